"""Small Pikesun configurations and weights for the tests: sizes that differ between the models and
from one another within a model (query/key size against value size, recurrence width against model
width), values of 1 (one head, one block, one tap, the first expert only), widths that no
matrix-core product takes, and weights drawn so that the mechanisms matter: decays near 1 (a long
memory), scores sharp enough that a key far back or at a window's edge decides a row."""
import json
import os

import torch


def rec(width, blocks, conv):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def att(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, base=10000.0, scale=0.5):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
             "rot": {"base": base, "dims": rot_dim}, "scale": scale}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def layer(mixer, mlp, weights_of=None):
    entry = dict(mixer, mlp=mlp)
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def config(width, vocab, layers, eps=1e-6, mult=0.7, scale=4.0):
    return {"architecture": "Pikesun", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "vocab": vocab, "width": width}


MODELS = {
    # attention first, a short window (9: edges everywhere), a recurrence wider than the model with
    # blocks of 24 channels and 3 taps, a shared layer, experts with a shared one; nothing a multiple of 32
    "P": dict(cfg=config(48, 131, [
        layer(att(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, window=9, base=100.0), moe(6, 2, 24, 1.5, (40, 1.0))),
        layer(rec(72, 3, 3), dense(80)),
        layer(rec(72, 3, 3), dense(80), weights_of=1),
        layer(att(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, window=9, base=100.0), moe(6, 2, 24, 1.5, (40, 1.0)),
              weights_of=0)], eps=1e-5, mult=0.5), page=8, seed=3),
    # the shapes the matrix-core forms take (multiples of 32 and 64), a window of 150 that crosses
    # pages of 64, one head, one block, every expert chosen, a layer without a feed-forward, no factors
    "Q": dict(cfg=config(128, 300, [
        layer(rec(128, 1, 4), None),
        layer(att(heads=1, dim=32, rot_dim=32, vdim=64, kv_rank=64, q_rank=32, window=150), moe(4, 4, 64, 2.5)),
        layer(rec(192, 3, 2), moe(8, 1, 32, 1.0, (64, 3.0))),
        layer(att(heads=4, dim=64, rot_dim=16, vdim=32, kv_rank=96, q_rank=64, window=40, base=5000.0, scale=0.3), dense(256))],
        eps=1e-6, mult=1.0, scale=1.0), page=64, seed=8),
    # one tap (no kept inputs), no window at all, two attention layers of different windows and ranks
    # (two page pools), an odd vocabulary
    "R": dict(cfg=config(64, 257, [
        layer(rec(64, 2, 1), dense(96)),
        layer(att(heads=2, dim=16, rot_dim=8, vdim=8, kv_rank=24, q_rank=40, window=0), dense(64)),
        layer(att(heads=5, dim=8, rot_dim=2, vdim=16, kv_rank=12, q_rank=8, window=33, scale=0.8), moe(3, 2, 16, 0.7))],
        eps=1e-4, mult=1.3, scale=9.0), page=16, seed=5),
    # recurrences only: no pages at all, a layer without a feed-forward between two that share tensors
    "S": dict(cfg=config(80, 140, [
        layer(rec(96, 4, 4), moe(5, 3, 24, 1.2)),
        layer(rec(160, 2, 2), None),
        layer(rec(96, 4, 4), moe(5, 3, 24, 1.2), weights_of=0)], eps=1e-6, mult=0.8, scale=2.0), page=32, seed=12),
    # sixteen heads and latents in sixteens: the matrix-core attention inside a whole model, with pages of 64
    "T": dict(cfg=config(64, 190, [
        layer(att(heads=16, dim=16, rot_dim=16, vdim=8, kv_rank=48, q_rank=32, window=75), dense(96)),
        layer(rec(64, 2, 3), moe(4, 2, 32, 2.0, (32, 2.0))),
        layer(att(heads=16, dim=16, rot_dim=16, vdim=8, kv_rank=48, q_rank=32, window=75), dense(96), weights_of=0)],
        eps=1e-5, mult=0.9, scale=3.0), page=64, seed=14),
}


def draw_weights(cfg, seed):
    """name -> float32 tensor of values that bfloat16 holds exactly (both compute dtypes and the
    plain implementation then start from the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def matrix(name, *shape, gain=1.0):
        W[name] = torch.randn(*shape, generator=g) * (gain / shape[-1] ** 0.5)

    def vector(name, *shape, mean=0.0, std=0.1):
        W[name] = torch.randn(*shape, generator=g) * std + mean

    width = cfg["width"]
    W["embed"] = torch.randn(cfg["vocab"], width, generator=g)
    vector("final.norm", width, mean=1.0)
    matrix("head", cfg["vocab"], width)
    for i, L in enumerate(cfg["layers"]):
        if "weights_of" in L:
            continue
        p, m = f"l{i}.", L["mixer"]
        vector(p + "norm1", width, mean=1.0)
        if L["type"] == "rglru":
            C, B = m["width"], m["blocks"]
            for n in ("y", "x"):
                matrix(p + "mix." + n, C, width)
                vector(p + "mix." + n + ".b", C)
            W[p + "mix.conv"] = torch.randn(C, m["conv"], generator=g) * 0.6
            vector(p + "mix.conv.b", C)
            for n in ("ra", "ri"):
                matrix(p + "mix." + n, B, C // B, C // B, gain=2.0)
                vector(p + "mix." + n + ".b", B, C // B, std=0.5)
            vector(p + "mix.lam", C, mean=-3.5, std=1.5)          # decays from about 0.5 to 0.999 a step
            matrix(p + "mix.o", width, C)
        else:
            H = m["heads"]
            matrix(p + "mix.dq", m["q_rank"], width)
            vector(p + "mix.dq.norm", m["q_rank"], mean=1.0)
            matrix(p + "mix.uq", H * (m["dim"] + m["rot_dim"]), m["q_rank"], gain=1.5)
            matrix(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], width)
            vector(p + "mix.dkv.norm", m["kv_rank"], mean=1.0)
            matrix(p + "mix.uk", H * m["dim"], m["kv_rank"], gain=1.5)
            matrix(p + "mix.uv", H * m["vdim"], m["kv_rank"])
            matrix(p + "mix.g", H * m["vdim"], width, gain=2.0)
            matrix(p + "mix.o", width, H * m["vdim"])
        mlp = L.get("mlp")
        if mlp is None:
            continue
        vector(p + "norm2", width, mean=1.0)
        if mlp["kind"] == "dense":
            matrix(p + "mlp.up", mlp["ff"], width, gain=1.5)
            matrix(p + "mlp.down", width, mlp["ff"])
        else:
            matrix(p + "mlp.router", mlp["router"]["experts"], width, gain=2.0)
            units = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                units.append(("shared.", mlp["shared"]["ff"]))
            for scope, ff in units:
                matrix(p + "mlp." + scope + "gate", ff, width, gain=2.0)      # wide enough to meet the clamps
                matrix(p + "mlp." + scope + "up", ff, width, gain=2.0)
                matrix(p + "mlp." + scope + "down", width, ff)
    return {k: v.to(torch.bfloat16).float() for k, v in W.items()}


def write_model(path, cfg, W):
    from axon_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path, exist_ok=True)
    write_safetensors(os.path.join(path, "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in W.items()], {"format": "pt"})
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return path


def make(path, name):
    m = MODELS[name]
    return write_model(path, m["cfg"], draw_weights(m["cfg"], m["seed"]))
