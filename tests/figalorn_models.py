"""Small Figalorn configurations and weights for the tests: sizes that differ between the models and
within a model (key size against value size, heads against key/value heads, rotated dims against the
key size), values of 1 (one head, one key/value head, a window of one position, one pass of the loop),
sizes that the matrix-core kernel takes and sizes it does not, a loop that starts behind the first
layer, layers without a feed-forward, and weights drawn so that scores are sharp: a key at a window's
or a chunk's edge decides a row."""
import json
import os

import torch


def diff(heads, kv_heads, dim, vdim, chunk, rot_dims, d=0.3, base=10000.0, scaling=(8.0, 1.0, 4.0, 64), scale=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": d, "mask": {"size": chunk},
             "rot": {"base": base, "dims": rot_dims}, "scale": scale if scale is not None else dim ** -0.5}
    if scaling:
        mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": mixer}


def keyed(heads, kv_heads, dim, window, rot_dims, softcap=30.0, base=10000.0, scaling=(4.0, 128, 32.0, 1.0), scale=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window},
             "rot": {"base": base, "dims": rot_dims}, "scale": scale if scale is not None else dim ** -0.5}
    if softcap:
        mixer["softcap"] = softcap
    if scaling:
        mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "attention_2", "mixer": mixer}


def layer(mixer, ff):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


def config(width, vocab, layers, loop=None, eps=1e-5):
    cfg = {"architecture": "Figalorn", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


MODELS = {
    # sizes the matrix-core kernel takes in 16 bits (keys in eights, values in sixteens, pages of 64); a loop over the
    # two middle layers, three times; a window (24) and chunks (40) that cross neither pages nor each other evenly
    "A": dict(cfg=config(64, 150, [
        layer(keyed(heads=4, kv_heads=2, dim=16, window=24, rot_dims=8), 96),
        layer(diff(heads=4, kv_heads=2, dim=8, vdim=32, chunk=40, rot_dims=4), 80),
        layer(keyed(heads=2, kv_heads=2, dim=32, window=70, rot_dims=32, softcap=5.0, scaling=None), None),
        layer(diff(heads=6, kv_heads=1, dim=24, vdim=16, chunk=64, rot_dims=24, d=0.1, scaling=(2.0, 1.0, 2.0, 32)), 72)],
        loop=(1, 3, 3)), page=64, seed=3),
    # nothing a multiple of eight: the kernel of any sizes in both builds; one key/value head, three query heads, a
    # window of one position (a token sees itself alone), chunks of seven, no loop, pages of 8
    "B": dict(cfg=config(40, 97, [
        layer(diff(heads=3, kv_heads=1, dim=6, vdim=10, chunk=7, rot_dims=6, d=0.5, base=100.0), 50),
        layer(keyed(heads=3, kv_heads=3, dim=12, window=1, rot_dims=4, base=50.0), 44),
        layer(keyed(heads=1, kv_heads=1, dim=20, window=13, rot_dims=10, softcap=2.0, scaling=(16.0, 32, 8.0, 2.0)), None)],
        eps=1e-4), page=8, seed=5),
    # the whole model in the loop, once (the stream is still rewritten at its start); twenty query heads on one
    # key/value head (more columns than a tile holds), chunks of exactly a page, a window of a page and one
    "C": dict(cfg=config(96, 211, [
        layer(diff(heads=20, kv_heads=1, dim=16, vdim=16, chunk=64, rot_dims=2, d=0.2), 64),
        layer(keyed(heads=8, kv_heads=4, dim=48, window=65, rot_dims=16, softcap=50.0), 128)],
        loop=(0, 2, 1), eps=1e-6), page=64, seed=8),
    # keys and values of more than 128 (the largest register tile), pages of 128, a loop at the end
    "D": dict(cfg=config(64, 120, [
        layer(keyed(heads=2, kv_heads=1, dim=144, window=100, rot_dims=64), 64),
        layer(diff(heads=2, kv_heads=2, dim=40, vdim=144, chunk=90, rot_dims=12), None)],
        loop=(1, 2, 2)), page=128, seed=13),
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
    vector("final.norm", width)
    matrix("head", cfg["vocab"], width)
    if "loop" in cfg:
        matrix("loop.in", width, 2 * width, gain=1.4)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        vector(p + "norm1", width)
        if L["type"] == "attention":
            matrix(p + "mix.q", H * 2 * d, width, gain=2.5)
            matrix(p + "mix.k", G * 2 * d, width, gain=2.5)
            matrix(p + "mix.v", G * dv, width)
            for n, rows in (("q", H * 2 * d), ("k", G * 2 * d), ("v", G * dv)):
                vector(p + "mix." + n + ".b", rows, std=0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vector(p + "mix." + n, d, std=0.4)
            matrix(p + "mix.g", H * dv, width, gain=2.0)
        else:
            matrix(p + "mix.q", H * d, width)
            matrix(p + "mix.k", G * d, width)
            vector(p + "mix.q.norm", d, mean=2.0, std=0.5)      # the norm's gain makes the scores sharp
            vector(p + "mix.k.norm", d, mean=2.0, std=0.5)
        matrix(p + "mix.o", width, H * dv)
        if L.get("mlp") is not None:
            vector(p + "norm2", width)
            matrix(p + "mlp.up", L["mlp"]["ff"], width, gain=1.5)
            matrix(p + "mlp.down", width, L["mlp"]["ff"])
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
