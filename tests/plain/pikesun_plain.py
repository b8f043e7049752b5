"""The Pikesun decoder, slowly and plainly: whole sequences, no cache, no state carried, float64.

One function per mechanism, written from the design's equations and sharing nothing with the
engine.  A model is (cfg, W): config.json as a dict and the tensors by name as float64.

Notation: h is a [T, width] input, positions are 0 .. T - 1, sigma is the logistic function.

    rms(x, g)        = x / sqrt(mean(x^2) + eps) * g
    layer            : x <- x + m rms(mixer(x), g1);  x <- x + m rms(ff(x), g2)
    recurrence       : y = gelu(Wy h + by); u = conv(Wx h + bx); per block b of channels
                       r = sigma(Ra_b u_b + ra_b), i = sigma(Ri_b u_b + ri_b);
                       a = exp(-8 r softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) i u; out = Wo (S y)
    latent attention : cq = rms(Wdq h, gq); q = Wuq cq = per head [qn | qr];
                       [c_raw | kr] = Wdkv h; c = rms(c_raw, gkv); kn = Wuk c; v = Wuv c (per head)
                       score(i, j) = (qn_i . kn_j + rot(qr_i, i) . rot(kr_j, j)) scale for 0 <= i - j < window
                       out = Wo (softmax(score) v * sigma(Wg h))
    experts          : z = Wr h; the `top` largest z, weights softmax over those;
                       expert(h) = Wd (g sigma(1.702 g) (u + 1)), g = min(Wg h, L), u = clamp(Wu h, -L, L)
"""
import json
import math
import os

import torch


def load_plain(model_dir):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    W = {k: v.double() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, W


# --------------------------------------------------------------------------- small pieces
def rms(x, gain, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigma(z):
    return 1.0 / (1.0 + torch.exp(-z))


def rotate(v, positions, dims, base):
    """Pairs (k, k + dims / 2) of the first `dims` places of v [T, ..., n] turned by position * base^(-2k / dims)."""
    half = dims // 2
    out = v.clone()
    for k in range(half):
        angle = positions.double() * base ** (-2.0 * k / dims)
        shape = [-1] + [1] * (v.dim() - 2)
        c, s = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
        a, b = v[..., k], v[..., k + half]
        out[..., k] = a * c - b * s
        out[..., k + half] = b * c + a * s
    return out


# --------------------------------------------------------------------------- the recurrent mixer
def causal_conv(x, taps_of_channel, bias):
    """x [T, C]; taps_of_channel [C, n]: the last column weighs the current token, zeros before the start."""
    T, C = x.shape
    n = taps_of_channel.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for k in range(n):
            src = t - (n - 1 - k)
            if src >= 0:
                out[t] += taps_of_channel[:, k] * x[src]
    return out + bias


def gated_recurrence(W, p, c, h, start_state=None):
    """p: the tensors' prefix ('l0.mix.'); c: the mixer's sizes (width, blocks, conv)."""
    T = h.shape[0]
    width, blocks = c["width"], c["blocks"]
    bw = width // blocks
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = causal_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    r, i = torch.zeros_like(u), torch.zeros_like(u)
    for b in range(blocks):
        part = slice(b * bw, (b + 1) * bw)
        r[:, part] = sigma(u[:, part] @ W[p + "ra"][b].T + W[p + "ra.b"][b])
        i[:, part] = sigma(u[:, part] @ W[p + "ri"][b].T + W[p + "ri.b"][b])
    a = torch.exp(-8.0 * r * torch.log1p(torch.exp(W[p + "lam"])))
    S = torch.zeros(width, dtype=h.dtype) if start_state is None else start_state
    rows = []
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        rows.append(S * y[t])
    return torch.stack(rows) @ W[p + "o"].T


# --------------------------------------------------------------------------- latent attention
def latent_attention(W, p, c, h, eps, window_override=None):
    T, H = h.shape[0], c["heads"]
    dim, rot, vdim, rank = c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    window = c["mask"]["size"] if c.get("mask") else 0
    if window_override is not None:
        window = window_override
    pos = torch.arange(T)
    q = (rms(h @ W[p + "dq"].T, W[p + "dq.norm"], eps) @ W[p + "uq"].T).view(T, H, dim + rot)
    down = h @ W[p + "dkv"].T
    latent = rms(down[:, :rank], W[p + "dkv.norm"], eps)
    shared_key = down[:, rank:]
    if rot:
        q = torch.cat([q[..., :dim], rotate(q[..., dim:], pos, c["rot"]["dims"], c["rot"]["base"])], dim=-1)
        shared_key = rotate(shared_key, pos, c["rot"]["dims"], c["rot"]["base"])
    keys = (latent @ W[p + "uk"].T).view(T, H, dim)
    values = (latent @ W[p + "uv"].T).view(T, H, vdim)
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for i in range(T):
        first = max(0, i - window + 1) if window > 0 else 0
        for head in range(H):
            s = (keys[first:i + 1, head] @ q[i, head, :dim] + shared_key[first:i + 1] @ q[i, head, dim:]) * c["scale"]
            w = torch.softmax(s, dim=0)
            out[i, head] = w @ values[first:i + 1, head]
    gated = out.reshape(T, H * vdim) * sigma(h @ W[p + "g"].T)
    return gated @ W[p + "o"].T


# --------------------------------------------------------------------------- feed-forwards
def dense_ff(W, p, h):
    return gelu_tanh(h @ W[p + "up"].T) @ W[p + "down"].T


def clamped_unit(W, p, h, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, min=-limit, max=limit)
    return (g * sigma(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def routed_ff(W, p, c, h):
    T = h.shape[0]
    z = h @ W[p + "router"].T
    top = c["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(T):
        order = sorted(range(z.shape[1]), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, order], dim=0)
        for share, e in zip(w, order):
            out[t] += share * clamped_unit(W, f"{p}e{e}.", h[t:t + 1], c["expert"]["limit"])[0]
    if c.get("shared"):
        out = out + clamped_unit(W, p + "shared.", h, c["shared"]["limit"])
    return out


def feed_forward(W, p, c, h):
    return dense_ff(W, p, h) if c["kind"] == "dense" else routed_ff(W, p, c, h)


# --------------------------------------------------------------------------- the model
def residual_stream(cfg, W, tokens, after_every_layer=None):
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = W["embed"][torch.as_tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{layer.get('weights_of', i)}."
        if layer["type"] == "rglru":
            mixed = gated_recurrence(W, p + "mix.", layer["mixer"], x)
        else:
            mixed = latent_attention(W, p + "mix.", layer["mixer"], x, eps)
        x = x + m * rms(mixed, W[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + m * rms(feed_forward(W, p + "mlp.", layer["mlp"], x), W[p + "norm2"], eps)
        if after_every_layer is not None:
            after_every_layer.append(x.clone())
    return x


def forward_logits(cfg, W, tokens):
    x = residual_stream(cfg, W, tokens)
    return rms(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T


def greedy_generate(cfg, W, prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        row = forward_logits(cfg, W, seq)[-1].float()
        best = max(range(row.numel()), key=lambda v: (float(row[v]), v))
        out.append(best)
        seq.append(best)
    return out
