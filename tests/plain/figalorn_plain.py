"""The Figalorn decoder, slowly and plainly: whole sequences, no cache, float64.

One function per mechanism, written from the design's equations and sharing nothing with the
engine.  A model is (cfg, W): config.json as a dict and the tensors by name as float64.

Notation: h is a [T, width] input, positions are 0 .. T - 1, sigma is the logistic function,
rms(x) = x / sqrt(mean(x^2) + eps).

    norm             : rms(x) (1 + w)
    layer            : x <- x + mixer(norm1 x);  x <- x + ff(norm2 x)
    loop             : layers start .. stop - 1 run `times` times over; each pass begins with
                       x <- W_in [x ; x0], x0 the embedding rows
    differential     : per head two score maps over one set of values, q = [q1 | q2], k = [k1 | k2];
    attention          pairs (2i, 2i + 1) of the first rot dims of each map turn by p f_i;
                       a_m = softmax(q_m k_m^T scale over the keys of the query's chunk) v;
                       lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff;
                       o = rms(a_1 - lam a_2) (1 - diff);  out = W_o (o sigma(W_g h))
    keys as values   : q, k per head through rms with a gain, then pairs (i, i + rot / 2) turn by
                       p f_i with cos and sin scaled by m; v = the keys as projected;
                       score = cap tanh(q . k scale / cap) for 0 <= i - j < window
    feed-forward     : W_down gelu(W_up h), gelu(z) = z (1 + erf(z / sqrt 2)) / 2
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
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def sigma(z):
    return 1.0 / (1.0 + torch.exp(-z))


# --------------------------------------------------------------------------- rotation
def base_frequencies(dims, base):
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def stretched_frequencies(dims, base, factor, low, high, original):
    """Long wavelengths are slowed by `factor`, short ones kept, those between blended."""
    out = []
    for f in base_frequencies(dims, base):
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelength - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


def ramped_frequencies(dims, base, factor, original, fast, slow):
    """A linear ramp over the pair index between the pairs that turn `fast` and `slow` times in
    `original` positions; returns (frequencies, the factor on cos and sin)."""
    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), dims - 1)
    out = []
    for i, f in enumerate(base_frequencies(dims, base)):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def turn(v, positions, freqs, pairing, magnitude=1.0):
    """v [T, ..., n]: pair i of the first 2 len(freqs) places turns by position * freqs[i];
    `pairing` "neighbours": places (2i, 2i + 1); "halves": places (i, i + len(freqs))."""
    n = len(freqs)
    out = v.clone()
    shape = [-1] + [1] * (v.dim() - 2)
    for i, f in enumerate(freqs):
        angle = positions.double() * f
        c, s = (torch.cos(angle) * magnitude).view(shape), (torch.sin(angle) * magnitude).view(shape)
        ia, ib = (2 * i, 2 * i + 1) if pairing == "neighbours" else (i, i + n)
        a, b = v[..., ia], v[..., ib]
        out[..., ia] = a * c - b * s
        out[..., ib] = b * c + a * s
    return out


# --------------------------------------------------------------------------- masks
def chunk_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def window_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (i - j >= 0) & (i - j < size)


def masked_softmax(scores, mask):
    scores = scores.masked_fill(~mask, float("-inf"))
    return torch.softmax(scores, dim=-1)


# --------------------------------------------------------------------------- mixers
def differential_attention(h, W, p, m, eps):
    """h [T, width]; W: tensors under the prefix p; m: the mixer's config."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, 2, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, 2, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    rot = m["rot"]
    sc = rot.get("scaling")
    freqs = (stretched_frequencies(rot["dims"], rot["base"], sc["factor"], sc["low"], sc["high"], sc["original"])
             if sc else base_frequencies(rot["dims"], rot["base"]))
    q, k = turn(q, pos, freqs, "neighbours"), turn(k, pos, freqs, "neighbours")
    mask = chunk_mask(T, m["mask"]["size"])
    diff = m["diff"]
    lam = math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + diff
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        a = [masked_softmax(q[:, hd, i] @ k[:, g, i].T * m["scale"], mask) @ v[:, g] for i in range(2)]
        heads.append(rms(a[0] - lam * a[1], eps) * (1.0 - diff))
    o = torch.cat(heads, dim=-1) * sigma(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def key_value_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, G, d)
    v = k
    q, k = rms(q, eps) * W[p + "q.norm"], rms(k, eps) * W[p + "k.norm"]
    rot = m["rot"]
    sc = rot.get("scaling")
    if sc:
        freqs, magnitude = ramped_frequencies(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"])
    else:
        freqs, magnitude = base_frequencies(rot["dims"], rot["base"]), 1.0
    q, k = turn(q, pos, freqs, "halves", magnitude), turn(k, pos, freqs, "halves", magnitude)
    mask = window_mask(T, m["mask"]["size"])
    cap = m.get("softcap")
    heads = []
    for hd in range(H):
        g = hd // (H // G)
        s = q[:, hd] @ k[:, g].T * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        heads.append(masked_softmax(s, mask) @ v[:, g])
    return torch.cat(heads, dim=-1) @ W[p + "o"].T


def feed_forward(h, W, p):
    return gelu_erf(h @ W[p + "up"].T) @ W[p + "down"].T


MIXERS = {"attention": differential_attention, "attention_2": key_value_attention}


# --------------------------------------------------------------------------- the model
def layer_order(cfg):
    """[(layer, starts a pass)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg, W, tokens, streams=None):
    """Logits [T, vocab] of a whole sequence; `streams`, a list, takes the residual stream after
    every layer run."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x0 = x
    for i, begins in layer_order(cfg):
        layer = cfg["layers"][i]
        if begins:
            x = torch.cat([x, x0], dim=-1) @ W["loop.in"].T
        p = f"l{i}."
        x = x + MIXERS[layer["type"]](norm(x, W[p + "norm1"], eps), W, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + feed_forward(norm(x, W[p + "norm2"], eps), W, p + "mlp.")
        if streams is not None:
            streams.append(x)
    return norm(x, W["final.norm"], eps) @ W["head"].T


def greedy_generate(cfg, W, prompt, n_new):
    """n_new tokens, each the largest logit after everything before it (ties to the larger id)."""
    seq, out = list(prompt), []
    for _ in range(n_new):
        row = forward(cfg, W, seq)[-1]
        best = float(row.max())
        tok = max(i for i in range(row.numel()) if float(row[i]) == best)
        seq.append(tok)
        out.append(tok)
    return out
