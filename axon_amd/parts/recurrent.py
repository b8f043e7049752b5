"""A recurrent mixer with a real-gated linear recurrence (the recurrent block of Griffin-like
models), with its state in the cache manager's state slots.

Two branches of `width` channels from the input h: y = gelu(Wy h + by) and u = conv(Wx h + bx), a
causal convolution of `conv` taps per channel.  The channels form `blocks` equal parts; in part b
the gates are r = sigmoid(Ra[b] u_b + ra[b]) and i = sigmoid(Ri[b] u_b + ri[b]).  Then
a = exp(-decay * r * softplus(lam)), S_t = a S_(t-1) + sqrt(1 - a^2) (i u) from S = 0, and the
output is Wo (S * y).  Gates, decays and the state are 32-bit; a request's state row holds S and
the convolution's last conv - 1 inputs, twice: the state behind position p in copy p & 1, so that a
decoding step reads one copy and writes the other and may be run again (the engine runs a step once
before it captures it into a graph) with the same result.

Parameters: `hidden_size`, `width`, `blocks`, `conv`, `decay` (default 8), `names` (the tensors'
names under the prefix: scope "mix.", y, x, conv, ra, ri, lam, o; a bias is the name + ".b").
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.base import ConfigError
from ..kernels import MODE_ADD_F32, MODE_STORE, MODE_STORE_F32
from .base import CacheBinding, Mixer, StateSpec, TensorDecl, register_mixer


def step_spans(ctx) -> Optional[torch.Tensor]:
    """The requests of a step as the scans want them: int32 [n, 3] = (slot, first token, tokens) on
    the device, made once a step; None in a step of single tokens (each its own request, read from
    the slots on the device, so that a captured graph holds nothing of one step)."""
    if ctx.decode_only:
        return None
    spans = ctx.shared.get("step_spans")
    if spans is None:
        rows = [[s.slot, s.q_start, s.q_len] for s in ctx.spans]
        spans = ctx.shared["step_spans"] = torch.tensor(rows, dtype=torch.int32).to(ctx.rt.device)
    return spans


class GatedRecurrence(Mixer):
    graph_safe = True
    stores_output = True

    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        p = params
        self.hidden, self.width = int(p["hidden_size"]), int(p["width"])
        self.blocks, self.taps, self.decay = int(p["blocks"]), int(p["conv"]), float(p.get("decay", 8.0))
        if self.blocks < 1 or self.width % self.blocks:
            raise ConfigError(f"a recurrence of {self.width} channels does not split into {self.blocks} equal blocks")
        if self.taps < 1:
            raise ConfigError(f"a convolution of {self.taps} taps")
        self.bw = self.width // self.blocks
        names = p.get("names", {})
        base = prefix + names.get("scope", "mix.")
        self.n = {k: base + names.get(k, k) for k in ("y", "x", "conv", "ra", "ri", "lam", "o")}

    def tensors(self) -> List[TensorDecl]:
        n, W, B, bw = self.n, self.width, self.blocks, self.bw
        return [TensorDecl(n["y"], (W, self.hidden)), TensorDecl(n["y"] + ".b", (W,), "bias"),
                TensorDecl(n["x"], (W, self.hidden)), TensorDecl(n["x"] + ".b", (W,), "bias"),
                TensorDecl(n["conv"], (W, self.taps)), TensorDecl(n["conv"] + ".b", (W,), "bias"),
                TensorDecl(n["ra"], (B, bw, bw)), TensorDecl(n["ra"] + ".b", (B, bw), "bias"),
                TensorDecl(n["ri"], (B, bw, bw)), TensorDecl(n["ri"] + ".b", (B, bw), "bias"),
                TensorDecl(n["lam"], (W,), "bias"), TensorDecl(n["o"], (self.hidden, W))]

    def state_spec(self) -> StateSpec:
        return StateSpec(2 * self.taps * self.width)

    def load(self, store, rt) -> None:
        n = self.n

        def together(a, b, dim=0):
            a, b = store.vector(a), store.vector(b)
            dt = torch.float32 if torch.float32 in (a.dtype, b.dtype) else a.dtype
            return torch.cat([a.to(dt), b.to(dt)], dim=dim).contiguous()
        self.w_yx = rt.k.prepare_weight(store.fused_matrix([n["y"], n["x"]]))
        self.b_yx = together(n["y"] + ".b", n["x"] + ".b")
        self.conv_w, self.conv_b = store.matrix(n["conv"]), store.vector(n["conv"] + ".b")
        # a block's rows of Ra, then its rows of Ri: one grouped product gives both gates
        self.w_gates = torch.cat([store.matrix(n["ra"]), store.matrix(n["ri"])], dim=1).contiguous()
        self.b_gates = together(n["ra"] + ".b", n["ri"] + ".b", dim=1)
        for name in (n["ra"], n["ri"]):
            store.forget(name)
        self.lam = store.vector(n["lam"])
        self.w_o = rt.k.prepare_weight(store.matrix(n["o"]))
        store.forget(n["o"])

    def forward(self, ctx, binding: CacheBinding, h, out, accumulate: bool = True) -> None:
        k, T, C = ctx.rt.k, h.shape[0], self.width
        state = ctx.cache.state(binding.state_index)
        yx = ctx.ws.take((T, 2 * C), ctx.rt.dtype)
        k.gemm(h, self.w_yx, yx, self.b_yx, MODE_STORE)
        y, x = yx[:, :C], yx[:, C:]
        u = ctx.ws.take((T, C), torch.float32)
        k.causal_conv(x, self.conv_w, self.conv_b, state, ctx.positions, ctx.seq_rows, u)
        gates = ctx.ws.take((T, 2 * C), torch.float32)
        k.grouped_gemm(u, self.w_gates, gates, x_group_stride=self.bw, out_group_stride=2 * self.bw, bias=self.b_gates)
        mixed = ctx.ws.take((T, C), ctx.rt.dtype)
        k.gated_scan(gates, u, y, x, self.lam, self.decay, state, step_spans(ctx), ctx.positions, ctx.seq_rows, mixed, self.bw,
                     self.taps)
        k.gemm(mixed, self.w_o, out, None, MODE_ADD_F32 if accumulate else MODE_STORE_F32)


register_mixer("gated_recurrence", GatedRecurrence)
