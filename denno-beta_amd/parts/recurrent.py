"""Mixers that keep a matrix per head instead of keys and values: S <- diag(w) S + a v^T, read with a query.
Both run the one scan kernel (kernels.ops.state_scan); what differs is how a token makes r, a, v and w."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import MIXERS, FixedState, Part
from .linear import Linear

F32 = torch.float32


@MIXERS.register("wkv")
class WKV(Part):
    """Every projection reads its own blend of the token's row and the row before it, h + (h' - h) mu.  r, k, v are
    plain projections, the gate silu(W_g .), the decay w = exp(-exp(W_2 tanh(W_1 .) + w0)) per head and key channel.
    o_t = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T; each head's o is divided by its root mean square,
    times a weight per column, times the gate, then the output projection.  State: S in 32-bit and the last row."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, head_dim: int, eps: float, lora: int, names: dict):
        """names: r, k, v, g, w1, w2, o (matrices); mu_r, mu_k, mu_v, mu_g, mu_w, w0, u, norm (vectors)."""
        self.width, self.n_heads, self.head_dim, self.eps, self.lora, self.names = width, n_heads, head_dim, eps, lora, dict(names)
        n = n_heads * head_dim
        self.inner = n
        self.r, self.k, self.v, self.g = (Linear(width, n, names[s], None) for s in "rkvg")
        self.w1, self.w2 = Linear(width, lora, names["w1"], None), Linear(lora, n, names["w2"], None)
        self.out = Linear(n, width, names["o"], None)

    def param_specs(self):
        n, W = self.inner, self.width
        specs = []
        for lin in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.out):
            specs += lin.param_specs()
        specs += [ParamSpec(self.names["mu_" + s], (W,), "vector", ("normal", 0.5, 0.15)) for s in "rkvgw"]
        specs += [ParamSpec(self.names["w0"], (n,), "vector", ("normal", -1.0, 0.7)),
                  ParamSpec(self.names["u"], (self.n_heads, self.head_dim), "vector", ("normal", 0.3, 0.3)),
                  ParamSpec(self.names["norm"], (n,), "vector", ("normal", 1.0, 0.1))]
        return specs

    def cache_spec(self):
        return FixedState((self.inner * self.head_dim + self.width,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        for lin in (self.r, self.k, self.v, self.g, self.w1, self.w2, self.out):
            lin.bind(tensors)
        self.mu = torch.stack([tensors[self.names["mu_" + s]] for s in "rkvgw"]).contiguous()
        self.w0, self.norm = tensors[self.names["w0"]], tensors[self.names["norm"]]
        self.u = tensors[self.names["u"]].reshape(-1).contiguous()

    def forward(self, h, ctx, cache, accumulate_into):
        act, T, n = self.runtime.act_dtype, h.shape[0], self.inner
        state, last = cache.state[:, :n * self.head_dim], cache.state[:, n * self.head_dim:]
        mixes = torch.empty((5, T, self.width), dtype=act, device=h.device)
        ops.shift_mix(h, last, self.mu, ctx.row_start, ctx.state_slots, mixes)
        if cache.writes:
            ops.history_update(h, last, ctx.row_start, ctx.state_slots)
        r, k, v, g = (lin(mixes[i], out_dtype=F32) for i, lin in enumerate((self.r, self.k, self.v, self.g)))
        low = ops.activate(self.w1(mixes[4], out_dtype=F32), "tanh", torch.empty((T, self.lora), dtype=act, device=h.device))
        w = self.w2(low, out_dtype=F32)
        ops.activate(w, "exp_neg_exp", w, bias=self.w0)
        o = torch.empty((T, n), dtype=F32, device=h.device)
        ops.state_scan(r, k, v, w, self.u, state, ctx.row_start, ctx.state_slots, self.n_heads, self.head_dim, self.head_dim, o)
        y = torch.empty((T, n), dtype=act, device=h.device)
        ops.head_norm(o, self.norm, self.eps, y, self.n_heads, gate=g, gate_kind="silu")
        self.out(y, residual=accumulate_into)


@MIXERS.register("hgrn2")
class HGRN2(Part):
    """The forget gate f = lower + (1 - lower) sigmoid(W_f h + b) per head and channel also decides what is written:
    S <- diag(f) S + (1 - f) v^T, o = S^T q with q = silu(W_q h); each head's o is normed over its value columns with
    one weight shared by the heads, then the output projection.  State: S in 32-bit."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, n_heads: int, head_dim: int, value_dim: int, eps: float, names: dict):
        """names: q, f, v, o (matrices); f_bias, lower, norm (vectors)."""
        self.width, self.n_heads, self.head_dim, self.value_dim, self.eps = width, n_heads, head_dim, value_dim, eps
        self.names = dict(names)
        self.qk, self.vw = n_heads * head_dim, n_heads * value_dim
        self.proj = Linear(width, 2 * self.qk + self.vw, names["q"] + "+f+v", None,
                           weight_sources=((names["q"], self.qk), (names["f"], self.qk), (names["v"], self.vw)))
        self.out = Linear(self.vw, width, names["o"], None)

    def param_specs(self):
        return self.proj.param_specs() + self.out.param_specs() + [
            ParamSpec(self.names["f_bias"], (self.qk,), "vector", ("normal", 0.0, 1.0)),
            ParamSpec(self.names["lower"], (self.qk,), "vector", ("uniform", 0.0, 0.9)),
            ParamSpec(self.names["norm"], (self.value_dim,), "vector", ("normal", 1.0, 0.1))]

    def cache_spec(self):
        return FixedState((self.qk * self.value_dim,))

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.proj.bind(tensors), self.out.bind(tensors)
        self.f_bias, self.lower, self.norm = (tensors[self.names[s]] for s in ("f_bias", "lower", "norm"))

    def forward(self, h, ctx, cache, accumulate_into):
        act, T = self.runtime.act_dtype, h.shape[0]
        z = self.proj(h, out_dtype=F32)
        q, f, v = z[:, :self.qk], z[:, self.qk:2 * self.qk], z[:, 2 * self.qk:]
        ops.activate(q, "silu", q)
        ops.activate(f, "bounded_sigmoid", f, bias=self.f_bias, lower=self.lower)
        o = torch.empty((T, self.vw), dtype=F32, device=h.device)
        ops.state_scan(q, None, v, f, None, cache.state, ctx.row_start, ctx.state_slots, self.n_heads, self.head_dim,
                       self.value_dim, o, read_after=True, key_from_decay=True)
        y = torch.empty((T, self.vw), dtype=act, device=h.device)
        ops.head_norm(o, self.norm, self.eps, y, self.n_heads)
        self.out(y, residual=accumulate_into)
