"""Input filters: what stands between a block's first norm and its mixer and changes the rows that the mixer reads."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import FILTERS, FixedState, Part


@FILTERS.register("none")
class NoFilter(Part):
    graph_safe = True

    def __init__(self):
        pass

    def cache_spec(self):
        return None

    def forward(self, h, ctx, cache):
        return h


@FILTERS.register("causal_conv")
class CausalConv(Part):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j): a convolution over time on every channel, nothing before a request's
    first token.  The last taps - 1 rows it has read are a request's state, so a prompt may come in portions.  It
    reads 32-bit rows and writes the engine's activation dtype."""
    graph_safe = True
    libraries = ("sequence",)
    in_dtype = torch.float32

    def __init__(self, width: int, taps: int, weight_name: str):
        if taps < 1:
            raise ValueError(f"causal_conv: {taps} taps")
        self.width, self.taps, self.weight_name = width, taps, weight_name

    def param_specs(self):
        return [ParamSpec(self.weight_name, (self.width, self.taps), "vector", ("normal", 0.0, 0.2))]

    def cache_spec(self):
        return FixedState(((self.taps - 1) * self.width,)) if self.taps > 1 else None

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.weight_name]

    def forward(self, h, ctx, cache):
        out = torch.empty(h.shape, dtype=self.runtime.act_dtype, device=h.device)
        ops.conv_rows(h, self.weight, cache.state, ctx.row_start, ctx.state_slots, out)
        if self.taps > 1 and cache.writes:
            ops.history_update(h, cache.state, ctx.row_start, ctx.state_slots)
        return out
