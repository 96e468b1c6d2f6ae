"""Feed-forwards: the parts that work on each token alone."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import FEED_FORWARDS, Part
from .linear import Linear

ACTIVATION_EPILOGUES = {"gelu_tanh": "gelu_tanh", "gelu_erf": "gelu_erf"}


@FEED_FORWARDS.register("dense_mlp")
class DenseMLP(Part):
    """act(h W_up + b_up) W_down + b_down, added into the residual stream
    (crates/denno-engine/src/model/gpt2.rs:211-219).  The activation runs in the first
    product's epilogue, in 32-bit, before the rounding to the activation dtype."""
    graph_safe = True

    def __init__(self, width: int, inner: int, activation: str, up_weight: str, up_bias, down_weight: str,
                 down_bias, stored_in_out: bool = False, down_init_std: float = 0.02):
        if activation not in ACTIVATION_EPILOGUES:
            raise ValueError(f"activation {activation!r}; known: {sorted(ACTIVATION_EPILOGUES)}")
        self.width, self.inner, self.activation = width, inner, activation
        self.up = Linear(width, inner, up_weight, up_bias, stored_in_out)
        self.down = Linear(inner, width, down_weight, down_bias, stored_in_out, down_init_std)

    def param_specs(self):
        return self.up.param_specs() + self.down.param_specs()

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.up.bind(tensors)
        self.down.bind(tensors)

    def packed_input(self, n_rows):
        return self.up.packed_input(n_rows)

    def prepare_lazy_norm(self, norm):
        self.up.fold_norm(norm)

    def takes_lazy_norm(self, n_rows, norm):
        return self.up.takes_lazy_norm(n_rows, norm)

    def writes_norm_stats(self, n_rows):
        return self.down.writes_norm_stats(n_rows)

    def defers_sum(self, n_rows):
        return self.down.defers(n_rows)

    def forward(self, h, ctx, accumulate_into, stats=None, deferred=None):
        n = h.shape[0]
        f = self.up(h, out_dtype=self.runtime.act_dtype, epilogue=ACTIVATION_EPILOGUES[self.activation],
                    packed_out=self.up.few_rows(n) and self.down.packed_input(n))
        self.down(f, residual=accumulate_into, stats=stats, deferred=deferred)


@FEED_FORWARDS.register("none")
class NoFeedForward(Part):
    """A block without a feed-forward: nothing is added to the stream (and the block does not run the norm before it)."""
    graph_safe = True
    absent = True

    def __init__(self):
        pass

    def forward(self, h, ctx, accumulate_into):
        return None


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(Part):
    """A mixture of small feed-forwards.  The router's scores are s = softmax(W_router h) over all experts, in 32-bit; a
    token's `top` experts are the ones with the largest s + correction, its weights their s divided by their sum
    (+ 1e-20).  An expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), W_down (g sigmoid(alpha g) (u + 1)).
    The step's (token, expert) pairs are sorted by expert on the device, each expert's products run over tiles of its
    own rows, and the results are added into the stream per token in the order of its choices."""
    graph_safe = True
    libraries = ("grouped",)

    def __init__(self, width: int, inner: int, n_experts: int, top: int, limit: float, alpha: float, router: str,
                 correction, gate: str, up: str, down: str):
        """gate, up, down: tensor names with {e} for the expert's number; correction: a name or None."""
        if not 1 <= top <= n_experts:
            raise ValueError(f"routed_experts: {top} of {n_experts} experts")
        self.width, self.inner, self.n_experts, self.top = width, inner, n_experts, top
        self.limit, self.alpha = float(limit), float(alpha)
        self.router = Linear(width, n_experts, router, None)
        self.correction_name = correction
        self.templates = dict(gate=gate, up=up, down=down)

    def _stacked(self, which):
        E = self.n_experts
        rows, cols = (self.width, self.inner) if which == "down" else (self.inner, self.width)
        t = self.templates[which]
        return ParamSpec(t.format(e="*"), (E * rows, cols), "matrix", ("normal", 0.0, cols ** -0.5),
                         sources=tuple((t.format(e=e), rows) for e in range(E)), concat_dim=0)

    def param_specs(self):
        specs = self.router.param_specs() + [self._stacked(w) for w in ("gate", "up", "down")]
        if self.correction_name:
            specs.append(ParamSpec(self.correction_name, (self.n_experts,), "vector", ("normal", 0.0, 0.02)))
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.router.bind(tensors)
        E = self.n_experts
        self.w_gate = tensors[self.templates["gate"].format(e="*")].view(E, self.inner, self.width)
        self.w_up = tensors[self.templates["up"].format(e="*")].view(E, self.inner, self.width)
        self.w_down = tensors[self.templates["down"].format(e="*")].view(E, self.width, self.inner)
        self.correction = tensors[self.correction_name] if self.correction_name else None
        # bfloat16 experts on the GPU are held packed for the matrix cores, the stack as one matrix, where an expert's
        # rows start at a block's border (the rows they came from are not kept)
        self.up_dims = self.down_dims = None
        if self.w_gate.dtype == torch.bfloat16 and self.w_gate.is_cuda:
            if ops.experts_packable(E, self.inner, self.width):
                self.w_gate = ops.pack_matrix(self.w_gate.view(E * self.inner, self.width))
                self.w_up = ops.pack_matrix(self.w_up.view(E * self.inner, self.width))
                self.up_dims = (E, self.inner, self.width)
            if ops.experts_packable(E, self.width, self.inner):
                self.w_down = ops.pack_matrix(self.w_down.view(E * self.width, self.inner))
                self.down_dims = (E, self.width, self.inner)
        self.w_dtype = torch.bfloat16 if isinstance(self.w_gate, ops.PackedMatrix) else self.w_gate.dtype

    def forward(self, h, ctx, accumulate_into):
        T, top, dev = h.shape[0], self.top, h.device
        wdt = self.w_dtype
        if h.dtype != wdt:        # (experts stored in 32-bit in a bfloat16 engine: their products run on widened rows)
            h = ops.cast(h.contiguous(), torch.empty(h.shape, dtype=wdt, device=dev))
        z = self.router(h, out_dtype=torch.float32)
        ids = torch.empty((T, top), dtype=torch.int32, device=dev)
        wts = torch.empty((T, top), dtype=torch.float32, device=dev)
        ops.moe_route(z, self.correction, top, ids, wts)
        offsets = torch.empty(self.n_experts + 1, dtype=torch.int32, device=dev)
        order = torch.empty(T * top, dtype=torch.int32, device=dev)
        ops.moe_plan(ids, self.n_experts, offsets, order)
        y = torch.empty((T * top, self.inner), dtype=wdt, device=dev)
        ops.moe_up(h, order, offsets, top, self.w_gate, self.w_up, self.limit, self.alpha, y, dims=self.up_dims)
        out = torch.empty((T * top, self.width), dtype=torch.float32, device=dev)
        ops.moe_down(y, order, offsets, self.w_down, out, dims=self.down_dims)
        ops.moe_combine(out, wts, accumulate_into)
