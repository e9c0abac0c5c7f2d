"""Feed-forward parts.  Here: the gated MLP  down( act(gate(h)) * up(h) ), dense.

crates/synaptix-models/llm/common/src/model.rs:1670-1691; activation silu(z) = z / (1 + e^-z) in
32-bit as crates/synaptix-kernels-cuda/src/cu/fused/mlp/silu_and_mul.cu:11-52.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.source import TensorSpec
from .base import Part
from .linear import Matrix, linear, linear_for_sum, deferred_product, as_rows, ScaledRows


class FeedForward(Part):
    """Interface: forward(h [N, hidden] activation type, ctx) -> residual delta [N, hidden] float."""

    takes_scaled_rows = False     # as Mixer.takes_scaled_rows

    def forward(self, h, ctx):
        raise NotImplementedError


class GatedMlp(FeedForward):
    takes_scaled_rows = True
    capturable = True

    NAMES = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "silu", names=None):
        """names: the tensors of the gate, up and down products behind `prefix` (default: NAMES)."""
        self.names = tuple(names or self.NAMES)
        try:
            ops.activation_code(activation)       # the kernels apply it by its code; an unknown name is refused here
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.prefix, self.hidden, self.intermediate, self.activation = prefix, hidden, intermediate, activation
        self.w_gate_up = self.w_down = None
        self.paired = False      # gate and up rows in turns of 16: the activation runs inside the product

    def tensor_specs(self):
        p, (gate, up, down) = self.prefix, self.names
        return {
            p + gate: TensorSpec((self.intermediate, self.hidden)),
            p + up: TensorSpec((self.intermediate, self.hidden)),
            p + down: TensorSpec((self.hidden, self.intermediate)),
        }

    def load(self, get):
        p = self.prefix
        gate, up = get(p + self.names[0]), get(p + self.names[1])
        self.paired = (gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                       and self.intermediate % ops.PAIR == 0 and self.hidden % 8 == 0)
        self.w_gate_up = Matrix(ops.pair_rows(gate, up) if self.paired else torch.cat([gate, up], 0))
        self.w_down = Matrix(get(p + self.names[2]))

    def forward(self, h, ctx):
        m = torch.empty((h.shape[0], self.intermediate), dtype=h.dtype, device=h.device)
        if self.paired and h.dtype == torch.bfloat16:
            if self.w_gate_up.packed is not None and h.shape[0] <= ops.PACKED_MAX_ROWS_GATED:
                if isinstance(h, ScaledRows):      # the norm's last step is the product's epilogue
                    ops.gemm_packed(h.rows, self.w_gate_up.packed, m, paired=True, activation=self.activation,
                                    row_scale=h.row_scale)
                else:
                    ops.gemm_packed(h, self.w_gate_up.packed, m, paired=True, activation=self.activation)
            else:
                ops.gemm_swiglu(as_rows(h), self.w_gate_up.data, m, self.activation)
        else:
            h = as_rows(h)
            ops.swiglu(linear(h, self.w_gate_up, h.dtype), m, self.activation)
        return deferred_product(m, self.w_down)


class RoutedExperts(FeedForward):
    """A mixture of small ungated experts: each token goes through the `top` experts whose router logits are largest,

        z = W_router h + b (32-bit sums of the framework's own product);   chosen: the `top` largest z;
        weights: softmax over the chosen logits only
        y = sum_chosen weight_e * W_down[e] act(W_up[e] h)

    The tokens are sorted by expert on the device (no count comes back to the host), and each expert's rows meet its
    matrices in one launch for all experts (ops.experts_product).  Returns the `top` weighted results of every token
    as partial sums [top, N, hidden], which whoever adds the residual sums up.
    Tensors: prefix + "e<j>.up" [ff, hidden], "e<j>.down" [hidden, ff], "router" [experts, hidden], "router.b"."""
    takes_scaled_rows = False
    capturable = True

    ACTIVATIONS = ("gelu",)       # the exact (erf) form, the products' epilogue

    def __init__(self, prefix: str, hidden: int, ff: int, n_experts: int, top: int, activation: str = "gelu",
                 router_bias: bool = True, names=("e{}.up", "e{}.down", "router", "router.b")):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"{prefix}: activation {activation!r} (the experts' products apply {self.ACTIVATIONS})")
        if not 0 < top <= n_experts:
            raise ValueError(f"{prefix}: the {top} largest of {n_experts} experts")
        self.prefix, self.hidden, self.ff, self.n_experts, self.top = prefix, hidden, ff, n_experts, top
        self.router_bias, self.names = bool(router_bias), tuple(names)
        self.w_up = self.w_down = self.w_router = self.b_router = None

    def tensor_specs(self):
        p, (up, down, router, bias) = self.prefix, self.names
        specs = {p + router: TensorSpec((self.n_experts, self.hidden))}
        if self.router_bias:
            specs[p + bias] = TensorSpec((self.n_experts,), "bias")
        for e in range(self.n_experts):
            specs[p + up.format(e)] = TensorSpec((self.ff, self.hidden))
            specs[p + down.format(e)] = TensorSpec((self.hidden, self.ff))
        return specs

    def load(self, get):
        p, (up, down, router, bias) = self.prefix, self.names
        # every expert's matrices kept once: in fragment order where type and sizes allow, else in plain rows
        w_up = torch.stack([get(p + up.format(e)) for e in range(self.n_experts)]).contiguous()
        packed = ops.pack_expert_weights(w_up)
        self.w_up = w_up if packed is None else packed
        del w_up, packed
        w_down = torch.stack([get(p + down.format(e)) for e in range(self.n_experts)]).contiguous()
        packed = ops.pack_expert_weights(w_down)
        self.w_down = w_down if packed is None else packed
        self.w_router = Matrix(get(p + router))
        self.b_router = get(p + bias).float().contiguous() if self.router_bias else None

    def check(self, dtype):
        if self.n_experts > ops.ROUTE_MAX_EXPERTS or self.top > ops.ROUTE_MAX_TOP:
            raise ValueError(f"{self.prefix}: {self.top} of {self.n_experts} experts "
                             f"(at most {ops.ROUTE_MAX_TOP} of {ops.ROUTE_MAX_EXPERTS})")

    def forward(self, h, ctx):
        h = as_rows(h)
        N, dev = h.shape[0], h.device
        ids = torch.empty((N, self.top), dtype=torch.int32, device=dev)
        weights = torch.empty((N, self.top), dtype=torch.float32, device=dev)
        ops.route_topk(linear(h, self.w_router, torch.float32), self.b_router, ids, weights)
        seg, tok_of, pair_of, part_of, weight_of = ops.route_sort(ids, weights, self.n_experts)
        mid = torch.empty((N * self.top, self.ff), dtype=h.dtype, device=dev)
        ops.experts_product(h, self.w_up, mid, seg, tok_of, pair_of, gelu=True)
        y = torch.empty((self.top, N, self.hidden), dtype=torch.float32, device=dev)
        ops.experts_product(mid, self.w_down, y.view(self.top * N, self.hidden), seg, pair_of, part_of,
                            row_weight=weight_of)
        return y
