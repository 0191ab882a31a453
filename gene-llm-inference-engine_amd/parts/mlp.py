"""Gated feed-forward: residual += down( act(gate(h)) * up(h) ); act is SiLU, silu(g) = g / (1 + exp(-g))
(SwiGLU; reference: src/model/transformer.cpp:437-450), or the tanh form of GELU where the spec says so.  gate and up run
as one product with the stacked matrix [gate; up]; in bfloat16 the gate is applied inside that product."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import FeedForward, register_feed_forward
from .linear import activation_dtype_for, linear, linear_onto, takes_handed_norm


class SwiGlu(FeedForward):
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True              # `forward(..., overwrite=True)` stores its result in `residual` instead of adding onto it

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        gate, up = tensors[spec.gate_proj], tensors[spec.up_proj]
        self.w_down = tensors[spec.down_proj]
        self.in_dtype = activation_dtype_for(gate, dtype)
        self.mid_dtype = activation_dtype_for(self.w_down, dtype)
        # bfloat16 throughout: the gate is applied inside the product (weights interleaved for it)
        self.activation = getattr(spec, "activation", "silu")
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"feed-forward: unknown activation {self.activation!r}; known: {', '.join(ops.ACTIVATIONS)}")
        self.limit = float(getattr(spec, "activation_limit", 0.0))
        self.fused = (self.in_dtype == torch.bfloat16 and self.mid_dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                      and spec.intermediate_size % 16 == 0 and spec.hidden_size % 8 == 0 and self.activation in ops.FUSED_GATE_ACTIVATIONS)
        self.w_gate_up = ops.interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], dim=0).contiguous()

    @classmethod
    def tensor_needs(cls, spec):
        i, d = spec.intermediate_size, spec.hidden_size
        return [TensorNeed(spec.gate_proj, (i, d)), TensorNeed(spec.up_proj, (i, d)), TensorNeed(spec.down_proj, (d, i))]

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and ops.gemm_bf16_takes_norm(n_rows, self.w_gate_up.shape[0], self.w_gate_up.shape[1], self.fused)

    def forward(self, h, residual, ctx, then=None, overwrite=False):
        T, inter = ctx.n_rows, self.spec.intermediate_size
        if self.fused:
            mid = torch.empty((T, inter), dtype=torch.bfloat16, device=ctx.device)
            linear(h, self.w_gate_up, mid, gated=self.activation, gate_limit=self.limit)
        else:
            gate_up = torch.empty((T, 2 * inter), dtype=torch.float32, device=ctx.device)
            linear(h, self.w_gate_up, gate_up)
            mid = torch.empty((T, inter), dtype=self.mid_dtype, device=ctx.device)
            ops.act_mul(gate_up, mid, self.activation, self.limit)
        if overwrite:
            linear(mid, self.w_down, residual)
            return None
        return linear_onto(mid, self.w_down, residual, then)


register_feed_forward("swiglu", SwiGlu)


class DenseMlp(FeedForward):
    """residual += down(act(up(h))): no gate.  The activation has parameters of its own (a tensor) and runs in 32-bit on the up
    product's rows, which it stores as the down product reads them."""
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and takes_handed_norm(self.w_up, n_rows)

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        if spec.activation != "xielu":
            raise ValueError(f"feed-forward: unknown activation {spec.activation!r} of a dense feed-forward; known: xielu")
        if spec.activation_params is None:
            raise ValueError("feed-forward: the activation xielu needs its two parameters")
        self.w_up, self.w_down = tensors[spec.up_proj], tensors[spec.down_proj]
        self.params = tensors[spec.activation_params].float().contiguous()
        self.in_dtype = activation_dtype_for(self.w_up, dtype)
        self.mid_dtype = activation_dtype_for(self.w_down, dtype)

    @classmethod
    def tensor_needs(cls, spec):
        i, d = spec.intermediate_size, spec.hidden_size
        return [TensorNeed(spec.up_proj, (i, d)), TensorNeed(spec.down_proj, (d, i)), TensorNeed(spec.activation_params, (2,))]

    def input_weight(self):          # (the first product's matrix, for a block that makes several parts' first products in one)
        return self.w_up

    def use_input_weight(self, view):
        self.w_up = view

    def forward(self, h, residual, ctx, then=None, overwrite=False, projected=None):
        T, inter = ctx.n_rows, self.spec.intermediate_size
        up = projected
        if up is None:
            up = torch.empty((T, inter), dtype=torch.float32, device=ctx.device)
            linear(h, self.w_up, up)
        mid = torch.empty((T, inter), dtype=self.mid_dtype, device=ctx.device)
        ops.xielu(up, mid, self.params)
        if overwrite:
            linear(mid, self.w_down, residual)
            return None
        return linear_onto(mid, self.w_down, residual, then)


register_feed_forward("dense_mlp", DenseMlp)
