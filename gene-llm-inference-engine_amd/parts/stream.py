"""Parts that change the residual stream between layers (`StreamPart`): a second input from the token itself behind a layer
(`config.spec.TokenSideInputSpec`), and the stream mixed with the token rows again before a run-order entry
(`config.spec.RejoinSpec`).  The residual stream stays 32-bit; what goes into a product is stored as the compute dtype stores
a product's rows."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import StreamPart, norm_class, register_stream_part
from .linear import activation_dtype_for, linear


class TokenSideInput(StreamPart):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if s.activation not in ops.ACTIVATIONS:
            raise ValueError(f"token side input: unknown activation {s.activation!r}; known: {', '.join(ops.ACTIVATIONS)}")
        if not 0 <= s.first_column <= s.table_width - s.dim:
            raise ValueError("token side input: the columns asked for lie outside the table")
        self.table, self.w_gate, self.w_out = tensors[s.table], tensors[s.gate_proj], tensors[s.out_proj]
        self.norm = norm_class(s.norm)(s.norm, tensors, dtype, device)
        if not hasattr(self.norm, "add_onto"):
            raise ValueError("token side input: the norm must be one that can add its result onto rows")
        self.in_dtype = activation_dtype_for(self.w_gate, dtype)
        self.mid_dtype = activation_dtype_for(self.w_out, dtype)

    @classmethod
    def tensor_needs(cls, spec):
        s = spec
        return ([TensorNeed(s.table, (s.vocab_size, s.table_width)), TensorNeed(s.gate_proj, (s.dim, s.hidden_size)), TensorNeed(s.out_proj, (s.hidden_size, s.dim))]
                + norm_class(s.norm).tensor_needs(s.norm))

    def weights_read_per_step(self):
        return [self.w_gate, self.w_out, self.norm]

    FEW_ROWS = 16      # up to so many rows (bfloat16) the stream's rounding, the first product and the gate are one kernel

    def forward(self, x, ctx):
        s, T, dev = self.spec, ctx.n_rows, ctx.device
        if (T <= self.FEW_ROWS and self.in_dtype == torch.bfloat16 and self.w_gate.dtype == self.table.dtype == self.mid_dtype == torch.bfloat16):
            g = torch.empty((T, s.dim), dtype=torch.bfloat16, device=dev)
            ops.gate_token_columns_rows(x, self.w_gate, self.table, s.first_column, ctx.tokens, g, s.activation)
            y = torch.empty((T, s.hidden_size), dtype=torch.float32, device=dev)
            linear(g, self.w_out, y)
            self.norm.add_onto(y, x)
            return
        rows = x if self.in_dtype == torch.float32 else ops.concat_rows(x, None, torch.empty((T, s.hidden_size), dtype=self.in_dtype, device=dev))
        u = torch.empty((T, s.dim), dtype=torch.float32, device=dev)
        linear(rows, self.w_gate, u)
        g = torch.empty((T, s.dim), dtype=self.mid_dtype, device=dev)
        ops.gate_token_columns(u, self.table, s.first_column, ctx.tokens, g, s.activation)
        y = torch.empty((T, s.hidden_size), dtype=torch.float32, device=dev)
        linear(g, self.w_out, y)
        self.norm.add_onto(y, x)


class Rejoin(StreamPart):
    graph_safe = True
    needs_token_rows = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.weight = tensors[spec.weight]
        self.offset = None if spec.offsets is None else tensors[spec.offsets][spec.row].contiguous()
        self.in_dtype = activation_dtype_for(self.weight, dtype)

    @classmethod
    def tensor_needs(cls, spec):
        needs = [TensorNeed(spec.weight, (spec.hidden_size, 2 * spec.hidden_size))]
        if spec.offsets is not None:
            if not 0 <= spec.row < spec.offsets_rows:
                raise ValueError("rejoin: the row of offsets asked for does not exist")
            needs.append(TensorNeed(spec.offsets, (spec.offsets_rows, spec.hidden_size)))
        return needs

    def weights_read_per_step(self):
        return [self.weight] + ([self.offset] if self.offset is not None else [])

    def forward(self, x, ctx):
        T, d = x.shape
        both = ops.concat_rows(x, ctx.memo["token_rows"], torch.empty((T, 2 * d), dtype=self.in_dtype, device=ctx.device))
        linear(both, self.weight, x)                   # (x is free to be overwritten: `both` holds what the product reads)
        if self.offset is not None:
            ops.add_vector(x, self.offset)


register_stream_part("token_side_input", TokenSideInput)
register_stream_part("rejoin", Rejoin)
