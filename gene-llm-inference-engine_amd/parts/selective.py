"""The selective scan as a mixer (`config.spec.SelectiveScanSpec` states the recurrence; the kernels are `csrc/selective.hip`).

One product gives the 32-bit [x | z] of a step's rows.  One kernel takes x through its short convolution (a request's rows
before this step come from its state) and SiLU; one keeps every request's last rows for the next step's convolution (in a step
of single rows the kernel before it does that on its way).  A second product makes [dt | B | C] of the convolved rows, a third
the channels' step sizes from dt (in bfloat16 steps of single rows the scan's kernel makes that one on its way).  One kernel steps the states over every request's rows, in order, from the request's state
slot and back into it, and stores (read-out + D x) * SiLU(z) as the output product reads it.  The step sizes (from the third
product on: bias, softplus), the decays and their exponentials, B, C, the state and the read-out are 32-bit, whatever the
compute dtype.  In bfloat16 a request's long run of rows (a prompt) is cut into chunks that run at once (`ops.ssm_scan`); in
float32 the rows are always taken one after the other, so that the bits do not depend on how a prompt was cut into steps.

A request's state: S [inner][state] and the convolution's last taps - 1 inputs, one run of 32-bit numbers in the slot the
cache manager gives it (zeroed when the request opens).  The runs of rows that belong to one request are found on the
device, so a captured pass may contain the mixer."""
from __future__ import annotations

import torch

from ..cache.needs import StateNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .attention import _pad_rows
from .base import Mixer, register_mixer
from .linear import activation_dtype_for, linear, linear_onto, takes_handed_norm


class SelectiveScan(Mixer):
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True
    out_scale = 1.0                   # multiplies the mixer's result (`set_out_scale`: inside the scan's kernel, before the output product)

    def set_out_scale(self, scale: float) -> bool:
        self.out_scale = float(scale)
        return True

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and takes_handed_norm(self.w_in, n_rows)

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if not 1 <= s.conv_taps <= ops.SSM_MAX_TAPS:
            raise ValueError(f"selective scan: {s.conv_taps} taps are outside what the kernel takes (1 to {ops.SSM_MAX_TAPS})")
        if not 1 <= s.state <= ops.SSM_MAX_STATES:
            raise ValueError(f"selective scan: {s.state} states a channel are outside what the kernel takes (1 to {ops.SSM_MAX_STATES})")
        self.w_in = _pad_rows(tensors[s.in_proj])
        self.w_x = _pad_rows(tensors[s.x_proj])
        self.w_dt = tensors[s.dt_proj]
        self.taps = tensors[s.conv].float().contiguous()
        self.conv_bias = tensors[s.conv_bias].float().contiguous()
        self.dt_bias = tensors[s.dt_bias].float().contiguous()
        self.a_log = tensors[s.a_log].float().contiguous()
        self.d_skip = tensors[s.d_skip].float().contiguous()
        self.w_o = tensors[s.o_proj]
        self.in_dtype = activation_dtype_for(self.w_in, dtype)
        self.low_dtype = activation_dtype_for(self.w_x, dtype)
        self.mid_dtype = activation_dtype_for(self.w_o, dtype)

    def weights_read_per_step(self):
        return [self.w_in, self.w_x, self.w_dt, self.taps, self.conv_bias, self.dt_bias, self.a_log, self.d_skip, self.w_o]

    def input_weight(self):
        return self.w_in

    def use_input_weight(self, view):
        self.w_in = view

    @classmethod
    def tensor_needs(cls, spec):
        s, d = spec, spec.hidden_size
        return [TensorNeed(s.in_proj, (2 * s.inner, d)), TensorNeed(s.conv, (s.inner, s.conv_taps)), TensorNeed(s.conv_bias, (s.inner,)),
                TensorNeed(s.x_proj, (s.dt_rank + 2 * s.state, s.inner)), TensorNeed(s.dt_proj, (s.inner, s.dt_rank)), TensorNeed(s.dt_bias, (s.inner,)),
                TensorNeed(s.a_log, (s.inner, s.state)), TensorNeed(s.d_skip, (s.inner,)), TensorNeed(s.o_proj, (d, s.inner))]

    @classmethod
    def cache_need(cls, spec):
        return StateNeed((ops.ssm_state_floats(spec.inner, spec.state, spec.conv_taps),), torch.float32)

    def forward(self, h, residual, ctx, cache, then=None, overwrite=False, projected=None):
        s, T, dev = self.spec, ctx.n_rows, ctx.device
        inner, N, R = s.inner, s.state, s.dt_rank
        proj = projected
        if proj is None:
            proj = torch.empty((T, self.w_in.shape[0]), dtype=torch.float32, device=dev)
            linear(h, self.w_in, proj)
        pre, z = proj[:, :inner], proj[:, inner:2 * inner]
        seg_start, seg_len = ops.segments(ctx)
        x = torch.empty((T, inner), dtype=torch.float32, device=dev)
        x_low = x if self.low_dtype == torch.float32 else torch.empty((T, inner), dtype=self.low_dtype, device=dev)
        single_rows = ctx.max_seg_len == 1            # (a step's shape, which a captured pass shares with its replays)
        ops.ssm_conv(pre, self.taps, self.conv_bias, ctx.row_slot, ctx.row_pos, cache.state, x, None if x_low is x else x_low, N, move_tail=single_rows)
        if not single_rows:
            ops.ssm_tail(pre, s.conv_taps, seg_start, seg_len, ctx.row_slot, cache.state, inner, N)
        low = torch.empty((T, self.w_x.shape[0]), dtype=torch.float32, device=dev)
        linear(x_low, self.w_x, low)
        mid = torch.empty((T, inner), dtype=self.mid_dtype, device=dev)
        dt_pre = dt_proj = None
        if single_rows and self.mid_dtype == torch.bfloat16 and self.w_dt.dtype == torch.bfloat16:
            dt_proj = (self.w_dt, 0)                    # (a step of single rows: the scan's kernel makes the step sizes' product on its way)
        else:
            dt_pre = torch.empty((T, inner), dtype=torch.float32, device=dev)
            linear(low[:, :R], self.w_dt, dt_pre)       # (32-bit rows: the step sizes' product keeps them)
        ops.ssm_scan(x, dt_pre, self.dt_bias, low, R, R + N, z, self.a_log, self.d_skip, seg_start, seg_len, ctx.row_slot, cache.state, mid, N,
                     rows_per_request=ctx.seg_len, out_scale=self.out_scale, dt_proj=dt_proj)
        if overwrite:
            linear(mid, self.w_o, residual)
            return None
        return linear_onto(mid, self.w_o, residual, then)


register_mixer("selective_scan", SelectiveScan)
