"""Attention through low-rank latents (`config.spec.LatentAttentionSpec` states the layer; the kernels between the products are
`csrc/latent.hip`).

What is cached per position is the normed key/value latent c [kv_rank] and one rotated key part [rotary_dim], nothing per
head.  The up projections are folded into the two sides of the attention instead of being applied to cached rows:
    score_j = (W_uk_h^T q_plain_h) . c_j + q_rot_h . k_rot_j        o_h = W_uv_h (sum_j p_j c_j)
so the attention kernel sees one key/value head, shared by all query heads, with keys [c; k_rot] of kv_rank + rotary_dim
channels and values c of kv_rank channels, and every step costs the same few products whatever the context holds.  The pages
are those of any layer whose values are shorter than its keys (the latent lies in them twice: as part of the key, and as the
value with the places innermost, which is how the kernels' second product reads it).

Steps of a pass: one product with [W_dq; W_dkv]; one kernel that norms both latents, turns the rotated key part and writes the
page; the product with W_uq; one kernel that parts every head's query into plain channels (rows for the folding product) and
turned channels (written where the attention reads them); the folding product with every head's W_uk_h^T; attention (in
bfloat16 on the matrix cores: 16 heads are the columns of one matrix instruction, for a single decoded row too); the product
with every head's W_uv_h; the output product onto the residual."""
from __future__ import annotations

import torch

from ..cache.needs import PagedKvNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .attention import _pad_rows
from .base import Mixer, position_class, register_mixer
from .linear import activation_dtype_for, linear, linear_onto, takes_handed_norm


def _head_product(a, w, out):
    """out = a @ w.T for one head's columns of wider rows: by `linear` where the matrix-core kernels' stores find their
    alignment in the view, by the exact kernel otherwise."""
    if out.data_ptr() % 16 or (out.stride(0) * out.element_size()) % 16 or a.data_ptr() % 16:
        return ops.gemm_exact(a, w, out)
    return linear(a, w, out)


def heads_product(a, w, out, n_heads, out_head_stride=None):
    """out[:, h*stride : h*stride + n] = a[:, h*k : (h+1)*k] @ w[h].T for every head: one launch in bfloat16, head by head otherwise."""
    k, n = w.shape[2], w.shape[1]
    stride = out_head_stride or n
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and ops.heads_product(a, w, out, n_heads, stride):
        return out
    for i in range(n_heads):
        _head_product(a[:, i * k:(i + 1) * k], w[i], out[:, i * stride:i * stride + n])
    return out


class LatentAttention(Mixer):
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and takes_handed_norm(self.w_down, n_rows)

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        self.key_dim = s.kv_rank + s.rotary_dim
        if not 0 < self.key_dim <= ops.attention_max_head_size():
            raise ValueError(f"latent attention: kv_rank + rotary_dim = {self.key_dim} is outside what the attention kernels take (up to {ops.attention_max_head_size()})")
        if s.rotary_dim % 2:
            raise ValueError("latent attention: the rotated channels come in pairs")
        self.position = None
        if s.rotary_dim:
            if s.position is None:
                raise ValueError("latent attention: rotated channels need a position encoding")
            self.position = position_class(s.position)(s.position, tensors, dtype, device)
            if not hasattr(self.position, "pair_tables") or s.position.rotary_dim != s.rotary_dim:
                raise ValueError("latent attention: the position encoding must give angles for rotary_dim / 2 neighbouring pairs")
        # one product for both latents and, where every head's output has a gate, the gates' logits behind them
        self.gate_at = s.q_rank + s.kv_rank + s.rotary_dim
        gates = [tensors[s.head_gate]] if getattr(s, "head_gate", None) is not None else []
        self.gated = bool(gates)
        self.w_down = _pad_rows(torch.cat([tensors[s.dq_proj], tensors[s.dkv_proj], *gates], dim=0).contiguous())
        self.q_norm, self.kv_norm = tensors[s.dq_norm], tensors[s.dkv_norm]
        self.w_uq = tensors[s.uq_proj]
        # per head: W_uk_h^T [kv_rank, head_dim] (folded into the queries) and W_uv_h [value_dim, kv_rank] (applied to the attended latent)
        self.w_uk_t = tensors[s.uk_proj].view(s.n_heads, s.head_dim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[s.uv_proj].view(s.n_heads, s.value_dim, s.kv_rank).contiguous()
        self.w_o = tensors[s.o_proj]
        self.in_dtype = activation_dtype_for(self.w_down, dtype)
        self.cq_dtype = activation_dtype_for(self.w_uq, dtype)
        self.plain_dtype = activation_dtype_for(self.w_uk_t, dtype)
        self.att_dtype = activation_dtype_for(self.w_o, dtype)
        self.graph_safe = self.position is None or bool(getattr(self.position, "graph_safe", False))
        if dtype == torch.bfloat16 and torch.device(device).type == "cuda":
            ops.latent_attention_prepare()

    def weights_read_per_step(self):
        return [self.w_down, self.q_norm, self.kv_norm, self.w_uq, self.w_uk_t, self.w_uv, self.w_o]

    def input_weight(self):          # (see `GatedDelta.input_weight`)
        return self.w_down

    def use_input_weight(self, view):
        self.w_down = view

    @classmethod
    def tensor_needs(cls, spec):
        s, d = spec, spec.hidden_size
        return [TensorNeed(s.dq_proj, (s.q_rank, d)), TensorNeed(s.dq_norm, (s.q_rank,), "norm"), TensorNeed(s.uq_proj, (s.n_heads * (s.head_dim + s.rotary_dim), s.q_rank)),
                TensorNeed(s.dkv_proj, (s.kv_rank + s.rotary_dim, d)), TensorNeed(s.dkv_norm, (s.kv_rank,), "norm"),
                TensorNeed(s.uk_proj, (s.n_heads * s.head_dim, s.kv_rank)), TensorNeed(s.uv_proj, (s.n_heads * s.value_dim, s.kv_rank)),
                TensorNeed(s.o_proj, (d, s.n_heads * s.value_dim))] + ([TensorNeed(s.head_gate, (s.n_heads, d))] if getattr(s, "head_gate", None) is not None else [])

    @classmethod
    def cache_need(cls, spec):
        return PagedKvNeed(1, spec.kv_rank + spec.rotary_dim, spec.window, spec.kv_rank, None)

    def forward(self, h, residual, ctx, cache, then=None, overwrite=False, projected=None):
        s, T, dev = self.spec, ctx.n_rows, ctx.device
        H, kd = s.n_heads, self.key_dim
        down = projected
        if down is None:
            down = torch.empty((T, self.w_down.shape[0]), dtype=torch.float32, device=dev)
            linear(h, self.w_down, down)
        cos, sin = self.position.pair_tables(ctx) if self.position is not None else (None, None)
        cq = torch.empty((T, s.q_rank), dtype=self.cq_dtype, device=dev)
        ops.latent_prepare(down, s.q_rank, s.kv_rank, s.rotary_dim, self.q_norm, self.kv_norm, s.norm_eps, cos, sin, ctx.row_pos, ctx.row_slot,
                           cache.table, cq, cache.kv, cache.page_size)
        q = torch.empty((T, H * (s.head_dim + s.rotary_dim)), dtype=torch.float32, device=dev)
        linear(cq, self.w_uq, q)
        plain = torch.empty((T, H * s.head_dim), dtype=self.plain_dtype, device=dev)
        folded = torch.empty((T, H * kd), dtype=cache.kv.dtype, device=dev)
        ops.latent_queries(q, cos, sin, plain, folded, H, s.head_dim, s.rotary_dim, s.kv_rank)
        heads_product(plain, self.w_uk_t, folded, H, kd)
        attended = torch.empty((T, H * s.kv_rank), dtype=cache.kv.dtype, device=dev)
        if cache.kv.dtype == torch.bfloat16 and ops.latent_attention_bf16_supports(kd, s.kv_rank, cache.page_size):
            ops.latent_attention_bf16(folded, cache.kv, attended, ctx, cache.table, H, kd, s.kv_rank, cache.page_size, s.window, s.scale)
        else:
            ops.attention_general(folded, cache.kv, attended, ctx, cache.table, H, 1, kd, page_size=cache.page_size, value_dim=s.kv_rank,
                                  window=s.window, scale=s.scale)
        if attended.dtype != activation_dtype_for(self.w_uv, self.dtype):
            attended = attended.to(activation_dtype_for(self.w_uv, self.dtype))
        att = torch.empty((T, H * s.value_dim), dtype=self.att_dtype, device=dev)
        heads_product(attended, self.w_uv, att, H)
        if self.gated:
            ops.head_gate(att, down[:, self.gate_at:self.gate_at + H], H, s.value_dim)
        if overwrite:
            linear(att, self.w_o, residual)
            return None
        return linear_onto(att, self.w_o, residual, then)


register_mixer("latent_attention", LatentAttention)
