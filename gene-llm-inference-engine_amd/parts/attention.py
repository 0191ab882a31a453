"""Causal attention with grouped key/value heads over the paged cache (optionally windowed).

Order of operations as the reference's pass (src/gpu/gpu_transformer.cpp:390-409): q, k, v
products; rotation of q and k; all new keys and values are written to their pages; then every
row attends over its request's pages up to its own position; output product added onto the
residual.  The three input products run as one with the stacked matrix [q; k; v].

The position encoding is a part of its own (`spec.position`).  One that turns the pairs
(i, i + head_dim/2) of whole heads hands over its cosines and sines, and the kernel that writes the
pages (or, for a few decoded rows, the attention kernel itself) applies them; any other encoding
changes q and k in place with its own kernels first, and the pages are then written unrotated."""
from __future__ import annotations

import torch

from ..cache.needs import PagedKvNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import Mixer, PositionEncoding, position_class, register_mixer
from .linear import activation_dtype_for, linear, linear_onto, takes_handed_norm
from .norm import HandedRows, NormedRows
from .rope import rotation_tables


def qkv_rotate_store_attend(h, w_qkv, ctx, cache, *, n_heads, n_kv_heads, head_dim, position=None, window=None, in_dtype=None,
                            before_rotation=None):
    """The front half of an attention-like mixer, for any mixer to call: the product with the stacked matrix [q; k; v], the
    position encoding on queries and keys, the new keys and values into the entry's pages, and every row's attention over its
    request's pages up to its own position.  Returns the heads' outputs [rows, n_heads*head_dim] in the cache's dtype.

    h                the mixer's input: rows, or a norm not yet (or half) applied, as `linear` takes it
    position         a `PositionEncoding` or None; one with `half_split_tables` is applied by the kernels that store and attend
    before_rotation  `f(q, k)`: changes the 32-bit products in place before the rotation (a norm or a scale per head; k is None
                     where the pages are another entry's).  With it the products are always written out in 32-bit; the kernels
                     that rotate, store and attend from them still serve.
    Which kernels serve is decided here by storage and shape alone: for some tens of rows and for the rows of prompts the
    product's own last step rotates and fills the pages; for a few decoded rows one kernel rotates, stores and attends;
    otherwise product, rotation + store and attention are three launches."""
    T, a_dim, kv_dim = ctx.n_rows, n_heads * head_dim, n_kv_heads * head_dim
    in_dtype = in_dtype if in_dtype is not None else activation_dtype_for(w_qkv, ctx.dtype)
    tables = position.half_split_tables(ctx) if position is not None else None
    cos, sin = tables if tables is not None else (None, None)
    att = torch.empty((T, a_dim), dtype=cache.kv.dtype, device=ctx.device)
    if (before_rotation is None and cache.writes and (tables is not None or position is None) and w_qkv.dtype == torch.bfloat16
            and cache.kv.dtype == torch.bfloat16 and in_dtype == torch.bfloat16
            and ops.gemm_bf16_qkv_rope_store_takes(T, w_qkv.shape[0], w_qkv.shape[1], head_dim)):
        # the product's own last step (the kernel that adds up the shares of k, or the epilogue over a tile) rotates and writes the pages
        # (this product finishes a norm handed on at every number of rows it is taken at, if the pieces are few enough)
        if (isinstance(h, HandedRows) and h.scaled.stride(0) % 8 == 0 and h.scaled.data_ptr() % 16 == 0
                and h.squares.shape[1] <= ops.gemm_bf16_qkv_rope_store_max_parts(T, w_qkv.shape[0], w_qkv.shape[1])):
            rows, norm_in = h.scaled, (h.squares, h.eps)
        else:
            rows, norm_in = (h.materialize() if isinstance(h, NormedRows) else h), None
        if ops.gemm_bf16_supports(rows, w_qkv, att):
            q_rot = torch.empty((T, a_dim), dtype=torch.bfloat16, device=ctx.device)
            ops.gemm_bf16_qkv_rope_store(rows, w_qkv, cos, sin, ctx.row_pos, ctx.row_slot, cache.table, q_rot, cache.kv, n_heads, n_kv_heads,
                                         head_dim, norm_in)
            return ops.attention(q_rot, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window)
        if norm_in is None:
            h = rows                  # (whole rows: what `linear` below would make of h)
    if cache.writes:
        qkv = torch.empty((T, a_dim + 2 * kv_dim), dtype=torch.float32, device=ctx.device)
        linear(h, w_qkv, qkv)
        q, k, v = qkv[:, :a_dim], qkv[:, a_dim:a_dim + kv_dim], qkv[:, a_dim + kv_dim:]
    else:                       # the pages are another layer's: only the queries are made
        q, k, v = torch.empty((T, a_dim), dtype=torch.float32, device=ctx.device), None, None
        linear(h, w_qkv[:a_dim], q)
    if before_rotation is not None:
        before_rotation(q, k)
    if position is not None and tables is None:          # an encoding with kernels of its own: q and k are turned in place
        position.apply(q, k, ctx, n_heads, n_kv_heads, head_dim)
    # a step of single decoded rows: one kernel rotates, writes the pages and attends
    if not ops.attention_from_products(q, k, v, cos, sin, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window):
        q_rot = torch.empty((T, a_dim), dtype=cache.kv.dtype, device=ctx.device)
        ops.rope_store(q, k, v, cos, sin, ctx.row_pos, ctx.row_slot, cache.table, q_rot, cache.kv, n_heads, n_kv_heads, head_dim)
        ops.attention(q_rot, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window)
    return att


def _pad_rows(w, multiple=16):
    """The stacked matrix with rows of zeros behind it up to a multiple of `multiple` (so that the product's 32-bit rows start at
    multiples of 16 bytes)."""
    extra = -w.shape[0] % multiple
    return w if not extra else torch.cat([w, torch.zeros((extra, w.shape[1]), dtype=w.dtype, device=w.device)], dim=0).contiguous()


class Attention(Mixer):
    """Plain (Llama) attention takes the kernels chosen in `qkv_rotate_store_attend`.  A spec that names any of the further
    features (value heads of another size, a scale of its own, a mask cut into chunks, sinks, norms on query and key heads or over
    the whole projections, a gate per head, a rotation of a part of the head, capped scores) takes the general path: one product with [q; k; v; head gates], one kernel
    that norms, turns and stores, and the attention kernel that knows all of these."""
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next
    can_overwrite = True              # `forward(..., overwrite=True)` stores its result in `residual` instead of adding onto it

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError("the number of heads must be a multiple of the number of key/value heads")
        if not 0 < s.head_dim <= ops.attention_max_head_size():
            raise ValueError(f"attention: head_dim = {s.head_dim} is outside what the attention kernels take (1 to {ops.attention_max_head_size()} channels a head)")
        self.a_dim, self.kv_dim = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim
        self.value_dim = s.value_dim or s.head_dim
        self.general = self._is_general(s)
        self.position = None if s.position is None else position_class(s.position)(s.position, tensors, dtype, device)
        if not 0 < self.value_dim <= ops.attention_max_head_size():
            raise ValueError(f"attention: value heads of {self.value_dim} channels are outside what the attention kernels take")
        if self.general:
            stacked = [tensors[s.q_proj]] + ([tensors[s.k_proj], tensors[s.v_proj]] if s.k_proj is not None else [])
            self.gate_at = sum(w.shape[0] for w in stacked)
            if s.head_gate is not None:
                stacked.append(tensors[s.head_gate])
            self.w_qkv = _pad_rows(torch.cat(stacked, dim=0).contiguous())
            self.sinks = None if s.sinks is None else tensors[s.sinks].float().contiguous()
            self.q_norm = None if s.q_norm is None else tensors[s.q_norm]
            self.k_norm = None if s.k_norm is None else tensors[s.k_norm]
            as_f32 = lambda name: None if name is None else tensors[name].float().contiguous()
            self.biases = (as_f32(s.q_bias), as_f32(s.k_bias), as_f32(s.v_bias))
            self.value_blend = None if s.value_blend is None else tensors[s.value_blend].float().reshape(1).contiguous()
            if s.value_blend is not None and s.value_family is None:
                raise ValueError("attention: a blend of values needs the family whose first layer's values are blended in")
            self.unit_rms = bool(getattr(s, "qk_unit_rms", False))
            self.norm_whole = bool(getattr(s, "qk_norm_whole", False))
            if self.norm_whole and (self.q_norm is None or (self.k_norm is None and s.k_proj is not None)):
                raise ValueError("attention: a norm over the whole query and key projections needs its weights")
            self.score_cap = getattr(s, "score_cap", None)
            if self.score_cap is not None and not self.score_cap > 0:
                raise ValueError("attention: the scores' cap must be positive")
            if self.unit_rms and (self.q_norm is not None or self.k_norm is not None):
                raise ValueError("attention: heads divided by their root mean square have no norm weights")
            if self.position is not None and hasattr(self.position, "pair_tables") and self.position.rotary_dim > s.head_dim:
                raise ValueError("attention: more channels to turn than a head has")
            if self.position is not None and not (hasattr(self.position, "partial_tables") or hasattr(self.position, "pair_tables")
                                                  or type(self.position).half_split_tables is not PositionEncoding.half_split_tables):
                if self.q_norm is not None or self.k_norm is not None or self.unit_rms:
                    raise ValueError("attention: norms on query and key heads come before the rotation, which needs a position encoding that hands over its cosines and sines")
        else:
            self.w_qkv = torch.cat([tensors[s.q_proj], tensors[s.k_proj], tensors[s.v_proj]], dim=0).contiguous()
        self.w_o = tensors[s.o_proj]
        self.in_dtype = activation_dtype_for(self.w_qkv, dtype)
        self.att_dtype = activation_dtype_for(self.w_o, dtype)
        self.graph_safe = self.position is None or bool(getattr(self.position, "graph_safe", False))

    @staticmethod
    def _is_general(s) -> bool:
        return (s.k_proj is None or any(v is not None for v in (s.value_dim, s.scale, s.chunk, s.sinks, s.q_norm, s.k_norm, s.head_gate, s.q_bias,
                                                                 s.k_bias, s.v_bias, s.value_family, s.value_blend, getattr(s, "score_cap", None)))
                or getattr(s, "qk_unit_rms", False) or getattr(s.position, "kind", None) in ("rotary_partial", "rotary_interleaved"))

    @classmethod
    def tensor_needs(cls, spec):
        a, kv, d, vd = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim, spec.hidden_size, spec.value_dim or spec.head_dim
        needs = [TensorNeed(spec.q_proj, (a, d))]
        if spec.k_proj is not None:            # (a layer that reads another layer's pages has no keys and values of its own)
            needs += [TensorNeed(spec.k_proj, (kv, d)), TensorNeed(spec.v_proj, (spec.n_kv_heads * vd, d))]
        needs.append(TensorNeed(spec.o_proj, (d, spec.n_heads * vd)))
        whole = getattr(spec, "qk_norm_whole", False)          # one norm over all heads of a projection, with a weight per channel of all heads
        if spec.q_norm is not None:
            needs.append(TensorNeed(spec.q_norm, (a if whole else spec.head_dim,), "norm"))
        if spec.k_norm is not None and spec.k_proj is not None:
            needs.append(TensorNeed(spec.k_norm, (kv if whole else spec.head_dim,), "norm"))
        if spec.sinks is not None:
            needs.append(TensorNeed(spec.sinks, (spec.n_heads,)))
        if spec.head_gate is not None:
            needs.append(TensorNeed(spec.head_gate, (spec.n_heads, d)))
        if spec.q_bias is not None:
            needs.append(TensorNeed(spec.q_bias, (a,)))
        if spec.k_proj is not None:
            if spec.k_bias is not None:
                needs.append(TensorNeed(spec.k_bias, (kv,)))
            if spec.v_bias is not None:
                needs.append(TensorNeed(spec.v_bias, (spec.n_kv_heads * vd,)))
            if spec.value_blend is not None:
                needs.append(TensorNeed(spec.value_blend, ()))
        return needs

    @classmethod
    def cache_need(cls, spec):
        return PagedKvNeed(spec.n_kv_heads, spec.head_dim, spec.window, None if spec.value_dim in (None, spec.head_dim) else spec.value_dim, spec.keep_chunk)

    def takes_handed_norm(self, n_rows: int) -> bool:
        if self.in_dtype == torch.bfloat16 and self.general:          # (the general path's one product goes through `linear`)
            return takes_handed_norm(self.w_qkv, n_rows)
        if self.in_dtype != torch.bfloat16:
            return False
        if ops.gemm_bf16_takes_norm(n_rows, self.w_qkv.shape[0], self.w_qkv.shape[1]):
            return True
        # the rows of prompts: the q/k/v product that rotates and fills the pages itself finishes the norm, where it serves
        half_split = self.position is None or getattr(type(self.position), "half_split_tables", None) is not PositionEncoding.half_split_tables
        return half_split and ops.gemm_bf16_qkv_rope_store_takes(n_rows, self.w_qkv.shape[0], self.w_qkv.shape[1], self.spec.head_dim)

    def _attend_general(self, h, ctx, cache, projected=None):
        """The heads' outputs [rows, heads * value_dim] by the general path."""
        s, T, vd = self.spec, ctx.n_rows, self.value_dim
        proj = projected
        if proj is None:
            proj = torch.empty((T, self.w_qkv.shape[0]), dtype=torch.float32, device=ctx.device)
            linear(h, self.w_qkv, proj)
        q, k, v = proj[:, :self.a_dim], None, None
        if s.k_proj is not None and cache.writes:
            k, v = proj[:, self.a_dim:self.a_dim + self.kv_dim], proj[:, self.a_dim + self.kv_dim:self.a_dim + self.kv_dim + s.n_kv_heads * vd]
        gate = proj[:, self.gate_at:self.gate_at + s.n_heads] if s.head_gate is not None else None
        neighbours = self.position is not None and hasattr(self.position, "pair_tables")          # pairs (2i, 2i + 1) of a head's first channels
        tables = (*self.position.pair_tables(ctx), self.position.rotary_dim) if neighbours else rotation_tables(self.position, ctx)
        if self.position is not None and tables is None:          # an encoding with kernels of its own turns q and k in place
            self.position.apply(q, k, ctx, s.n_heads, s.n_kv_heads, s.head_dim)
        cos, sin, turned = tables if tables is not None else (None, None, 0)
        q_ready = torch.empty((T, self.a_dim), dtype=cache.kv.dtype, device=ctx.device)
        blend = keep = None
        if s.value_family is not None and k is not None:
            family = ("value_family", s.value_family)
            if self.value_blend is None:          # the family's first layer: its values stay for the others
                keep = ctx.memo[family] = torch.empty((T, s.n_kv_heads * vd), dtype=torch.float32, device=ctx.device)
            else:
                if family not in ctx.memo:
                    raise RuntimeError(f"attention: no earlier layer of this pass has left the values of family {s.value_family!r}")
                blend = (ctx.memo[family], self.value_blend)
        biases = self.biases if k is not None else (self.biases[0], None, None)
        ops.norm_rope_store(q, k, v, self.q_norm, self.k_norm if k is not None else None, s.qk_norm_eps, cos, sin, turned, ctx.row_pos, ctx.row_slot,
                            cache.table, q_ready, cache.kv, cache.page_size, s.n_heads, s.n_kv_heads, s.head_dim, vd,
                            biases=biases if any(b is not None for b in biases) else None, blend=blend, keep=keep, neighbours=neighbours,
                            unit_rms=self.unit_rms, norm_last=self.unit_rms, v_scale=self.out_scale, norm_all=self.norm_whole)
        att = torch.empty((T, s.n_heads * vd), dtype=cache.kv.dtype, device=ctx.device)
        return ops.attention_general(q_ready, cache.kv, att, ctx, cache.table, s.n_heads, s.n_kv_heads, s.head_dim, page_size=cache.page_size,
                                     value_dim=vd, window=s.window, chunk=s.chunk, scale=s.scale, sinks=self.sinks, gate=gate, cap=self.score_cap)

    out_scale = 1.0

    def set_out_scale(self, scale: float) -> bool:
        """Multiplies the mixer's result by `scale`, where that costs nothing: the general path's values are weighed on their way into
        the layer's own pages (the attention is linear in them).  False: the caller weighs the result itself.  (Another layer that
        reads these pages would read the weighed values: a layer whose pages are shared is not asked.)"""
        s = self.spec
        if not (self.general and s.k_proj is not None and s.value_family is None and s.head_gate is None):
            return False
        self.out_scale = float(scale)
        return True

    def input_weight(self):
        """The first product's matrix, for a block that makes several parts' first products in one; None where the plain path's
        kernels make that product themselves."""
        return self.w_qkv if self.general and self.spec.k_proj is not None else None

    def use_input_weight(self, view):
        self.w_qkv = view

    def forward(self, h, residual, ctx, cache, then=None, overwrite=False, projected=None):
        s = self.spec
        if self.general:
            att = self._attend_general(h, ctx, cache, projected if cache.writes else None)
            if att.dtype != self.att_dtype:
                att = att.to(self.att_dtype)
            if overwrite:
                linear(att, self.w_o, residual)
                return None
            return linear_onto(att, self.w_o, residual, then)
        if overwrite:
            residual.zero_()
        att = qkv_rotate_store_attend(h, self.w_qkv, ctx, cache, n_heads=s.n_heads, n_kv_heads=s.n_kv_heads, head_dim=s.head_dim,
                                      position=self.position, window=s.window, in_dtype=self.in_dtype)
        if att.dtype != self.att_dtype:
            att = att.to(self.att_dtype)
        return linear_onto(att, self.w_o, residual, then)


register_mixer("attention", Attention)
