"""Layers over several copies of the residual stream, and the blend of a mixer's input with the input of the token before.

"multistream" block (`LayerSpec.block`): the model carries n copies x_0 .. x_(n-1) of the residual stream side by side in a row
(float32 [T, n * hidden]; `ModelSpec.n_streams`).  Each half of the layer (mixer, feed-forward), with its `StreamAccessSpec`:
    u = sum_s read[s] x_s;   y = half(norm(u));   x_t <- sum_s mix[s, t] x_s + c * write[t] * y   (all copies from the old ones)
with c the layer's `residual_scale`.  A half without such a spec (one copy only) is x <- x + c * half(norm(x)).  A half's result
lies in rows of its own (32-bit) on its way into the copies.

`TokenShift` (a mixer around a mixer, `TokenShiftSpec`): what the inner mixer reads is h + (h_before - h) * w, with h_before the
row the request's token before brought (before its own blending; zeros at position 0).  The last row's h of every request is
kept in a state slot beside the inner mixer's cache, so the blend goes on across steps however a prompt is cut.  Under any block
it takes the normed rows in 32-bit, blends and hands them on; the multistream block, when its norm is an RMS norm, makes the
copies' sum, the norm and the blend in one kernel and calls the inner mixer itself.

Everything here is read from the device (positions and slots of the rows), so a pass may be captured; the one thing taken from
the host is whether every request of the step brings a single row, which is the step's shape."""
from __future__ import annotations

import torch

from ..cache.needs import JointNeed, StateNeed, paged_need, state_need
from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import LayerCache, Mixer, feed_forward_class, mixer_class, norm_class, register_block, register_mixer
from .norm import NormedRows, RmsNorm


def _blend(x, n_streams, out, ctx, *, read, norm_weight, eps, shift, state):
    """out = the blended, normed sum of the copies (see `ops.streams_norm_shift`), the requests' slots of `state` brought up to date."""
    if shift is None:
        return ops.streams_norm_shift(x, n_streams, out, read=read, norm_weight=norm_weight, eps=eps)
    common = dict(read=read, norm_weight=norm_weight, eps=eps, shift=shift, state=state, positions=ctx.row_pos, slots=ctx.row_slot)
    if ctx.max_seg_len == 1:                  # a row reads its slot before it writes it
        return ops.streams_norm_shift(x, n_streams, out, mode=3, **common)
    ops.streams_norm_shift(x, n_streams, out, mode=1, **common)       # a portion's first row reads the slot its last row writes: two launches
    ops.streams_norm_shift(x, n_streams, out, mode=2, **common)
    return out


class TokenShift(Mixer):
    in_dtype = torch.float32          # the normed rows come in 32-bit: the blend is made of them before anything is rounded

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.inner = mixer_class(spec.inner)(spec.inner, tensors, dtype, device)
        self.can_overwrite = bool(getattr(self.inner, "can_overwrite", False))
        self.weight = tensors[spec.weight].float().contiguous()
        self.inner_in_dtype = getattr(self.inner, "in_dtype", dtype)
        self.graph_safe = bool(getattr(self.inner, "graph_safe", False))
        self._inner_need = mixer_class(spec.inner).cache_need(spec.inner)

    @classmethod
    def tensor_needs(cls, spec):
        return [TensorNeed(spec.weight, (spec.hidden_size,))] + mixer_class(spec.inner).tensor_needs(spec.inner)

    @classmethod
    def cache_need(cls, spec):
        inner = mixer_class(spec.inner).cache_need(spec.inner)
        if state_need(inner) is not None:
            raise ValueError("token shift: the mixer inside keeps a fixed-size state of its own; one state per layer is served")
        return JointNeed(paged_need(inner), StateNeed((spec.hidden_size,), torch.float32))

    def pages_are_shared(self):
        shared = getattr(self.inner, "pages_are_shared", None)
        if shared is not None:
            shared()

    def weights_read_per_step(self):
        return [self.weight, self.inner]

    def inner_cache(self, cache: LayerCache) -> LayerCache:
        if paged_need(self._inner_need) is None:
            return LayerCache()
        return LayerCache(kv=cache.kv, page_size=cache.page_size, table=cache.table, writes=cache.writes)

    def forward(self, h, residual, ctx, cache, overwrite=False, **told):
        rows = h.materialize() if isinstance(h, NormedRows) else h
        if rows.dtype != torch.float32:
            raise ValueError("token shift: the rows to blend must be 32-bit")
        blended = torch.empty(rows.shape, dtype=self.inner_in_dtype, device=rows.device)
        _blend(rows, 1, blended, ctx, read=None, norm_weight=None, eps=0.0, shift=self.weight, state=cache.state)
        kw = dict(told)
        if overwrite:
            kw["overwrite"] = True
        return self.inner.forward(blended, residual, ctx, self.inner_cache(cache), **kw)


register_mixer("token_shift", TokenShift)


class _Access:
    """One half's weights on the copies, in 32-bit on the device."""

    def __init__(self, spec, tensors, n_streams):
        if spec is None:
            if n_streams != 1:
                raise ValueError(f"a layer over {n_streams} copies of the residual stream must say how each half reads and writes them")
            self.read = self.write = self.mix = None
            return
        if spec.n_streams != n_streams:
            raise ValueError("a layer's halves must use as many copies of the residual stream as the layer carries")
        f32 = lambda name: tensors[name].float().contiguous()
        self.read, self.write, self.mix = f32(spec.read), f32(spec.write), f32(spec.mix)

    @staticmethod
    def tensor_needs(spec):
        if spec is None:
            return []
        n = spec.n_streams
        return [TensorNeed(spec.read, (n,)), TensorNeed(spec.write, (n,)), TensorNeed(spec.mix, (n, n))]


class MultiStreamBlock:
    stream_aware = True               # its x is [T, n_streams * hidden]
    FUSE = True                       # the copies' sum, the norm and the blend with the row before in one kernel, and the mixer's result written into
                                      # the copies together with the feed-forward's input read out of them (off: one after the other)

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        if spec.mixer_post_norm is not None or spec.feed_forward_post_norm is not None:
            raise ValueError("a multistream layer has a norm before each half and none behind")
        self.n_streams = spec.mixer_streams.n_streams if spec.mixer_streams is not None else 1
        if not 1 <= self.n_streams <= ops.streams_max():
            raise ValueError(f"1 to {ops.streams_max()} copies of the residual stream are served, not {self.n_streams}")
        self.scale = float(spec.residual_scale)
        self.mixer_norm = norm_class(spec.mixer_norm)(spec.mixer_norm, tensors, dtype, device)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.mixer_access = _Access(spec.mixer_streams, tensors, self.n_streams)
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = norm_class(spec.feed_forward_norm)(spec.feed_forward_norm, tensors, dtype, device)
            self.feed_forward = feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)
            self.feed_forward_access = _Access(spec.feed_forward_streams, tensors, self.n_streams)

    def _parts(self):
        return [self.mixer_norm, self.mixer] + ([self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else [])

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in self._parts())

    @classmethod
    def tensor_needs(cls, spec):
        needs = norm_class(spec.mixer_norm).tensor_needs(spec.mixer_norm) + mixer_class(spec.mixer).tensor_needs(spec.mixer) + _Access.tensor_needs(spec.mixer_streams)
        if spec.feed_forward is not None:
            needs += (norm_class(spec.feed_forward_norm).tensor_needs(spec.feed_forward_norm) + feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward)
                      + _Access.tensor_needs(spec.feed_forward_streams))
        return needs

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    def weights_read_per_step(self):
        return self._parts()

    def _input(self, x, ctx, norm, part, access, shift=None, state=None):
        """The rows a half reads: norm(sum_s read[s] x_s), blended with the row before where the half's mixer asks for it."""
        T, width = ctx.n_rows, x.shape[1] // self.n_streams
        dtype = getattr(part, "in_dtype", ctx.dtype)
        if self.FUSE and type(norm) is RmsNorm:
            out = torch.empty((T, width), dtype=dtype, device=x.device)
            return _blend(x, self.n_streams, out, ctx, read=access.read, norm_weight=norm.weight, eps=norm.eps, shift=shift, state=state)
        u = x
        if self.n_streams > 1 or access.read is not None:
            u = ops.streams_norm_shift(x, self.n_streams, torch.empty((T, width), dtype=torch.float32, device=x.device), read=access.read)
        if shift is None:
            return norm(u, dtype)
        out = torch.empty((T, width), dtype=dtype, device=x.device)
        return _blend(norm(u, torch.float32), 1, out, ctx, read=None, norm_weight=None, eps=0.0, shift=shift, state=state)

    def _output(self, x, y, access):
        ops.streams_write(x, self.n_streams, y, access.mix, access.write, self.scale)

    @staticmethod
    def _run(part, h, ctx, *cache):
        """The half's result in rows of its own."""
        y = torch.empty((ctx.n_rows, h.shape[1]), dtype=torch.float32, device=h.device)
        if getattr(part, "can_overwrite", False):
            part.forward(h, y, ctx, *cache, overwrite=True)
        else:
            y.zero_()
            part.forward(h, y, ctx, *cache)
        return y

    def _traced(self, tag, x, ctx):
        if ctx.trace is not None:              # (what a reader of one stream would see: the sum of the copies)
            width = x.shape[1] // self.n_streams
            ctx.trace(tag, x if self.n_streams == 1 else ops.streams_norm_shift(x, self.n_streams, torch.empty((ctx.n_rows, width), dtype=torch.float32, device=x.device)))

    def forward(self, x, ctx, cache):
        if x.shape[1] != self.n_streams * self.mixer_norm.spec.size:
            raise ValueError("a multistream layer was handed rows of another number of copies than it carries")
        if isinstance(self.mixer, TokenShift):          # the block makes the blend itself and calls the mixer inside
            h = self._input(x, ctx, self.mixer_norm, self.mixer.inner, self.mixer_access, shift=self.mixer.weight, state=cache.state)
            y = self._run(self.mixer.inner, h, ctx, self.mixer.inner_cache(cache))
        else:
            h = self._input(x, ctx, self.mixer_norm, self.mixer, self.mixer_access)
            y = self._run(self.mixer, h, ctx, cache)
        h = None
        if (self.feed_forward is not None and self.FUSE and type(self.feed_forward_norm) is RmsNorm and ctx.trace is None
                and ops.streams_write_norm_takes(self.n_streams, x.shape[1] // self.n_streams)):
            # the mixer's result into the copies and the feed-forward's input out of them in one kernel
            a, b = self.mixer_access, self.feed_forward_access
            h = torch.empty((ctx.n_rows, x.shape[1] // self.n_streams), dtype=getattr(self.feed_forward, "in_dtype", ctx.dtype), device=x.device)
            ops.streams_write_norm(x, self.n_streams, y, a.mix, a.write, self.scale, b.read, self.feed_forward_norm.weight, self.feed_forward_norm.eps, h)
        else:
            self._output(x, y, self.mixer_access)
        self._traced("attn_out", x, ctx)
        if self.feed_forward is not None:
            if h is None:
                h = self._input(x, ctx, self.feed_forward_norm, self.feed_forward, self.feed_forward_access)
            y = self._run(self.feed_forward, h, ctx)
            self._output(x, y, self.feed_forward_access)
        self._traced("ffn_out", x, ctx)


register_block("multistream", MultiStreamBlock)
