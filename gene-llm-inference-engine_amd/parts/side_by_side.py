"""Several mixers that read the same rows: residual += sum_i weights[i] * member_i(h)  (`config.spec.SideBySideSpec`).

Every member is built from its own spec and keeps the cache or state it would keep alone; the entry's need is the members' needs
side by side (`JointNeed`: pages for at most one member, a fixed-size state for at most one).  Each member stores its result in
rows of its own (32-bit), and one kernel adds their weighted sum onto the residual stream: the weights touch no matrix, so a
member's arithmetic is what it is alone."""
from __future__ import annotations

import torch

from ..cache.needs import JointNeed, paged_need, state_need
from ..kernels import ops
from .base import LayerCache, Mixer, mixer_class, register_mixer


class SideBySide(Mixer):
    accepts_deferred_norm = False

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.members = [mixer_class(m)(m, tensors, dtype, device) for m in spec.members]
        for m in self.members:
            if not getattr(m, "can_overwrite", False):
                raise ValueError(f"mixers side by side: a {type(m).__name__} cannot store its result in rows of its own")
        self.weights = [float(w) for w in spec.weights]
        dtypes = {getattr(m, "in_dtype", None) for m in self.members}
        self.in_dtype = dtypes.pop() if len(dtypes) == 1 else None
        self.graph_safe = all(getattr(m, "graph_safe", False) for m in self.members)
        self._needs = [mixer_class(m).cache_need(m) for m in spec.members]

    @classmethod
    def tensor_needs(cls, spec):
        return [n for m in spec.members for n in mixer_class(m).tensor_needs(m)]

    @classmethod
    def cache_need(cls, spec):
        needs = [mixer_class(m).cache_need(m) for m in spec.members]
        paged = [paged_need(n) for n in needs if paged_need(n) is not None]
        state = [state_need(n) for n in needs if state_need(n) is not None]
        if len(paged) > 1 or len(state) > 1:
            raise ValueError("mixers side by side: at most one member with pages and one with a fixed-size state")
        if not paged and not state:
            return None
        return JointNeed(paged[0] if paged else None, state[0] if state else None)

    def _member_cache(self, need, cache: LayerCache) -> LayerCache:
        view = LayerCache()
        if paged_need(need) is not None:
            view = LayerCache(kv=cache.kv, page_size=cache.page_size, table=cache.table, writes=cache.writes)
        if state_need(need) is not None:
            view.state = cache.state
        return view

    def forward(self, h, residual, ctx, cache, then=None, overwrite=False):
        outs = []
        for member, need in zip(self.members, self._needs):
            rows = h if torch.is_tensor(h) or getattr(member, "accepts_deferred_norm", False) else h.materialize()
            out = torch.empty_like(residual)
            member.forward(rows, out, ctx, self._member_cache(need, cache), overwrite=True)
            outs.append(out)
        if overwrite:
            residual.zero_()
        for i in range(0, len(outs), 2):
            pair = outs[i:i + 2]
            ops.add_weighted(residual, pair[0], self.weights[i], pair[1] if len(pair) > 1 else None, self.weights[i + 1] if len(pair) > 1 else 0.0)
        return None


register_mixer("side_by_side", SideBySide)
