"""Several mixers that read the same rows: residual += sum_i weights[i] * member_i(h)  (`config.spec.SideBySideSpec`).

Every member is built from its own spec and keeps the cache or state it would keep alone; the entry's need is the members' needs
side by side (`JointNeed`: pages for at most one member, a fixed-size state for at most one).  Where every member says which
matrix its first product reads (`input_weight`), the matrices are laid one behind the other and one product serves all members.
Where every member can weigh its own result on the way (`set_out_scale`: a scan in its kernel, an attention on its values), each
adds straight onto the residual stream; otherwise each member stores its result in rows of its own (32-bit) and one kernel adds
their weighted sum.  The weights touch no matrix either way."""
from __future__ import annotations

import torch

from ..cache.needs import JointNeed, paged_need, state_need
from ..kernels import ops
from .base import LayerCache, Mixer, mixer_class, register_mixer
from .linear import linear


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
        # one first product for all members
        self.w_first, self._cuts = None, []
        first = [getattr(m, "input_weight", lambda: None)() for m in self.members]
        if (self.in_dtype is not None and all(w is not None for w in first) and len({w.dtype for w in first}) == 1 and len({w.shape[1] for w in first}) == 1
                and all((w.shape[0] * w.shape[1] * w.element_size()) % 16 == 0 for w in first)):
            self.w_first = torch.cat(first, dim=0).contiguous()
            at = 0
            for m, w in zip(self.members, first):
                m.use_input_weight(self.w_first[at:at + w.shape[0]])
                self._cuts.append((at, at + w.shape[0]))
                at += w.shape[0]
        # every member weighs its own result
        self.weigh_inside = all(hasattr(m, "set_out_scale") for m in self.members) and all([m.set_out_scale(w) for m, w in zip(self.members, self.weights)])
        if not self.weigh_inside:
            self.pages_are_shared()

    def pages_are_shared(self):
        """Another run-order entry reads this one's pages: nothing but the members' own keys and values may lie there."""
        self.weigh_inside = False
        for m in self.members:
            if hasattr(m, "set_out_scale"):
                m.set_out_scale(1.0)

    def weights_read_per_step(self):
        return self.members

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
        rows = h if torch.is_tensor(h) else h.materialize()
        told = [{} for _ in self.members]
        if self.w_first is not None:
            both = torch.empty((ctx.n_rows, self.w_first.shape[0]), dtype=torch.float32, device=residual.device)
            linear(rows, self.w_first, both)
            for own, (lo, hi) in zip(told, self._cuts):
                own["projected"] = both[:, lo:hi]
        if self.weigh_inside:
            for i, (member, need) in enumerate(zip(self.members, self._needs)):
                member.forward(rows, residual, ctx, self._member_cache(need, cache), overwrite=overwrite and i == 0, **told[i])
            return None
        outs = []
        for member, need, own in zip(self.members, self._needs, told):
            out = torch.empty_like(residual)
            member.forward(rows, out, ctx, self._member_cache(need, cache), overwrite=True, **own)
            outs.append(out)
        if overwrite:
            residual.zero_()
        for i in range(0, len(outs), 2):
            pair = outs[i:i + 2]
            ops.add_weighted(residual, pair[0], self.weights[i], pair[1] if len(pair) > 1 else None, self.weights[i + 1] if len(pair) > 1 else 0.0)
        return None


register_mixer("side_by_side", SideBySide)
