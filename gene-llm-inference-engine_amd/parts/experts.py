"""A mixture of gated feed-forwards behind a router (`config.spec.RoutedExpertsSpec` states the rules; kernels: `csrc/experts.hip`).

The router's logits are a 32-bit product of the normed rows (as the compute dtype stores them) with the router's matrix; the
same kernel turns them into every row's choice of experts and their weights.  The experts' matrices lie in stacks
[experts, ...] (in bfloat16 an expert's gates and up products interleaved in one matrix, for the product with the gate inside).
A few (row, choice) items walk their own expert's matrices each; many are put in the order of their experts on the device and
go through the matrix cores, all experts in one launch.  Either way nothing of a step's shape depends on the router's choices,
so a captured pass may contain the part.  A shared feed-forward, if the spec names one, is a part of its own kind and adds onto the
same rows."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import FeedForward, feed_forward_class, register_feed_forward
from .linear import activation_dtype_for, linear
from .norm import NormedRows


class RoutedExperts(FeedForward):
    graph_safe = True
    can_overwrite = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if s.score not in ops.ROUTER_SCORES:
            raise ValueError(f"routed experts: unknown score {s.score!r}; known: {', '.join(ops.ROUTER_SCORES)}")
        if s.weigh not in ("input", "output"):
            raise ValueError(f"routed experts: the weights weigh an expert's 'input' or its 'output', not {s.weigh!r}")
        if s.activation not in ops.ACTIVATIONS:
            raise ValueError(f"routed experts: unknown activation {s.activation!r}; known: {', '.join(ops.ACTIVATIONS)}")
        if s.n_experts > ops.ROUTER_MAX_EXPERTS or s.top > ops.ROUTER_MAX_TOP:
            raise ValueError(f"routed experts: at most {ops.ROUTER_MAX_EXPERTS} experts and {ops.ROUTER_MAX_TOP} a row")
        self.router = tensors[s.router]
        self.limit = float(getattr(s, "activation_limit", 0.0))
        self.groups = (s.n_groups, s.groups_kept) if getattr(s, "n_groups", 1) > 1 else None
        self.floor = float(getattr(s, "renormalize_floor", 0.0))
        # the shared feed-forward's gate is one more row of the router's matrix: its logit comes out of the router's product, in 32-bit
        self.shared_gated = getattr(s, "shared_gate", None) is not None
        self.router_all = torch.cat([self.router, tensors[s.shared_gate].reshape(1, -1)], dim=0).contiguous() if self.shared_gated else self.router
        self.w_down = torch.stack([tensors[n] for n in s.down_projs]).contiguous()
        if self.w_down.dtype == torch.bfloat16 and dtype == torch.bfloat16 and s.intermediate_size % ops.EXPERT_ROW_GROUP == 0:
            # gates and up products in one stack, as the product with the gate inside reads them
            self.w_gate = torch.stack([ops.interleave_gate_up(tensors[g], tensors[u]) for g, u in zip(s.gate_projs, s.up_projs)]).contiguous()
            self.w_up = None
        else:
            self.w_gate = torch.stack([tensors[n] for n in s.gate_projs]).contiguous()
            self.w_up = torch.stack([tensors[n] for n in s.up_projs]).contiguous()
        self.in_dtype = activation_dtype_for(self.w_gate, dtype)
        self.mid_dtype = activation_dtype_for(self.w_down, dtype)
        self.shared = None if s.shared is None else feed_forward_class(s.shared)(s.shared, tensors, dtype, device)
        if self.shared is not None and getattr(self.shared, "in_dtype", self.in_dtype) != self.in_dtype:
            raise ValueError("routed experts: the shared feed-forward must read rows stored as the experts read them")
        self.graph_safe = self.shared is None or bool(getattr(self.shared, "graph_safe", False))

    @classmethod
    def tensor_needs(cls, spec):
        s, d, i = spec, spec.hidden_size, spec.intermediate_size
        needs = [TensorNeed(s.router, (s.n_experts, d))]
        for g, u, w in zip(s.gate_projs, s.up_projs, s.down_projs):
            needs += [TensorNeed(g, (i, d)), TensorNeed(u, (i, d)), TensorNeed(w, (d, i))]
        if s.shared is not None:
            needs += feed_forward_class(s.shared).tensor_needs(s.shared)
        if getattr(s, "shared_gate", None) is not None:
            needs.append(TensorNeed(s.shared_gate, (1, d)))
        return needs

    def weights_read_per_step(self):
        """What a step of few rows reads: the router, `top` experts a row at most (here: of one row), the shared feed-forward."""
        s = self.spec
        share = [w[:min(s.top, s.n_experts)] for w in (self.w_gate, self.w_up, self.w_down) if w is not None]
        return [self.router_all, *share] + ([self.shared] if self.shared is not None else [])

    def forward(self, h, residual, ctx, then=None, overwrite=False):
        s, T, dev = self.spec, ctx.n_rows, ctx.device
        rows = h.materialize() if isinstance(h, NormedRows) else h
        ids = torch.empty((T, s.top), dtype=torch.int32, device=dev)
        weights = torch.empty((T, s.top), dtype=torch.float32, device=dev)
        gate = torch.empty((T, 1), dtype=torch.float32, device=dev) if self.shared_gated else None          # (its logit comes out of the router's product)
        ops.route_rows(rows, self.router_all, s.top, ids, weights, s.score, s.renormalize, groups=self.groups, floor=self.floor, extra=gate)
        ops.routed_experts(rows, self.w_gate, self.w_up, self.w_down, ids, weights, residual, accumulate=not overwrite, weigh=s.weigh, activation=s.activation,
                           limit=self.limit)
        if self.shared is not None and not self.shared_gated:
            self.shared.forward(rows, residual, ctx)
        elif self.shared is not None:          # its result in rows of its own, added times the row's gate
            if getattr(self.shared, "can_overwrite", False):
                y = torch.empty_like(residual)
                self.shared.forward(rows, y, ctx, overwrite=True)
            else:
                y = torch.zeros_like(residual)
                self.shared.forward(rows, y, ctx)
            ops.add_rows_gated(residual, y, gate)
        return None


register_feed_forward("routed_experts", RoutedExperts)
