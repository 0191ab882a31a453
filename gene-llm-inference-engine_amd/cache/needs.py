"""What a mixer asks of the cache manager for one layer of the run order."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedKvNeed:
    """Keys and values of every position (or of the last `window` positions, or of the positions of the chunk of `chunk`
    positions that the request is in: what no later position can see is given back) in pages.  `value_dim`: channels of a
    value head where they differ from a key head's `head_dim`."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None
    chunk: Optional[int] = None

    def elements_per_position(self) -> int:
        return self.n_kv_heads * (self.head_dim + (self.value_dim or self.head_dim))

    def first_visible(self, position: int) -> int:
        """The earliest position that the row at `position` (and so every later row) may still see."""
        first = 0
        if self.window is not None:
            first = max(first, position - self.window + 1)
        if self.chunk is not None:
            first = max(first, position - position % self.chunk)
        return first

    @property
    def forgets(self) -> bool:
        return self.window is not None or self.chunk is not None


@dataclass(frozen=True)
class StateNeed:
    """A state of fixed size per request (for instance a recurrent state), zeroed when a request starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class JointNeed:
    """What a mixer made of several mixers asks for one run-order entry: pages and a fixed-size state side by side (at most one
    of each; either may be absent)."""
    paged: Optional[PagedKvNeed] = None
    state: Optional[StateNeed] = None


def paged_need(need) -> Optional[PagedKvNeed]:
    """The pages an entry's need asks for, or None."""
    if isinstance(need, JointNeed):
        return need.paged
    return need if isinstance(need, PagedKvNeed) else None


def state_need(need) -> Optional[StateNeed]:
    """The fixed-size state an entry's need asks for, or None."""
    if isinstance(need, JointNeed):
        return need.state
    return need if isinstance(need, StateNeed) else None
