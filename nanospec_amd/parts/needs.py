"""What a mixer asks of the cache manager: pages (``PagedNeed``), state of fixed size (``StateNeed``), nothing (None), or a
tuple of these for a mixer made of several (it is then handed a tuple of views in the same order)."""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class PagedNeed:
    """Keys and values per token, in pages.  Mixers with equal needs share a group of pages."""

    kv_heads: int
    head_dim: int
    window: int = 0  # 0 = every earlier token stays
    value_dim: int = 0  # size of a value head if it is not ``head_dim``

    @property
    def v_dim(self) -> int:
        return self.value_dim or self.head_dim

    @property
    def group_name(self) -> str:
        return (f"kv{self.kv_heads}x{self.head_dim}" + (f"v{self.value_dim}" if self.value_dim not in (0, self.head_dim) else "")
                + (f"w{self.window}" if self.window else ""))


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request, kept in the request's slot; zeroed when a request is admitted."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


def each_need(need):
    """The single needs of what ``cache_need()`` returned, in order."""
    if isinstance(need, (tuple, list)):
        for n in need:
            yield from each_need(n)
    elif need is not None:
        yield need
