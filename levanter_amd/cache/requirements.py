"""What a mixer asks of the cache manager. A mixer returns one of these from
``cache_requirement()`` (or None); cache units with equal requirements form a group."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple, Union


@dataclass(frozen=True)
class PagedKv:
    """Keys and values of every past token (or of the last ``window`` tokens), in pages."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None  # None: all keys. w: a query at position p reads keys p-w+1 .. p
    value_dim: Optional[int] = None  # size of a value head where it differs from a key head's (None: head_dim)
    chunk: Optional[int] = None  # c: a query at position p reads only keys of its own chunk, (p // c) * c .. p
    keep_first: int = 0  # the first so many positions of a request stay readable whatever window and chunk say

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def reach(self) -> Optional[int]:
        """The most keys any query reads (None: all keys so far)."""
        both = [n for n in (self.window, self.chunk) if n is not None]
        return min(both) + self.keep_first if both else None

    def first_needed(self, length: int) -> int:
        """The first position that a query at position ``length`` or later can still read."""
        lo = 0
        if self.window is not None:
            lo = max(lo, length - self.window + 1)
        if self.chunk is not None:
            lo = max(lo, (length // self.chunk) * self.chunk)
        return lo


@dataclass(frozen=True)
class SlotState:
    """A tensor of fixed shape per live request, zeroed when the request is admitted."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class Combined:
    """What a mixer made of several mixers asks for: one cache unit that holds pages and a state tensor at once (at most
    one ``PagedKv`` and one ``SlotState``). The unit's view in a step has both filled in."""

    parts: Tuple[Union[PagedKv, SlotState], ...]

    def __post_init__(self):
        kinds = [type(p) for p in self.parts]
        if any(k not in (PagedKv, SlotState) for k in kinds) or len(set(kinds)) != len(kinds):
            raise TypeError(f"a combined cache requirement takes one PagedKv and one SlotState at most, got {self.parts!r}")

    def paged(self) -> Optional[PagedKv]:
        return next((p for p in self.parts if isinstance(p, PagedKv)), None)

    def slot_state(self) -> Optional[SlotState]:
        return next((p for p in self.parts if isinstance(p, SlotState)), None)
