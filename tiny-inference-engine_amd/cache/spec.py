"""What a mixer needs from the cache, and how a model's needs are grouped.

A mixer declares one need (or none): paged keys and values, all of them or a
window of them, or a state of fixed size per request; a mixer that keeps several
things (keys and the last inputs of a short convolution, two mixers side by side)
declares a tuple of needs and is bound to a tuple of caches in the same order.
Run-order entries with
equal needs share a *group*: one page pool, one block table per request and one
tensor whose leading dimension counts the entries (planes) of the group. The
reference has a single group - every layer is full attention with the same head
geometry (``src/kv/paged_kv_cache.h:27-30``) - and no fixed-size state at all.
"""

from __future__ import annotations

import dataclasses
import functools
from typing import List, Optional, Sequence, Tuple, Union

from ..errors import InvalidArgument


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values of every cached position, in pages.

    ``window`` = None keeps all positions; ``window`` = w means a query at
    position p reads keys p-w+1 .. p, so pages wholly before that range can be
    given back while the request still runs. ``chunk`` = n means a query at position p
    reads the keys of its own chunk, from p - p % n on (chunks of n positions counted from 0):
    pages wholly before the chunk of the next query can go as well. At most one of the two.
    ``keep_first`` = f (with a window only) means every query also reads the keys of positions below f, at their
    true positions, however far back they lie: the pages that hold them stay with the request to its end.
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    chunk: Optional[int] = None
    keep_first: int = 0

    def __post_init__(self):
        if self.num_kv_heads <= 0 or self.head_dim <= 0:
            raise InvalidArgument("a paged cache needs positive num_kv_heads and head_dim")
        if self.window is not None and self.window <= 0:
            raise InvalidArgument(f"an attention window must be positive, got {self.window}")
        if self.chunk is not None and self.chunk <= 0:
            raise InvalidArgument(f"an attention chunk must be positive, got {self.chunk}")
        if self.window is not None and self.chunk is not None:
            raise InvalidArgument("a paged cache has a window or chunks, not both")
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise InvalidArgument(f"first positions are kept ({self.keep_first}) beside a window only, and not a "
                                  f"negative number of them")

    @property
    def reach(self) -> Optional[int]:
        """The most positions a query reads (None: all of them): what a request must hold at a time."""
        if self.window is not None:
            return self.window + self.keep_first
        return self.chunk

    def first_needed(self, position: int) -> int:
        """The first key any query at ``position`` or later reads."""
        if self.window is not None:
            return max(0, position - self.window + 1)
        if self.chunk is not None:
            return position - position % self.chunk
        return 0


@dataclasses.dataclass(frozen=True)
class FixedState:
    """A state of fixed shape per request (per run-order entry), kept in a slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self):
        if any(d <= 0 for d in self.shape):
            raise InvalidArgument(f"a state needs positive dimensions, got {self.shape}")


CacheNeed = Union[PagedKV, FixedState]


class CallCaches(tuple):
    """Where a run-order entry whose mixer declared several needs finds them: one ``CallCache`` a need, in order."""


@dataclasses.dataclass(frozen=True)
class CacheGroup:
    need: CacheNeed
    num_planes: int


@dataclasses.dataclass(frozen=True)
class CallCache:
    """Where one run-order entry finds its cache: a plane of a group, written or only read."""

    group: int
    plane: int
    writes: bool


@dataclasses.dataclass(frozen=True)
class CachePlan:
    groups: Tuple[CacheGroup, ...]
    calls: Tuple[Union[None, CallCache, CallCaches], ...]

    @functools.cached_property
    def paged_groups(self) -> List[int]:
        return [i for i, g in enumerate(self.groups) if isinstance(g.need, PagedKV)]

    @functools.cached_property
    def state_groups(self) -> List[int]:
        return [i for i, g in enumerate(self.groups) if isinstance(g.need, FixedState)]


def plan_cache(needs: Sequence[Optional[CacheNeed]], reads_cache_of: Sequence[Optional[int]]) -> CachePlan:
    """Groups the needs of the run-order entries.

    ``needs[i]`` is what entry i's mixer needs (None for a mixer without cache, a tuple for
    a mixer that needs several things: its entry of ``calls`` is then a ``CallCaches``);
    ``reads_cache_of[i]`` is an earlier entry whose plane entry i reads instead
    of owning one, and whose need must equal its own.
    """
    if len(needs) != len(reads_cache_of):
        raise InvalidArgument("plan_cache: one need and one sharing entry per run-order entry")
    group_of = {}
    planes: List[int] = []
    calls: List[Union[None, CallCache, CallCaches]] = []

    def own(need) -> CallCache:
        if need not in group_of:
            group_of[need] = len(planes)
            planes.append(0)
        g = group_of[need]
        planes[g] += 1
        return CallCache(g, planes[g] - 1, True)

    for i, need in enumerate(needs):
        src = reads_cache_of[i]
        if need is None or (isinstance(need, (tuple, list)) and not need):
            if src is not None:
                raise InvalidArgument(f"run order entry {i} reads a cache but its mixer needs none")
            calls.append(None)
            continue
        several = isinstance(need, (tuple, list))
        if src is not None:
            owner = calls[src] if 0 <= src < i else None
            owners = owner if isinstance(owner, CallCaches) else (owner,)
            if owner is None or not all(o.writes for o in owners):
                raise InvalidArgument(f"run order entry {i} reads the cache of entry {src}, which owns none")
            theirs = needs[src]
            if (tuple(theirs) if isinstance(theirs, (tuple, list)) else theirs) != (tuple(need) if several else need):
                raise InvalidArgument(
                    f"run order entry {i} needs {need} but reads the cache of entry {src}, which holds {needs[src]}")
            read = [CallCache(o.group, o.plane, False) for o in owners]
            calls.append(CallCaches(read) if several else read[0])
            continue
        calls.append(CallCaches(own(n) for n in need) if several else own(need))
    ordered = sorted(group_of.items(), key=lambda kv: kv[1])
    groups = tuple(CacheGroup(need, planes[g]) for need, g in ordered)
    return CachePlan(groups, tuple(calls))
