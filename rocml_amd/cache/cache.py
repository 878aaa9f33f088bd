"""The cache: a slot per sequence, keys and values per cache line in pages, and
per-sequence state of fixed size.

The reference holds one sequence: per layer two planes ``[Hkv, max_seq, D]`` and one
scalar position (rocml/src/cache.rs:45-138, rocml/src/forward/mod.rs:84); a reset
only sets the position to zero because rows beyond it are never read
(rocml/src/forward/mod.rs:224-232), while the fixed-size state of its other
architecture is zeroed on reset (rocml/src/qwen35/cache/mod.rs:289-298).  Both rules
are kept here, for many sequences:

* a **slot** stands for one live sequence and knows its length;
* cache lines (one per execution of a layer that owns a cache) with the same needs form
  a **group** with storage of its own.  A key/value group is a pool of pages of
  ``page_size`` positions, keys laid out ``[line, page, Hkv, page_size, D]`` and values
  ``[line, page, Hkv, D, page_size]``, so that one head's part of a page is contiguous;
  each slot maps its logical pages to pool pages.  A group with a window gives pages back as soon as no later query can see them;
* a **state group** is ``[line, slot, *shape]`` and a slot's part is zeroed when the
  slot is handed out;
* pages are not cleared when a slot is freed or handed out again.

All bookkeeping is on the host and works without a GPU; only the storage is on the
device.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import CacheFullError, MemoryBudgetError, RocmlError
from ..parts.base import KVCacheRequest, StateRequest

PAGE_SIZE = 64


def pages_for(length: int, page_size: int = PAGE_SIZE) -> int:
    return (length + page_size - 1) // page_size


class SlotAllocator:
    """Hands out the integers ``0 .. n-1``; lowest free number first, so that freed
    slots are used again at once."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free = list(range(n_slots - 1, -1, -1))
        self._live = set()

    def alloc(self) -> int:
        if not self._free:
            raise CacheFullError(f"all {self.n_slots} sequence slots are in use")
        slot = self._free.pop()
        self._live.add(slot)
        return slot

    def free(self, slot: int) -> None:
        if slot not in self._live:
            raise RocmlError(f"slot {slot} is not in use (freed twice, or never handed out)")
        self._live.remove(slot)
        self._free.append(slot)
        self._free.sort(reverse=True)

    def is_live(self, slot: int) -> bool:
        return slot in self._live

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def live(self):
        return frozenset(self._live)


@dataclass(frozen=True)
class Geometry:
    """What a cache was asked to hold; every group sizes its storage from it."""
    n_pages: int                  # pages of page_size positions for live sequences together
    page_size: int
    n_slots: int                  # most live sequences
    max_seqs: Optional[int]       # the caller's bound on live sequences, if it gave one
    step_tokens: Optional[int]    # most tokens one piece of a step brings, if bounded
    dtype: torch.dtype            # the model's compute type
    device: object


class CacheGroup:
    """Storage shared by the cache lines with one request.  The cache tells every group when a
    sequence starts (``open``), reaches a length (``committed``) and ends (``close``); a group
    hands a mixer its part of the storage with ``view``.  A group with ``paged`` true also keeps
    a page table per sequence (``PagedGroup``)."""
    paged = False

    def __init__(self, name: str, request, n_lines: int):
        self.name = name
        self.request = request
        self.n_lines = n_lines

    @staticmethod
    def planned_bytes(request, n_lines: int, geo: "Geometry") -> int:
        return 0

    def open(self, slot: int) -> None:
        pass

    def committed(self, slot: int, length: int) -> None:
        pass

    def close(self, slot: int) -> None:
        pass

    def check(self) -> None:
        pass

    def view(self, line: int, step) -> "CacheLineView":
        raise NotImplementedError


class PagedGroup(CacheGroup):
    """Page bookkeeping of a group that stores something per position: a pool of pages and, per
    sequence, the pool pages of its logical pages.  ``window`` (None: everything is kept) lets
    the group give pages back once no later query can see them.  Storage is the subclass's."""
    paged = True

    def __init__(self, name: str, request, n_lines: int, n_pages: int, page_size: int, window: Optional[int]):
        super().__init__(name, request, n_lines)
        self.n_pages = n_pages
        self.page_size = page_size
        self.window = window
        self._free = list(range(n_pages - 1, -1, -1))
        self._pages: Dict[int, List[int]] = {}   # slot -> logical page -> pool page, -1 once released

    @staticmethod
    def pool_pages(window: Optional[int], geo: Geometry) -> int:
        """Pages of the pool.  A group with a window holds, per sequence, the pages its window
        spans (one more than the window's pages, as it rarely starts on a page's edge) and the
        page being filled; while a step runs it also holds the pages of the step's own tokens,
        which are only given back when the step's piece is committed.  With a bound on the
        sequences and on the tokens of a piece the group needs no more than that, however long
        the sequences grow; without them it is sized like a group that keeps everything."""
        if window is not None and geo.max_seqs is not None and geo.step_tokens is not None:
            return min(geo.n_pages, geo.max_seqs * (pages_for(window, geo.page_size) + 2)
                       + pages_for(geo.step_tokens, geo.page_size))
        return geo.n_pages

    # -- bookkeeping -----------------------------------------------------------------
    @property
    def n_free_pages(self) -> int:
        return len(self._free)

    def open(self, slot: int) -> None:
        self._pages[slot] = []

    def pages_needed(self, slot: int, new_len: int) -> int:
        return max(0, pages_for(new_len, self.page_size) - len(self._pages[slot]))

    def grow(self, slot: int, new_len: int) -> None:
        need = self.pages_needed(slot, new_len)
        if need > len(self._free):
            raise CacheFullError(f"cache group {self.name}: {need} more pages of {self.page_size} "
                                 f"positions are needed, {len(self._free)} of {self.n_pages} are free")
        table = self._pages[slot]
        for _ in range(need):
            table.append(self._free.pop())

    def grow_together(self, slots: Sequence[int], new_lens: Sequence[int]) -> None:
        """Pages for several sequences at once, a page per sequence and round.  Sequences that
        run side by side then hold the pages of one position side by side in the pool, and the
        decode attention, which reads the same positions of all sequences at about the same
        time, reads one window of memory instead of as many as there are sequences (11 % of its
        time at batch 64).  The caller has checked that the pages are there."""
        need = [self.pages_needed(s, n) for s, n in zip(slots, new_lens)]
        for level in range(max(need, default=0)):
            for s, k in zip(slots, need):
                if level < k:
                    self._pages[s].append(self._free.pop())

    def committed(self, slot: int, length: int) -> None:
        self.trim(slot, length)

    def trim(self, slot: int, length: int) -> None:
        """After a sequence reached ``length``: a group with a window releases the pages
        whose positions no query at ``length`` or later can see."""
        w = self.window
        if w is None:
            return
        first_needed = max(0, length - w + 1) // self.page_size
        table = self._pages[slot]
        for i in range(min(first_needed, len(table))):
            if table[i] >= 0:
                self._free.append(table[i])
                table[i] = -1

    def close(self, slot: int) -> None:
        for page in self._pages.pop(slot):
            if page >= 0:
                self._free.append(page)

    def page_table(self, slot: int) -> List[int]:
        return self._pages[slot]

    def check(self) -> None:
        """No page lost, none held twice, none both free and held."""
        held = [p for table in self._pages.values() for p in table if p >= 0]
        everything = sorted(held + self._free)
        if everything != list(range(self.n_pages)):
            raise RocmlError(f"cache group {self.name}: pages out of balance "
                             f"({len(held)} held, {len(self._free)} free, {self.n_pages} in all)")

    def bytes_per_token(self) -> int:
        return 0


class KVGroup(PagedGroup):
    """Paged keys and values of the cache lines that share one ``KVCacheRequest``."""

    def __init__(self, name: str, request: KVCacheRequest, n_lines: int, geo: Geometry):
        super().__init__(name, request, n_lines, self.pool_pages(request.window, geo), geo.page_size, request.window)
        # Values are transposed inside a page, which is the order the attention kernels
        # multiply them in.  Zeroed once: rows beyond a sequence's length are never counted,
        # but they are multiplied by a zero weight and so must stay finite.
        h, d = request.n_kv_heads, request.head_dim
        self.k = torch.zeros((n_lines, self.n_pages, h, self.page_size, d), dtype=geo.dtype, device=geo.device)
        self.v = torch.zeros((n_lines, self.n_pages, h, d, self.page_size), dtype=geo.dtype, device=geo.device)

    @staticmethod
    def planned_bytes(request: KVCacheRequest, n_lines: int, geo: Geometry) -> int:
        size = torch.empty((), dtype=geo.dtype).element_size()
        return (2 * n_lines * PagedGroup.pool_pages(request.window, geo) * geo.page_size
                * request.n_kv_heads * request.head_dim * size)

    def view(self, line: int, step) -> "CacheLineView":
        return CacheLineView(group=self, line=line, k=self.k[line], v=self.v[line],
                             block_table=step.block_tables[self.name])

    def bytes_per_token(self) -> int:
        r = self.request
        return 2 * self.n_lines * r.n_kv_heads * r.head_dim * self.k.element_size()


class StateGroup(CacheGroup):
    """Fixed-size per-sequence state of the cache lines that share one ``StateRequest``."""

    def __init__(self, name: str, request: StateRequest, n_lines: int, geo: Geometry):
        super().__init__(name, request, n_lines)
        self.state = torch.zeros((n_lines, geo.n_slots) + tuple(request.shape), dtype=request.dtype, device=geo.device)

    @staticmethod
    def planned_bytes(request: StateRequest, n_lines: int, geo: Geometry) -> int:
        n = 1
        for dim in request.shape:
            n *= dim
        return n_lines * geo.n_slots * n * torch.empty((), dtype=request.dtype).element_size()

    def open(self, slot: int) -> None:
        self.state[:, slot].zero_()

    def view(self, line: int, step) -> "CacheLineView":
        return CacheLineView(group=self, line=line, state=self.state[line], slots=step.seq_slots)


# Which group class serves which kind of request.  A mixer with needs of its own brings a request
# class and a group class (both may live outside this package) and registers the pair.
_GROUP_KINDS: Dict[type, type] = {}


def register_cache_group(request_type: type, group_type: type) -> None:
    """``group_type(name, request, n_lines, geometry)`` builds the storage for ``request_type``;
    its static ``planned_bytes(request, n_lines, geometry)`` says how much that will be."""
    _GROUP_KINDS[request_type] = group_type


def _group_type(req) -> type:
    # the request's own class first, then its bases from the nearest on: a request class that
    # derives from a registered one and registers a group of its own gets that group
    for rt in type(req).__mro__:
        if rt in _GROUP_KINDS:
            return _GROUP_KINDS[rt]
    raise RocmlError(f"unknown cache request {req!r}")


register_cache_group(KVCacheRequest, KVGroup)
register_cache_group(StateRequest, StateGroup)


@dataclass
class CacheLineView:
    """What a mixer sees of the cache for one execution of its layer in one step."""
    group: object
    line: int
    k: Optional[torch.Tensor] = None            # [pages, Hkv, page_size, D]
    v: Optional[torch.Tensor] = None            # [pages, Hkv, D, page_size]
    block_table: Optional[torch.Tensor] = None  # [B, width] int32 on the device, per step
    state: Optional[torch.Tensor] = None        # [slots, *shape]
    slots: Optional[torch.Tensor] = None        # [B] int32 on the device, per step


# Memory left free beside the cache for activations and the runtime: the reference keeps
# 768 MiB of headroom when it checks a context length against hipMemGetInfo
# (rocml/src/budget/mod.rs:37, rocml/src/forward/mod.rs:148-161).
HEADROOM_BYTES = 768 << 20


def _geometry(max_tokens: int, dtype, device, max_seqs: Optional[int], page_size: int,
              step_tokens: Optional[int]) -> Geometry:
    n_pages = max(1, pages_for(max_tokens, page_size))
    return Geometry(n_pages=n_pages, page_size=page_size, n_slots=max_seqs if max_seqs is not None else n_pages,
                    max_seqs=max_seqs, step_tokens=step_tokens, dtype=dtype, device=device)


def _by_request(requests: Sequence[Optional[object]]) -> Dict[object, List[int]]:
    by_request: Dict[object, List[int]] = {}
    for entry, req in enumerate(requests):
        if req is not None:
            by_request.setdefault(req, []).append(entry)
    return by_request


def planned_bytes(requests: Sequence[Optional[object]], max_tokens: int, dtype: torch.dtype,
                  max_seqs: Optional[int] = None, page_size: int = PAGE_SIZE,
                  step_tokens: Optional[int] = None) -> int:
    """Bytes the cache for these requests will allocate: per key/value line
    ``2 * pages * page_size * Hkv * D * bytes`` (rocml/src/budget/mod.rs:47-59), per state
    line ``slots * elements * bytes``."""
    geo = _geometry(max_tokens, dtype, None, max_seqs, page_size, step_tokens)
    return sum(_group_type(req).planned_bytes(req, len(entries), geo)
               for req, entries in _by_request(requests).items())


def check_budget(need: int, free: int, headroom: int = HEADROOM_BYTES, max_tokens: Optional[int] = None) -> None:
    """Raises when ``need`` bytes and the headroom do not fit ``free``; names, as the reference's
    budget does (rocml/src/budget/mod.rs:70-83), about how many positions would fit."""
    if need + headroom > free:
        hint = ""
        if max_tokens is not None and need > 0:
            hint = f" (about {max(0, free - headroom) * max_tokens // need} positions would fit)"
        raise MemoryBudgetError(
            f"the cache needs {need / 2**30:.2f} GiB and {headroom / 2**20:.0f} MiB are kept free beside it, but the "
            f"device has {free / 2**30:.2f} GiB free: ask for fewer positions or sequences{hint}")


class Cache:
    """Slots, groups and the mapping from schedule entries to cache lines.

    ``requests[i]`` is what schedule entry ``i`` asks for (``None`` for an entry that
    owns no cache line).  ``max_tokens`` is the number of positions live sequences may
    hold together, each rounded up to whole pages; ``max_seqs`` bounds the live sequences.
    ``step_tokens`` is the most tokens one piece of a step brings; with it and ``max_seqs`` a
    group with a window is sized for its windows instead of for whole sequences.
    With ``free_bytes`` (the free memory of the device) the storage is checked against it,
    less ``headroom`` bytes for activations and the runtime, before anything is allocated."""

    def __init__(self, requests: Sequence[Optional[object]], max_tokens: int, dtype: torch.dtype,
                 device, max_seqs: Optional[int] = None, page_size: int = PAGE_SIZE,
                 free_bytes: Optional[int] = None, step_tokens: Optional[int] = None,
                 headroom: int = HEADROOM_BYTES):
        if free_bytes is not None:
            check_budget(planned_bytes(requests, max_tokens, dtype, max_seqs, page_size, step_tokens), free_bytes,
                         headroom=headroom, max_tokens=max_tokens)
        geo = _geometry(max_tokens, dtype, device, max_seqs, page_size, step_tokens)
        self.page_size = page_size
        self.n_pages = geo.n_pages
        self.max_seqs = geo.n_slots
        self.slots = SlotAllocator(self.max_seqs)
        self.lengths: Dict[int, int] = {}
        self.groups: List[CacheGroup] = []
        self._line_of: Dict[int, Tuple[CacheGroup, int]] = {}
        for req, entries in _by_request(requests).items():
            kind = _group_type(req)
            tag = kind.__name__.replace("Group", "").lower()
            name = f"{tag}{sum(1 for g in self.groups if type(g) is kind)}"
            if getattr(req, "window", None) is not None:
                name += f"w{req.window}"
            group = kind(name, req, len(entries), geo)
            self.groups.append(group)
            for line, entry in enumerate(entries):
                self._line_of[entry] = (group, line)
        self.kv_groups: List[PagedGroup] = [g for g in self.groups if g.paged]       # every group with pages
        self.state_groups: List[CacheGroup] = [g for g in self.groups if not g.paged]

    # -- sequences -------------------------------------------------------------------
    def new_sequence(self) -> int:
        slot = self.slots.alloc()
        self.lengths[slot] = 0
        for g in self.groups:
            g.open(slot)
        return slot

    def free_sequence(self, slot: int) -> None:
        self.slots.free(slot)
        del self.lengths[slot]
        for g in self.groups:
            g.close(slot)

    def length(self, slot: int) -> int:
        return self.lengths[slot]

    def reserve(self, slots: Sequence[int], new_lens: Sequence[int], which: str = "all") -> None:
        """Pages for every sequence to reach its new length, or none at all.  ``which``: ``all``
        groups, only those that keep every position (``kept``) or only those with a window
        (``windowed``): a step of several pieces takes the pages of the former for all its
        sequences at once, so that they lie side by side in the pool as ``grow_together`` wants
        them, and those of the latter piece by piece, between which such a group gives pages back."""
        groups = [g for g in self.kv_groups
                  if which == "all" or (g.window is None) == (which == "kept")]
        for g in groups:
            need = sum(g.pages_needed(s, n) for s, n in zip(slots, new_lens))
            if need > g.n_free_pages:
                raise CacheFullError(
                    f"cache group {g.name}: the step needs {need} more pages of {g.page_size} "
                    f"positions, {g.n_free_pages} of {g.n_pages} are free")
        for g in groups:
            g.grow_together(slots, new_lens)

    def fits(self, pieces: Sequence[Sequence[Tuple[object, int]]],
             final: Optional[Sequence[Tuple[object, int]]] = None) -> Optional[str]:
        """Whether the pieces of a step can be reserved and committed one after the other.
        A piece is a list of ``(sequence, length after the piece)``; a sequence is a live slot
        or any other key, which stands for a sequence that would start empty.  ``final`` names
        the lengths the sequences will grow to afterwards, a token at a time.  Only page counts
        are followed, nothing changes.  Returns None when everything fits, else what is short."""
        for g in self.kv_groups:
            free = g.n_free_pages
            size: Dict[object, int] = {}
            released: Dict[object, int] = {}
            w = g.window
            for piece in pieces:
                need = 0
                for key, n in piece:
                    if key not in size:
                        table = g._pages.get(key, []) if isinstance(key, int) else []
                        size[key] = len(table)
                        released[key] = sum(1 for p in table if p < 0)
                    want = pages_for(n, g.page_size)
                    if want > size[key]:
                        need += want - size[key]
                        size[key] = want
                if need > free:
                    return (f"cache group {g.name}: the step needs {need} more pages of {g.page_size} "
                            f"positions, {free} of {g.n_pages} are free")
                free -= need
                if w is not None:        # what the commit of this piece gives back
                    for key, n in piece:
                        first_needed = min(max(0, n - w + 1) // g.page_size, size[key])
                        if first_needed > released[key]:
                            free += first_needed - released[key]
                            released[key] = first_needed
            if final:
                # a token at a time: a sequence of a windowed group then never holds more than
                # the pages its window spans and the one being filled
                need = 0
                for key, n in final:
                    held = size.get(key, 0) - released.get(key, 0)
                    want = pages_for(n, g.page_size) - released.get(key, 0)
                    if w is not None:
                        want = min(want, max(held, pages_for(w, g.page_size) + 2))
                    need += max(0, want - held)
                if need > free:
                    return (f"cache group {g.name}: the sequences would need {need} more pages of "
                            f"{g.page_size} positions, {free} of {g.n_pages} are free")
        return None

    def commit(self, slots: Sequence[int], new_lens: Sequence[int]) -> None:
        for s, n in zip(slots, new_lens):
            self.lengths[s] = n
            for g in self.groups:
                g.committed(s, n)

    # -- per step --------------------------------------------------------------------
    def block_table(self, group: PagedGroup, slots: Sequence[int], width: int) -> np.ndarray:
        table = np.full((len(slots), width), -1, dtype=np.int32)
        for row, slot in enumerate(slots):
            pages = group.page_table(slot)
            table[row, :len(pages)] = pages
        return table

    def table_width(self, slots: Sequence[int]) -> int:
        return max([1] + [len(g.page_table(s)) for g in self.kv_groups for s in slots])

    def line(self, entry: int) -> Tuple[object, int]:
        return self._line_of[entry]

    def has_line(self, entry: int) -> bool:
        return entry in self._line_of

    def check(self) -> None:
        for g in self.groups:
            g.check()
        for g in self.kv_groups:
            if set(g._pages) != set(self.lengths):
                raise RocmlError(f"cache group {g.name}: slots and page tables disagree")
        if set(self.lengths) != set(self.slots.live):
            raise RocmlError("slot allocator and length table disagree")

    def bytes_per_token(self) -> int:
        """``2 * lines * Hkv * D * bytes`` summed over groups (rocml/src/budget/mod.rs:47-59)."""
        return sum(g.bytes_per_token() for g in self.kv_groups)
