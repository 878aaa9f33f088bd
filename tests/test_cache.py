"""The cache's bookkeeping (no GPU): no slot or page is lost, held twice or freed twice;
groups have storage of their own; a window gives pages back early; state starts at zero."""
import random

import pytest
import torch

from rocml_amd.cache import Cache, SlotAllocator, pages_for
from rocml_amd.errors import CacheFullError, RocmlError
from rocml_amd.parts import KVCacheRequest, StateRequest

FULL = KVCacheRequest(2, 16, None)
WIN = KVCacheRequest(2, 16, 100)
STATE = StateRequest((3, 4))


def _cache(requests, max_tokens, **kw):
    return Cache(requests, max_tokens, torch.float32, "cpu", **kw)


def test_slot_allocator():
    a = SlotAllocator(3)
    s = [a.alloc(), a.alloc(), a.alloc()]
    assert sorted(s) == [0, 1, 2]
    with pytest.raises(CacheFullError):
        a.alloc()
    a.free(1)
    with pytest.raises(RocmlError, match="freed twice"):
        a.free(1)
    assert a.alloc() == 1                      # a freed slot is used again at once
    with pytest.raises(RocmlError):
        a.free(7)


def test_groups_have_their_own_storage_and_lines():
    c = _cache([FULL, WIN, FULL, None, STATE, WIN], 64 * 10, max_seqs=4)
    assert len(c.kv_groups) == 2 and len(c.state_groups) == 1
    full, win = c.kv_groups
    assert full.n_lines == 2 and win.n_lines == 2
    assert full.k.shape == (2, 10, 2, 64, 16) and full.v.shape == (2, 10, 2, 16, 64)
    assert win.n_pages == min(10, 4 * (pages_for(100) + 1))
    assert c.line(0) == (full, 0) and c.line(2) == (full, 1) and c.line(5) == (win, 1)
    assert not c.has_line(3)
    assert c.state_groups[0].state.shape == (1, 4, 3, 4)
    assert c.bytes_per_token() == 2 * (2 + 2) * 2 * 16 * 4


def test_pages_follow_lengths_and_reserve_is_all_or_nothing():
    c = _cache([FULL], 64 * 4)
    a, b = c.new_sequence(), c.new_sequence()
    c.reserve([a, b], [65, 64])
    c.commit([a, b], [65, 64])
    g = c.kv_groups[0]
    assert len(g.page_table(a)) == 2 and len(g.page_table(b)) == 1 and g.n_free_pages == 1
    with pytest.raises(CacheFullError):
        c.reserve([a, b], [129, 129])          # needs 1 + 2 pages, 1 is free
    assert g.n_free_pages == 1 and len(g.page_table(a)) == 2      # nothing was taken
    c.reserve([a], [128])                      # no new page
    assert g.n_free_pages == 1
    c.check()
    table = c.block_table(g, [b, a], 4)
    assert table.shape == (2, 4) and list(table[0, 1:]) == [-1, -1, -1] and table[1, 1] >= 0
    c.free_sequence(a)
    with pytest.raises(RocmlError):
        c.free_sequence(a)
    assert g.n_free_pages == 3
    c.check()


def test_sequences_of_a_step_get_neighbouring_pages():
    """A step's sequences take their pages a page per sequence and round: page p of all of them
    lies side by side in the pool, and a longer sequence goes on alone."""
    c = _cache([FULL], 64 * 16)
    s = [c.new_sequence() for _ in range(3)]
    c.reserve(s, [130, 64, 200])               # 3, 1 and 4 pages
    c.commit(s, [130, 64, 200])
    g = c.kv_groups[0]
    t = [g.page_table(x) for x in s]
    assert [len(x) for x in t] == [3, 1, 4]
    assert sorted([t[0][0], t[1][0], t[2][0]]) == [0, 1, 2]       # first pages of all three
    assert sorted([t[0][1], t[2][1]]) == [3, 4] and sorted([t[0][2], t[2][2]]) == [5, 6]
    assert t[2][3] == 7
    c.reserve(s, [193, 65, 257])               # one more page each: again side by side
    assert sorted([t[0][3], t[1][1], t[2][4]]) == [8, 9, 10]
    c.check()


def test_window_releases_pages_no_query_can_see():
    c = _cache([WIN], 64 * 8)
    s = c.new_sequence()
    g = c.kv_groups[0]
    c.reserve([s], [300])
    assert g.n_free_pages == 8 - 5
    c.commit([s], [300])
    # a query at position 300 sees keys from 201 on: pages 0..2 (positions 0..191) are free again
    assert g.page_table(s)[:3] == [-1, -1, -1] and g.page_table(s)[3] >= 0
    assert g.n_free_pages == 6
    c.reserve([s], [301])
    c.commit([s], [301])
    assert len(g.page_table(s)) == 5
    c.check()
    c.free_sequence(s)
    assert g.n_free_pages == 8


def test_state_is_zero_when_a_slot_is_handed_out():
    c = _cache([STATE], 64 * 2, max_seqs=2)
    s = c.new_sequence()
    c.state_groups[0].state[:, s] = 5.0
    c.free_sequence(s)
    assert c.new_sequence() == s
    assert float(c.state_groups[0].state[:, s].abs().max()) == 0.0


def test_random_traffic_keeps_the_books_balanced():
    rng = random.Random(0)
    c = _cache([FULL, WIN], 64 * 40, max_seqs=12)
    live = {}
    for _ in range(3000):
        op = rng.random()
        if op < 0.25 and len(live) < 12:
            live[c.new_sequence()] = 0
        elif op < 0.4 and live:
            s = rng.choice(list(live))
            c.free_sequence(s)
            del live[s]
        elif live:
            some = rng.sample(list(live), k=min(len(live), rng.randint(1, 4)))
            new = [live[s] + rng.randint(1, 90) for s in some]
            try:
                c.reserve(some, new)
            except CacheFullError:
                c.check()
                continue
            c.commit(some, new)
            for s, n in zip(some, new):
                live[s] = n
        c.check()
        for s, n in live.items():
            assert c.length(s) == n
            for g in c.kv_groups:
                table = g.page_table(s)
                assert len(table) >= pages_for(n)
                first = 0 if g.request.window is None else max(0, n - g.request.window + 1) // 64
                assert all(p >= 0 for p in table[first:])          # every page a query may read is held
    held = [p for g in c.kv_groups[:1] for s in live for p in g.page_table(s) if p >= 0]
    assert len(held) == len(set(held))                              # no page held twice


def test_storage_is_checked_against_free_memory_before_it_is_allocated():
    """Bytes per position as the reference counts them (2 * lines * Hkv * D * bytes,
    rocml/src/budget/mod.rs:47-59), 768 MiB kept free beside the cache, and a refusal that
    allocates nothing."""
    from rocml_amd.cache.cache import HEADROOM_BYTES, check_budget, planned_bytes
    from rocml_amd.errors import MemoryBudgetError
    full = KVCacheRequest(n_kv_heads=8, head_dim=128, window=None)
    windowed = KVCacheRequest(n_kv_heads=2, head_dim=64, window=100)
    state = StateRequest(shape=(4, 16), dtype=torch.float32)
    need = planned_bytes([full, full, None, windowed, state], max_tokens=64 * 1000, dtype=torch.bfloat16, max_seqs=10,
                         step_tokens=640)
    kv_full = 2 * 2 * 64 * 1000 * 8 * 128 * 2                       # two lines of 1000 pages
    # a window of 100 is two pages, one more as it starts inside a page, one being filled, per
    # sequence; and the ten pages of a piece's own 640 tokens
    kv_window = 2 * (10 * 4 + 10) * 64 * 2 * 64 * 2
    # without a bound on the pieces a windowed group is sized like one that keeps everything
    assert planned_bytes([windowed], 64 * 1000, torch.bfloat16, max_seqs=10) == 2 * 1000 * 64 * 2 * 64 * 2
    assert need == kv_full + kv_window + 10 * 64 * 4
    check_budget(need, need + HEADROOM_BYTES)
    with pytest.raises(MemoryBudgetError, match="GiB free"):
        check_budget(need, need + HEADROOM_BYTES - 1)
    with pytest.raises(MemoryBudgetError):
        Cache([full], max_tokens=1 << 40, dtype=torch.bfloat16, device="cpu", free_bytes=1 << 30)
    cache = Cache([full], max_tokens=128, dtype=torch.float32, device="cpu", free_bytes=HEADROOM_BYTES + (1 << 20))
    assert cache.n_pages == 2


def test_a_windowed_group_takes_prompts_far_longer_than_its_window():
    """Pieces are reserved and committed one after the other; the windowed group, sized for its
    windows and one piece, gives pages back between them, and the plan is checked as a whole
    before anything is reserved."""
    full = KVCacheRequest(n_kv_heads=1, head_dim=16, window=None)
    windowed = KVCacheRequest(n_kv_heads=1, head_dim=16, window=70)
    c = Cache([full, windowed], max_tokens=4096, dtype=torch.float32, device="cpu", max_seqs=2, step_tokens=256)
    g_full, g_win = c.kv_groups
    assert g_full.n_pages == 64 and g_win.n_pages == 2 * 4 + 4
    a, b = c.new_sequence(), c.new_sequence()
    pieces = [[(a, 256)], [(a, 512)], [(a, 768)], [(a, 1000), (b, 24)], [(b, 280)], [(b, 300)]]
    assert c.fits(pieces) is None
    for piece in pieces:
        slots, lens = [s for s, _ in piece], [n for _, n in piece]
        c.reserve(slots, lens)
        c.commit(slots, lens)
        c.check()
        for s, n in piece:                                         # the window's pages are all held
            table = g_win.page_table(s)
            assert all(p >= 0 for p in table[max(0, n - 70 + 1) // 64:])
    assert c.length(a) == 1000 and c.length(b) == 300
    assert g_win.n_pages - g_win.n_free_pages <= 2 * 3
    # a token at a time to the end of the full group's room: never more than the window's pages
    for n in range(1001, 1200):
        c.reserve([a], [n])
        c.commit([a], [n])
    assert g_win.n_pages - g_win.n_free_pages <= 2 * 3
    # a plan that does not fit is refused whole and says which group is short
    short = c.fits([[(a, 1200 + 256)], [(a, 1200 + 512)], [(a, 4097)]])
    assert short is not None and "kv0" in short
    c.check()
    # new sequences are counted from nothing; a final length counts a windowed group by its window
    c.free_sequence(a)
    c.free_sequence(b)
    assert c.fits([[("x", 256)], [("x", 512)]], final=[("x", 4096)]) is None
    assert c.fits([[("x", 256)]], final=[("x", 4097)]) is not None


def test_a_cache_group_kind_of_its_own_needs_no_change_to_the_cache():
    """A mixer with needs of its own (here: one narrow vector per position, in pages, beside a
    counter per sequence) brings a request class and a group class and registers the pair; the
    cache opens, commits, closes and checks it like its own kinds."""
    from dataclasses import dataclass
    from rocml_amd.cache import CacheLineView, PagedGroup, register_cache_group

    @dataclass(frozen=True)
    class LatentRequest:
        width: int
        window: int = None

    class LatentGroup(PagedGroup):
        def __init__(self, name, request, n_lines, geo):
            super().__init__(name, request, n_lines, self.pool_pages(request.window, geo), geo.page_size, request.window)
            self.latent = torch.zeros((n_lines, self.n_pages, geo.page_size, request.width), dtype=geo.dtype, device=geo.device)
            self.tokens_seen = {}

        @staticmethod
        def planned_bytes(request, n_lines, geo):
            return n_lines * PagedGroup.pool_pages(request.window, geo) * geo.page_size * request.width * 4

        def open(self, slot):
            super().open(slot)
            self.tokens_seen[slot] = 0

        def committed(self, slot, length):
            super().committed(slot, length)
            self.tokens_seen[slot] = length

        def close(self, slot):
            super().close(slot)
            del self.tokens_seen[slot]

        def view(self, line, step):
            return CacheLineView(group=self, line=line, k=self.latent[line], block_table=step.block_tables[self.name])

    register_cache_group(LatentRequest, LatentGroup)
    from rocml_amd.cache.cache import planned_bytes
    full = KVCacheRequest(n_kv_heads=1, head_dim=16)
    reqs = [full, LatentRequest(24), LatentRequest(24), None, LatentRequest(24, window=100)]
    assert planned_bytes(reqs, 64 * 10, torch.float32) == 2 * 640 * 16 * 4 + 2 * 640 * 24 * 4 + 640 * 24 * 4
    c = Cache(reqs, max_tokens=64 * 10, dtype=torch.float32, device="cpu")
    assert [g.name for g in c.kv_groups] == ["kv0", "latent0", "latent1w100"] and c.kv_groups[1].n_lines == 2
    a, b = c.new_sequence(), c.new_sequence()
    c.reserve([a, b], [200, 5])
    c.commit([a, b], [200, 5])
    latent = c.kv_groups[1]
    assert latent.tokens_seen == {a: 200, b: 5} and len(latent.page_table(a)) == 4
    assert c.kv_groups[2].page_table(a)[0] == -1                     # the windowed one gave its first page back
    table = c.block_table(latent, [a, b], 4)
    assert table.shape == (2, 4) and table[1, 1] == -1
    c.free_sequence(a)
    c.check()
    assert latent.tokens_seen == {b: 5} and c.line(2)[0] is latent and c.line(2)[1] == 1


def test_a_request_class_derived_from_a_registered_one_gets_its_own_group():
    """The nearest registered class of a request decides: a subclass of the key/value request that
    registers a group of its own is served by that group, an unregistered subclass by its base's."""
    from dataclasses import dataclass
    from rocml_amd.cache import register_cache_group
    from rocml_amd.cache.cache import KVGroup, _group_type

    @dataclass(frozen=True)
    class WideRequest(KVCacheRequest):
        pass

    @dataclass(frozen=True)
    class PlainChild(KVCacheRequest):
        pass

    class WideGroup(KVGroup):
        pass

    register_cache_group(WideRequest, WideGroup)
    assert _group_type(WideRequest(1, 16)) is WideGroup
    assert _group_type(PlainChild(1, 16)) is KVGroup and _group_type(KVCacheRequest(1, 16)) is KVGroup
    c = Cache([WideRequest(1, 16), KVCacheRequest(1, 16)], max_tokens=128, dtype=torch.float32, device="cpu")
    assert type(c.line(0)[0]) is WideGroup and type(c.line(1)[0]) is KVGroup


def test_workspace_views_are_kept_until_their_buffer_moves():
    """A step asks for the same few views over and over; the workspace hands the same view out
    again, and forgets a buffer's views when the buffer has to grow (a recorded graph is then
    stale, which ``generation`` says)."""
    from rocml_amd.engine import Workspace
    ws = Workspace("cpu")
    a = ws.get("x", (4, 8), torch.float32)
    g0 = ws.generation
    assert ws.get("x", (4, 8), torch.float32) is a and ws.generation == g0
    b = ws.get("x", (2, 8), torch.float32)                    # a smaller view of the same buffer
    assert b.data_ptr() == a.data_ptr() and ws.generation == g0 and tuple(b.shape) == (2, 8)
    other = ws.get("x", (4, 8), torch.bfloat16)               # another type is another buffer
    assert other.dtype == torch.bfloat16 and ws.generation == g0 + 1
    big = ws.get("x", (16, 8), torch.float32)                 # the buffer grows: its views are dropped
    assert ws.generation == g0 + 2 and tuple(big.shape) == (16, 8)
    again = ws.get("x", (4, 8), torch.float32)
    assert again is not a and again.data_ptr() == big.data_ptr()
    assert ws.get("x", (4, 8), torch.bfloat16) is other       # the other buffer's views stay
