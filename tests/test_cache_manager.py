"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice, under
random orders of requests; windows give pages back; slots and state."""
import random

import pytest
import torch

from torchlet_amd.cache.manager import CacheError, CacheManager, OutOfPages, PagePool
from torchlet_amd.parts.base import PagedNeed, StateNeed

FULL = PagedNeed(num_heads=2, head_dim=16)
WIN = PagedNeed(num_heads=2, head_dim=16, window=20)


def manager(plan, pages=10, page=8, slots=3, device=None):
    return CacheManager(plan, page_size=page, num_pages=pages, max_requests=slots, device=device)


def test_pool_is_lifo_and_guards_misuse():
    p = PagePool(5)
    assert p.free == 4
    a = p.take(2)
    assert a == [4, 3] and 0 not in a
    p.give([3])
    assert p.take(1) == [3]                    # the page freed last is reused first
    with pytest.raises(OutOfPages):
        p.take(3)
    assert p.free == 2                         # a failed take leaves the pool as it was
    p.give([3])
    with pytest.raises(CacheError, match="freed twice"):
        p.give([3])
    with pytest.raises(CacheError, match="does not belong"):
        p.give([0])


def test_layers_with_equal_needs_share_a_group_and_shared_caches_follow_their_owner():
    m = manager([(FULL, None, None), (WIN, None, None), (FULL, None, None), (None, None, 1)], device="cpu")
    assert len(m.groups) == 2 and m.groups[0].runs == [0, 2] and m.groups[1].runs == [1]
    assert [tuple(t.shape) for t in m.groups[0].tensors] == [(2, 10, 2, 8, 16)] * 2
    c0, c2, c3 = m.layer_cache(0), m.layer_cache(2), m.layer_cache(3)
    assert c0.group == c2.group == 0 and c0.writable and c0.planes[0].data_ptr() != c2.planes[0].data_ptr()
    assert c3.group == 1 and not c3.writable and c3.planes[0].data_ptr() == m.layer_cache(1).planes[0].data_ptr()


def test_reserve_is_all_or_nothing_and_tables_are_sentinel_padded():
    m = manager([(FULL, None, None)], pages=6)
    m.add_request("a")
    assert m.pages_missing("a", 17) == [3]
    assert m.reserve("a", 17) and m.free_pages() == [2]
    m.commit("a", 17)
    assert m.pages_missing("a", 24) == [0] and m.pages_missing("a", 25) == [1]
    m.add_request("b")
    assert not m.reserve("b", 17) and m.free_pages() == [2]          # needs 3, 2 free: nothing taken
    assert m.reserve("b", 16)
    bt = m.block_table(0, ["a", "b"], 4)
    assert bt.shape == (2, 4) and bt[0, 3] == 0 and bt[1, 2] == 0 and set(bt[0, :3]) | set(bt[1, :2]) == {1, 2, 3, 4, 5}
    m.check()
    with pytest.raises(CacheError, match="cannot shrink"):
        m.reserve("a", 3)


def test_release_returns_everything_and_guards():
    m = manager([(FULL, None, None), (WIN, None, None)], pages=8)
    m.add_request("a"); m.reserve("a", 30); m.commit("a", 30)
    m.release("a")
    assert m.free_pages() == [7, 7] and m.free_slots() == 3
    with pytest.raises(CacheError, match="released twice"):
        m.release("a")
    with pytest.raises(CacheError, match="not in the cache"):
        m.length("a")
    m.add_request("x")
    with pytest.raises(CacheError, match="already"):
        m.add_request("x")
    m.add_request("y"); m.add_request("z")
    with pytest.raises(OutOfPages, match="slot"):
        m.add_request("w")


def test_window_gives_pages_back_as_it_passes():
    m = manager([(WIN, None, None)], pages=8, page=8)
    m.add_request("a")
    assert m.reserve("a", 40)
    assert m.free_pages() == [2]               # a 40-token portion needs all five pages while it runs
    m.commit("a", 40)
    # queries from position 40 on read keys from 21 on: blocks 0 and 1 (keys 0..15) are dead
    assert m.free_pages() == [4]
    assert list(m.block_table(0, ["a"], 6)[0][:2]) == [0, 0]
    for n in range(41, 120):
        assert m.reserve("a", n)
        m.commit("a", n)
        m.check()
        live = sum(1 for p in m.block_table(0, ["a"])[0] if p)
        assert live <= 20 // 8 + 2             # window / page + the two partly filled ends
    m.release("a")
    assert m.free_pages() == [7]


def test_state_slots_are_zeroed_when_handed_out():
    m = manager([(None, StateNeed((4,)), None), (FULL, StateNeed((2, 2), torch.float32), None)], device="cpu")
    s = m.add_request("a")
    c0, c1 = m.layer_cache(0), m.layer_cache(1)
    # three slots and the row of the padding requests of fixed-shape steps, which belongs to no request
    assert c0.group is None and c0.state.shape == (4, 4) and c1.state.shape == (4, 2, 2) and c1.group == 0 and m.pad_slot == 3
    c0.state[s] = 7.0
    m.release("a")
    assert m.add_request("b") == s             # slots are reused, last freed first
    assert float(c0.state[s].abs().sum()) == 0.0


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    m = manager([(FULL, None, None), (WIN, None, None), (FULL, None, None)], pages=24, page=4, slots=5)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.free_slots():
            counter += 1
            live[f"r{counter}"] = 0
            m.add_request(f"r{counter}")
        elif op < 0.85 and live:
            r = rng.choice(list(live))
            n = live[r] + rng.choice([1, 1, 1, 2, 5, 13, 30])
            before = m.free_pages()
            if m.reserve(r, n):
                m.commit(r, n)
                live[r] = n
            else:
                assert m.free_pages() == before
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.check()
        for r, n in live.items():
            assert m.length(r) == n
            full = m.block_table(0, [r])[0]
            assert all(full[b] for b in range(-(-n // 4)))          # every block of a full-attention group is held
    for r in list(live):
        m.release(r)
    assert m.free_pages() == [23, 23] and m.free_slots() == 5


def test_planes_of_different_widths_and_an_element_type_of_their_own():
    """A mixer may keep planes that differ in heads and width (a compressed latent beside a small rotated
    part) and in element type; runs with the same such need still share a group."""
    latent = PagedNeed(num_heads=1, head_dim=0, planes=((1, 24), (1, 8), (3, 2)), dtype=torch.float32)
    m = CacheManager([(latent, None, None), (FULL, None, None), (latent, None, None)], page_size=4, num_pages=6,
                     max_requests=2, dtype=torch.bfloat16, device="cpu")
    assert len(m.groups) == 2 and m.groups[0].runs == [0, 2]
    assert [tuple(t.shape) for t in m.groups[0].tensors] == [(2, 6, 1, 4, 24), (2, 6, 1, 4, 8), (2, 6, 3, 4, 2)]
    assert {t.dtype for t in m.groups[0].tensors} == {torch.float32} and m.groups[1].tensors[0].dtype == torch.bfloat16
    c = m.layer_cache(2)
    assert [tuple(p.shape) for p in c.planes] == [(6, 1, 4, 24), (6, 1, 4, 8), (6, 3, 4, 2)]
    assert c.planes[0].data_ptr() == m.groups[0].tensors[0][1].data_ptr()
    assert m.bytes_per_page() == 2 * 4 * (24 + 8 + 6) * 4 + 2 * (2 * 4 * 16) * 2
    assert FULL.plane_shapes == ((2, 16), (2, 16))


@pytest.mark.parametrize("seed", range(4))
def test_a_windowed_groups_pool_is_sized_by_the_window_when_steps_are_bounded(seed):
    """With steps of at most 12 tokens a request holds at most (20 + 12 - 2) // 4 + 2 = 9 pages of a group
    with a window of 20 at pages of 4: three slots need 27 pages and the sentinel, however many pages the
    full-attention group has; sequences far longer than that pool still fit, and nothing is lost."""
    rng = random.Random(seed)
    m = CacheManager([(FULL, None, None), (WIN, None, None)], page_size=4, num_pages=200, max_requests=3, max_step_tokens=12)
    assert m.capacity() == [199, 27] and m.pages_for(400) == [100, 9]
    lengths: dict[str, int] = {}
    for step in range(400):
        if len(lengths) < 3 and rng.random() < 0.3:
            r = f"r{step}"
            m.add_request(r)
            lengths[r] = 0
        for r in list(lengths):
            n = rng.choice([1, 1, 1, 5, 12])
            if lengths[r] + n > 260 or rng.random() < 0.02:
                m.release(r)
                del lengths[r]
                continue
            assert m.reserve(r, lengths[r] + n), "a bounded step must always find its pages in the windowed pool"
            lengths[r] += n
            m.commit(r, lengths[r])
        m.check()
    for r in lengths:
        m.release(r)
    assert m.free_pages() == [199, 27]
