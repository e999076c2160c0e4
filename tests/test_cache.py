"""The page pool and the cache manager on the host: no page lost, held twice or freed twice,
under random orders of requests (reference scenarios: engine/tests/test_allocator.cu:23-113)."""
import random

import pytest
import torch

from bare_cuda_4gib_amd.cache import CacheManager, FixedState, PagedKV, PagePool
from bare_cuda_4gib_amd.errors import EngineError, OutOfPages


def test_pool_exhaust_and_refill():
    pool = PagePool(4)
    assert [pool.acquire() for _ in range(4)] == [0, 1, 2, 3]       # a fresh pool hands out 0, 1, 2, ...
    assert pool.acquire() == -1 and pool.free_count == 0 and pool.high_water_mark == 4
    assert pool.release(2) and pool.acquire() == 2                  # LIFO
    assert not pool.release(7) and not pool.release(-1)             # invalid
    assert pool.release(1) and not pool.release(1)                  # double free refused
    assert pool.pages_in_use == 3


def test_pool_random_stress_against_a_model():
    rng = random.Random(0)
    pool, held = PagePool(37), set()
    pool.shuffle_free_list(5)
    for _ in range(100000):
        if held and (rng.random() < 0.5 or len(held) == 37):
            page = rng.choice(sorted(held))
            assert pool.release(page)
            held.discard(page)
        else:
            page = pool.acquire()
            assert (page == -1) == (len(held) == 37)
            if page >= 0:
                assert page not in held and 0 <= page < 37
                held.add(page)
        assert pool.pages_in_use == len(held) and pool.free_count == 37 - len(held)


def _manager(num_pages=12, window=0, extra=None, **kw):
    streams = {0: PagedKV(2, 8), 1: PagedKV(2, 8)}
    if window:
        streams["w"] = PagedKV(1, 4, window=window)
    if extra:
        streams.update(extra)
    return CacheManager(streams, page_tokens=4, num_pages=num_pages, max_requests=4, max_tokens=40,
                        dtype=torch.float32, device="cpu", **kw)


def _check_invariants(cm, lengths):
    for gkey, group in cm.groups.items():
        held = []
        for rid in cm.live_requests():
            table = cm.table(gkey, rid)
            assert len(table) == cm.pages_for(lengths.get(rid, cm.length(rid))) or len(table) >= cm.pages_for(cm.length(rid))
            held.extend(p for p in table if p >= 0)
        assert len(held) == len(set(held)), "a page is held twice"
        assert all(group.pool.in_use(p) for p in held)
        assert group.pool.pages_in_use == len(held), "a page is lost"
        assert group.pool.pages_in_use + group.pool.free_count == group.pool.num_pages
        # the arrays by slot say what the lists say, and nothing in the rows of free slots
        mirror = cm.tables_by_slot[gkey]
        live_slots = set()
        for rid in cm.live_requests():
            slot, table = cm.slot(rid), cm.table(gkey, rid)
            live_slots.add(slot)
            assert mirror[slot, :len(table)].tolist() == table and (mirror[slot, len(table):] == -1).all()
            assert cm.lengths_by_slot[slot] == cm.length(rid)
        for slot in range(cm.max_requests):
            if slot not in live_slots:
                assert (mirror[slot] == -1).all() and cm.lengths_by_slot[slot] == 0


def test_reserve_is_all_or_nothing_and_pages_are_lazy():
    cm = _manager(num_pages=5)
    cm.admit("a"), cm.admit("b")
    cm.reserve([("a", 9)])                                           # 3 pages
    assert cm.pages_in_use() == 3 and cm.table(("window", 0), "a") == [0, 1, 2]
    cm.advance("a", 9)
    cm.reserve([("a", 3)])                                           # fits the third page: nothing new
    assert cm.pages_in_use() == 3
    with pytest.raises(OutOfPages):
        cm.reserve([("a", 4), ("b", 5)])                             # needs 1 + 2, only 2 are free
    assert cm.pages_in_use() == 3 and cm.table(("window", 0), "b") == []
    assert not cm.can_reserve([("a", 4), ("b", 5)]) and cm.can_reserve([("b", 8)])
    cm.reserve([("b", 8)])
    assert cm.pages_in_use() == 5
    cm.release("a")
    assert cm.pages_in_use() == 2 and cm.free_slots == 3
    cm.release("b")
    assert cm.pages_in_use() == 0


def test_errors():
    cm = _manager()
    with pytest.raises(EngineError):
        cm.reserve([("nobody", 1)])
    cm.admit("a")
    with pytest.raises(EngineError):
        cm.admit("a")
    with pytest.raises(EngineError):
        cm.reserve([("a", 41)])                                      # beyond max_tokens per request
    with pytest.raises(EngineError):
        cm.reserve([("a", 1), ("a", 1)])
    with pytest.raises(EngineError):
        cm.advance("a", 1)                                           # nothing reserved
    for r in "bcd":
        cm.admit(r)
    with pytest.raises(EngineError):
        cm.admit("e")                                                # all slots taken
    cm.release("a")
    with pytest.raises(EngineError):
        cm.release("a")


def test_groups_have_pages_of_their_own_and_windows_give_pages_back():
    cm = _manager(num_pages=6, window=6)
    full, win = ("window", 0), ("window", 6)
    assert set(cm.groups) == {full, win} and cm.groups[full].streams == [0, 1] and cm.groups[win].streams == ["w"]
    cm.admit("a")
    length = 0
    for n in (5, 2, 9, 1, 1, 6):
        cm.reserve([("a", n)])
        cm.advance("a", n)
        length += n
        table_full, table_win = cm.table(full, "a"), cm.table(win, "a")
        assert all(p >= 0 for p in table_full) and len(table_full) == cm.pages_for(length)
        first_needed = max(0, length - 6 + 1) // 4                   # the next query reads keys from length - 5
        assert [p >= 0 for p in table_win] == [i >= first_needed for i in range(len(table_win))]
        _check_invariants(cm, {})
    assert cm.pages_in_use(full) == 6 and cm.pages_in_use(win) <= 3
    cm.release("a")
    assert cm.pages_in_use() == 0


def test_state_slots_are_zeroed_at_admission():
    cm = _manager(extra={"s": FixedState((3,), "float32")})
    view = cm.view("s")
    assert tuple(view.state.shape) == (4, 3)
    slot = cm.admit("a")
    view.state[slot] += 5.0
    cm.release("a")
    assert cm.admit("b") == slot and torch.equal(view.state[slot], torch.zeros(3))
    assert cm.view(0).k.shape == (12, 2, 4, 8) and cm.view(0).group == ("window", 0)


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    cm = _manager(num_pages=14, window=5, poison=True)
    cm.shuffle_free_pages(seed)
    lengths, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        live = cm.live_requests()
        if action < 0.25 and cm.free_slots:
            cm.admit(next_id)
            lengths[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            asks = []
            for rid in rng.sample(live, rng.randint(1, len(live))):
                n = rng.randint(1, 9)
                if lengths[rid] + n <= 40:
                    asks.append((rid, n))
            before = {g: cm.pages_in_use(g) for g in cm.groups}
            try:
                cm.reserve(asks)
            except OutOfPages:
                assert {g: cm.pages_in_use(g) for g in cm.groups} == before       # nothing was taken
                continue
            for rid, n in asks:
                cm.advance(rid, n)
                lengths[rid] += n
        elif live:
            rid = rng.choice(live)
            cm.release(rid)
            del lengths[rid]
        _check_invariants(cm, lengths)
    cm.release_all()
    assert cm.pages_in_use() == 0 and cm.free_slots == 4


def test_a_spec_says_its_own_storage():
    """The manager allocates what a spec names and knows no spec by name: a spec of the test's own,
    with one tensor per page in a dtype of its own and a window, gets its pages, its group and its
    poison; a spec that says nothing of the kind is refused."""
    import dataclasses
    from bare_cuda_4gib_amd.cache import bytes_per_page
    from bare_cuda_4gib_amd.errors import EngineError

    @dataclasses.dataclass(frozen=True)
    class Latent:
        width: int
        window: int = 0
        per_token = True

        def page_tensors(self, page_tokens):
            return {"c": (page_tokens, self.width), "scale": ((page_tokens,), "float32")}

    @dataclasses.dataclass(frozen=True)
    class Counters:
        per_token = False

        def slot_tensors(self):
            return {"hits": ((2,), "int32"), "sum": ((5,), "float32")}

    cm = CacheManager({"kv": PagedKV(2, 8), "lat": Latent(6), "lat_w": Latent(3, window=9), "n": Counters()},
                      page_tokens=4, num_pages=10, max_requests=3, max_tokens=40, dtype=torch.bfloat16, device="cpu",
                      poison=True)
    lat, lat_w, n = cm.view("lat"), cm.view("lat_w"), cm.view("n")
    assert lat.c.shape == (10, 4, 6) and lat.c.dtype == torch.bfloat16 and lat.scale.dtype == torch.float32
    assert lat.group == cm.view("kv").group == ("window", 0) and lat_w.group == ("window", 9) and lat_w.window == 9
    assert torch.isnan(lat.c.float()).all() and torch.isnan(lat.scale).all()
    assert n.hits.shape == (3, 2) and n.hits.dtype == torch.int32 and not n.paged and lat.paged
    with pytest.raises(AttributeError, match="no tensor 'k'"):
        lat.k
    assert bytes_per_page(cm.specs.values(), 4, torch.bfloat16) == 2 * (2 * 4 * 8 * 2) + (4 * 6 * 2 + 4 * 4) + (4 * 3 * 2 + 4 * 4)
    slot = cm.admit("a")
    n.sum[slot] += 1.0
    cm.reserve([("a", 6)])
    cm.advance("a", 6)
    lat.c[cm.table(("window", 0), "a")[0]] = 1.0
    page = cm.table(("window", 0), "a")[0]
    cm.release("a")
    assert torch.isnan(lat.c[page].float()).all()                       # poisoned again when given back
    assert cm.admit("b") == slot and float(n.sum[slot].sum()) == 0.0     # zeroed at admission
    with pytest.raises(EngineError, match="neither"):
        CacheManager({"x": object()}, page_tokens=4, num_pages=2, max_requests=1, max_tokens=8, dtype=torch.float32, device="cpu")
