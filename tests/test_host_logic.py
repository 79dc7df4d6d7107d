"""Host logic through the C-ABI, no GPU: pool allocator invariants, LRU policy against the
restatement of the reference's LRUEvictor and against a brute-force model, and the
controller / executor state machine of a host-only engine (TP_FLAG_HOST_ONLY: no HIP calls, no
compute - ops are validated, tracked and recorded but not launched)."""
import ctypes as C
import random
import re

import numpy as np
import pytest

from oracle.host_ref import FixedBlocksRef, LruRef
from torpor_amd import _lib
from torpor_amd._lib import TorporError
from torpor_amd.functions import resnet
from torpor_amd.server import (ACK_INAVAIL, ACK_OK, OP_ADD, OP_COPY2D, OP_NCHW_TO_NHWC, OP_RELU, REQ_EXECUTE,
                               REQ_EXECUTE_AFTER_LOAD, REQ_LOAD,
                               REQ_UNLOAD, Server)

SLAB = 2 << 20
NOFIT = (1 << 64) - 1


# ---------------------------------------------------------------------------------- pool
class Pool:
    def __init__(self, cap, policy=None):
        self.l = _lib.lib()
        self.p = self.l.tp_pool_create(cap) if policy is None else self.l.tp_pool_create_policy(cap, policy)
        assert self.p

    def cached(self):
        b, n = C.c_uint64(), C.c_uint64()
        assert self.l.tp_pool_cached(self.p, C.byref(b), C.byref(n)) == 0
        return b.value, n.value

    def trim(self):
        return self.l.tp_pool_trim(self.p)

    def alloc(self, n):
        return self.l.tp_pool_alloc(self.p, n)

    def release(self, off):
        return self.l.tp_pool_release(self.p, off)

    def query(self):
        v = [C.c_uint64() for _ in range(5)]
        assert self.l.tp_pool_query(self.p, *[C.byref(x) for x in v]) == 0
        return dict(zip(("capacity", "used", "largest_free", "live", "free_extents"), [x.value for x in v]))

    def __del__(self):
        self.l.tp_pool_destroy(self.p)


def test_pool_basic_and_coalescing():
    p = Pool(16 * SLAB + 12345)             # capacity rounds down to whole slabs
    assert p.query()["capacity"] == 16 * SLAB
    a = p.alloc(1)                          # rounds up to one slab
    b = p.alloc(3 * SLAB)
    c = p.alloc(SLAB + 1)                   # two slabs
    assert (a, b, c) == (0, SLAB, 4 * SLAB)
    assert p.query()["used"] == 6 * SLAB
    assert p.release(b) == 0 and p.release(b) != 0          # double free is refused
    assert p.release(12345) != 0                            # not an extent start
    d = p.alloc(2 * SLAB)                   # best fit: the 3-slab hole, not the 10-slab tail
    assert d == SLAB
    assert p.release(a) == 0 and p.release(d) == 0 and p.release(c) == 0
    q = p.query()
    assert q["used"] == 0 and q["free_extents"] == 1 and q["largest_free"] == 16 * SLAB   # fully coalesced
    assert p.alloc(17 * SLAB) == NOFIT and p.alloc(16 * SLAB) == 0


def test_pool_random_invariants():
    """No overlap, inside the arena, slab aligned, used = sum of live extents, free + used =
    capacity, no two adjacent free extents (largest_free == capacity once everything is freed)."""
    rng = random.Random(0)
    cap = 64 * SLAB
    p = Pool(cap)
    live = {}
    for step in range(3000):
        if live and (rng.random() < 0.45 or len(live) > 20):
            off = rng.choice(list(live))
            assert p.release(off) == 0
            del live[off]
        else:
            n = rng.randint(1, 9 * SLAB)
            off = p.alloc(n)
            need = -(-n // SLAB) * SLAB
            if off == NOFIT:
                # refusal is only legal when no hole is large enough
                assert p.query()["largest_free"] < need
                continue
            assert off % SLAB == 0 and off + need <= cap
            for o, s in live.items():
                assert off + need <= o or o + s <= off, "extents overlap"
            live[off] = need
        q = p.query()
        assert q["used"] == sum(live.values()) and q["live"] == len(live)
    for off in list(live):
        assert p.release(off) == 0
    q = p.query()
    assert q["used"] == 0 and q["largest_free"] == cap and q["free_extents"] == 1


POOL_FIXED = 1


def test_fixed_blocks_restatement_on_a_hand_worked_trace():
    """Read off block_manager.hpp:188-258 by hand: budget 10; sizes in arbitrary units."""
    r = FixedBlocksRef(10)
    a, reused, freed = r.acquire(4)
    assert (a, reused, freed, r.budget) == (0, False, [], 6)
    b, _, _ = r.acquire(4)
    c, _, _ = r.acquire(2)
    assert (b, c, r.budget) == (1, 2, 0)
    r.evict(a, 4)
    r.evict(b, 4)
    r.evict(c, 2)
    assert r.acquire(4) == (b, True, [])                       # same size: the one released last, no budget change
    assert r.budget == 0
    # a size nobody has released: idle blocks are freed largest size first (the 4 before the 2) until it fits
    d, reused, freed = r.acquire(3)
    assert (reused, freed, r.budget) == (False, [(a, 4)], 1)
    e, reused, freed = r.acquire(3)                            # 1 + 2 covers it: the idle 2 goes
    assert (reused, freed, r.budget, r.over_budget) == (False, [(c, 2)], 0, 0)
    f, reused, freed = r.acquire(5)                            # nothing left to free: allocated beyond the budget
    assert (reused, freed, r.over_budget) == (False, [], 1)
    assert len({a, b, c, d, e, f}) == 6


def test_fixed_size_pool_matches_the_restatement_and_keeps_the_pool_invariants():
    """The fixed-size policy of the pool against FixedBlocksRef on random traces of a few recurring sizes
    (models come in a few sizes): a request served from the idle list gets the extent released last at
    that size in both; when a new size needs room, the idle extents given back are the restatement's, in
    its order, until the request fits (the pool may need more of them than the byte budget alone says,
    because its extents must be contiguous - never fewer); and the best-fit invariants hold throughout:
    no overlap, inside the arena, used = sum of live extents."""
    rng = random.Random(11)
    cap = 96 * SLAB
    sizes = [1 * SLAB, 3 * SLAB, 7 * SLAB, 12 * SLAB, 20 * SLAB]
    for trial in range(6):
        p = Pool(cap, POOL_FIXED)
        ref = FixedBlocksRef(cap)
        live = {}          # offset -> (size, ref block)
        where = {}         # ref block -> offset of the extent that stands for it
        reuses = trims = 0
        for step in range(1500):
            if live and (rng.random() < 0.5 or sum(s for s, _ in live.values()) > 0.8 * cap):
                off = rng.choice(sorted(live))
                sz, blk = live.pop(off)
                assert p.release(off) == 0
                ref.evict(blk, sz)
                continue
            sz = rng.choice(sizes)
            idle_before = {s: list(b) for s, b in ref.idle.items()}
            cached_before, n_before = p.cached()
            assert cached_before == ref.idle_bytes() and n_before == sum(len(b) for b in ref.idle.values())
            off = p.alloc(sz - rng.randint(0, SLAB - 1))        # any byte count that rounds to this size
            if idle_before.get(sz):
                blk, reused, freed = ref.acquire(sz)
                assert reused and off == where[blk], "the extent released last at this size is reused"
                live[off] = (sz, blk)
                reuses += 1
                continue
            # a new size: the order in which idle extents would go, largest size first, newest first
            order = [(b, s) for s in sorted(idle_before, reverse=True) for b in reversed(idle_before[s])]
            cached_after, n_after = p.cached()
            k = n_before - n_after
            assert cached_before - cached_after == sum(s for _, s in order[:k])
            # bring the restatement to the same state: it frees by bytes, the pool until a contiguous fit
            ref.budget = max(ref.budget, 0)
            for b, s in order[:k]:
                ref.idle[s].remove(b)
                ref.budget += s
                del where[b]
            trims += k
            if off == NOFIT:
                assert k == len(order), "refused only after every idle extent has been given back"
                assert p.query()["largest_free"] < sz
                continue
            blk = ref.next_block
            ref.next_block += 1
            ref.budget -= sz
            where[blk] = off
            live[off] = (sz, blk)
            assert off % SLAB == 0 and off + sz <= cap
            spans = sorted([(o, o + s) for o, (s, _) in live.items()] + [(where[b], where[b] + s) for s, bl in ref.idle.items() for b in bl])
            for (a0, a1), (b0, b1) in zip(spans, spans[1:]):
                assert a1 <= b0, "live and idle extents never overlap"
            q = p.query()
            assert q["used"] == sum(s for s, _ in live.values()) and q["live"] == len(live)
        assert reuses > 200 and trims > 5
        for off in list(live):
            assert p.release(off) == 0
        n_idle = p.cached()[1]
        assert p.trim() == n_idle and p.cached() == (0, 0)
        q = p.query()
        assert q["used"] == 0 and q["largest_free"] == cap and q["free_extents"] == 1


def test_host_only_engine_with_the_fixed_size_pool_reuses_a_models_extents(monkeypatch):
    """BLOCK_MANAGER=Fixed (memory_manager.hpp:46-52): a model swapped out and in again lands where it was,
    and the idle extents are visible in the pool statistics."""
    monkeypatch.setenv("BLOCK_MANAGER", "Fixed")
    with Server(mem_limit_bytes=1 << 30, pool_bytes=1 << 30, host_only=True) as s:
        _register(s, 0)
        _register(s, 1, seed=1)
        before = (s.model_info(0)["weight_off"], s.model_info(0)["act_off"])
        st0 = s.pool_stats()      # the per-allocation extents of the tracked runs wait in the idle lists already
        assert s.signal(REQ_UNLOAD, 0)[0] == ACK_OK
        st = s.pool_stats()
        assert st["pool_idle_extents"] == st0["pool_idle_extents"] + 2
        assert st["pool_cached_bytes"] == st0["pool_cached_bytes"] + s.model_info(0)["total_bytes"]
        assert st["used"] == st0["used"] - s.model_info(0)["total_bytes"]
        assert s.signal(REQ_LOAD, 0)[0] == ACK_OK
        assert (s.model_info(0)["weight_off"], s.model_info(0)["act_off"]) == before
        assert s.pool_stats()["pool_idle_extents"] == st0["pool_idle_extents"]


def test_pool_at_288_gb_with_ten_thousand_live_extents():
    """The arena of a whole MI355X (288 GB) full of small models: invariants hold, best fit agrees with a
    brute-force scan of the holes, and an allocation stays a tree search (the bound below is generous for a
    call through ctypes: a linear scan of ~10^4 holes would not meet it in the steady state)."""
    import time
    rng = random.Random(7)
    cap = 288 * 10 ** 9
    p = Pool(cap)
    cap = p.query()["capacity"]
    live = {}
    while True:                                  # fill it: 2 .. 20 MiB extents
        n = rng.randint(1, 10) * SLAB
        off = p.alloc(n)
        if off == NOFIT:
            break
        live[off] = n
    assert len(live) > 20000
    for off in rng.sample(sorted(live), len(live) // 2):   # punch ~12 000 holes
        assert p.release(off) == 0
        del live[off]
    q = p.query()
    assert q["live"] == len(live) >= 10000 and q["used"] == sum(live.values())
    assert q["free_extents"] > 5000

    def holes():
        out, pos = [], 0
        for off in sorted(live):
            if off > pos:
                out.append((pos, off - pos))
            pos = off + live[off]
        if pos < cap:
            out.append((pos, cap - pos))
        return out
    for _ in range(40):                          # best fit == brute force: smallest hole that fits, lowest address
        n = rng.randint(1, 30) * SLAB
        fit = [(ln, o) for o, ln in holes() if ln >= n]
        off = p.alloc(n)
        if not fit:
            assert off == NOFIT
            continue
        assert off == min(fit)[1]
        live[off] = n
    assert p.query()["largest_free"] == max(ln for _, ln in holes())
    ops = 20000
    offs = sorted(live)
    t0 = time.perf_counter()
    for i in range(ops):                         # steady state: release one, allocate one
        off = offs[(i * 7919) % len(offs)]
        if off in live:
            assert p.release(off) == 0
            n = live.pop(off)
            o2 = p.alloc(n)
            assert o2 != NOFIT
            live[o2] = n
    per_op_us = (time.perf_counter() - t0) / ops * 1e6
    assert per_op_us < 50.0, per_op_us
    srt = sorted(live.items())
    assert all(a[0] + a[1] <= b[0] for a, b in zip(srt, srt[1:])) and srt[-1][0] + srt[-1][1] <= cap
    assert p.query()["used"] == sum(live.values())
    assert p.alloc(cap + SLAB) == NOFIT and p.alloc((1 << 64) - 1) == NOFIT


def test_pool_layout_is_deterministic():
    seq = [(1, 5 * SLAB), (1, SLAB), (0, 0), (1, 2 * SLAB), (1, 7 * SLAB), (0, 1), (1, 3 * SLAB)]
    outs = []
    for _ in range(2):
        p, got, offs = Pool(32 * SLAB), [], []
        for kind, v in seq:
            if kind:
                offs.append(p.alloc(v))
                got.append(offs[-1])
            else:
                p.release(offs[v])
        outs.append(got)
    assert outs[0] == outs[1]


# ---------------------------------------------------------------------------------- LRU
class Lru:
    def __init__(self, budget):
        self.l = _lib.lib()
        self.p = self.l.tp_lru_create(budget)

    def check_and_add(self, f, sz):
        buf = C.create_string_buffer(4096)
        n, over = C.c_int32(), C.c_int32()
        assert self.l.tp_lru_check_and_add(self.p, f.encode(), sz, buf, 4096, C.byref(n), C.byref(over)) == 0
        v = buf.value.decode().split("\n") if buf.value else []
        assert len(v) == n.value
        return v, bool(over.value)

    def force_evict(self, f):
        return self.l.tp_lru_force_evict(self.p, f.encode())

    def lock(self, f):
        self.l.tp_lru_lock(self.p, f.encode())

    def unlock(self, f):
        self.l.tp_lru_unlock(self.p, f.encode())

    def used(self):
        return self.l.tp_lru_used(self.p)

    def __del__(self):
        self.l.tp_lru_destroy(self.p)


def test_lru_textbook_cases():
    l = Lru(100)
    assert l.check_and_add("a", 40) == ([], False)
    assert l.check_and_add("b", 40) == ([], False)
    assert l.check_and_add("a", 40) == ([], False)            # hit: a becomes most recent
    assert l.check_and_add("c", 40) == (["b"], False)         # 80 + 40 >= 100 -> evict the oldest = b
    assert l.used() == 80
    assert l.check_and_add("d", 20) == (["a"], False)         # '>=': 80 + 20 == budget still evicts
    l.lock("c")
    assert l.check_and_add("e", 60) == (["d"], True)          # c is locked: over budget, reported
    l.unlock("c")
    assert l.force_evict("zzz") == 0 and l.force_evict("e") == 1
    assert l.used() == 40


def test_lru_matches_reference_restatement_on_random_traces():
    for seed in range(5):
        rng = random.Random(seed)
        budget = 1000
        mine, ref = Lru(budget), LruRef(budget)
        brute = []          # brute-force model: list, most recent first
        sizes = {f"{i}": rng.randint(50, 400) for i in range(12)}
        for step in range(2000):
            f = str(rng.randrange(12))
            r = rng.random()
            if r < 0.8:
                got, _ = mine.check_and_add(f, sizes[f])
                want = ref.check_and_add(f, sizes[f])
                assert got == want, (seed, step)
                # brute force (no locks in this trace)
                if f in brute:
                    brute.remove(f)
                    exp = []
                else:
                    exp = []
                    while sum(sizes[x] for x in brute) + sizes[f] >= budget and brute:
                        exp.append(brute.pop())
                brute.insert(0, f)
                assert got == exp
            else:
                assert bool(mine.force_evict(f)) == ref.force_evict(f)
                if f in brute:
                    brute.remove(f)
            assert mine.used() == ref.cur == sum(sizes[x] for x in brute)
            assert mine.used() < budget or len(brute) == 1


def test_lru_locked_entries_are_never_evicted():
    rng = random.Random(7)
    mine, ref = Lru(500), LruRef(500)
    locked = set()
    for step in range(1500):
        f = str(rng.randrange(8))
        r = rng.random()
        if r < 0.6:
            got, _ = mine.check_and_add(f, 120)
            assert got == ref.check_and_add(f, 120)
            assert not (set(got) & locked)
        elif r < 0.8:
            mine.lock(f)
            ref.lock(f)
            if f in ref.items:
                locked.add(f)
        else:
            mine.unlock(f)
            ref.unlock(f)
            locked.discard(f)


# ---------------------------------------------------------------------------------- engine state machine
def _register(s, fid, image=32, seed=0):
    fn = resnet.ResNet(s, fid, "resnet50", batch=1, seed=seed, image=image)
    x = np.zeros((1, 3, image, image), np.float32)
    with pytest.raises(TorporError) as e:        # host-only: the request completes, but there is no data
        fn.register([x])
    assert e.value.code == -19
    return fn


@pytest.fixture(scope="module")
def host_server():
    s = Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20, request_timeout_ms=200)
    yield s
    s.close()


def test_register_invoke_unload_flow(host_server):
    s = host_server
    fn = _register(s, 0)
    info = s.model_info(0)
    assert info["registered"] and info["resident"] and info["n_params"] == 267 and info["n_ops"] == 58
    assert info["image_bytes"] % 256 == 0 and info["param_bytes"] == sum(v.nbytes for v in fn.weights().values())
    assert s.pool_stats()["lru_models"] == 1 and s.pool_stats()["live_extents"] == 2
    # Execute (resident) -> ack OK, gpu 0 ; ops from another client are refused while 0 is active
    assert s.signal(REQ_EXECUTE, 0, "") == (ACK_OK, 0, False)
    with pytest.raises(TorporError) as e:
        s.malloc(5, 64)
    assert e.value.code == -72
    # a second request while busy is queued: no ack yet (controller.hpp:177)
    assert s.signal(REQ_EXECUTE, 0, "")[2] is True
    assert s.take_deferred_ack() is None
    # Unload of the active function is refused
    assert s.signal(REQ_UNLOAD, 0, "")[0] == ACK_INAVAIL
    # the request ends with its async D2H (here through replay); the queued one is then started
    packed, outbuf, _ = fn.pack([np.zeros((1, 3, 32, 32), np.float32)])
    with pytest.raises(TorporError):
        s.replay(0, packed, outbuf)
    assert s.take_deferred_ack() == (ACK_OK, 0)
    with pytest.raises(TorporError):
        s.replay(0, packed, outbuf)
    assert s.take_deferred_ack() is None
    # Unload: ack OK, resp -1, pool back to empty, LRU forgets the model
    assert s.signal(REQ_UNLOAD, 0, "")[:2] == (ACK_OK, -1)
    st = s.pool_stats()
    assert not s.resident(0) and st["used"] == 0 and st["lru_models"] == 0 and st["free_extents"] == 1
    # Load = prefetch
    assert s.signal(REQ_LOAD, 0, "")[0] == ACK_OK and s.resident(0)
    assert s.signal(REQ_UNLOAD, 0, "")[0] == ACK_OK


def test_eviction_under_budget_and_deterministic_offsets(host_server):
    s = host_server
    fns = [_register(s, i, seed=i) for i in range(1, 5)]
    total = s.model_info(1)["total_bytes"]
    assert 3 * total < (330 << 20) <= 4 * total
    assert [s.resident(i) for i in range(1, 5)] == [False, True, True, True]
    ref = LruRef(330 << 20)
    for i in (2, 3, 4):
        ref.check_and_add(str(i), total)
    rng = random.Random(1)
    for step in range(200):
        i = rng.randint(1, 4)
        victims = ref.check_and_add(str(i), total)
        ack, resp, dfr = s.signal(REQ_EXECUTE, i, "")
        assert (ack, resp, dfr) == (ACK_OK, 0, False)
        for v in victims:
            assert not s.resident(int(v))
        assert s.resident(i)
        assert sorted(ref.items) == sorted(str(j) for j in range(1, 5) if s.resident(j))
        st = s.pool_stats()
        assert st["lru_used"] == ref.cur and st["used"] == len(ref.items) * total
        # extents of resident models never overlap
        ext = []
        for j in range(1, 5):
            if s.resident(j):
                mi = s.model_info(j)
                ext += [(mi["weight_off"], mi["image_bytes"]), (mi["act_off"], mi["act_bytes"])]
        ext.sort()
        for (a, n), (b, _) in zip(ext, ext[1:]):
            assert a + n <= b
        packed, outbuf, _ = fns[i - 1].pack([np.zeros((1, 3, 32, 32), np.float32)])
        with pytest.raises(TorporError):
            s.replay(i, packed, outbuf)
    for i in range(1, 5):
        s.signal(REQ_UNLOAD, i, "")
    assert s.pool_stats()["used"] == 0


def test_load_while_busy_never_evicts_the_running_model():
    """controller.hpp:208-215 accepts Load while an executor is busy; the model that is running must
    not be the victim of the eviction that makes room for it."""
    s = Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20, request_timeout_ms=60000)
    try:
        fns = [_register(s, i, seed=i) for i in range(1, 5)]
        assert [s.resident(i) for i in range(1, 5)] == [False, True, True, True]
        assert s.signal(REQ_EXECUTE, 2, "") == (ACK_OK, 0, False)       # LRU order, oldest first: 3, 4, 2
        for other in (1, 3, 4, 1, 3, 4):                                 # each Load evicts a model that is not 2
            assert s.signal(REQ_LOAD, other, "")[0] == ACK_OK
            assert s.resident(2) and s.resident(other)
            assert sum(s.resident(i) for i in range(1, 5)) == 3
        packed, outbuf, _ = fns[1].pack([np.zeros((1, 3, 32, 32), np.float32)])
        with pytest.raises(TorporError):
            s.replay(2, packed, outbuf)
        # once the request is over the model is an ordinary candidate again: 2 is the oldest entry now
        assert s.signal(REQ_LOAD, 1, "")[0] == ACK_OK
        assert not s.resident(2)
    finally:
        s.close()


def test_executor_log_has_the_reference_sections(tmp_path, monkeypatch):
    """EXECUTOR_LOG_LEVEL (cuda_server.hpp:61-69) switches on log_executor_<gpu>.txt with the sections the
    reference times: CheckMalloc (memory_manager.hpp:499-501), Evict (258), request completion
    (cuda_server.hpp:294-295).  Unset, the engine writes nothing."""
    monkeypatch.setenv("TORPOR_LOG_DIR", str(tmp_path))
    monkeypatch.delenv("EXECUTOR_LOG_LEVEL", raising=False)
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20):
        pass
    assert not list(tmp_path.iterdir())
    monkeypatch.setenv("EXECUTOR_LOG_LEVEL", "info")
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20) as s:
        fn = _register(s, 7)
        assert s.signal(REQ_UNLOAD, 7, "")[0] == ACK_OK
        assert s.signal(REQ_EXECUTE, 7, "") == (ACK_OK, 0, False)
        packed, outbuf, _ = fn.pack([np.zeros((1, 3, 32, 32), np.float32)])
        with pytest.raises(TorporError):
            s.replay(7, packed, outbuf)
    text = (tmp_path / "log_executor_0.txt").read_text()
    lines = text.splitlines()
    assert all(re.match(r"\[\d{4}-\d\d-\d\d \d\d:\d\d:\d\d\.\d{6}\] \[info\] ", ln) for ln in lines), text
    order = [next(i for i, ln in enumerate(lines) if key in ln) for key in
             ("Executor 0 started", "Evict model 7 elasped", "CheckMalloc model 7 elasped", "Request of model 7 completed in")]
    assert order == sorted(order)
    assert "(swapped in)" in lines[order[-1]]
    monkeypatch.setenv("EXECUTOR_LOG_LEVEL", "err")      # info lines are below this level
    (tmp_path / "log_executor_0.txt").unlink()
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20) as s:
        _register(s, 8)
        s.signal(REQ_UNLOAD, 8, "")
    assert (tmp_path / "log_executor_0.txt").read_text() == ""


def _register_level(s, fid, level):
    fn = resnet.ResNet(s, fid, "resnet50", batch=1, seed=fid, image=32, level=level)
    with pytest.raises(TorporError):
        fn.register([np.zeros((1, 3, 32, 32), np.float32)])
    return fn


def test_model_levels_select_the_two_class_policy_or_plain_lru():
    """controller.hpp:103-109, 142-152: by default a light model (level 0) is evicted before median / heavy
    ones whatever its recency; with the LRU policy the level is ignored."""
    for lru in (False, True):
        s = Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20, request_timeout_ms=200,
                   evict_lru=lru)
        f1 = _register_level(s, 1, 1)
        _register_level(s, 2, 2), _register_level(s, 3, 0)
        assert [s.resident(i) for i in (1, 2, 3)] == [True, True, True]
        assert s.signal(REQ_EXECUTE, 1, "")[0] == ACK_OK      # recency now 2 < 3 < 1; the budget holds three models
        packed, outbuf, _ = f1.pack([np.zeros((1, 3, 32, 32), np.float32)])
        with pytest.raises(TorporError):                      # host-only: completes the request without data
            s.replay(1, packed, outbuf)
        _register_level(s, 4, 1)
        # two-class: the light model 3 goes although 2 is older; LRU: the oldest, 2
        assert [s.resident(i) for i in (1, 2, 3, 4)] == ([True, False, True, True] if lru else [True, True, False, True])
        s.close()


def test_tables_looked_up_by_index_are_last_in_the_image():
    """First-access order (model_repo.hpp:102-109) with one exception: the word-embedding table,
    read first but only a few rows of it, follows every tensor the forward pass streams through.
    The other embedding operands (position and type tables, LayerNorm) keep their early place."""
    from torpor_amd.functions import bert
    cfg = dict(layers=2, hidden=64, heads=2, ffn=128)
    weights = bert.init_weights(seed=1, vocab=500, max_pos=32, cfg=cfg)
    with Server(host_only=True, mem_limit_bytes=64 << 20, pool_bytes=128 << 20) as s:
        fn = bert.Bert(s, 0, batch=1, seq=16, weights=weights, cfg=cfg)
        with pytest.raises(TorporError) as e:
            fn.register([np.zeros((1, 16), np.int64)])
        assert e.value.code == -19
        off = {k: s.weight_offset(0, va) for k, va in fn.w.items()}
        assert off["embeddings.word_embeddings.weight"] == max(off.values())
        assert off["embeddings.position_embeddings.weight"] == 0
        first_layer = min(v for k, v in off.items() if k.startswith("encoder.layer.0."))
        assert off["embeddings.LayerNorm.weight"] < first_layer
        last = max(v for k, v in off.items() if k.startswith("pooler."))
        assert last < off["embeddings.word_embeddings.weight"]


def test_pinned_result_buffers_are_tracked(host_server):
    import ctypes as C
    from torpor_amd import _lib
    L, h = _lib.lib(), host_server._h
    p = C.c_void_p()
    assert L.tp_host_alloc(h, 0, C.byref(p)) == -22 and L.tp_host_alloc(h, 64, None) == -22
    assert L.tp_host_alloc(h, 4096, C.byref(p)) == 0 and p.value
    a = host_server.host_empty(100)
    a[:] = 7
    assert a.sum() == 700
    assert L.tp_host_free(h, C.c_void_p(p.value + 8)) == -22      # not the start of a buffer
    assert L.tp_host_free(h, p) == 0 and L.tp_host_free(h, p) == -22
    # the device expansion hook needs a device
    w = np.zeros(8, np.uint32)
    payload = np.zeros(216, np.uint8)
    tab = np.zeros(1, np.uint32)
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 8, 0, None, 0, tab.ctypes.data, 0, 8, w.ctypes.data) == -19


def test_request_timeout_completes_the_request(host_server):
    """cuda_server.hpp:257-264: an Execute that sends no ops is force-completed after the timeout
    (200 ms here) and the executor becomes available again."""
    import time
    s = host_server
    _register(s, 10)
    assert s.signal(REQ_EXECUTE, 10, "")[0] == ACK_OK
    assert s.signal(REQ_EXECUTE, 10, "")[2] is True          # busy -> queued
    assert not s.poll()
    time.sleep(0.25)
    assert s.poll()                                          # timed out, completed, queued one started
    assert s.take_deferred_ack() == (ACK_OK, 0)
    time.sleep(0.25)
    assert s.poll()
    assert s.signal(REQ_UNLOAD, 10, "")[0] == ACK_OK


def test_error_paths(host_server):
    s = host_server
    assert s.signal(REQ_EXECUTE, 777, "")[0] == ACK_INAVAIL          # never registered
    assert s.signal(REQ_LOAD, 777, "")[0] == ACK_INAVAIL
    assert s.signal(REQ_UNLOAD, 777, "")[:2] == (ACK_OK, -1)
    assert s.signal(10, 1, "")[0] == ACK_INAVAIL                     # ExecuteForRecord is refused
    assert s.signal(11, 1, "")[0] == ACK_INAVAIL                     # Replay signal is refused
    with pytest.raises(TorporError):
        s.signal(REQ_EXECUTE, "abc", "")                             # function must be a decimal id
    with pytest.raises(TorporError) as e:
        s.signal(REQ_EXECUTE_AFTER_LOAD, 65536, "1")                 # ids are 0 .. 65535
    assert e.value.code == -34 and "range" in str(e.value)
    assert s.signal(REQ_EXECUTE, 65535, "")[0] == ACK_INAVAIL        # in range, never registered
    with pytest.raises(TorporError):
        s.malloc(0, 16)                                              # no active function
    # registration: ops before the end of the upload phase are refused; uploads outside a block too
    assert s.signal(REQ_EXECUTE_AFTER_LOAD, 20, "2")[0] == ACK_OK
    va = s.malloc(20, 1024)
    s.h2d(20, va, np.arange(256, dtype=np.float32))
    with pytest.raises(TorporError):
        s.h2d(20, va + 512, np.zeros(256, np.float32))               # runs past the block
    with pytest.raises(TorporError):
        s.launch(20, OP_RELU, [va, va], [4])                         # still uploading
    with pytest.raises(TorporError):
        s.device_synchronize(20)       # ends the upload phase, and reports the refused ops above (once)
    assert s.model_info(20)["level"] == 2
    act = s.malloc(20, 1024)
    with pytest.raises(TorporError):
        s.h2d(20, va, np.zeros(4, np.float32))                       # weights are read-only after registration
    with pytest.raises(TorporError):
        s.free(20, va)                                               # freeing a model block is refused
    s.launch(20, OP_RELU, [va, act], [256])
    with pytest.raises(TorporError):
        s.launch(20, OP_RELU, [va, act], [257])                      # longer than the buffers
    with pytest.raises(TorporError):
        s.launch(20, OP_RELU, [va, 0x1234], [4])                     # not an address of this server
    s.free(20, act)
    with pytest.raises(TorporError):
        s.launch(20, OP_RELU, [va, act], [4])                        # freed
    out = np.empty(4, np.float32)
    act = s.malloc(20, 1024)
    s.d2h_async(20, out, act)
    with pytest.raises(TorporError):
        s.stream_synchronize(20)                                     # sticky op errors + no device
    assert s.model_info(20)["registered"] == 1
    assert s.signal(REQ_UNLOAD, 20, "")[0] == ACK_OK


def test_arguments_whose_spans_would_wrap_are_refused(host_server):
    """Element counts and byte counts arrive unvalidated from wire clients; their products must not wrap
    into a span that passes the bounds test (64-bit products of dims, off + span, the cast of a byte count
    to a signed 64-bit integer)."""
    s = host_server
    assert s.signal(REQ_EXECUTE_AFTER_LOAD, 21, "1")[0] == ACK_OK
    w = s.malloc(21, 1024)
    s.h2d(21, w, np.zeros(256, np.float32))
    s.device_synchronize(21)   # the upload phase ends
    a = s.malloc(21, 1024)
    b = s.malloc(21, 1024)

    def refused(fn, *args, **kw):
        with pytest.raises(TorporError) as e:
            fn(*args, **kw)
        assert e.value.code in (-22, -14, -12, -38), e.value.code
    s.launch(21, OP_RELU, [a, b], [256])
    refused(s.launch, 21, OP_RELU, [a, b], [257])
    refused(s.launch, 21, OP_RELU, [a, b], [1 << 62])            # 2^62 elements x 4 bytes = 2^64
    refused(s.launch, 21, OP_RELU, [a, b], [(1 << 62) + 1])
    refused(s.launch, 21, OP_NCHW_TO_NHWC, [a, b], [1 << 16] * 4)  # N*C*H*W = 2^64
    refused(s.launch, 21, OP_NCHW_TO_NHWC, [a, b], [1 << 15, 1 << 16, 1 << 16, 1 << 16])
    refused(s.launch, 21, OP_NCHW_TO_NHWC, [a, b], [(1 << 32) + 1, 1, 1, 1])   # would be narrowed to int 1
    refused(s.launch, 21, OP_COPY2D, [a, b], [1 << 40, 4, 1 << 40, 1 << 40])
    refused(s.launch, 21, OP_ADD, [a, b, a], [-1, 0])
    refused(s.d2d, 21, a, b, (1 << 64) - 1)
    refused(s.d2d, 21, a, b, (1 << 63) + 16)
    refused(s.d2d, 21, a + 8, b, (1 << 64) - 4)                  # off + span wraps to a small value
    refused(s.memset, 21, a, 0, (1 << 64) - 1)
    refused(s.memset, 21, a + 16, 0, (1 << 64) - 8)
    refused(s.malloc, 21, (1 << 64) - 1)
    refused(s.gemm, 21, a, w, b, 1 << 31, 1 << 31, 4, xs_r=4, ys_c=4, ldc=1 << 31)
    refused(s.gemm, 21, a, w, b, 4, 4, 4, xs_r=(1 << 62), ys_c=4, ldc=4)
    refused(s.gemm, 21, a, w, b, 2, 2, 2, xs_r=2, ys_c=2, ldc=2, nb0=1 << 20, nb1=1 << 20)
    refused(s.conv, 21, a, w, b, 1 << 20, 1 << 20, 1 << 20, 1 << 4, 1, 1, 1)
    refused(s.bn, 21, a, b, w, w, w, w, 1e-5, 1 << 50, 4)
    s.d2d(21, a, b, 1024)                                         # what fits still passes
    s.memset(21, a, 0, 1024)
    s.gemm(21, a, w, b, 4, 4, 4, xs_r=4, ys_c=4, ldc=4)
    out = np.empty(4, np.float32)
    s.d2h_async(21, out, a)
    with pytest.raises(TorporError):
        s.stream_synchronize(21)
    assert s.signal(REQ_UNLOAD, 21, "")[0] == ACK_OK


def test_deferred_acks_carry_tickets_and_can_be_cancelled():
    """Queued signals are matched to their acks by ticket; a cancelled ticket never produces an ack, and a
    request that had been started for a peer that is gone is completed at once (controller.hpp:242-262 hands
    the executor to the oldest queued signal)."""
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20, request_timeout_ms=60000) as s:
        fns = {fid: _register(s, fid) for fid in (1, 2, 3, 4)}
        assert s.signal_ticket(REQ_EXECUTE, 1)[:3] == (ACK_OK, 0, False)
        t2 = s.signal_ticket(REQ_EXECUTE, 2)
        t3 = s.signal_ticket(REQ_EXECUTE, 3)
        t4 = s.signal_ticket(REQ_EXECUTE, 4)
        assert [t[2] for t in (t2, t3, t4)] == [True] * 3
        assert t2[3] < t3[3] < t4[3] and t2[3] >= 1
        assert s.take_deferred_ack_ticket() is None
        # the peer of the first queued signal goes away while still queued: no ack for it, ever
        assert s.cancel_deferred(t2[3]) == 1
        assert s.cancel_deferred(t2[3]) == 0
        assert s.cancel_deferred(12345) == 0
        x = np.zeros((1, 3, 32, 32), np.float32)

        def drive(fid):     # the data plane of a request that the engine has already started
            packed, outbuf, _ = fns[fid].pack([x])
            with pytest.raises(TorporError) as e:
                s.replay(fid, packed, outbuf)
            assert e.value.code == -19              # host-only: the request completes, there is no data
        drive(1)
        assert s.take_deferred_ack_ticket() == (ACK_OK, 0, t3[3])   # function 3 was started, not 2
        assert s.take_deferred_ack_ticket() is None
        with pytest.raises(TorporError) as e:
            s.malloc(2, 64)
        assert e.value.code == -72                  # function 2 is not the active one
        assert s.check_address(2, 0, 4) == -72
        assert s.check_address(3, 0x1234, 4) == -14
        # function 3 finishes, function 4 is started; its peer disappears before the ack is taken:
        drive(3)
        assert s.cancel_deferred(t4[3]) == 2        # ack dropped, the started request completed at once
        assert s.take_deferred_ack_ticket() is None
        assert s.signal_ticket(REQ_EXECUTE, 1)[:3] == (ACK_OK, 0, False)   # the executor is free again


def test_an_ack_that_could_not_be_delivered_withdraws_the_request_it_started():
    """A front end takes the ack of a queued signal and then finds the peer gone (or the send fails).  The
    request was started for nobody: tp_cancel_deferred on its ticket completes it at once -- an Execute
    would otherwise hold the executor until the request timeout, a queued registration for good (no
    timeout applies while a model is being uploaded) -- and forgets a half-made registration."""
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20, request_timeout_ms=60000) as s:
        fns = {fid: _register(s, fid) for fid in (1, 2)}
        x = np.zeros((1, 3, 32, 32), np.float32)

        def drive(fid):
            packed, outbuf, _ = fns[fid].pack([x])
            with pytest.raises(TorporError):
                s.replay(fid, packed, outbuf)
        used0 = s.pool_stats()["used"]
        assert s.signal_ticket(REQ_EXECUTE, 1)[:3] == (ACK_OK, 0, False)
        t_exec = s.signal_ticket(REQ_EXECUTE, 2)            # queued behind function 1
        t_reg = s.signal_ticket(REQ_EXECUTE_AFTER_LOAD, 9, "1")   # a registration queued behind that
        assert t_exec[2] and t_reg[2]
        drive(1)
        assert s.take_deferred_ack_ticket() == (ACK_OK, 0, t_exec[3])   # function 2 started, ack handed out ...
        assert s.cancel_deferred(t_exec[3]) == 2                         # ... and could not be delivered
        assert s.cancel_deferred(t_exec[3]) == 0
        # the executor went on to the queued registration; its ack meets the same fate after an upload
        assert s.take_deferred_ack_ticket() == (ACK_OK, 0, t_reg[3])
        va = s.malloc(9, 4096)
        s.h2d(9, va, np.ones(1024, np.float32))
        assert s.cancel_deferred(t_reg[3]) == 2
        with pytest.raises(TorporError) as e:
            s.model_info(9)
        assert e.value.code == -2                            # the half-made model is forgotten
        assert s.pool_stats()["used"] == used0
        assert s.signal_ticket(REQ_EXECUTE, 1)[:3] == (ACK_OK, 0, False)   # the executor is free again
        drive(1)
        # a ticket whose request has ended by itself is no longer known
        t_late = s.signal_ticket(REQ_EXECUTE, 1)
        assert not t_late[2]
        assert s.cancel_deferred(t_exec[3]) == 0


def test_function_ids_up_to_65535_register_and_run():
    with Server(host_only=True, mem_limit_bytes=330 << 20, pool_bytes=512 << 20) as s:
        fn = _register(s, 65535, seed=1)
        assert s.model_info(65535)["registered"] == 1 and s.resident(65535)
        assert (fn.w["conv1.weight"] >> 40) & 0xFFFF == 65535       # the id travels in every address
        assert s.signal(REQ_UNLOAD, 65535, "")[0] == ACK_OK and not s.resident(65535)
        assert s.signal(REQ_LOAD, 65535, "")[0] == ACK_OK and s.resident(65535)
