"""Control-plane policy objects for several GPUs (decision logic only; runs on the CPU):
the two-class interference-aware evictor (evictor.hpp:28-188) and the placement / scheduling
decisions of the controller (controller.hpp:271-389), through the C-ABI, against the
restatements in oracle/host_ref.py and against what the policies' definitions fix."""
import ctypes as C
import itertools
import random

import numpy as np

import pytest

from oracle.host_ref import IaRef, LruRef, SchedRef
from torpor_amd import _lib

LRU, IA = 0, 1
RANDOM_POLICY, IA_POLICY = 0, 1


class Evictor:
    def __init__(self, policy, gpus, budget):
        self.l = _lib.lib()
        self.h = self.l.tp_evictor_create(policy, gpus, budget)
        assert self.h

    def __del__(self):
        self.l.tp_evictor_destroy(self.h)

    def set_level(self, f, lv):
        assert self.l.tp_evictor_set_level(self.h, f.encode(), lv) == 0

    def check_and_add(self, gpu, f, sz):
        buf = C.create_string_buffer(4096)
        n, over = C.c_int32(), C.c_int32()
        assert self.l.tp_evictor_check_and_add(self.h, gpu, f.encode(), sz, buf, 4096, C.byref(n), C.byref(over)) == 0
        v = buf.value.decode().split("\n") if buf.value else []
        assert len(v) == n.value
        return v, bool(over.value)

    def force_evict(self, gpu, f):
        return self.l.tp_evictor_force_evict(self.h, gpu, f.encode())

    def lock(self, gpu, f):
        assert self.l.tp_evictor_lock(self.h, gpu, f.encode()) == 0

    def unlock(self, gpu, f):
        assert self.l.tp_evictor_unlock(self.h, gpu, f.encode()) == 0

    def used(self, gpu):
        return self.l.tp_evictor_used(self.h, gpu)

    def protected(self, gpu, f):
        return self.l.tp_evictor_is_protected(self.h, gpu, f.encode()) == 1

    def order(self, gpu):
        buf = C.create_string_buffer(4096)
        n = self.l.tp_evictor_order(self.h, gpu, buf, 4096)
        v = buf.value.decode().split("\n") if buf.value else []
        assert len(v) == n
        return v


# ------------------------------------------------------------------------------------------ evictor
class _Both:
    """Drives the library and the restatement together; the expected values in the test are hand-derived."""

    def __init__(self, gpus, budget):
        self.e, self.ref = Evictor(IA, gpus, budget), IaRef(gpus, budget)

    def set_level(self, f, lv):
        self.e.set_level(f, lv)
        self.ref.level[f] = lv

    def check_and_add(self, g, f, sz):
        got = self.e.check_and_add(g, f, sz)
        assert got[0] == self.ref.check_and_add(g, f, sz)
        return got

    def order(self, g):
        assert self.e.order(g) == self.ref.order(g)
        return self.e.order(g)

    def used(self, g):
        assert self.e.used(g) == self.ref.cur[g]
        return self.e.used(g)

    def protected(self, g, f):
        assert self.e.protected(g, f) == any(x[0] == f for x in self.ref.first[g])
        return self.e.protected(g, f)


def test_ia_hand_worked_two_gpu_trace():
    """Expected victims worked out from the policy's definition with explicit sums."""
    e = _Both(2, 100)
    for f, lv in (("L", 0), ("M", 1), ("H", 2), ("N", 1)):
        e.set_level(f, lv)
    for f in ("M", "L", "H"):
        assert e.check_and_add(0, f, 30) == ([], False)      # 0, 30, 60 (+30) < 100
    assert e.check_and_add(1, "M", 30) == ([], False)
    assert not e.protected(0, "M") and not e.protected(1, "M") and e.protected(0, "H")
    assert e.check_and_add(0, "N", 20) == (["L"], False)     # 90+20 >= 100 -> L ; 60+20 < 100
    assert e.used(0) == 80
    # 80+40 >= 100 -> M (unprotected, older than nothing else unprotected); 50+40 = 90 < 100 -> stop
    assert e.check_and_add(0, "L", 40) == (["M"], False)
    assert e.protected(1, "M")                               # the copy on GPU 1 is the last one
    assert e.order(0) == ["L", "H", "N"]                     # light first, then protected by recency
    # 90+30 >= 100 -> L ; 50+30 < 100
    assert e.check_and_add(0, "M", 30) == (["L"], False)
    assert not e.protected(1, "M") and not e.protected(0, "M")
    assert e.order(0) == ["M", "H", "N"]


def test_ia_equals_lru_on_one_gpu_with_one_level():
    """One GPU and a single level: only one of the two classes is ever used, so the policy is LRU."""
    for level in (0, 1, 2):
        rng = random.Random(level)
        ia, ia_ref, lru = Evictor(IA, 1, 1000), IaRef(1, 1000), LruRef(1000)
        lru_c = Evictor(LRU, 1, 1000)
        sizes = {str(i): rng.randint(50, 400) for i in range(12)}
        for f in sizes:
            ia.set_level(f, level)
            ia_ref.level[f] = level
        for step in range(3000):
            f = str(rng.randrange(12))
            r = rng.random()
            if r < 0.7:
                want = lru.check_and_add(f, sizes[f])
                assert ia_ref.check_and_add(0, f, sizes[f]) == want, (level, step)
                assert ia.check_and_add(0, f, sizes[f])[0] == want, (level, step)
                assert lru_c.check_and_add(0, f, sizes[f])[0] == want
            elif r < 0.85:
                want = lru.force_evict(f)
                assert ia_ref.force_evict(0, f) == want
                assert bool(ia.force_evict(0, f)) == want
                assert bool(lru_c.force_evict(0, f)) == want
            elif r < 0.93:
                if f in lru.items:          # the LRU policy ignores a lock on an untracked name, the two-class one keeps it
                    lru.lock(f), ia_ref.lock(0, f), ia.lock(0, f), lru_c.lock(0, f)
            else:
                lru.unlock(f), ia_ref.unlock(0, f), ia.unlock(0, f), lru_c.unlock(0, f)
            assert ia.used(0) == lru.cur == ia_ref.cur[0] == lru_c.used(0)
        assert ia.order(0) == list(lru.items) == lru_c.order(0)


@pytest.mark.parametrize("gpus", [2, 4, 8])
def test_ia_random_traces_match_restatement_and_invariants(gpus):
    for seed in range(4):
        rng = random.Random(100 * gpus + seed)
        budget = 1000
        e, ref = Evictor(IA, gpus, budget), IaRef(gpus, budget)
        names = [str(i) for i in range(16)]
        sizes = {f: rng.randint(60, 380) for f in names}
        for f in names:
            lv = rng.randrange(3)
            e.set_level(f, lv)
            ref.level[f] = lv
        forced = False
        for step in range(4000):
            g, f, r = rng.randrange(gpus), rng.choice(names), rng.random()
            if r < 0.75:
                got, over = e.check_and_add(g, f, sizes[f])
                assert got == ref.check_and_add(g, f, sizes[f]), (seed, step)
                assert not (set(got) & ref.locked[g])
                if over:            # nothing unlocked was left to evict
                    assert all(x in ref.locked[g] for x in ref.order(g) if x != f)
            elif r < 0.80 and seed >= 2:
                assert bool(e.force_evict(g, f)) == ref.force_evict(g, f)
                forced = True
            elif r < 0.90:
                e.lock(g, f), ref.lock(g, f)
            else:
                e.unlock(g, f), ref.unlock(g, f)
            if step % 50 == 0 or step > 3950:
                for k in range(gpus):
                    assert e.order(k) == ref.order(k), (seed, step, k)
                    assert e.used(k) == ref.cur[k] == sum(s for _, s in ref.first[k] + ref.second[k])
                # the policy's definition: a tracked model of level >= 1 is protected exactly when one GPU
                # holds it (force_evict does not re-classify the surviving copy, so only without it)
                if not forced:
                    for f2 in names:
                        holders = [k for k in range(gpus) if f2 in e.order(k)]
                        for k in holders:
                            assert e.protected(k, f2) == (ref.level[f2] >= 1 and len(holders) == 1), (seed, step, f2)


def test_ia_all_locked_reports_over_budget_instead_of_spinning():
    e = Evictor(IA, 1, 100)
    e.set_level("a", 2), e.set_level("b", 2)
    assert e.check_and_add(0, "a", 60) == ([], False)
    e.lock(0, "a")
    assert e.check_and_add(0, "b", 60) == ([], True)     # the reference would never return (evictor.hpp:85-97)
    assert e.used(0) == 120
    e.unlock(0, "a")
    assert e.check_and_add(0, "c", 10) == (["a"], False)        # 120+10 >= 100 -> a ; 60+10 < 100


def test_evictor_argument_errors():
    l = _lib.lib()
    assert not l.tp_evictor_create(7, 1, 100) and not l.tp_evictor_create(IA, 0, 100)
    e = Evictor(IA, 2, 100)
    n = C.c_int32()
    assert l.tp_evictor_check_and_add(e.h, 2, b"a", 1, None, 0, C.byref(n), None) == -22
    assert l.tp_evictor_force_evict(e.h, -1, b"a") == -22
    assert l.tp_evictor_used(e.h, 9) == 0


# ---------------------------------------------------------------------------------------- scheduler
class Sched:
    def __init__(self, gpus, sibling=None, link=None):
        self.l = _lib.lib()
        self.h = self.l.tp_sched_create(gpus)
        assert self.h
        if sibling:
            for g, o in enumerate(sibling):
                assert self.l.tp_sched_set_sibling(self.h, g, o) == 0
        if link:
            for a, row in enumerate(link):
                for b, k in enumerate(row):
                    assert self.l.tp_sched_set_link(self.h, a, b, k) == 0

    def __del__(self):
        self.l.tp_sched_destroy(self.h)

    def decide(self, policy, f, draw=0):
        d, s, st = C.c_int32(), C.c_int32(), C.c_int32()
        assert self.l.tp_sched_decide(self.h, policy, f.encode(), draw, C.byref(d), C.byref(s), C.byref(st)) == 0
        return d.value, s.value, st.value


REF_SIBLING = (1, 0, 3, 2)                                                   # controller.hpp:117
REF_LINK = ((0, 1, 1, 2), (1, 0, 2, 1), (1, 2, 0, 2), (2, 1, 2, 0))          # controller.hpp:118


def _pair(statuses, resident, levels):
    s, ref = Sched(4, REF_SIBLING, REF_LINK), SchedRef()
    for g, st in enumerate(statuses):
        assert s.l.tp_sched_set_status(s.h, g, st) == 0
        ref.status[g] = st
    for f, gs in resident.items():
        for g in gs:
            s.l.tp_sched_set_resident(s.h, f.encode(), g, 1)
        ref.resident[f] = set(gs)
    for f, lv in levels.items():
        s.l.tp_sched_set_level(s.h, f.encode(), lv)
        ref.level[f] = lv
    return s, ref


def test_schedule_hand_worked_cases_on_the_reference_topology():
    A = -1
    # resident on an idle GPU: run there, no swap
    s, _ = _pair([0, A, A, A], {"f": [2]}, {"f": 2})
    assert s.decide(IA_POLICY, "f") == (2, -1, 0) and s.decide(RANDOM_POLICY, "f", 5) == (2, -1, 0)
    # resident only on busy GPU 0; idle 1, 2, 3; the fast links of 0 go to 3 only -> copy 0 -> 3
    s, _ = _pair([0, A, A, A], {"f": [0]}, {"f": 2})
    assert s.decide(IA_POLICY, "f") == (3, 0, 1)
    # no fast link between any idle GPU and a holder: first idle GPU, lowest holder
    s, _ = _pair([0, A, 3, 3], {"f": [0]}, {"f": 1})
    assert s.decide(IA_POLICY, "f") == (1, 0, 1)
    # holders 0 and 1 busy, idle 2 and 3: GPU 2 is fast to 1, GPU 3 is fast to 0; the last idle GPU's pair is kept
    s, _ = _pair([0, 0, A, A], {"f": [0, 1]}, {"f": 1})
    assert s.decide(IA_POLICY, "f") == (3, 0, 1)
    # nowhere resident: host swap on the idle GPU whose PCIe sibling is least busy.  idle 1 (sibling 0 runs a
    # heavy swap = 4) and 3 (sibling 2 runs locally = 0) -> GPU 3; the status is the model's level + 2
    s, _ = _pair([4, A, 0, A], {}, {"f": 2, "g": 0})
    assert s.decide(IA_POLICY, "f") == (3, -1, 4) and s.decide(IA_POLICY, "g") == (3, -1, 2)
    # an idle sibling (-1) beats everything; ties keep the first
    s, _ = _pair([A, A, 0, A], {}, {"f": 1})
    assert s.decide(IA_POLICY, "f") == (0, -1, 3)
    # random policy: the draw indexes the idle GPUs
    s, _ = _pair([0, A, 0, A], {}, {"f": 1})
    assert s.decide(RANDOM_POLICY, "f", 0) == (1, -1, 3) and s.decide(RANDOM_POLICY, "f", 7) == (3, -1, 3)
    # nothing idle
    s, _ = _pair([0, 1, 2, 3], {"f": [1]}, {"f": 1})
    assert s.decide(IA_POLICY, "f") == (-1, -1, -1) and s.decide(RANDOM_POLICY, "f", 1) == (-1, -1, -1)


def test_schedule_exhaustive_against_restatement_and_properties():
    """Every assignment of {idle, local, heavy swap} to 4 executors x every residency set."""
    for statuses in itertools.product([-1, 0, 4], repeat=4):
        for mask in range(16):
            holders = [g for g in range(4) if mask >> g & 1]
            s, ref = _pair(list(statuses), {"f": holders} if holders else {}, {"f": 1})
            idle = [g for g in range(4) if statuses[g] == -1]
            for draw in (0, 1, 2, 3):
                assert s.decide(RANDOM_POLICY, "f", draw) == ref.random_schedule("f", draw)
            got = s.decide(IA_POLICY, "f")
            assert got == ref.interference_aware_schedule("f"), (statuses, holders)
            dst, src, st = got
            if not idle:
                assert got == (-1, -1, -1)
                continue
            assert dst in idle                                   # never a busy executor
            local = [g for g in holders if g in idle]
            if local:
                assert got == (local[0], -1, 0)                  # resident and idle always wins
            elif holders:
                assert st == 1 and src in holders and src not in idle
                fast = [(i, j) for i in idle for j in holders if REF_LINK[i][j] == 2]
                assert (REF_LINK[dst][src] == 2) == bool(fast)   # a fast link is used whenever one exists
            else:
                assert src == -1 and st == 3
                assert statuses[REF_SIBLING[dst]] == min(statuses[REF_SIBLING[g]] for g in idle)


def test_placement_round_robin():
    s, ref = Sched(4), SchedRef()
    seq = []
    for step in range(12):
        if step == 5:
            s.l.tp_sched_set_status(s.h, 2, 5), s.l.tp_sched_set_status(s.h, 1, 5)
            ref.status[2] = ref.status[1] = 5
        g = s.l.tp_sched_placement(s.h)
        assert g == ref.placement()
        seq.append(g)
    # 0 1 2 3 0 | cursor at 1 which is busy -> first idle = 0, cursor stays
    assert seq[:5] == [0, 1, 2, 3, 0] and seq[5:8] == [0, 0, 0]
    for g in range(4):
        s.l.tp_sched_set_status(s.h, g, 0)
    assert s.l.tp_sched_placement(s.h) == -1


def test_default_topology_is_an_eight_gpu_all_to_all_node():
    s = Sched(8)
    for g in range(8):
        s.l.tp_sched_set_status(s.h, g, 0)
    s.l.tp_sched_set_status(s.h, 5, -1)
    s.l.tp_sched_set_resident(s.h, b"f", 2, 1)
    assert s.decide(IA_POLICY, "f") == (5, 2, 1)                 # every pair has a direct link
    s.l.tp_sched_set_status(s.h, 0, -1)                          # sibling of 0 is 1 (busy local), of 5 is 4 (busy local)
    s.l.tp_sched_set_status(s.h, 4, 4)
    assert s.decide(IA_POLICY, "g") == (0, -1, 2)                # GPU 5's sibling runs a heavy host swap


# ------------------------------------------------------------ the engine's own victims vs the oracle
_ACT_VA = {}   # function id -> address of its activation block


def _tiny_function(s, fid, level, weight_mib):
    """Registers a function of `weight_mib` MiB of weights and one 1 KiB activation through the C-ABI of a
    host-only engine (no device): the LRU charges round_up(weights) + round_up(activations) slabs."""
    from torpor_amd.server import ACK_OK, OP_RELU, REQ_EXECUTE_AFTER_LOAD
    assert s.signal(REQ_EXECUTE_AFTER_LOAD, fid, str(level))[:2] == (ACK_OK, 0)
    w = s.malloc(fid, weight_mib << 20)
    s.h2d(fid, w, np.zeros((weight_mib << 20) // 4, np.float32))
    s.device_synchronize(fid)
    a = s.malloc(fid, 1024)
    s.launch(fid, OP_RELU, [w, a], [256])
    out = np.empty(256, np.float32)
    s.d2h_async(fid, out, a)       # the request-finished marker: the registration completes here
    try:
        s.stream_synchronize(fid)
    except Exception:              # host-only: no data to deliver (-19)
        pass
    _ACT_VA[fid] = a
    return s.model_info(fid)["total_bytes"]


@pytest.mark.parametrize("policy", ["two_class", "lru"])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_engine_victims_follow_the_oracle_on_levelled_traces(policy, seed):
    """include/server/evictor.hpp:28-264 + controller.hpp:141-216,392-400 as the engine runs them: after every
    Execute / Load / Unload signal (with requests left running in between, so that the active function is
    locked) the set of resident functions and the charged bytes equal those of the oracle evictor fed the
    same trace.  The pool is twice the budget, so the contiguous-extent fallback never adds victims."""
    from oracle.host_ref import IaRef, LruRef
    from torpor_amd.server import ACK_INAVAIL, ACK_OK, REQ_EXECUTE, REQ_LOAD, REQ_UNLOAD, Server

    rng = np.random.default_rng(100 + seed)
    budget = 96 << 20
    two = policy == "two_class"
    with Server(host_only=True, mem_limit_bytes=budget, pool_bytes=2 * budget + (64 << 20), request_timeout_ms=60000,
                evict_lru=not two) as s:
        ref = IaRef(1, budget) if two else LruRef(budget)
        n = 14
        level = {fid: int(rng.integers(0, 3)) for fid in range(n)}
        size = {}

        def ref_add(fid):
            if two:
                ref.level[fid] = level[fid]
                return ref.check_and_add(0, fid, size[fid])
            return ref.check_and_add(fid, size[fid])

        def ref_resident(fid):
            return (0 in ref.gpus.get(fid, set())) if two else (fid in ref.items)

        def check(what):
            got = [s.resident(f) for f in size]
            want = [ref_resident(f) for f in size]
            assert got == want, (what, got, want)
            used = ref.cur[0] if two else ref.cur
            assert s.pool_stats()["lru_used"] == used, what

        for fid in range(n):
            size[fid] = _tiny_function(s, fid, level[fid], int(rng.integers(2, 20)))
            ref_add(fid)           # controller.hpp:223-227: the eviction check of a finished cold start
            check(f"register {fid}")
        active = None
        for step in range(600):
            fid = int(rng.integers(0, n))
            r = rng.random()
            if active is not None and r < 0.35:
                assert s.model_info(active)["resident"] == 1
                _finish(s, active)     # the running request ends
                if two:
                    ref.unlock(0, active)
                else:
                    ref.unlock(active)
                active = None
                check(f"step {step}: complete")
            elif r < 0.6:
                if active is None:
                    assert s.signal(REQ_EXECUTE, fid)[:2] == (ACK_OK, 0)
                    ref_add(fid)
                    if two:
                        ref.lock(0, fid)
                    else:
                        ref.lock(fid)
                    active = fid
                    check(f"step {step}: execute {fid}")
            elif r < 0.85:
                ack = s.signal(REQ_LOAD, fid)[0]
                if fid == active:
                    assert ack == ACK_INAVAIL
                else:
                    assert ack == ACK_OK
                    ref_add(fid)
                check(f"step {step}: load {fid}")
            else:
                ack = s.signal(REQ_UNLOAD, fid)[0]
                if fid == active:
                    assert ack == ACK_INAVAIL
                else:
                    assert ack == ACK_OK
                    if two:
                        ref.force_evict(0, fid)
                    else:
                        ref.force_evict(fid)
                check(f"step {step}: unload {fid}")
        st = s.pool_stats()
        assert st["evictions"] > 50 and st["swap_ins"] > 50     # the budget did bind


def _finish(s, fid):
    """Ends the running request of `fid` the way a function does: one asynchronous device-to-host copy of
    its activation (the completion marker, cuda_server.hpp:1044) and the stream synchronisation."""
    from torpor_amd._lib import TorporError
    s.d2h_async(fid, np.empty(256, np.float32), _ACT_VA[fid])
    try:
        s.stream_synchronize(fid)
    except TorporError:
        pass
