"""Router queueing policies, senders and the dispatch loop (CPU; a fake backend with a virtual
clock stands for the server).  Expected values are hand-worked or follow from the policies'
definitions; oracle/router_ref.py is the restatement both are compared with on random traces."""
import random

import numpy as np
import pytest

from oracle.router_ref import FifoRef, SaRef
from torpor_amd import router as R


class Clock:
    def __init__(self):
        self.t = 0.0

    def __call__(self):
        return self.t


class FakeBackend:
    """Serves a batch in service[f] * (1 + 0.5 * (n - 1)) seconds of virtual time."""

    def __init__(self, clock, service):
        self.clock, self.service = clock, service
        self.log, self.levels = [], {}

    def launch(self, f, level):
        self.levels[f] = level

    def execute(self, f, n):
        self.log.append((f, n))
        self.clock.t += self.service[f] * (1 + 0.5 * (n - 1))

    def unload(self, f):
        self.log.append(("unload", f))

    def load(self, f):
        self.log.append(("load", f))


def test_mixed_zoo_levels():
    # router.py:39,44-53: three ResNets median, four light models, BERT question answering heavy
    assert [R.mixed_model_level(i) for i in range(8)] == [1, 1, 1, 0, 0, 0, 0, 2]
    assert R.mixed_model_name(15) == "bertqa" and R.mixed_model_level(15) == 2 and R.mixed_model_name(8) == "resnet50"


def test_fifo_batches_runs_of_the_same_function_at_the_head():
    st = R._Stats()
    p = R.FifoPolicy(st, 0.98)
    for i, f in enumerate([3, 3, 3, 1, 3, 3]):
        p.insert(f, float(i))
    assert p.next_batch(lambda f: 2) == (3, [0.0, 1.0])        # limit 2
    assert p.next_batch(lambda f: 8) == (3, [2.0])             # the run ends at function 1
    assert p.next_batch(lambda f: 8) == (1, [3.0])
    assert p.next_batch(lambda f: 8) == (3, [4.0, 5.0])
    assert p.next_batch(lambda f: 8) is None


def _policy_with(stats_rows, slo=0.9):
    st = R._Stats()
    for f, row in stats_rows.items():
        st.add(f)
        st.stat[f] = list(row)
    p = R.SloAwarePolicy(st, slo)
    for f in stats_rows:
        p.add_function(f)
    return st, p


def test_sa_urgency_and_ranking_hand_worked():
    # [on time, requests, summed latency]; slo 0.9
    #  f0: mean 0.10, short of 0.9*10-9 = 0    -> urgency 0
    #  f1: mean 0.20, short of 9-7 = 2         -> 0.4
    #  f2: mean 0.05, short of 18-10 = 8       -> 0.4
    #  f3: mean 0.10, ahead by 1 (9-10 = -1)   -> -0.1
    #  f4: mean 0.50, short of 9-5 = 4         -> 2.0
    st, p = _policy_with({0: (9, 10, 1.0), 1: (7, 10, 2.0), 2: (10, 20, 1.0), 3: (10, 10, 1.0), 4: (5, 10, 5.0)})
    assert [round(p.urgency(f), 9) for f in range(5)] == [0.0, 0.4, 0.4, -0.1, 2.0]
    # alpha = 1: everything is high priority
    p.update()
    assert p.high == {0, 1, 2, 3, 4} and p.low == set()
    # alpha = 0.5: positive urgencies 0.4 + 0.4 + 2.0 = 2.8 -> budget 1.4; ascending 0.4, 0.8 fit, 2.8 does not
    p.alpha = 0.5
    p.update()
    assert p.high == {0, 1, 2, 3} and p.low == {4}
    # alpha = 0.25: budget 0.7: the first 0.4 fits, the second (0.8) does not; stable sort keeps f1 before f2
    p.alpha = 0.25
    p.update()
    assert p.high == {0, 1, 3} and p.low == {2, 4}
    # alpha = 0: nothing with a positive urgency stays; those at or ahead of their target do
    p.alpha = 0.0
    p.update()
    assert p.high == {0, 3} and p.low == {1, 2, 4}


def test_sa_queue_order_and_dispatch():
    st, p = _policy_with({0: (9, 10, 1.0), 1: (7, 10, 2.0), 2: (10, 20, 1.0), 3: (10, 10, 1.0), 4: (5, 10, 5.0)})
    p.alpha = 0.25
    p.update()                                                    # high {0,1,3}  low {2,4}
    for i, f in enumerate([3, 0, 1, 4, 2, 1, 0]):
        p.insert(f, float(i))
    # high queue: most urgent first, equal urgencies in arrival order; low queue: least urgent first
    assert [f for f, _ in p.high_q] == [1, 1, 0, 0, 3] and [a for f, a in p.high_q if f == 1] == [2.0, 5.0]
    assert [f for f, _ in p.low_q] == [2, 4]
    st.avail[1] = False                                           # function 1 has a request in flight
    assert p.next_batch(lambda f: 4) == (0, [1.0, 6.0])           # skips 1; batches both requests of 0
    st.avail[1] = True
    assert p.next_batch(lambda f: 1) == (1, [2.0])
    assert p.next_batch(lambda f: 4) == (1, [5.0])
    assert p.next_batch(lambda f: 4) == (3, [0.0])
    assert p.next_batch(lambda f: 4) == (2, [4.0])                # high queue empty: low queue
    assert p.next_batch(lambda f: 4) == (4, [3.0]) and p.next_batch(lambda f: 4) is None


def test_sa_alpha_adaptation_sequence():
    st, p = _policy_with({0: (10, 10, 1.0), 1: (0, 10, 1.0)}, slo=0.9)   # half of the functions meet the target
    alphas = []
    for step in range(1, 101):
        if step == 41:
            st.stat[1] = [10, 10, 1.0]      # ratio 0.5 -> 1.0 : +100 %
        if step == 61:
            st.stat[0] = [0, 10, 1.0]       # ratio 1.0 -> 0.5 : -50 %
        p.update()
        if step % 20 == 0:
            alphas.append(p.alpha)
    # window 1: no previous ratio counts as a rise -> min(1, 2) = 1 and 0.5 remembered; window 2: unchanged -> 1.01
    # capped at 1; window 3: rise -> 1; window 4: fall -> 0.5; window 5: unchanged -> 0.505
    assert alphas == [1, 1, 1, 0.5, 0.5 * 1.01]


@pytest.mark.parametrize("batch", [1, 3])
def test_policies_match_restatement_on_random_event_streams(batch):
    for seed in range(6):
        rng = random.Random(seed)
        nf = 10
        st = R._Stats()
        mine, ref = R.SloAwarePolicy(st, 0.95), SaRef(0.95, batch)
        fifo, fifo_ref = R.FifoPolicy(R._Stats(), 0.95), FifoRef(batch)
        for f in range(nf):
            st.add(f), mine.add_function(f), ref.add(f)
        inflight, t, served, offered = [], 0.0, 0, 0
        for step in range(6000):
            r = rng.random()
            t += rng.random() * 0.01
            if r < 0.45:
                f = rng.randrange(nf)
                mine.insert(f, t), ref.request(f, t), fifo.insert(f, t), fifo_ref.request(f, t)
                offered += 1
            elif r < 0.75:
                got = mine.next_batch(lambda f: batch)
                assert got == ref.dispatch(), (seed, step)
                assert fifo.next_batch(lambda f: batch) == fifo_ref.dispatch()
                if got:
                    st.avail[got[0]] = False
                    inflight.append(got)
                    served += len(got[1])
                    assert len(got[1]) <= batch
            elif r < 0.97:
                if inflight:
                    f, arrs = inflight.pop(rng.randrange(len(inflight)))
                    lats = [t - a + rng.random() * 0.2 for a in arrs]
                    st.record(f, lats, 0.1), ref.complete(f, lats, 0.1)
            else:
                assert mine.update() == ref.update()
                assert mine.alpha == ref.alpha and mine.high == ref.high_func and mine.low == ref.low_func
                assert mine.high_q == ref.high_q and mine.low_q == ref.low_q
                # right after a re-ranking both queues are sorted by urgency
                hu = [mine.urgency(f) for f, _ in mine.high_q]
                lu = [mine.urgency(f) for f, _ in mine.low_q]
                assert hu == sorted(hu, reverse=True) and lu == sorted(lu)
                assert not (mine.high & mine.low)
            assert st.stat == ref.func_stat
        # conservation: nothing lost, nothing served twice
        for f, arrs in inflight:
            st.avail[f] = True
            ref.func_avail[f] = True
        while True:
            got = mine.next_batch(lambda f: batch)
            assert got == ref.dispatch()
            if not got:
                break
            ref.func_avail[got[0]] = True          # served at once
            served += len(got[1])
        assert served == offered and len(mine) == 0


def test_router_loop_serves_everything_once_and_tracks_deadlines():
    clock = Clock()
    be = FakeBackend(clock, {0: 0.010, 1: 0.030, 2: 0.080})
    r = R.Router(be, slo_percentile=0.9, deadline_s=0.05, batch_limit=2, policy="sa", clock=clock, deadlines={2: 0.2})
    for f in range(3):
        r.launch(f, level=f)
    assert be.levels == {0: 0, 1: 1, 2: 2}
    rng = np.random.default_rng(0)
    arrivals = R.fixed_rate_arrivals(3, 600, 1, rng)            # 30 req/s offered, capacity about 25-40 req/s
    t, i = 0.0, 0
    stamps = np.cumsum([g for g, _ in arrivals])
    while i < len(arrivals) or r.queued():
        while i < len(arrivals) and stamps[i] <= clock.t:
            r.submit(arrivals[i][1], float(stamps[i]))
            i += 1
        if r.pump() == 0 and i < len(arrivals):
            clock.t = max(clock.t, float(stamps[i]))
    s = r.summary()
    assert s["requests"] == len(arrivals) == sum(n for _, n in be.log)
    assert set(s["batches"]) <= {1, 2} and s["queued"] == 0
    for f in range(3):
        met, n, total = r.stats.stat[f]
        lats = np.asarray(r.latencies[f])
        assert n == len(lats) == sum(1 for _, g in arrivals if g == f)
        assert met == int((lats <= (0.2 if f == 2 else 0.05)).sum()) and abs(total - lats.sum()) < 1e-9
        assert lats.min() >= be.service[f] - 1e-12                # latency includes the service time
    assert len(r.slo_history) >= 20                               # re-ranked every 2 s of a 60 s trace
    assert r.force_evict(1) is None and be.log[-1] == ("unload", 1)


def test_router_takes_a_failing_function_out_of_service():
    clock = Clock()

    class Failing(FakeBackend):
        def execute(self, f, n):
            if f == 1:
                raise RuntimeError("timeout")
            super().execute(f, n)

    r = R.Router(Failing(clock, {0: 0.01, 1: 0.01}), policy="fifo", clock=clock)
    r.launch(0, 1), r.launch(1, 1)
    r.submit(1), r.submit(0)
    with pytest.raises(RuntimeError):
        r.pump()
    assert r.unhealthy == {1} and not r.submit(1)                 # router.py:434-435
    assert r.pump() == 1 and r.summary()["requests"] == 1


def test_senders():
    rng = np.random.default_rng(1)
    a = R.fixed_rate_arrivals(4, 30, 3, rng)
    assert len(a) == 3 * 120                                      # rate x functions requests per minute
    gaps = np.array([g for g, _ in a])
    assert abs(gaps.mean() - 0.5) < 0.005 and abs(gaps.sum() - 180) < 3     # mean gap 60 s / 120
    assert np.allclose(gaps * 1000, np.round(gaps * 1000))        # whole milliseconds (Poisson counts)
    assert abs(gaps.var() * 1e6 / 500 - 1) < 0.25                 # Poisson: variance = mean (in ms)
    assert set(f for _, f in a) == {0, 1, 2, 3}
    pat = np.array([[60, 0, 120], [0, 0, 60]])
    b = R.trace_arrivals(pat, 50, np.random.default_rng(2))
    rows = pat[np.random.default_rng(2).choice(2, 50)]
    assert len(b) == rows.sum()                                   # per minute: the summed rate; the empty minute adds none
    syn = R.synthetic_rate_patterns(203, 31, np.random.default_rng(3))
    assert syn.shape == (203, 31) and syn.dtype == np.int64 and 8 < syn.mean() < 12 and syn.min() >= 0
    ka = R.keepalive_p99([(1.0, 0), (1.0, 1), (1.0, 0), (5.0, 0), (1.0, 1)])
    assert ka[0] == pytest.approx(np.percentile([2.0, 5.0], 99)) and ka[1] == pytest.approx(7.0)


class HintBackend(FakeBackend):
    def execute(self, f, n, prefetch=None):
        self.log.append((f, n, prefetch))
        self.clock.t += self.service[f]


@pytest.mark.parametrize("policy", ["fifo", "sa"])
def test_prefetch_names_the_function_the_queue_hands_out_next(policy):
    """With prefetch on, every dispatch names the function of the request that the policy hands out next (never the
    one being served, nothing when nobody else waits), and the order of service is what it is without prefetch."""
    def run(prefetch):
        clock = Clock()
        backend = (HintBackend if prefetch else FakeBackend)(clock, {f: 0.010 for f in range(4)})
        r = R.Router(backend, 0.98, 0.1, 1, policy, clock=clock, prefetch=prefetch)
        for f in range(4):
            r.launch(f, 1)
        rng = random.Random(5)
        for i in range(60):
            r.submit(rng.randrange(4), arrival=0.001 * i)
        while r.pump():
            pass
        return r, backend.log

    r1, hinted = run(True)
    _, plain = run(False)
    assert [(f, n) for f, n, _ in hinted] == plain
    for i, (f, _, nxt) in enumerate(hinted):
        assert nxt != f
        later = [g for g, _, _ in hinted[i + 1:] if g != f]
        if policy == "fifo":
            assert nxt == (later[0] if later else None), i      # FIFO: the first later request of another function
        elif nxt is not None:
            assert nxt in later, i
    assert r1.prefetch_hints == sum(1 for _, _, nxt in hinted if nxt is not None) > 20
    assert r1.summary()["prefetch_hints"] == r1.prefetch_hints


class SwapBackend(FakeBackend):
    """A server with room for `capacity` models (LRU): a request of a swapped-out model ends when its bytes have
    crossed the link, swap[f] after the swap-in was started, and not before forward[f] of its own."""

    def __init__(self, clock, swap, forward, capacity, resident=()):
        super().__init__(clock, forward)
        self.swap, self.forward, self.capacity = swap, forward, capacity
        self.lru = list(resident)
        self.load_start = {}

    def _bring_in(self, f):
        if f not in self.lru:
            if len(self.lru) >= self.capacity:
                self.lru.pop(0)
            self.load_start[f] = self.clock.t
        else:
            self.lru.remove(f)
        self.lru.append(f)

    def resident(self, f):
        return f in self.lru

    def load_estimate(self, f):
        return self.swap[f], self.forward[f]

    def load(self, f):
        self.log.append(("load", f, self.clock.t))
        self._bring_in(f)

    def execute(self, f, n, prefetch=None):
        self._bring_in(f)
        start = self.clock.t
        end = start + self.forward[f]
        t0 = self.load_start.pop(f, None)
        if t0 is not None:
            end = max(end, t0 + self.swap[f] + 0.1 * self.forward[f])
        self.log.append((f, n, start))
        self.clock.t = end


def _run_trace(clock, router, arrivals):
    """serve_arrivals on the virtual clock: the busy-wait of the real loop becomes a jump."""
    i, n = 0, len(arrivals)
    while i < n or router.queued():
        while i < n and arrivals[i][0] <= clock.t:
            router.submit(arrivals[i][1], arrivals[i][0])
            i += 1
        if router.pump() == 0:
            wake = [t for t in (arrivals[i][0] if i < n else None, router.wake_time()) if t is not None]
            assert wake, "nothing to serve and nothing to wait for"
            clock.t = max(clock.t, min(wake))


@pytest.mark.parametrize("policy", ["fifo", "sa"])
def test_miss_aware_router_serves_hits_while_a_model_streams_in(policy):
    """Function 2 is swapped out (5 ms of link, 1 ms forward), 0 and 1 are resident.  In queue order the two hits
    wait out the swap-in; miss-aware they run at once, the Load goes out when the miss reaches the head of the
    queue, and the miss is served at 5 - 1 = 4 ms and ends at 5.1 ms as it would have anyway."""
    ms = 1e-3
    swap, fwd = {0: 5 * ms, 1: 5 * ms, 2: 5 * ms}, {0: 1 * ms, 1: 1 * ms, 2: 1 * ms}
    arrivals = [(0.0, 2), (0.5 * ms, 0), (1.0 * ms, 1)]
    out = {}
    for aware in (False, True):
        clock = Clock()
        be = SwapBackend(clock, swap, fwd, capacity=3, resident=(0, 1))
        r = R.Router(be, policy=policy, clock=clock, miss_aware=aware, margin_s=0.0)
        for f in range(3):
            r.launch(f, 1)
        _run_trace(clock, r, arrivals)
        out[aware] = ([e for e in be.log if e[0] != "load"], {f: v for f, v in r.latencies.items()})
    runs, lats = out[False]
    assert [(f, round(t / ms, 3)) for f, _, t in runs] == [(2, 0.0), (0, 5.1), (1, 6.1)]
    runs, lats = out[True]
    assert [(f, round(t / ms, 3)) for f, _, t in runs] == [(0, 0.5), (1, 1.5), (2, 4.0)]
    assert lats[2][0] == pytest.approx(5.1 * ms) and lats[0][0] == pytest.approx(1.0 * ms) and lats[1][0] == pytest.approx(1.5 * ms)


@pytest.mark.parametrize("policy", ["fifo", "sa"])
@pytest.mark.parametrize("seed", range(4))
def test_miss_aware_router_serves_every_request_once_one_at_a_time_one_swap_in_at_a_time(policy, seed):
    rng = random.Random(seed)
    nf, cap = 10, 4
    swap = {f: rng.uniform(1e-3, 6e-3) for f in range(nf)}
    fwd = {f: rng.uniform(0.4e-3, 2e-3) for f in range(nf)}
    t, arrivals = 0.0, []
    for _ in range(300):
        t += rng.expovariate(1 / 1.5e-3)
        arrivals.append((t, rng.choices(range(nf), [1 / (i + 1) for i in range(nf)])[0]))
    res = {}
    for aware in (False, True):
        clock = Clock()
        be = SwapBackend(clock, swap, fwd, capacity=cap, resident=tuple(range(cap)))
        r = R.Router(be, policy=policy, clock=clock, miss_aware=aware, batch_limit=1)
        for f in range(nf):
            r.launch(f, 1)
        _run_trace(clock, r, arrivals)
        runs = [e for e in be.log if e[0] != "load"]
        assert len(runs) == len(arrivals) and sum(len(v) for v in r.latencies.values()) == len(arrivals)
        starts = [t0 for _, _, t0 in runs]
        assert starts == sorted(starts)                              # one active function: no overlap
        loads = [e for e in be.log if e[0] == "load"]
        for a, b in zip(loads, loads[1:]):                           # one swap-in at a time: the earlier one has been
            assert any(f == a[1] and a[2] <= t0 <= b[2] for f, _, t0 in runs)   # handed over before the next starts
        res[aware] = np.sort(np.concatenate([np.asarray(v) for v in r.latencies.values()]))
        assert r.summary()["dispatch"] == ("miss-aware" if aware else "queue order")
    assert res[True].mean() <= res[False].mean() * 1.02              # what it is for: nobody waits out others' swap-ins
