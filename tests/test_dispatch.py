"""Dispatch order of one executor (CPU, virtual clock): the miss-aware dispatcher of torpor_amd/dispatch.py driven
by a simulated server, against hand-worked traces and against the whole-trace simulations of
oracle/router_ref.py.  Times are in milliseconds here (the dispatcher does not care about the unit)."""
import random

import pytest

from oracle.router_ref import _Residency, _service_end, in_order_trace, miss_aware_trace
from torpor_amd.dispatch import InOrderDispatcher, MissAwareDispatcher


def drive(dispatcher, arrivals, fids, est, capacity, resident=()):
    """The serving loop of torpor_amd/multitenant.py with a simulated server: residency with LRU eviction, a
    request of a model whose swap-in was started at `load_start` ends when its bytes have crossed the link."""
    res = _Residency(capacity, resident)
    load_start = {}
    n, nxt, t = len(arrivals), 0, 0.0
    events, ends = [], {}
    while len(ends) < n:
        while nxt < n and arrivals[nxt] <= t:
            dispatcher.arrive(nxt, fids[nxt], arrivals[nxt])
            nxt += 1
        kind, what = dispatcher.decide(t, res.has)
        if kind == "load":
            f = what.fid
            res.bring_in(f)
            load_start[f] = t
            swap, fwd = est[f]
            dispatcher.load_started(f, t, swap, fwd)
            events.append(("load", what.seq, t))
        elif kind == "run":
            f = what.fid
            swap, fwd = est[f]
            if not res.has(f):          # the in-order dispatcher starts the swap-in with the request
                res.bring_in(f)
                load_start[f] = t
                events.append(("load", what.seq, t))
            res.touch(f)
            events.append(("run", what.seq, t))
            t = ends[what.seq] = _service_end(t, fwd, load_start.pop(f, None), swap)
        else:
            wake = [arrivals[nxt]] if nxt < n else []
            if what is not None:
                wake.append(what)
            assert wake, "idle with nothing to wait for and requests outstanding"
            t = max(t, min(wake))
    return events, ends


EST = {0: (5.0, 1.0), 1: (5.0, 1.0), 2: (5.0, 1.0), 3: (2.0, 3.0)}


def test_hits_are_served_while_a_swap_in_streams_hand_worked():
    """Model 2 is swapped out (5 ms of link, 1 ms forward), 0 and 1 are resident.  In arrival order the two
    hits wait out the swap-in; miss-aware they run at once and the miss still ends at 5.1 ms = 5 ms of link +
    a tenth of its forward pass."""
    arrivals, fids = [0.0, 0.5, 1.0], [2, 0, 1]
    ev, ends = drive(InOrderDispatcher(), arrivals, fids, EST, 3, resident=(0, 1))
    assert ev == [("load", 0, 0.0), ("run", 0, 0.0), ("run", 1, 5.1), ("run", 2, 6.1)]
    assert ends == {0: 5.1, 1: 6.1, 2: 7.1}
    ev, ends = drive(MissAwareDispatcher(margin_s=0.0), arrivals, fids, EST, 3, resident=(0, 1))
    # load at 0; nothing can run until the first hit arrives; the miss is started at 5 - 1 = 4
    assert ev == [("load", 0, 0.0), ("run", 1, 0.5), ("run", 2, 1.5), ("run", 0, 4.0)]
    assert ends == {1: 1.5, 2: 2.5, 0: 5.1}


def test_a_hit_that_runs_into_the_start_time_delays_the_miss_by_its_own_length_at_most():
    arrivals, fids = [0.0, 3.9], [2, 0]
    ev, ends = drive(MissAwareDispatcher(margin_s=0.0), arrivals, fids, EST, 3, resident=(0, 1))
    assert ev == [("load", 0, 0.0), ("run", 1, 3.9), ("run", 0, 4.9)]
    assert ends[0] == pytest.approx(5.9)            # 0.8 later than 5.1: the overlap of the hit with its start time
    ev, ends = drive(MissAwareDispatcher(margin_s=1.0), arrivals, fids, EST, 3, resident=(0, 1))
    assert ev == [("load", 0, 0.0), ("run", 0, 3.0), ("run", 1, 5.1)]   # started a hit's length early: ends on time
    assert ends[0] == pytest.approx(5.1)


def test_a_model_whose_forward_pass_outlasts_its_swap_in_starts_at_once():
    ev, ends = drive(MissAwareDispatcher(margin_s=0.0), [0.0, 0.1], [3, 0], EST, 3, resident=(0, 1))
    assert ev == [("load", 0, 0.0), ("run", 0, 0.0), ("run", 1, 3.0)]
    assert ends[0] == pytest.approx(3.0)


def test_requests_of_one_function_keep_their_order_and_one_swap_in_runs_at_a_time():
    # two misses (2, then 3) and a second request of 2 behind them; capacity 4 so nothing is evicted
    arrivals, fids = [0.0, 0.1, 0.2, 0.3], [2, 3, 2, 0]
    ev, ends = drive(MissAwareDispatcher(margin_s=0.0), arrivals, fids, EST, 4, resident=(0, 1))
    # t=0 load 2 (start time 4.0).  The hit (seq 3) runs 0.3-1.3.  Model 3 is not loaded before 2 has been
    # handed over: at 4.0 seq 0 runs (ends 5.1), then 3 is loaded at 5.1 (start time 5.1: forward 3 > swap 2)
    # and runs at once; the second request of 2 follows as a hit.
    assert ev == [("load", 0, 0.0), ("run", 3, 0.3), ("run", 0, 4.0), ("load", 1, 5.1), ("run", 1, 5.1),
                  ("run", 2, 8.1)]


def invariants(ev, ends, arrivals, fids):
    runs = [(s, t) for k, s, t in ev if k == "run"]
    assert sorted(s for s, _ in runs) == list(range(len(arrivals))), "every request runs exactly once"
    for s, t in runs:
        assert t >= arrivals[s] and ends[s] > t
    last = {}
    for s, _ in runs:                      # per function: arrival order
        assert last.get(fids[s], -1) < s
        last[fids[s]] = s
    times = [t for _, _, t in ev]
    assert times == sorted(times)
    prev_end = 0.0
    for s, t in runs:                      # one active function: runs do not overlap
        assert t >= prev_end - 1e-12
        prev_end = ends[s]


@pytest.mark.parametrize("seed", range(8))
def test_dispatcher_equals_the_restated_policy_on_random_traces(seed):
    rng = random.Random(seed)
    n_models = 12
    est = {f: (rng.uniform(1.0, 6.0), rng.uniform(0.4, 2.0)) for f in range(n_models)}
    n = 400
    t, arrivals = 0.0, []
    for _ in range(n):
        t += rng.expovariate(1 / 1.2)
        arrivals.append(t)
    weights = [1 / (i + 1) ** 1.1 for i in range(n_models)]
    fids = rng.choices(range(n_models), weights, k=n)
    cap = 5
    resident = tuple(range(cap))
    ev, ends = drive(MissAwareDispatcher(margin_s=0.3), arrivals, fids, est, cap, resident)
    ev_ref, ends_ref = miss_aware_trace(arrivals, fids, est, cap, resident, margin=0.3)
    assert ev == ev_ref and ends == ends_ref
    invariants(ev, ends, arrivals, fids)
    ev_io, ends_io = drive(InOrderDispatcher(), arrivals, fids, est, cap, resident)
    ev_io_ref, ends_io_ref = in_order_trace(arrivals, fids, est, cap, resident)
    assert ev_io == ev_io_ref and ends_io == ends_io_ref
    invariants(ev_io, ends_io, arrivals, fids)
    # what the policy is for: requests that found their model resident wait less, in the tail above all
    hit_io = sorted(ends_io[s] - arrivals[s] for k, s, _ in ev_io if k == "run" and ("load", s, _) not in ev_io)
    hit_ma = sorted(ends[s] - arrivals[s] for k, s, _ in ev if k == "run" and not any(e[0] == "load" and e[1] == s for e in ev))
    assert hit_ma[int(0.95 * len(hit_ma))] <= hit_io[int(0.95 * len(hit_io))]
