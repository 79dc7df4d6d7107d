"""TEST INFRASTRUCTURE ONLY: the reference router's queueing decisions, restated in its own shape.

  SaRef    scripts/router.py:218-378 (`sa_schedule`): the two request lists, `calc_metric`,
           the two binary-search insertions, `get_req` over `func_avail`, batching, and the
           periodic re-ranking with its alpha adaptation.  Events that the reference takes from
           its schedule queue are method calls here: `request` (type 0), `update` (type 1),
           `dispatch` (the queue-empty branch), `complete` (router.py:481-489).
  FifoRef  scripts/router.py:156-216 (`baseline_schedule`).

  miss_aware_trace  the miss-aware dispatch order of torpor_amd/dispatch.py as a simulation of a whole trace.
           The reference has no such policy (its router serves in arrival order, scripts/router.py:289-313; the
           controller queues while the executor is busy, include/server/controller.hpp:163-186,242-262); what is
           kept from it is the one-active-function rule and the Load signal (controller.hpp:208-215) that starts
           a swap-in ahead of the request.  in_order_trace is the reference's order under the same timing model.

Pinning (tests/test_router.py): hand-worked rankings and alpha sequences, sortedness of both
lists after every re-ranking, and conservation (every request is dispatched exactly once); the two dispatch
simulations on hand-worked traces whose answers follow from the rules by arithmetic, and by their invariants (each
request runs once, never before it arrives, requests of one function in arrival order, one swap-in at a time).
"""


class SaRef:
    def __init__(self, slo_percentile, batch_size_limit=1):
        self.slo = slo_percentile
        self.batch = batch_size_limit
        self.func_stat, self.func_avail = {}, {}
        self.high_func, self.low_func = set(), set()
        self.high_q, self.low_q = [], []
        self.alpha = 1
        self.alpha_adj_cur, self.old_slo_ratio = 0, 0

    def add(self, f):                                   # router.py:475-479
        self.func_stat[f] = [0, 0, 0]
        self.high_func.add(f)
        self.func_avail[f] = True

    def calc_metric(self, f):                           # router.py:224-225
        s = self.func_stat[f]
        return (s[2] / s[1]) * (self.slo * s[1] - s[0]) if s[1] > 0 else 0

    def request(self, f, arr):                          # router.py:227-250
        m = self.calc_metric
        if f in self.high_func:
            a, b = 0, len(self.high_q)
            while a < b:
                mid = (a + b) // 2
                if m(self.high_q[mid][0]) < m(f):
                    b = mid
                else:
                    a = mid + 1
            self.high_q.insert(a, (f, arr))
        elif f in self.low_func:
            a, b = 0, len(self.low_q)
            while a < b:
                mid = (a + b) // 2
                if m(self.low_q[mid][0]) >= m(f):
                    b = mid
                else:
                    a = mid + 1
            self.low_q.insert(a, (f, arr))

    def _get(self, out=True):                           # router.py:252-272
        for q in (self.high_q, self.low_q):
            for i in range(len(q)):
                if self.func_avail[q[i][0]]:
                    return q.pop(i) if out else q[i]
        return None

    def dispatch(self):                                 # router.py:300-316
        req = self._get()
        if req is None:
            return None
        f, arr = req
        arrs = [arr]
        while True:
            nxt = self._get(False)
            if nxt is None or nxt[0] != f or len(arrs) >= self.batch:
                break
            arrs.append(self._get()[1])
        self.func_avail[f] = False
        return f, arrs

    def complete(self, f, lats, ddl):                   # router.py:481-489
        for lat in lats:
            self.func_stat[f][2] += lat
            self.func_stat[f][1] += 1
            if lat <= ddl:
                self.func_stat[f][0] += 1
        self.func_avail[f] = True

    def update(self):                                   # router.py:318-376
        slo = self.slo
        self.alpha_adj_cur += 1
        exp = [(f, (s[2] / s[1]) * (slo * s[1] - s[0]) / (1 - slo)) for f, s in self.func_stat.items() if s[1] > 0]
        exp.sort(key=lambda x: x[1])
        total = sum(v for _, v in exp if v >= 0) * self.alpha
        borderline, agg = -1, 0
        for i in range(len(exp)):
            if exp[i][1] > 0:
                agg += exp[i][1]
                if agg > total:
                    borderline = i - 1
                    break
        if agg <= total:
            borderline = len(exp) - 1
        for i in range(len(exp)):
            if i <= borderline:
                self.high_func.add(exp[i][0]); self.low_func.discard(exp[i][0])
            else:
                self.high_func.discard(exp[i][0]); self.low_func.add(exp[i][0])
        old_h, old_l = self.high_q, self.low_q
        self.high_q, self.low_q = [], []
        for f, a in old_h + old_l:
            self.request(f, a)
        seen = [s for s in self.func_stat.values() if s[1] > 0]
        if not seen:
            return None
        ratio = len([s for s in seen if s[0] / s[1] >= slo]) / len(seen)
        if self.alpha_adj_cur >= 20:
            d = (ratio - self.old_slo_ratio) / self.old_slo_ratio if self.old_slo_ratio > 0 else 0.04
            if d >= 0.04:
                self.alpha = min(1, self.alpha * 2.0)
                self.old_slo_ratio = ratio
            elif d < -0.04:
                self.alpha = self.alpha / 2.0
                self.old_slo_ratio = ratio
            else:
                self.alpha = min(1, self.alpha * 1.01)
            self.alpha_adj_cur = 0
        return ratio


class FifoRef:
    def __init__(self, batch_size_limit=1):
        self.batch = batch_size_limit
        self.q = []

    def request(self, f, arr):
        self.q.append((f, arr))

    def dispatch(self):                                 # router.py:179-199
        if not self.q:
            return None
        f, arr = self.q.pop(0)
        arrs = [arr]
        while self.q and self.q[0][0] == f and len(arrs) < self.batch:
            arrs.append(self.q.pop(0)[1])
        return f, arrs


# ------------------------------------------------------------------------------------------- dispatch order
class _Residency:
    """Which models are in device memory: at most `capacity` of them, the least recently used one leaves when a
    swap-in needs room (never the one that is running or being swapped in)."""

    def __init__(self, capacity, resident):
        self.capacity = capacity
        self.order = list(resident)   # least recent first

    def has(self, f):
        return f in self.order

    def touch(self, f):
        self.order.remove(f)
        self.order.append(f)

    def bring_in(self, f, keep=()):
        while len(self.order) >= self.capacity:
            victim = next((g for g in self.order if g not in keep), None)
            if victim is None:
                break
            self.order.remove(victim)
        self.order.append(f)


def _service_end(start, forward, load_start, swap):
    """When a request ends that starts at `start`: its forward pass, but not before the bytes it waits for have
    crossed the link (the engine pipelines the copy with the forward pass), plus a tenth of a forward pass for the
    layers behind the last transfer group."""
    if load_start is None:
        return start + forward
    return max(start + forward, load_start + swap + 0.1 * forward)


def in_order_trace(arrivals, fids, est, capacity, resident=()):
    """The reference's order: each request holds the executor from its start to its end, a request of a
    swapped-out model starts its swap-in when it starts.  Returns [(kind, seq, time)] with kind "run" / "load",
    and the end time of every request."""
    res = _Residency(capacity, resident)
    t, events, ends = 0.0, [], {}
    for seq, (a, f) in enumerate(zip(arrivals, fids)):
        t = max(t, a)
        swap, fwd = est[f]
        if res.has(f):
            res.touch(f)
            end = _service_end(t, fwd, None, swap)
        else:
            res.bring_in(f)
            events.append(("load", seq, t))
            end = _service_end(t, fwd, t, swap)
        events.append(("run", seq, t))
        ends[seq] = end
        t = end
    return events, ends


def miss_aware_trace(arrivals, fids, est, capacity, resident=(), margin=0.0003):
    """State machine over the moments at which the executor is free.  waiting = the one request whose swap-in is
    on its way: (seq, load start, earliest start)."""
    n = len(arrivals)
    res = _Residency(capacity, resident)
    pending = []                 # seqs that have arrived and not run, arrival order
    nxt = 0                      # next arrival to admit
    waiting = None
    t = 0.0
    events, ends = [], {}
    while len(ends) < n:
        while nxt < n and arrivals[nxt] <= t:
            pending.append(nxt)
            nxt += 1
        if waiting is None:                                   # start the oldest miss's swap-in
            for s in pending:
                if not res.has(fids[s]):
                    swap, fwd = est[fids[s]]
                    res.bring_in(fids[s])
                    waiting = (s, t, t + max(0.0, swap - fwd - margin))
                    events.append(("load", s, t))
                    break
        choice = None
        if waiting is not None and waiting[2] <= t:           # its time has come
            # the oldest queued request of that function (it is the one the swap-in was started for)
            choice = next(s for s in pending if fids[s] == fids[waiting[0]])
        else:
            busy = fids[waiting[0]] if waiting is not None else None
            choice = next((s for s in pending if fids[s] != busy and res.has(fids[s])), None)
        if choice is None:                                    # nothing to do: the next thing that can change that
            wake = [arrivals[nxt]] if nxt < n else []
            if waiting is not None:
                wake.append(waiting[2])
            t = max(t, min(wake))
            continue
        f = fids[choice]
        swap, fwd = est[f]
        load_start = None
        if waiting is not None and fids[waiting[0]] == f:
            load_start = waiting[1]
            waiting = None
        res.touch(f)
        events.append(("run", choice, t))
        pending.remove(choice)
        t = ends[choice] = _service_end(t, fwd, load_start, swap)
    return events, ends
