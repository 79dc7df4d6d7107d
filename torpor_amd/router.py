"""Request router: the layer that calls the server's signal boundary.

What the reference's scripts/router.py does around the GPU server, without its docker / HTTP
plumbing: functions are launched (ExecuteAfterLoad with the model level as payload,
router.py:381-387), requests arrive from senders, wait in a FIFO queue (router.py:156-216) or
in the SLO-aware pair of queues (router.py:218-378), are batched per function up to `-b`
(router.py:186-189, 352-355) and dispatched with an Execute signal; completions feed the
per-function statistics [requests within the deadline, requests, summed latency]
(router.py:481-489) from which the SLO-aware policy re-ranks functions every two seconds
(router.py:495-498) and adapts its admission factor alpha every 20 re-rankings.

The reference runs one manager process per GPU and lets several functions execute at once on
different GPUs; with one GPU the executor serves one request at a time, so `Router.pump`
dispatches synchronously: drain the inbox, then run one batch to completion.

Senders (scripts/sender_fix_rate.py, scripts/sender_from_trace.py) are functions that return
the arrival list [(seconds since the previous request, function)], and `keepalive_p99`
is tools/export_keepalive.py:24-27.
"""
import argparse
import collections
import json
import time

import numpy as np

# scripts/router.py:39 ; levels from get_mixed_model_level (router.py:44-53)
MIXED_MODELS = ("resnet50", "resnet101", "resnet152", "densenet169", "densenet201", "inception", "efficientnet",
                "bertqa")


def mixed_model_name(func_id, models=MIXED_MODELS):
    return models[func_id % len(models)]


def mixed_model_level(func_id, models=MIXED_MODELS):
    i = func_id % len(models)
    if i < 3:
        return 1
    if i < 7:
        return 0
    return 2 if i == 7 else 1


# ----------------------------------------------------------------------------------------- policies
class _Stats:
    """Per function: [requests that met the deadline, requests, summed latency] (router.py:133-136)."""

    def __init__(self):
        self.stat = {}
        self.avail = {}

    def add(self, f):
        self.stat[f] = [0, 0, 0.0]
        self.avail[f] = True

    def record(self, f, latencies, deadline):       # router.py:481-489
        s = self.stat[f]
        for lat in latencies:
            s[2] += lat
            s[1] += 1
            if lat <= deadline:
                s[0] += 1
        self.avail[f] = True

    def slo_ratio(self, slo):
        """Share of the functions with at least one request whose hit rate reaches the target."""
        seen = [s for s in self.stat.values() if s[1] > 0]
        if not seen:
            return None
        return sum(1 for s in seen if s[0] / s[1] >= slo) / len(seen)


class FifoPolicy:
    """Arrival order; batches are runs of the same function at the head (router.py:156-216)."""
    name = "fifo"

    def __init__(self, stats, slo):
        self.stats, self.slo = stats, slo
        self.queue = collections.deque()
        self.blocked = set()            # functions the router holds back (their model is on its way): skipped

    def add_function(self, f):
        pass

    def insert(self, f, arrival):
        self.queue.append((f, arrival))

    def __len__(self):
        return len(self.queue)

    def next_batch(self, limit):
        if not self.queue:
            return None
        if self.blocked:
            return self._next_unblocked(limit)
        f, arr = self.queue.popleft()
        arrivals = [arr]
        while self.queue and self.queue[0][0] == f and len(arrivals) < limit(f):
            arrivals.append(self.queue.popleft()[1])
        return f, arrivals

    def _next_unblocked(self, limit):
        """The first request of a function that is not held back, with the requests of the same function that
        follow it directly among those not held back."""
        f, arrivals, keep, closed = None, [], [], False
        for g, arr in self.queue:
            if closed or g in self.blocked:         # held-back requests stay where they are and do not end a run
                keep.append((g, arr))
            elif f is None:
                f, arrivals = g, [arr]
            elif g == f and len(arrivals) < limit(f):
                arrivals.append(arr)
            else:
                closed = True
                keep.append((g, arr))
        if f is None:
            return None
        self.queue = collections.deque(keep)
        return f, arrivals

    def head(self):
        """The function next_batch would serve now."""
        return next((f for f, _ in self.queue if f not in self.blocked), None)

    def peek(self, running):
        """The function of the first waiting request that is not `running`'s (what follows the batch just taken)."""
        for f, _ in self.queue:
            if f != running:
                return f
        return None

    def update(self):
        return self.stats.slo_ratio(self.slo)


class SloAwarePolicy:
    """Two queues (router.py:218-378).

    A function's urgency is  mean latency x (slo x requests - requests on time): the time it would
    take to serve the on-time requests it is short of.  High-priority requests are kept most urgent
    first, low-priority ones least urgent first; dispatch takes the first request of a function
    that has none in flight, high queue before low.  `update` re-ranks: functions are sorted by
    urgency / (1 - slo), and the least urgent ones whose positive urgencies add up to at most
    alpha x (sum of positive urgencies) are high priority, the rest low - with alpha < 1 the
    functions furthest from their target are sacrificed so that the others meet theirs.  Every
    `window` updates alpha doubles (capped at 1) if the share of functions meeting the target rose
    by 4 % or more, halves if it fell by more than 4 %, and creeps up by 1 % otherwise.

    Positions in the queues come from a binary search with the urgencies of the moment, as in the
    reference (router.py:229-248); the queues are re-sorted only by `update`, so between updates the
    probe sequence decides where a request lands and is kept the same: mid = (lo + hi) // 2.
    """
    name = "sa"

    def __init__(self, stats, slo, window=20, diff_threshold=0.04, scale=2.0, low_scale=1.01):
        self.stats, self.slo = stats, slo
        self.high_q, self.low_q = [], []
        self.high, self.low = set(), set()
        self.blocked = set()            # functions the router holds back (their model is on its way): skipped
        self.alpha = 1.0
        self.window, self.diff_threshold, self.scale, self.low_scale = window, diff_threshold, scale, low_scale
        self._updates = 0
        self._old_ratio = 0.0

    def add_function(self, f):          # router.py:475-479: new functions start as high priority
        self.high.add(f)

    def urgency(self, f):               # router.py:224-225
        met, n, total = self.stats.stat[f]
        return (total / n) * (self.slo * n - met) if n > 0 else 0

    def insert(self, f, arrival):
        if f in self.high:
            q, before = self.high_q, lambda other, mine: other < mine
        elif f in self.low:
            q, before = self.low_q, lambda other, mine: other >= mine
        else:
            return False
        mine = self.urgency(f)
        lo, hi = 0, len(q)
        while lo < hi:
            mid = (lo + hi) // 2
            if before(self.urgency(q[mid][0]), mine):
                hi = mid
            else:
                lo = mid + 1
        q.insert(lo, (f, arrival))
        return True

    def __len__(self):
        return len(self.high_q) + len(self.low_q)

    def _first_available(self):
        for q in (self.high_q, self.low_q):
            for i, (f, _) in enumerate(q):
                if self.stats.avail[f] and f not in self.blocked:
                    return q, i
        return None, None

    def head(self):
        """The function next_batch would serve now."""
        q, i = self._first_available()
        return None if q is None else q[i][0]

    def peek(self, running):
        """The function next_batch would take now (`running` has been marked unavailable by the caller)."""
        q, i = self._first_available()
        return None if q is None or q[i][0] == running else q[i][0]

    def next_batch(self, limit):
        q, i = self._first_available()
        if q is None:
            return None
        f, arr = q.pop(i)
        arrivals = [arr]
        while len(arrivals) < limit(f):
            q, i = self._first_available()
            if q is None or q[i][0] != f:
                break
            arrivals.append(q.pop(i)[1])
        return f, arrivals

    def update(self):                   # router.py:318-376
        self._updates += 1
        slo = self.slo
        ranked = [(f, (s[2] / s[1]) * (slo * s[1] - s[0]) / (1 - slo)) for f, s in self.stats.stat.items() if s[1] > 0]
        ranked.sort(key=lambda x: x[1])
        budget = sum(v for _, v in ranked if v >= 0) * self.alpha
        border, acc = -1, 0
        for i, (_, v) in enumerate(ranked):
            if v > 0:
                acc += v
                if acc > budget:
                    border = i - 1
                    break
        if acc <= budget:
            border = len(ranked) - 1
        for i, (f, _) in enumerate(ranked):
            if i <= border:
                self.high.add(f)
                self.low.discard(f)
            else:
                self.high.discard(f)
                self.low.add(f)
        old_high, old_low = self.high_q, self.low_q
        self.high_q, self.low_q = [], []
        for f, arr in old_high:
            self.insert(f, arr)
        for f, arr in old_low:
            self.insert(f, arr)
        ratio = self.stats.slo_ratio(slo)
        if ratio is None:
            return None
        if self._updates >= self.window:
            diff = (ratio - self._old_ratio) / self._old_ratio if self._old_ratio > 0 else self.diff_threshold
            if diff >= self.diff_threshold:
                self.alpha = min(1, self.alpha * self.scale)
                self._old_ratio = ratio
            elif diff < -self.diff_threshold:
                self.alpha = self.alpha / self.scale
                self._old_ratio = ratio
            else:
                self.alpha = min(1, self.alpha * self.low_scale)
            self._updates = 0
        return ratio


# ------------------------------------------------------------------------------------------- router
class Router:
    """`backend.launch(func_id, level)` registers a function and `backend.execute(func_id, n)` serves
    a batch of n requests of it, blocking until the answers are back (see `FunctionBackend`)."""

    UPDATE_PERIOD_S = 2.0               # router.py:495

    def __init__(self, backend, slo_percentile=0.98, deadline_s=0.1, batch_limit=1, policy="sa", clock=time.monotonic,
                 deadlines=None, batch_limits=None, prefetch=False, miss_aware=False, margin_s=0.0003):
        self.backend = backend
        # miss_aware: a request whose model is swapped out does not hold the executor for its swap-in.  Its model
        # is asked for at once (the Load signal), requests of resident models that the queue would serve next run
        # meanwhile, and the waiting function is served when the rest of its copy is about as long as its forward
        # pass (torpor_amd/dispatch.py has the rule and its reasons; one swap-in at a time, a function's own
        # requests keep their order).  Needs a backend that can say whether a model is resident and how long its
        # swap-in takes (`resident`, `load_estimate`).
        self.miss_aware = miss_aware and hasattr(backend, "resident") and hasattr(backend, "load_estimate")
        self.margin_s = margin_s
        self.loading = {}               # function -> time from which it is served
        self.loads = 0
        # prefetch: when a batch is dispatched, the function whose request the queue would hand out next is named
        # to the backend, which asks the server to load its model (the Load signal) while this batch runs
        self.prefetch = prefetch
        self.prefetch_hints = 0
        self.slo = slo_percentile
        self.deadline_s = deadline_s
        self.deadlines = dict(deadlines or {})          # per-function overrides (router.py:18: 0.2 s for BERT)
        self.batch_limit = batch_limit
        self.batch_limits = dict(batch_limits or {})    # router.py:20,186
        self.clock = clock
        self.stats = _Stats()
        self.policy = SloAwarePolicy(self.stats, self.slo) if policy == "sa" else FifoPolicy(self.stats, self.slo)
        self.inbox = collections.deque()
        self.unhealthy = set()                          # router.py:491-493
        self.latencies = collections.defaultdict(list)
        self.batches = collections.Counter()
        self._last_update = None
        self.slo_history = []

    def launch(self, func_id, level=None):
        """router.py:381-387 + the manager's reply (router.py:475-479)."""
        self.backend.launch(func_id, mixed_model_level(func_id) if level is None else level)
        self.stats.add(func_id)
        self.policy.add_function(func_id)

    def force_evict(self, func_id):     # router.py:408-412
        self.backend.unload(func_id)

    def load_all(self):                 # router.py:462-468
        for f in self.stats.stat:
            self.backend.load(f)

    def submit(self, func_id, arrival=None):
        """A request from a sender (router.py:429-437)."""
        if func_id in self.unhealthy:
            return False
        self.inbox.append((func_id, self.clock() if arrival is None else arrival))
        return True

    def _limit(self, f):
        return self.batch_limits.get(f, self.batch_limit)

    def pump(self):
        """One turn of the scheduling loop: queue what has arrived, re-rank when due, then dispatch one
        batch and wait for it.  Returns the number of requests served."""
        now = self.clock()
        if self._last_update is None:
            self._last_update = now
        while self.inbox:
            f, arr = self.inbox.popleft()
            self.policy.insert(f, arr)
        if now - self._last_update > self.UPDATE_PERIOD_S:
            self._last_update = now
            ratio = self.policy.update()
            if ratio is not None:
                self.slo_history.append((now, ratio, getattr(self.policy, "alpha", None), len(self.policy)))
        if self.miss_aware and not self._hold_back_misses(now):
            return 0
        got = self.policy.next_batch(self._limit)
        if got is None:
            return 0
        f, arrivals = got
        self.loading.pop(f, None)       # (a function whose swap-in was started is handed over with its first batch)
        self.stats.avail[f] = False
        try:
            nxt = self.policy.peek(f) if self.prefetch else None
            if nxt is not None:
                self.prefetch_hints += 1
                self.backend.execute(f, len(arrivals), prefetch=nxt)
            else:
                self.backend.execute(f, len(arrivals))
        except Exception:
            self.unhealthy.add(f)       # router.py:104-106: a function that fails is taken out of service
            self.stats.avail[f] = True
            raise
        end = self.clock()
        lats = [end - a for a in arrivals]
        self.stats.record(f, lats, self.deadlines.get(f, self.deadline_s))
        self.latencies[f].extend(lats)
        self.batches[len(arrivals)] += 1
        return len(arrivals)

    def _hold_back_misses(self, now):
        """Miss-aware dispatch: decide which functions the policy must pass over in this turn.  Returns False
        when nothing can be served yet (every waiting request is of a model that is still on its way)."""
        blocked = self.policy.blocked
        blocked.clear()
        for f, due in self.loading.items():
            if due > now:
                blocked.add(f)          # its copy has not come far enough
        while True:
            f = self.policy.head()
            if f is None:
                blocked.clear()
                return False
            if f in self.loading or self.backend.resident(f):
                return True             # resident, or a swap-in that has come far enough: served next
            if not self.loading:        # one swap-in at a time: this one's starts now
                self.backend.load(f)
                swap_s, forward_s = self.backend.load_estimate(f)
                self.loading[f] = now + max(0.0, swap_s - forward_s - self.margin_s)
                self.loads += 1
                if self.loading[f] <= now:
                    return True
            blocked.add(f)              # waits for its copy, or for its turn to be copied

    def wake_time(self):
        """When a function that waits for its swap-in is due (miss-aware dispatch), else None."""
        return min(self.loading.values()) if self.loading else None

    def queued(self):
        return len(self.policy) + len(self.inbox)

    def summary(self):
        all_lat = np.sort(np.concatenate([np.asarray(v) for v in self.latencies.values()])) if self.latencies else np.zeros(0)

        def pct(q):
            return float(all_lat[min(len(all_lat) - 1, int(round(q * (len(all_lat) - 1))))]) * 1e3 if len(all_lat) else None

        per_func = {f: s[0] / s[1] for f, s in self.stats.stat.items() if s[1] > 0}
        return dict(policy=self.policy.name, requests=int(len(all_lat)), p50_ms=pct(0.5), p99_ms=pct(0.99),
                    mean_ms=float(all_lat.mean() * 1e3) if len(all_lat) else None,
                    functions_meeting_slo=self.stats.slo_ratio(self.slo),
                    requests_within_deadline=(sum(s[0] for s in self.stats.stat.values()) /
                                              max(1, sum(s[1] for s in self.stats.stat.values()))),
                    worst_function_hit_rate=min(per_func.values()) if per_func else None,
                    alpha=getattr(self.policy, "alpha", None), batches=dict(self.batches), queued=self.queued(),
                    prefetch_hints=self.prefetch_hints, dispatch="miss-aware" if self.miss_aware else "queue order",
                    early_loads=self.loads)


def serve_arrivals(router, arrivals, clock=time.monotonic, drain=True):
    """Open-loop replay of an arrival list [(gap_s, function)] against the wall clock: requests are
    submitted when due, whatever the backlog (sender_from_trace.py:51-57)."""
    t0 = clock()
    due, i, n = 0.0, 0, len(arrivals)
    if n:
        due = float(arrivals[0][0])
    while i < n or (drain and router.queued()):
        now = clock() - t0
        while i < n and due <= now:
            router.submit(int(arrivals[i][1]), t0 + due)
            i += 1
            if i < n:
                due += float(arrivals[i][0])
        if router.pump() == 0:
            # nothing to serve: until the next arrival, or until a model that is on its way has come far enough
            wake = router.wake_time()
            until = min(t0 + due if i < n else float("inf"), wake if wake is not None else float("inf"))
            while until != float("inf") and clock() < until:
                pass
    return clock() - t0


# ------------------------------------------------------------------------------------------ senders
def fixed_rate_arrivals(func_num, rate_per_min, mins, rng):
    """scripts/sender_fix_rate.py:46-56: every function at `rate_per_min`; per minute, as many gaps as
    requests, each drawn (in milliseconds) from a Poisson law whose mean is the mean gap."""
    out = []
    overall = int(rate_per_min * func_num)
    for _ in range(mins):
        gaps = rng.poisson(60 * 1000 / overall, overall)
        funcs = rng.choice(func_num, overall)
        out += [(g / 1000, int(f)) for g, f in zip(gaps, funcs)]
    return out


def trace_arrivals(patterns, func_num, rng):
    """scripts/sender_from_trace.py:19-32: each function follows one row of `patterns` (requests per
    minute, one column per minute), rows drawn with replacement."""
    patterns = np.asarray(patterns)
    rows = patterns[rng.choice(len(patterns), func_num)]
    out = []
    for minute in range(patterns.shape[1]):
        rates = rows[:, minute].astype(np.float64)
        overall = int(rates.sum())
        if overall <= 0:
            continue
        gaps = rng.poisson(60 * 1000 / overall, overall)
        funcs = rng.choice(func_num, overall, p=rates / rates.sum())
        out += [(g / 1000, int(f)) for g, f in zip(gaps, funcs)]
    return out


def synthetic_rate_patterns(n, mins, rng, mean_rpm=10.0):
    """Stand-in for the reference's trace sample (tools/samples.npy: 203 functions x 31 minutes of
    requests per minute, mean about 10, range 0..33): a per-function base rate with Poisson
    minute-to-minute variation."""
    base = rng.gamma(shape=6.0, scale=mean_rpm / 6.0, size=n)
    return rng.poisson(base[:, None], size=(n, mins)).astype(np.int64)


def keepalive_p99(arrivals):
    """tools/export_keepalive.py:13-27: per function, the 99th percentile of its inter-arrival times."""
    t, stamps = 0.0, collections.defaultdict(list)
    for gap, f in arrivals:
        t += gap
        stamps[int(f)].append(t)
    return {f: float(np.percentile(np.diff(s), 99)) for f, s in stamps.items() if len(s) > 1}


# ------------------------------------------------------------------------------------------ backend
class FunctionBackend:
    """Functions of `torpor_amd.functions` behind a server (in-process `Server` or wire `Client`).

    The reference's function container runs the model at batch = number of batched requests
    (tests/endpoint.py:84-92).  A function is registered at the router's batch limit; a full batch
    replays the recorded op stream in one call, a smaller one is issued op by op at its own size
    (`Function.invoke_rows`)."""

    def __init__(self, server, factory, example_inputs):
        # `server`: one in-process Server for every function, or a callable func_id -> connection
        # (each function container of the reference is a client of its own: RemoteServer(dir, client_id))
        self._owned = callable(server)
        self.server_for = server if callable(server) else (lambda func_id: server)
        self.factory, self.example_inputs = factory, example_inputs
        self.fn = {}
        self.conn = {}
        self.first = {}                 # answers of the registration run
        self.inputs = {}
        self.last = {}                  # answers of the last request when it ran below the registered batch

    def launch(self, func_id, level):
        self.conn[func_id] = self.server_for(func_id)
        fn = self.factory(self.conn[func_id], func_id, level)
        inputs = self.example_inputs(fn)
        first = fn.register(inputs)
        fn._weights = None              # the server's pinned store holds the authoritative copy now
        packed, outbuf, views = fn.pack(inputs)
        self.fn[func_id] = (fn, packed, outbuf, views)
        self.inputs[func_id] = inputs
        self.first[func_id] = [np.array(a, copy=True) for a in first]
        self.last[func_id] = None

    def outputs(self, func_id):
        """Answers of the last request of the function."""
        if self.last[func_id] is not None:
            return self.last[func_id]
        fn, _, _, views = self.fn[func_id]
        return fn.postprocess(views)

    def execute(self, func_id, n, prefetch=None):
        fn, packed, outbuf, _ = self.fn[func_id]
        batch = getattr(fn, "batch", n)
        if 0 < n < batch:               # fewer requests than the registered batch: run at that size
            self.last[func_id] = fn.invoke_rows([a[:n] for a in self.inputs[func_id]], n)
            return
        ack, _, deferred = self.conn[func_id].signal(1, func_id, "")
        if ack != 0 or deferred:
            raise RuntimeError(f"execute {func_id}: ack={ack} deferred={deferred}")
        if prefetch is not None and prefetch != func_id and prefetch in self.conn:
            # its copies queue behind this request's on the server's copy thread and run while this one computes
            self.conn[prefetch].signal(2, prefetch, "")
        self.conn[func_id].replay(func_id, packed, outbuf)
        self.last[func_id] = None

    def unload(self, func_id):
        self.conn[func_id].signal(3, func_id, "")

    def load(self, func_id):
        self.conn[func_id].signal(2, func_id, "")

    def resident(self, func_id):
        """Is the function's model in device memory (from the moment a swap-in has been started)?  An in-process
        server answers; over the wire there is no such query and every model counts as resident."""
        conn = self.conn[func_id]
        return conn.resident(func_id) if hasattr(conn, "resident") else True

    def load_estimate(self, func_id):
        """(swap-in, forward pass) in seconds, from the engine's own figures."""
        conn = self.conn[func_id]
        if not hasattr(conn, "load_estimate"):
            return 0.0, 0.0
        swap_ms, forward_ms = conn.load_estimate(func_id)
        return swap_ms * 1e-3, forward_ms * 1e-3

    def close(self):
        """Closes the per-function connections this backend opened (nothing for a shared server)."""
        if self._owned:
            for c in self.conn.values():
                c.close()
        self.conn.clear()


def build_function(server, func_id, level, model, batch):
    """One of the reference's served models (tests/endpoint.py:16-40) with seeded random weights."""
    from .functions import bert, densenet, efficientnet, inception, mobilenet, resnet
    name = mixed_model_name(func_id) if model == "mixed" else model
    if name in ("resnet50", "resnet101", "resnet152"):
        return resnet.ResNet(server, func_id, name, batch=batch, seed=func_id, level=level)
    if name in ("densenet121", "densenet169", "densenet201"):
        return densenet.DenseNet(server, func_id, name, batch=batch, seed=func_id, level=level)
    if name == "inception":
        return inception.InceptionV3(server, func_id, batch=batch, seed=func_id, level=level)
    if name == "efficientnet":
        return efficientnet.EfficientNetB0(server, func_id, batch=batch, seed=func_id, level=level)
    if name == "mobilenet":
        return mobilenet.MobileNetV2(server, func_id, batch=batch, seed=func_id, level=level)
    if name in ("bert", "bert-base"):
        return bert.Bert(server, func_id, "bert-base", batch=batch, seq=128, seed=func_id, level=level)
    if name == "bertqa":
        w = bert.init_weights("bert-large", seed=func_id, qa_head=True)
        return bert.Bert(server, func_id, "bert-large", batch=batch, seq=512, weights=w, level=level, token_types=True)
    raise ValueError(f"unknown model {name}")


def ones_inputs(fn):
    """The reference's endpoints feed all-ones inputs (tests/endpoint.py:53,66)."""
    return [np.ones(shape, dtype=dt) for shape, dt in fn.input_specs()]


def main(argv=None):
    ap = argparse.ArgumentParser(description="serve a synthetic request trace through the router on one GPU")
    ap.add_argument("-m", default="resnet152", help="model name or 'mixed' (router.py:502)")
    ap.add_argument("-f", type=int, default=1, help="number of functions")
    ap.add_argument("-t", type=int, default=98, help="SLO percentile")
    ap.add_argument("-d", type=int, default=100, help="latency deadline in ms (BERT question answering: twice that)")
    ap.add_argument("-b", type=int, default=1, help="batch size limit")
    ap.add_argument("-p", default="sa", choices=["sa", "fifo"])
    ap.add_argument("--rate", type=float, default=0.0, help="requests per minute per function; 0: trace patterns")
    ap.add_argument("--mins", type=int, default=1)
    ap.add_argument("--patterns", default=None, help=".npy of requests per minute [functions x minutes]")
    ap.add_argument("--speedup", type=float, default=1.0, help="divide every gap by this")
    ap.add_argument("--mem-gb", type=float, default=24.0)
    ap.add_argument("--connect", default=None, metavar="DIR",
                    help="serve through a running torpor_server whose sockets are in DIR (one connection per function) "
                         "instead of an in-process server")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--prefetch", action="store_true",
                    help="while a batch runs, ask the server to load the model of the request the queue hands out next")
    ap.add_argument("--dispatch", default="queue", choices=["queue", "miss-aware"],
                    help="miss-aware: requests of resident models are served while a swapped-out model streams in")
    a = ap.parse_args(argv)

    from .server import Server
    rng = np.random.default_rng(a.seed)
    if a.rate > 0:
        arrivals = fixed_rate_arrivals(a.f, a.rate, a.mins, rng)
    else:
        pat = np.load(a.patterns) if a.patterns else synthetic_rate_patterns(203, a.mins, rng)
        arrivals = trace_arrivals(pat[:, :a.mins], a.f, rng)
    arrivals = [(g / a.speedup, f) for g, f in arrivals]
    qa = {f for f in range(a.f) if a.m == "mixed" and mixed_model_name(f) == "bertqa"}

    def serve(server_or_factory, stats):
        backend = FunctionBackend(server_or_factory, lambda s, fid, lv: build_function(s, fid, lv, a.m, a.b), ones_inputs)
        router = Router(backend, a.t / 100, a.d / 1000, a.b, a.p, deadlines={f: 2 * a.d / 1000 for f in qa},
                        batch_limits={f: 1 for f in qa}, prefetch=a.prefetch,
                        miss_aware=a.dispatch == "miss-aware")
        for f in range(a.f):
            router.launch(f, mixed_model_level(f) if a.m == "mixed" else 1)
        for f in range(a.f):
            router.force_evict(f)
        wall = serve_arrivals(router, arrivals)
        out = router.summary()
        out.update(wall_s=wall, offered=len(arrivals), model=a.m, functions=a.f, **stats())
        backend.close()
        print(json.dumps(out))

    if a.connect:
        from .client import RemoteServer
        serve(lambda fid: RemoteServer(a.connect, client_id=fid), lambda: {"transport": "wire"})
    else:
        limit = int(a.mem_gb * 2 ** 30)
        with Server(mem_limit_bytes=limit, pool_bytes=limit + (2 << 30)) as server:
            serve(server, lambda: {"transport": "in-process", "pool": server.pool_stats()})


if __name__ == "__main__":
    main()
