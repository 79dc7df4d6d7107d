"""Miss-aware dispatch for one executor.

The reference's router hands requests to the server one after the other (scripts/router.py:289-313) and the
controller queues an Execute while the executor is busy (include/server/controller.hpp:163-186, 242-262), so a
request of a swapped-out model holds up every request behind it for the whole swap-in.  The executor itself is
mostly idle during that time: it waits for the host link.  This dispatcher keeps the reference's rule of one
active function per executor and changes only the order in which a queue of arrived requests is handed over:

  * the oldest queued request whose model is swapped out gets its swap-in started at once with the
    reference's prefetch signal, Load (controller.hpp:208-215) -- one swap-in at a time, in arrival order;
  * while it streams, queued requests of resident models are served, oldest first;
  * the request that waits for the swap-in is started when the rest of its copy is about as long as its forward
    pass (from the engine's own estimate: link time of the bytes the request waits for, forward time measured at
    registration), so that it ends when it would have ended had it held the executor from the start -- the
    engine pipelines the tail of the copy with the forward pass either way;
  * requests of one function are never reordered among themselves.

Pure decision logic on a clock the caller owns (seconds as floats): nothing here touches the server.  The serving
loop in torpor_amd/multitenant.py drives it; oracle/router_ref.py restates the policy as a whole-trace simulation.
"""


class Request:
    __slots__ = ("seq", "fid", "arrival", "miss")

    def __init__(self, seq, fid, arrival):
        self.seq, self.fid, self.arrival = seq, fid, arrival
        self.miss = False


class MissAwareDispatcher:
    """decide(now, resident) -> ("load", request) | ("run", request) | ("idle", wake_time or None).

    After a "load" the caller sends the Load signal and reports load_started(fid, now, swap_s, forward_s); after a
    "run" it executes the request (which leaves the queue with the decision).  `resident(fid)` is the engine's
    residency test (true from the moment a swap-in has been started).  margin_s: how much earlier than
    (end of copy - forward pass) a waiting request is started, to absorb the service time of a request of a
    resident model that happens to be running then."""

    def __init__(self, margin_s=0.0003, max_loading=1):
        self.queue = []          # arrival order
        self.loading = {}        # fid -> time from which its oldest request is started
        self.margin_s = margin_s
        self.max_loading = max_loading
        self.loads = 0

    def arrive(self, seq, fid, arrival):
        self.queue.append(Request(seq, fid, arrival))

    def __len__(self):
        return len(self.queue)

    def load_started(self, fid, now, swap_s, forward_s):
        self.loading[fid] = now + max(0.0, swap_s - forward_s - self.margin_s)
        self.loads += 1

    def load_failed(self, fid):
        self.loading.pop(fid, None)

    def decide(self, now, resident):
        q = self.queue
        # 1. the oldest request of a swapped-out model: start its swap-in (one at a time)
        if len(self.loading) < self.max_loading:
            for r in q:
                if r.fid not in self.loading and not resident(r.fid):
                    r.miss = True
                    return ("load", r)
        # 2. a request whose swap-in has come far enough: it goes first, so that waiting costs it nothing
        due = None
        for r in q:
            t = self.loading.get(r.fid)
            if t is not None and t <= now:
                due = r
                break
        if due is not None:
            q.remove(due)
            del self.loading[due.fid]
            return ("run", due)
        # 3. the oldest request of a resident model that is not being swapped in
        for r in q:
            if r.fid not in self.loading and resident(r.fid):
                q.remove(r)
                return ("run", r)
        # 4. nothing can run: sleep until the waiting request's time (or the next arrival, whichever the caller sees first)
        if self.loading:
            waiting = [t for f, t in self.loading.items() if any(r.fid == f for r in q)]
            if waiting:
                return ("idle", min(waiting))
            self.loading.clear()   # loads whose requests are gone (cannot happen through this interface)
        return ("idle", None)


class InOrderDispatcher:
    """Arrival order, as the reference serves (scripts/router.py:289-313): the comparison case."""

    def __init__(self):
        self.queue = []
        self.loads = 0

    def arrive(self, seq, fid, arrival):
        self.queue.append(Request(seq, fid, arrival))

    def __len__(self):
        return len(self.queue)

    def load_started(self, fid, now, swap_s, forward_s):
        pass

    def load_failed(self, fid):
        pass

    def decide(self, now, resident):
        if not self.queue:
            return ("idle", None)
        r = self.queue.pop(0)
        r.miss = not resident(r.fid)
        return ("run", r)
