"""TEST INFRASTRUCTURE ONLY: Python restatement of the reference's host-side decisions.

  LruRef      include/server/evictor.hpp:190-264 (LRUEvictor), single GPU.  One difference is
              made explicit: where the reference would loop forever (nothing unlocked left to
              evict, evictor.hpp:211-224) `check_and_add` stops evicting and inserts anyway.
  IaRef       include/server/evictor.hpp:28-188 (InterferenceAwareEvictor), any number of GPUs,
              kept in the reference's own shape (two recency lists per GPU).  Same explicit
              difference: the search of the protected list stops when nothing unlocked is left
              (the reference would loop forever, evictor.hpp:85-97).
  SchedRef    include/server/controller.hpp:271-389: round-robin placement and the random /
              interference-aware scheduling decisions over executor states, residency and the
              PCIe-sibling and peer-link tables (defaults: the reference's 4-GPU tables,
              controller.hpp:117-118).
  FixedBlocksRef  include/server/block_manager.hpp:188-258 (FixedSizeBlockManager): a byte budget over
              raw device allocations, idle lists per exact size (taken from the back), and idle blocks
              freed largest size first (the map is ordered by std::greater, common/include/types.hpp:31)
              when the budget does not cover a new size.  Blocks are numbered instead of addressed.
  signal_*    proto3 wire bytes of proto/signal.proto:5-30, written from the protobuf encoding
              spec (varint field keys, length-delimited strings, default values omitted).

Pinning: LruRef is checked against a brute-force list model on random traces
(tests/test_host_logic.py); IaRef against LruRef where the two policies must coincide (one GPU,
one level), against the policy's defining invariant (a model of level >= 1 is protected exactly
when one GPU holds it) on random multi-GPU traces, and on hand-worked traces; SchedRef on
hand-worked cases over the reference's 4-GPU tables and against exhaustive properties (never a
busy GPU, a resident idle GPU always wins, the sibling-status minimum); the codec against the known-answer byte strings derived by hand from
the proto3 spec and against the installed `google.protobuf` runtime with a descriptor built in
code (tests/test_wire.py); FixedBlocksRef on a hand-worked trace read off the reference's code and by
conservation (budget + bytes of live and idle blocks is constant, tests/test_host_logic.py).
"""
from collections import OrderedDict


class LruRef:
    def __init__(self, budget):
        self.budget = budget
        self.items = OrderedDict()   # most recent last
        self.locked = set()
        self.cur = 0

    def check_and_add(self, func, sz):
        if func in self.items:                     # evictor.hpp:202-206
            self.items.move_to_end(func)
            return []
        victims = []
        while self.cur + sz >= self.budget:        # evictor.hpp:211
            cand = next((f for f in self.items if f not in self.locked), None)   # oldest unlocked
            if cand is None:
                break
            victims.append(cand)
            self.cur -= self.items.pop(cand)
        self.items[func] = sz                      # evictor.hpp:230-232
        self.cur += sz
        return victims

    def force_evict(self, func):                   # evictor.hpp:237-247
        if func in self.items:
            self.cur -= self.items.pop(func)
            return True
        return False

    def lock(self, func):
        if func in self.items:
            self.locked.add(func)

    def unlock(self, func):
        self.locked.discard(func)


class FixedBlocksRef:
    def __init__(self, budget):
        self.budget = budget
        self.idle = {}            # size -> [block ids], released last at the back
        self.next_block = 0
        self.over_budget = 0      # block_manager.hpp:222-234: allocated although the budget was spent

    def acquire(self, size):
        """Returns (block, reused, freed): the block handed out, whether it came from the idle list of
        its size, and the idle blocks freed to make room, in order."""
        lst = self.idle.get(size)
        if lst:                                            # block_manager.hpp:193-198
            return lst.pop(), True, []
        freed = []
        if self.budget < size:                             # block_manager.hpp:205-221
            for sz in sorted(self.idle, reverse=True):     # std::map<..., std::greater<>>: largest first
                blocks = self.idle[sz]
                while blocks:
                    freed.append((blocks.pop(), sz))
                    self.budget += sz
                    if self.budget >= size:
                        break
                if self.budget >= size:
                    break
        if self.budget >= size:
            self.budget -= size
        else:
            self.over_budget += 1
        block = self.next_block
        self.next_block += 1
        return block, False, freed

    def evict(self, block, size):                          # block_manager.hpp:243-252, free_flag == false
        self.idle.setdefault(size, []).append(block)

    def idle_bytes(self):
        return sum(sz * len(b) for sz, b in self.idle.items())


class IaRef:
    """Two recency lists per GPU; index 0 of a list is the most recent entry (evictor.hpp:181-186)."""

    def __init__(self, gpu_count, budget):
        self.budget = budget
        self.first = [[] for _ in range(gpu_count)]     # protected: [name, size], evicted last
        self.second = [[] for _ in range(gpu_count)]
        self.locked = [set() for _ in range(gpu_count)]
        self.cur = [0] * gpu_count
        self.gpus = {}                                   # model_to_gpus
        self.level = {}                                  # model_level_map (controller.hpp:472)

    @staticmethod
    def _find(lst, func):
        return next((i for i, e in enumerate(lst) if e[0] == func), None)

    def _move(self, src, dst, func):
        i = self._find(src, func)
        if i is None:
            return False
        dst.insert(0, src.pop(i))
        return True

    def check_and_add(self, gpu, func, sz):
        if gpu in self.gpus.get(func, set()):            # evictor.hpp:43-60
            if not self._move(self.first[gpu], self.first[gpu], func):
                self._move(self.second[gpu], self.second[gpu], func)
            return []
        victims = []
        for lst in (self.second[gpu], self.first[gpu]):  # evictor.hpp:65-97
            while self.cur[gpu] + sz >= self.budget:
                i = next((k for k in range(len(lst) - 1, -1, -1) if lst[k][0] not in self.locked[gpu]), None)
                if i is None:
                    break
                name, size = lst.pop(i)
                victims.append(name)
                self.cur[gpu] -= size
        holders = self.gpus.setdefault(func, set())
        heavy = self.level.get(func, 0) >= 1
        if heavy and not holders:                        # evictor.hpp:99-103
            self.first[gpu].insert(0, [func, sz])
        else:                                            # evictor.hpp:104-122
            self.second[gpu].insert(0, [func, sz])
            if heavy:
                for g in sorted(holders):
                    self._move(self.first[g], self.second[g], func)
        holders.add(gpu)
        self.cur[gpu] += sz
        for mod in victims:                              # evictor.hpp:126-144
            left = self.gpus.setdefault(mod, set())
            left.discard(gpu)
            if self.level.get(mod, 0) >= 1 and len(left) == 1:
                g = next(iter(left))
                self._move(self.second[g], self.first[g], mod)
        return victims

    def force_evict(self, gpu, func):                    # evictor.hpp:149-170
        hit = False
        for lst in (self.first[gpu], self.second[gpu]):
            i = self._find(lst, func)
            if i is not None:
                self.cur[gpu] -= lst.pop(i)[1]
                hit = True
                break
        self.gpus.setdefault(func, set()).discard(gpu)
        return hit

    def lock(self, gpu, func):                           # evictor.hpp:172-174
        self.locked[gpu].add(func)

    def unlock(self, gpu, func):                         # evictor.hpp:176-180
        self.locked[gpu].discard(func)

    def order(self, gpu):
        """Eviction order, first victim first."""
        return [e[0] for e in reversed(self.second[gpu])] + [e[0] for e in reversed(self.first[gpu])]


class SchedRef:
    AVAIL, LOCAL, PEER, HOST_LIGHT, HOST_MEDIAN, HOST_HEAVY, COLD = -1, 0, 1, 2, 3, 4, 5   # controller.hpp:18-24

    def __init__(self, gpu_count=4, sibling=(1, 0, 3, 2),
                 link=((0, 1, 1, 2), (1, 0, 2, 1), (1, 2, 0, 2), (2, 1, 2, 0))):   # controller.hpp:117-118
        self.n = gpu_count
        self.status = [self.AVAIL] * gpu_count
        self.sibling = list(sibling)
        self.link = [list(r) for r in link]
        self.resident = {}
        self.level = {}
        self.rr = 0

    def _host_status(self, func):                        # controller.hpp:26-32
        lv = self.level.get(func, 0)
        return lv + self.HOST_LIGHT if 0 <= lv <= 2 else self.HOST_MEDIAN

    def placement(self):                                 # controller.hpp:271-294
        if self.status[self.rr] == self.AVAIL:
            g = self.rr
            self.rr = (self.rr + 1) % self.n
            return g
        return next((i for i in range(self.n) if self.status[i] == self.AVAIL), -1)

    def random_schedule(self, func, draw):               # controller.hpp:296-319 ; draw stands for rand()
        idle = [i for i in range(self.n) if self.status[i] == self.AVAIL]
        if not idle:
            return (-1, -1, -1)
        for g in sorted(self.resident.get(func, ())):
            if self.status[g] == self.AVAIL:
                return (g, -1, self.LOCAL)
        return (idle[draw % len(idle)], -1, self._host_status(func))

    def interference_aware_schedule(self, func):         # controller.hpp:321-389
        idle = [i for i in range(self.n) if self.status[i] == self.AVAIL]
        if not idle:
            return (-1, -1, -1)
        holders = sorted(self.resident.get(func, ()))
        if holders:
            for g in holders:
                if self.status[g] == self.AVAIL:
                    return (g, -1, self.LOCAL)
            dst, src = idle[0], holders[0]
            for i in idle:                               # controller.hpp:347-355: the inner break only
                for j in holders:
                    if self.link[i][j] == 2:
                        dst, src = i, j
                        break
            return (dst, src, self.PEER)
        best, best_status = idle[0], self.status[self.sibling[idle[0]]]
        for g in idle:                                   # controller.hpp:379-385
            if self.status[self.sibling[g]] < best_status:
                best_status = self.status[self.sibling[g]]
                best = g
        return (best, -1, self._host_status(func))


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def signal_request_bytes(req_type, function, payload=""):
    """SignalRequest{type=1 enum, function=2 string, payload=3 string} (signal.proto:16-20)."""
    out = b""
    if req_type:
        out += b"\x08" + _varint(req_type)
    if function:
        f = function.encode()
        out += b"\x12" + _varint(len(f)) + f
    if payload:
        p = payload.encode()
        out += b"\x1a" + _varint(len(p)) + p
    return out


def signal_ack_bytes(ack, resp):
    """SignalAck{ack=1 enum, resp=2 int32} (signal.proto:27-30); negative int32 = 10-byte varint."""
    out = b""
    if ack:
        out += b"\x08" + _varint(ack)
    if resp:
        out += b"\x10" + _varint(resp)
    return out
