"""TEST INFRASTRUCTURE ONLY: Python restatement of the reference's host-side decisions.

  LruRef      include/server/evictor.hpp:190-264 (LRUEvictor), single GPU.  One difference is
              made explicit: where the reference would loop forever (nothing unlocked left to
              evict, evictor.hpp:211-224) `check_and_add` stops evicting and inserts anyway.
  signal_*    proto3 wire bytes of proto/signal.proto:5-30, written from the protobuf encoding
              spec (varint field keys, length-delimited strings, default values omitted).

Pinning: LruRef is checked against a brute-force list model on random traces
(tests/test_host_logic.py); the codec against the known-answer byte strings derived by hand from
the proto3 spec and against the installed `google.protobuf` runtime with a descriptor built in
code (tests/test_wire.py).
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
