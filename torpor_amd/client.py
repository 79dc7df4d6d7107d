"""Client library for the server's wire interface (pure Python, no pyzmq / protoc needed).

Speaks ZMTP 3.0 over `ipc://` (AF_UNIX) and the proto3 messages of torpor_amd/proto/*.proto:
  - control plane: REQ to ipc://<dir>/signal_0, one SignalRequest -> one SignalAck
    (reference scripts/router.py:389-394 `send_signal`);
  - data plane: PUSH to ipc://<dir>/server_0 with QueryList batches, replies on a PULL bound at
    ipc://<dir>/client_<id>.  Batching follows the reference shim's AsyncSender
    (include/client/async_sender.hpp:13-14,50-98): asynchronous queries are queued and sent when 30
    are pending or 50 us have passed since the last send; a synchronous query flushes the queue
    and waits for exactly one reply.  Which query types are asynchronous follows
    common/include/cuda_common.hpp:80-106.

`RemoteServer` offers the same methods as `torpor_amd.server.Server`, so a served function
(torpor_amd/functions) runs unchanged in-process or over the wire.
"""
import os
import socket
import struct
import time

import numpy as np

from .server import ACT_NONE, NHWC

Q_DEVICE_SYNC, Q_STREAM_SYNC = 14, 23
Q_MALLOC, Q_FREE, Q_MEMCPY, Q_MEMCPY_ASYNC, Q_MEMSET_ASYNC = 30, 31, 32, 33, 34
Q_LAUNCH, Q_SGEMM, Q_SGEMM_BATCHED, Q_CONV, Q_BN, Q_GEMM, Q_REPLAY = 50, 104, 105, 211, 212, 300, 301
KIND_H2D, KIND_D2H, KIND_D2D = 1, 2, 3
BATCH_MAX_QUERIES = 30          # async_sender.hpp:13
BATCH_WINDOW_S = 50e-6          # async_sender.hpp:14


class WireError(RuntimeError):
    def __init__(self, code, what=""):
        self.code = code
        super().__init__(f"{what}: server error {code}")


# ------------------------------------------------------------------------------- proto3
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while v >= 0x80:
        out.append((v & 0x7F) | 0x80)
        v >>= 7
    out.append(v)
    return bytes(out)


class Msg:
    """proto3 writer: default-valued scalars are omitted."""

    def __init__(self):
        self.b = bytearray()

    def u(self, field, v):
        v = int(v)
        if v:
            self.b += _varint(field << 3) + _varint(v)
        return self

    def f32(self, field, v):
        raw = struct.pack("<f", v)
        if raw != b"\0\0\0\0":
            self.b += _varint((field << 3) | 5) + raw
        return self

    def f64(self, field, v):
        raw = struct.pack("<d", v)
        if raw != b"\0" * 8:
            self.b += _varint((field << 3) | 1) + raw
        return self

    def by(self, field, data):
        if len(data):
            self.b += _varint((field << 3) | 2) + _varint(len(data))
            self.b += data
        return self

    def sub(self, field, data):   # embedded message / repeated element, emitted even when empty
        self.b += _varint((field << 3) | 2) + _varint(len(data))
        self.b += data
        return self

    def packed(self, field, values):
        if len(values):
            self.sub(field, b"".join(_varint(int(v)) for v in values))
        return self

    def packed_f32(self, field, values):
        if len(values):
            self.sub(field, struct.pack(f"<{len(values)}f", *values))
        return self

    def bytes(self):
        return bytes(self.b)


def parse(data):
    """-> {field: [values]}; varints as int, fixed32/64 as raw bytes, length-delimited as memoryview."""
    out, mv, pos, n = {}, memoryview(data), 0, len(data)

    def varint():
        nonlocal pos
        v = shift = 0
        while True:
            b = mv[pos]
            pos += 1
            v |= (b & 0x7F) << shift
            if not b & 0x80:
                return v
            shift += 7

    while pos < n:
        key = varint()
        field, wt = key >> 3, key & 7
        if wt == 0:
            val = varint()
        elif wt == 1:
            val = bytes(mv[pos:pos + 8])
            pos += 8
        elif wt == 2:
            ln = varint()
            val = mv[pos:pos + ln]
            pos += ln
        elif wt == 5:
            val = bytes(mv[pos:pos + 4])
            pos += 4
        else:
            raise ValueError("bad wire type")
        out.setdefault(field, []).append(val)
    return out


def _i32(v):
    """int32 field value from its (sign-extended 64-bit) varint."""
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >> 63 else v


def signal_request(req_type, function, payload=""):
    return Msg().u(1, req_type).by(2, str(function).encode()).by(3, str(payload).encode()).bytes()


def parse_signal_ack(data):
    f = parse(data)
    return _i32(f.get(1, [0])[0]), _i32(f.get(2, [0])[0])


# ------------------------------------------------------------------------------- ZMTP 3.0
def _greeting():
    g = bytearray(64)
    g[0], g[9], g[10], g[11] = 0xFF, 0x7F, 3, 0
    g[12:16] = b"NULL"
    return bytes(g)


def _frame(body, more=False, command=False):
    flags = (1 if more else 0) | (4 if command else 0)
    if len(body) > 255:
        return bytes([flags | 2]) + struct.pack(">Q", len(body)) + bytes(body)
    return bytes([flags, len(body)]) + bytes(body)


def _ready(sock_type):
    body = b"\x05READY"
    props = [(b"Socket-Type", sock_type.encode())]
    if sock_type == "REQ":
        props.append((b"Identity", b""))
    for k, v in props:
        body += bytes([len(k)]) + k + struct.pack(">I", len(v)) + v
    return _frame(body, command=True)


_COMPAT = {"REQ": ("REP", "ROUTER"), "REP": ("REQ", "DEALER"), "PUSH": ("PULL",), "PULL": ("PUSH",)}


class ZConn:
    """One ZMTP peer connection over a connected AF_UNIX socket (blocking)."""

    def __init__(self, sock, sock_type, timeout=30.0):
        self.s, self.type = sock, sock_type
        self.s.settimeout(timeout)
        self.buf = bytearray()
        self.s.sendall(_greeting() + _ready(sock_type))
        g = self._read(64)
        if g[0] != 0xFF or g[9] != 0x7F or g[10] < 3 or bytes(g[12:17]) != b"NULL\0":
            raise ConnectionError("peer is not ZMTP 3.x / NULL")
        self.peer_type = None
        while self.peer_type is None:
            flags, body = self._read_frame()
            if flags & 4 and body[1:1 + body[0]] == b"READY":
                self.peer_type = self._parse_ready(body)
        if self.peer_type not in _COMPAT[sock_type]:
            raise ConnectionError(f"{sock_type} cannot talk to {self.peer_type}")

    @staticmethod
    def _parse_ready(body):
        p, t = 1 + body[0], ""
        while p < len(body):
            kl = body[p]
            key = bytes(body[p + 1:p + 1 + kl])
            p += 1 + kl
            (vl,) = struct.unpack(">I", body[p:p + 4])
            p += 4
            if key == b"Socket-Type":
                t = bytes(body[p:p + vl]).decode()
            p += vl
        return t

    def _read(self, n):
        while len(self.buf) < n:
            chunk = self.s.recv(1 << 20)
            if not chunk:
                raise ConnectionError("peer closed")
            self.buf += chunk
        out = self.buf[:n]
        del self.buf[:n]
        return out

    def _read_frame(self):
        h = self._read(2)
        flags, ln = h[0], h[1]
        if flags & 2:
            rest = self._read(7)
            (ln,) = struct.unpack(">Q", bytes(h[1:2]) + bytes(rest))
        return flags, self._read(ln)

    def send(self, frames):
        self.s.sendall(b"".join(_frame(f, more=(i + 1 < len(frames))) for i, f in enumerate(frames)))

    def recv(self):
        frames = []
        while True:
            flags, body = self._read_frame()
            if flags & 4:
                continue   # commands (PING/PONG) are not part of messages
            frames.append(bytes(body))
            if not flags & 1:
                return frames

    def close(self):
        try:
            self.s.close()
        except OSError:
            pass


def connect(path, sock_type, timeout=30.0, retry_s=5.0):
    deadline = time.time() + retry_s
    while True:
        s = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
        try:
            s.connect(path)
            return ZConn(s, sock_type, timeout)
        except (FileNotFoundError, ConnectionRefusedError):
            s.close()
            if time.time() > deadline:
                raise
            time.sleep(0.01)


class ZListener:
    """A bound socket that serves exactly one peer at a time (the client's PULL end)."""

    def __init__(self, path, sock_type, timeout=30.0):
        self.path, self.type, self.timeout = path, sock_type, timeout
        if os.path.exists(path):
            os.unlink(path)
        self.l = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
        self.l.bind(path)
        self.l.listen(8)
        self.l.settimeout(timeout)
        self.conn = None

    def recv(self):
        if self.conn is None:
            s, _ = self.l.accept()
            self.conn = ZConn(s, self.type, self.timeout)
        return self.conn.recv()

    def close(self):
        if self.conn:
            self.conn.close()
        self.l.close()
        if os.path.exists(self.path):
            os.unlink(self.path)


# ------------------------------------------------------------------------------- remote server
class RemoteServer:
    """Same surface as torpor_amd.server.Server, over the wire, for one client id."""

    def __init__(self, ipc_dir="/cuda", client_id=0, timeout=60.0):
        self.dir, self.cid = ipc_dir, int(client_id)
        self.pull = ZListener(os.path.join(ipc_dir, f"client_{self.cid}"), "PULL", timeout)
        self.req = connect(os.path.join(ipc_dir, "signal_0"), "REQ", timeout)
        self.push = connect(os.path.join(ipc_dir, "server_0"), "PUSH", timeout)
        self.queue = []
        self.last_send = time.perf_counter()
        self.d2h_targets = {}
        self.messages_sent = 0
        self.queries_sent = 0

    def close(self):
        for c in (self.req, self.push, self.pull):
            c.close()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # ---- control plane
    def signal(self, req_type, function, payload=""):
        self.req.send([b"", signal_request(req_type, function, payload)])
        frames = self.req.recv()
        ack, resp = parse_signal_ack(frames[-1])
        return ack, resp, False

    # ---- batching (async_sender.hpp:50-98)
    def _wrap(self, qtype, body, need_sync):
        return Msg().u(1, qtype).by(2, body).u(3, self.cid).u(4, 1 if need_sync else 0).bytes()

    def _flush(self):
        if not self.queue:
            return
        m = Msg()
        for q in self.queue:
            m.sub(1, q)
        self.push.send([m.bytes()])
        self.messages_sent += 1
        self.queries_sent += len(self.queue)
        self.queue = []
        self.last_send = time.perf_counter()

    def _async(self, qtype, body):
        self.queue.append(self._wrap(qtype, body, False))
        if len(self.queue) >= BATCH_MAX_QUERIES or time.perf_counter() - self.last_send >= BATCH_WINDOW_S:
            self._flush()

    def _sync(self, qtype, body):
        self.queue.append(self._wrap(qtype, body, True))
        self._flush()
        return parse(self.pull.recv()[-1])

    @staticmethod
    def _check(fields, what):
        err = _i32(fields.get(1, [0])[0])
        if err:
            raise WireError(err, what)

    # ---- data plane
    def malloc(self, fid, nbytes):
        f = self._sync(Q_MALLOC, Msg().u(1, nbytes).bytes())
        self._check(f, "malloc")
        return f.get(2, [0])[0]

    def free(self, fid, va):
        self._check(self._sync(Q_FREE, Msg().u(1, va).bytes()), "free")

    def h2d(self, fid, dst_va, array):
        a = np.ascontiguousarray(array)
        body = Msg().u(1, KIND_H2D).u(3, dst_va).u(4, a.nbytes).by(5, a.reshape(-1).view(np.uint8).data).bytes()
        self._async(Q_MEMCPY_ASYNC, body)

    def d2h_async(self, fid, out_array, src_va):
        key = out_array.ctypes.data
        self.d2h_targets[key] = out_array
        self._async(Q_MEMCPY_ASYNC, Msg().u(1, KIND_D2H).u(2, src_va).u(3, key).u(4, out_array.nbytes).bytes())

    def d2h(self, fid, out_array, src_va):
        f = self._sync(Q_MEMCPY, Msg().u(1, KIND_D2H).u(2, src_va).u(4, out_array.nbytes).bytes())
        self._check(f, "memcpy d2h")
        out_array.reshape(-1).view(np.uint8)[:] = np.frombuffer(f[2][0], dtype=np.uint8)

    def d2d(self, fid, dst_va, src_va, nbytes):
        self._async(Q_MEMCPY_ASYNC, Msg().u(1, KIND_D2D).u(2, src_va).u(3, dst_va).u(4, nbytes).bytes())

    def memset(self, fid, dst_va, value, nbytes):
        self._async(Q_MEMSET_ASYNC, Msg().u(1, dst_va).u(2, value).u(3, nbytes).bytes())

    def device_synchronize(self, fid):
        self._check(self._sync(Q_DEVICE_SYNC, b""), "device_synchronize")

    def stream_synchronize(self, fid):
        f = self._sync(Q_STREAM_SYNC, b"")
        err = _i32(f.get(1, [0])[0])
        for r in f.get(2, []):
            e = parse(r)
            target = self.d2h_targets.pop(e.get(1, [0])[0], None)
            if target is not None and not err and 2 in e:
                target.reshape(-1).view(np.uint8)[:] = np.frombuffer(e[2][0], dtype=np.uint8)
        if err:
            raise WireError(err, "stream_synchronize")

    @staticmethod
    def _ep(alpha=1.0, beta=0.0, bias=0, bn=None, bn_eps=1e-5, residual=0, ldr=0, act=ACT_NONE):
        m = Msg().f32(1, alpha).f32(2, beta).u(3, bias)
        if bn is not None:
            m.u(4, bn[0]).u(5, bn[1]).u(6, bn[2]).u(7, bn[3])
        return m.f32(8, bn_eps).u(9, act).u(10, residual).u(11, ldr).bytes()

    def gemm(self, fid, x, y, c, m, n, k, xs_r, ys_c, ldc, xs_k=1, ys_k=1, nb0=1, nb1=1,
             xb0=0, xb1=0, yb0=0, yb1=0, cb0=0, cb1=0, **ep):
        b = Msg().u(1, x).u(2, y).u(3, c).u(4, m).u(5, n).u(6, k).u(7, xs_r).u(8, xs_k).u(9, ys_c).u(10, ys_k)
        b.u(11, ldc).u(12, nb0).u(13, nb1).u(14, xb0).u(15, xb1).u(16, yb0).u(17, yb1).u(18, cb0).u(19, cb1)
        # explicit zero strides must survive proto3 default elision: xs_k / ys_k default to 1 on the server
        b.sub(20, self._ep(**ep))
        self._async(Q_GEMM, b.bytes())

    def sgemm(self, fid, transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
        body = Msg().u(2, transa).u(3, transb).u(4, m).u(5, n).u(6, k).f32(7, alpha).u(8, a).u(9, lda).u(10, b)
        self._async(Q_SGEMM, body.u(11, ldb).f32(12, beta).u(13, c).u(14, ldc).bytes())

    def sgemm_strided_batched(self, fid, transa, transb, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta, c, ldc, sc,
                              count):
        body = Msg().u(2, transa).u(3, transb).u(4, m).u(5, n).u(6, k).f32(7, alpha).u(8, a).u(9, lda).u(10, b)
        body.u(11, ldb).f32(12, beta).u(13, c).u(14, ldc).u(15, sa).u(16, sb).u(17, sc).u(18, count)
        self._async(Q_SGEMM_BATCHED, body.bytes())

    def conv(self, fid, x, w, y, n, h, w_in, cin, cout, kh, kw, stride=1, pad=0, x_layout=NHWC, y_layout=NHWC,
             groups=1, x_pitch=0, y_pitch=0, **ep):
        sh, sw = (stride, stride) if isinstance(stride, int) else stride
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        b = Msg().u(4, x).u(6, w).u(13, y).u(20, n).u(21, h).u(22, w_in).u(23, cin).u(24, cout).u(25, kh).u(26, kw)
        b.u(27, sh).u(28, sw).u(29, ph).u(30, pw).u(31, groups).u(32, x_layout).u(33, y_layout)
        b.sub(34, self._ep(**ep)).u(35, x_pitch).u(36, y_pitch)
        self._async(Q_CONV, b.bytes())

    def bn(self, fid, x, y, scale, bias, mean, var, eps, rows, channels, hw=1, layout=NHWC, relu=False, x_pitch=0):
        b = Msg().u(6, x).u(8, y).u(10, scale).u(11, bias).u(12, mean).u(13, var).f64(14, eps)
        b.u(20, rows).u(21, channels).u(22, hw).u(23, layout).u(24, int(relu)).u(25, x_pitch)
        self._async(Q_BN, b.bytes())

    def launch(self, fid, op_id, ptrs, ints=(), floats=()):
        # packed repeated fields keep zero elements (a null pointer slot must stay in place)
        self._async(Q_LAUNCH, Msg().u(20, op_id).packed(21, ptrs).packed(22, ints).packed_f32(23, floats).bytes())

    def replay(self, fid, input_array, output_array):
        """One message per request: the server re-issues the op stream it recorded at registration."""
        a = np.ascontiguousarray(input_array)
        f = self._sync(Q_REPLAY, Msg().by(1, a.reshape(-1).view(np.uint8).data).u(2, output_array.nbytes).bytes())
        self._check(f, "replay")
        output_array.reshape(-1).view(np.uint8)[:] = np.frombuffer(f[2][0], dtype=np.uint8)
