"""Wire layer on the CPU: proto3 codec against hand-derived known-answer bytes and against the
installed protobuf runtime (descriptors built in code, no protoc); ZMTP framing constants; and
the whole request flow client -> torpor_server (host-only engine) over ipc:// sockets."""
import os
import signal
import subprocess
import tempfile
import time

import numpy as np
import pytest

from oracle import host_ref
from torpor_amd import client as wire
from torpor_amd.functions import resnet
from torpor_amd.server import ACK_INAVAIL, ACK_OK, OP_RELU, REQ_EXECUTE, REQ_EXECUTE_AFTER_LOAD, REQ_LOAD, REQ_UNLOAD

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SERVER_BIN = os.path.join(ROOT, "torpor_amd", "bin", "torpor_server")


# --------------------------------------------------------------------------------- codec
def test_signal_known_answer_bytes():
    """Derived by hand from the proto3 encoding rules for proto/signal.proto:16-30."""
    assert wire.signal_request(1, "7") == bytes.fromhex("0801120137")
    assert wire.signal_request(0, "0", "1") == bytes.fromhex("120130" "1a0131")       # enum 0 is omitted
    assert wire.signal_request(3, "12") == bytes.fromhex("0803" "12023132")
    assert host_ref.signal_ack_bytes(0, 0) == b""
    assert host_ref.signal_ack_bytes(0, -1) == bytes.fromhex("10ffffffffffffffffff01")   # int32 -1: 10-byte varint
    assert host_ref.signal_ack_bytes(1, 2) == bytes.fromhex("08011002")
    assert wire.parse_signal_ack(b"") == (0, 0)
    assert wire.parse_signal_ack(bytes.fromhex("10ffffffffffffffffff01")) == (0, -1)
    assert wire.parse_signal_ack(bytes.fromhex("08011002")) == (1, 2)
    for t, f, p in [(1, "7", ""), (0, "0", "1"), (2, "33", "0"), (3, "4095", "")]:
        assert wire.signal_request(t, f, p) == host_ref.signal_request_bytes(t, f, p)


def _pb_classes():
    """signal.proto and a few data-plane messages as runtime descriptors of google.protobuf."""
    pb = pytest.importorskip("google.protobuf")
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    T = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="t.proto", package="t", syntax="proto3")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, num, typ, rep in fields:
            m.field.add(name=fname, number=num, type=typ,
                        label=T.LABEL_REPEATED if rep else T.LABEL_OPTIONAL)
        return m

    msg("SignalRequest", [("type", 1, T.TYPE_INT32, 0), ("function", 2, T.TYPE_STRING, 0), ("payload", 3, T.TYPE_STRING, 0)])
    msg("SignalAck", [("ack", 1, T.TYPE_INT32, 0), ("resp", 2, T.TYPE_INT32, 0)])
    msg("WapperQuery", [("type", 1, T.TYPE_INT32, 0), ("query", 2, T.TYPE_BYTES, 0), ("client_id", 3, T.TYPE_INT32, 0),
                        ("need_sync", 4, T.TYPE_BOOL, 0)])
    msg("LaunchQuery", [("op_id", 20, T.TYPE_INT32, 0), ("ptrs", 21, T.TYPE_UINT64, 1), ("ints", 22, T.TYPE_INT64, 1),
                        ("floats", 23, T.TYPE_FLOAT, 1)])
    msg("SgemmQuery", [("transa", 2, T.TYPE_INT32, 0), ("transb", 3, T.TYPE_INT32, 0), ("m", 4, T.TYPE_INT32, 0),
                       ("n", 5, T.TYPE_INT32, 0), ("k", 6, T.TYPE_INT32, 0), ("alpha", 7, T.TYPE_FLOAT, 0),
                       ("matrix_a", 8, T.TYPE_UINT64, 0), ("lda", 9, T.TYPE_INT32, 0), ("matrix_b", 10, T.TYPE_UINT64, 0),
                       ("ldb", 11, T.TYPE_INT32, 0), ("beta", 12, T.TYPE_FLOAT, 0), ("matrix_c", 13, T.TYPE_UINT64, 0),
                       ("ldc", 14, T.TYPE_INT32, 0)])
    msg("BnQuery", [("x", 6, T.TYPE_UINT64, 0), ("epsilon", 14, T.TYPE_DOUBLE, 0), ("rows", 20, T.TYPE_INT64, 0)])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("t." + n))
            for n in ("SignalRequest", "SignalAck", "WapperQuery", "LaunchQuery", "SgemmQuery", "BnQuery")}


def test_codec_matches_protobuf_runtime():
    cls = _pb_classes()
    for t, f, p in [(1, "7", ""), (0, "0", "1"), (3, "12", "0"), (11, "", "x" * 300)]:
        ref = cls["SignalRequest"](type=t, function=f, payload=p).SerializeToString()
        assert wire.signal_request(t, f, p) == ref
    for ack, resp in [(0, 0), (0, -1), (1, 2), (0, 2 ** 31 - 1), (1, -2 ** 31)]:
        ref = cls["SignalAck"](ack=ack, resp=resp).SerializeToString()
        assert host_ref.signal_ack_bytes(ack, resp) == ref
        assert wire.parse_signal_ack(ref) == (ack, resp)
    # data plane: what the client writes parses to the same values in the protobuf runtime
    body = wire.Msg().u(20, 7).packed(21, [0x7A00000000000100, 0, 5]).packed(22, [128, 768]).packed_f32(23, [1e-12]).bytes()
    m = cls["LaunchQuery"].FromString(body)
    assert (m.op_id, list(m.ptrs), list(m.ints)) == (7, [0x7A00000000000100, 0, 5], [128, 768])
    assert np.float32(m.floats[0]) == np.float32(1e-12)
    assert body == cls["LaunchQuery"](op_id=7, ptrs=[0x7A00000000000100, 0, 5], ints=[128, 768],
                                      floats=[np.float32(1e-12)]).SerializeToString()
    sg = wire.Msg().u(2, 1).u(4, 768).u(5, 128).u(6, 768).f32(7, 1.0).u(8, 11).u(9, 768).u(10, 22).u(11, 768).u(13, 33).u(14, 768).bytes()
    ref = cls["SgemmQuery"](transa=1, m=768, n=128, k=768, alpha=1.0, matrix_a=11, lda=768, matrix_b=22, ldb=768,
                            matrix_c=33, ldc=768).SerializeToString()
    assert sg == ref
    bn = wire.Msg().u(6, 99).f64(14, 1e-5).u(20, 3136).bytes()
    assert bn == cls["BnQuery"](x=99, epsilon=1e-5, rows=3136).SerializeToString()
    wq = wire.Msg().u(1, 33).by(2, b"abc").u(3, 5).u(4, 1).bytes()
    assert wq == cls["WapperQuery"](type=33, query=b"abc", client_id=5, need_sync=True).SerializeToString()
    f = wire.parse(ref)
    assert f[4] == [768] and f[7] == [np.float32(1.0).tobytes()]


def test_zmtp_constants():
    """ZMTP 3.0 (rfc.zeromq.org/spec/23): greeting layout, READY command, short and long frames."""
    g = wire._greeting()
    assert len(g) == 64 and g[0] == 0xFF and g[1:9] == b"\0" * 8 and g[9] == 0x7F
    assert g[10:12] == b"\x03\x00" and g[12:32] == b"NULL" + b"\0" * 16 and g[32] == 0 and g[33:] == b"\0" * 31
    assert wire._ready("REP") == b"\x04\x19\x05READY\x0bSocket-Type\x00\x00\x00\x03REP"
    assert wire._ready("REQ").endswith(b"\x08Identity\x00\x00\x00\x00")
    assert wire._frame(b"hi") == b"\x00\x02hi" and wire._frame(b"", more=True) == b"\x01\x00"
    big = wire._frame(b"x" * 300)
    assert big[0] == 0x02 and big[1:9] == (300).to_bytes(8, "big") and len(big) == 309


# --------------------------------------------------------------------------------- end to end
@pytest.fixture(scope="module")
def wire_server():
    d = tempfile.mkdtemp(prefix="tpipc")
    env = dict(os.environ, TORPOR_IPC_DIR=d, TORPOR_HOST_ONLY="1", TORPOR_MEM_LIMIT_BYTES=str(330 << 20),
               TORPOR_POOL_BYTES=str(512 << 20), TORPOR_REQUEST_TIMEOUT_MS="300")
    p = subprocess.Popen([SERVER_BIN], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    line = p.stdout.readline()
    assert b"listening" in line, line
    yield d
    p.send_signal(signal.SIGTERM)
    try:
        p.wait(timeout=10)
    except subprocess.TimeoutExpired:
        p.kill()
    assert not os.path.exists(os.path.join(d, "signal_0"))


def test_request_flow_over_the_wire(wire_server):
    with wire.RemoteServer(wire_server, client_id=3) as rs:
        assert rs.signal(REQ_EXECUTE, 3)[0] == ACK_INAVAIL             # not registered yet
        assert rs.signal(REQ_UNLOAD, 3)[:2] == (ACK_OK, -1)
        # register: signal, upload, device sync, tracked first inference
        fn = resnet.ResNet(rs, 3, "resnet50", batch=1, seed=0, image=32)
        x = np.zeros((1, 3, 32, 32), np.float32)
        with pytest.raises(wire.WireError) as e:
            fn.register([x])                                           # host-only: completes, no data (-19)
        assert e.value.code == -19
        # 267 uploads + 58 ops went out in far fewer messages than queries (batching)
        assert rs.queries_sent > 600 and rs.messages_sent < rs.queries_sent
        assert rs.signal(REQ_EXECUTE, 3)[:2] == (ACK_OK, 0)
        with pytest.raises(wire.WireError):
            rs.malloc(3, 1 << 20)        # the activation arena is frozen after the first inference (-12)
        out = np.empty(1000, np.float32)
        with pytest.raises(wire.WireError) as e:
            rs.replay(3, x, out)
        assert e.value.code == -19
        assert rs.signal(REQ_UNLOAD, 3)[:2] == (ACK_OK, -1)
        assert rs.signal(REQ_LOAD, 3)[:2] == (ACK_OK, -1)
        assert rs.signal(REQ_UNLOAD, 3)[:2] == (ACK_OK, -1)
        assert rs.signal(10, 3)[0] == ACK_INAVAIL                      # ExecuteForRecord is refused


def test_deferred_ack_and_timeout_over_the_wire(wire_server):
    """A second Execute while the executor is busy gets its ack only after the first request ends
    (here by the 300 ms request timeout, cuda_server.hpp:257-264)."""
    with wire.RemoteServer(wire_server, client_id=4) as a, wire.RemoteServer(wire_server, client_id=5) as b:
        for rs, cid in ((a, 4), (b, 5)):
            assert rs.signal(REQ_EXECUTE_AFTER_LOAD, cid, "1")[0] == ACK_OK
            va = rs.malloc(cid, 1024)
            rs.h2d(cid, va, np.ones(256, np.float32))
            rs.device_synchronize(cid)
            act = rs.malloc(cid, 1024)
            rs.launch(cid, OP_RELU, [va, act], [256])
            out = np.empty(256, np.float32)
            rs.d2h_async(cid, out, act)
            with pytest.raises(wire.WireError):
                rs.stream_synchronize(cid)
        assert a.signal(REQ_EXECUTE, 4)[:2] == (ACK_OK, 0)
        t0 = time.time()
        assert b.signal(REQ_EXECUTE, 5)[:2] == (ACK_OK, 0)            # blocks until client 4's request times out
        assert 0.2 < time.time() - t0 < 5.0
        time.sleep(0.4)                                               # client 5's own request times out too
        assert a.signal(REQ_UNLOAD, 4)[0] == ACK_OK and b.signal(REQ_UNLOAD, 5)[0] == ACK_OK


def test_ack_of_a_queued_peer_that_died_is_not_handed_to_the_next_one(wire_server):
    """Two Execute signals are queued behind a running request; the first sender disconnects before its
    ack.  The second must get the ack of *its own* request and find itself active (its data-plane calls
    are accepted), not the orphaned ack of the dead peer's request."""
    ids = (6, 7, 8)
    conns = {cid: wire.RemoteServer(wire_server, client_id=cid) for cid in ids}
    try:
        for cid, rs in conns.items():
            assert rs.signal(REQ_EXECUTE_AFTER_LOAD, cid, "1")[0] == ACK_OK
            va = rs.malloc(cid, 1024)
            rs.h2d(cid, va, np.ones(256, np.float32))
            rs.device_synchronize(cid)
            act = rs.malloc(cid, 1024)
            rs.launch(cid, OP_RELU, [va, act], [256])
            rs.d2h_async(cid, np.empty(256, np.float32), act)
            with pytest.raises(wire.WireError):
                rs.stream_synchronize(cid)
        assert conns[6].signal(REQ_EXECUTE, 6)[:2] == (ACK_OK, 0)     # runs until its 300 ms timeout
        # client 7 queues an Execute and goes away without waiting for the ack
        conns[7].req.send([b"", wire.signal_request(REQ_EXECUTE, 7, "")])
        time.sleep(0.05)
        conns[7].close()
        t0 = time.time()
        assert conns[8].signal(REQ_EXECUTE, 8)[:2] == (ACK_OK, 0)     # answered when client 6's request ends
        assert 0.1 < time.time() - t0 < 5.0
        with pytest.raises(wire.WireError) as e:
            conns[8].malloc(8, 1 << 20)
        assert e.value.code == -12        # active (the frozen arena refuses); -72 would mean "not the active function"
        time.sleep(0.4)
        for cid in (6, 8):
            assert conns[cid].signal(REQ_UNLOAD, cid)[0] == ACK_OK
    finally:
        for cid in (6, 8):
            conns[cid].close()
