"""Swap engine, pool and LRU on the device: eviction under a binding budget, repeated
swap-in / swap-out, prefetch (Load), gate ordering with a poisoned pool."""
import os

import numpy as np
import pytest

from torpor_amd.functions import bert, resnet
from torpor_amd.functions.base import Function
from torpor_amd.server import ACK_INAVAIL, ACK_OK, REQ_EXECUTE, REQ_LOAD, REQ_UNLOAD, Server

pytestmark = pytest.mark.gpu


def _mk(server, fid, seed, image=64):
    fn = resnet.ResNet(server, fid, "resnet50", batch=1, seed=seed, image=image)
    x = np.random.default_rng(seed).standard_normal((1, 3, image, image)).astype(np.float32)
    (y,) = fn.register([x])
    return fn, x, y


def test_lru_eviction_and_identity():
    """Budget fits two ResNet-50s: registering / invoking a third evicts the least recently
    used one; every model still answers with its own bits after being swapped back in."""
    with Server(mem_limit_bytes=300 << 20, pool_bytes=512 << 20, chunk_bytes=1 << 20) as s:
        fns = [_mk(s, i, seed=i) for i in range(3)]
        info = s.model_info(0)
        assert 2 * info["total_bytes"] < (300 << 20) <= 3 * info["total_bytes"]
        assert [s.resident(i) for i in range(3)] == [False, True, True]
        order = [0, 1, 2, 2, 0, 1, 0, 2, 1, 1, 0]
        for i in order:
            fn, x, y = fns[i]
            (got,) = fn.invoke([x])
            assert np.array_equal(got, y), f"model {i} changed its answer after swapping"
            assert s.resident(i)
            assert sum(s.resident(j) for j in range(3)) <= 2
            st = s.pool_stats()
            assert st["lru_used"] < st["lru_budget"] and st["used"] <= st["capacity"]
        st = s.pool_stats()
        assert st["evictions"] >= 5 and st["swap_ins"] >= 5
        for i in range(3):
            if s.resident(i):
                assert np.array_equal(s.readback_weights(i), s.host_weights(i))


def test_prefetch_then_invoke(gpu_server):
    fn, x, y = _mk(gpu_server, 20, seed=7)
    assert fn.unload()[0] == ACK_OK and not gpu_server.resident(20)
    ack, resp, _ = fn.load()
    assert ack == ACK_OK and gpu_server.resident(20)
    assert np.array_equal(gpu_server.readback_weights(20), gpu_server.host_weights(20))
    (got,) = fn.invoke([x])
    assert np.array_equal(got, y)
    fn.unload()


def test_unknown_and_active_function(gpu_server):
    ack, _, _ = gpu_server.signal(REQ_EXECUTE, 3999, "")
    assert ack == ACK_INAVAIL
    ack, resp, _ = gpu_server.signal(REQ_UNLOAD, 3999, "")
    assert ack == ACK_OK and resp == -1
    assert gpu_server.signal(REQ_LOAD, 3999, "")[0] == ACK_INAVAIL


def test_gate_orders_compute_after_copy():
    """Tiny gate groups (BUFFER_SIZE=1-style ablation): every op waits for exactly its own
    tensor.  The pool is poisoned between swap-out and swap-in by another model's weights, so
    an op that ran ahead of its copy would read foreign bytes and change the logits."""
    with Server(mem_limit_bytes=200 << 20, pool_bytes=384 << 20, chunk_bytes=256, chunk_max_bytes=64 << 10) as s:
        a, xa, ya = _mk(s, 0, seed=11)
        b, xb, yb = _mk(s, 1, seed=12)   # evicts model 0 (budget holds one)
        assert not s.resident(0) and s.resident(1)
        for _ in range(3):
            (ga,) = a.invoke([xa])
            assert np.array_equal(ga, ya)
            assert s.swap_stats(0)["gate_waits"] > 50
            (gb,) = b.invoke([xb])
            assert np.array_equal(gb, yb)


def test_graph_replays_match_eager_and_follow_the_placement(monkeypatch):
    """TORPOR_GRAPH_MIN_OPS: warm requests launch the compute part of the program as one HIP graph.
    Every replay of the graph must equal the eager answer, with other models' eager work and
    synchronisations in between, and a swap-out / swap-in (new addresses) must re-capture."""
    monkeypatch.setenv("TORPOR_GRAPH_MIN_OPS", "8")
    with Server(mem_limit_bytes=300 << 20, pool_bytes=512 << 20) as s:
        fa, xa, ya = _mk(s, 0, seed=3)
        fb, xb, yb = _mk(s, 1, seed=4)
        for rnd in range(3):
            for i in range(5):                      # the second warm request captures, the rest replay
                (got,) = fa.invoke([xa])
                assert np.array_equal(got, ya), (rnd, i)
                (gb,) = fb.invoke([xb], replay=False)    # eager, op by op, between the replays
                assert np.array_equal(gb, yb)
            x2 = xa + 1.0                            # new inputs through the same graph
            (g2,) = fa.invoke([x2])
            (e2,) = fa.invoke([x2], replay=False)
            assert np.array_equal(g2, e2) and not np.array_equal(g2, ya)
            assert fa.unload()[0] == ACK_OK          # placement is dropped ...
            _mk(s, 2 + rnd, seed=5 + rnd)            # ... and the pool re-used, so it comes back elsewhere or not
            (cold,) = fa.invoke([xa])
            assert np.array_equal(cold, ya)


@pytest.mark.parametrize("host_gather", [True, False])
def test_embedding_table_travels_last_and_is_read_in_place_meanwhile(host_gather, monkeypatch):
    """The word-embedding table is looked up by row, so it is the last tensor of the image, and a
    cold request reads its rows from the pinned host store while the table is still on its way;
    with the option off the lookup waits for the table.  Either way cold answers equal warm ones
    bit for bit and the device copy ends up identical to the host store."""
    monkeypatch.delenv("TORPOR_HOST_GATHER", raising=False)   # the flag under test, not the environment
    cfg = dict(layers=2, hidden=512, heads=8, ffn=1024)
    weights = bert.init_weights(seed=21, vocab=30522, max_pos=128, cfg=cfg)   # table: 62 MB of 71
    ids = np.random.default_rng(4).integers(0, 30522, (2, 64))
    with Server(mem_limit_bytes=1 << 30, host_gather=host_gather) as s:
        fn = bert.Bert(s, 3, batch=2, seq=64, weights=weights, cfg=cfg)
        first = fn.register([ids])
        off = {k: s.weight_offset(3, va) for k, va in fn.w.items()}
        assert off["embeddings.word_embeddings.weight"] == max(off.values())
        assert off["embeddings.position_embeddings.weight"] < off["encoder.layer.0.output.dense.weight"]
        for _ in range(3):
            fn.unload()
            cold = fn.invoke([ids])
            st = s.swap_stats(3)
            assert st["host_gathers"] == (1 if host_gather else 0)
            warm = fn.invoke([ids])
            assert s.swap_stats(3)["host_gathers"] == 0
            for a, b, c in zip(first, cold, warm):
                assert np.array_equal(a, b) and np.array_equal(a, c)
            assert np.array_equal(s.readback_weights(3), s.host_weights(3))
        fn.unload()


def _assert_host_store_holds_the_upload(s, fn, host):
    """Every uploaded tensor sits unmodified at its offset of the host copy of the image."""
    for name, arr in fn.weights().items():
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        off = s.weight_offset(fn.fid, fn.w[name])
        assert np.array_equal(host[off:off + raw.size], raw), name


@pytest.mark.parametrize("keep", [False, True])
def test_host_store_is_the_transfer_image_plus_the_tables(keep, monkeypatch):
    """By default a packed model's raw image is released once its transfer image has been decoded back to it
    on the host: pinned memory holds the transfer image and a raw copy of the tables that lookups read in place
    during a swap-in.  tp_host_weights then decodes on demand, and what it returns is the upload, byte for
    byte; cold requests still read table rows from host memory and answer as at registration."""
    monkeypatch.delenv("TORPOR_SLIM_HOST", raising=False)
    monkeypatch.delenv("TORPOR_PACK", raising=False)
    monkeypatch.delenv("TORPOR_HOST_GATHER", raising=False)
    cfg = dict(layers=2, hidden=512, heads=8, ffn=1024)
    weights = bert.init_weights(seed=22, vocab=30522, max_pos=128, cfg=cfg)   # word table: 62 MB of 71
    ids = np.random.default_rng(5).integers(0, 30522, (2, 64))
    with Server(mem_limit_bytes=1 << 30, keep_host_image=keep) as s:
        fn = bert.Bert(s, 3, batch=2, seq=64, weights=weights, cfg=cfg)
        first = fn.register([ids])
        info = s.model_info(3)
        image = info["image_bytes"]
        st = s.pool_stats()
        table = weights["embeddings.word_embeddings.weight"].nbytes
        assert 0.82 * image < st["host_transfer_bytes"] < 0.91 * image
        if keep:
            assert st["host_image_bytes"] == image
        else:
            assert table <= st["host_image_bytes"] < table + (1 << 20)   # the table (plus alignment), nothing else
        host = s.host_weights(3)
        _assert_host_store_holds_the_upload(s, fn, host)
        for _ in range(3):
            fn.unload()
            cold = fn.invoke([ids])
            assert s.swap_stats(3)["host_gathers"] == 1
            for a, b in zip(first, cold):
                assert np.array_equal(a, b)
            assert np.array_equal(s.readback_weights(3), host)
        assert np.array_equal(s.host_weights(3), host)
        fn.unload()


@pytest.mark.parametrize("pack", [True, False])
def test_packed_transfer_is_lossless_for_any_bits(pack, monkeypatch):
    """Weights cross the link in the packed format and are expanded on the device.  Doctored tensors
    (zeros, denormals, infinities, NaNs, exponents spread over 60 binades, one tensor of arbitrary
    bits, one of zeros only) must come back bit for bit, swap-in after swap-in, and a request must
    answer as it did at registration."""
    monkeypatch.delenv("TORPOR_PACK", raising=False)
    weights = resnet.init_weights("resnet50", seed=5)
    rng = np.random.default_rng(6)
    flat = weights["layer1.0.conv1.weight"].reshape(-1).view(np.uint32)
    flat[::97] = 0
    flat[1::101] = 0x00000001
    flat[2::103] = 0x7F800000
    flat[3::107] = 0x7FC00001
    flat[5::109] = 0xFF800000
    big = weights["layer2.0.conv2.weight"]
    weights["layer2.0.conv2.weight"] = rng.integers(0, 1 << 32, big.size, dtype=np.uint64).astype(np.uint32).view(np.float32).reshape(big.shape)
    weights["layer3.0.conv1.weight"][:] = 0
    w4 = weights["layer4.0.conv2.weight"]
    w4 *= np.exp(rng.uniform(-20, 20, w4.shape)).astype(np.float32)
    x = rng.standard_normal((1, 3, 64, 64)).astype(np.float32)
    with Server(mem_limit_bytes=1 << 30, pack=pack) as s:
        fn = resnet.ResNet(s, 2, "resnet50", batch=1, weights=weights, image=64)
        first = fn.register([x])
        host = s.host_weights(2).copy()
        image = s.model_info(2)["image_bytes"]
        assert np.array_equal(s.readback_weights(2), host)
        _assert_host_store_holds_the_upload(s, fn, host)
        st = s.pool_stats()
        # packed: the transfer image is the host store (the raw image was released after decoding back to it)
        slim = os.environ.get("TORPOR_SLIM_HOST", "1") != "0"      # the process-wide switch keeps the raw image too
        assert st["host_image_bytes"] == (0 if pack and slim else image)
        assert (0.82 * image < st["host_transfer_bytes"] < 0.91 * image) if pack else st["host_transfer_bytes"] == 0
        for _ in range(3):
            fn.unload()
            cold = fn.invoke([x])
            assert np.array_equal(first[0], cold[0], equal_nan=True)
            assert np.array_equal(s.readback_weights(2), host)
            sent = s.swap_stats(2)["bytes"]
            assert (0.82 * image < sent < 0.91 * image) if pack else sent == image
        fn.unload()


@pytest.mark.parametrize("image", [64, 320])
def test_requests_from_and_into_pinned_buffers_equal_requests_through_staging(gpu_server, image):
    """tp_host_alloc: an input that lies in such a buffer is read by the device where it is, a result whose
    destination lies in one is written by the device itself (by copy kernel while a swap-in runs and for small
    copies, by the copy engine otherwise: 64 x 64 images are below the size bound, 320 x 320 above); same
    bytes as the staged path, warm and cold, in every combination."""
    s = gpu_server
    fn, x, y = _mk(s, 7, seed=31, image=image)
    in_plain, out_plain, views_plain = fn.pack([x])
    in_pinned, out_pinned, views_pinned = fn.pack([x], pinned=True)
    assert np.array_equal(in_plain, in_pinned)
    for cold in (False, True, True, False):
        for packed in (in_pinned, in_plain):
            for out in (out_pinned, out_plain):
                if cold:
                    fn.unload()
                out[:] = 0
                assert s.signal(REQ_EXECUTE, 7, "")[0] == ACK_OK
                s.replay(7, packed, out)
            assert np.array_equal(views_plain[0], y) and np.array_equal(views_pinned[0], y)
    # the pinned input is read at request time, not captured earlier: a changed input changes the answer
    in_pinned[:] = fn.pack([x * np.float32(0.5)])[0]
    assert s.signal(REQ_EXECUTE, 7, "")[0] == ACK_OK
    s.replay(7, in_pinned, out_pinned)
    assert not np.array_equal(views_pinned[0], y)
    fn.unload()


class _Chain(Function):
    """y = x W^T applied `depth` times with one square weight: a long run of device work behind very
    few calls, so that the request's host side is over long before the device is."""

    def __init__(self, server, fid, seed, n=2048, depth=24):
        super().__init__(server, fid)
        self.n, self.depth, self.batch = n, depth, 1
        rng = np.random.default_rng(seed)
        self._w = (rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float32)

    def weights(self):
        return {"w": self._w}

    def input_specs(self):
        return [((self.n, self.n), np.float32)]

    def forward(self, inputs):
        n = self.n
        a, b = inputs[0], self.alloc(4 * n * n)
        for _ in range(self.depth):
            self.s.gemm(self.fid, a.va, self.w["w"], b.va, n, n, n, n, n, n)
            a, b = b, a
        return [(a, (n, n), np.float32)]


def test_memory_of_a_finished_request_is_not_reused_while_its_kernels_run():
    """A request is over for the controller once its result copy is queued (cuda_server.hpp:1044), which
    can be milliseconds before the device has run it.  The next request may evict that model at once;
    its weights, activations and result must stay intact until the device is done with them."""
    with Server(mem_limit_bytes=80 << 20, pool_bytes=256 << 20) as s:
        a, b = _Chain(s, 0, seed=1), _Chain(s, 1, seed=2)
        x = np.random.default_rng(3).standard_normal((a.n, a.n)).astype(np.float32)
        (ya,) = a.register([x])
        (yb,) = b.register([x])                      # the budget holds one model: this evicts 0
        assert not s.resident(0) and s.resident(1)
        assert np.abs(ya).max() > 0 and not np.array_equal(ya, yb)
        for _ in range(3):
            # request for model 0, issued op by op, left unsynchronised after the result copy
            assert s.signal(REQ_EXECUTE, 0, "") == (ACK_OK, 0, False)
            a._alloc_pos = 0
            buf = a.alloc(x.nbytes)
            s.h2d(0, buf.va, x)
            ((out, shape, dt),) = a.forward([buf])
            got_a = np.empty(shape, dt)
            s.d2h_async(0, got_a, out.va)
            # the executor is free again: model 1 is started at once, which evicts model 0
            assert s.signal(REQ_EXECUTE, 1, "") == (ACK_OK, 0, False)
            assert not s.resident(0) and s.resident(1)
            packed, outbuf, views = b.pack([x])
            s.replay(1, packed, outbuf)
            s.stream_synchronize(0)
            assert np.array_equal(got_a, ya), "model 0's result was damaged by the swap-in that followed it"
            assert np.array_equal(views[0], yb)
            assert np.array_equal(s.readback_weights(1), s.host_weights(1))


def test_executor_log_reports_every_swap_in(tmp_path, monkeypatch):
    """The Transfer line of the executor log (memory_manager.hpp:425-431) carries what tp_swap_stats reports."""
    import re
    monkeypatch.setenv("TORPOR_LOG_DIR", str(tmp_path))
    monkeypatch.setenv("EXECUTOR_LOG_LEVEL", "info")
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        fn, x, y = _mk(s, 0, seed=5)
        stats = []
        for _ in range(3):
            fn.unload()
            (got,) = fn.invoke([x])
            assert np.array_equal(got, y)
            stats.append(s.swap_stats(0))
        fn.unload()
    lines = (tmp_path / "log_executor_0.txt").read_text().splitlines()
    xfer = [re.search(r"Transfer model 0: (\d+) bytes over the link in (\d+) groups on (\d) streams, overall elasped (\d+) us", ln)
            for ln in lines if "Transfer model" in ln]
    assert len(xfer) == 3 and all(xfer)
    for m, st in zip(xfer, stats):
        assert int(m.group(1)) == st["bytes"] and int(m.group(2)) == st["chunks"] and int(m.group(3)) == st["copy_streams"]
        assert abs(int(m.group(4)) - st["copy_ms"] * 1e3) <= 2
    assert sum("Request of model 0 completed" in ln and "(swapped in)" in ln for ln in lines) == 3


def test_device_image_equals_host_image_wherever_it_lands():
    """Functions of different architectures take turns on the same pool memory: after every swap-in the
    device image equals the host image byte for byte, the alignment gaps between tensors included (they hold
    zeros in the host copy, and whatever the previous tenant left in the pool memory a swap-in lands in)."""
    from torpor_amd.functions import mobilenet
    with Server(mem_limit_bytes=260 << 20, pool_bytes=400 << 20) as s:
        rng = np.random.default_rng(3)
        a, xa, ya = _mk(s, 0, seed=1)
        cfg = dict(bert.CONFIGS["bert-base"], layers=2)
        b = bert.Bert(s, 1, "bert-base", batch=1, seq=32, seed=2, cfg=cfg, vocab=60000)   # 230 MB: the pair cannot both stay
        ids = rng.integers(0, 60000, (1, 32))
        yb = b.register([ids])
        c = mobilenet.MobileNetV2(s, 2, batch=1, weights=mobilenet.init_weights(seed=3))
        xc = rng.standard_normal((1, 3, 224, 224)).astype(np.float32)
        (yc,) = c.register([xc])
        # 0xFF everywhere the models do not write: activations of a poisoning function
        for turn in range(3):
            for fn, x, want in ((a, [xa], [ya]), (b, [ids], yb), (c, [xc], [yc])):
                got = fn.invoke(x)
                for g, w in zip(got, want):
                    assert np.array_equal(g, w)
                assert np.array_equal(s.readback_weights(fn.fid), s.host_weights(fn.fid)), (turn, fn.fid)
        assert s.pool_stats()["evictions"] >= 4


@pytest.mark.parametrize("trials", [0, 1, 2])
def test_copy_plan_settles_after_its_trial_requests_and_never_changes_an_answer(trials, monkeypatch):
    """The number of copy streams of a swap-in may follow the model's own cold requests (the first `trials`
    under the estimated plan, the next `trials` under the other one when the two estimates are close, then the
    better of the two for good).  Whatever it does, every cold answer has the registration run's bits, the
    weights land byte for byte, and the plan is the same for every swap-in after the trial requests."""
    monkeypatch.setenv("TORPOR_PLAN_TRIALS", str(trials))
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        fn, x, y = _mk(s, 5, seed=11, image=160)
        plans, groups = [], []
        for i in range(9):
            assert fn.unload()[0] == ACK_OK and not s.resident(5)
            (got,) = fn.invoke([x])
            assert np.array_equal(got, y), f"cold request {i} changed the answer"
            s.stream_synchronize(5)
            st = s.swap_stats(5)
            assert st["copy_streams"] in (1, 2) and st["chunks"] == s.model_info(5)["n_chunks"]
            plans.append(st["copy_streams"])
            groups.append(st["chunks"])
            assert np.array_equal(s.readback_weights(5), s.host_weights(5))
        settled = plans[2 * trials:]
        assert len(set(settled)) == 1, f"plan still changing after the trial requests: {plans}"
        if trials == 0:
            assert len(set(plans)) == 1 and len(set(groups)) == 1, "without trials the estimate alone decides"
