"""The pool at the size of the part: one arena as large as the device grants (MI355X: 288 GB of HBM3E),
a function placed above the 128 GiB mark of it, answers against the PyTorch CPU forward and swapped
weights byte-identical up there (pooled allocation of the whole device: block_manager.hpp:260-418,
memory_manager.hpp:38-53)."""
import numpy as np
import pytest
import torch

from oracle import models as om
from tests.harness import assert_close
from torpor_amd._lib import TorporError
from torpor_amd.functions import resnet
from torpor_amd.server import ACK_OK, OP_FILL, REQ_EXECUTE_AFTER_LOAD, Server

pytestmark = pytest.mark.gpu
GIB = 1 << 30


def _ballast(s, fid, act_bytes):
    """A function whose activation arena is `act_bytes`: it pins that much of the pool below whatever is
    placed next.  Only the first KiB is ever touched."""
    assert s.signal(REQ_EXECUTE_AFTER_LOAD, fid, "2")[:2] == (ACK_OK, 0)
    w = s.malloc(fid, 1024)
    s.h2d(fid, w, np.zeros(256, np.float32))
    s.device_synchronize(fid)
    a = s.malloc(fid, act_bytes)
    s.launch(fid, OP_FILL, [a], [256], [1.5])
    out = np.empty(256, np.float32)
    s.d2h_async(fid, out, a)
    s.stream_synchronize(fid)
    assert (out == 1.5).all()


def test_a_function_above_128_gib_of_a_whole_device_arena():
    server = None
    for arena_gib in (256, 248, 240, 224, 208, 200):
        try:
            server = Server(mem_limit_bytes=(arena_gib - 2) * GIB, pool_bytes=arena_gib * GIB)
            break
        except TorporError as e:
            print(f"arena of {arena_gib} GiB refused: {e}", flush=True)
    assert server is not None, "the device granted no arena of 200 GiB or more"
    with server as s:
        st = s.pool_stats()
        assert st["capacity"] >= 200 * GIB
        print(f"arena {st['capacity'] / GIB:.0f} GiB", flush=True)
        _ballast(s, 0, 130 * GIB)
        assert s.model_info(0)["act_bytes"] >= 130 * GIB
        weights = resnet.init_weights("resnet50", seed=4)
        x = torch.randn(2, 3, 224, 224, generator=torch.Generator().manual_seed(5)).numpy()
        fn = resnet.ResNet(s, 1, "resnet50", batch=2, weights=weights)
        (first,) = fn.register([x])
        model = om.load_numpy_state(om.ResNet("resnet50"), weights)
        with torch.no_grad():
            want = model(torch.from_numpy(x)).numpy()
        assert_close(first, want, 1e-3, "logits above 128 GiB")
        for turn in range(3):     # swapped out and back in: it lands above the ballast every time
            fn.unload()
            (cold,) = fn.invoke([x])
            assert np.array_equal(cold, first)
            info = s.model_info(1)
            assert info["weight_off"] >= 128 * GIB and info["act_off"] >= 128 * GIB, info
            assert np.array_equal(s.readback_weights(1), s.host_weights(1))
        st = s.pool_stats()
        assert st["used"] >= 130 * GIB and st["lru_models"] == 2 and st["fragmentation_evictions"] == 0
        # a second tenant up there, then the first one again: placement stays deterministic
        fn2 = resnet.ResNet(s, 2, "resnet50", batch=1, seed=6)
        x2 = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(7)).numpy()
        (y2,) = fn2.register([x2])
        assert s.model_info(2)["weight_off"] > s.model_info(1)["weight_off"]
        (again,) = fn.invoke([x])
        assert np.array_equal(again, first)
        (y2b,) = fn2.invoke([x2])
        assert np.array_equal(y2b, y2)
