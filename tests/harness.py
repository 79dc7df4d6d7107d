"""Op-level test session over the C-ABI: registers a scratch function, uploads "weights",
switches to the tracked mode and lets a test run any ops and read buffers back."""
import itertools

import numpy as np

from torpor_amd.server import ACK_OK, REQ_EXECUTE_AFTER_LOAD, REQ_UNLOAD

_fids = itertools.count(100)


class OpSession:
    def __init__(self, server, weights=()):
        self.s = server
        self.fid = next(_fids)
        ack, resp, deferred = server.signal(REQ_EXECUTE_AFTER_LOAD, self.fid, "1")
        assert ack == ACK_OK and not deferred
        self.w = []
        for a in weights:
            a = np.ascontiguousarray(a)
            va = server.malloc(self.fid, a.nbytes)
            server.h2d(self.fid, va, a)
            self.w.append(va)
        server.device_synchronize(self.fid)
        self._bufs = []

    def act(self, array):
        a = np.ascontiguousarray(array)
        va = self.s.malloc(self.fid, max(a.nbytes, 4))
        if a.nbytes:
            self.s.h2d(self.fid, va, a)
        return va

    def empty(self, nbytes):
        return self.s.malloc(self.fid, max(int(nbytes), 4))

    def read(self, va, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self.s.d2h(self.fid, out, va)
        return out

    def close(self):
        # finish the tracked request (the async D2H is the completion marker), then swap out
        dummy = np.empty(1, np.float32)
        va = self.s.malloc(self.fid, 4)
        self.s.launch(self.fid, 13, [va], [1], [0.0])
        self.s.d2h_async(self.fid, dummy, va)
        self.s.stream_synchronize(self.fid)
        self.s.signal(REQ_UNLOAD, self.fid, "")

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()


def assert_close(got, ref, rtol=1e-4, what=""):
    """max |got - ref| <= rtol * max(|ref|, tiny): the whole-tensor relative bound used for logits."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values"
    scale = max(float(np.abs(ref).max()), 1e-30)
    err = float(np.abs(got - ref).max()) / scale
    assert err <= rtol, f"{what}: rel err {err:.3e} > {rtol:.1e}"
    return err
