"""A served function: what runs inside the reference's function container
(tests/endpoint.py: build the model, move it to the GPU, answer each request with one
forward pass), driving the server through its request flow instead of through an
intercepted CUDA runtime.

Life cycle (reference scripts/router.py:381-394 `launch`, 306-313 `Execute`):
  register(): ExecuteAfterLoad signal -> one alloc + upload per weight tensor -> device
              synchronise -> one warm-up inference, which the server tracks to learn the
              weight access order and to record the op stream
  invoke():   Execute signal -> ops (or one replay call) -> outputs
  unload():   Unload signal
"""
from collections import OrderedDict

import numpy as np

from ..server import ACK_OK, REQ_EXECUTE, REQ_EXECUTE_AFTER_LOAD, REQ_LOAD, REQ_UNLOAD, Server


class Buf:
    """An activation allocation on the server."""
    __slots__ = ("va", "nbytes")

    def __init__(self, va, nbytes):
        self.va, self.nbytes = va, nbytes


class Function:
    def __init__(self, server: Server, fid: int, level: int = 1):
        self.s = server
        self.fid = int(fid)
        self.level = level
        self.w = OrderedDict()  # weight name -> virtual address
        self._alloc_log = []    # activation allocations of the first run, in order
        self._alloc_pos = None  # None while recording, else cursor into _alloc_log
        self.registered = False
        self.out_specs = None   # [(shape, dtype)] of the outputs, set by the first run

    # -- to be provided by the model ------------------------------------------------
    def weights(self):
        """OrderedDict name -> np.ndarray, in upload order."""
        raise NotImplementedError

    def forward(self, inputs):
        """Emit the ops of one inference; `inputs` are device buffers.  Returns
        [(Buf, shape, dtype)] for the outputs."""
        raise NotImplementedError

    def input_specs(self):
        """[(shape, dtype)] of the request inputs."""
        raise NotImplementedError

    # -- activation buffers -------------------------------------------------------------
    def alloc(self, nbytes):
        nbytes = int(nbytes)
        if self._alloc_pos is None:
            b = Buf(self.s.malloc(self.fid, nbytes), nbytes)
            self._alloc_log.append(b)
            return b
        b = self._alloc_log[self._alloc_pos]
        self._alloc_pos += 1
        # a request with fewer rows than the registered batch re-uses the recorded buffers
        assert b.nbytes >= nbytes, "allocation sequence differs from the recorded run"
        return b

    def release(self, buf):
        if self._alloc_pos is None:
            self.s.free(self.fid, buf.va)

    # -- request flow ---------------------------------------------------------------------
    def _run(self, inputs):
        specs = self.input_specs()
        assert len(inputs) == len(specs)
        if self._alloc_pos is not None:
            self._alloc_pos = 0
        dev_in = []
        for a, (shape, dtype) in zip(inputs, specs):
            a = np.ascontiguousarray(a, dtype=dtype)
            assert tuple(a.shape) == tuple(shape), (a.shape, shape)
            b = self.alloc(a.nbytes)
            self.s.h2d(self.fid, b.va, a)
            dev_in.append(b)
        outs = self.forward(dev_in)
        host = [np.empty(shape, dtype=dtype) for (_, shape, dtype) in outs]
        self.out_specs = [(shape, dtype) for (_, shape, dtype) in outs]
        for h, (b, _, _) in zip(host, outs):
            self.s.d2h_async(self.fid, h, b.va)
        self.s.stream_synchronize(self.fid)
        if self._alloc_pos is None:
            self._alloc_pos = 0
        return self.postprocess(host)

    def postprocess(self, host):
        """Turn the raw output buffers of a request into the model's outputs."""
        return host

    def register(self, example_inputs):
        ack, resp, deferred = self.s.signal(REQ_EXECUTE_AFTER_LOAD, self.fid, str(self.level))
        if ack != ACK_OK or deferred:
            raise RuntimeError(f"register {self.fid}: ack={ack} deferred={deferred}")
        for name, arr in self.weights().items():
            arr = np.ascontiguousarray(arr)
            va = self.s.malloc(self.fid, arr.nbytes)
            self.s.h2d(self.fid, va, arr)
            self.w[name] = va
        self.s.device_synchronize(self.fid)
        out = self._run(example_inputs)
        self.registered = True
        return out

    def invoke(self, inputs, replay=True):
        ack, resp, deferred = self.s.signal(REQ_EXECUTE, self.fid, "")
        if ack != ACK_OK or deferred:
            raise RuntimeError(f"execute {self.fid}: ack={ack} deferred={deferred}")
        if not replay:
            return self._run(inputs)
        packed, outbuf, views = self.pack(inputs)
        self.s.replay(self.fid, packed, outbuf)
        return self.postprocess(views)

    def invoke_rows(self, inputs, rows):
        """One request with `rows` <= the registered batch, at the cost of `rows`: the reference's
        function container runs the model at the batch the router hands it (tests/endpoint.py:84-92).
        The recorded op stream is for the registered batch, so a smaller one is issued op by op,
        in the activation buffers of the registered run."""
        if rows == self.batch:
            return self.invoke(inputs)
        if not 0 < rows < self.batch:
            raise ValueError(f"rows must be in 1..{self.batch}")
        ack, resp, deferred = self.s.signal(REQ_EXECUTE, self.fid, "")
        if ack != ACK_OK or deferred:
            raise RuntimeError(f"execute {self.fid}: ack={ack} deferred={deferred}")
        saved = (self.batch, self.out_specs)
        self.batch = rows
        try:
            return self._run(inputs)
        finally:
            self.batch, self.out_specs = saved

    def pack(self, inputs, pinned=False):
        """Request inputs as one byte string and one output buffer with per-output views,
        in the order the recorded H2D / D2H copies consume them.  `pinned`: both buffers are pinned
        memory of the server (the device reads the inputs and writes the results in place, without a
        staging copy on either side; they live as long as the server)."""
        specs = self.input_specs()
        parts = [np.ascontiguousarray(a, dtype=dt).reshape(-1).view(np.uint8) for a, (_, dt) in zip(inputs, specs)]
        packed = np.concatenate(parts) if len(parts) > 1 else parts[0]
        if pinned:
            staged = self.s.host_empty(packed.size)
            staged[:] = packed
            packed = staged
        sizes = [int(np.prod(shape)) * np.dtype(dt).itemsize for shape, dt in self.out_specs]
        outbuf = self.s.host_empty(sum(sizes)) if pinned else np.empty(sum(sizes), dtype=np.uint8)
        views, pos = [], 0
        for (shape, dt), n in zip(self.out_specs, sizes):
            views.append(outbuf[pos:pos + n].view(dt).reshape(shape))
            pos += n
        return packed, outbuf, views

    def load(self):
        return self.s.signal(REQ_LOAD, self.fid, "")

    def unload(self):
        return self.s.signal(REQ_UNLOAD, self.fid, "")
