"""Python mirror of the server's two interfaces, over the C-ABI.

`Server.signal` is the control plane (SignalRequest -> SignalAck, reference
include/server/controller.hpp:131-216); the remaining methods are the data
plane a function container drives (reference include/server/cuda_server.hpp:301-455),
with the HIP-native op vocabulary of include/torpor_amd.h.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import TorporError

REQ_EXECUTE_AFTER_LOAD, REQ_EXECUTE, REQ_LOAD, REQ_UNLOAD = 0, 1, 2, 3
ACK_OK, ACK_INAVAIL = 0, 1
EUNSUPPORTED = -38   # TP_EUNSUPPORTED: shape / option not implemented (the caller takes another route)
ACT_NONE, ACT_RELU, ACT_GELU, ACT_TANH, ACT_RELU6, ACT_SILU, ACT_SIGMOID = 0, 1, 2, 3, 4, 5, 6
NCHW, NHWC = 0, 1
(OP_RELU, OP_ADD, OP_BIAS_ACT, OP_GELU, OP_MAXPOOL, OP_AVGPOOL, OP_LAYERNORM, OP_SOFTMAX, OP_EMBEDDING,
 OP_NCHW_TO_NHWC, OP_NHWC_TO_NCHW, OP_SUM, OP_FILL, OP_ATTENTION, OP_AVGPOOL2D, OP_COPY2D,
 OP_SCALE_CHANNELS, OP_BN_CONV1X1) = range(1, 19)
FLAG_HOST_ONLY = 1
FLAG_EVICT_LRU = 2   # plain LRU instead of the two-class policy (as env EVICT_POLICY=LRU)
FLAG_NO_PACK = 8   # weights cross the link as they are
FLAG_NO_HOST_GATHER = 4   # embedding lookups wait for their table instead of reading it from host memory
FLAG_KEEP_HOST_IMAGE = 16   # keep the raw weight image in pinned memory beside the packed transfer image
FLAG_POOL_FIXED = 32   # the reference's FixedSizeBlockManager policy for the HBM pool (as env BLOCK_MANAGER=Fixed)


def _chk(code, what):
    if code != 0:
        raise TorporError(code, what)


def _as_bytes_view(a):
    a = np.ascontiguousarray(a)
    return a, a.ctypes.data_as(C.c_void_p), a.nbytes


def gemm_noalloc(x, y, c, m, n, k, xs_r, ys_c, ldc, xs_k=1, ys_k=1, nb0=1, nb1=1, xb0=0, xb1=0, yb0=0, yb1=0,
                 cb0=0, cb1=0, stream=0, **ep):
    """tp_gemm_noalloc: the GEMM of Server.gemm on raw device addresses of the current HIP device, enqueued on
    `stream` (a hipStream_t as an integer, 0 = default stream); allocates nothing.  Returns the status code."""
    d = _lib.GemmDesc()
    d.x, d.y, d.c, d.m, d.n, d.k = x, y, c, m, n, k
    d.xs_r, d.xs_k, d.ys_c, d.ys_k, d.ldc = xs_r, xs_k, ys_c, ys_k, ldc
    d.nb0, d.nb1, d.xb0, d.xb1, d.yb0, d.yb1, d.cb0, d.cb1 = nb0, nb1, xb0, xb1, yb0, yb1, cb0, cb1
    Server._epilogue(d.ep, **ep)
    return _lib.lib().tp_gemm_noalloc(C.byref(d), C.c_void_p(stream))


class Server:
    def __init__(self, mem_limit_bytes=0, pool_bytes=0, chunk_bytes=0, chunk_max_bytes=0, workspace_bytes=0,
                 device=0, host_only=False, request_timeout_ms=0, copy_streams=0, evict_lru=False, host_gather=True, pack=True,
                 keep_host_image=False, pool_fixed=False):
        self._l = _lib.lib()
        cfg = _lib.Config()
        cfg.struct_size = C.sizeof(_lib.Config)
        cfg.device = device
        cfg.mem_limit_bytes = mem_limit_bytes
        cfg.pool_bytes = pool_bytes
        cfg.chunk_bytes = chunk_bytes
        cfg.chunk_max_bytes = chunk_max_bytes
        cfg.workspace_bytes = workspace_bytes
        cfg.flags = (FLAG_HOST_ONLY if host_only else 0) | (FLAG_EVICT_LRU if evict_lru else 0) | \
            (0 if host_gather else FLAG_NO_HOST_GATHER) | (0 if pack else FLAG_NO_PACK) | \
            (FLAG_KEEP_HOST_IMAGE if keep_host_image else 0) | (FLAG_POOL_FIXED if pool_fixed else 0)
        cfg.request_timeout_ms = request_timeout_ms
        cfg.copy_streams = copy_streams
        h = C.c_void_p()
        _chk(self._l.tp_server_create(C.byref(cfg), C.byref(h)), "tp_server_create")
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._l.tp_server_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---------------------------------------------------------------- control plane
    def signal(self, req_type, function, payload=""):
        """Returns (ack, resp, deferred)."""
        ack, resp, dfr = C.c_int32(), C.c_int32(), C.c_int32()
        _chk(self._l.tp_signal(self._h, req_type, str(function).encode(), str(payload).encode(),
                               C.byref(ack), C.byref(resp), C.byref(dfr)), "tp_signal")
        return ack.value, resp.value, bool(dfr.value)

    def take_deferred_ack(self):
        ack, resp = C.c_int32(), C.c_int32()
        r = self._l.tp_take_deferred_ack(self._h, C.byref(ack), C.byref(resp))
        if r < 0:
            raise TorporError(r, "tp_take_deferred_ack")
        return (ack.value, resp.value) if r == 1 else None

    def signal_ticket(self, req_type, function, payload=""):
        """Returns (ack, resp, deferred, ticket); ticket is 0 unless the signal was queued."""
        ack, resp, dfr, tk = C.c_int32(), C.c_int32(), C.c_int32(), C.c_uint64()
        _chk(self._l.tp_signal_ticket(self._h, req_type, str(function).encode(), str(payload).encode(),
                                      C.byref(ack), C.byref(resp), C.byref(dfr), C.byref(tk)), "tp_signal_ticket")
        return ack.value, resp.value, bool(dfr.value), tk.value

    def take_deferred_ack_ticket(self):
        ack, resp, tk = C.c_int32(), C.c_int32(), C.c_uint64()
        r = self._l.tp_take_deferred_ack_ticket(self._h, C.byref(ack), C.byref(resp), C.byref(tk))
        if r < 0:
            raise TorporError(r, "tp_take_deferred_ack_ticket")
        return (ack.value, resp.value, tk.value) if r == 1 else None

    def cancel_deferred(self, ticket):
        r = self._l.tp_cancel_deferred(self._h, int(ticket))
        if r < 0:
            raise TorporError(r, "tp_cancel_deferred")
        return r

    def check_address(self, fid, va, nbytes):
        return self._l.tp_check_address(self._h, fid, int(va), int(nbytes))

    def poll(self):
        r = self._l.tp_poll(self._h)
        if r < 0:
            raise TorporError(r, "tp_poll")
        return r == 1

    # ---------------------------------------------------------------- data plane
    def malloc(self, fid, nbytes):
        va = C.c_uint64()
        _chk(self._l.tp_malloc(self._h, fid, int(nbytes), C.byref(va)), "tp_malloc")
        return va.value

    def free(self, fid, va):
        _chk(self._l.tp_free(self._h, fid, va), "tp_free")

    def h2d(self, fid, dst_va, array):
        a, p, n = _as_bytes_view(array)
        _chk(self._l.tp_memcpy_h2d(self._h, fid, dst_va, p, n), "tp_memcpy_h2d")

    def d2h_async(self, fid, out_array, src_va):
        assert out_array.flags["C_CONTIGUOUS"]
        _chk(self._l.tp_memcpy_d2h_async(self._h, fid, out_array.ctypes.data_as(C.c_void_p), src_va,
                                         out_array.nbytes), "tp_memcpy_d2h_async")

    def d2h(self, fid, out_array, src_va):
        assert out_array.flags["C_CONTIGUOUS"]
        _chk(self._l.tp_memcpy_d2h(self._h, fid, out_array.ctypes.data_as(C.c_void_p), src_va,
                                   out_array.nbytes), "tp_memcpy_d2h")

    def d2d(self, fid, dst_va, src_va, nbytes):
        _chk(self._l.tp_memcpy_d2d(self._h, fid, dst_va, src_va, nbytes), "tp_memcpy_d2d")

    def memset(self, fid, dst_va, value, nbytes):
        _chk(self._l.tp_memset_async(self._h, fid, dst_va, value, nbytes), "tp_memset_async")

    def device_synchronize(self, fid):
        _chk(self._l.tp_device_synchronize(self._h, fid), "tp_device_synchronize")

    def stream_synchronize(self, fid):
        _chk(self._l.tp_stream_synchronize(self._h, fid), "tp_stream_synchronize")

    @staticmethod
    def _epilogue(ep, alpha=1.0, beta=0.0, bias=0, bn=None, bn_eps=1e-5, residual=0, ldr=0, act=ACT_NONE):
        ep.alpha, ep.beta, ep.bias = alpha, beta, bias
        if bn is not None:
            ep.bn_scale, ep.bn_bias, ep.bn_mean, ep.bn_var = bn
        ep.bn_eps, ep.residual, ep.ldr, ep.act = bn_eps, residual, ldr, act

    def gemm(self, fid, x, y, c, m, n, k, xs_r, ys_c, ldc, xs_k=1, ys_k=1, nb0=1, nb1=1,
             xb0=0, xb1=0, yb0=0, yb1=0, cb0=0, cb1=0, **ep):
        d = _lib.GemmDesc()
        d.x, d.y, d.c, d.m, d.n, d.k = x, y, c, m, n, k
        d.xs_r, d.xs_k, d.ys_c, d.ys_k, d.ldc = xs_r, xs_k, ys_c, ys_k, ldc
        d.nb0, d.nb1, d.xb0, d.xb1, d.yb0, d.yb1, d.cb0, d.cb1 = nb0, nb1, xb0, xb1, yb0, yb1, cb0, cb1
        self._epilogue(d.ep, **ep)
        _chk(self._l.tp_gemm(self._h, fid, C.byref(d)), "tp_gemm")

    def sgemm(self, fid, transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
        _chk(self._l.tp_sgemm(self._h, fid, transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc), "tp_sgemm")

    def sgemm_strided_batched(self, fid, transa, transb, m, n, k, alpha, a, lda, sa, b, ldb, sb, beta, c, ldc, sc,
                              count):
        _chk(self._l.tp_sgemm_strided_batched(self._h, fid, transa, transb, m, n, k, alpha, a, lda, sa, b, ldb, sb,
                                              beta, c, ldc, sc, count), "tp_sgemm_strided_batched")

    def conv(self, fid, x, w, y, n, h, w_in, cin, cout, kh, kw, stride=1, pad=0, x_layout=NHWC, y_layout=NHWC,
             groups=1, x_pitch=0, y_pitch=0, **ep):
        d = _lib.ConvDesc()
        d.x, d.w, d.y = x, w, y
        d.n, d.h, d.w_in, d.cin, d.cout, d.kh, d.kw = n, h, w_in, cin, cout, kh, kw
        sh, sw = (stride, stride) if isinstance(stride, int) else stride
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        d.stride_h, d.stride_w, d.pad_h, d.pad_w, d.groups = sh, sw, ph, pw, groups
        d.x_layout, d.y_layout = x_layout, y_layout
        d.x_pitch, d.y_pitch = x_pitch, y_pitch
        self._epilogue(d.ep, **ep)
        _chk(self._l.tp_conv_forward(self._h, fid, C.byref(d)), "tp_conv_forward")

    def bn(self, fid, x, y, scale, bias, mean, var, eps, rows, channels, hw=1, layout=NHWC, relu=False, x_pitch=0):
        _chk(self._l.tp_bn_inference_pitched(self._h, fid, x, y, scale, bias, mean, var, eps, rows, channels, hw,
                                             layout, int(relu), x_pitch), "tp_bn_inference")

    def launch(self, fid, op_id, ptrs, ints=(), floats=()):
        P = (C.c_uint64 * max(1, len(ptrs)))(*ptrs)
        I = (C.c_int64 * max(1, len(ints)))(*ints)
        F = (C.c_float * max(1, len(floats)))(*floats)
        _chk(self._l.tp_launch(self._h, fid, op_id, P, len(ptrs), I, len(ints), F, len(floats)), "tp_launch")

    def replay(self, fid, input_array, output_array):
        a, p, n = _as_bytes_view(input_array)
        assert output_array.flags["C_CONTIGUOUS"]
        _chk(self._l.tp_replay(self._h, fid, p, n, output_array.ctypes.data_as(C.c_void_p), output_array.nbytes),
             "tp_replay")

    # ---------------------------------------------------------------- introspection
    def resident(self, fid):
        r = self._l.tp_model_resident(self._h, fid)
        if r < 0:
            raise TorporError(r, "tp_model_resident")
        return bool(r)

    def loaded(self, fid):
        """True when the function is resident and its last swap-in has landed completely."""
        r = self._l.tp_model_loaded(self._h, fid)
        if r < 0:
            raise TorporError(r, "tp_model_loaded")
        return bool(r)

    def load_estimate(self, fid):
        """(ms the host link is busy before a request of the swapped-out function can complete, ms of its forward pass)."""
        a, b = C.c_double(), C.c_double()
        _chk(self._l.tp_get_load_estimate(self._h, fid, C.byref(a), C.byref(b)), "tp_get_load_estimate")
        return a.value, b.value

    def model_info(self, fid):
        o = _lib.ModelInfo()
        _chk(self._l.tp_get_model_info(self._h, fid, C.byref(o)), "tp_get_model_info")
        return {n: getattr(o, n) for n, _ in o._fields_}

    def pool_stats(self):
        o = _lib.PoolStats()
        _chk(self._l.tp_get_pool_stats(self._h, C.byref(o)), "tp_get_pool_stats")
        return {n: getattr(o, n) for n, _ in o._fields_}

    def swap_stats(self, fid):
        o = _lib.SwapStats()
        _chk(self._l.tp_get_swap_stats(self._h, fid, C.byref(o)), "tp_get_swap_stats")
        return {n: getattr(o, n) for n, _ in o._fields_}

    def readback_weights(self, fid):
        n = self.model_info(fid)["image_bytes"]
        out = np.empty(n, dtype=np.uint8)
        _chk(self._l.tp_readback_weights(self._h, fid, out.ctypes.data_as(C.c_void_p), n), "tp_readback_weights")
        return out

    def host_weights(self, fid):
        p, n = C.c_void_p(), C.c_uint64()
        _chk(self._l.tp_host_weights(self._h, fid, C.byref(p), C.byref(n)), "tp_host_weights")
        buf = (C.c_uint8 * n.value).from_address(p.value)
        return np.frombuffer(buf, dtype=np.uint8).copy()

    def weight_offset(self, fid, va):
        o = C.c_uint64()
        _chk(self._l.tp_weight_offset(self._h, fid, va, C.byref(o)), "tp_weight_offset")
        return o.value

    def last_kernel(self):
        return self._l.tp_last_kernel().decode()

    def host_empty(self, nbytes):
        """uint8 array over pinned host memory of the server: a request result whose destination lies
        in it is written by the device directly.  Valid until the server is closed."""
        p = C.c_void_p()
        _chk(self._l.tp_host_alloc(self._h, max(1, nbytes), C.byref(p)), "tp_host_alloc")
        buf = (C.c_uint8 * max(1, nbytes)).from_address(p.value)
        return np.frombuffer(buf, dtype=np.uint8, count=nbytes)

    def measure_h2d(self, nbytes=256 << 20, iters=10):
        g = C.c_double()
        _chk(self._l.tp_measure_h2d(self._h, nbytes, iters, C.byref(g)), "tp_measure_h2d")
        return g.value

    def profile_begin(self):
        _chk(self._l.tp_profile_begin(self._h), "tp_profile_begin")

    def profile_end(self):
        """Returns ({kernel: {launches, total_us, flops, bytes}}, empty_bracket_us)."""
        _chk(self._l.tp_profile_end(self._h), "tp_profile_end")
        out, empty, i = {}, 0.0, 0
        while True:
            st = _lib.KernelStat()
            r = self._l.tp_profile_read(self._h, i, C.byref(st))
            if r != 0:
                break
            i += 1
            name = st.name.decode()
            if name == "__empty_bracket__":
                empty = st.total_us
            else:
                out[name] = dict(launches=st.launches, total_us=st.total_us, flops=st.flops, bytes=st.bytes)
        return out, empty

    def time_op(self, fid, op_index=-1, iters=20):
        t = C.c_double()
        _chk(self._l.tp_time_op(self._h, fid, op_index, iters, C.byref(t)), "tp_time_op")
        return t.value
