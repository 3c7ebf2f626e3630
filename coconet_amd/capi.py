"""ctypes binding of libcoconet_hip.so (include/coconet_hip.h).

Thin by design: every function below forwards device pointers and sizes to the C ABI and raises
CoconetError on a non-zero return code.  torch is used by callers only to own device memory and streams;
arguments here are raw addresses (ints), torch tensors (their data_ptr() is taken) or None.

There is no CPU fallback: if the shared library is missing, loading raises.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libcoconet_hip.so")

CCN_OK = 0
CCN_EINVAL = -22
CCN_ENOMEM = -12
CCN_ENODEV = -19
CCN_EHIP = -5
CCN_ERANGE = -34
CCN_MAX_RANKS = 16
LAMB_TRUST_RATIO = 0
LAMB_REFERENCE = 1
LAMB_NCCL_GLOBAL = 2

# every symbol include/coconet_hip.h declares
SYMBOLS = [
    "ccn_version", "ccn_init", "ccn_device_info", "ccn_malloc", "ccn_free", "ccn_memcpy_h2d", "ccn_memcpy_d2h",
    "ccn_memcpy_d2d", "ccn_fill_f32", "ccn_stream_create", "ccn_stream_destroy", "ccn_stream_sync",
    "ccn_event_create", "ccn_event_destroy", "ccn_event_record", "ccn_stream_wait_event", "ccn_event_elapsed_ms", "ccn_last_hip_error",
    "ccn_strerror", "ccn_reduce_f32", "ccn_sgd_f32", "ccn_sgd_axpby_f32", "ccn_pseudo_adam_f32", "ccn_adam_f32",
    "ccn_adam_f16g", "ccn_overflow_check_f16", "ccn_fused_adam_ref_f16g", "ccn_lamb_plan_create", "ccn_lamb_plan_create_parented",
    "ccn_lamb_plan_destroy", "ccn_lamb_f32", "ccn_lamb_plan_norms", "ccn_lamb_plan_tune", "ccn_mlp_outproj_bf16",
    "ccn_bias_dropout_residual", "ccn_graph_begin", "ccn_graph_end", "ccn_graph_launch", "ccn_graph_destroy",
    "ccn_scatter_plan_create", "ccn_scatter_plan_destroy", "ccn_sgd_f32_scattered", "ccn_adam_f32_scattered",
    "ccn_lamb_f32_scattered", "ccn_adam_bf16g", "ccn_lamb_nccl_f16g", "ccn_lamb_f32_static",
    "ccn_mlp_outproj_bf16_ex", "ccn_bias_dropout_residual_ex", "ccn_matmul_bf16_f32",
    "ccn_mlp_outproj_f16_ex", "ccn_bias_dropout_residual_f16_ex", "ccn_matmul_f16_f32",
    "ccn_matmul_bf16", "ccn_matmul_f16",
]


class CoconetError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__(f"{what}: error {code} ({strerror(code)})")


_lib = None


def load():
    """Load the library (once).  Raises OSError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is missing: run `python -m coconet_amd.build` (needs hipcc)")
        L = C.CDLL(LIB_PATH)
        _declare(L)
        _lib = L
    return _lib


_vp, _i, _f, _sz, _u64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint64
_pp = C.POINTER(C.c_void_p)


def _declare(L):
    def sig(name, args, res=_i):
        fn = getattr(L, name)
        fn.argtypes = args
        fn.restype = res

    sig("ccn_version", [])
    sig("ccn_init", [_i])
    sig("ccn_device_info", [C.POINTER(_i), C.POINTER(_sz), C.c_char_p, _sz])
    sig("ccn_malloc", [_pp, _sz])
    sig("ccn_free", [_vp])
    sig("ccn_memcpy_h2d", [_vp, _vp, _sz, _vp])
    sig("ccn_memcpy_d2h", [_vp, _vp, _sz, _vp])
    sig("ccn_memcpy_d2d", [_vp, _vp, _sz, _vp])
    sig("ccn_fill_f32", [_vp, _f, _sz, _vp])
    sig("ccn_stream_create", [_pp])
    sig("ccn_stream_destroy", [_vp])
    sig("ccn_stream_sync", [_vp])
    sig("ccn_event_create", [_pp])
    sig("ccn_event_destroy", [_vp])
    sig("ccn_event_record", [_vp, _vp])
    sig("ccn_stream_wait_event", [_vp, _vp])
    sig("ccn_event_elapsed_ms", [_vp, _vp, C.POINTER(_f)])
    sig("ccn_last_hip_error", [])
    sig("ccn_strerror", [_i], C.c_char_p)
    sig("ccn_reduce_f32", [_pp, _i, _vp, _sz, _vp])
    sig("ccn_sgd_f32", [_pp, _i, _vp, _sz, _f, _vp])
    sig("ccn_sgd_axpby_f32", [_pp, _i, _vp, _sz, _f, _f, _vp])
    sig("ccn_pseudo_adam_f32", [_pp, _i, _vp, _vp, _vp, _sz, _f, _f, _f, _vp])
    sig("ccn_adam_f32", [_pp, _i, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i, _vp])
    sig("ccn_adam_f16g", [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i, _f, _vp, _vp])
    sig("ccn_adam_bf16g", [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i, _f, _vp, _vp])
    sig("ccn_overflow_check_f16", [_pp, _i, _sz, _vp, _vp])
    sig("ccn_fused_adam_ref_f16g", [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f, _vp])
    sig("ccn_lamb_plan_create", [C.POINTER(_sz), _i, _pp])
    sig("ccn_lamb_plan_create_parented", [C.POINTER(_sz), C.POINTER(_sz), _i, _pp])
    sig("ccn_lamb_plan_destroy", [_vp])
    sig("ccn_lamb_f32", [_vp, _pp, _i, _vp, _vp, _vp, _f, _f, _f, _f, _f, _i, _i, _vp])
    sig("ccn_lamb_plan_norms", [_vp, _vp, _vp])
    sig("ccn_lamb_plan_tune", [_vp, _i, C.c_long])
    sig("ccn_lamb_f32_static", [_pp, _i, _vp, _vp, _vp, _sz, _sz, _f, _f, _f, _f, _f, _i, _i, _vp, _vp])
    sig("ccn_lamb_f32_scattered", [_vp, _pp, _i, _pp, _vp, _vp, _f, _f, _f, _f, _f, _i, _i, _vp])
    sig("ccn_lamb_nccl_f16g", [_vp, _pp, _i, _vp, _vp, _vp, _vp, _f, _f, _f, _f, _vp])
    sig("ccn_mlp_outproj_bf16", [_vp, _vp, _pp, _i, _vp, _vp, _vp, _i, _i, _i, _f, _u64, _vp])
    sig("ccn_bias_dropout_residual", [_vp, _pp, _i, _vp, _vp, _vp, _i, _i, _f, _u64, _vp])
    sig("ccn_mlp_outproj_bf16_ex", [_vp, _vp, _pp, _i, _vp, _vp, _vp, _i, _i, _i, _f, _u64, _i, _vp])
    sig("ccn_bias_dropout_residual_ex", [_vp, _pp, _i, _vp, _vp, _vp, _i, _i, _f, _u64, _i, _sz, _vp])
    sig("ccn_matmul_bf16_f32", [_vp, _vp, _vp, _i, _i, _i, _vp])
    sig("ccn_mlp_outproj_f16_ex", [_vp, _vp, _pp, _i, _vp, _vp, _vp, _i, _i, _i, _f, _u64, _i, _vp])
    sig("ccn_bias_dropout_residual_f16_ex", [_vp, _pp, _i, _vp, _vp, _vp, _i, _i, _f, _u64, _i, _sz, _vp])
    sig("ccn_matmul_f16_f32", [_vp, _vp, _vp, _i, _i, _i, _vp])
    sig("ccn_matmul_bf16", [_vp, _vp, _vp, _i, _i, _i, _vp])
    sig("ccn_matmul_f16", [_vp, _vp, _vp, _i, _i, _i, _vp])
    sig("ccn_scatter_plan_create", [C.POINTER(_sz), _i, _pp])
    sig("ccn_scatter_plan_destroy", [_vp])
    sig("ccn_sgd_f32_scattered", [_vp, _pp, _i, _pp, _f, _vp])
    sig("ccn_adam_f32_scattered", [_vp, _pp, _i, _pp, _vp, _vp, _f, _f, _f, _f, _i, _vp])
    sig("ccn_graph_begin", [_vp])
    sig("ccn_graph_end", [_vp, _pp])
    sig("ccn_graph_launch", [_vp, _vp])
    sig("ccn_graph_destroy", [_vp])


def strerror(code):
    return load().ccn_strerror(int(code)).decode()


def _check(rc, what):
    if rc != CCN_OK:
        raise CoconetError(rc, what)


def addr(x):
    """Device address of a torch tensor, or an int / None passed through."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def ptr_table(bufs):
    """Host array of device pointers (what the ABI calls `g` or `partials`)."""
    tbl = (C.c_void_p * max(len(bufs), 1))()
    for k, b in enumerate(bufs):
        tbl[k] = addr(b)
    return C.cast(tbl, _pp), tbl


def current_stream():
    """The HIP stream torch is currently issuing work on, as an address."""
    import torch
    return torch.cuda.current_stream().cuda_stream


# ---- runtime ---------------------------------------------------------------------------------------------------------
def version():
    return load().ccn_version()


def init(device=0):
    _check(load().ccn_init(device), "ccn_init")


def device_info():
    cu, hbm, arch = _i(0), _sz(0), C.create_string_buffer(64)
    _check(load().ccn_device_info(C.byref(cu), C.byref(hbm), arch, 64), "ccn_device_info")
    return {"cu_count": cu.value, "hbm_bytes": hbm.value, "arch": arch.value.decode()}


def malloc(nbytes):
    """ccn_malloc: device memory whose start is staggered against HBM channel conflicts.  Returns the address."""
    h = C.c_void_p()
    _check(load().ccn_malloc(C.byref(h), nbytes), "ccn_malloc")
    return h.value or 0


def free(address):
    _check(load().ccn_free(address), "ccn_free")


def memcpy_d2d(dst, src, nbytes, stream=None):
    _check(load().ccn_memcpy_d2d(addr(dst), addr(src), nbytes, stream), "ccn_memcpy_d2d")


def memcpy_h2d(dst, src_host, nbytes, stream=None):
    _check(load().ccn_memcpy_h2d(addr(dst), src_host, nbytes, stream), "ccn_memcpy_h2d")


def memcpy_d2h(dst_host, src, nbytes, stream=None):
    _check(load().ccn_memcpy_d2h(dst_host, addr(src), nbytes, stream), "ccn_memcpy_d2h")


def fill_f32(dst, value, n, stream=None):
    _check(load().ccn_fill_f32(addr(dst), value, n, stream), "ccn_fill_f32")


class Event:
    def __init__(self):
        h = C.c_void_p()
        _check(load().ccn_event_create(C.byref(h)), "ccn_event_create")
        self.h = h

    def record(self, stream=None):
        _check(load().ccn_event_record(self.h, stream.h if isinstance(stream, Stream) else stream), "ccn_event_record")

    def close(self):
        if self.h:
            _check(load().ccn_event_destroy(self.h), "ccn_event_destroy")
            self.h = None

    def elapsed_ms(self, stop):
        ms = _f(0)
        _check(load().ccn_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "ccn_event_elapsed_ms")
        return ms.value

    def __del__(self):
        try:
            if self.h:
                load().ccn_event_destroy(self.h)
        except Exception:
            pass


class ScatterPlan:
    """Tile table for nbuff separate gradient / weight buffers of the given element counts (ccn_scatter_plan)."""

    def __init__(self, counts):
        self.counts = [int(c) for c in counts]
        arr = (_sz * len(self.counts))(*self.counts)
        h = C.c_void_p()
        _check(load().ccn_scatter_plan_create(arr, len(self.counts), C.byref(h)), "ccn_scatter_plan_create")
        self.h = h

    def _tables(self, g, w):
        """g: P lists of nbuff buffers; w: nbuff buffers."""
        nb = len(self.counts)
        assert len(w) == nb and all(len(gp) == nb for gp in g)
        gt = (C.c_void_p * (len(g) * nb))(*[addr(x) for gp in g for x in gp])
        wt = (C.c_void_p * nb)(*[addr(x) for x in w])
        return gt, wt

    def sgd(self, g, w, lr, stream=None):
        gt, wt = self._tables(g, w)
        _check(load().ccn_sgd_f32_scattered(self.h, gt, len(g), wt, lr, stream), "ccn_sgd_f32_scattered")

    def adam(self, g, w, m, v, lr, beta1, beta2, eps, step, stream=None):
        gt, wt = self._tables(g, w)
        _check(load().ccn_adam_f32_scattered(self.h, gt, len(g), wt, addr(m), addr(v), lr, beta1, beta2, eps, step, stream),
               "ccn_adam_f32_scattered")

    def close(self):
        if self.h:
            _check(load().ccn_scatter_plan_destroy(self.h), "ccn_scatter_plan_destroy")
            self.h = None


class Stream:
    """A stream of the library's own (ccn_stream_create); pass `.h` wherever a stream is taken."""

    def __init__(self):
        h = C.c_void_p()
        _check(load().ccn_stream_create(C.byref(h)), "ccn_stream_create")
        self.h = h

    def sync(self):
        _check(load().ccn_stream_sync(self.h), "ccn_stream_sync")

    def wait_event(self, event):
        _check(load().ccn_stream_wait_event(self.h, event.h), "ccn_stream_wait_event")

    def close(self):
        if self.h:
            _check(load().ccn_stream_destroy(self.h), "ccn_stream_destroy")
            self.h = None


class Graph:
    """Records the update calls made on `stream` inside the with-block; launch() replays them."""

    def __init__(self, stream):
        self.stream, self.h = stream, None

    def __enter__(self):
        _check(load().ccn_graph_begin(self.stream.h), "ccn_graph_begin")
        return self

    def __exit__(self, exc_type, exc, tb):
        h = C.c_void_p()
        rc = load().ccn_graph_end(self.stream.h, C.byref(h))
        if exc_type is None:
            _check(rc, "ccn_graph_end")
            self.h = h
        return False

    def launch(self, stream=None):
        _check(load().ccn_graph_launch(self.h, (stream or self.stream).h), "ccn_graph_launch")

    def close(self):
        if self.h:
            _check(load().ccn_graph_destroy(self.h), "ccn_graph_destroy")
            self.h = None


# ---- hot path --------------------------------------------------------------------------------------------------------
def reduce_f32(g, out, n, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_reduce_f32(p, len(g), addr(out), n, stream), "ccn_reduce_f32")


def sgd_f32(g, w, n, lr, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_sgd_f32(p, len(g), addr(w), n, lr, stream), "ccn_sgd_f32")


def sgd_axpby_f32(g, w, n, alpha, beta, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_sgd_axpby_f32(p, len(g), addr(w), n, alpha, beta, stream), "ccn_sgd_axpby_f32")


def pseudo_adam_f32(g, w, m, v, n, lr, beta1, beta2, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_pseudo_adam_f32(p, len(g), addr(w), addr(m), addr(v), n, lr, beta1, beta2, stream),
           "ccn_pseudo_adam_f32")


def adam_f32(g, w, m, v, n, lr, beta1, beta2, eps, step, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_adam_f32(p, len(g), addr(w), addr(m), addr(v), n, lr, beta1, beta2, eps, step, stream),
           "ccn_adam_f32")


def adam_f16g(g, w, m, v, w16, n, lr, beta1, beta2, eps, step, inv_scale, overflow_flag, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_adam_f16g(p, len(g), addr(w), addr(m), addr(v), addr(w16), n, lr, beta1, beta2, eps, step,
                                inv_scale, addr(overflow_flag), stream), "ccn_adam_f16g")


def adam_bf16g(g, w, m, v, w16, n, lr, beta1, beta2, eps, step, inv_scale, overflow_flag, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_adam_bf16g(p, len(g), addr(w), addr(m), addr(v), addr(w16), n, lr, beta1, beta2, eps, step,
                                 inv_scale, addr(overflow_flag), stream), "ccn_adam_bf16g")


def overflow_check_f16(g, n, overflow_flag, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_overflow_check_f16(p, len(g), n, addr(overflow_flag), stream), "ccn_overflow_check_f16")


def fused_adam_ref_f16g(g, w, halfw, m, v, n, lr, beta1, beta2, stream=None):
    p, _keep = ptr_table(g)
    _check(load().ccn_fused_adam_ref_f16g(p, len(g), addr(w), addr(halfw), addr(m), addr(v), n, lr, beta1, beta2,
                                          stream), "ccn_fused_adam_ref_f16g")


LAMB_KNOB_SPIN_LIMIT, LAMB_KNOB_TWO_PASS, LAMB_KNOB_WITHHOLD = 0, 1, 2
# knobs every new LambPlan is tuned with ({knob: value}): how the tests run whole files under another kernel path
LAMB_DEFAULT_KNOBS = {}


class LambPlan:
    """Device-side segment tables for one segmentation of [0, N) (ccn_lamb_plan)."""

    def __init__(self, seg_offsets, buf_sizes=None, buf_parent=None, knobs=None):
        """seg_offsets: nseg+1 element offsets, one buffer per segment.  Or buf_sizes / buf_parent (seg_offsets None):
        segments made of several buffers each, buffer i belonging to segment buf_parent[i].
        knobs: {LAMB_KNOB_*: value} passed to ccn_lamb_plan_tune (default: LAMB_DEFAULT_KNOBS)."""
        h = C.c_void_p()
        if buf_sizes is not None:
            sizes, parent = [int(x) for x in buf_sizes], [int(x) for x in buf_parent]
            assert len(sizes) == len(parent)
            self.nbuf = len(sizes)
            self.nseg = parent[-1] + 1 if parent else 0
            _check(load().ccn_lamb_plan_create_parented((_sz * len(sizes))(*sizes), (_sz * len(parent))(*parent), self.nbuf,
                                                        C.byref(h)), "ccn_lamb_plan_create_parented")
        else:
            offs = [int(x) for x in seg_offsets]
            self.nseg = self.nbuf = len(offs) - 1
            arr = (_sz * len(offs))(*offs)
            _check(load().ccn_lamb_plan_create(arr, self.nseg, C.byref(h)), "ccn_lamb_plan_create")
        self.h = h
        for knob, value in (LAMB_DEFAULT_KNOBS if knobs is None else knobs).items():
            self.tune(knob, value)

    def tune(self, knob, value):
        _check(load().ccn_lamb_plan_tune(self.h, knob, value), "ccn_lamb_plan_tune")

    def step(self, g, w, m, v, lr, beta1, beta2, eps, wd, step, mode=LAMB_TRUST_RATIO, stream=None):
        p, _keep = ptr_table(g)
        _check(load().ccn_lamb_f32(self.h, p, len(g), addr(w), addr(m), addr(v), lr, beta1, beta2, eps, wd, step, mode,
                                   stream), "ccn_lamb_f32")

    def step_scattered(self, g, w, m, v, lr, beta1, beta2, eps, wd, step, mode=LAMB_TRUST_RATIO, stream=None):
        """g: P lists of nbuf buffers; w: nbuf buffers (one per buffer of the plan); m, v: single arrays."""
        assert len(w) == self.nbuf and all(len(gp) == self.nbuf for gp in g)
        gt = (C.c_void_p * (len(g) * self.nbuf))(*[addr(x) for gp in g for x in gp])
        wt = (C.c_void_p * self.nbuf)(*[addr(x) for x in w])
        _check(load().ccn_lamb_f32_scattered(self.h, gt, len(g), wt, addr(m), addr(v), lr, beta1, beta2, eps, wd, step, mode,
                                             stream), "ccn_lamb_f32_scattered")

    def step_nccl_f16g(self, g, w, halfw, m, v, lr, beta1, beta2, wd, stream=None):
        """The modified NCCL's mixed-precision LAMB: g are fp16 bit patterns, halfw receives fp16(w)."""
        p, _keep = ptr_table(g)
        _check(load().ccn_lamb_nccl_f16g(self.h, p, len(g), addr(w), addr(halfw), addr(m), addr(v), lr, beta1, beta2, wd,
                                         stream), "ccn_lamb_nccl_f16g")

    def norms(self, stream=None):
        import numpy as np
        out = np.empty((self.nseg, 2), np.float64)
        _check(load().ccn_lamb_plan_norms(self.h, out.ctypes.data_as(C.c_void_p), stream), "ccn_lamb_plan_norms")
        return out

    def close(self):
        if self.h:
            _check(load().ccn_lamb_plan_destroy(self.h), "ccn_lamb_plan_destroy")
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


LAMB_STATIC_MAX_N = 1 << 28
LAMB_STATIC_MAX_SEGS = 4096


def lamb_f32_static(g, w, m, v, n, seg_len, lr, beta1, beta2, eps, wd, step, mode=LAMB_TRUST_RATIO, norms=None, stream=None):
    """ccn_lamb_f32_static: the two-pass LAMB step on uniform segments, scratch in the library's static device array."""
    p, _keep = ptr_table(g)
    _check(load().ccn_lamb_f32_static(p, len(g), addr(w), addr(m), addr(v), n, seg_len, lr, beta1, beta2, eps, wd, step,
                                      mode, addr(norms), stream), "ccn_lamb_f32_static")


DROPOUT_INVERTED, DROPOUT_REF_DSL, DROPOUT_REF_NCCL, DROPOUT_REF_NCCL_SAT = 0, 1, 2, 3


def mlp_outproj_bf16(X, W, partials, bias, resid, out, M, N, K, p_drop, seed, stream=None, dropout_mode=None, half=False):
    """half=True: X, W, resid and out are IEEE half instead of bfloat16 (ccn_mlp_outproj_f16_ex)."""
    p, _keep = ptr_table(partials)
    if half:
        _check(load().ccn_mlp_outproj_f16_ex(addr(X), addr(W), p, len(partials), addr(bias), addr(resid), addr(out), M, N,
                                             K, p_drop, seed, dropout_mode or 0, stream), "ccn_mlp_outproj_f16_ex")
    elif dropout_mode is None:
        _check(load().ccn_mlp_outproj_bf16(addr(X), addr(W), p, len(partials), addr(bias), addr(resid), addr(out), M, N, K,
                                           p_drop, seed, stream), "ccn_mlp_outproj_bf16")
    else:
        _check(load().ccn_mlp_outproj_bf16_ex(addr(X), addr(W), p, len(partials), addr(bias), addr(resid), addr(out), M, N,
                                              K, p_drop, seed, dropout_mode, stream), "ccn_mlp_outproj_bf16_ex")


def bias_dropout_residual(acc, partials, bias, resid, out, M, N, p_drop, seed, stream=None, dropout_mode=None, first_row=0,
                          half=False):
    p, _keep = ptr_table(partials)
    if half:
        _check(load().ccn_bias_dropout_residual_f16_ex(addr(acc), p, len(partials), addr(bias), addr(resid), addr(out), M, N,
                                                       p_drop, seed, dropout_mode or 0, first_row, stream),
               "ccn_bias_dropout_residual_f16_ex")
    elif dropout_mode is None and first_row == 0:
        _check(load().ccn_bias_dropout_residual(addr(acc), p, len(partials), addr(bias), addr(resid), addr(out), M, N,
                                                p_drop, seed, stream), "ccn_bias_dropout_residual")
    else:
        _check(load().ccn_bias_dropout_residual_ex(addr(acc), p, len(partials), addr(bias), addr(resid), addr(out), M, N,
                                                   p_drop, seed, dropout_mode or 0, first_row, stream),
               "ccn_bias_dropout_residual_ex")


def matmul_bf16_f32(X, W, Cmat, M, N, K, stream=None, half=False):
    if half:
        _check(load().ccn_matmul_f16_f32(addr(X), addr(W), addr(Cmat), M, N, K, stream), "ccn_matmul_f16_f32")
    else:
        _check(load().ccn_matmul_bf16_f32(addr(X), addr(W), addr(Cmat), M, N, K, stream), "ccn_matmul_bf16_f32")


def matmul_16(X, W, Cmat, M, N, K, stream=None, half=False):
    """The product alone with C in the operands' 16-bit type (ccn_matmul_bf16 / ccn_matmul_f16)."""
    if half:
        _check(load().ccn_matmul_f16(addr(X), addr(W), addr(Cmat), M, N, K, stream), "ccn_matmul_f16")
    else:
        _check(load().ccn_matmul_bf16(addr(X), addr(W), addr(Cmat), M, N, K, stream), "ccn_matmul_bf16")
