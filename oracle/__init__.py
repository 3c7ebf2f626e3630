"""ctypes binding of the CPU oracle (oracle/ccn_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg
of bench.py as the checker.  The product package (coconet_amd) never imports this module.

All array arguments are numpy arrays; state arrays (w, m, v) are updated in place.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_pp = C.POINTER(C.c_void_p)
_f = C.c_float
_sz = C.c_size_t
_vp = C.c_void_p
_i = C.c_int


def _declare(L):
    L.orc_f32_to_f16.restype = C.c_uint16
    L.orc_f32_to_f16.argtypes = [_f]
    L.orc_f16_to_f32.restype = _f
    L.orc_f16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_f32_to_bf16.argtypes = [_f]
    L.orc_bf16_to_f32.restype = _f
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    for n in ("orc_f32_to_f16_array", "orc_f16_to_f32_array", "orc_f32_to_bf16_array", "orc_bf16_to_f32_array"):
        getattr(L, n).restype = None
        getattr(L, n).argtypes = [_vp, _vp, _sz]
    L.orc_eqFloat_1e3.restype = _i
    L.orc_eqFloat_1e3.argtypes = [_f, _f]
    L.orc_eq_float_1e5.restype = _i
    L.orc_eq_float_1e5.argtypes = [_f, _f]
    L.orc_reduce_f32.restype = None
    L.orc_reduce_f32.argtypes = [_pp, _i, _sz, _vp]
    L.orc_sgd_f32.restype = None
    L.orc_sgd_f32.argtypes = [_pp, _i, _vp, _sz, _f]
    L.orc_sgd_axpby_f32.restype = None
    L.orc_sgd_axpby_f32.argtypes = [_pp, _i, _vp, _sz, _f, _f]
    L.orc_pseudo_adam_f32.restype = None
    L.orc_pseudo_adam_f32.argtypes = [_pp, _i, _vp, _vp, _vp, _sz, _f, _f, _f]
    L.orc_fused_adam_a3.restype = None
    L.orc_fused_adam_a3.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f]
    L.orc_adam_f32.restype = None
    L.orc_adam_f32.argtypes = [_pp, _i, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i]
    L.orc_adam_f16g.restype = C.c_uint32
    L.orc_adam_f16g.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i, _f]
    L.orc_adam_bf16g.restype = C.c_uint32
    L.orc_adam_bf16g.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, _sz, _f, _f, _f, _f, _i, _f]
    L.orc_overflow_f16.restype = C.c_uint32
    L.orc_overflow_f16.argtypes = [_pp, _i, _sz]
    L.orc_lamb_nccl_f16g.restype = None
    L.orc_lamb_nccl_f16g.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, _vp, _i, _f, _f, _f, _f, _vp]
    L.orc_lamb_f32.restype = None
    L.orc_lamb_f32.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, _i, _f, _f, _f, _f, _f, _i, _i, _vp]
    L.orc_philox4x32_10.restype = None
    L.orc_philox4x32_10.argtypes = [_vp, _vp, _vp]
    L.orc_dropout_keep.restype = _i
    L.orc_dropout_keep.argtypes = [C.c_uint64, C.c_uint64, _f]
    L.orc_dropout_mask.restype = None
    L.orc_dropout_mask.argtypes = [C.c_uint64, C.c_uint64, _sz, _f, _vp]
    L.orc_mlp_outproj.restype = None
    L.orc_mlp_outproj.argtypes = [_vp, _vp, _pp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, C.c_uint64]
    L.orc_mlp_outproj_mode.restype = None
    L.orc_mlp_outproj_mode.argtypes = [_vp, _vp, _pp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, C.c_uint64, _i]
    L.orc_mlp_outproj_typed.restype = None
    L.orc_mlp_outproj_typed.argtypes = [_vp, _vp, _pp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, C.c_uint64, _i, _i]
    L.orc_dsl_lamb_f32.restype = None
    L.orc_dsl_lamb_f32.argtypes = [_pp, _i, _vp, _vp, _vp, _vp, C.c_size_t, _f, _f, _f, _f, _f, _f, _i, _f, _vp]
    L.orc_mlp_outproj_rows.restype = None
    L.orc_mlp_outproj_rows.argtypes = [_vp, _vp, _pp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _f, C.c_uint64, _i, _i, _vp]
    L.orc_epilogue_value.restype = _f
    L.orc_epilogue_value.argtypes = [_f, _f, _f, _i, _f, _i]
    L.orc_epilogue_value_typed.restype = _f
    L.orc_epilogue_value_typed.argtypes = [_f, _f, _f, _i, _f, _i, _i]


def set_num_threads(n):
    """Host threads for the oracle's element-, segment- and row-parallel loops (1 = as the reference runs its checker)."""
    lib().orc_set_num_threads(int(n))


def _ptr(a, dtype):
    assert isinstance(a, np.ndarray) and a.dtype == dtype and a.flags["C_CONTIGUOUS"], (a.dtype, dtype)
    return a.ctypes.data_as(C.c_void_p)


def _ptrs(arrs, dtype):
    """Host table of P pointers."""
    tbl = (C.c_void_p * len(arrs))()
    for k, a in enumerate(arrs):
        tbl[k] = _ptr(a, dtype).value
    return C.cast(tbl, _pp), tbl


f32 = np.dtype(np.float32)
u16 = np.dtype(np.uint16)


# ---- conversions ---------------------------------------------------------------------------------
def f32_to_f16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_f16_array(_ptr(a, f32), _ptr(out, u16), a.size)
    return out


def f16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_f16_to_f32_array(_ptr(a, u16), _ptr(out, f32), a.size)
    return out


def f32_to_bf16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_bf16_array(_ptr(a, f32), _ptr(out, u16), a.size)
    return out


def bf16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_bf16_to_f32_array(_ptr(a, u16), _ptr(out, f32), a.size)
    return out


def eqFloat(u, v):
    """examples/header.h eqFloat (rel 1e-3)."""
    return bool(lib().orc_eqFloat_1e3(float(u), float(v)))


def eq_float(u, v):
    """nccl-overlap/samples/multi-process-adam-scattered.cpp eq_float (rel 1e-5)."""
    return bool(lib().orc_eq_float_1e5(float(u), float(v)))


# ---- optimizers ----------------------------------------------------------------------------------
def reduce_f32(g):
    out = np.empty_like(g[0])
    p, _k = _ptrs(g, f32)
    lib().orc_reduce_f32(p, len(g), g[0].size, _ptr(out, f32))
    return out


def sgd_f32(g, w, lr):
    p, _k = _ptrs(g, f32)
    lib().orc_sgd_f32(p, len(g), _ptr(w, f32), w.size, lr)


def sgd_axpby_f32(g, w, alpha, beta):
    p, _k = _ptrs(g, f32)
    lib().orc_sgd_axpby_f32(p, len(g), _ptr(w, f32), w.size, alpha, beta)


def pseudo_adam_f32(g, w, m, v, lr, beta1, beta2):
    p, _k = _ptrs(g, f32)
    lib().orc_pseudo_adam_f32(p, len(g), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), w.size, lr, beta1, beta2)


def dsl_lamb_f32(g, w, m, v, lr, beta1, beta2, gamma, c1=None, c2=None, eps=None):
    """The DSL example's LAMB (examples/lamb/lamb.cpp:20-28): m, v updated in place; returns (new weights, (rNorm, wNorm)).
    c1, c2 default to the example's fp32 (1 - beta); eps=None leaves the square root alone as the example does."""
    one = np.float32(1)
    c1 = np.float32(one - np.float32(beta1)) if c1 is None else np.float32(c1)
    c2 = np.float32(one - np.float32(beta2)) if c2 is None else np.float32(c2)
    p, _k = _ptrs(g, f32)
    out = np.empty_like(w)
    norms = np.empty(2, np.float32)
    lib().orc_dsl_lamb_f32(p, len(g), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), _ptr(out, f32), w.size, lr, beta1, beta2,
                           float(c1), float(c2), 0.0 if eps is None else eps, 0 if eps is None else 1, gamma, _ptr(norms, f32))
    return out, norms


def fused_adam_a3(g16, w, m, v, halfw, lr, beta1, beta2):
    p, _k = _ptrs(g16, u16)
    lib().orc_fused_adam_a3(p, len(g16), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), _ptr(halfw, u16), w.size,
                            lr, beta1, beta2)


def adam_f32(g, w, m, v, lr, beta1, beta2, eps, step):
    p, _k = _ptrs(g, f32)
    lib().orc_adam_f32(p, len(g), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), w.size, lr, beta1, beta2, eps, step)


def adam_f16g(g16, w, m, v, w16, lr, beta1, beta2, eps, step, inv_scale):
    p, _k = _ptrs(g16, u16)
    return int(lib().orc_adam_f16g(p, len(g16), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), _ptr(w16, u16), w.size,
                                   lr, beta1, beta2, eps, step, inv_scale))


def adam_bf16g(g16, w, m, v, w16, lr, beta1, beta2, eps, step, inv_scale):
    p, _k = _ptrs(g16, u16)
    return int(lib().orc_adam_bf16g(p, len(g16), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), _ptr(w16, u16), w.size,
                                    lr, beta1, beta2, eps, step, inv_scale))


def overflow_f16(g16):
    p, _k = _ptrs(g16, u16)
    return int(lib().orc_overflow_f16(p, len(g16), g16[0].size))


def lamb_f32(g, w, m, v, seg_offsets, lr, beta1, beta2, eps, wd, step, mode=0):
    """Returns norms (nseg, 2): [W_b, R_b]."""
    p, _k = _ptrs(g, f32)
    so = np.ascontiguousarray(seg_offsets, dtype=np.uint64)
    nseg = so.size - 1
    assert so[-1] == w.size and so[0] == 0
    norms = np.zeros((nseg, 2), np.float64)
    lib().orc_lamb_f32(p, len(g), _ptr(w, f32), _ptr(m, f32), _ptr(v, f32), so.ctypes.data_as(C.c_void_p), nseg,
                       lr, beta1, beta2, eps, wd, step, mode, norms.ctypes.data_as(C.c_void_p))
    return norms


def lamb_nccl_f16g(g16, w, halfw, m, v, seg_offsets, lr, beta1, beta2, wd):
    """The modified NCCL's mixed-precision LAMB (fp16 gradients, fp16 weight copy).  Returns norms (nseg, 2)."""
    p, _k = _ptrs(g16, u16)
    so = np.ascontiguousarray(seg_offsets, dtype=np.uint64)
    nseg = so.size - 1
    assert so[-1] == w.size and so[0] == 0
    norms = np.zeros((nseg, 2), np.float64)
    lib().orc_lamb_nccl_f16g(p, len(g16), _ptr(w, f32), _ptr(halfw, u16), _ptr(m, f32), _ptr(v, f32),
                             so.ctypes.data_as(C.c_void_p), nseg, lr, beta1, beta2, wd,
                             norms.ctypes.data_as(C.c_void_p))
    return norms


# ---- RNG / dropout / GEMM epilogue ------------------------------------------------------------------
def philox4x32_10(ctr, key):
    c = np.ascontiguousarray(ctr, dtype=np.uint32)
    k = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.empty(4, np.uint32)
    lib().orc_philox4x32_10(c.ctypes.data_as(C.c_void_p), k.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    return out


def dropout_mask(seed, first_idx, n, p_drop):
    keep = np.empty(n, np.uint8)
    lib().orc_dropout_mask(seed, first_idx, n, p_drop, keep.ctypes.data_as(C.c_void_p))
    return keep


def epilogue_value(s, b, r, kept_inverted, p_drop, mode, half=False):
    """One output element of the epilogue under dropout form `mode`; kept_inverted is the draw's u >= p.
    half=True: IEEE-half operands (only the saturating form then differs: it rounds to half after each add)."""
    if half:
        return float(lib().orc_epilogue_value_typed(s, b, r, int(kept_inverted), p_drop, mode, 1))
    return float(lib().orc_epilogue_value(s, b, r, int(kept_inverted), p_drop, mode))


def mlp_outproj(X, W, partials, bias, resid, M, N, K, p_drop, seed, mode=0, half=False, row_ids=None):
    """X, W, resid: uint16 bit patterns, bfloat16 or (half=True) IEEE half. Returns (out_bits, out_f32).
    mode: dropout form, 0 = standard.  row_ids: the M rows handed in are these rows of a larger output (the dropout
    draw of an element depends on its index in the whole output)."""
    out = np.empty((M, N), np.uint16)
    outf = np.empty((M, N), np.float32)
    if partials:
        p, _k = _ptrs(partials, f32)
    else:
        p, _k = C.cast(None, _pp), None
    ids = None
    if row_ids is not None:
        ids = np.ascontiguousarray(row_ids, dtype=np.int64)
        assert ids.shape == (M,)
    lib().orc_mlp_outproj_rows(_ptr(X, u16), _ptr(W, u16), p, len(partials), _ptr(bias, f32),
                               _ptr(resid, u16) if resid is not None else None, _ptr(out, u16), _ptr(outf, f32),
                               M, N, K, p_drop, seed, mode, 1 if half else 0,
                               ids.ctypes.data_as(C.c_void_p) if ids is not None else None)
    return out, outf
