"""Pins the CPU oracle (oracle/ccn_oracle.c) before anything is compared against it.

Each routine is checked against evidence that does not come from the oracle itself: the reference's own
fixtures and known answers, closed forms, library routines (numpy / torch on the CPU) and float64 brute
force.  None of these tests needs a GPU.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from util import REF_BUFF_SIZES_TAIL, grads_f32, ref_integer_pattern, rel_err, rng, weights_f32


# ---------------------------------------------------------------------------------------------------------------------
# conversions
# ---------------------------------------------------------------------------------------------------------------------
def test_f16_exhaustive_decode_and_roundtrip():
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    got = orc.f16_to_f32(allh)
    finite_or_inf = ~np.isnan(ref)
    assert np.array_equal(got.view(np.uint32)[finite_or_inf], ref.view(np.uint32)[finite_or_inf])
    assert np.all(np.isnan(got[~finite_or_inf]))
    assert np.array_equal(orc.f32_to_f16(got)[finite_or_inf], allh[finite_or_inf])


def test_f32_to_f16_rne_against_numpy():
    r = rng(1)
    x = (r.standard_normal(1 << 20) * np.exp(r.uniform(-20, 12, 1 << 20))).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f32_to_f16(x), x.astype(np.float16).view(np.uint16))
    # every tie between two neighbouring halfs, both signs
    h = np.arange(0, 0x7bff, dtype=np.uint16)
    mid = ((orc.f16_to_f32(h).astype(np.float64) + orc.f16_to_f32(h + 1).astype(np.float64)) / 2).astype(np.float32)
    for s in (1.0, -1.0):
        m = (mid * np.float32(s)).astype(np.float32)
        assert np.array_equal(orc.f32_to_f16(m), m.astype(np.float16).view(np.uint16))
    special = np.array([np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -25, 2.0 ** -24, 0.0, -0.0], np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f32_to_f16(special), special.astype(np.float16).view(np.uint16))
    assert (orc.f32_to_f16(np.array([np.nan], np.float32))[0] & 0x7c00) == 0x7c00


def test_bf16_against_torch():
    r = rng(2)
    x = (r.standard_normal(1 << 20) * np.exp(r.uniform(-30, 30, 1 << 20))).astype(np.float32)
    t = torch.from_numpy(x).to(torch.bfloat16)
    assert np.array_equal(orc.f32_to_bf16(x).view(np.int16), t.view(torch.int16).numpy())
    allb = np.arange(65536, dtype=np.uint16)
    back = torch.from_numpy(allb.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    got = orc.bf16_to_f32(allb)
    ok = ~np.isnan(back)
    assert np.array_equal(got.view(np.uint32)[ok], back.view(np.uint32)[ok])


# ---------------------------------------------------------------------------------------------------------------------
# comparators of the reference
# ---------------------------------------------------------------------------------------------------------------------
def test_reference_comparators():
    assert orc.eqFloat(1.0, 1.0005) and not orc.eqFloat(1.0, 1.002)
    assert orc.eqFloat(0.0, 0.0) and not orc.eqFloat(0.0, 1e-9)
    assert orc.eq_float(1.0, 1.000005) and not orc.eq_float(1.0, 1.00002)
    assert orc.eq_float(0.0, 0.0)


# ---------------------------------------------------------------------------------------------------------------------
# reduce / SGD
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("P", [1, 2, 4, 8, 16])
def test_reduce_integers_exact_and_order(P):
    N = 1000
    g = [np.full(N, p + 1, np.float32) for p in range(P)]
    assert np.array_equal(orc.reduce_f32(g), np.full(N, P * (P + 1) / 2, np.float32))
    # order: ascending p, one fp32 rounding per add.  1 + 2^-24 + 2^-24 is 1 when added left to right in
    # fp32 (each 2^-24 is a tie that rounds to even), but 1 + 2^-23 if the small terms were paired first.
    if P >= 3:
        g = [np.zeros(4, np.float32) for _ in range(P)]
        g[0][:] = 1.0
        g[1][:] = 2.0 ** -24
        g[2][:] = 2.0 ** -24
        assert np.all(orc.reduce_f32(g) == np.float32(1.0))
    gr = grads_f32(3, P, N, 1e-2)
    seq = gr[0].copy()
    for p in range(1, P):
        seq = seq + gr[p]
    assert np.array_equal(orc.reduce_f32(gr), seq)
    # permutation bound: any order agrees within P ulps of sum |g|
    rev = orc.reduce_f32(gr[::-1])
    bound = P * np.finfo(np.float32).eps * np.sum(np.abs(np.stack(gr)), axis=0)
    assert np.all(np.abs(rev - seq) <= bound)


def test_sgd_closed_form_and_axpy():
    P, N = 4, 64
    g = [np.full(N, p + 1, np.float32) for p in range(P)]           # sum = 10
    w = np.full(N, 8.0, np.float32)
    orc.sgd_f32(g, w, 0.5)
    assert np.all(w == 3.0)
    gr = grads_f32(4, P, 1 << 12, 1e-2)
    w0 = weights_f32(4, 1 << 12, 0.1)
    w = w0.copy()
    orc.sgd_f32(gr, w, np.float32(0.01))
    s = ((gr[0] + gr[1]) + gr[2]) + gr[3]
    assert np.array_equal(w, w0 - np.float32(0.01) * s)
    # independent library cross-check in float64
    ref = w0.astype(np.float64) - 0.01 * np.sum(np.stack(gr).astype(np.float64), axis=0)
    assert rel_err(w, ref) < 1e-6
    w = w0.copy()
    orc.sgd_axpby_f32(gr, w, np.float32(0.75), np.float32(-0.01))
    assert np.array_equal(w, np.float32(0.75) * w0 + np.float32(-0.01) * s)


# ---------------------------------------------------------------------------------------------------------------------
# the DSL example's pseudo-Adam and the modified NCCL's fused kernel: known answers held by the reference
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("P", [1, 2, 4, 8, 16])
def test_pseudo_adam_known_answer(P):
    # examples/test-adam.cu:73-88: g = 1, w = m = v = 0, lr = 1, beta1 = beta2 = 0.5  =>  w = -1/P
    N = 257
    g = [np.ones(N, np.float32) for _ in range(P)]
    w, m, v = (np.zeros(N, np.float32) for _ in range(3))
    orc.pseudo_adam_f32(g, w, m, v, 1.0, 0.5, 0.5)
    assert np.all(w == np.float32(-1.0 / P))
    assert np.all(m == np.float32(P / 2)) and np.all(v == np.float32(P * P / 2))


@pytest.mark.parametrize("P", [2, 4, 8])
def test_fused_adam_a3_known_answer(P):
    # nccl/src/collectives/device/common_kernel.h:658-660: same inputs => w == -1.0, fp16 copy == 0xBC00
    N = 129
    g = [np.full(N, 0x3C00, np.uint16) for _ in range(P)]       # 1.0 in fp16
    w, m, v = (np.zeros(N, np.float32) for _ in range(3))
    hw = np.zeros(N, np.uint16)
    orc.fused_adam_a3(g, w, m, v, hw, 1.0, 0.5, 0.5)
    assert np.all(w == -1.0) and np.all(hw == 0xBC00)


def test_fused_adam_a3_first_moment_decays_with_beta2():
    """The kernel runs its first-moment functor through `.mixedbinOp1(beta2, mval, ...)`
    (nccl/src/collectives/device/common_kernel.h:878): m decays with beta2, and only the division S3 = m/beta1 (:879)
    sees beta1.  With beta1 != beta2 the two readings differ; values by hand, one rank, g = 1, w = m = v = 0, lr = 1,
    beta1 = 1/2, beta2 = 1/4 (every intermediate is exact in binary):
      step 1: v = 3/4, S4 = v/beta2 = 3;  m = (1 - beta2) = 3/4 (1 - beta1 would give 1/2);  S3 = m/beta1 = 3/2;
              w = -(3/2)/sqrt(3)
      step 2: m = 3/4 * 1/4 + 3/4 = 15/16 (beta1 would give 3/4), v = 15/16, S4 = 15/4, S3 = 15/8;
              w -= (15/8)/sqrt(15/4)"""
    g = [np.array([0x3C00], np.uint16)]
    w, m, v = (np.zeros(1, np.float32) for _ in range(3))
    hw = np.zeros(1, np.uint16)
    f = np.float32
    orc.fused_adam_a3(g, w, m, v, hw, 1.0, 0.5, 0.25)
    assert m[0] == f(0.75) and v[0] == f(0.75)
    w1 = f(0) - f(1.5) / np.sqrt(f(3.0))
    assert w[0] == w1
    orc.fused_adam_a3(g, w, m, v, hw, 1.0, 0.5, 0.25)
    assert m[0] == f(15 / 16) and v[0] == f(15 / 16)
    assert w[0] == w1 - f(15 / 8) / np.sqrt(f(15 / 4))
    assert hw[0] == np.float16(w[0]).view(np.uint16)


def test_fused_adam_a3_half_precision_effects():
    # the sum is carried in fp16: 2048 + 1 is not representable in half (spacing 2), so the second rank's
    # gradient is lost; an fp32 sum would give 2049.  The square is also rounded to half: 3.001^2.
    g = [np.array([0x6800], np.uint16), np.array([0x3C00], np.uint16)]      # 2048, 1
    w, m, v = (np.zeros(1, np.float32) for _ in range(3))
    hw = np.zeros(1, np.uint16)
    orc.fused_adam_a3(g, w, m, v, hw, 1.0, 0.5, 0.5)
    assert m[0] == np.float32(2048 * 0.5)                    # (1-beta2) * fp16 sum; 2049 would give 1024.5
    g = [np.array([0x4201], np.uint16)]                      # 3.001953125
    w[:] = 0; m[:] = 0; v[:] = 0
    orc.fused_adam_a3(g, w, m, v, hw, 1.0, 0.5, 0.5)
    x = np.float16(3.001953125)
    assert v[0] == np.float32(np.float16(x * x)) * np.float32(0.5)


# ---------------------------------------------------------------------------------------------------------------------
# bias-corrected Adam
# ---------------------------------------------------------------------------------------------------------------------
def test_adam_step1_closed_form():
    # m = v = 0 and one rank: mhat = c, vhat = c^2, update = lr*c/(|c|+eps), whatever the betas are
    N = 4096
    c = grads_f32(5, 1, N, 1e-3)
    for b1, b2 in [(0.9, 0.999), (0.5, 0.5), (0.0, 0.99)]:
        w0 = weights_f32(5, N, 0.05)
        w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
        orc.adam_f32(c, w, m, v, 1e-3, b1, b2, 1e-6, 1)
        cd = c[0].astype(np.float64)
        upd = 1e-3 * cd / (np.abs(cd) + 1e-6)
        assert rel_err(w0.astype(np.float64) - w.astype(np.float64), upd) < 5e-4   # w-w0 cancels ~13 bits
        assert np.max(np.abs(w.astype(np.float64) - (w0.astype(np.float64) - upd))) < 4e-9   # one ulp of |w| <= 0.05
        omb1, omb2 = float(np.float32(1) - np.float32(b1)), float(np.float32(1) - np.float32(b2))   # fp32 betas
        assert rel_err(m, omb1 * cd) < 1e-6 and rel_err(v, omb2 * cd * cd) < 1e-6


def test_adam_against_torch_optim():
    # textbook Adam from a library (torch.optim.Adam on the CPU), 10 steps of benchmark configuration 2 at small N
    P, N = 8, 1 << 14
    w0 = weights_f32(6, N, 0.05)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    tw = torch.nn.Parameter(torch.from_numpy(w0.astype(np.float64)))
    f32 = lambda x: float(np.float32(x))      # the library sees the same fp32-rounded hyper-parameters
    opt = torch.optim.Adam([tw], lr=f32(1e-3), betas=(f32(0.9), f32(0.999)), eps=f32(1e-6))
    for t in range(1, 11):
        g = grads_f32(6, P, N, 1e-3, step=t)
        orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
        tw.grad = torch.from_numpy(orc.reduce_f32(g).astype(np.float64))   # the reduce is pinned separately
        opt.step()
    st = opt.state[tw]
    # torch adds eps to sqrt(v)/sqrt(1-b2^t) exactly as the checker adds it to sqrt(vhat); float64 vs fp32 state
    tw_np = tw.detach().numpy()
    assert np.max(np.abs(w - tw_np)) < 1e-6 * np.max(np.abs(tw_np))
    big = np.abs(tw_np) > 1e-3                      # relative error where w is not itself near zero
    assert rel_err(w[big], tw_np[big]) < 1e-5
    d, dref = w - w0.astype(np.float64), tw_np - w0           # the accumulated update itself
    assert np.max(np.abs(d - dref)) < 1e-5 * np.max(np.abs(dref))
    assert np.max(np.abs(m - st["exp_avg"].numpy())) < 1e-6 * np.max(np.abs(m))
    assert np.max(np.abs(v - st["exp_avg_sq"].numpy())) < 1e-6 * np.max(np.abs(v))


@pytest.mark.parametrize("P", [1, 2, 4])
def test_adam_reference_integer_fixture(P):
    # the reference's fixture: every rank holds g = w0 = (i%2+1)*(index%20+1), beta = .5, alpha = +1 (lr = -1),
    # eps 1e-6, 5 checked steps.  With a constant gradient G = P*g: mhat = G, vhat = G^2, so every step adds
    # alpha*G/(G+eps) = 1 - eps/(G+eps).
    for buff in (0, 1):
        n = 2048
        g0 = ref_integer_pattern(buff, n)
        w, m, v = g0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
        G = P * g0.astype(np.float64)
        for t in range(1, 6):
            orc.adam_f32([g0] * P, w, m, v, -1.0, 0.5, 0.5, 1e-6, t)
            expect = g0.astype(np.float64) + t * (1.0 - 1e-6 / (G + 1e-6))
            assert rel_err(w, expect) < 1e-6
            assert rel_err(m, (1 - 0.5 ** t) * G) < 1e-6
            assert rel_err(v, (1 - 0.5 ** t) * G * G) < 1e-6


# ---------------------------------------------------------------------------------------------------------------------
# LAMB
# ---------------------------------------------------------------------------------------------------------------------
def lamb_float64(g, w, m, v, seg_offsets, lr, b1, b2, eps, wd, step, mode):
    """Independent float64 restatement of LAMB with RMS-normalised per-segment norms (numpy, vectorised).
    Hyper-parameters are first rounded to fp32, as the fp32 routine receives them."""
    lr, b1, b2, eps, wd = (float(np.float32(x)) for x in (lr, b1, b2, eps, wd))
    gs = np.sum(np.stack(g).astype(np.float64), axis=0)
    m = b1 * m.astype(np.float64) + (1 - b1) * gs
    v = b2 * v.astype(np.float64) + (1 - b2) * gs * gs
    mh, vh = m / (1 - b1 ** step), v / (1 - b2 ** step)
    w = w.astype(np.float64)
    r = mh / (np.sqrt(vh) + eps) + wd * w
    out = w.copy()
    norms = []
    for b in range(len(seg_offsets) - 1):
        lo, hi = seg_offsets[b], seg_offsets[b + 1]
        W = np.sqrt(np.mean(w[lo:hi] ** 2))
        R = np.sqrt(np.mean(r[lo:hi] ** 2))
        ratio = (W / R if R > 0 else 1.0) if W > 0 else 1.0
        scale = ratio / R if mode == 1 else ratio
        out[lo:hi] = w[lo:hi] - lr * scale * r[lo:hi]
        norms.append((W, R))
    return out, m, v, np.array(norms)


@pytest.mark.parametrize("mode", [0, 1])
def test_lamb_float64_brute_force(mode):
    P = 4
    segs = [0, 5, 1029, 1030, 4096, 10000]
    N = segs[-1]
    g = grads_f32(7, P, N, 1e-3)
    w0 = weights_f32(7, N, 0.05)
    m0 = (rng(7, 50).standard_normal(N) * 1e-3).astype(np.float32)
    v0 = (rng(7, 51).uniform(0, 1e-5, N)).astype(np.float32)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    norms = orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 3, mode)
    ew, em, ev, en = lamb_float64(g, w0, m0, v0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 3, mode)
    assert rel_err(norms, en) < 1e-6
    assert np.max(np.abs(w - ew)) < 1e-6 * np.max(np.abs(ew))
    assert np.max(np.abs(m - em)) < 1e-6 * np.max(np.abs(em)) and np.max(np.abs(v - ev)) < 1e-6 * np.max(np.abs(ev))
    # the update itself (w - w0), not only w: a wrong scale would hide behind w's magnitude otherwise
    d, dref = w.astype(np.float64) - w0, ew - w0
    assert np.max(np.abs(d - dref)) < 1e-3 * np.max(np.abs(dref))     # fp32 rounding of w is ~2e-4 of a step here


def test_lamb_special_cases():
    P, n = 2, 3000
    g = grads_f32(8, P, n, 1e-3)
    # w == 0: W = 0 => ratio 1; trust-ratio mode steps by lr*r, reference mode by lr*r/R
    for mode in (0, 1):
        w, m, v = (np.zeros(n, np.float32) for _ in range(3))
        norms = orc.lamb_f32(g, w, m, v, [0, n], 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, mode)
        gs = (g[0] + g[1]).astype(np.float64)
        r = gs / (np.abs(gs) + 1e-6)          # step 1, m = v = 0: mhat/(sqrt(vhat)+eps) = gs/(|gs|+eps)
        R = np.sqrt(np.mean(r * r))
        assert norms[0, 0] == 0.0 and abs(norms[0, 1] - R) < 1e-6 * R
        expect = -1e-3 * r / (R if mode == 1 else 1.0)
        assert rel_err(w, expect) < 1e-5
    # segments are independent: a 3-segment call equals three 1-segment calls
    segs = [0, 1000, 1001, n]
    w0 = weights_f32(8, n, 0.05)
    w, m, v = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0)
    for b in range(3):
        lo, hi = segs[b], segs[b + 1]
        ws, ms, vs = w0[lo:hi].copy(), np.zeros(hi - lo, np.float32), np.zeros(hi - lo, np.float32)
        orc.lamb_f32([x[lo:hi].copy() for x in g], ws, ms, vs, [0, hi - lo], 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0)
        assert np.array_equal(ws, w[lo:hi]) and np.array_equal(ms, m[lo:hi])


def test_lamb_reference_integer_fixture():
    # reference fixture (multi-process-adam-scattered.cpp:221-226 and the tail of its buffer list): constant
    # gradient G per element, so step 1 gives r = G/(G+eps) + w with w = g; reference mode (second /R kept).
    P = 2
    sizes = REF_BUFF_SIZES_TAIL
    segs = np.concatenate([[0], np.cumsum(sizes)])
    g0 = np.concatenate([ref_integer_pattern(i, n) for i, n in enumerate(sizes)])
    w, m, v = g0.copy(), np.zeros_like(g0), np.zeros_like(g0)
    orc.lamb_f32([g0] * P, w, m, v, segs, 1.0, 0.5, 0.5, 1e-6, 1.0, 1, 1)
    G = P * g0.astype(np.float64)
    r = G / (G + 1e-6) + g0
    for b in range(len(sizes)):
        lo, hi = segs[b], segs[b + 1]
        W, R = np.sqrt(np.mean(g0[lo:hi].astype(np.float64) ** 2)), np.sqrt(np.mean(r[lo:hi] ** 2))
        expect = g0[lo:hi] - (W / R / R) * r[lo:hi]
        assert np.max(np.abs(w[lo:hi] - expect)) < 1e-5 * np.max(np.abs(g0[lo:hi]))


# ---------------------------------------------------------------------------------------------------------------------
# mixed-precision Adam with overflow flag (build-defined semantics, pinned by reduction to orc_adam_f32)
# ---------------------------------------------------------------------------------------------------------------------
def test_adam_f16g_reduces_to_adam_and_flags():
    P, N = 8, 1 << 13
    scale = 2.0 ** 16
    g32 = grads_f32(9, P, N, 1e-3)
    g16 = [orc.f32_to_f16(x * np.float32(scale)) for x in g32]
    w0 = weights_f32(9, N, 0.05)
    # no overflow: equals fp32 Adam on the decoded, unscaled gradients, bit for bit; flag 0
    w, m, v, w16 = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    flag = orc.adam_f16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(1 / scale))
    dec = [orc.f16_to_f32(x) * np.float32(1 / scale) for x in g16]
    wr, mr, vr = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    orc.adam_f32(dec, wr, mr, vr, 1e-3, 0.9, 0.999, 1e-6, 1)
    assert flag == 0 and orc.overflow_f16(g16) == 0
    assert np.array_equal(w, wr) and np.array_equal(m, mr) and np.array_equal(v, vr)
    assert np.array_equal(w16, w.astype(np.float16).view(np.uint16))
    # plant +inf, -inf and a nan in different ranks: flag 1, exactly those elements keep their state
    bad = {17: (0, 0x7C00), 4096: (3, 0xFC00), N - 1: (7, 0x7E01)}
    for i, (p, bits) in bad.items():
        g16[p][i] = bits
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    flag = orc.adam_f16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(1 / scale))
    assert flag == 1 and orc.overflow_f16(g16) == 1
    keep = np.ones(N, bool)
    keep[list(bad)] = False
    assert np.array_equal(w[keep], wr[keep]) and np.array_equal(m[keep], mr[keep])
    assert np.array_equal(w[~keep], w0[~keep]) and np.all(m[~keep] == 0) and np.all(v[~keep] == 0)
    assert np.array_equal(w16, w.astype(np.float16).view(np.uint16))
    assert np.all(np.isfinite(w)) and np.all(np.isfinite(m)) and np.all(np.isfinite(v))
    # the largest finite half (exponent 0x1E) is not an overflow
    g16[0][5] = 0x7BFF
    for i, (p, bits) in bad.items():
        g16[p][i] = 0
    assert orc.overflow_f16(g16) == 0


# ---------------------------------------------------------------------------------------------------------------------
# Philox, dropout mask, GEMM epilogue
# ---------------------------------------------------------------------------------------------------------------------
def test_philox_known_answers():
    # Random123 known-answer vectors for philox4x32-10
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for ctr, key, out in kat:
        assert [int(x) for x in orc.philox4x32_10(ctr, key)] == out


def test_dropout_mask_definition():
    n = 1 << 16
    keep = orc.dropout_mask(0, 0, n, 0.1)
    assert abs(keep.mean() - 0.9) < 0.005
    assert np.array_equal(keep, orc.dropout_mask(0, 0, n, 0.1))
    assert not np.array_equal(keep, orc.dropout_mask(1, 0, n, 0.1))
    assert np.array_equal(keep[4096:], orc.dropout_mask(0, 4096, n - 4096, 0.1))      # counter-based: offsets compose
    assert orc.dropout_mask(0, 0, n, 0.0).all()
    # word -> uniform mapping, element 6 = word 2 of block 1
    word = int(orc.philox4x32_10([1, 0, 0, 0], [0, 0])[2])
    u = np.float32(word >> 8) * np.float32(2.0 ** -24)
    for p in (0.05, 0.5, 0.95):
        assert bool(orc.dropout_mask(0, 6, 1, p)[0]) == bool(u >= np.float32(p))


def _bf16(x):
    return orc.f32_to_bf16(np.ascontiguousarray(x, np.float32))


def test_mlp_outproj_float64_brute_force_and_all_ones():
    M, N, K, nP = 8, 12, 16, 3
    r = rng(10)
    X = _bf16(r.standard_normal((M, K)))
    W = _bf16(r.standard_normal((K, N)) * 0.02)
    parts = [r.standard_normal((M, N)).astype(np.float32) for _ in range(nP)]
    bias = r.standard_normal(N).astype(np.float32)
    resid = _bf16(r.standard_normal((M, N)))
    out, outf = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 0.1, 0)
    acc = orc.bf16_to_f32(X).astype(np.float64) @ orc.bf16_to_f32(W).astype(np.float64)
    s = acc + np.sum(np.stack(parts).astype(np.float64), axis=0) + bias
    keep = orc.dropout_mask(0, 0, M * N, 0.1).reshape(M, N).astype(bool)
    y = np.where(keep, s / 0.9, 0.0) + orc.bf16_to_f32(resid)
    assert np.max(np.abs(outf - y)) < 1e-5
    assert np.array_equal(out, _bf16(outf))
    # reference's only check at this boundary: all-ones operands give C == K*ranks
    # (nccl-overlap/samples/matmul-allreduce-bias-dropout-layernorm.cu:520-526)
    X1, W1 = _bf16(np.ones((M, K))), _bf16(np.ones((K, N)))
    parts1 = [np.full((M, N), K, np.float32) for _ in range(7)]
    _, outf = orc.mlp_outproj(X1, W1, parts1, np.zeros(N, np.float32), None, M, N, K, 0.0, 0)
    assert np.all(outf == K * 8)


def test_mlp_outproj_in_ieee_half():
    """The same routine with X, W, resid and out in IEEE half (the type of the reference's model-parallel example):
    float64 brute force over numpy's own float16 values, the output rounded by numpy's float16 cast, and the
    reference's all-ones check."""
    M, N, K, nP = 8, 12, 16, 3
    r = rng(11)
    Xh = r.standard_normal((M, K)).astype(np.float16)
    Wh = (r.standard_normal((K, N)) * 0.02).astype(np.float16)
    Rh = r.standard_normal((M, N)).astype(np.float16)
    parts = [r.standard_normal((M, N)).astype(np.float32) for _ in range(nP)]
    bias = r.standard_normal(N).astype(np.float32)
    out, outf = orc.mlp_outproj(Xh.view(np.uint16), Wh.view(np.uint16), parts, bias, Rh.view(np.uint16), M, N, K, 0.1, 0,
                                half=True)
    s = Xh.astype(np.float64) @ Wh.astype(np.float64) + np.sum(np.stack(parts).astype(np.float64), axis=0) + bias
    keep = orc.dropout_mask(0, 0, M * N, 0.1).reshape(M, N).astype(bool)
    y = np.where(keep, s / 0.9, 0.0) + Rh.astype(np.float64)
    assert np.max(np.abs(outf - y)) < 1e-5
    assert np.array_equal(out, outf.astype(np.float16).view(np.uint16))
    # the two 16-bit types give different answers on the same bits: the argument is not ignored
    out_b, _ = orc.mlp_outproj(Xh.view(np.uint16), Wh.view(np.uint16), parts, bias, Rh.view(np.uint16), M, N, K, 0.1, 0)
    assert not np.array_equal(out, out_b)
    ones = lambda shape: np.ones(shape, np.float16).view(np.uint16)
    parts1 = [np.full((M, N), K, np.float32) for _ in range(7)]
    o, outf = orc.mlp_outproj(ones((M, K)), ones((K, N)), parts1, np.zeros(N, np.float32), None, M, N, K, 0.0, 0, half=True)
    assert np.all(outf == K * 8) and np.all(o.view(np.float16) == K * 8)


# ---------------------------------------------------------------------------------------------------------------------
# the modified NCCL's global-norm LAMB arithmetic (mode 2)
# ---------------------------------------------------------------------------------------------------------------------
def test_lamb_nccl_global_all_ones_closed_form():
    # all-ones gradients on P ranks, w = m = v = 0, beta = .5, lr = 1 (the inputs of examples/test-adam.cu:73-88):
    # v = P^2/2, S4 = P^2, m = P/2, S3 = P, r = P/P + 0 = 1, W = 0, R = sqrt(N), scale = 1/R, w = -1/sqrt(N)
    for P in (2, 8):
        N = 4096
        g = [np.ones(N, np.float32) for _ in range(P)]
        w, m, v = (np.zeros(N, np.float32) for _ in range(3))
        norms = orc.lamb_f32(g, w, m, v, [0, N], 1.0, 0.5, 0.5, 0.0, 1.0, 1, 2)
        assert np.all(m == P / 2) and np.all(v == P * P / 2)
        assert norms[0, 0] == 0.0 and norms[0, 1] == 64.0
        assert np.all(w == np.float32(-1.0 / 64.0))


def test_lamb_nccl_global_float64_brute_force():
    P, N = 4, 5000
    g = grads_f32(60, P, N, 1e-2)
    w0 = weights_f32(60, N, 0.05)
    m0 = (rng(60, 50).standard_normal(N) * 1e-2).astype(np.float32)
    v0 = (rng(60, 51).uniform(1e-5, 1e-3, N)).astype(np.float32)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    b1, b2, lr = float(np.float32(0.9)), float(np.float32(0.999)), float(np.float32(1e-3))
    norms = orc.lamb_f32(g, w, m, v, [0, N], lr, b1, b2, 0.0, 1.0, 1, 2)
    gs = np.sum(np.stack(g).astype(np.float64), axis=0)
    vv = v0 * b2 + gs * gs * (1 - b2)
    mm = m0 * b1 + gs * (1 - b1)
    r = (mm / b1) / np.sqrt(vv / b2) + w0
    W, R = np.sqrt(np.sum(w0.astype(np.float64) ** 2)), np.sqrt(np.sum(r ** 2))
    assert abs(norms[0, 0] / W - 1) < 1e-6 and abs(norms[0, 1] / R - 1) < 1e-6
    expect = w0 - lr * (W / R / R) * r
    assert np.max(np.abs(w - expect)) < 1e-6 * np.max(np.abs(expect))
    assert np.max(np.abs(m - mm)) < 1e-6 * np.max(np.abs(mm)) and np.max(np.abs(v - vv)) < 1e-6 * np.max(np.abs(vv))


def test_adam_bf16g_reduces_to_adam_and_flags():
    """bfloat16 gradients: same pins as the fp16 variant, with torch's bfloat16 cast as the independent conversion."""
    import torch
    P, N = 8, 1 << 13
    scale = 2.0 ** 7
    g32 = grads_f32(10, P, N, 1e-3)
    g16 = [orc.f32_to_bf16(x * np.float32(scale)) for x in g32]
    for x32, x16 in zip(g32, g16):
        t = (torch.from_numpy(x32) * scale).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(x16, t)
    w0 = weights_f32(10, N, 0.05)
    w, m, v, w16 = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    flag = orc.adam_bf16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(1 / scale))
    dec = [orc.bf16_to_f32(x) * np.float32(1 / scale) for x in g16]
    wr, mr, vr = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    orc.adam_f32(dec, wr, mr, vr, 1e-3, 0.9, 0.999, 1e-6, 1)
    assert flag == 0
    assert np.array_equal(w, wr) and np.array_equal(m, mr) and np.array_equal(v, vr)
    want16 = torch.from_numpy(w).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(w16, want16)
    # finite values near 2^121, whose bits read as fp16 would be inf/nan patterns, are not overflows
    big = [orc.f32_to_bf16(x * np.float32(2.0 ** 100) * np.float32(2.0 ** 31)) for x in g32]
    assert all(np.isfinite(orc.bf16_to_f32(x)).all() for x in big)
    assert any(((x & 0x7C00) == 0x7C00).any() for x in big)
    wb, mb, vb = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    assert orc.adam_bf16g(big, wb, mb, vb, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(2.0 ** -120)) == 0
    assert np.isfinite(vb).all() and (mb != 0).any()
    # +inf, -inf and a nan
    bad = {17: (0, 0x7F80), 4096: (3, 0xFF80), N - 1: (7, 0x7FC1)}
    for i, (p, bits) in bad.items():
        g16[p][i] = bits
    dec = [orc.bf16_to_f32(x) * np.float32(1 / scale) for x in g16]
    for i, (p, _) in bad.items():
        dec[p][i] = 0
    wr, mr, vr = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    orc.adam_f32(dec, wr, mr, vr, 1e-3, 0.9, 0.999, 1e-6, 1)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    flag = orc.adam_bf16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(1 / scale))
    assert flag == 1
    keep = np.ones(N, bool)
    keep[list(bad)] = False
    assert np.array_equal(w[keep], wr[keep]) and np.array_equal(m[keep], mr[keep]) and np.array_equal(v[keep], vr[keep])
    assert np.array_equal(w[~keep], w0[~keep]) and np.all(m[~keep] == 0) and np.all(v[~keep] == 0)
    assert np.all(np.isfinite(w)) and np.isfinite(m).all() and np.isfinite(v).all()


# ---------------------------------------------------------------------------------------------------------------------
# the modified NCCL's mixed-precision LAMB (fp16 gradients)
# ---------------------------------------------------------------------------------------------------------------------
def test_lamb_nccl_f16g_equals_fp32_variant_where_fp16_is_exact():
    """Small-integer gradients: the fp16 sum and the fp16 square are exact, so every bit of m, v, w and the norms must
    equal the fp32 variant (mode 2) on the same values; a wrong beta, a dropped term or a swapped operand shows."""
    P, segs = 8, [0, 700, 701, 5000, 8192]
    N = segs[-1]
    r = rng(61)
    gi = [r.integers(-2, 3, N).astype(np.float32) for _ in range(P)]        # |sum| <= 16, square <= 256
    g16 = [orc.f32_to_f16(x) for x in gi]
    w0 = weights_f32(61, N, 0.05)
    m0 = weights_f32(62, N, 0.01)
    v0 = np.abs(weights_f32(63, N, 1e-2)) + np.float32(1e-3)
    w, m, v, hw = w0.copy(), m0.copy(), v0.copy(), np.zeros(N, np.uint16)
    n16 = orc.lamb_nccl_f16g(g16, w, hw, m, v, segs, 0.01, 0.9, 0.999, 1.0)
    wr, mr, vr = w0.copy(), m0.copy(), v0.copy()
    n32 = orc.lamb_f32(gi, wr, mr, vr, segs, 0.01, 0.9, 0.999, 0.0, 1.0, 1, mode=2)
    assert np.array_equal(m, mr) and np.array_equal(v, vr) and np.array_equal(w, wr)
    assert np.array_equal(n16, n32)
    assert np.array_equal(hw, w.astype(np.float16).view(np.uint16))


def test_lamb_nccl_f16g_half_chain_against_numpy_float16():
    """Where fp16 rounds: the sum chain and the square, restated with numpy's float16 (correctly rounded, an
    independent implementation), must give the same m and v."""
    P, N = 5, 4096
    g32 = grads_f32(64, P, N, 3.0)
    g16 = [orc.f32_to_f16(x) for x in g32]
    w0 = weights_f32(64, N, 0.05)
    m0 = weights_f32(65, N, 0.01)
    v0 = np.abs(weights_f32(66, N, 1e-2)) + np.float32(1e-3)
    w, m, v, hw = w0.copy(), m0.copy(), v0.copy(), np.zeros(N, np.uint16)
    orc.lamb_nccl_f16g(g16, w, hw, m, v, [0, N], 0.01, 0.9, 0.999, 1.0)
    S0 = g16[0].view(np.float16).copy()
    for x in g16[1:]:
        S0 = (S0 + x.view(np.float16)).astype(np.float16)
    sq = (S0 * S0).astype(np.float16)
    assert np.any(sq.astype(np.float32) != S0.astype(np.float32) ** 2)      # the square does round somewhere
    b1, b2 = np.float32(0.9), np.float32(0.999)
    want_v = (v0 * b2) + (sq.astype(np.float32) * (np.float32(1) - b2))
    want_m = (m0 * b1) + (S0.astype(np.float32) * (np.float32(1) - b1))
    assert np.array_equal(v, want_v.astype(np.float32)) and np.array_equal(m, want_m.astype(np.float32))
    # and the update, in float64, from those m and v
    r = (want_m.astype(np.float64) / 0.9) / np.sqrt(want_v.astype(np.float64) / np.float64(b2)) + w0
    scale = (np.sqrt(np.sum(w0.astype(np.float64) ** 2)) / np.sqrt(np.sum(r ** 2))) / np.sqrt(np.sum(r ** 2))
    assert np.max(np.abs(w - (w0 - 0.01 * scale * r))) <= 1e-6 * np.max(np.abs(w0))
    assert np.array_equal(hw, w.astype(np.float16).view(np.uint16))


# ---------------------------------------------------------------------------------------------------------------------
# the reference's dropout forms (keep with probability p, no rescale): pinned by what the arithmetic fixes
# ---------------------------------------------------------------------------------------------------------------------
def test_reference_dropout_forms_closed_forms():
    """src/codegen.cpp:634-640 emits (curand_uniform < p ? x : 0): p = 0 keeps nothing, p = 1 everything, and nothing
    is rescaled.  FuncDropout (nccl-overlap/.../reduce_kernel.h:192-213) drops the sum only, then adds bias and
    residual, with saturation to [0, 1] in its half form."""
    r = rng(61)
    M, N, K, nP = 4, 8, 16, 3
    X = orc.f32_to_bf16(r.standard_normal((M, K), dtype=np.float32))
    W = orc.f32_to_bf16(r.standard_normal((K, N), dtype=np.float32) * np.float32(0.1))
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, N), dtype=np.float32))
    rf = orc.bf16_to_f32(resid)
    s = (orc.bf16_to_f32(X).astype(np.float64) @ orc.bf16_to_f32(W).astype(np.float64)).astype(np.float32)
    for q in parts:
        s = s + q
    # p = 0: nothing survives.  DSL form: the residual alone; fused-kernel form: bias + residual
    _, y = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 0.0, 3, mode=1)
    assert np.array_equal(y, rf)
    _, y = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 0.0, 3, mode=2)
    assert np.array_equal(y, (np.float32(0) + bias[None, :]) + rf)
    # p = 1: everything survives, unscaled
    _, y = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 1.0, 3, mode=1)
    assert np.array_equal(y, (s + bias[None, :]) + rf)
    _, y = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 1.0, 3, mode=2)
    assert np.array_equal(y, (s + bias[None, :]) + rf)
    # in between: the survivors of "keep with probability p" are exactly the elements "drop with probability p" drops
    p = 0.3
    dropped_by_standard = ~orc.dropout_mask(3, 0, M * N, p).reshape(M, N).astype(bool)
    _, y = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 3, mode=1)
    assert np.array_equal(y, np.where(dropped_by_standard, s + bias[None, :], np.float32(0)) + rf)
    _, y0 = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 3, mode=0)
    scale = np.float32(1) / (np.float32(1) - np.float32(p))
    assert np.array_equal(y0, np.where(dropped_by_standard, np.float32(0), (s + bias[None, :]) * scale) + rf)
    assert 0 < dropped_by_standard.sum() < M * N


def test_reference_saturating_dropout_form():
    """__hadd2_sat clamps every sum to [0, 1]: all-ones inputs give 1 (not 3), a negative kept sum gives
    sat(sat(s + b) + r) with the inner clamp at 0 applied before the residual is added."""
    one = np.float32(1.0)
    assert orc.epilogue_value(one, one, one, 0, 0.5, 3) == 1.0          # kept: sat(sat(1 + 1) + 1)
    assert orc.epilogue_value(one, one, one, 1, 0.5, 3) == 1.0          # dropped: sat(sat(0 + 1) + 1)
    assert orc.epilogue_value(-2.0, 0.5, 0.25, 0, 0.5, 3) == 0.25       # sat(-1.5) = 0, then 0 + 0.25
    assert orc.epilogue_value(-2.0, 0.5, 0.25, 0, 0.5, 2) == -1.25      # unsaturated: (-2 + 0.5) + 0.25
    assert orc.epilogue_value(0.25, 0.25, 0.25, 0, 0.5, 3) == 0.75 and orc.epilogue_value(0.25, 0.25, -1.0, 0, 0.5, 3) == 0.0
    assert orc.epilogue_value(float("nan"), 0.0, 0.0, 0, 0.5, 3) == 0.0  # NaN saturates to zero


def test_saturating_form_in_half_rounds_after_each_add():
    """FuncDropout<half> (nccl-overlap/src/collectives/device/reduce_kernel.h:199-213) holds value, bias and residual as
    halves and each __hadd2_sat rounds to half.  Hand-computed: at 0.5 a half's spacing is 2^-11, so 0.5 + 2^-12 is a
    tie and rounds to even (0.5) -- twice; one fp32 sum rounded once would give 0.5 + 2^-11.  numpy's float16
    arithmetic (an independent library) rounds after each add too."""
    h = np.float32(2.0 ** -12)
    assert orc.epilogue_value(0.5, h, h, 0, 0.5, 3, half=True) == 0.5
    assert orc.epilogue_value(0.5, h, h, 0, 0.5, 3) == 0.5 + 2.0 ** -11           # the fp32 form adds first, rounds never
    # the sum itself is rounded to half before the first add (the reference's value is a half): 0.5 + 2^-13 -> 0.5
    assert orc.epilogue_value(0.5 + 2.0 ** -13, 0.0, 0.0, 0, 0.5, 3, half=True) == 0.5
    # the other forms do not change with the operand type
    for mode in (0, 1, 2):
        assert orc.epilogue_value(0.3, 0.2, 0.1, 0, 0.5, mode, half=True) == orc.epilogue_value(0.3, 0.2, 0.1, 0, 0.5, mode)
    r = rng(62)
    s = (r.standard_normal(4000) * 0.3).astype(np.float16)
    b = (r.standard_normal(4000) * 0.3).astype(np.float16)
    res = (r.standard_normal(4000) * 0.3).astype(np.float16)
    sat = lambda x: np.clip(x, np.float16(0), np.float16(1))
    want = sat(sat(s + b) + res)                                                   # float16 arithmetic throughout
    got = np.array([orc.epilogue_value(float(s[i]), float(b[i]), float(res[i]), 0, 0.5, 3, half=True) for i in range(4000)])
    assert np.array_equal(got.astype(np.float16), want) and np.array_equal(got, want.astype(np.float64))


def test_row_subset_of_the_out_projection_equals_the_whole_call():
    """orc.mlp_outproj(row_ids=...) on gathered rows gives the rows of the whole-output call, mask included; and the
    product behind it is the float64 brute force whatever the loop order."""
    r = rng(63)
    M, N, K, nP, p = 24, 16, 40, 2, 0.4
    X = orc.f32_to_bf16(r.standard_normal((M, K), dtype=np.float32))
    W = orc.f32_to_bf16(r.standard_normal((K, N), dtype=np.float32))
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, N), dtype=np.float32))
    whole, whole_f = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 11)
    rows = np.array([23, 0, 7, 8, 15])
    sub, sub_f = orc.mlp_outproj(np.ascontiguousarray(X[rows]), W, [np.ascontiguousarray(q[rows]) for q in parts], bias,
                                 np.ascontiguousarray(resid[rows]), len(rows), N, K, p, 11, row_ids=rows)
    assert np.array_equal(sub, whole[rows]) and np.array_equal(sub_f, whole_f[rows])
    # brute force, k innermost, float64: the product of one element
    xf, wf = orc.bf16_to_f32(X).astype(np.float64), orc.bf16_to_f32(W).astype(np.float64)
    keep = orc.dropout_mask(11, 0, M * N, p).reshape(M, N).astype(bool)
    for (i, j) in [(0, 0), (23, 15), (7, 3)]:
        acc = 0.0
        for k in range(K):
            acc += xf[i, k] * wf[k, j]
        s = np.float32(acc)
        for q in parts:
            s = np.float32(s + q[i, j])
        t = np.float32(s + bias[j])
        y = np.float32((np.float32(t * (np.float32(1) / (np.float32(1) - np.float32(p)))) if keep[i, j] else np.float32(0))
                       + orc.bf16_to_f32(resid[i:i + 1, j:j + 1])[0, 0])
        assert whole_f[i, j] == y


# ---------------------------------------------------------------------------------------------------------------------
# the LAMB of the DSL example (examples/lamb/lamb.cpp:20-28): what the programs emitted from it are checked against
# ---------------------------------------------------------------------------------------------------------------------
def test_dsl_lamb_all_ones_closed_form():
    """g = 1 on P ranks, m = v = 0, w = 1, beta = 1/2, gamma = 1: m1 = P/2, v1 = P^2/2, m_ = P, v_ = P^2, r = 1 + 1 = 2,
    rNorm = 2 sqrt(N), wNorm = sqrt(N), w1 = 1 - lr * (1/2) * 2 = 1 - lr; every step exact for N a power of four."""
    for P in (1, 4, 8):
        N = 4096
        g = [np.ones(N, np.float32) for _ in range(P)]
        w, m, v = np.ones(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.float32)
        w1, norms = orc.dsl_lamb_f32(g, w, m, v, 0.25, 0.5, 0.5, 1.0)
        assert np.all(m == P / 2) and np.all(v == P * P / 2)
        assert norms[0] == 2 * 64 and norms[1] == 64
        assert np.all(w1 == 0.75) and np.all(w == 1.0)
    # gamma = 0 and a known r: w = 3, P = 2, g = 1: r = 1, wNorm/rNorm = 3, w1 = 3 - lr*3
    g = [np.ones(16, np.float32) for _ in range(2)]
    w1, norms = orc.dsl_lamb_f32(g, np.full(16, 3, np.float32), np.zeros(16, np.float32), np.zeros(16, np.float32), 0.5, 0.5, 0.5, 0.0)
    assert norms[0] == 4 and norms[1] == 12 and np.all(w1 == 1.5)


def test_dsl_lamb_against_a_float64_restatement():
    """An independent numpy restatement in float64 from the text of examples/lamb/lamb.cpp:20-28: fp32 results within
    a few ulp; a wrong operand order, a missing square root, a norm over r instead of w or the division the other way
    round are all far outside."""
    r = rng(71)
    N, P = 5000, 4
    g = [r.uniform(0, 1, N).astype(np.float32) for _ in range(P)]
    w, m0, v0 = (r.uniform(0, 1, N).astype(np.float32) for _ in range(3))
    lr, b1, b2, gamma = 0.01, 0.9, 0.99, 0.1
    m, v = m0.copy(), v0.copy()
    w1, norms = orc.dsl_lamb_f32(g, w, m, v, lr, b1, b2, gamma)
    G = np.sum(np.stack(g).astype(np.float64), axis=0)
    fb1, fb2 = np.float64(np.float32(b1)), np.float64(np.float32(b2))
    M = fb1 * m0 + (1.0 - fb1) * G
    V = fb2 * v0 + (1.0 - fb2) * G * G
    R = (M / (1.0 - fb1)) / np.sqrt(V / (1.0 - fb2)) + np.float64(np.float32(gamma)) * w
    rn, wn = np.sqrt(np.sum(R * R)), np.sqrt(np.sum(w.astype(np.float64) ** 2))
    W1 = w - np.float64(np.float32(lr)) * (wn / rn) * R
    assert np.max(np.abs(m - M) / np.abs(M)) < 4e-7 and np.max(np.abs(v - V) / np.abs(V)) < 4e-7
    assert abs(norms[0] - rn) / rn < 2e-7 and abs(norms[1] - wn) / wn < 2e-7
    assert np.max(np.abs(w1 - W1)) < 1e-6 * np.max(np.abs(W1))
    # with bias corrections and an epsilon handed in (the build's own lamb program)
    m, v = m0.copy(), v0.copy()
    w2, _ = orc.dsl_lamb_f32(g, w, m, v, lr, b1, b2, gamma, c1=0.3, c2=0.7, eps=1e-3)
    R2 = (M / np.float64(np.float32(0.3))) / (np.sqrt(V / np.float64(np.float32(0.7))) + np.float64(np.float32(1e-3))) + np.float64(np.float32(gamma)) * w
    W2 = w - np.float64(np.float32(lr)) * (wn / np.sqrt(np.sum(R2 * R2))) * R2
    assert np.max(np.abs(w2 - W2)) < 1e-6 * np.max(np.abs(W2))
