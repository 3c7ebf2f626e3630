"""GPU parity tests: the HIP kernels behind the C ABI against the CPU oracle on identical seeded inputs.

Bars (north star of the benchmark): fp32 state within 1e-6 relative, fp16 weight copies within 1e-3, overflow
flags exact.  The kernels are written to round where the oracle rounds, so the tests first ask for
bit-identical results and report the largest ulp distance if that ever fails.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from util import (REF_BUFF_SIZES_HEAD, REF_BUFF_SIZES_TAIL, grads_f32, ref_integer_pattern, rel_err, rng, ulp_diff_f32,
                  weights_f32)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP32_TOL = 1e-6


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def dev_u16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def host_u16(t):
    torch.cuda.synchronize()
    return t.cpu().numpy().view(np.uint16)


def assert_f32_parity(got, want, what):
    """North-star bar, then the stronger bit-exact claim."""
    scale = max(float(np.max(np.abs(want))), 1e-30) if want.size else 1.0
    assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)), initial=0.0) <= FP32_TOL * scale, what
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
        f"{what}: not bit-identical, max ulp distance {ulp_diff_f32(got, want)}, rel {rel_err(got, want):.3g}"


SIZES = [1, 3, 4, 5, 255, 1024, 4099, (1 << 20) + 3]
RANKS = [1, 2, 3, 4, 7, 8, 9, 16]


# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("P", RANKS)
def test_reduce_and_sgd_ranks(ccn, P):
    N = 70001
    g = grads_f32(11, P, N, 1e-2)
    gd = [dev(x) for x in g]
    out = torch.empty(N, device=DEV)
    ccn.reduce_f32(gd, out, N)
    assert_f32_parity(host(out), orc.reduce_f32(g), f"reduce P={P}")
    w0 = weights_f32(11, N, 0.1)
    wd = dev(w0)
    ccn.sgd_f32(gd, wd, N, 0.01)
    w = w0.copy()
    orc.sgd_f32(g, w, 0.01)
    assert_f32_parity(host(wd), w, f"sgd P={P}")
    ccn.sgd_axpby_f32(gd, wd, N, 0.75, -0.01)
    orc.sgd_axpby_f32(g, w, 0.75, -0.01)
    assert_f32_parity(host(wd), w, f"axpby P={P}")


@pytest.mark.parametrize("N", SIZES)
def test_sgd_sizes_and_tails(ccn, N):
    P = 4
    g = grads_f32(12, P, N, 1e-2)
    w0 = weights_f32(12, N, 0.1)
    # guard elements after the end must stay untouched
    wd = torch.full((N + 8,), 7.0, device=DEV)
    wd[:N] = dev(w0)
    ccn.sgd_f32([dev(x) for x in g], wd, N, 0.01)
    w = w0.copy()
    orc.sgd_f32(g, w, 0.01)
    got = host(wd)
    assert_f32_parity(got[:N], w, f"sgd N={N}")
    assert np.all(got[N:] == 7.0)


def test_sgd_config1_full_size(ccn):
    # benchmark configuration 1: N = 2^20, P = 4, g ~ N(0, 1e-2), w ~ U(-0.1, 0.1), lr = 0.01
    P, N = 4, 1 << 20
    g = grads_f32(0, P, N, 1e-2)
    w0 = weights_f32(0, N, 0.1)
    wd = dev(w0)
    ccn.sgd_f32([dev(x) for x in g], wd, N, 0.01)
    w = w0.copy()
    orc.sgd_f32(g, w, 0.01)
    got = host(wd)
    assert_f32_parity(got, w, "config 1")
    # the reference's own acceptance test for this program (examples/test-sgd.cu:19, eqFloat rel 1e-3)
    assert all(orc.eqFloat(a, b) for a, b in zip(w[::997], got[::997]))


def test_sgd_more_than_2_to_32_elements(ccn):
    """Element indices that do not fit 32 bits (17 GB per buffer): slices at the start, across 2^32 and at the ragged
    end go through the oracle bit for bit, the whole array through a torch expression at the 1e-6 bar."""
    P, N = 2, (1 << 32) + 4099
    gen = torch.Generator(device=DEV)
    gen.manual_seed(99)
    g = [torch.empty(N, device=DEV).normal_(0.0, 1e-2, generator=gen) for _ in range(P)]
    w = torch.empty(N, device=DEV).uniform_(-0.1, 0.1, generator=gen)
    windows = [(0, 8192), ((1 << 32) - 4096, (1 << 32) + 4099)]
    keep = [(host(w[a:b]).copy(), [host(x[a:b]).copy() for x in g]) for a, b in windows]
    want_all = w - (g[0] + g[1]) * 0.01
    ccn.sgd_f32(g, w, N, 0.01)
    torch.cuda.synchronize()
    assert float((w - want_all).abs().max()) <= FP32_TOL * 0.2
    del want_all
    for (a, b), (w0, g0) in zip(windows, keep):
        orc.sgd_f32(g0, w0, 0.01)
        assert_f32_parity(host(w[a:b]), w0, f"elements {a}..{b}")


def test_reduce_in_place_and_empty(ccn):
    P, N = 4, 5000
    g = grads_f32(13, P, N, 1e-2)
    gd = [dev(x) for x in g]
    ccn.reduce_f32(gd, gd[0], N)            # all-reduce in place, as the reference does
    assert_f32_parity(host(gd[0]), orc.reduce_f32(g), "in-place reduce")
    ccn.sgd_f32(gd, gd[1], 0, 0.1)          # N == 0 is a no-op
    assert np.array_equal(host(gd[1]), g[1])


def test_misaligned_buffers_take_the_scalar_path(ccn):
    P, N = 3, 10007
    g = grads_f32(14, P, N, 1e-2)
    w0 = weights_f32(14, N, 0.1)
    # shift every buffer by one element so that no pointer is 16-byte aligned
    gbuf = [torch.zeros(N + 1, device=DEV) for _ in range(P)]
    for b, x in zip(gbuf, g):
        b[1:] = dev(x)
    wbuf = torch.zeros(N + 1, device=DEV)
    wbuf[1:] = dev(w0)
    mbuf = torch.zeros(N + 1, device=DEV)
    vbuf = torch.zeros(N + 1, device=DEV)
    ccn.adam_f32([b[1:] for b in gbuf], wbuf[1:], mbuf[1:], vbuf[1:], N, 1e-3, 0.9, 0.999, 1e-6, 1)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, 1)
    assert_f32_parity(host(wbuf)[1:], w, "misaligned adam w")
    assert_f32_parity(host(mbuf)[1:], m, "misaligned adam m")
    assert host(wbuf)[0] == 0.0


# ---------------------------------------------------------------------------------------------------------------------
def test_pseudo_adam_known_answer_and_parity(ccn):
    for P in (1, 4, 8):
        N = 3001
        ones = [torch.ones(N, device=DEV) for _ in range(P)]
        w, m, v = (torch.zeros(N, device=DEV) for _ in range(3))
        ccn.pseudo_adam_f32(ones, w, m, v, N, 1.0, 0.5, 0.5)
        assert np.all(host(w) == np.float32(-1.0 / P))          # examples/test-adam.cu:73-88
    P, N = 8, 50001
    g = grads_f32(15, P, N, 1e-2)
    w0, m0 = weights_f32(15, N, 0.1), weights_f32(16, N, 0.01)
    v0 = np.abs(weights_f32(17, N, 0.01)) + np.float32(1e-3)
    wd, md, vd = dev(w0), dev(m0), dev(v0)
    ccn.pseudo_adam_f32([dev(x) for x in g], wd, md, vd, N, 0.1, 0.9, 0.99)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    orc.pseudo_adam_f32(g, w, m, v, 0.1, 0.9, 0.99)
    assert_f32_parity(host(wd), w, "pseudo-adam w")
    assert_f32_parity(host(md), m, "pseudo-adam m")
    assert_f32_parity(host(vd), v, "pseudo-adam v")


@pytest.mark.parametrize("P,N", [(8, 1 << 20), (8, 4099), (1, 1000), (5, 12345), (12, 7777)])
def test_adam_config2_ten_steps(ccn, P, N):
    # benchmark configuration 2 at reduced N: fresh gradients every step, bias correction at t = 1..10
    w0 = weights_f32(0, N, 0.05)
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    for t in range(1, 11):
        g = grads_f32(0, P, N, 1e-3, step=t)
        ccn.adam_f32([dev(x) for x in g], wd, md, vd, N, 1e-3, 0.9, 0.999, 1e-6, t)
        orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    assert_f32_parity(host(wd), w, "adam w")
    assert_f32_parity(host(md), m, "adam m")
    assert_f32_parity(host(vd), v, "adam v")


def test_adam_reference_fixture(ccn):
    """The reference's own harness (multi-process-adam-scattered.cpp:156-369): integer pattern, beta = .5,
    alpha = +1, 5 checked steps, judged with its eq_float (rel 1e-5)."""
    P = 4
    for buff, n in enumerate(REF_BUFF_SIZES_TAIL):
        g0 = ref_integer_pattern(buff, n)
        gd = [dev(g0) for _ in range(P)]
        wd, md, vd = dev(g0), torch.zeros(n, device=DEV), torch.zeros(n, device=DEV)
        w, m, v = g0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
        for epoch in range(5):
            ccn.adam_f32(gd, wd, md, vd, n, -1.0, 0.5, 0.5, 1e-6, epoch + 1)
            orc.adam_f32([g0] * P, w, m, v, -1.0, 0.5, 0.5, 1e-6, epoch + 1)
            got = host(wd)
            assert all(orc.eq_float(a, b) for a, b in zip(w, got))
            assert_f32_parity(got, w, f"fixture buff {buff} epoch {epoch}")


def test_adam_full_size_sampled(ccn):
    """benchmark configuration 2 at its full size (N = 2^28, P = 8).  Adam is elementwise, so the oracle is run on
    the elements gathered at sampled indices (first/last elements, block edges and random positions)."""
    P, N = 8, 1 << 28
    gen = torch.Generator(device=DEV)
    gen.manual_seed(1234)
    g = [torch.randn(N, device=DEV, generator=gen) * 1e-3 for _ in range(P)]
    w = (torch.rand(N, device=DEV, generator=gen) - 0.5) * 0.1
    m = torch.zeros(N, device=DEV)
    v = torch.zeros(N, device=DEV)
    r = rng(20)
    idx = np.unique(np.concatenate([
        np.arange(0, 4096), np.arange(N - 4096, N), r.integers(0, N, 200000),
        (np.arange(1, 2048) * 131072)[:, None].repeat(8, 1).ravel() + np.tile(np.arange(-4, 4), 2047),
    ]))
    it = torch.from_numpy(idx).to(DEV)
    hw, hm, hv = (host(x[it]).copy() for x in (w, m, v))
    for t in (1, 2, 3):
        hg = [host(x[it]).copy() for x in g]
        ccn.adam_f32(g, w, m, v, N, 1e-3, 0.9, 0.999, 1e-6, t)
        orc.adam_f32(hg, hw, hm, hv, 1e-3, 0.9, 0.999, 1e-6, t)
        for x in g:            # next step's gradients: a cheap deterministic change of every buffer
            x.mul_(-0.5)
    assert_f32_parity(host(w[it]), hw, "full-size adam w")
    assert_f32_parity(host(m[it]), hm, "full-size adam m")
    assert_f32_parity(host(v[it]), hv, "full-size adam v")
    # size-independent property: with m, v restarted at zero and every rank holding the same g, the step-1
    # update is lr*G/(|G|+eps) with G = P*g, on every one of the 2^28 elements
    m.zero_(); v.zero_()
    w_before = w.clone()
    ccn.adam_f32([g[0]] * P, w, m, v, N, 1e-3, 0.9, 0.999, 1e-6, 1)
    G = g[0].double() * P
    expect = w_before.double() - 1e-3 * G / (G.abs() + 1e-6)
    assert float((w.double() - expect).abs().max()) < 1e-8


# ---------------------------------------------------------------------------------------------------------------------
def _mixed_inputs(seed, P, N, plant):
    scale = np.float32(2.0 ** 16)
    g16 = [orc.f32_to_f16(x * scale) for x in grads_f32(seed, P, N, 1e-3)]
    r = rng(seed, 77)
    for _ in range(plant):
        g16[int(r.integers(0, P))][int(r.integers(0, N))] = [0x7C00, 0xFC00, 0x7E00][int(r.integers(0, 3))]
    return g16


@pytest.mark.parametrize("P,N,plant", [(8, 1 << 20, 0), (8, 1 << 20, 1), (8, 100003, 5), (3, 8, 1), (9, 4099, 2),
                                       (1, 1, 1), (8, 7, 0)])
def test_mixed_precision_adam(ccn, P, N, plant):
    g16 = _mixed_inputs(21, P, N, plant)
    w0 = weights_f32(21, N, 0.05)
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w16d = torch.zeros(N, dtype=torch.int16, device=DEV)
    flag = torch.full((1,), 123, dtype=torch.int32, device=DEV)      # stale value must be overwritten
    gd = [dev_u16(x) for x in g16]
    w, m, v, w16 = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    for t in (1, 2):
        ccn.adam_f16g(gd, wd, md, vd, w16d, N, 1e-3, 0.9, 0.999, 1e-6, t, 2.0 ** -16, flag)
        want = orc.adam_f16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, t, np.float32(2.0 ** -16))
        assert int(host(flag)[0]) == want == (1 if plant else 0)
    assert_f32_parity(host(wd), w, "mixed w")
    assert_f32_parity(host(md), m, "mixed m")
    assert_f32_parity(host(vd), v, "mixed v")
    got16 = host_u16(w16d)
    assert rel_err(orc.f16_to_f32(got16), orc.f16_to_f32(w16)) <= 1e-3
    assert np.array_equal(got16, w16)
    ccn.overflow_check_f16(gd, N, flag)
    assert int(host(flag)[0]) == orc.overflow_f16(g16)


@pytest.mark.parametrize("P,N,plant,log2scale", [(8, 1 << 20, 0, 7), (8, 100003, 4, 7), (3, 8, 1, 7), (9, 4099, 2, 7),
                                                 (1, 1, 1, 7), (8, 65539, 0, 131)])
def test_mixed_precision_adam_bf16(ccn, P, N, plant, log2scale):
    """bfloat16 gradients and weight copy; overflow = exponent 0xFF.  At scale 2^131 the finite gradients sit near
    2^121, where their bits read as fp16 would be inf/nan patterns: the flag must stay 0."""
    inv = float(np.float32(2.0 ** -min(log2scale, 120)))      # kept a normal number
    g16 = [orc.f32_to_bf16(x * np.float32(2.0 ** (log2scale - 31)) * np.float32(2.0 ** 31))
           for x in grads_f32(23, P, N, 1e-3)]
    r = rng(23, 77)
    for _ in range(plant):
        g16[int(r.integers(0, P))][int(r.integers(0, N))] = [0x7F80, 0xFF80, 0x7FC0][int(r.integers(0, 3))]
    if log2scale > 100:
        assert any(((x & 0x7C00) == 0x7C00).any() for x in g16)
        assert all(np.isfinite(orc.bf16_to_f32(x)).all() for x in g16)
    w0 = weights_f32(23, N, 0.05)
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w16d = torch.zeros(N, dtype=torch.int16, device=DEV)
    flag = torch.full((1,), 123, dtype=torch.int32, device=DEV)
    gd = [dev_u16(x) for x in g16]
    w, m, v, w16 = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    for t in (1, 2):
        ccn.adam_bf16g(gd, wd, md, vd, w16d, N, 1e-3, 0.9, 0.999, 1e-6, t, inv, flag)
        want = orc.adam_bf16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, t, np.float32(inv))
        assert int(host(flag)[0]) == want == (1 if plant else 0)
    assert_f32_parity(host(wd), w, "bf16 w")
    assert_f32_parity(host(md), m, "bf16 m")
    assert_f32_parity(host(vd), v, "bf16 v")
    assert np.array_equal(host_u16(w16d), w16)


def test_mixed_precision_full_size_flag_and_skips(ccn):
    """benchmark configuration 3 at full size: one in 2^20 entries forced to inf.  Checked through properties:
    flag == 1, exactly the planted elements keep their state, fp16 copy == fp16(w) everywhere."""
    P, N = 8, 1 << 28
    gen = torch.Generator(device=DEV)
    gen.manual_seed(99)
    g = [(torch.randn(N, device=DEV, generator=gen) * (1e-3 * 65536.0)).to(torch.float16) for _ in range(P)]
    r = rng(22)
    planted = np.unique(r.integers(0, N, (N * P) >> 20))
    ranks = r.integers(0, P, planted.size)
    inf16 = torch.tensor(float("inf"), dtype=torch.float16, device=DEV)
    for p in range(P):
        sel = torch.from_numpy(planted[ranks == p]).to(DEV)
        g[p][sel] = inf16
    w = (torch.rand(N, device=DEV, generator=gen) - 0.5) * 0.1
    w0 = w.clone()
    m = torch.zeros(N, device=DEV)
    v = torch.zeros(N, device=DEV)
    w16 = torch.zeros(N, dtype=torch.float16, device=DEV)
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    ccn.adam_f16g(g, w, m, v, w16, N, 1e-3, 0.9, 0.999, 1e-6, 1, 2.0 ** -16, flag)
    assert int(host(flag)[0]) == 1
    # which elements overflow, and which have an exactly zero gradient sum, recomputed with torch
    bad = torch.zeros(N, dtype=torch.bool, device=DEV)
    gs = torch.zeros(N, device=DEV)
    for p in range(P):
        bad |= ~torch.isfinite(g[p])
        gs = g[p].float() * (2.0 ** -16) if p == 0 else gs + g[p].float() * (2.0 ** -16)
    assert np.array_equal(torch.nonzero(bad).flatten().cpu().numpy(), planted)
    unchanged = (w == w0) & (m == 0) & (v == 0)
    assert bool(torch.equal(unchanged, bad | (gs == 0)))      # exactly the overflowing elements are skipped
    del bad, gs, unchanged
    assert bool(torch.equal(w16, w.to(torch.float16)))
    assert bool(torch.isfinite(w).all()) and bool(torch.isfinite(m).all()) and bool(torch.isfinite(v).all())
    # sampled parity against the oracle, planted positions included
    idx = np.unique(np.concatenate([planted[:2000], r.integers(0, N, 100000), np.arange(N - 64, N)]))
    it = torch.from_numpy(idx).to(DEV)
    hg = [host(x[it]).view(np.uint16).copy() for x in g]
    hw, hm, hv = host(w0[it]).copy(), np.zeros(idx.size, np.float32), np.zeros(idx.size, np.float32)
    h16 = np.zeros(idx.size, np.uint16)
    orc.adam_f16g(hg, hw, hm, hv, h16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(2.0 ** -16))
    assert_f32_parity(host(w[it]), hw, "full-size mixed w")
    assert_f32_parity(host(v[it]), hv, "full-size mixed v")
    assert np.array_equal(host(w16[it]).view(np.uint16), h16)


def test_fused_adam_reference_variant(ccn):
    # the modified NCCL's kernel arithmetic: known answer (common_kernel.h:658-660) and parity on random data
    for P in (2, 8):
        N = 5003
        ones = [torch.ones(N, dtype=torch.float16, device=DEV) for _ in range(P)]
        w, m, v = (torch.zeros(N, device=DEV) for _ in range(3))
        hw = torch.zeros(N, dtype=torch.int16, device=DEV)
        ccn.fused_adam_ref_f16g(ones, w, hw, m, v, N, 1.0, 0.5, 0.5)
        assert np.all(host(w) == -1.0) and np.all(host_u16(hw) == 0xBC00)
    # beta1 != beta2, by hand: the kernel decays the first moment with beta2 (common_kernel.h:878) and divides it by
    # beta1 (:879).  One rank, g = 1, lr = 1, beta1 = 1/2, beta2 = 1/4: m = 3/4 then 15/16; w = -(3/2)/sqrt(3), then
    # minus (15/8)/sqrt(15/4); with beta1 in the decay m would be 1/2 then 3/4.
    N = 777
    one = [torch.ones(N, dtype=torch.float16, device=DEV)]
    w, m, v = (torch.zeros(N, device=DEV) for _ in range(3))
    hw = torch.zeros(N, dtype=torch.int16, device=DEV)
    f = np.float32
    ccn.fused_adam_ref_f16g(one, w, hw, m, v, N, 1.0, 0.5, 0.25)
    w1 = f(0) - f(1.5) / np.sqrt(f(3.0))
    assert np.all(host(m) == f(0.75)) and np.all(host(v) == f(0.75)) and np.all(host(w) == w1)
    ccn.fused_adam_ref_f16g(one, w, hw, m, v, N, 1.0, 0.5, 0.25)
    assert np.all(host(m) == f(15 / 16)) and np.all(host(w) == w1 - f(15 / 8) / np.sqrt(f(15 / 4)))
    P, N = 8, 100001
    g16 = [orc.f32_to_f16(x) for x in grads_f32(23, P, N, 0.5)]
    w0 = weights_f32(23, N, 0.05)
    m0 = weights_f32(24, N, 0.05)
    v0 = np.abs(weights_f32(25, N, 0.05)) + np.float32(0.01)
    wd, md, vd = dev(w0), dev(m0), dev(v0)
    hwd = torch.zeros(N, dtype=torch.int16, device=DEV)
    ccn.fused_adam_ref_f16g([dev_u16(x) for x in g16], wd, hwd, md, vd, N, 0.01, 0.9, 0.99)
    w, m, v, hw = w0.copy(), m0.copy(), v0.copy(), np.zeros(N, np.uint16)
    orc.fused_adam_a3(g16, w, m, v, hw, 0.01, 0.9, 0.99)
    assert_f32_parity(host(wd), w, "A3 w")
    assert_f32_parity(host(md), m, "A3 m")
    assert_f32_parity(host(vd), v, "A3 v")
    assert np.array_equal(host_u16(hwd), hw)


# ---------------------------------------------------------------------------------------------------------------------
def _lamb_compare(ccn, g, w0, segs, lr, b1, b2, eps, wd_, steps, mode, what, m0=None, v0=None):
    N = w0.size
    gd = [dev(x) for x in g]
    wd, md, vd = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    plan = ccn.LambPlan(segs)
    for t in range(1, steps + 1):
        plan.step(gd, wd, md, vd, lr, b1, b2, eps, wd_, t, mode)
        norms = orc.lamb_f32(g, w, m, v, segs, lr, b1, b2, eps, wd_, t, mode)
        gn = plan.norms()
        assert rel_err(gn, norms) < 1e-9, what           # float64 sums, different association only
    gw, gm, gv = host(wd), host(md), host(vd)
    plan.close()
    # m and v do not depend on the norms: bit-exact.  w goes through scale = (float)(W/R): 1e-6 bar.
    assert_f32_parity(gm, m, what + " m")
    assert_f32_parity(gv, v, what + " v")
    scale = float(np.max(np.abs(w)))
    assert np.max(np.abs(gw.astype(np.float64) - w)) <= FP32_TOL * scale, what
    return ulp_diff_f32(gw, w)


# How a plan runs its segments: the one-tile-per-workgroup kernel for segments short enough to stay on chip (the
# default), the same with a spin limit of zero (every tile whose segment is not ready at the first poll goes through the
# deferred list), or the two-pass kernels only.  Knobs of ccn_lamb_plan_tune, applied to every plan the tests create.
SPIN, TWO_PASS, WITHHOLD = 0, 1, 2
LAMB_VARIANTS = {
    "one-tile": {},
    "one-tile-deferred": {SPIN: 0},
    "two-pass": {TWO_PASS: 1},
    # a patience of a poll or two: some tiles see their segment's scale in time, the others go to the trailing kernel
    "one-tile-short-patience": {SPIN: 6},
    # the workgroup that adds a segment up keeps the result to itself, as it does when a tile sum has not arrived: every
    # tile runs out of patience and the trailing kernel adds the segments up from the sums in memory
    "one-tile-withheld": {WITHHOLD: 1, SPIN: 8},
}


@pytest.fixture(params=list(LAMB_VARIANTS))
def lamb_variant(request, ccn, monkeypatch):
    monkeypatch.setattr(ccn, "LAMB_DEFAULT_KNOBS", dict(LAMB_VARIANTS[request.param]))
    return request.param


@pytest.mark.parametrize("mode", [0, 1])
def test_lamb_ragged_segments(ccn, mode, lamb_variant):
    P = 4
    segs = [0, 5, 1029, 1030, 4096, 10000, 10000 + 8192, 10000 + 3 * 8192 + 1, 70001]
    N = segs[-1]
    g = grads_f32(26, P, N, 1e-3)
    w0 = weights_f32(26, N, 0.05)
    ulps = _lamb_compare(ccn, g, w0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 3, mode, f"ragged mode {mode}")
    assert ulps <= 2


@pytest.mark.parametrize("P", [1, 5, 7, 9, 16])
@pytest.mark.parametrize("path", ["one-tile", "two-pass"])
def test_lamb_rank_counts(ccn, monkeypatch, P, path):
    """Every rank count has its own instantiation up to 8 and a looped one beyond; segments around the 8192-element
    tile of the one-tile kernel."""
    monkeypatch.setattr(ccn, "LAMB_DEFAULT_KNOBS", {TWO_PASS: 1} if path == "two-pass" else {})
    segs = [0, 8192, 8192 + 8191, 3 * 8192 + 5, 5 * 8192 + 5]
    N = segs[-1]
    g = grads_f32(40 + P, P, N, 1e-3)
    w0 = weights_f32(40, N, 0.05)
    ulps = _lamb_compare(ccn, g, w0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 2, 0, f"ranks {P} {path}")
    assert ulps <= 2


def test_lamb_config4_reduced(ccn, lamb_variant):
    # benchmark configuration 4 layout at reduced size: 16 segments of 2^16, P = 8, wd = 0.01, two-pass norm + update
    P, nseg, seglen = 8, 16, 1 << 16
    N = nseg * seglen
    segs = [i * seglen for i in range(nseg + 1)]
    g = grads_f32(0, P, N, 1e-3)
    w0 = weights_f32(0, N, 0.05)
    _lamb_compare(ccn, g, w0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 3, 0, "config 4 reduced")


def test_lamb_unaligned_buffers(ccn, lamb_variant):
    """Buffers that start 4 bytes past a 16-byte boundary take the element-wise path of every kernel."""
    P, segs = 3, [0, 700, 4096 + 700, 4096 + 701, 30011]
    N = segs[-1]
    g = grads_f32(71, P, N, 1e-3)
    w0 = weights_f32(71, N, 0.05)
    gd = [dev(np.concatenate([[np.float32(0)], x]))[1:] for x in g]
    wd = dev(np.concatenate([[np.float32(0)], w0]))[1:]
    md, vd = torch.zeros(N + 1, device=DEV)[1:], torch.zeros(N + 1, device=DEV)[1:]
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    plan = ccn.LambPlan(segs)
    for t in (1, 2):
        plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
        orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
    plan.close()
    assert_f32_parity(host(md), m, "unaligned m")
    assert_f32_parity(host(vd), v, "unaligned v")
    assert ulp_diff_f32(host(wd), w) <= 2


@pytest.mark.parametrize("long_seg", [4_000_000])
def test_lamb_mixed_resident_and_two_pass(ccn, long_seg):
    """One segment too long to stay on chip between short ones: the long one takes the two-pass kernels, the others
    the one-tile kernel, in one call.  The one-tile kernel keeps segments of up to half the tiles the GPU runs at once
    (384 tiles of 8192 elements)."""
    P = 2
    segs = [0, 3000, 3000 + long_seg, 3000 + long_seg + 8192, 3000 + long_seg + 8192 + 100_001]
    N = segs[-1]
    g = grads_f32(72, P, N, 1e-3)
    w0 = weights_f32(72, N, 0.05)
    ulps = _lamb_compare(ccn, g, w0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 2, 0, "mixed")
    assert ulps <= 2


def test_lamb_long_segment_two_level_sums(ccn):
    """A segment of more than 4096 two-pass tiles (5 M elements: too long to stay on chip) has its tile sums folded in
    groups before the finalize step; short segments on either side take the resident kernel in the same call."""
    P = 2
    segs = [0, 4097, 4097 + 5_000_001, 4097 + 5_000_001 + 70_000]
    N = segs[-1]
    g = grads_f32(73, P, N, 1e-3)
    w0 = weights_f32(73, N, 0.05)
    ulps = _lamb_compare(ccn, g, w0, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 2, 1, "long segment")
    assert ulps <= 2


def test_lamb_reference_fixture(ccn):
    """Reference harness for LAMB (multi-process-adam-scattered.cpp:464-698): integer pattern, beta = .5,
    alpha = 1, weight decay 1.0, reference scale; head and tail of its buffer-size list scaled to fit a test."""
    P = 2
    sizes = [s // 16 if s > 1 << 20 else s for s in REF_BUFF_SIZES_HEAD] + REF_BUFF_SIZES_TAIL
    segs = np.concatenate([[0], np.cumsum(sizes)]).tolist()
    g0 = np.concatenate([ref_integer_pattern(i, n) for i, n in enumerate(sizes)])
    N = g0.size
    gd = [dev(g0) for _ in range(P)]
    wd, md, vd = dev(g0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = g0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    plan = ccn.LambPlan(segs)
    for epoch in range(5):
        plan.step(gd, wd, md, vd, 1.0, 0.5, 0.5, 1e-6, 1.0, epoch + 1, ccn.LAMB_REFERENCE)
        orc.lamb_f32([g0] * P, w, m, v, segs, 1.0, 0.5, 0.5, 1e-6, 1.0, epoch + 1, 1)
        got = host(wd)
        bad = [i for i in range(0, N, 37) if not orc.eq_float(w[i], got[i])]      # the reference's comparator
        assert not bad, (epoch, bad[:5])
        assert np.max(np.abs(got.astype(np.float64) - w)) <= FP32_TOL * np.max(np.abs(w))
    plan.close()


def test_lamb_full_size_segments(ccn):
    """benchmark configuration 4 at full size (N = 2^28 as 256 segments of 2^20, P = 8): the oracle is run on four
    whole segments (first, two inner, last); segments are independent, so this is exact for them.  The norms of all
    256 segments are then checked against float64 norms and against the two-pass kernels' norms of the same step."""
    P, nseg, seglen = 8, 256, 1 << 20
    N = nseg * seglen
    gen = torch.Generator(device=DEV)
    gen.manual_seed(4321)
    g = [torch.randn(N, device=DEV, generator=gen) * 1e-3 for _ in range(P)]
    w = (torch.rand(N, device=DEV, generator=gen) - 0.5) * 0.1
    m = torch.zeros(N, device=DEV)
    v = torch.zeros(N, device=DEV)
    check = [0, 77, 200, 255]
    hg = {b: [host(x[b * seglen:(b + 1) * seglen]).copy() for x in g] for b in check}
    hw = {b: host(w[b * seglen:(b + 1) * seglen]).copy() for b in check}
    w0 = w.clone()
    plan = ccn.LambPlan([i * seglen for i in range(nseg + 1)])
    plan.step(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, ccn.LAMB_TRUST_RATIO)
    norms = plan.norms()
    for b in check:
        ww, mm, vv = hw[b].copy(), np.zeros(seglen, np.float32), np.zeros(seglen, np.float32)
        on = orc.lamb_f32(hg[b], ww, mm, vv, [0, seglen], 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0)
        assert rel_err(norms[b], on[0]) < 1e-9
        sl = slice(b * seglen, (b + 1) * seglen)
        assert_f32_parity(host(m[sl]), mm, f"segment {b} m")
        assert np.max(np.abs(host(w[sl]).astype(np.float64) - ww)) <= FP32_TOL * np.max(np.abs(ww))
    plan.close()
    assert norms.shape == (nseg, 2) and np.all(norms > 0)
    # Every segment, not only the four above.  The one-tile kernel passes tile sums between workgroups of one launch: a
    # tile sum that arrived late or stale would show in that segment's norms and nowhere else.  (a) against float64
    # norms computed by torch on the device from the weights before the step and the moments after it; (b) against the
    # two-pass kernels, which exchange nothing inside a launch, on the same inputs: their sums associate differently, so
    # equal to rounding, not to the bit.
    b1, b2, eps, wd = (float(np.float32(x)) for x in (0.9, 0.999, 1e-6, 0.01))      # the scalars as the C ABI receives them
    ref = np.empty((nseg, 2))
    for b in range(nseg):
        sl = slice(b * seglen, (b + 1) * seglen)
        mh = (m[sl].double() / (1 - b1)).float()
        vh = (v[sl].double() / (1 - b2)).float()
        r = mh.double() / (vh.sqrt().double() + eps) + wd * w0[sl].double()
        ref[b] = [float(w0[sl].double().pow(2).mean().sqrt()), float(r.pow(2).mean().sqrt())]
    assert rel_err(norms, ref) < 1e-6, rel_err(norms, ref)
    w2, m2, v2 = w0, torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    plan2 = ccn.LambPlan([i * seglen for i in range(nseg + 1)], knobs={TWO_PASS: 1})
    plan2.step(g, w2, m2, v2, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, ccn.LAMB_TRUST_RATIO)
    norms2 = plan2.norms()
    plan2.close()
    assert rel_err(norms, norms2) < 1e-12, rel_err(norms, norms2)
    assert torch.equal(m, m2) and torch.equal(v, v2)
    ulps = (w.view(torch.int32).long() - w2.view(torch.int32).long()).abs().max().item()
    assert ulps <= 2, ulps
    del g


def test_lamb_nccl_global_variant(ccn):
    """The modified NCCL's global-norm LAMB arithmetic (mode 2): its all-ones known answer and parity on random data.
    m, v bit-exact; the norms are rounded to fp32 from float64 sums on both sides; w within 1e-6."""
    for P in (2, 8):
        N = 4096
        ones = [torch.ones(N, device=DEV) for _ in range(P)]
        w, m, v = (torch.zeros(N, device=DEV) for _ in range(3))
        plan = ccn.LambPlan([0, N])
        plan.step(ones, w, m, v, 1.0, 0.5, 0.5, 0.0, 1.0, 1, ccn.LAMB_NCCL_GLOBAL)
        assert np.all(host(w) == np.float32(-1.0 / 64.0)) and np.all(host(m) == P / 2)
        plan.close()
    P, N = 8, 200003
    g = grads_f32(61, P, N, 1e-2)
    w0 = weights_f32(61, N, 0.05)
    m0 = weights_f32(62, N, 0.01)
    v0 = np.abs(weights_f32(63, N, 1e-3)) + np.float32(1e-5)
    wd, md, vd = dev(w0), dev(m0), dev(v0)
    plan = ccn.LambPlan([0, N])
    plan.step([dev(x) for x in g], wd, md, vd, 1e-3, 0.9, 0.999, 0.0, 1.0, 1, ccn.LAMB_NCCL_GLOBAL)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    norms = orc.lamb_f32(g, w, m, v, [0, N], 1e-3, 0.9, 0.999, 0.0, 1.0, 1, 2)
    assert_f32_parity(host(md), m, "nccl-lamb m")
    assert_f32_parity(host(vd), v, "nccl-lamb v")
    assert rel_err(plan.norms(), norms) < 1e-6
    assert np.max(np.abs(host(wd).astype(np.float64) - w)) <= FP32_TOL * np.max(np.abs(w))
    plan.close()


# ---------------------------------------------------------------------------------------------------------------------
def test_recorded_steps_replay_like_eager_calls(ccn):
    """ccn_graph_*: eight SGD steps and a mixed-precision Adam step recorded on a stream, replayed three times with
    eager work and synchronisations of the program's own in between; every replay is checked against the oracle."""
    P, N = 4, (1 << 20) + 3
    g = grads_f32(81, P, N, 1e-2)
    w0 = weights_f32(81, N, 0.1)
    g16 = [orc.f32_to_f16(x * np.float32(64.0)) for x in grads_f32(82, P, N, 1e-2)]
    g16[1][12345] = np.uint16(0x7c00)                       # one overflowing element
    gd, wd = [dev(x) for x in g], dev(w0)
    g16d = [dev_u16(x) for x in g16]
    w2d, m2d, v2d = dev(w0), torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w16d = torch.zeros(N, dtype=torch.int16, device=DEV)
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    stream = ccn.Stream()
    with ccn.Graph(stream) as graph:
        for _ in range(8):
            ccn.sgd_f32(gd, wd, N, 0.01, stream.h)
        ccn.adam_f16g(g16d, w2d, m2d, v2d, w16d, N, 1e-3, 0.9, 0.999, 1e-6, 1, 1.0 / 64.0, flag, stream.h)
    assert np.array_equal(host(wd), w0)                     # recording runs nothing
    w = w0.copy()
    w2, m2, v2, w16 = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    scratch = torch.zeros(1 << 22, device=DEV)
    for replay in range(3):
        graph.launch()
        stream.sync()
        for _ in range(8):
            orc.sgd_f32(g, w, 0.01)
        want_flag = orc.adam_f16g(g16, w2, m2, v2, w16, 1e-3, 0.9, 0.999, 1e-6, 1, 1.0 / 64.0)
        assert_f32_parity(host(wd), w, f"replay {replay}: sgd w")
        assert_f32_parity(host(w2d), w2, f"replay {replay}: adam w")
        assert_f32_parity(host(v2d), v2, f"replay {replay}: adam v")
        assert np.array_equal(host_u16(w16d), w16) and int(flag.item()) == want_flag == 1
        flag.zero_()                                        # the recorded call clears and sets it again
        scratch.add_(1.0)                                   # eager work between replays
        ccn.sgd_f32(gd, scratch[:N], N, 0.0)
        torch.cuda.synchronize()
    graph.close()
    stream.close()


def test_recorded_lamb_step_replays(ccn):
    """A LAMB step through the one-tile kernel (segments that stay on chip), recorded after one eager call and replayed twice."""
    P, segs = 3, [0, 5000, 5000 + 40960, 5000 + 40960 + 12289]
    N = segs[-1]
    g = grads_f32(83, P, N, 1e-3)
    w0 = weights_f32(83, N, 0.05)
    gd, wd = [dev(x) for x in g], dev(w0)
    md, vd = torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    plan = ccn.LambPlan(segs)
    stream = ccn.Stream()
    plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0, stream.h)
    stream.sync()
    orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0)
    with ccn.Graph(stream) as graph:
        plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, 2, 0, stream.h)
    for replay in range(2):
        graph.launch()
        stream.sync()
        orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 2, 0)
        assert_f32_parity(host(md), m, f"replay {replay}: m")
        assert_f32_parity(host(vd), v, f"replay {replay}: v")
        assert ulp_diff_f32(host(wd), w) <= 2
        torch.cuda.synchronize()
    graph.close()
    plan.close()
    stream.close()


def test_lamb_on_chip_kernel_shares_the_gpu(ccn):
    """The one-tile kernel counts on a segment's tiles running at the same time.  With another stream keeping the GPU busy
    that need not hold: waits may run out and tiles go through the deferred list.  Whatever happens, the result is the same."""
    P, nseg, seglen = 4, 16, 1 << 20
    N = nseg * seglen
    segs = [i * seglen for i in range(nseg + 1)]
    g = grads_f32(91, P, N, 1e-3)
    w0 = weights_f32(91, N, 0.05)
    gd, wd = [dev(x) for x in g], dev(w0)
    md, vd = torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    # the competing work: Adam steps over other buffers on a second stream
    M = 1 << 26
    og = [torch.zeros(M, device=DEV) for _ in range(8)]
    ow, om, ov = (torch.zeros(M, device=DEV) for _ in range(3))
    plan = ccn.LambPlan(segs)
    a, b = ccn.Stream(), ccn.Stream()
    torch.cuda.synchronize()
    for t in (1, 2, 3):
        for _ in range(6):
            ccn.adam_f32(og, ow, om, ov, M, 1e-3, 0.9, 0.999, 1e-6, 1, b.h)
        plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0, a.h)
    a.sync()
    b.sync()
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    for t in (1, 2, 3):
        orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
    assert_f32_parity(host(md), m, "shared GPU: m")
    assert_f32_parity(host(vd), v, "shared GPU: v")
    assert ulp_diff_f32(host(wd), w) <= 2
    plan.close()
    a.close()
    b.close()


# ---------------------------------------------------------------------------------------------------------------------
MIXED_LAMB_SHAPES = [(8, [0, 1 << 18], 0), (3, [0, 700, 701, 5000, 8192 + 3], 0), (8, [0, 4096, 8192, 12288], 0),
                     (11, [0, 1000, 70001], 0), (2, [0, 4099], 1), (1, [0, 1], 0)]
# ... and one segment of more than 4096 tiles, which takes the two-pass kernels whatever the path: run once
MIXED_LAMB_CASES = [(P, segs, shift, path) for (P, segs, shift) in MIXED_LAMB_SHAPES
                    for path in ("one-tile", "one-tile-deferred", "two-pass")] + [(8, [0, 5 * 1024 * 4096 + 17], 0, "one-tile")]


@pytest.mark.parametrize("P,segs,shift,path", MIXED_LAMB_CASES)
def test_lamb_nccl_mixed_precision(ccn, monkeypatch, P, segs, shift, path):
    """The modified NCCL's LAMB with fp16 gradients: m and v bit for bit, w within the fp32 bar (the order of the
    float64 norm sums differs), the fp16 weight copy within one fp16 ulp and equal to fp16 of the kernel's own w.
    shift = 1: every array starts one element past an aligned address (scalar path).  The last case has a segment of
    more than 4096 tiles: it takes the two-pass kernels whatever the path, with its partial sums folded in two levels."""
    monkeypatch.setattr(ccn, "LAMB_DEFAULT_KNOBS", {"one-tile": {}, "one-tile-deferred": {SPIN: 0}, "two-pass": {TWO_PASS: 1}}[path])
    N = segs[-1]
    g16 = [orc.f32_to_f16(x) for x in grads_f32(71 + P, P, N, 0.5)]
    w0 = weights_f32(71, N, 0.05)
    m0 = weights_f32(72, N, 0.01)
    v0 = np.abs(weights_f32(73, N, 1e-2)) + np.float32(1e-3)

    def place(a, dt):
        if not shift:
            return dev(a) if dt == "f" else dev_u16(a)
        pad = np.concatenate([np.zeros(1, a.dtype), a])
        return (dev(pad) if dt == "f" else dev_u16(pad))[1:]

    gd = [place(x, "h") for x in g16]
    wd, md, vd = place(w0, "f"), place(m0, "f"), place(v0, "f")
    hwd = place(np.zeros(N, np.uint16), "h")
    w, m, v, hw = w0.copy(), m0.copy(), v0.copy(), np.zeros(N, np.uint16)
    plan = ccn.LambPlan(segs)
    for _ in range(2):
        plan.step_nccl_f16g(gd, wd, hwd, md, vd, 0.01, 0.9, 0.999, 1.0)
        want_norms = orc.lamb_nccl_f16g(g16, w, hw, m, v, segs, 0.01, 0.9, 0.999, 1.0)
    got_norms = plan.norms()
    plan.close()
    assert_f32_parity(host(md), m, "mixed lamb m")
    assert_f32_parity(host(vd), v, "mixed lamb v")
    got_w = host(wd)
    assert np.max(np.abs(got_w.astype(np.float64) - w)) <= FP32_TOL * np.max(np.abs(w))
    assert np.max(np.abs(got_norms - want_norms) / want_norms) <= 1e-6
    got_hw = host_u16(hwd)
    assert np.array_equal(got_hw, got_w.astype(np.float16).view(np.uint16))
    assert rel_err(orc.f16_to_f32(got_hw), orc.f16_to_f32(hw)) <= 1e-3


# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("P", [1, 3, 8, 11])
@pytest.mark.parametrize("counts", [[1, 255, 256, 257, 1000, 4096, 70001, 3],
                                    [1] * 70 + [300] + [2] * 40 + [9000, 8192, 5] + [256] * 33])
def test_scattered_adam_and_sgd(ccn, P, counts):
    """Gradients and weights in separate buffers of ragged sizes (two of them misaligned by 4 bytes), moments in single
    arrays over the concatenation: the same results, bit for bit, as the oracle on the concatenated arrays.  The second
    list has runs of buffers smaller than a tile, so that many buffers end inside one group of tiles."""
    offs = np.concatenate([[0], np.cumsum(counts)])
    N = int(offs[-1])
    g = grads_f32(95 + P, P, N, 1e-3)
    w0 = weights_f32(95, N, 0.05)

    def pieces(flat, shift_some):
        out = []
        for b, n in enumerate(counts):
            lo = int(offs[b])
            if shift_some and b in (3, 5):      # a buffer that starts 4 bytes past a 16-byte boundary
                out.append(dev(np.concatenate([[np.float32(0)], flat[lo:lo + n]]))[1:])
            else:
                out.append(dev(flat[lo:lo + n]))
        return out

    gd = [pieces(x, True) for x in g]
    wd = pieces(w0, True)
    md, vd = torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    plan = ccn.ScatterPlan(counts)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    for t in (1, 2, 3):
        plan.adam(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, t)
        orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    plan.sgd(gd, wd, 0.01)
    orc.sgd_f32(g, w, 0.01)
    got_w = np.concatenate([host(x) for x in wd])
    assert_f32_parity(got_w, w, "scattered w")
    assert_f32_parity(host(md), m, "scattered m")
    assert_f32_parity(host(vd), v, "scattered v")
    # new weight buffers: the pointer table follows
    wd2 = pieces(w0, False)
    plan.sgd(gd, wd2, 0.5)
    w2 = w0.copy()
    orc.sgd_f32(g, w2, 0.5)
    assert_f32_parity(np.concatenate([host(x) for x in wd2]), w2, "scattered w after a pointer change")
    plan.close()


@pytest.mark.parametrize("mode", [0, 2])
def test_scattered_lamb(ccn, mode, lamb_variant):
    """LAMB with every segment's gradients and weights in a buffer of its own (one of them misaligned by 4 bytes in a
    second run), moments over the concatenation: same results as the oracle on the concatenated arrays."""
    P = 3
    counts = [700, 4096 + 5, 1, 30000, 8192]
    segs = np.concatenate([[0], np.cumsum(counts)]).tolist()
    N = segs[-1]
    g = grads_f32(97, P, N, 1e-3)
    w0 = weights_f32(97, N, 0.05)
    eps, wd_ = (1e-6, 0.01) if mode == 0 else (0.0, 1.0)
    for shift in (False, True):
        def pieces(flat):
            out = []
            for b, n in enumerate(counts):
                lo = segs[b]
                if shift and b == 3:
                    out.append(dev(np.concatenate([[np.float32(0)], flat[lo:lo + n]]))[1:])
                else:
                    out.append(dev(flat[lo:lo + n]))
            return out
        gd, wd = [pieces(x) for x in g], pieces(w0)
        m0 = weights_f32(98, N, 0.01)
        v0 = np.abs(weights_f32(99, N, 1e-3)) + np.float32(1e-5)
        md, vd = dev(m0), dev(v0)
        w, m, v = w0.copy(), m0.copy(), v0.copy()
        plan = ccn.LambPlan(segs)
        for t in (1, 2):
            plan.step_scattered(gd, wd, md, vd, 1e-3, 0.9, 0.999, eps, wd_, t, mode)
            orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, eps, wd_, t, mode)
        plan.close()
        assert_f32_parity(host(md), m, "scattered lamb m")
        assert_f32_parity(host(vd), v, "scattered lamb v")
        got = np.concatenate([host(x) for x in wd])
        assert np.max(np.abs(got.astype(np.float64) - w)) <= FP32_TOL * np.max(np.abs(w))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("max_buf", [1000, 4096, 20000])
def test_scattered_lamb_with_parent_buffers(ccn, mode, max_buf, lamb_variant):
    """The reference cuts every parameter tensor into small buffers of at most maxBuffSize elements and maps them back
    with buffIdToParentBufferId (nccl-overlap/samples/multi-process-adam-scattered.cpp:505-517); the norms are per
    parent.  Every small buffer is an allocation of its own here; results must be the oracle's on the concatenated
    arrays with one segment per parent, and the parents' norms those of the plan that takes the parents whole."""
    P = 3
    parents = [700, 4096 + 5, 1, 30000, 8192, 2 * max_buf]
    sizes, parent_of = [], []
    for i, n in enumerate(parents):
        for lo in range(0, n, max_buf):
            sizes.append(min(max_buf, n - lo))
            parent_of.append(i)
    segs = np.concatenate([[0], np.cumsum(parents)]).tolist()
    offs = np.concatenate([[0], np.cumsum(sizes)]).tolist()
    N = segs[-1]
    g = grads_f32(197, P, N, 1e-3)
    w0 = weights_f32(197, N, 0.05)
    pieces = lambda flat: [dev(flat[offs[q]:offs[q + 1]]) for q in range(len(sizes))]
    gd, wd = [pieces(x) for x in g], pieces(w0)
    m0 = weights_f32(198, N, 0.01)
    v0 = np.abs(weights_f32(199, N, 1e-3)) + np.float32(1e-5)
    md, vd = dev(m0), dev(v0)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    plan = ccn.LambPlan(None, buf_sizes=sizes, buf_parent=parent_of)
    assert plan.nseg == len(parents) and plan.nbuf == len(sizes)
    for t in (1, 2):
        plan.step_scattered(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, mode)
        orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, mode)
    norms = plan.norms()
    plan.close()
    assert_f32_parity(host(md), m, "parented lamb m")
    assert_f32_parity(host(vd), v, "parented lamb v")
    got = np.concatenate([host(x) for x in wd])
    assert np.max(np.abs(got.astype(np.float64) - w)) <= FP32_TOL * np.max(np.abs(w))
    # the same two steps with the parents whole: the norms of the second step agree to the last few bits (the tile sums
    # are cut differently, so the float64 additions associate differently)
    whole = ccn.LambPlan(segs)
    wd2, md2, vd2 = dev(w0), dev(m0), dev(v0)
    gd2 = [dev(x) for x in g]
    for t in (1, 2):
        whole.step(gd2, wd2, md2, vd2, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, mode)
    want = whole.norms()
    whole.close()
    assert norms.shape == want.shape == (len(parents), 2)
    assert np.max(np.abs(norms - want) / np.maximum(np.abs(want), 1e-300)) < 1e-12


@pytest.mark.parametrize("which,ranks,max_buff", [("adam", 2, 0), ("adam", 8, 0), ("lamb", 2, 0), ("lamb", 3, 0),
                                                  ("lamb", 2, 65536), ("lamb", 3, 5000)])
def test_cpp_harness_in_the_shape_of_the_reference_sample(which, ranks, max_buff):
    """tests/harness/adam_lamb_scattered.cpp: the flow of the reference's multi-process-adam-scattered.cpp (its buffer
    list, integer inputs, five checked epochs, its comparator) through the scattered entry points, from C++."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "harness", "build", "adam_lamb_scattered")
    if not os.path.exists(exe):
        pytest.skip("harness not built (make -C tests/harness)")
    # max_buff > 0: the parents cut into small buffers with the sample's parent map (LAMB)
    r = subprocess.run([exe, which, str(ranks), "16", str(max_buff)], capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and "Success" in r.stdout, (r.stdout[-1500:], r.stderr[-500:])
    assert r.stdout.count("weights match the checker") == 5


# ---------------------------------------------------------------------------------------------------------------------
def _placed(a, shift, kind):
    """Device copy of `a` that starts `shift` elements past an aligned address."""
    if shift == 0:
        return dev(a) if kind == "f" else dev_u16(a)
    pad = np.concatenate([np.zeros(shift, a.dtype), a])
    return (dev(pad) if kind == "f" else dev_u16(pad))[shift:]


@pytest.mark.parametrize("case", range(24))
def test_seeded_random_shapes(ccn, case):
    """Seeded random rank counts, sizes, starting alignments and segmentations through every optimizer entry point:
    the same bits as the oracle (LAMB: m, v the same bits, w within 2 ulp)."""
    r = rng(1000 + case)
    P = int(r.integers(1, 17))
    N = int(r.choice([1, 2, 3, 5, 63, 64, 65, 255, 257, 1023, 4097, 8191, 8193, 40_000, 100_003, 262_147]))
    shifts = [int(x) for x in r.integers(0, 4, P + 3)] if case % 3 else [0] * (P + 3)
    op = ["sgd", "adam", "adam16", "lamb", "lamb16"][case % 5]
    w0 = weights_f32(2000 + case, N, 0.05)
    m0 = weights_f32(3000 + case, N, 0.01)
    v0 = np.abs(weights_f32(4000 + case, N, 1e-2)) + np.float32(1e-4)
    g = grads_f32(5000 + case, P, N, 1e-3)
    w, m, v = w0.copy(), m0.copy(), v0.copy()
    wd, md, vd = _placed(w0, shifts[P], "f"), _placed(m0, shifts[P + 1], "f"), _placed(v0, shifts[P + 2], "f")
    what = f"case {case}: {op} P={P} N={N} shifts={shifts}"
    if op in ("sgd", "adam", "lamb"):
        gd = [_placed(x, shifts[p], "f") for p, x in enumerate(g)]
    else:
        g16 = [orc.f32_to_f16(x * np.float32(256.0)) for x in g]
        gd = [_placed(x, shifts[p], "h") for p, x in enumerate(g16)]
    if op == "sgd":
        ccn.sgd_f32(gd, wd, N, 0.01)
        orc.sgd_f32(g, w, 0.01)
        assert_f32_parity(host(wd), w, what)
        return
    if op == "adam":
        for t in (1, 2):
            ccn.adam_f32(gd, wd, md, vd, N, 1e-3, 0.9, 0.999, 1e-6, t)
            orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    elif op == "adam16":
        w16d = _placed(np.zeros(N, np.uint16), shifts[0], "h")
        w16 = np.zeros(N, np.uint16)
        flag = torch.zeros(1, dtype=torch.int32, device=DEV)
        for t in (1, 2):
            ccn.adam_f16g(gd, wd, md, vd, w16d, N, 1e-3, 0.9, 0.999, 1e-6, t, 1.0 / 256.0, flag)
            want = orc.adam_f16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, t, np.float32(1.0 / 256.0))
            assert int(host(flag)[0]) == want == 0
        assert np.array_equal(host_u16(w16d), w16), what
    else:
        cuts = sorted(set(int(x) for x in r.integers(1, max(N, 2), min(5, N)) if 0 < x < N))
        segs = [0] + cuts + [N]
        plan = ccn.LambPlan(segs)
        if op == "lamb":
            mode = int(r.integers(0, 3))
            eps, wdec = (1e-6, 0.01) if mode != 2 else (0.0, 1.0)
            for t in (1, 2):
                plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, eps, wdec, t, mode)
                orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, eps, wdec, t, mode)
        else:
            hwd = _placed(np.zeros(N, np.uint16), shifts[0], "h")
            hw = np.zeros(N, np.uint16)
            for _ in (1, 2):
                plan.step_nccl_f16g(gd, wd, hwd, md, vd, 0.01, 0.9, 0.999, 1.0)
                orc.lamb_nccl_f16g(g16, w, hw, m, v, segs, 0.01, 0.9, 0.999, 1.0)
            got_w = host(wd)
            assert np.array_equal(host_u16(hwd), got_w.astype(np.float16).view(np.uint16)), what
        plan.close()
        assert_f32_parity(host(md), m, what + " m")
        assert_f32_parity(host(vd), v, what + " v")
        got_w = host(wd)
        assert np.max(np.abs(got_w.astype(np.float64) - w)) <= FP32_TOL * max(float(np.max(np.abs(w))), 1e-30), what
        return
    assert_f32_parity(host(wd), w, what + " w")
    assert_f32_parity(host(md), m, what + " m")
    assert_f32_parity(host(vd), v, what + " v")


@pytest.mark.parametrize("case", range(8))
def test_seeded_random_scattered_buffers(ccn, case):
    """Seeded random buffer lists (sizes from one element to a few tiles, some buffers misaligned) through the scattered
    Adam, SGD and LAMB entry points: the same bits as the oracle on the concatenation."""
    r = rng(7000 + case)
    P = int(r.integers(1, 12))
    nbuff = int(r.integers(1, 60))
    counts = [int(x) for x in r.choice([1, 2, 3, 4, 100, 255, 256, 257, 1000, 5000, 8192, 20_001], nbuff)]
    offs = np.concatenate([[0], np.cumsum(counts)])
    N = int(offs[-1])
    g = grads_f32(7100 + case, P, N, 1e-3)
    w0 = weights_f32(7200 + case, N, 0.05)
    shift = [int(x) for x in r.integers(0, 2, nbuff)]

    def pieces(flat):
        return [_placed(flat[int(offs[b]):int(offs[b + 1])], shift[b], "f") for b in range(nbuff)]

    gd, wd = [pieces(x) for x in g], pieces(w0)
    md, vd = torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    plan = ccn.ScatterPlan(counts)
    for t in (1, 2):
        plan.adam(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, t)
        orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    plan.sgd(gd, wd, 0.01)
    orc.sgd_f32(g, w, 0.01)
    plan.close()
    what = f"case {case}: P={P} counts={counts}"
    assert_f32_parity(np.concatenate([host(x) for x in wd]), w, what + " w")
    assert_f32_parity(host(md), m, what + " m")
    assert_f32_parity(host(vd), v, what + " v")
    lplan = ccn.LambPlan([int(x) for x in offs])
    for t in (3, 4):
        lplan.step_scattered(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
        orc.lamb_f32(g, w, m, v, [int(x) for x in offs], 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
    lplan.close()
    assert_f32_parity(host(md), m, what + " lamb m")
    assert_f32_parity(host(vd), v, what + " lamb v")
    got = np.concatenate([host(x) for x in wd])
    assert np.max(np.abs(got.astype(np.float64) - w)) <= FP32_TOL * float(np.max(np.abs(w))), what


def test_lamb_plan_knobs_reject_what_they_do_not_know(ccn):
    """ccn_lamb_plan_tune: unknown knobs and negative values are CCN_EINVAL and change nothing; a spin limit beyond 2^31-1
    is CCN_ERANGE; setting and clearing the two-pass knob between steps gives the oracle's result either way."""
    segs = [0, 8192, 3 * 8192, 3 * 8192 + 777]
    N = segs[-1]
    plan = ccn.LambPlan(segs, knobs={})
    for knob, value, code in [(7, 1, ccn.CCN_EINVAL), (-1, 0, ccn.CCN_EINVAL), (SPIN, -5, ccn.CCN_EINVAL), (SPIN, 1 << 40, ccn.CCN_ERANGE)]:
        with pytest.raises(ccn.CoconetError) as e:
            plan.tune(knob, value)
        assert e.value.code == code, (knob, value)
    g = grads_f32(97, 3, N, 1e-3)
    w0 = weights_f32(97, N, 0.05)
    gd, wd = [dev(x) for x in g], dev(w0)
    md, vd = torch.zeros(N, device=DEV), torch.zeros(N, device=DEV)
    w, m, v = w0.copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    for t, two_pass in ((1, 0), (2, 1), (3, 0)):
        plan.tune(TWO_PASS, two_pass)
        plan.step(gd, wd, md, vd, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
        want = orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, t, 0)
        assert rel_err(plan.norms(), want) < 1e-9, (t, two_pass)
    assert_f32_parity(host(md), m, "knobs m")
    assert_f32_parity(host(vd), v, "knobs v")
    assert ulp_diff_f32(host(wd), w) <= 4
    plan.close()
