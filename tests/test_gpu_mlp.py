"""GPU parity tests of the model-parallel MLP out-projection (bf16 MFMA GEMM + fused epilogue) and of the
standalone bias/dropout/residual epilogue, against the CPU oracle.

Bars: dropout masks exact; the standalone epilogue is fp32 elementwise work and is bit-exact; the fused GEMM
accumulates K bf16 products in fp32 inside the MFMA (order differs from the oracle's float64 sum), so its
pre-rounding value is bounded by K*2^-24*sum|x||w| and the bf16 output may differ by one bf16 ulp where that
error straddles a rounding boundary.
"""
import numpy as np
import pytest
import torch

import oracle as orc
from util import rng

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bf16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV)


def bf16_host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy().view(np.uint16)


def make_case(seed, M, N, K, nP):
    r = rng(seed)
    X = orc.f32_to_bf16(r.standard_normal((M, K), dtype=np.float32))
    W = orc.f32_to_bf16(r.standard_normal((K, N), dtype=np.float32) * np.float32(0.02))
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, N), dtype=np.float32))
    return X, W, parts, bias, resid


def bf16_ulp_distance(a, b):
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7fff), x)
    return np.abs(key(a) - key(b))


def assert_within_fp32_sum_error(got_bits, want_bits, want_f32, mag, terms):
    """The fused kernel's bar on many outputs: the same bfloat16 or its neighbour, except where the sum cancels (a small
    result of large terms), where the error must stay within what an fp32 sum of `terms` terms of total magnitude `mag`
    may be off by, plus the rounding to bfloat16."""
    d = bf16_ulp_distance(got_bits, want_bits)
    assert (d > 0).mean() < 0.02, f"{(d > 0).mean():.4f} of the outputs differ"
    far = d > 1
    assert far.mean() < 1e-4, f"{far.mean():.6f} of the outputs differ by more than one ulp"
    if far.any():
        err = np.abs(orc.bf16_to_f32(got_bits[far]).astype(np.float64) - want_f32[far])
        ulp = np.abs(want_f32[far]).astype(np.float64) * 2.0 ** -8 + 1e-38
        assert np.all(err <= terms * 2.0 ** -24 * mag[far] + ulp), float(np.max(err / (terms * 2.0 ** -24 * mag[far] + ulp)))
    return d


@pytest.mark.parametrize("M,N,K,nP,p", [(128, 128, 64, 7, 0.1), (256, 384, 192, 7, 0.1), (128, 256, 1024, 3, 0.5),
                                         (384, 128, 128, 0, 0.0), (128, 128, 64, 1, 0.0)])
def test_outproj_against_oracle(ccn, M, N, K, nP, p):
    X, W, parts, bias, resid = make_case(30 + nP, M, N, K, nP)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV),
                         bf16_dev(resid), out, M, N, K, p, 0)
    got = bf16_host(out).reshape(M, N)
    want, want_f32 = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 0)
    # dropout mask: a dropped element is exactly the residual
    keep = orc.dropout_mask(0, 0, M * N, p).reshape(M, N).astype(bool)
    assert np.array_equal(got[~keep], resid[~keep])
    d = bf16_ulp_distance(got, want)
    assert d.max() <= 1, f"max bf16 ulp distance {d.max()}"
    assert (d > 0).mean() < 0.02, f"{(d > 0).mean():.4f} of the outputs differ by one ulp"
    gf = orc.bf16_to_f32(got)
    assert np.max(np.abs(gf - want_f32) / (np.abs(want_f32) + 1.0)) < 2.0 ** -7


@pytest.mark.parametrize("M,N,K,nP,p,mode", [(100, 128, 64, 7, 0.1, None), (128, 132, 64, 2, 0.0, None), (128, 128, 72, 3, 0.3, None),
                                              (1, 4, 1, 0, 0.0, None), (67, 36, 129, 7, 0.5, 1), (300, 260, 200, 8, 0.25, 3),
                                              (130, 64, 31, 1, 0.2, 2)])
def test_outproj_shapes_that_are_not_whole_tiles(ccn, M, N, K, nP, p, mode):
    """Any M and K, N a multiple of 4: the vector-ALU kernel behind the same entry points (the reference's cuBLAS call
    takes any shape), same epilogue, same bar as the matrix-core kernel."""
    X, W, parts, bias, resid = make_case(90 + nP, M, N, K, nP)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV),
                         bf16_dev(resid), out, M, N, K, p, 5, dropout_mode=mode)
    got = bf16_host(out).reshape(M, N)
    want, want_f32 = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 5, mode=mode or 0)
    d = bf16_ulp_distance(got, want)
    assert d.max() <= 1, f"max bf16 ulp distance {d.max()}"
    assert (d > 0).mean() < 0.03, f"{(d > 0).mean():.4f} of the outputs differ by one ulp"
    if mode is None:
        keep = orc.dropout_mask(5, 0, M * N, p).reshape(M, N).astype(bool)
        assert np.array_equal(got[~keep], resid[~keep])


@pytest.mark.parametrize("M,N,K", [(100, 132, 70), (1, 4, 1), (129, 128, 64), (64, 64, 33)])
def test_plain_product_of_any_shape(ccn, M, N, K):
    X, W, _, _, _ = make_case(95, M, N, K, 0)
    Cd = torch.full((M, N), -1.0, device=DEV)
    ccn.matmul_bf16_f32(bf16_dev(X), bf16_dev(W), Cd, M, N, K)
    torch.cuda.synchronize()
    xf, wf = orc.bf16_to_f32(X).astype(np.float64), orc.bf16_to_f32(W).astype(np.float64)
    bound = K * 2.0 ** -24 * (np.abs(xf) @ np.abs(wf))
    assert np.all(np.abs(Cd.cpu().numpy().astype(np.float64) - xf @ wf) <= bound + 1e-30)


def u16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV)


def f16_ulp_distance(a, b):
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7fff), x)
    return np.abs(key(a) - key(b))


@pytest.mark.parametrize("M,N,K,nP,p,mode", [(128, 128, 64, 7, 0.1, 0), (256, 384, 192, 3, 0.3, 0), (128, 256, 1024, 7, 0.5, 1),
                                              (256, 128, 128, 2, 0.25, 2), (128, 128, 64, 1, 0.5, 3), (100, 36, 70, 7, 0.1, 0),
                                              (1, 4, 1, 0, 0.0, 0)])
def test_outproj_in_ieee_half(ccn, M, N, K, nP, p, mode):
    """X, W, resid and out in IEEE half (ccn_mlp_outproj_f16_ex): the element type the reference's model-parallel example
    declares.  Same bar as for bfloat16, with the unit in the last place of a half: the fp32 accumulation order differs
    from the oracle's float64 sum, so an output may land on the neighbouring half where the error straddles a
    rounding boundary."""
    r = rng(130 + nP)
    X = r.standard_normal((M, K)).astype(np.float16).view(np.uint16)
    W = (r.standard_normal((K, N)) * 0.02).astype(np.float16).view(np.uint16)
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = r.standard_normal((M, N)).astype(np.float16).view(np.uint16)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(u16_dev(X), u16_dev(W), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV),
                         u16_dev(resid), out, M, N, K, p, 9, dropout_mode=mode, half=True)
    got = bf16_host(out).reshape(M, N)
    want, want_f32 = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 9, mode=mode, half=True)
    d = f16_ulp_distance(got, want)
    # A half has 3 more mantissa bits than a bfloat16, so the same fp32 error crosses a rounding boundary 8 times as
    # often; and where the dropped-and-scaled sum cancels against the residual the result is small while the error of the
    # fp32 sum is not (a half resolves 6e-8 near zero), so "one ulp" is the bar only away from cancellation.  Everywhere:
    # the error is within what an fp32 sum of K products and nP + 3 terms of these magnitudes may have, plus the rounding
    # to half.
    assert (d > 0).mean() < 0.08, f"{(d > 0).mean():.4f} of the outputs differ"
    assert (d > 1).mean() < 0.002, f"{(d > 1).mean():.5f} of the outputs differ by more than one ulp"
    xf, wf = X.view(np.float16).astype(np.float64), W.view(np.float16).astype(np.float64)
    scale = 1.0 / (1.0 - p) if mode == 0 else 1.0
    mag = (np.abs(xf) @ np.abs(wf) + sum(np.abs(q).astype(np.float64) for q in parts) + np.abs(bias)) * scale \
        + np.abs(resid.view(np.float16).astype(np.float64))
    gf = got.view(np.float16).astype(np.float64)
    ulp = np.spacing(np.abs(want_f32).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(gf - want_f32) <= (K + nP + 4) * 2.0 ** -24 * mag + ulp)
    if mode == 0:
        keep = orc.dropout_mask(9, 0, M * N, p).reshape(M, N).astype(bool)
        assert np.array_equal(got[~keep], resid[~keep])


def test_half_product_and_standalone_epilogue(ccn):
    """ccn_matmul_f16_f32 against float64 within the fp32 accumulation bound, all-ones C == K, and the standalone epilogue
    in half bit for bit against the oracle's per-element routine."""
    M, N, K = 256, 128, 192
    r = rng(140)
    Xh = r.standard_normal((M, K)).astype(np.float16)
    Wh = (r.standard_normal((K, N)) * 0.02).astype(np.float16)
    Cd = torch.full((M, N), -1.0, device=DEV)
    ccn.matmul_bf16_f32(u16_dev(Xh.view(np.uint16)), u16_dev(Wh.view(np.uint16)), Cd, M, N, K, half=True)
    torch.cuda.synchronize()
    xf, wf = Xh.astype(np.float64), Wh.astype(np.float64)
    bound = K * 2.0 ** -24 * (np.abs(xf) @ np.abs(wf))
    assert np.all(np.abs(Cd.cpu().numpy().astype(np.float64) - xf @ wf) <= bound + 1e-30)
    ones = lambda shape: u16_dev(np.ones(shape, np.float16).view(np.uint16))
    ccn.matmul_bf16_f32(ones((M, K)), ones((K, N)), Cd, M, N, K, half=True)
    torch.cuda.synchronize()
    assert torch.all(Cd == K)
    acc = r.standard_normal((M, N), dtype=np.float32)
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(2)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = r.standard_normal((M, N)).astype(np.float16)
    for mode in (0, 1, 2, 3, 3):
        if mode == 3:       # values inside and around [0, 1]: both clamps and the roundings between the two adds matter
            acc, parts, bias = acc * np.float32(0.2), [q * np.float32(0.2) for q in parts], bias * np.float32(0.3)
        out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
        ccn.bias_dropout_residual(torch.from_numpy(acc).to(DEV), [torch.from_numpy(q).to(DEV) for q in parts],
                                  torch.from_numpy(bias).to(DEV), u16_dev(resid.view(np.uint16)), out, M, N, 0.3, 7,
                                  dropout_mode=mode, half=True)
        s = (acc + parts[0]) + parts[1]
        kept = orc.dropout_mask(7, 0, M * N, 0.3).reshape(M, N)
        y = np.array([[orc.epilogue_value(s[i, j], bias[j], np.float32(resid[i, j]), int(kept[i, j]), 0.3, mode, half=True)
                       for j in range(N)] for i in range(M)], np.float32)
        assert np.array_equal(bf16_host(out).reshape(M, N), y.astype(np.float16).view(np.uint16)), mode
        if mode == 3:
            # the reference's half specialisation rounds to half after each saturating add: float16 arithmetic throughout
            # (numpy's, an independent library) gives the same bits, one fp32 sum rounded once does not
            sat = lambda x: np.clip(x, np.float16(0), np.float16(1))
            v = np.where(kept.astype(bool), np.float16(0), s.astype(np.float16))
            assert np.array_equal(y.astype(np.float16), sat(sat(v + bias.astype(np.float16)[None, :]) + resid))
            once = np.array([[orc.epilogue_value(s[i, j], bias[j], np.float32(resid[i, j]), int(kept[i, j]), 0.3, 3)
                              for j in range(N)] for i in range(M)], np.float32).astype(np.float16)
            assert (once != y.astype(np.float16)).any()


def test_outproj_all_ones_known_answer(ccn):
    # the reference's own check at this boundary: all-ones operands give C == K*ranks
    # (nccl-overlap/samples/matmul-allreduce-bias-dropout-layernorm.cu:520-526)
    M, N, K = 256, 256, 128
    ones = lambda shape: orc.f32_to_bf16(np.ones(shape, np.float32))
    parts = [torch.full((M, N), float(K), device=DEV) for _ in range(7)]
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(ones((M, K))), bf16_dev(ones((K, N))), parts, torch.zeros(N, device=DEV), None, out,
                         M, N, K, 0.0, 0)
    assert np.all(orc.bf16_to_f32(bf16_host(out)) == K * 8)


def test_outproj_tile_order_and_indexing(ccn):
    # X = one-hot rows, W = distinct small integers: C[m][n] = W[k(m)][n] exactly, so any transposed or
    # swizzled index in the tile loads shows up as a wrong integer
    M, N, K = 256, 256, 128
    r = rng(40)
    sel = r.integers(0, K, M)
    Xf = np.zeros((M, K), np.float32)
    Xf[np.arange(M), sel] = 1.0
    Wf = r.integers(-64, 64, (K, N)).astype(np.float32)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(orc.f32_to_bf16(Xf)), bf16_dev(orc.f32_to_bf16(Wf)), [], torch.zeros(N, device=DEV), None,
                         out, M, N, K, 0.0, 0)
    assert np.array_equal(orc.bf16_to_f32(bf16_host(out)).reshape(M, N), Wf[sel])


def _awkward_probabilities():
    """Drop probabilities around the places where the kernels' integer form of the keep decision (draw >= ceil(p * 2^24))
    could part from the oracle's float comparison u >= p: multiples of 2^-24 and their float neighbours, the smallest and
    the largest probabilities, and a few arbitrary ones."""
    f = np.float32
    ps = [f(2.0 ** -24), np.nextafter(f(2.0 ** -24), f(1)), np.nextafter(f(2.0 ** -24), f(0)), f(2.0 ** -30),
          f(0.25), np.nextafter(f(0.25), f(1)), np.nextafter(f(0.25), f(0)), f(1.0) - f(2.0 ** -24),
          np.nextafter(f(1.0), f(0)), f(3 * 2.0 ** -24), f(0.1), f(1.0 / 3.0), f(0.999)]
    return [float(x) for x in ps]


@pytest.mark.parametrize("p", _awkward_probabilities())
def test_dropout_decision_matches_the_oracle_for_awkward_probabilities(ccn, p):
    """The mask, element by element: with a zero product, zero bias and a residual of zero, an output element is zero
    exactly where the element was dropped (the inputs are bounded away from zero).  2^20 draws per probability, through
    the stand-alone epilogue and through the fused kernel."""
    M, N, K = 1024, 1024, 64
    acc = np.full((M, N), 1.0, dtype=np.float32)
    zero_bias = np.zeros(N, dtype=np.float32)
    keep = orc.dropout_mask(5, 0, M * N, p).reshape(M, N).astype(bool)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.bias_dropout_residual(torch.from_numpy(acc).to(DEV), [], torch.from_numpy(zero_bias).to(DEV), None, out, M, N, p, 5)
    assert np.array_equal(bf16_host(out).reshape(M, N) != 0, keep)
    # fused kernel: X = 0, so the product is zero and the partial buffer carries the ones
    X = torch.zeros(M, K, dtype=torch.int16, device=DEV)
    W = torch.zeros(K, N, dtype=torch.int16, device=DEV)
    out2 = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(X, W, [torch.from_numpy(acc).to(DEV)], torch.from_numpy(zero_bias).to(DEV), None, out2, M, N, K, p, 5)
    assert np.array_equal(bf16_host(out2).reshape(M, N) != 0, keep)


@pytest.mark.parametrize("M,N,nP,p", [(64, 128, 7, 0.1), (3, 20, 2, 0.3), (1000, 36, 0, 0.0), (17, 4, 7, 0.9)])
def test_standalone_epilogue_bit_exact(ccn, M, N, nP, p):
    r = rng(50 + nP)
    acc = r.standard_normal((M, N), dtype=np.float32)
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, N), dtype=np.float32))
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.bias_dropout_residual(torch.from_numpy(acc).to(DEV), [torch.from_numpy(q).to(DEV) for q in parts],
                              torch.from_numpy(bias).to(DEV), bf16_dev(resid), out, M, N, p, 7)
    # oracle: the same epilogue with the product replaced by acc (K = 0 GEMM + acc as the first partial)
    s = acc.copy()
    for q in parts:
        s = s + q
    t = s + bias[None, :]
    keep = orc.dropout_mask(7, 0, M * N, p).reshape(M, N).astype(bool)
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(p))
    y = np.where(keep, t * scale, np.float32(0)) + orc.bf16_to_f32(resid)
    assert np.array_equal(bf16_host(out).reshape(M, N), orc.f32_to_bf16(y.astype(np.float32)))


def test_outproj_config5_shape_in_ieee_half(ccn):
    """The shape of benchmark configuration 5 with the operands, residual and output in IEEE half: mask exact on sampled
    rows, drop rate over all 2^26 outputs, values within the fp32-sum bound plus the rounding to half."""
    M = N = 8192
    K = 1024
    gen = torch.Generator(device=DEV)
    gen.manual_seed(6)
    X = torch.randn(M, K, device=DEV, generator=gen).to(torch.float16)
    W = (torch.randn(K, N, device=DEV, generator=gen) * 0.02).to(torch.float16)
    parts = [torch.randn(M, N, device=DEV, generator=gen) for _ in range(7)]
    bias = torch.randn(N, device=DEV, generator=gen)
    resid = torch.randn(M, N, device=DEV, generator=gen).to(torch.float16)
    out = torch.empty(M, N, dtype=torch.float16, device=DEV)
    ccn.mlp_outproj_bf16(X, W, parts, bias, resid, out, M, N, K, 0.1, 0, dropout_mode=0, half=True)
    torch.cuda.synchronize()
    rows = [0, 1, 127, 128, 4095, 4096, 8191]
    keep_rows = np.stack([orc.dropout_mask(0, r * N, N, 0.1) for r in rows]).astype(bool)
    xf = X[rows].cpu().numpy().astype(np.float64)
    wf = W.cpu().numpy().astype(np.float64)
    ph = [q[rows].cpu().numpy() for q in parts]
    rh = resid[rows].cpu().numpy()
    got = out[rows].cpu().numpy()
    s = (xf @ wf).astype(np.float32)
    for q in ph:
        s = s + q
    t = s + bias.cpu().numpy()[None, :]
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(0.1))
    y = np.where(keep_rows, t * scale, np.float32(0)) + rh.astype(np.float32)
    assert np.array_equal(got[~keep_rows].view(np.uint16), rh[~keep_rows].view(np.uint16))
    mag = (np.abs(xf) @ np.abs(wf) + sum(np.abs(q).astype(np.float64) for q in ph) + np.abs(bias.cpu().numpy())) * float(scale) \
        + np.abs(rh.astype(np.float64))
    ulp = np.spacing(np.abs(y).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - y) <= (K + 11) * 2.0 ** -24 * mag + ulp)
    d = f16_ulp_distance(got.view(np.uint16), y.astype(np.float16).view(np.uint16))
    assert (d > 1).mean() < 0.002 and (d > 0).mean() < 0.08
    dropped = float((out == resid).float().mean())
    assert abs(dropped - 0.1) < 2e-3


def test_outproj_config5_full_size(ccn):
    """benchmark configuration 5 at full size (8192 x 1024 x 8192, 7 partials, p = 0.1, seed 0).  Checked by the oracle
    itself on every row of three 128-row tile rows (the first, one in the middle, the last: every row position inside a
    tile, so every wavefront and both halves of its walk, over all 64 tile columns), and over the whole output by the
    drop rate (dropped outputs equal the residual, kept ones almost never do)."""
    M = N = 8192
    K = 1024
    gen = torch.Generator(device=DEV)
    gen.manual_seed(5)
    X = torch.randn(M, K, device=DEV, generator=gen).to(torch.bfloat16)
    W = (torch.randn(K, N, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
    parts = [torch.randn(M, N, device=DEV, generator=gen) for _ in range(7)]
    bias = torch.randn(N, device=DEV, generator=gen)
    resid = torch.randn(M, N, device=DEV, generator=gen).to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ccn.mlp_outproj_bf16(X, W, parts, bias, resid, out, M, N, K, 0.1, 0)
    torch.cuda.synchronize()
    rows = np.concatenate([np.arange(0, 128), np.arange(37 * 128, 38 * 128), np.arange(M - 128, M)])
    ridx = torch.from_numpy(rows).to(DEV)
    bits = lambda t: t[ridx].view(torch.int16).cpu().numpy().view(np.uint16)
    Xh, rh, got = bits(X), bits(resid), bits(out)
    Wh = W.view(torch.int16).cpu().numpy().view(np.uint16)
    ph = [q[ridx].cpu().numpy() for q in parts]
    want, want_f32 = orc.mlp_outproj(Xh, Wh, ph, bias.cpu().numpy(), rh, len(rows), N, K, 0.1, 0, row_ids=rows)
    keep_rows = np.stack([orc.dropout_mask(0, int(r) * N, N, 0.1) for r in rows]).astype(bool)
    assert np.array_equal(got[~keep_rows], rh[~keep_rows])                 # mask exact on the sampled rows
    mag = (torch.abs(X[ridx].float()) @ torch.abs(W.float())).cpu().numpy().astype(np.float64)
    mag = (mag + sum(np.abs(q).astype(np.float64) for q in ph) + np.abs(bias.cpu().numpy())) / 0.9 + np.abs(orc.bf16_to_f32(rh))
    d = assert_within_fp32_sum_error(got, want, want_f32, mag, K + 11)
    per_row = (d > 0).reshape(3, 128, N).mean(axis=(0, 2))                 # no row position inside a tile stands out
    assert per_row.max() < 0.03, f"in-tile row {int(per_row.argmax())}: {per_row.max():.4f} of its outputs differ"
    dropped = float((out == resid).float().mean())
    assert abs(dropped - 0.1) < 2e-3


def test_fused_call_takes_8_byte_aligned_residual_and_output(ccn):
    """The 16-bit residual and output of the fused call need 8-byte alignment only (they move a quad of columns at a
    time), as the header says: both 8 bytes off a 16-byte boundary, whole-tile shape (matrix-core kernel) and an odd
    one (any-shape kernel)."""
    for (M, N, K) in [(128, 256, 128), (100, 36, 70)]:
        X, W, parts, bias, resid = make_case(33, M, N, K, 2)
        rbuf = torch.zeros(M * N + 4, dtype=torch.int16, device=DEV)
        obuf = torch.zeros(M * N + 4, dtype=torch.int16, device=DEV)
        rbuf[4:] = bf16_dev(resid).reshape(-1)
        rview, oview = rbuf[4:], obuf[4:]
        assert rview.data_ptr() % 16 == 8 and oview.data_ptr() % 16 == 8
        ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV),
                             rview, oview, M, N, K, 0.2, 4)
        got = bf16_host(oview).reshape(M, N)
        want, _ = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, 0.2, 4)
        d = bf16_ulp_distance(got, want)
        assert d.max() <= 1 and (d > 0).mean() < 0.03
        assert np.array_equal(bf16_host(obuf)[:4], np.zeros(4, np.uint16))     # nothing written in front of the output
        with pytest.raises(ccn.CoconetError) as e:                              # 4 bytes off is refused
            ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), [], torch.from_numpy(bias).to(DEV), None, obuf[2:], M, N, K, 0.0, 0)
        assert e.value.code == ccn.CCN_EINVAL


def test_rows_longer_than_a_buffer_descriptor_spans(ccn):
    """N = 2^21 + 128 (whole tiles, but a row of fp32 partials is longer than the 2 GiB window the matrix-core kernel
    addresses 128 rows through): the entry point hands over to the any-shape kernel.  Oracle on a few rows."""
    M, K = 128, 64
    N = (1 << 21) + 128
    gen = torch.Generator(device=DEV)
    gen.manual_seed(12)
    X = torch.randn(M, K, device=DEV, generator=gen).to(torch.bfloat16)
    W = (torch.randn(K, N, device=DEV, generator=gen) * 0.1).to(torch.bfloat16)
    part = torch.randn(M, N, device=DEV, generator=gen)
    bias = torch.randn(N, device=DEV, generator=gen)
    resid = torch.randn(M, N, device=DEV, generator=gen).to(torch.bfloat16)
    out = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    ccn.mlp_outproj_bf16(X, W, [part], bias, resid, out, M, N, K, 0.1, 3)
    torch.cuda.synchronize()
    rows = np.array([0, 1, 63, 126, 127])
    ridx = torch.from_numpy(rows).to(DEV)
    bits = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)
    want, want_f32 = orc.mlp_outproj(bits(X[ridx]), bits(W), [part[ridx].cpu().numpy()], bias.cpu().numpy(), bits(resid[ridx]),
                                     len(rows), N, K, 0.1, 3, row_ids=rows)
    got = bits(out[ridx])
    mag = (torch.abs(X[ridx].float()) @ torch.abs(W.float())).cpu().numpy().astype(np.float64)
    mag = (mag + np.abs(part[ridx].cpu().numpy()) + np.abs(bias.cpu().numpy())) / 0.9 + np.abs(orc.bf16_to_f32(bits(resid[ridx])))
    assert_within_fp32_sum_error(got, want, want_f32, mag, K + 5)
    keep_rows = np.stack([orc.dropout_mask(3, int(r) * N, N, 0.1) for r in rows]).astype(bool)
    assert np.array_equal(got[~keep_rows], bits(resid[ridx])[~keep_rows])
    dropped = float((out == resid).float().mean())
    assert abs(dropped - 0.1) < 2e-3
    Cd = torch.empty(M, N, device=DEV)                                          # the plain product hands over as well
    ccn.matmul_bf16_f32(X, W, Cd, M, N, K)
    torch.cuda.synchronize()
    ref = X[ridx].double() @ W.double()
    assert float((Cd[ridx].double() - ref).abs().max()) <= K * 2.0 ** -24 * float((X[ridx].double().abs() @ W.double().abs()).max())


@pytest.mark.parametrize("case", range(8))
def test_seeded_random_shapes(ccn, case):
    """Seeded random tile counts, depths, partial counts, drop rates and seeds through the fused kernel (every count of
    partial buffers has an instantiation of its own), without a residual in some cases."""
    r = rng(900 + case)
    M, N, K = 128 * int(r.integers(1, 4)), 128 * int(r.integers(1, 4)), 64 * int(r.integers(1, 6))
    nP = case % 9 if case < 8 else 8
    p = float(r.choice([0.0, 0.1, 0.5]))
    seed = int(r.integers(0, 1 << 40))
    with_resid = case % 3 != 0
    X, W, parts, bias, resid = make_case(950 + case, M, N, K, nP)
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV),
                         bf16_dev(resid) if with_resid else None, out, M, N, K, p, seed)
    got = bf16_host(out).reshape(M, N)
    zero = np.zeros_like(resid)
    want, want_f32 = orc.mlp_outproj(X, W, parts, bias, resid if with_resid else zero, M, N, K, p, seed)
    keep = orc.dropout_mask(seed, 0, M * N, p).reshape(M, N).astype(bool)
    assert np.array_equal(got[~keep], (resid if with_resid else zero)[~keep])
    d = bf16_ulp_distance(got, want)
    assert d.max() <= 1 and (d > 0).mean() < 0.02, f"case {case}: M={M} N={N} K={K} nP={nP} p={p}: {d.max()} {(d > 0).mean():.4f}"


# ---- the reference's dropout forms and the unfused pieces ---------------------------------------------------------------
@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("p", [0.0, 0.1, 1.0])
def test_reference_dropout_forms(ccn, mode, p):
    """Keep with probability p and no rescale (src/codegen.cpp:634-640), the fused kernel's placement of bias and
    residual and its saturating adds (nccl-overlap/.../reduce_kernel.h:192-213): the standalone epilogue bit for bit
    against the oracle, the fused GEMM within its one-ulp bar.  p = 0 keeps nothing, p = 1 everything."""
    M, N, K, nP = 128, 256, 128, 3
    X, W, parts, bias, resid = make_case(70 + mode, M, N, K, nP)
    if mode == 3:       # values inside and around [0, 1] so that both clamps are exercised
        parts = [q * np.float32(0.2) for q in parts]
        bias = bias * np.float32(0.3)
    pd = [torch.from_numpy(q).to(DEV) for q in parts]
    out = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.mlp_outproj_bf16(bf16_dev(X), bf16_dev(W), pd, torch.from_numpy(bias).to(DEV), bf16_dev(resid), out, M, N, K, p, 9,
                         dropout_mode=mode)
    got = bf16_host(out).reshape(M, N)
    want, want_f32 = orc.mlp_outproj(X, W, parts, bias, resid, M, N, K, p, 9, mode=mode)
    d = bf16_ulp_distance(got, want)
    assert d.max() <= 1 and (d > 0).mean() < 0.02
    if mode == 1 and p == 0.0:
        assert np.array_equal(got, resid)                   # nothing kept: the residual alone
    # standalone epilogue on the exact product: bit for bit
    acc = (orc.bf16_to_f32(X).astype(np.float64) @ orc.bf16_to_f32(W).astype(np.float64)).astype(np.float32)
    out2 = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.bias_dropout_residual(torch.from_numpy(acc).to(DEV), pd, torch.from_numpy(bias).to(DEV), bf16_dev(resid), out2, M, N, p, 9,
                              dropout_mode=mode)
    assert np.array_equal(bf16_host(out2).reshape(M, N), want)
    if mode == 3:
        f = orc.bf16_to_f32(want)
        assert f.min() >= 0.0 and f.max() <= 1.0 and (f == 0).any() and (f == 1).any()


def test_reference_dropout_forms_reject_bad_probabilities(ccn):
    M = N = 128
    K = 64
    z16 = torch.zeros(M * N, dtype=torch.int16, device=DEV)
    zf = torch.zeros(N, device=DEV)
    for mode, p, ok in [(0, 1.0, False), (1, 1.0, True), (1, 1.5, False), (2, -0.1, False), (4, 0.1, False)]:
        call = lambda: ccn.mlp_outproj_bf16(z16, z16, [], zf, None, z16, M, N, K, p, 0, dropout_mode=mode)
        if ok:
            call()
        else:
            with pytest.raises(ccn.CoconetError) as e:
                call()
            assert e.value.code == ccn.CCN_EINVAL


def test_epilogue_in_row_bands_draws_the_same_mask(ccn):
    """One rank's slice of the output (a band of rows) through ccn_bias_dropout_residual_ex with first_row: the union of
    the bands is the whole-call result, mask included."""
    M, N, nP, p = 96, 64, 2, 0.4
    r = rng(77)
    acc = r.standard_normal((M, N), dtype=np.float32)
    parts = [r.standard_normal((M, N), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(N, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, N), dtype=np.float32))
    accd, pd, bd, rd = torch.from_numpy(acc).to(DEV), [torch.from_numpy(q).to(DEV) for q in parts], torch.from_numpy(bias).to(DEV), bf16_dev(resid)
    whole = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    ccn.bias_dropout_residual(accd, pd, bd, rd, whole, M, N, p, 5)
    banded = torch.zeros(M, N, dtype=torch.int16, device=DEV)
    for r0 in range(0, M, 32):
        ccn.bias_dropout_residual(accd[r0:r0 + 32], [q[r0:r0 + 32] for q in pd], bd, rd[r0:r0 + 32], banded[r0:r0 + 32], 32, N, p, 5,
                                  dropout_mode=0, first_row=r0)
    assert torch.equal(whole, banded)


def test_plain_product(ccn):
    """ccn_matmul_bf16_f32, the unfused schedule's GEMM: exact on small integers (all-ones gives K, the reference's own
    check at this boundary), fp32-accumulation close to float64 on random operands."""
    M, N, K = 256, 384, 192
    ones = lambda shape: orc.f32_to_bf16(np.ones(shape, np.float32))
    Cd = torch.zeros(M, N, device=DEV)
    ccn.matmul_bf16_f32(bf16_dev(ones((M, K))), bf16_dev(ones((K, N))), Cd, M, N, K)
    torch.cuda.synchronize()
    assert torch.all(Cd == K)
    X, W, _, _, _ = make_case(81, M, N, K, 0)
    ccn.matmul_bf16_f32(bf16_dev(X), bf16_dev(W), Cd, M, N, K)
    torch.cuda.synchronize()
    xf, wf = orc.bf16_to_f32(X).astype(np.float64), orc.bf16_to_f32(W).astype(np.float64)
    ref = xf @ wf
    bound = K * 2.0 ** -24 * (np.abs(xf) @ np.abs(wf))           # fp32 accumulation of K exact products
    assert np.all(np.abs(Cd.cpu().numpy().astype(np.float64) - ref) <= bound + 1e-30)
    with pytest.raises(ccn.CoconetError) as e:
        ccn.matmul_bf16_f32(bf16_dev(X), bf16_dev(W), Cd, M, N - 2, K)   # a quad of columns must stay inside a row
    assert e.value.code == ccn.CCN_ERANGE


@pytest.mark.parametrize("M,N,K,half", [(2048, 4096, 64, False), (4096, 2304, 192, False), (2560, 3328, 320, False), (2048, 4096, 1024, True),
                                        (8192, 1024, 128, False), (4096, 8192, 64, True), (256, 256, 64, False), (768, 1280, 320, False)])
def test_plain_product_on_large_tiles(ccn, M, N, K, half):
    """Whole multiples of 256 rows and columns, at least 128 tiles of 256 x 256 (half of the CUs), take the large-tile kernel
    of the plain product; the last two shapes are fewer tiles and stay on 128 x 128 tiles.  Exact on small integers (a
    one-hot X picks rows of an integer W: any transposed, swizzled or mis-dealt index shows as a wrong integer; all-ones
    gives K, the reference's own check at this boundary), within the fp32-accumulation bound of float64 on random operands.
    Tile counts that do and do not divide into the blocks of 4 x 8 tiles the workgroups are dealt in; K of 2, 4, 6, 10 and
    32 ring steps (whole trips of four and the two left over)."""
    r = rng(300 + M // 256 + N // 256)
    to16 = (lambda a: a.astype(np.float16).view(np.uint16)) if half else (lambda a: orc.f32_to_bf16(a.astype(np.float32)))
    wide = (lambda b: b.view(np.float16).astype(np.float64)) if half else (lambda b: orc.bf16_to_f32(b).astype(np.float64))
    Cd = torch.full((M, N), -7.0, device=DEV)
    sel = r.integers(0, K, M)
    Xf = np.zeros((M, K), np.float32)
    Xf[np.arange(M), sel] = 1.0
    Wf = r.integers(-64, 64, (K, N)).astype(np.float32)
    ccn.matmul_bf16_f32(u16_dev(to16(Xf)), u16_dev(to16(Wf)), Cd, M, N, K, half=half)
    torch.cuda.synchronize()
    assert np.array_equal(Cd.cpu().numpy(), Wf[sel])
    ones = lambda shape: u16_dev(to16(np.ones(shape, np.float32)))
    ccn.matmul_bf16_f32(ones((M, K)), ones((K, N)), Cd, M, N, K, half=half)
    torch.cuda.synchronize()
    assert torch.all(Cd == K)
    X = to16(r.standard_normal((M, K)))
    W = to16(r.standard_normal((K, N)) * 0.02)
    ccn.matmul_bf16_f32(u16_dev(X), u16_dev(W), Cd, M, N, K, half=half)
    torch.cuda.synchronize()
    xf, wf = wide(X), wide(W)
    bound = K * 2.0 ** -24 * (np.abs(xf) @ np.abs(wf))
    assert np.all(np.abs(Cd.cpu().numpy().astype(np.float64) - xf @ wf) <= bound + 1e-30)


def test_plain_product_config5_shape(ccn):
    """8192 x 1024 x 8192 through the large-tile kernel: sampled rows against float64 (every row position inside a tile in
    the first and the last tile row), and a checksum over the whole product: sum_ij C_ij = sum_k (sum_i X_ik)(sum_j W_kj)."""
    M = N = 8192
    K = 1024
    gen = torch.Generator(device=DEV)
    gen.manual_seed(15)
    X = torch.randn(M, K, device=DEV, generator=gen).to(torch.bfloat16)
    W = (torch.randn(K, N, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
    Cd = torch.empty(M, N, device=DEV)
    ccn.matmul_bf16_f32(X, W, Cd, M, N, K)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, 256), torch.arange(M - 256, M)]).to(DEV)
    ref = X[rows].double() @ W.double()
    bound = K * 2.0 ** -24 * (X[rows].double().abs() @ W.double().abs())
    assert bool(((Cd[rows].double() - ref).abs() <= bound + 1e-30).all())
    total = float(Cd.double().sum())
    want = float((X.double().sum(dim=0) * W.double().sum(dim=1)).sum())
    mag = float((X.double().abs().sum(dim=0) * W.double().abs().sum(dim=1)).sum())
    assert abs(total - want) <= K * 2.0 ** -24 * mag


def test_plain_product_with_w_beyond_2_gib(ccn):
    """W of 1088 x 2^20 16-bit elements is 2.1 GiB, more than one buffer descriptor spans: the large-tile kernel moves the
    descriptor's base with every K-step.  A one-hot X picks rows of an integer W, so every element of C is known exactly
    without a product on the host; the picked k are spread over the first and the last steps."""
    M, N, K = 256, 1 << 20, 1088
    gen = torch.Generator(device=DEV)
    gen.manual_seed(77)
    W = torch.randint(-64, 64, (K, N), device=DEV, generator=gen, dtype=torch.int16).to(torch.bfloat16)
    sel = torch.cat([torch.arange(0, 64), torch.arange(K - 64, K), torch.randint(0, K, (M - 128,), generator=torch.Generator().manual_seed(3))]).to(DEV)
    X = torch.zeros(M, K, device=DEV, dtype=torch.bfloat16)
    X[torch.arange(M, device=DEV), sel] = 1.0
    Cd = torch.full((M, N), -7.0, device=DEV)
    ccn.matmul_bf16_f32(X, W, Cd, M, N, K)
    torch.cuda.synchronize()
    for m0 in range(0, M, 64):   # in pieces: the comparison's temporaries stay small
        assert torch.equal(Cd[m0:m0 + 64], W[sel[m0:m0 + 64]].float())


@pytest.mark.parametrize("M,N,K,half", [(2048, 4096, 192, False), (2560, 3328, 64, True), (768, 1280, 320, False), (256, 384, 192, True),
                                        (100, 36, 70, False), (1, 4, 1, True)])
def test_plain_product_with_16_bit_c(ccn, M, N, K, half):
    """ccn_matmul_bf16 / ccn_matmul_f16 (C in the operands' type, as the reference's emitted GEMM call writes it) on the
    large-tile kernel, on 128 x 128 tiles and on the any-shape kernel: a one-hot X picks rows of an integer W exactly;
    random operands land on the 16-bit neighbour of the float64 product that fp32 accumulation allows (the oracle's
    round-to-nearest-even conversion of the float64 value, one unit in the last place where the fp32 error straddles a
    rounding boundary); and every element equals the fp32-C call's, rounded to nearest even."""
    r = rng(700 + M + N)
    to16 = (lambda a: a.astype(np.float16).view(np.uint16)) if half else (lambda a: orc.f32_to_bf16(a.astype(np.float32)))
    wide = (lambda b: b.view(np.float16).astype(np.float64)) if half else (lambda b: orc.bf16_to_f32(b).astype(np.float64))
    C16 = torch.full((M, N), 0x7e01, dtype=torch.int16, device=DEV)
    sel = r.integers(0, K, M)
    Xf = np.zeros((M, K), np.float32)
    Xf[np.arange(M), sel] = 1.0
    Wf = r.integers(-64, 64, (K, N)).astype(np.float32)
    ccn.matmul_16(u16_dev(to16(Xf)), u16_dev(to16(Wf)), C16, M, N, K, half=half)
    torch.cuda.synchronize()
    assert np.array_equal(wide(bf16_host(C16).reshape(M, N)), Wf[sel].astype(np.float64))
    X = to16(r.standard_normal((M, K)))
    W = to16(r.standard_normal((K, N)) * 0.02)
    C32 = torch.empty(M, N, device=DEV)
    ccn.matmul_16(u16_dev(X), u16_dev(W), C16, M, N, K, half=half)
    ccn.matmul_bf16_f32(u16_dev(X), u16_dev(W), C32, M, N, K, half=half)
    torch.cuda.synchronize()
    got = bf16_host(C16).reshape(M, N)
    c32 = C32.cpu().numpy()
    rounded = c32.astype(np.float16).view(np.uint16) if half else orc.f32_to_bf16(c32)
    assert np.array_equal(got, rounded)
    ref = wide(X) @ wide(W)
    want = ref.astype(np.float16).view(np.uint16) if half else orc.f32_to_bf16(ref.astype(np.float32))
    d = f16_ulp_distance(got, want)
    bound = K * 2.0 ** -24 * (np.abs(wide(X)) @ np.abs(wide(W)))
    ulp = np.maximum(np.abs(wide(want)) * 2.0 ** (-10 if half else -7), 1e-30)
    assert np.all((d <= 1) | (np.abs(wide(got) - ref) <= bound + ulp))
    with pytest.raises(ccn.CoconetError) as e:
        ccn.matmul_16(u16_dev(X), u16_dev(W), C16, M, N + 2, K, half=half)
    assert e.value.code == ccn.CCN_ERANGE
    if M % 256 == 0 and N % 256 == 0:   # a C that is only 8-byte aligned: same values from the kernel that stores 8 bytes per lane
        pad = torch.full((M * N + 4,), 0x7e01, dtype=torch.int16, device=DEV)
        C8 = pad[4:].view(M, N)
        assert C8.data_ptr() % 16 == 8
        ccn.matmul_16(u16_dev(X), u16_dev(W), C8, M, N, K, half=half)
        torch.cuda.synchronize()
        assert torch.equal(C8, C16)
