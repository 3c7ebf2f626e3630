"""Writes the small golden fixtures under tests/golden/ (run from the repository root: python tests/golden/make_fixtures.py).

Inputs come from the build's seeded generator (tests/util.py); expected outputs from the CPU oracle after it has
been pinned by tests/test_oracle.py.  The reference itself is never imported or run here: its own fixtures for this
path are formulas (integer patterns, all-ones known answers), which tests/util.py restates.  The fixtures let the GPU
parity tests and the oracle tests detect any drift of either side without the other."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle as orc  # noqa: E402
from util import grads_f32, rng, weights_f32  # noqa: E402


def main():
    out = {}
    # config 1 shape, small: SGD
    P, N = 4, 1027
    g = grads_f32(100, P, N, 1e-2)
    w = weights_f32(100, N, 0.1)
    out["sgd_g"], out["sgd_w0"] = np.stack(g), w.copy()
    orc.sgd_f32(g, w, 0.01)
    out["sgd_w1"] = w
    # config 2 shape, small: 3 Adam steps with the same gradients
    P, N = 8, 1029
    g = grads_f32(101, P, N, 1e-3)
    w, m, v = weights_f32(101, N, 0.05), np.zeros(N, np.float32), np.zeros(N, np.float32)
    out["adam_g"], out["adam_w0"] = np.stack(g), w.copy()
    for t in (1, 2, 3):
        orc.adam_f32(g, w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    out["adam_w3"], out["adam_m3"], out["adam_v3"] = w, m, v
    # config 3 shape, small: fp16 gradients with two planted overflows
    P, N = 8, 515
    g16 = [orc.f32_to_f16(x * np.float32(65536.0)) for x in grads_f32(102, P, N, 1e-3)]
    g16[2][17] = 0x7C00
    g16[5][300] = 0xFE00
    w, m, v = weights_f32(102, N, 0.05), np.zeros(N, np.float32), np.zeros(N, np.float32)
    w16 = np.zeros(N, np.uint16)
    out["mixed_g16"], out["mixed_w0"] = np.stack(g16), w.copy()
    out["mixed_flag"] = np.array([orc.adam_f16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(2.0 ** -16))], np.uint32)
    out["mixed_w1"], out["mixed_m1"], out["mixed_v1"], out["mixed_w16"] = w, m, v, w16
    # config 4 shape, small: LAMB over ragged segments, both scale modes
    P = 4
    segs = np.array([0, 7, 1031, 2048, 5000], np.uint64)
    N = int(segs[-1])
    g = grads_f32(103, P, N, 1e-3)
    out["lamb_g"], out["lamb_segs"] = np.stack(g), segs
    for mode in (0, 1):
        w, m, v = weights_f32(103, N, 0.05), np.zeros(N, np.float32), np.zeros(N, np.float32)
        out["lamb_w0"] = w.copy()
        norms = orc.lamb_f32(g, w, m, v, segs, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, mode)
        out[f"lamb_w1_mode{mode}"], out[f"lamb_norms_mode{mode}"] = w, norms
        out["lamb_m1"], out["lamb_v1"] = m, v
    # config 5 shape, one tile: GEMM + epilogue
    M, Nn, K, nP = 128, 128, 64, 7
    r = rng(104)
    X = orc.f32_to_bf16(r.standard_normal((M, K), dtype=np.float32))
    W = orc.f32_to_bf16(r.standard_normal((K, Nn), dtype=np.float32) * np.float32(0.02))
    parts = [r.standard_normal((M, Nn), dtype=np.float32) for _ in range(nP)]
    bias = r.standard_normal(Nn, dtype=np.float32)
    resid = orc.f32_to_bf16(r.standard_normal((M, Nn), dtype=np.float32))
    o16, of32 = orc.mlp_outproj(X, W, parts, bias, resid, M, Nn, K, 0.1, 0)
    out.update(mlp_X=X, mlp_W=W, mlp_parts=np.stack(parts), mlp_bias=bias, mlp_resid=resid, mlp_out=o16, mlp_out_f32=of32,
               mlp_keep=orc.dropout_mask(0, 0, M * Nn, 0.1))
    np.savez_compressed(os.path.join(HERE, "fixtures.npz"), **out)
    print("wrote", os.path.join(HERE, "fixtures.npz"), {k: v.shape for k, v in out.items()})


def main_16bit():
    """fixtures_16bit.npz: the bfloat16-gradient Adam step and the modified NCCL's mixed-precision LAMB."""
    out = {}
    P, N = 8, 515
    g16 = [orc.f32_to_bf16(x * np.float32(128.0)) for x in grads_f32(105, P, N, 1e-3)]
    g16[1][40] = 0x7F80
    g16[6][511] = 0xFFC0
    w, m, v = weights_f32(105, N, 0.05), np.zeros(N, np.float32), np.zeros(N, np.float32)
    w16 = np.zeros(N, np.uint16)
    out["bf16_g16"], out["bf16_w0"] = np.stack(g16), w.copy()
    out["bf16_flag"] = np.array([orc.adam_bf16g(g16, w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1, np.float32(2.0 ** -7))], np.uint32)
    out["bf16_w1"], out["bf16_m1"], out["bf16_v1"], out["bf16_w16"] = w, m, v, w16
    P = 4
    segs = np.array([0, 7, 1031, 2048, 9000], np.uint64)
    N = int(segs[-1])
    g16 = [orc.f32_to_f16(x) for x in grads_f32(106, P, N, 0.5)]
    w = weights_f32(106, N, 0.05)
    m = weights_f32(107, N, 0.01)
    v = np.abs(weights_f32(108, N, 1e-2)) + np.float32(1e-3)
    hw = np.zeros(N, np.uint16)
    out.update(lamb16_g16=np.stack(g16), lamb16_segs=segs, lamb16_w0=w.copy(), lamb16_m0=m.copy(), lamb16_v0=v.copy())
    out["lamb16_norms"] = orc.lamb_nccl_f16g(g16, w, hw, m, v, segs, 0.01, 0.9, 0.999, 1.0)
    out.update(lamb16_w1=w, lamb16_m1=m, lamb16_v1=v, lamb16_hw=hw)
    np.savez_compressed(os.path.join(HERE, "fixtures_16bit.npz"), **out)
    print("wrote", os.path.join(HERE, "fixtures_16bit.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
    main_16bit()
