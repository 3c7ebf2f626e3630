"""Golden fixtures (tests/golden/fixtures.npz, written by tests/golden/make_fixtures.py).
CPU: the oracle still reproduces them bit for bit.  GPU: the HIP kernels reproduce them without the oracle."""
import os

import numpy as np
import pytest

import oracle as orc

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.npz"))


def test_oracle_reproduces_the_fixtures():
    f = FIX
    w = f["sgd_w0"].copy()
    orc.sgd_f32(list(f["sgd_g"]), w, 0.01)
    assert np.array_equal(w, f["sgd_w1"])
    N = f["adam_w0"].size
    w, m, v = f["adam_w0"].copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
    for t in (1, 2, 3):
        orc.adam_f32([np.ascontiguousarray(x) for x in f["adam_g"]], w, m, v, 1e-3, 0.9, 0.999, 1e-6, t)
    assert np.array_equal(w, f["adam_w3"]) and np.array_equal(m, f["adam_m3"]) and np.array_equal(v, f["adam_v3"])
    N = f["mixed_w0"].size
    w, m, v, w16 = f["mixed_w0"].copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    flag = orc.adam_f16g([np.ascontiguousarray(x) for x in f["mixed_g16"]], w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1,
                         np.float32(2.0 ** -16))
    assert flag == int(f["mixed_flag"][0]) == 1
    assert np.array_equal(w, f["mixed_w1"]) and np.array_equal(w16, f["mixed_w16"])
    for mode in (0, 1):
        N = f["lamb_w0"].size
        w, m, v = f["lamb_w0"].copy(), np.zeros(N, np.float32), np.zeros(N, np.float32)
        norms = orc.lamb_f32([np.ascontiguousarray(x) for x in f["lamb_g"]], w, m, v, f["lamb_segs"], 1e-3, 0.9, 0.999, 1e-6,
                             0.01, 1, mode)
        assert np.array_equal(w, f[f"lamb_w1_mode{mode}"]) and np.array_equal(norms, f[f"lamb_norms_mode{mode}"])
    o16, of32 = orc.mlp_outproj(f["mlp_X"], f["mlp_W"], [np.ascontiguousarray(x) for x in f["mlp_parts"]], f["mlp_bias"],
                                f["mlp_resid"], 128, 128, 64, 0.1, 0)
    assert np.array_equal(o16, f["mlp_out"]) and np.array_equal(orc.dropout_mask(0, 0, 128 * 128, 0.1), f["mlp_keep"])


@pytest.mark.gpu
def test_gpu_reproduces_the_fixtures(ccn):
    import torch
    f = FIX
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    dev16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()
    host = lambda t: (torch.cuda.synchronize(), t.cpu().numpy())[1]
    # SGD, Adam: bit-exact
    w = dev(f["sgd_w0"])
    ccn.sgd_f32([dev(x) for x in f["sgd_g"]], w, w.numel(), 0.01)
    assert np.array_equal(host(w), f["sgd_w1"])
    N = f["adam_w0"].size
    w, m, v = dev(f["adam_w0"]), torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda")
    g = [dev(x) for x in f["adam_g"]]
    for t in (1, 2, 3):
        ccn.adam_f32(g, w, m, v, N, 1e-3, 0.9, 0.999, 1e-6, t)
    assert np.array_equal(host(w), f["adam_w3"]) and np.array_equal(host(m), f["adam_m3"]) and np.array_equal(host(v), f["adam_v3"])
    # mixed precision: state bit-exact, fp16 copy exact, flag exact
    N = f["mixed_w0"].size
    w, m, v = dev(f["mixed_w0"]), torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda")
    w16 = torch.zeros(N, dtype=torch.int16, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    ccn.adam_f16g([dev16(x) for x in f["mixed_g16"]], w, m, v, w16, N, 1e-3, 0.9, 0.999, 1e-6, 1, 2.0 ** -16, flag)
    assert int(host(flag)[0]) == int(f["mixed_flag"][0])
    assert np.array_equal(host(w), f["mixed_w1"]) and np.array_equal(host(m), f["mixed_m1"])
    assert np.array_equal(host(w16).view(np.uint16), f["mixed_w16"])
    # LAMB: m, v bit-exact; norms to 1e-9; w within 1e-6 (float64 sums associate differently)
    for mode in (0, 1):
        N = f["lamb_w0"].size
        w, m, v = dev(f["lamb_w0"]), torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda")
        plan = ccn.LambPlan(f["lamb_segs"].tolist())
        plan.step([dev(x) for x in f["lamb_g"]], w, m, v, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, mode)
        assert np.array_equal(host(m), f["lamb_m1"]) and np.array_equal(host(v), f["lamb_v1"])
        assert np.max(np.abs(plan.norms() / f[f"lamb_norms_mode{mode}"] - 1)) < 1e-9
        want = f[f"lamb_w1_mode{mode}"]
        assert np.max(np.abs(host(w).astype(np.float64) - want)) <= 1e-6 * np.max(np.abs(want))
        plan.close()
    # GEMM + epilogue: mask exact, output within one bf16 ulp
    out = torch.zeros(128, 128, dtype=torch.int16, device="cuda")
    ccn.mlp_outproj_bf16(dev16(f["mlp_X"]), dev16(f["mlp_W"]), [dev(x) for x in f["mlp_parts"]], dev(f["mlp_bias"]),
                         dev16(f["mlp_resid"]), out, 128, 128, 64, 0.1, 0)
    got = host(out).view(np.uint16)
    keep = f["mlp_keep"].reshape(128, 128).astype(bool)
    assert np.array_equal(got[~keep], f["mlp_resid"][~keep])
    key = lambda x: np.where(x.astype(np.int32) & 0x8000, -(x.astype(np.int32) & 0x7fff), x.astype(np.int32))
    assert np.max(np.abs(key(got) - key(f["mlp_out"]))) <= 1


FIX16 = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures_16bit.npz"))


def test_oracle_reproduces_the_16bit_fixtures():
    f = FIX16
    N = f["bf16_w0"].size
    w, m, v, w16 = f["bf16_w0"].copy(), np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(N, np.uint16)
    flag = orc.adam_bf16g([np.ascontiguousarray(x) for x in f["bf16_g16"]], w, m, v, w16, 1e-3, 0.9, 0.999, 1e-6, 1,
                          np.float32(2.0 ** -7))
    assert flag == int(f["bf16_flag"][0]) == 1
    assert np.array_equal(w, f["bf16_w1"]) and np.array_equal(m, f["bf16_m1"]) and np.array_equal(v, f["bf16_v1"])
    assert np.array_equal(w16, f["bf16_w16"])
    w, m, v = f["lamb16_w0"].copy(), f["lamb16_m0"].copy(), f["lamb16_v0"].copy()
    hw = np.zeros(w.size, np.uint16)
    norms = orc.lamb_nccl_f16g([np.ascontiguousarray(x) for x in f["lamb16_g16"]], w, hw, m, v, f["lamb16_segs"], 0.01, 0.9,
                               0.999, 1.0)
    assert np.array_equal(w, f["lamb16_w1"]) and np.array_equal(m, f["lamb16_m1"]) and np.array_equal(v, f["lamb16_v1"])
    assert np.array_equal(hw, f["lamb16_hw"]) and np.array_equal(norms, f["lamb16_norms"])


@pytest.mark.gpu
def test_gpu_reproduces_the_16bit_fixtures(ccn):
    import torch
    f = FIX16
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    dev16 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()
    host = lambda t: (torch.cuda.synchronize(), t.cpu().numpy())[1]
    # bfloat16-gradient Adam: state, bfloat16 copy and flag exact
    N = f["bf16_w0"].size
    w, m, v = dev(f["bf16_w0"]), torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda")
    w16 = torch.zeros(N, dtype=torch.int16, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    ccn.adam_bf16g([dev16(x) for x in f["bf16_g16"]], w, m, v, w16, N, 1e-3, 0.9, 0.999, 1e-6, 1, 2.0 ** -7, flag)
    assert int(host(flag)[0]) == int(f["bf16_flag"][0])
    assert np.array_equal(host(w), f["bf16_w1"]) and np.array_equal(host(m), f["bf16_m1"]) and np.array_equal(host(v), f["bf16_v1"])
    assert np.array_equal(host(w16).view(np.uint16), f["bf16_w16"])
    # mixed-precision LAMB: m, v exact; norms to 1e-6 (fp32 roundings of float64 sums); w within 1e-6; fp16 copy within an ulp
    N = f["lamb16_w0"].size
    w, m, v = dev(f["lamb16_w0"]), dev(f["lamb16_m0"]), dev(f["lamb16_v0"])
    hw = torch.zeros(N, dtype=torch.int16, device="cuda")
    plan = ccn.LambPlan(f["lamb16_segs"].tolist())
    plan.step_nccl_f16g([dev16(x) for x in f["lamb16_g16"]], w, hw, m, v, 0.01, 0.9, 0.999, 1.0)
    assert np.array_equal(host(m), f["lamb16_m1"]) and np.array_equal(host(v), f["lamb16_v1"])
    assert np.max(np.abs(plan.norms() / f["lamb16_norms"] - 1)) < 1e-6
    plan.close()
    want = f["lamb16_w1"]
    got = host(w)
    assert np.max(np.abs(got.astype(np.float64) - want)) <= 1e-6 * np.max(np.abs(want))
    assert np.array_equal(host(hw).view(np.uint16), got.astype(np.float16).view(np.uint16))
    d = np.abs(orc.f16_to_f32(host(hw).view(np.uint16)).astype(np.float64) - orc.f16_to_f32(f["lamb16_hw"]))
    assert np.max(d / np.maximum(np.abs(orc.f16_to_f32(f["lamb16_hw"])), 1e-30)) <= 1e-3
