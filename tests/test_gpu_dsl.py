"""GPU tests of the programs the HIP code-generation target emits: each binary (cross-compiled in-tree by
`make -C coconet_amd/dsl gen`) runs its pipeline on the GPU, re-executes it on the CPU stage by stage with the
fixed-order P-way sum, compares, and prints the reference's "{SZ: ..., Epochs: ..., <step>: ms, Total: ms}" lines."""
import os
import re
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "coconet_amd", "dsl", "build", "gen")
LINE = re.compile(r"^\{SZ: (\d+), Epochs: (\d+)((?:, \w+: [0-9.eE+-]+)+)\}$")

OWN = ["sgd-fused", "sgd-unfused", "biasadd-fused", "biasadd-unfused", "biasstage-unfused", "clipsgd-fused", "clipsgd-unfused", "reduction-fused", "reduction-unfused", "adam-fused", "adam-unfused", "adamf16-fused", "lamb-fused", "lamb-unfused"]
REF = ["ref-sgd-ar-c", "ref-sgd-rs-c-ag", "ref-sgd-fuse-rs-c-ag", "ref-adam-ar-c", "ref-adam-rs-c-ag",
       "ref-adam-fuse-rs-c-ag", "ref-lamb-ar-c", "ref-lamb-rs-c-ag", "ref-lamb-fuse-rs-c-ag"]


def as_the_reference_scraper_reads(line):
    """The reference's result scraper quotes the keys of every {...} line and evaluates it as a dict literal
    (experiments/generate-pdf/process_hypercluster_data.py:41-54); the emitted lines must survive that."""
    import ast
    quoted = line.replace("{", '{"').replace(":", '":').replace(",", ',"')
    return {k.strip(): v for k, v in ast.literal_eval(quoted).items()}


def run_raw(name, *args, env=None):
    exe = os.path.join(GEN, name)
    if not os.path.exists(exe):
        pytest.skip(f"{name} was not built (make -C coconet_amd/dsl gen)")
    full = dict(os.environ)
    full.update({k: str(v) for k, v in (env or {}).items()})
    return subprocess.run([exe, *map(str, args)], capture_output=True, text=True, timeout=240, env=full)


def run_program(name, *args, env=None):
    r = run_raw(name, *args, env=env)
    assert "do not match" not in r.stdout and "Mismatch" not in r.stdout, r.stdout[-2000:]
    assert r.returncode == 0, (r.returncode, r.stdout[-2000:], r.stderr[-2000:])
    rows = []
    for line in r.stdout.splitlines():
        m = LINE.match(line.strip())
        if m:
            fields = dict(re.findall(r"(\w+): ([0-9.eE+-]+)", m.group(3)))
            rows.append((int(m.group(1)), int(m.group(2)), {k: float(v) for k, v in fields.items()}))
            d = as_the_reference_scraper_reads(line.strip())
            assert d["SZ"] == rows[-1][0] and d["Epochs"] == rows[-1][1] and abs(d["Total"] - rows[-1][2]["Total"]) < 1e-9
    return rows


@pytest.mark.parametrize("name", OWN)
@pytest.mark.parametrize("ranks", [1, 4, 8, 11])
def test_own_programs_check_themselves(name, ranks):
    # sizes 2^10 .. 2^21 with the CPU re-execution switched on (biasadd walks a B x H matrix with B = H = 2^k)
    if name.startswith("bias"):
        rows = run_program(name, 2, ranks, 1, 10, 1)
        assert [r[0] for r in rows] == [1 << (2 * k) for k in range(1, 11)]
    else:
        rows = run_program(name, 2, ranks, 10, 21, 1)
        assert [r[0] for r in rows] == [1 << k for k in range(10, 22)]
    for size, epochs, f in rows:
        assert epochs == 2 and abs(sum(v for k, v in f.items() if k != "Total") - f["Total"]) < 1e-3
    steps = set(rows[0][2]) - {"Total"}
    if name == "biasstage-unfused":     # the [H] update and the [B, H] update are kernels of their own
        assert steps == {"AllReduce", "kernel0", "kernel1"}
    else:
        assert steps == ({"kernel0"} if name.endswith("-fused") else {"AllReduce", "kernel0"})


@pytest.mark.parametrize("name", REF)
def test_programs_emitted_from_the_reference_examples(name):
    """The reference's examples/{sgd,adam,lamb}/*.cpp, compiled unmodified against this front end, every schedule."""
    rows = run_program(name, 2, 4, 10, 20, 1)
    assert len(rows) == 11
    steps = set(rows[0][2]) - {"Total"}
    if "fuse" in name:
        assert steps == {"kernel0"}
    elif "rs-c-ag" in name:
        assert steps == {"ReduceScatter", "kernel0", "AllGather"}
    else:
        assert steps == {"AllReduce", "kernel0"}


@pytest.mark.parametrize("name", ["adam-fused", "adam-unfused", "lamb-fused", "adamf16-fused", "ref-adam-rs-c-ag"])
@pytest.mark.parametrize("n,misalign", [(4099, 0), (4099, 1), (1 << 12, 1), (3, 0), (1, 1)])
def test_odd_sizes_and_unaligned_arrays(name, n, misalign):
    """A size that leaves an n % 4 tail behind the 16-byte packs, and arrays that start 4 bytes (2 for fp16) past a
    16-byte boundary, which take the element-wise instantiation: each program still agrees with its CPU re-execution."""
    rows = run_program(name, 2, 3, 10, 10, 1, env={"CCN_GEN_N": n, "CCN_GEN_MISALIGN": misalign})
    assert [r[0] for r in rows] == [n]


def splitmix_uniform(seed, n):
    """The emitted programs' input stream (ccn_gen::uniform01): splitmix64 of seed + golden * (i + 1), top 24 bits."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + np.uint64(0x9E3779B97F4A7C15) * (np.arange(n, dtype=np.uint64) + np.uint64(1))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return (((z >> np.uint64(40)) + np.uint64(1)).astype(np.float32) * np.float32(2.0 ** -24)).astype(np.float32)


def emitted_inputs(ranks, n, replicated):
    """Inputs as the emitted main() seeds them: the reduced tensor comes first in the examples' argument lists (seed
    1234 + 100 + rank), the other tensors follow with seeds 1234 + 101, 1234 + 102, ..."""
    g = [splitmix_uniform(1234 + 100 + p, n) for p in range(ranks)]
    return g, [splitmix_uniform(1234 + 101 + k, n) for k in range(replicated)]


@pytest.mark.parametrize("schedule", ["ar-c", "rs-c-ag", "fuse-rs-c-ag"])
@pytest.mark.parametrize("n,ranks", [(1 << 16, 4), (4099, 4), (4099, 7), (10, 4), (5, 8)])
def test_emitted_sgd_and_adam_against_the_oracle(tmp_path, schedule, n, ranks):
    """The programs emitted from the reference's examples/sgd and examples/adam, every schedule, against the oracle's
    restatement of the reference checkers on the same inputs, bit for bit.  The rs-c-ag schedules run rank by rank, each
    call updating its slice [DIVUP(n, ranks) * rank, ...) only: the union must be the whole update, also when n is not a
    multiple of the rank count or smaller than it.  lr = 1 and beta = 1/2 are the reference checker's own settings
    (examples/test-adam.cu:84-88); with them the example's w - m_/v_ and (1 - beta2)*g*g equal the checker's
    w - (lr*S3)/S4 and (1 - beta2)*(g*g) exactly."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    env = {"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_lr": 1.0}
    rows = run_program(f"ref-sgd-{schedule}", 1, ranks, 10, 10, 1, env=env)
    assert rows[0][0] == n
    g, (w,) = emitted_inputs(ranks, n, 1)
    orc.sgd_f32(g, w, 1.0)
    got = np.fromfile(f"{prefix}.w.{n}.f32", dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), w.view(np.uint32)), ("sgd", schedule)
    run_program(f"ref-adam-{schedule}", 1, ranks, 10, 10, 1, env=env)
    g, (w, m, v) = emitted_inputs(ranks, n, 3)
    orc.pseudo_adam_f32(g, w, m, v, 1.0, 0.5, 0.5)
    for name, want in (("w", w), ("m", m), ("v", v)):
        got = np.fromfile(f"{prefix}.{name}.{n}.f32", dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), ("adam", schedule, name)


def dumped(prefix, name, count):
    return np.fromfile(f"{prefix}.{name}.{count}.f32", dtype=np.float32)


def same_bits(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("schedule", ["ar-c", "rs-c-ag", "fuse-rs-c-ag"])
@pytest.mark.parametrize("n,ranks", [(4099, 4), (4099, 7), (1 << 16, 4), (1 << 16, 7), (5, 8)])
def test_emitted_lamb_against_the_oracle(tmp_path, schedule, n, ranks):
    """The programs emitted from the reference's examples/lamb/lamb.cpp, every schedule, against the oracle's restatement
    of that text (whole-tensor norms): m and v bit for bit; the norms' float64 sums are added up in another order by the
    two-pass kernels, so the new weights are held to 1e-6.  The AR_C schedule leaves its result in a stage buffer (S8)
    and w untouched, the RS_C_AG ones write it back into w."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    lr, b1, b2, gamma = 0.25, 0.75, 0.5, 0.125
    env = {"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_lr": lr, "CCN_GEN_beta1": b1, "CCN_GEN_beta2": b2, "CCN_GEN_gamma": gamma}
    run_program(f"ref-lamb-{schedule}", 1, ranks, 10, 10, 1, env=env)
    g, (w, m, v) = emitted_inputs(ranks, n, 3)
    want_w, _ = orc.dsl_lamb_f32(g, w, m, v, lr, b1, b2, gamma)
    assert same_bits(dumped(prefix, "m", n), m) and same_bits(dumped(prefix, "v", n), v), schedule
    got_w = dumped(prefix, "S8" if schedule == "ar-c" else "w", n)
    assert np.max(np.abs(got_w - want_w)) <= 1e-6 * np.max(np.abs(want_w)), schedule
    assert np.max(np.abs(got_w - w)) > 1e-3                                  # ... and it is an update, not the old weights


@pytest.mark.parametrize("name", ["lamb-fused", "lamb-unfused"])
@pytest.mark.parametrize("n,ranks", [(4099, 3), (1 << 16, 8)])
def test_own_lamb_program_against_the_oracle(tmp_path, name, n, ranks):
    """The build's own LAMB program (bias corrections and epsilon passed as scalars, one global trust ratio)."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    sc = {"lr": 0.25, "beta1": 0.75, "beta2": 0.5, "eps": 0.015625, "wd": 0.125, "bias1": 0.25, "bias2": 0.5}
    env = {"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix}
    env.update({f"CCN_GEN_{k}": x for k, x in sc.items()})
    run_program(name, 1, ranks, 10, 10, 1, env=env)
    g, (w, m, v) = emitted_inputs(ranks, n, 3)
    want_w, _ = orc.dsl_lamb_f32(g, w, m, v, sc["lr"], sc["beta1"], sc["beta2"], sc["wd"], c1=sc["bias1"], c2=sc["bias2"], eps=sc["eps"])
    assert same_bits(dumped(prefix, "m", n), m) and same_bits(dumped(prefix, "v", n), v)
    assert np.max(np.abs(dumped(prefix, "w", n) - want_w)) <= 1e-6 * np.max(np.abs(want_w))


@pytest.mark.parametrize("n,ranks", [(4099, 4), (1 << 16, 7), (3, 2)])
def test_emitted_fp16_gradient_adam_against_the_oracle(tmp_path, n, ranks):
    """The pipeline of the reference's examples/test-adamf16.cu (fp16 gradients widened and summed in fp32, the DSL
    example's Adam, an fp16 copy of the new weights): its checker there is the loop of examples/test-adam.cu on the widened
    gradients, i.e. the oracle's orc_pseudo_adam_f32.  Bit for bit, the fp16 copy included."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    run_program("adamf16-fused", 1, ranks, 10, 10, 1, env={"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_lr": 1.0})
    g = [orc.f16_to_f32(orc.f32_to_f16(splitmix_uniform(1234 + 100 + p, n))) for p in range(ranks)]
    w, m, v = (splitmix_uniform(1234 + k, n) for k in (101, 103, 104))
    orc.pseudo_adam_f32(g, w, m, v, 1.0, 0.5, 0.5)
    for name, want in (("w", w), ("m", m), ("v", v)):
        assert same_bits(dumped(prefix, name, n), want), name
    assert same_bits(dumped(prefix, "halfw", n), orc.f16_to_f32(orc.f32_to_f16(w)))


@pytest.mark.parametrize("name", ["reduction-fused", "reduction-unfused"])
@pytest.mark.parametrize("n,ranks", [(4099, 4), (1 << 16, 7)])
def test_emitted_reduction_against_a_float64_sum(tmp_path, name, n, ranks):
    """The pipeline of the reference's examples/test-reduction.cu: S1 = w + sum_p g, S2 = the sum of S1 over the tensor,
    w <- w - (damp * S2) * S0.  The whole-tensor sum against numpy's float64 sum rounded to fp32."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    damp = 2.0 ** -18
    run_program(name, 1, ranks, 10, 10, 1, env={"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_damp": damp})
    g, (w,) = emitted_inputs(ranks, n, 1)
    s0 = orc.reduce_f32(g)
    s2 = np.float32(np.sum((w + s0).astype(np.float64)))
    want = w - (np.float32(damp) * s2) * s0
    got = dumped(prefix, "w", n)
    assert np.max(np.abs(got - want)) <= 1e-6 * np.max(np.abs(want)) and np.max(np.abs(got - w)) > 1e-3


@pytest.mark.parametrize("name", ["clipsgd-fused", "clipsgd-unfused"])
def test_emitted_clipped_sgd_against_numpy(tmp_path, name):
    """Ite and comparisons: the summed gradient clipped to [-clip, clip] element by element, bit for bit against numpy's
    select on the oracle's fixed-order sum (uniform inputs on 4 ranks sum to (0, 4]: the upper clip at 2 cuts half)."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    n, ranks, lr, clip = 4099, 4, 0.25, 2.0
    run_program(name, 1, ranks, 10, 10, 1, env={"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_lr": lr, "CCN_GEN_clip": clip})
    g, (w,) = emitted_inputs(ranks, n, 1)
    gs = orc.reduce_f32(g)
    c = np.float32(clip)
    gc = np.where(gs > c, c, np.where(-c > gs, -c, gs)).astype(np.float32)
    assert 0.2 < float((gs > c).mean()) < 0.8
    assert same_bits(dumped(prefix, "w", n), w - np.float32(lr) * gc)


@pytest.mark.parametrize("name", ["biasadd-fused", "biasadd-unfused", "biasstage-unfused"])
def test_emitted_broadcast_programs_against_numpy(tmp_path, name):
    """A [H] operand broadcast over the rows of a [B, H] update, as a tensor (biasadd) and as the value of an Update stage
    over [H] read from the updated tensor's buffer (biasstage): bit for bit against numpy broadcasting.  B = H = 67."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    B = H = 67
    ranks, lr, decay = 3, 0.25, 0.75
    run_program(name, 1, ranks, 1, 1, 1, env={"CCN_GEN_N": B, "CCN_GEN_DUMP": prefix, "CCN_GEN_lr": lr, "CCN_GEN_decay": decay})
    g = [splitmix_uniform(1234 + 100 + p, B * H) for p in range(ranks)]
    w = splitmix_uniform(1234 + 101, B * H)
    b = splitmix_uniform(1234 + 102, H)
    if name.startswith("biasstage"):
        b = b * np.float32(decay)
        assert same_bits(dumped(prefix, "b", H), b)
    gs = orc.reduce_f32(g).reshape(B, H)
    want = w.reshape(B, H) - np.float32(lr) * (gs + b[None, :])
    assert same_bits(dumped(prefix, "w", B * H), want.reshape(-1).astype(np.float32))


@pytest.mark.parametrize("schedule", ["rs-c-ag", "fuse-rs-c-ag"])
@pytest.mark.parametrize("n,ranks,rank", [(10, 4, 0), (10, 4, 3), (4099, 4, 2), (5, 8, 6)])
def test_one_rank_updates_its_slice_only(tmp_path, schedule, n, ranks, rank):
    """The emitted driver takes the reference's (comm_size, rank) pair and runs that rank's share: elements
    [DIVUP(n, ranks) * rank, + DIVUP(n, ranks)) clipped at n (src/codegen.cpp:485-499 of the reference).  With n = 10 on 4
    ranks the slices are [0,3) [3,6) [6,9) [9,10); with 5 elements on 8 ranks, ranks 5 to 7 have nothing to do."""
    import oracle as orc
    prefix = str(tmp_path / "out")
    run_program(f"ref-sgd-{schedule}", 1, ranks, 10, 10, 1,
                env={"CCN_GEN_N": n, "CCN_GEN_DUMP": prefix, "CCN_GEN_ONLY_RANK": rank})
    g, (w0,) = emitted_inputs(ranks, n, 1)
    w = w0.copy()
    orc.sgd_f32(g, w, 0.5)
    per = -(-n // ranks)
    lo, hi = min(per * rank, n), min(per * rank + per, n)
    want = w0.copy()
    want[lo:hi] = w[lo:hi]
    got = np.fromfile(f"{prefix}.w.{n}.f32", dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (lo, hi)


def test_the_emitted_check_catches_a_wrong_result():
    """One device value corrupted by a part in a thousand before the comparison: the program must say so and exit 2."""
    for name in ("sgd-fused", "ref-adam-rs-c-ag", "lamb-fused"):
        r = run_raw(name, 1, 4, 12, 12, 1, env={"CCN_GEN_PERTURB": 1})
        assert r.returncode == 2, (name, r.returncode, r.stdout[-500:])
        assert "Mismatch in" in r.stdout and "Results do not match the CPU re-execution" in r.stdout
        ok = run_raw(name, 1, 4, 12, 12, 1)
        assert ok.returncode == 0 and "do not match" not in ok.stdout


MLP_STEPS = {"ref-model-parallel-mm-ar-c": {"MatMul", "AllReduce", "kernel0"},
             "ref-model-parallel-mm-rs-c-ag": {"MatMul", "ReduceScatter", "kernel0", "AllGather"},
             "ref-model-parallel-ol-mm-fuse-rs-c-ag": {"MatMulFused"},
             "ref-pipeline-parallel-ar-p2p-c": {"MatMul", "AllReduce", "kernel0"},
             "ref-pipeline-parallel-rs-p2p-c-ag": {"MatMul", "ReduceScatter", "kernel0", "AllGather"},
             "ref-pipeline-parallel-ol-rs-fuse-p2p-c-ag": {"MatMulFused"}}


@pytest.mark.parametrize("name", list(MLP_STEPS))
def test_model_parallel_programs(name):
    """Every schedule of the reference's examples/model-parallel/model-parallel.cpp (the last one has no bias and no
    dropout in its expression) and of examples/pipeline-parallel/pipeline-parallel.cpp (product, sum over ranks and
    residual; what that example sends on to the next pipeline stage is this output): the unfused ones run the product, the sum over ranks and the pointwise part as separate
    steps (rank by rank on bands of rows after the ReduceScatter), the overlapped one as the one fused kernel; each
    emitted program checks its result against its own CPU re-execution."""
    rows = run_program(name, 2, 8, 1)
    # B in {8, 16}, S = 1024, H = 3072: M = B*S rows, N = 3072
    assert [r[0] for r in rows] == [8 * 1024 * 3072, 16 * 1024 * 3072]
    assert all(set(r[2]) - {"Total"} == MLP_STEPS[name] for r in rows)


@pytest.mark.parametrize("name", ["mlp-unfused", "mlpepi-fused", "mlp-fused", "ref-model-parallel-mm-rs-c-ag"])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
def test_mlp_programs_under_every_dropout_form(name, mode):
    """Small shapes (one rank's K-slice 256 x 128 . 128 x 1024 on 8 ranks), every schedule, every dropout form of the
    library (CCN_DROPOUT_*): the emitted self-check mirrors the form on the host."""
    rows = run_program(name, 1, 8, 1, env={"CCN_GEN_B": 1, "CCN_GEN_S": 256, "CCN_GEN_H": 1024, "CCN_GEN_DROPOUT_MODE": mode})
    assert [r[0] for r in rows] == [256 * 1024]


@pytest.mark.parametrize("name", ["mlp-unfused", "mlpepi-fused", "mlp-fused", "ref-model-parallel-mm-rs-c-ag"])
def test_mlp_programs_on_shapes_that_are_not_whole_tiles(name):
    """104 rows, 132 columns, a K-slice 17 deep (132 over 8 ranks, rounded up): the library's any-shape kernel behind the
    same calls; the emitted self-check is the same."""
    rows = run_program(name, 1, 8, 1, env={"CCN_GEN_B": 1, "CCN_GEN_S": 104, "CCN_GEN_H": 132})
    assert [r[0] for r in rows] == [104 * 132]


def test_fusing_the_epilogue_into_the_gemm_pays_off_at_config5_size():
    """Benchmark configuration 5 from the DSL (8 ranks, B*S = 8192 rows, H = 8192: one rank's K-slice is 1024 deep) in
    three schedules: the fused kernel writes the product nowhere, the unfused ones write it to memory as fp32 and read
    it back (once more when the sum over ranks is a step of its own)."""
    t = {}
    for name in ("mlp-fused", "mlpepi-fused", "mlp-unfused"):
        t[name] = run_program(name, 5, 8, 0, 2)[0][2]["Total"]
    assert t["mlp-fused"] < 0.9 * t["mlpepi-fused"] and t["mlpepi-fused"] < t["mlp-unfused"], t


def test_fusion_pays_off_at_config2_size():
    """The point of CoCoNet's fusion on one GPU, measured: at N = 2^28, P = 8 the fused schedule streams 56 bytes per
    element, all-reduce-then-update 64 (the summed gradient is written and read again), so once the first, cold epoch
    is left out (sixth argument: untimed warm-up epochs) the fused program must be faster by a clear margin."""
    fused = run_program("adam-fused", 5, 8, 28, 28, 0, 1)[0][2]["Total"]
    unfused = run_program("adam-unfused", 5, 8, 28, 28, 0, 1)[0][2]["Total"]
    assert fused < 0.95 * unfused, (fused, unfused)


def test_warmup_epochs_are_not_timed():
    cold = run_program("sgd-fused", 2, 4, 24, 24, 1)[0]
    warm = run_program("sgd-fused", 2, 4, 24, 24, 1, 2)[0]
    assert cold[1] == warm[1] == 2 and warm[2]["Total"] <= cold[2]["Total"]
