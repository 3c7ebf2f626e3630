"""GPU tests of the programs the HIP code-generation target emits: each binary (cross-compiled in-tree by
`make -C coconet_amd/dsl gen`) runs its pipeline on the GPU, re-executes it on the CPU stage by stage with the
fixed-order P-way sum, compares, and prints the reference's "{SZ: ..., Epochs: ..., <step>: ms, Total: ms}" lines."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "coconet_amd", "dsl", "build", "gen")
LINE = re.compile(r"^\{SZ: (\d+), Epochs: (\d+)((?:, \w+: [0-9.eE+-]+)+)\}$")

OWN = ["sgd-fused", "sgd-unfused", "clipsgd-fused", "clipsgd-unfused", "reduction-fused", "reduction-unfused", "adam-fused", "adam-unfused", "adamf16-fused", "lamb-fused", "lamb-unfused"]
REF = ["ref-sgd-ar-c", "ref-sgd-rs-c-ag", "ref-sgd-fuse-rs-c-ag", "ref-adam-ar-c", "ref-adam-rs-c-ag",
       "ref-adam-fuse-rs-c-ag", "ref-lamb-ar-c", "ref-lamb-rs-c-ag", "ref-lamb-fuse-rs-c-ag"]


def as_the_reference_scraper_reads(line):
    """The reference's result scraper quotes the keys of every {...} line and evaluates it as a dict literal
    (experiments/generate-pdf/process_hypercluster_data.py:41-54); the emitted lines must survive that."""
    import ast
    quoted = line.replace("{", '{"').replace(":", '":').replace(",", ',"')
    return {k.strip(): v for k, v in ast.literal_eval(quoted).items()}


def run_program(name, *args):
    exe = os.path.join(GEN, name)
    if not os.path.exists(exe):
        pytest.skip(f"{name} was not built (make -C coconet_amd/dsl gen)")
    r = subprocess.run([exe, *map(str, args)], capture_output=True, text=True, timeout=240)
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
    # sizes 2^10 .. 2^21 with the CPU re-execution switched on
    rows = run_program(name, 2, ranks, 10, 21, 1)
    assert [r[0] for r in rows] == [1 << k for k in range(10, 22)]
    for size, epochs, f in rows:
        assert epochs == 2 and abs(sum(v for k, v in f.items() if k != "Total") - f["Total"]) < 1e-3
    steps = set(rows[0][2]) - {"Total"}
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


def test_unaligned_size_takes_scalar_tail():
    # 2^k sizes never leave a tail; an odd size comes from the explicit bounds path of another program, so run the
    # smallest sweep point with 3 ranks instead: the kernel's n % 4 tail code is covered by N = 2^10 only when
    # buffers are unaligned -- here we simply make sure tiny sizes work
    rows = run_program("adam-fused", 1, 3, 1, 9, 1)
    assert [r[0] for r in rows] == [1 << k for k in range(1, 10)]


@pytest.mark.parametrize("name", ["ref-model-parallel-mm-ar-c", "ref-model-parallel-mm-rs-c-ag",
                                  "ref-model-parallel-ol-mm-fuse-rs-c-ag"])
def test_model_parallel_programs(name):
    """Every schedule of the reference's examples/model-parallel/model-parallel.cpp (the last one has no bias and no
    dropout in its expression): each emitted program checks its GEMM + epilogue against its own CPU re-execution."""
    rows = run_program(name, 2, 8, 1)
    # B in {8, 16}, S = 1024, H = 3072: M = B*S rows, N = 3072
    assert [r[0] for r in rows] == [8 * 1024 * 3072, 16 * 1024 * 3072]
    assert all("MatMulFused" in r[2] for r in rows)


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
