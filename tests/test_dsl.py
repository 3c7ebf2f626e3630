"""The C++ DSL front end and the HIP code-generation target (CPU side): API conformance with the reference's
example programs, fusion legality, storage classes, the error convention, and the text of emitted kernels."""
import ast
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DSL = os.path.join(ROOT, "coconet_amd", "dsl")
BUILD = os.path.join(DSL, "build")
REF = "/root/reference"


@pytest.fixture(scope="module")
def dsl_build():
    subprocess.check_call(["make", "-C", DSL, "-s", "-j8", "all"])
    return BUILD


def run(exe, *args, cwd=None):
    return subprocess.run([exe, *args], capture_output=True, text=True, cwd=cwd)


def test_storage_classes_and_fusion_groups(dsl_build):
    chk = os.path.join(dsl_build, "ccn-dsl-check")
    unf = run(chk, "print_unfused").stdout
    assert unf.count("kernel ") == 6 and "register" not in unf          # every stage is its own kernel, all in memory
    fused = run(chk, "print_fused").stdout
    assert fused.count("kernel ") == 2
    # reference rule (src/pipeline.hpp:360-387): values consumed only inside the fused kernel stay in registers,
    # Update targets and outputs are memory
    assert "S3 [Replicated, register]" in fused and "S4 [Replicated, register]" in fused
    assert "S0 [Replicated, memory] = AllReduce(g)" in fused
    assert "S5 [Replicated, memory, output] = Update(w" in fused
    allf = run(chk, "print_all_fused").stdout
    assert allf.count("kernel ") == 1 and "S0 [Replicated, register] = AllReduce(g)" in allf
    sl = run(chk, "sliced_layouts").stdout
    assert "S0 [Sliced" in sl and "S1 [Sliced" in sl and "S2 [Replicated, memory, output] = Update(w, AllGather(S1))" in sl


@pytest.mark.parametrize("case,needle", [
    ("fuse_skips_consumer", "fuse:"),               # reference spec hint: tests/fusion-test.cpp:68-83
    ("fuse_unreachable", "not reachable"),          # tests/fusion-test.cpp:34-49
    ("allreduce_of_replicated", "must be Local"),
    ("allgather_of_replicated", "must be Sliced"),
    ("local_read_without_collective", "is Local"),
    ("missing_argument", "not a pipeline argument"),
    # operands of one pointwise operation must have the same dimensions, or trailing ones (src/pipeline.cpp:14-90 of the
    # reference): anything else would make the emitted kernel read an operand past its end
    ("dims_mismatch_leading", "do not match"),
    ("dims_mismatch_same_rank", "do not match"),
    ("dims_mismatch_in_select", "do not match"),
    ("update_with_more_dims", "more dimensions"),
    # a MatMul pipeline that is not MatMul -> AllReduce|ReduceScatter -> [+bias] -> [Dropout] -> [+residual] -> [AllGather]
    # is refused, not lowered to the nearest thing the library has
    ("mlp_scaled_sum", "must have the shape"),
    ("mlp_two_dropouts", "must have the shape"),
    ("mlp_residual_before_dropout", "must have the shape"),
    ("mlp_no_collective", "must have the shape"),
    ("mlp_mixed_types", "one 16-bit type"),
])
def test_invalid_programs_abort_with_a_message(dsl_build, case, needle):
    """Error convention of the reference (src/ast.hpp:33-44): message on stderr, then std::terminate()."""
    r = run(os.path.join(dsl_build, "ccn-dsl-check"), case)
    assert r.returncode != 0 and "not rejected" not in r.stdout
    assert "ASSERT failed" in r.stderr and needle in r.stderr


def test_trailing_dimensions_broadcast(dsl_build):
    """x[B,S,H] op b[H] and op sh[S,H]: the smaller operand is read at element index modulo its own element count, in the
    kernel and in the emitted CPU re-execution (the reference's `%` of src/codegen.cpp:495-496); the full-size operands
    stay plain streamed inputs."""
    r = run(os.path.join(dsl_build, "ccn-dsl-check"), "broadcast_bias")
    assert r.returncode == 0, r.stderr
    text = r.stdout
    assert "s.bc_b[idx % s.bcn_b]" in text and "s.bc_sh[idx % s.bcn_sh]" in text
    assert "const float* bc_b; size_t bcn_b;" in text
    assert "args0.s.bc_b = b;" in text and "args0.s.bcn_b = (size_t)H;" in text and "args0.s.bcn_sh = (size_t)S * H;" in text
    assert "h.b[i0 % h.b.size()]" in text and "h.sh[i0 % h.sh.size()]" in text and "h.x[i0]" in text
    assert "NIN = 1" in text            # x alone is streamed; g comes through the rank fold


def test_broadcast_of_a_stage_value_is_named_after_its_buffer(dsl_build, tmp_path):
    """An Update stage over [H] read by a kernel over [B, H]: the value lives in the updated tensor's buffer, and the
    broadcast pointer is declared, filled and read under that buffer's name (the stage's own name would not compile)."""
    out = tmp_path / "biasstage.hip"
    r = run(os.path.join(dsl_build, "ccn-programs"), "biasstage", "unfused", str(out))
    assert r.returncode == 0, r.stderr
    text = out.read_text()
    assert "const float* bc_b; size_t bcn_b;" in text and "s.bc_b[idx % s.bcn_b]" in text
    assert ".s.bc_b = b;" in text and ".s.bcn_b = (size_t)H;" in text
    assert not re.search(r"bc_S\d", text)
    assert "h.b[i0 % h.b.size()]" in text or "h.S1[i0 % h.S1.size()]" in text


def test_matmul_chain_is_matched_by_structure_and_lowered_by_schedule(dsl_build, tmp_path):
    """The chain may be written with its sums' operands in either order and without bias and dropout; what is emitted
    follows the schedule: separate steps when nothing is fused (the reference emits a cuBLAS call, an all-reduce and
    pointwise kernels, src/codegen.cpp:1058-1136, 4146-4189), one epilogue call when the collective is fused with what
    follows it, one kernel when the MatMul is."""
    chk = os.path.join(dsl_build, "ccn-dsl-check")
    swapped = run(chk, "mlp_operands_swapped")
    assert swapped.returncode == 0, swapped.stderr
    # Float16 tensors (what the reference's example declares) go to the library's IEEE-half calls
    assert "ccn_matmul_f16_f32(X, W, C" in swapped.stdout and "ccn_reduce_f32(tbl__, comm_size, C + off__" in swapped.stdout
    assert "ccn_bias_dropout_residual_f16_ex(C + off__, nullptr, 0, bias, R + off__, out + off__" in swapped.stdout
    assert "ccn_gen::f32_to_f16_bits(" in swapped.stdout and "bf16" not in swapped.stdout.split("int main")[1]
    assert "const float p_drop = (float)0.5" in swapped.stdout
    bf = run(chk, "mlp_bfloat16")        # the same chain declared in BFloat16: the bfloat16 calls
    assert bf.returncode == 0, bf.stderr
    assert "ccn_matmul_bf16_f32(X, W, C" in bf.stdout and "ccn_bias_dropout_residual_ex(C + off__, nullptr, 0" in bf.stdout
    assert "ccn_gen::f32_to_bf16(" in bf.stdout and "_f16_" not in bf.stdout.split("int main")[1]
    plain = run(chk, "mlp_no_bias_no_dropout")
    assert plain.returncode == 0, plain.stderr
    assert "ccn_bias_dropout_residual_f16_ex(C + off__, tbl__, nPartials" in plain.stdout and "ccn_reduce_f32" not in plain.stdout
    assert "hB[i] = 0.0f" in plain.stdout and "CCN_DROPOUT_INVERTED ? 0.0f : 1.0f" in plain.stdout
    prog = os.path.join(dsl_build, "ccn-programs")
    texts = {}
    for name, sched in (("mlp", "unfused"), ("mlp", "fused"), ("mlpepi", "fused")):
        out = tmp_path / f"{name}-{sched}.hip"
        assert run(prog, name, sched, str(out)).returncode == 0
        texts[(name, sched)] = out.read_text()
    assert "ccn_mlp_outproj_bf16_ex(" in texts[("mlp", "fused")] and "ccn_matmul_bf16_f32" not in texts[("mlp", "fused")]
    assert "MatMul: %f, AllReduce: %f, kernel0: %f, Total" in texts[("mlp", "unfused")]
    assert "MatMul: %f, kernel0: %f, Total" in texts[("mlpepi", "fused")]
    # the reference's dropout form on request, at generation time
    env = dict(os.environ, CCN_DSL_DROPOUT="reference")
    out = tmp_path / "ref.hip"
    assert subprocess.run([prog, "mlp", "fused", str(out)], env=env).returncode == 0
    assert 'env_size("CCN_GEN_DROPOUT_MODE", CCN_DROPOUT_REF_DSL)' in out.read_text()
    assert 'env_size("CCN_GEN_DROPOUT_MODE", CCN_DROPOUT_INVERTED)' in texts[("mlp", "fused")]


def test_unwritable_output_reports_and_returns(dsl_build):
    r = run(os.path.join(dsl_build, "ccn-dsl-check"), "bad_file")       # src/pipeline.hpp:656-663
    assert r.returncode == 0 and "Error opening file" in r.stdout


# ---- emitted text --------------------------------------------------------------------------------------------------------
def canon(expr, rename):
    """Expression tree with identifiers renamed and the operands of + and * sorted: equal canon() means equal
    grouping, i.e. the same floating-point result (commuting a single + or * does not change it)."""
    def go(n):
        if isinstance(n, ast.BinOp):
            op = type(n.op).__name__
            a, b = go(n.left), go(n.right)
            if op in ("Add", "Mult"):
                a, b = sorted([a, b], key=repr)
            return (op, a, b)
        if isinstance(n, ast.Call):
            return ("call", go(n.func), tuple(go(a) for a in n.args))
        if isinstance(n, ast.Name):
            return rename.get(n.id, n.id)
        if isinstance(n, ast.Constant):
            return float(n.value)
        if isinstance(n, ast.UnaryOp):
            return ("neg", go(n.operand))
        raise AssertionError(ast.dump(n))
    return go(ast.parse(expr, mode="eval").body)


def emitted_statements(text):
    text = re.sub(r"\bs\.", "", text)
    return dict(re.findall(r"const float (v_S\d+) = (.*);", text))


def test_emitted_expressions_keep_the_users_grouping(dsl_build, tmp_path):
    exe = os.path.join(dsl_build, "ccn-programs")
    out = tmp_path / "adam.hip"
    assert run(exe, "adam", "fused", str(out)).returncode == 0
    st = emitted_statements(out.read_text())
    ren = {"in_m": "m", "in_v": "v", "in_w": "w", "v_S0": "gs", "red": "gs", "v_S1": "m1", "v_S2": "v1", "v_S3": "mh", "v_S4": "vh"}
    assert canon(st["v_S1"], ren) == canon("beta1*m + (1 - beta1)*gs", ren)
    assert canon(st["v_S2"], ren) == canon("beta2*v + ((1 - beta2)*gs)*gs", ren)          # left to right, as the checker
    assert canon(st["v_S2"], ren) != canon("beta2*v + (1 - beta2)*(gs*gs)", ren)
    assert canon(st["v_S5"], ren) == canon("w - (lr*mh)/(sqrtf(vh) + eps)", ren)
    text = out.read_text()
    assert "HAS_RED = true" in text and "ccn_reduce_f32" not in text                       # reduce fused into the kernel
    unf = tmp_path / "adam-u.hip"
    assert run(exe, "adam", "unfused", str(unf)).returncode == 0
    t2 = unf.read_text()
    assert "ccn_reduce_f32(g, comm_size, g[0]" in t2 and "HAS_RED = false" in t2
    assert re.search(r'printf\("\{SZ: %ld, Epochs: %d, AllReduce: %f, kernel0: %f, Total: %f\}', t2)   # reference line format


def test_ite_lowers_to_a_conditional_in_kernel_and_checker(dsl_build, tmp_path):
    """Ite(cond, a, b) prints (cond ? a : b) as the reference's generator does (src/codegen.cpp:660-666), nested
    selects included, in the device body and in the emitted CPU re-execution alike."""
    exe = os.path.join(dsl_build, "ccn-programs")
    out = tmp_path / "clipsgd.hip"
    assert run(exe, "clipsgd", "fused", str(out)).returncode == 0
    text = out.read_text()
    assert "((v_S0 > s.clip) ? s.clip : (((0 - s.clip) > v_S0) ? (0 - s.clip) : v_S0))" in text
    assert "((h.S0[i0] > clip) ? clip : (((0 - clip) > h.S0[i0]) ? (0 - clip) : h.S0[i0]))" in text
    assert "HAS_RED = true" in text


def test_fp16_gradients_are_widened_inside_the_fused_kernel(dsl_build, tmp_path):
    """A Float16 Local tensor (the reference's examples/test-adamf16.cu pipeline) is read as 16-bit patterns by the fused
    kernel and summed in fp32; reducing it outside a fused kernel is refused with a message."""
    exe = os.path.join(dsl_build, "ccn-programs")
    out = tmp_path / "adamf16.hip"
    assert run(exe, "adamf16", "fused", str(out)).returncode == 0
    text = out.read_text()
    assert "using RedT = uint16_t;" in text and "uint16_t* const* g" in text and "fill_uniform_f16(g[p_]" in text
    assert "sizeof(uint16_t)" in text
    # the fp16 copy of the weights: an Update target of type Float16 is stored as halves, output slot 3 of the body
    assert "static constexpr unsigned OUT_F16 = 8u;" in text and "uint16_t* halfw" in text
    assert 'compare("halfw", h.halfw, halfw' in text
    r = run(exe, "adamf16", "unfused", str(tmp_path / "x.hip"))
    assert r.returncode != 0 and "fused schedule only" in r.stderr


def test_reduce_stage_is_a_plain_sum(dsl_build, tmp_path):
    """ReduceStage(stage, Summation) (the S2 loop of the reference's examples/test-reduction.cu:17-19) accumulates the
    values, not their squares, and finishes without a square root; it shares the two-pass lowering with Norm."""
    exe = os.path.join(dsl_build, "ccn-programs")
    out = tmp_path / "reduction.hip"
    assert run(exe, "reduction", "fused", str(out)).returncode == 0
    text = out.read_text()
    assert "acc[0] += (double)(v_S1);" in text and "x_ * x_" not in text
    assert re.search(r"finalize_norms\(partials__, [^;]*, 1, 0u, norms__, stream\)", text)       # one accumulator, no sqrt
    assert "a_ += (double)(h.S1[i0])" in text.replace("(h.S1[i0])", "(h.S1[i0])") and "(float)a_" in text
    lamb = tmp_path / "lamb.hip"
    assert run(exe, "lamb", "fused", str(lamb)).returncode == 0
    assert re.search(r"finalize_norms\(partials__, [^;]*, 2, 3u, norms__, stream\)", lamb.read_text())    # two norms, both sqrt


def test_two_pass_lowering_of_norms(dsl_build, tmp_path):
    exe = os.path.join(dsl_build, "ccn-programs")
    out = tmp_path / "lamb.hip"
    assert run(exe, "lamb", "fused", str(out)).returncode == 0
    text = out.read_text()
    assert "lamb_body0_pass1" in text and "lamb_body0_pass2" in text and "finalize_norms" in text
    p1 = text[text.index("struct lamb_body0_pass1"):text.index("struct lamb_body0_pass2")]
    p2 = text[text.index("struct lamb_body0_pass2"):text.index("void lamb(")]
    assert "NACC = 2" in p1 and p1.count("acc[") == 2 and "out[2]" not in p1       # pass 1 stores m, v only
    assert "NNORM = 2" in p2 and "HAS_RED = false" in p2                            # pass 2 does not re-read gradients
    assert "nrm[1] / nrm[0]" in p2                                                   # wNorm / rNorm


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not present")
def test_reference_examples_compile_unmodified_and_generate(dsl_build, tmp_path):
    """API conformance: the reference's own DSL programs build against these headers from where they lie and every
    schedule produces a program."""
    for ex, schedules in [("sgd", ["AR_C", "RS_C_AG", "fuse_RS_C_AG"]), ("adam", ["AR_C", "RS_C_AG", "fuse_RS_C_AG"]),
                          ("lamb", ["AR_C", "RS_C_AG", "fuse_RS_C_AG"]),
                          ("model-parallel", ["MM_AR_C", "MM_RS_C_AG", "ol_MM_fuse_RS_C_AG"]),
                          ("pipeline-parallel", ["AR_P2P_C", "RS_P2P_C_AG", "ol_RS_fuse_P2P_C_AG"])]:
        exe = os.path.join(dsl_build, "ex-" + ex)
        assert os.path.exists(exe), exe
        for s in schedules:
            r = run(exe, s, cwd=tmp_path)
            assert r.returncode == 0, r.stderr
    made = sorted(f for f in os.listdir(tmp_path) if f.endswith(".hip"))
    assert len(made) == 15 and "adam-fuse-rs-c-ag.hip" in made
    fused = (tmp_path / "adam-fuse-rs-c-ag.hip").read_text()
    assert "HAS_RED = true" in fused and "ccn_memcpy_d2d" not in fused       # RS + compute + AG in one kernel
    unf = (tmp_path / "adam-rs-c-ag.hip").read_text()
    # ReduceScatter, kernel, AllGather, each on the rank's slice: every array moved on by DIVUP(N, comm_size) * rank
    assert "ccn_reduce_f32(tbl__, comm_size, g[0] + off__, cnt__" in unf and "ccn_memcpy_d2d(w + off__, S5 + off__, cnt__" in unf
    assert "n__ = (size_t)N, per__ = DIVUP(n__, (size_t)comm_size), off__ = per__ * (size_t)r_" in unf
    assert "args0.in[0] = m + off__" in unf and "args0.n = cnt__" in unf and "int comm_size, int rank" in unf
    arc = (tmp_path / "adam-ar-c.hip").read_text()
    assert "off__" not in arc and "ccn_reduce_f32(g, comm_size, g[0], (size_t)N" in arc     # Replicated: the whole range
    # the model-parallel example: unfused schedules as separate steps, the overlapped one as the one fused kernel
    mlp = (tmp_path / "model-parallel-mm-ar-c.hip").read_text()
    # (the example declares Float16: the library's IEEE-half calls)
    assert "ccn_matmul_f16_f32" in mlp and "ccn_bias_dropout_residual_f16_ex" in mlp and "p_drop = (float)0.5" in mlp
    assert "ccn_mlp_outproj_" not in mlp and "MatMul: %f, AllReduce: %f, kernel0: %f, Total" in mlp
    rs = (tmp_path / "model-parallel-mm-rs-c-ag.hip").read_text()
    assert "MatMul: %f, ReduceScatter: %f, kernel0: %f, AllGather: %f, Total" in rs and "ccn_memcpy_d2d(out + off__, scOut + off__" in rs
    ol = (tmp_path / "model-parallel-ol-mm-fuse-rs-c-ag.hip").read_text()
    assert "ccn_mlp_outproj_f16_ex" in ol and "MatMulFused: %f" in ol
    # the pipeline-parallel example: the same chain with neither bias nor dropout (every element kept), residual added
    pp = (tmp_path / "pipeline-parallel-ar-p2p-c.hip").read_text()
    assert "MatMul: %f, AllReduce: %f, kernel0: %f, Total" in pp and "ccn_matmul_f16_f32" in pp
    assert "no Dropout in the pipeline" in pp and "hB[i] = 0.0f" in pp and "bias, R + off__" in pp
    pprs = (tmp_path / "pipeline-parallel-rs-p2p-c-ag.hip").read_text()
    assert "MatMul: %f, ReduceScatter: %f, kernel0: %f, AllGather: %f, Total" in pprs
    ppol = (tmp_path / "pipeline-parallel-ol-rs-fuse-p2p-c-ag.hip").read_text()
    assert "ccn_mlp_outproj_f16_ex(X, W, partials.data(), nPartials, bias, R, out" in ppol


@pytest.mark.skipif(not os.path.exists(os.path.join(ROOT, "oracle", "_ref", "ref-adam")), reason="oracle/_ref not built")
def test_expression_grouping_matches_the_reference_generator(dsl_build, tmp_path):
    """Text oracle: the reference's own generator (built from its sources into oracle/_ref) and this target must
    emit expressions with the same grouping for the reference's adam program."""
    ref_dir = tmp_path / "ref"
    ref_dir.mkdir()
    assert run(os.path.join(ROOT, "oracle", "_ref", "ref-adam"), "AR_C", cwd=ref_dir).returncode == 0
    cu = (ref_dir / "adam-ar-c.cu").read_text()
    cu = cu.replace("[i0]", "")
    ref_stmt = dict(re.findall(r"^\s*(\w+) = (.*);$", cu[:cu.index("void adam(")], flags=re.M))
    mine_dir = tmp_path / "mine"
    mine_dir.mkdir()
    assert run(os.path.join(dsl_build, "ex-adam"), "AR_C", cwd=mine_dir).returncode == 0
    st = emitted_statements((mine_dir / "adam-ar-c.hip").read_text())
    mine_ren = {"in_m": "m", "in_v": "v", "in_w": "w", "in_S0": "g", "v_S1": "m", "v_S2": "v", "v_S3": "S3", "v_S4": "S4"}
    assert canon(st["v_S1"], mine_ren) == canon(ref_stmt["m"], {})
    assert canon(st["v_S2"], mine_ren) == canon(ref_stmt["v"], {})
    assert canon(st["v_S3"], mine_ren) == canon(ref_stmt["S3"], {})
    assert canon(st["v_S5"], mine_ren) == canon(ref_stmt["w"], {})


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_emitted_programs_were_cross_compiled(dsl_build):
    """__graft_entry__.build() runs `make gen`; the binaries are what the GPU tests execute."""
    gen = os.path.join(dsl_build, "gen")
    if not os.path.isdir(gen):
        subprocess.check_call(["make", "-C", DSL, "-s", "-j8", "gen"])
    for name in ("sgd-fused", "adam-fused", "adam-unfused", "lamb-fused"):
        assert os.access(os.path.join(gen, name), os.X_OK), name


def test_the_emitted_programs_comparison_catches_a_wrong_value(tmp_path):
    """The host half of the emitted self-check (ccn_gen::compare_host, the reference's eqFloat loop of
    src/codegen.cpp:4421-4581 and examples/header.h:55-62): equal vectors pass, a value off by a part in a thousand is
    reported as a mismatch, at the 1e-6 bar a value off by 3e-6 is too, and one off by 1e-7 is not.  Host code only."""
    src = tmp_path / "cmp.cpp"
    src.write_text(r'''
#include "ccn_codegen_rt.hpp"
int main() {
  std::vector<float> ref(1000), got(1000);
  for (size_t i = 0; i < ref.size(); i++) ref[i] = got[i] = 0.25f + (float)i;
  if (!ccn_gen::compare_host("same", ref, got, 1e-6f)) return 10;
  got[500] = ref[500] * 1.001f;
  if (ccn_gen::compare_host("w", ref, got, 1e-6f)) return 11;
  got[500] = ref[500] * (1.0f + 3e-6f);
  if (ccn_gen::compare_host("w", ref, got, 1e-6f)) return 12;
  if (!ccn_gen::compare_host("w", ref, got, 1e-5f)) return 13;
  got[500] = ref[500] * (1.0f + 1.2e-7f);
  if (!ccn_gen::compare_host("w", ref, got, 1e-6f)) return 14;
  got[500] = ref[500];
  got[7] = std::nanf("");
  if (ccn_gen::compare_host("w", ref, got, 1e-6f)) return 15;
  return 0;
}
''')
    exe = tmp_path / "cmp"
    lib = os.path.join(ROOT, "coconet_amd", "lib")
    subprocess.check_call(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O1", "-std=c++17", "-I", os.path.join(ROOT, "include"),
                           "-I", os.path.join(DSL, "include"), str(src), "-L", lib, "-lcoconet_hip", "-Wl,-rpath," + lib,
                           "-o", str(exe)], stderr=subprocess.DEVNULL)
    r = run(str(exe))
    assert r.returncode == 0, (r.returncode, r.stdout)
    assert r.stdout.count("Mismatch in w at 500") == 2 and "Mismatch in w at 7" in r.stdout
