// Lowering of the model-parallel MLP pipeline (examples/model-parallel/model-parallel.cpp of the reference; the
// programs of examples/pipeline-parallel/pipeline-parallel.cpp are the same chain without bias and dropout, and what
// they hand to the next pipeline stage is the output this rank computes):
//
//   layer = MatMul(in, w);  sum = AllReduce | ReduceScatter (layer);  [sum2 = sum + b;]  [Dropout(., p)]  [+ r | + Scatter(r)]
//   [out = AllGather(.)]
//
// The pipeline's stages are matched against exactly this chain (bias, dropout, residual and the gather are optional, the
// operands of a sum may come in either order, the chain may be cut into stages anywhere); anything else is rejected with
// an ASSERT rather than lowered to something the program did not say.
//
// What is emitted follows the schedule, as the reference's generator does (src/codegen.cpp:1058-1136, 4249-4277):
//   nothing fused (MM_AR_C, MM_RS_C_AG)      MatMul:  ccn_matmul_{f16,bf16}_f32, the product alone, fp32
//                                            AllReduce / ReduceScatter:  ccn_reduce_f32 over the ranks' partial products
//                                            kernel0:  ccn_bias_dropout_residual_ex on the reduced product
//                                            AllGather (after ReduceScatter):  every rank's band of rows copied into place
//   collective fused with what follows it    MatMul, then kernel0 = ccn_bias_dropout_residual_ex with the other ranks'
//                                            partial products as its partial buffers (the reduce happens in the epilogue)
//   MatMul fused or overlapped with the      MatMulFused:  ccn_mlp_outproj_{f16,bf16}_ex, everything in the GEMM's tile
//   collective (ol_MM_fuse_RS_C_AG)          write-back
// After a ReduceScatter the unfused steps run rank by rank on bands of M / comm_size rows (the reference's slices of
// DIVUP(M*N, comm_size) elements, src/codegen.cpp:485-499; the band must be whole rows).
//
// 16-bit tensors keep the type the program declares: Float16 (what the reference's example uses) goes to the library's
// IEEE-half calls, BFloat16 (this build's addition to the element types) to the bfloat16 ones.  The reference
// accumulates the product in fp16 (src/codegen.cpp:1131), this backend in fp32.
// Dropout: standard by default; with CCN_DSL_DROPOUT=reference in the generator's environment the emitted calls ask for
// the reference's form (keep with probability p, no rescale, src/codegen.cpp:634-640).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <set>
#include <sstream>

#include "pipeline.hpp"

namespace ACCCDSL {
using namespace ir;

namespace {
struct Chain {
  NodePtr matmul, in, w, bias, resid, collective;
  bool dropout = false, gathered = false;
  float p_drop = 0.f;
  std::set<const Node*> stagesSeen;
};

const char* kShape =
    "HIP target: a MatMul pipeline must have the shape MatMul -> AllReduce | ReduceScatter -> [+ bias] -> [Dropout] -> "
    "[+ residual] -> [AllGather]";

struct Matcher {
  Chain& c;
  explicit Matcher(Chain& ch) : c(ch) {}

  NodePtr peel(NodePtr n) {
    while (n->kind == Kind::Stage) {
      c.stagesSeen.insert(n.get());
      n = n->args[0];
    }
    return n;
  }
  bool is_add(const NodePtr& n) { return n->kind == Kind::Binary && n->bin == BinOp::Add; }
  bool reduced_product(NodePtr n) {
    n = peel(n);
    if (n->kind != Kind::Collective || (n->coll != CollOp::AllReduce && n->coll != CollOp::ReduceScatter)) return false;
    if (n->red != Summation) return false;
    NodePtr m = peel(n->args[0]);
    if (m->kind != Kind::MatMul || m->args[0]->kind != Kind::Tensor || m->args[1]->kind != Kind::Tensor) return false;
    c.collective = n;
    c.matmul = m;
    c.in = m->args[0];
    c.w = m->args[1];
    return true;
  }
  bool bias_tensor(NodePtr n) {   // one dimension: the product's last
    n = peel(n);
    return n->kind == Kind::Tensor && c.matmul && n->dims.size() == 1 && n->dims[0] == c.matmul->dims.back();
  }
  bool resid_tensor(NodePtr n, NodePtr& out) {   // the product's dimensions, read whole or through Scatter()
    n = peel(n);
    if (n->kind == Kind::Collective && n->coll == CollOp::Scatter) n = peel(n->args[0]);
    if (n->kind != Kind::Tensor || !c.matmul || n->dims != c.matmul->dims) return false;
    out = n;
    return true;
  }
  bool with_bias(NodePtr n) {
    n = peel(n);
    if (reduced_product(n)) return true;
    if (!is_add(n)) return false;
    for (int k = 0; k < 2; k++) {
      if (reduced_product(n->args[k]) && bias_tensor(n->args[1 - k])) {
        c.bias = peel(n->args[1 - k]);
        return true;
      }
    }
    return false;
  }
  bool with_dropout(NodePtr n) {
    n = peel(n);
    if (n->kind == Kind::Dropout) {
      c.dropout = true;
      c.p_drop = n->prob;
      return with_bias(n->args[0]);
    }
    return with_bias(n);
  }
  bool with_resid(NodePtr n) {
    n = peel(n);
    if (is_add(n)) {
      for (int k = 0; k < 2; k++) {
        // the product side first: it sets the dimensions the residual is checked against
        Chain saved = c;
        if (with_dropout(n->args[k]) && resid_tensor(n->args[1 - k], c.resid)) return true;
        c = saved;
      }
    }
    return with_dropout(n);
  }
  bool whole(NodePtr n) {
    n = peel(n);
    if (n->kind == Kind::Collective && n->coll == CollOp::AllGather) {
      c.gathered = true;
      n = peel(n->args[0]);
    }
    return with_resid(n);
  }
};

std::string product(const std::vector<NodePtr>& dims, size_t lo, size_t hi) {
  std::string s;
  for (size_t k = lo; k < hi; k++) s += (s.empty() ? "" : " * ") + dims[k]->name;
  return s.empty() ? "1" : s;
}
}  // namespace

std::string generateMLP(const Pipeline& p, const std::vector<CodeGenVarBounds>& bounds) {
  // ---- the chain, matched structurally from the single output
  int outputs = 0, outStage = -1;
  for (size_t k = 0; k < p.stages().size(); k++)
    if (p.isOutput((int)k)) { outputs++; outStage = (int)k; }
  ASSERT(outputs == 1, kShape << " with one output stage");
  Chain c;
  Matcher m(c);
  ASSERT(m.whole(p.stages()[outStage]), kShape << " (pipeline '" << p.name() << "')");
  for (auto& st : p.stages())
    ASSERT(c.stagesSeen.count(st.get()), kShape << ": stage " << st->name << " is not part of that chain");
  ASSERT(c.in->dims.size() >= 2 && c.w->dims.size() == 2, "MatMul needs [.., K] x [K, N] tensors");
  ASSERT(c.in->dims.back() == c.w->dims[0], "MatMul: the last dimension of '" << c.in->name << "' is not the first of '" << c.w->name << "'");
  const bool scattered = c.collective->coll == CollOp::ReduceScatter;
  ASSERT(!c.gathered || scattered, kShape << ": AllGather of a value that is not Sliced");

  // ---- the schedule: which stages share a kernel
  auto stage_of = [&](const Node* def) {
    for (size_t k = 0; k < p.stages().size(); k++) if (p.stages()[k]->args[0].get() == def) return (int)k;
    return -1;
  };
  std::vector<int> groupOf(p.stages().size(), -1);
  {
    int g = 0;
    for (auto& grp : p.groupsInOrder()) {
      for (int s : grp.stages) groupOf[s] = g;
      g++;
    }
  }
  const int sMat = stage_of(c.matmul.get()), sColl = stage_of(c.collective.get());
  ASSERT(sMat >= 0 && sColl >= 0, kShape << ": MatMul and the collective are stages of their own");
  const bool fusedAll = groupOf[sMat] == groupOf[sColl];
  bool collAlone = true;   // the collective's kernel holds nothing else
  for (size_t k = 0; k < p.stages().size(); k++) collAlone = collAlone && ((int)k == sColl || groupOf[k] != groupOf[sColl]);
  const bool epilogueIsLast = sColl == outStage;   // nothing follows the collective: no bias, dropout or residual stage
  const int level = fusedAll ? 2 : (collAlone && !epilogueIsLast ? 0 : 1);
  const char* env = std::getenv("CCN_DSL_DROPOUT");
  const bool refDropout = env && std::strcmp(env, "reference") == 0;

  std::vector<NodePtr> dimVars;
  auto addDim = [&](const NodePtr& d) {
    for (auto& q : dimVars) if (q == d) return;
    dimVars.push_back(d);
  };
  for (auto& d : c.in->dims) addDim(d);
  for (auto& d : c.w->dims) addDim(d);

  std::vector<std::string> labels;
  if (level == 2) labels = {"MatMulFused"};
  else {
    labels.push_back("MatMul");
    if (level == 0) labels.push_back(scattered ? "ReduceScatter" : "AllReduce");
    labels.push_back("kernel0");
    if (scattered && c.gathered) labels.push_back("AllGather");
  }

  std::ostringstream o;
  o << "// Generated by the coconet_amd HIP target from pipeline \"" << p.name() << "\".  Do not edit.\n";
  o << "// One rank's K-slice of the MLP out-projection.  Schedule: "
    << (level == 2 ? "the product, the sum over the ranks' partial products, bias, dropout and residual in one kernel"
                   : (level == 1 ? "the product, then one kernel for the sum over ranks and what follows it"
                                 : "the product, the sum over ranks and the pointwise part as separate steps"))
    << ".\n";
  o << "// 16-bit tensors keep the program's type (" << (c.in->elem == Float16 ? "Float16: IEEE half" : "BFloat16")
    << "); the product accumulates in fp32.\n";
  o << "// Run:   ./a.out <epochs> [ranks=8] [check=1] [untimed_warmup_epochs=0]\n";
  o << "// Environment: CCN_GEN_<dimension>=<n> replaces the sizes of a dimension variable; CCN_GEN_DROPOUT_MODE=0..3 the\n"
       "//        dropout form (CCN_DROPOUT_* of coconet_hip.h).\n";
  o << "#include \"ccn_codegen_rt.hpp\"\n\n";
  o << "int main(int argc, char** argv) {\n";
  o << "  if (argc < 2) { printf(\"Specify epochs as command arg\"); return 1; }\n";
  o << "  const int epochs = atoi(argv[1]);\n  const int comm_size = argc > 2 ? atoi(argv[2]) : 8;\n";
  o << "  const bool check__ = argc > 3 ? atoi(argv[3]) != 0 : true;\n";
  o << "  const int warmup__ = argc > 4 && atoi(argv[4]) > 0 ? atoi(argv[4]) : 0;\n";
  o << "  if (comm_size < 1 || comm_size > 9) { printf(\"ranks must be 1..9\\n\"); return 1; }\n";
  o << "  const int mode__ = (int)ccn_gen::env_size(\"CCN_GEN_DROPOUT_MODE\", " << (refDropout ? "CCN_DROPOUT_REF_DSL" : "CCN_DROPOUT_INVERTED") << ");\n";
  o << "  CCNCHECK(ccn_init(0));\n  void* stream;\n  CCNCHECK(ccn_stream_create(&stream));\n  bool allOk__ = true;\n";
  std::string ind = "  ";
  int depth = 0;
  for (auto& d : dimVars) {
    const CodeGenVarBounds* b = nullptr;
    for (auto& q : bounds) if (q.var.impl() == d) b = &q;
    o << ind << "for (size_t " << d->name << " : ccn_gen::env_sizes(\"CCN_GEN_" << d->name << "\", {";
    if (b) for (size_t k = 0; k < b->values.size(); k++) o << (k ? ", " : "") << b->values[k];
    else o << "1024";
    o << "})) {\n";
    ind += "  ";
    depth++;
  }
  // the 16-bit type of the program's tensors picks the library's calls and the host-side conversions of the self-check
  const bool half = c.in->elem == Float16;
  ASSERT(c.in->elem == Float16 || c.in->elem == BFloat16, "HIP target: MatMul operands must be Float16 or BFloat16");
  ASSERT(c.w->elem == c.in->elem && (!c.resid || c.resid->elem == c.in->elem),
         "HIP target: the operands and the residual of a MatMul pipeline must have one 16-bit type");
  const std::string cv_to = half ? "ccn_gen::f32_to_f16_bits" : "ccn_gen::f32_to_bf16";
  const std::string cv_from = half ? "ccn_gen::f16_bits_to_f32" : "ccn_gen::bf16_to_f32";
  const std::string fn_fused = half ? "ccn_mlp_outproj_f16_ex" : "ccn_mlp_outproj_bf16_ex";
  const std::string fn_matmul = half ? "ccn_matmul_f16_f32" : "ccn_matmul_bf16_f32";
  const std::string fn_epi = half ? "ccn_bias_dropout_residual_f16_ex" : "ccn_bias_dropout_residual_ex";
  const size_t nd = c.in->dims.size();
  o << ind << "const size_t M = " << product(c.in->dims, 0, nd - 1) << ", Kfull = " << c.in->dims[nd - 1]->name << ", N = "
    << c.w->dims[1]->name << ";\n";
  o << ind << "const size_t K = DIVUP(Kfull, (size_t)comm_size);   // this rank's slice of the reduction dimension\n";
  o << ind << "if (N % 4) { printf(\"skipping N=%zu: the row length must be a multiple of 4\\n\", N); continue; }\n";
  if (level < 2 && scattered)
    o << ind << "if (M % (size_t)comm_size) { printf(\"skipping M=%zu: a rank's slice must be whole rows\\n\", M); continue; }\n";
  o << ind << "const int nPartials = comm_size - 1;   // the other ranks' partial products, resident as fp32 [M,N]\n";
  o << ind << "std::vector<uint16_t> hX(M * K), hW(K * N), hR(M * N);\n";
  o << ind << "std::vector<float> hB(N);\n";
  o << ind << "for (size_t i = 0; i < M * K; i++) hX[i] = " << cv_to << "(2.0f * ccn_gen::uniform01(1234, i) - 1.0f);\n";
  o << ind << "for (size_t i = 0; i < K * N; i++) hW[i] = " << cv_to << "(0.04f * ccn_gen::uniform01(1235, i) - 0.02f);\n";
  o << ind << "for (size_t i = 0; i < M * N; i++) hR[i] = " << cv_to << "(" << (c.resid ? "2.0f * ccn_gen::uniform01(1236, i) - 1.0f" : "0.0f") << ");\n";
  o << ind << "for (size_t i = 0; i < N; i++) hB[i] = " << (c.bias ? "2.0f * ccn_gen::uniform01(1237, i) - 1.0f" : "0.0f") << ";\n";
  o << ind << "uint16_t *X, *W, *R, *out, *scOut = nullptr;\n" << ind << "float *bias, *C = nullptr;\n"
    << ind << "std::vector<float*> partials(nPartials > 0 ? nPartials : 1, nullptr);\n";
  o << ind << "std::vector<std::vector<float>> hP(nPartials);\n";
  o << ind << "CCNCHECK(ccn_malloc((void**)&X, M * K * 2));\n" << ind << "CCNCHECK(ccn_malloc((void**)&W, K * N * 2));\n";
  o << ind << "CCNCHECK(ccn_malloc((void**)&R, M * N * 2));\n" << ind << "CCNCHECK(ccn_malloc((void**)&out, M * N * 2));\n";
  o << ind << "CCNCHECK(ccn_malloc((void**)&bias, N * 4));\n";
  if (level < 2) o << ind << "CCNCHECK(ccn_malloc((void**)&C, M * N * 4));   // the product (and, reduced in place, the sum over ranks)\n";
  if (level < 2 && scattered && c.gathered) o << ind << "CCNCHECK(ccn_malloc((void**)&scOut, M * N * 2));   // the Sliced value the gather reads\n";
  o << ind << "CCNCHECK(ccn_memcpy_h2d(X, hX.data(), M * K * 2, nullptr));\n" << ind << "CCNCHECK(ccn_memcpy_h2d(W, hW.data(), K * N * 2, nullptr));\n";
  o << ind << "CCNCHECK(ccn_memcpy_h2d(R, hR.data(), M * N * 2, nullptr));\n" << ind << "CCNCHECK(ccn_memcpy_h2d(bias, hB.data(), N * 4, nullptr));\n";
  o << ind << "for (int q = 0; q < nPartials; q++) {\n";
  o << ind << "  CCNCHECK(ccn_malloc((void**)&partials[q], M * N * 4));\n";
  o << ind << "  ccn_gen::fill_uniform(partials[q], M * N, 2000 + q, check__ ? &hP[q] : nullptr);\n" << ind << "}\n";
  o << ind << "CCNCHECK(ccn_stream_sync(nullptr));\n";
  for (auto& l : labels) o << ind << "float elapsedTime" << l << " = 0;\n";
  o << ind << "void *start__, *stop__;\n" << ind << "CCNCHECK(ccn_event_create(&start__));\n" << ind << "CCNCHECK(ccn_event_create(&stop__));\n";
  o << ind << "const float p_drop = " << (c.dropout ? "(float)" + std::to_string(c.p_drop) : std::string("mode__ == CCN_DROPOUT_INVERTED ? 0.0f : 1.0f"))
    << ";" << (c.dropout ? "" : "   // no Dropout in the pipeline: every element kept") << "\n";
  o << ind << "const uint64_t seed__ = 0;\n";
  const std::string resid = c.resid ? "R" : "nullptr";
  auto timed = [&](const std::string& label, const std::string& body) {
    o << ind << "  CCNCHECK(ccn_event_record(start__, stream));\n" << body;
    o << ind << "  CCNCHECK(ccn_event_record(stop__, stream));\n";
    o << ind << "  CCNCHECK(ccn_event_elapsed_ms(start__, stop__, &elapsedTime));\n";
    o << ind << "  elapsedTime" << label << " += elapsedTime;\n";
  };
  o << ind << "for (int iter = -warmup__; iter < epochs; iter++) {\n";
  o << ind << "  float elapsedTime;\n";
  o << ind << "  if (iter == 0) {";
  for (auto& l : labels) o << " elapsedTime" << l << " = 0;";
  o << " }\n";
  if (level == 2) {
    timed("MatMulFused", ind + "  CCNCHECK(" + fn_fused + "(X, W, partials.data(), nPartials, bias, " + resid +
                             ", out, (int)M, (int)N, (int)K, p_drop, seed__, mode__, stream));\n");
  } else {
    timed("MatMul", ind + "  CCNCHECK(" + fn_matmul + "(X, W, C, (int)M, (int)N, (int)K, stream));\n");
    // bands of rows: one per rank after a ReduceScatter, the whole output otherwise
    const std::string bands = scattered ? "comm_size" : "1";
    const std::string loop = ind + "  for (int r_ = 0; r_ < " + bands + "; r_++) {\n" + ind + "    const size_t rows__ = M / " + bands +
                             ", row0__ = rows__ * r_, off__ = row0__ * N;\n";
    const std::string dst = (scattered && c.gathered) ? "scOut" : "out";
    if (level == 0) {
      timed(scattered ? "ReduceScatter" : "AllReduce",
            loop + ind + "    const float* tbl__[9];\n" + ind + "    tbl__[0] = C + off__;\n" + ind +
                "    for (int q = 0; q < nPartials; q++) tbl__[1 + q] = partials[q] + off__;\n" + ind +
                "    CCNCHECK(ccn_reduce_f32(tbl__, comm_size, C + off__, rows__ * N, stream));\n" + ind + "  }\n");
      timed("kernel0", loop + ind + "    CCNCHECK(" + fn_epi + "(C + off__, nullptr, 0, bias, " +
                           (c.resid ? "R + off__" : "nullptr") + ", " + dst + " + off__, (int)rows__, (int)N, p_drop, seed__, mode__, row0__, stream));\n" +
                           ind + "  }\n");
    } else {
      timed("kernel0", loop + ind + "    const float* tbl__[8];\n" + ind +
                           "    for (int q = 0; q < nPartials; q++) tbl__[q] = partials[q] + off__;\n" + ind +
                           "    CCNCHECK(" + fn_epi + "(C + off__, tbl__, nPartials, bias, " +
                           (c.resid ? "R + off__" : "nullptr") + ", " + dst + " + off__, (int)rows__, (int)N, p_drop, seed__, mode__, row0__, stream));\n" +
                           ind + "  }\n");
    }
    if (scattered && c.gathered)
      timed("AllGather", loop + ind + "    CCNCHECK(ccn_memcpy_d2d(out + off__, scOut + off__, rows__ * N * 2, stream));\n" + ind + "  }\n");
  }
  o << ind << "  if (check__ && iter == -warmup__) {\n";
  o << ind << "    // CPU re-execution on a few rows: float64 product, then the sum over ranks and the pointwise part in order\n";
  o << ind << "    std::vector<uint16_t> got(M * N);\n";
  o << ind << "    CCNCHECK(ccn_memcpy_d2h(got.data(), out, M * N * 2, nullptr));\n";
  o << ind << "    size_t bad = 0, seen = 0;\n";
  o << ind << "    for (size_t m : std::vector<size_t>{0, 1, M / 2 - 1, M / 2, M - 1}) {\n";
  o << ind << "      for (size_t n = 0; n < N; n++) {\n";
  o << ind << "        double acc = 0.0, mag = 0.0;   // mag: the magnitudes that went into the element, for the tolerance\n";
  o << ind << "        for (size_t k = 0; k < K; k++) {\n";
  o << ind << "          const double x = (double)" << cv_from << "(hX[m * K + k]), w = (double)" << cv_from << "(hW[k * N + n]);\n";
  o << ind << "          acc += x * w;\n" << ind << "          mag += fabs(x * w);\n" << ind << "        }\n";
  o << ind << "        float s = (float)acc;\n";
  o << ind << "        for (int q = 0; q < nPartials; q++) { s = s + hP[q][m * N + n]; mag += fabs((double)hP[q][m * N + n]); }\n";
  o << ind << "        const float r = " << (c.resid ? cv_from + "(hR[m * N + n])" : std::string("0.0f")) << ";\n";
  o << ind << "        const float y = ccn_gen::epilogue_value(s, hB[n], r, p_drop, seed__, m * N + n, mode__, " << (half ? "true" : "false") << ");\n";
  o << ind << "        mag = (mag + fabs((double)hB[n])) * (mode__ == CCN_DROPOUT_INVERTED ? 1.0 / (1.0 - (double)p_drop) : 1.0) + fabs((double)r);\n";
  o << ind << "        const int want = " << cv_to << "(y), have = got[m * N + n];\n";
  o << ind << "        seen++;\n";
  o << ind << "        // the same 16-bit value or its neighbour; where the sum cancels, within what an fp32 sum of these magnitudes may be off\n";
  o << ind << "        const bool near = abs((want & 0x7fff) - (have & 0x7fff)) <= 1 && (!((want ^ have) & 0x8000) || (want & 0x7fff) <= 1);\n";
  o << ind << "        if (!near && !(fabs((double)" << cv_from << "((uint16_t)have) - (double)y) <= 4e-6 * mag)) {\n";
  o << ind << "          if (bad++ < 5) printf(\"Mismatch at [%zu,%zu]: ref 0x%04x computed 0x%04x\\n\", m, n, want, have);\n";
  o << ind << "        }\n      " << ind << "}\n" << ind << "    }\n";
  o << ind << "    if (bad) { printf(\"Results do not match the CPU re-execution (%zu of %zu)\\n\", bad, seen); allOk__ = false; }\n";
  o << ind << "  }\n" << ind << "}\n";
  o << ind << "printf(\"{SZ: %ld, Epochs: %d";
  for (auto& l : labels) o << ", " << l << ": %f";
  o << ", Total: %f}\\n\", (long)(M * N), epochs";
  std::string total;
  for (auto& l : labels) {
    o << ", elapsedTime" << l;
    total += (total.empty() ? "" : " + ") + ("elapsedTime" + l);
  }
  o << ", " << total << ");\n";
  o << ind << "CCNCHECK(ccn_free(X)); CCNCHECK(ccn_free(W)); CCNCHECK(ccn_free(R)); CCNCHECK(ccn_free(out)); CCNCHECK(ccn_free(bias));\n";
  o << ind << "CCNCHECK(ccn_free(C)); CCNCHECK(ccn_free(scOut));\n";
  o << ind << "for (int q = 0; q < nPartials; q++) CCNCHECK(ccn_free(partials[q]));\n";
  o << ind << "CCNCHECK(ccn_event_destroy(start__)); CCNCHECK(ccn_event_destroy(stop__));\n";
  for (int k = 0; k < depth; k++) {
    ind.resize(ind.size() - 2);
    o << ind << "}\n";
  }
  o << "  CCNCHECK(ccn_stream_destroy(stream));\n  return allOk__ ? 0 : 2;\n}\n";
  return o.str();
}

}  // namespace ACCCDSL
