// Small pipelines exercising the front end's rules, one per command-line case; driven by tests/test_dsl.py.
// A case either prints the pipeline (Pipeline::print) and exits 0, or is expected to abort through ASSERT.
#include <dsl.hpp>
#include <pipeline.hpp>

#include <sstream>

using namespace ACCCDSL;

struct AdamParts {
  Variable N{Int32, "N"};
  Variable lr{Float32, "lr"}, beta1{Float32, "beta1"}, beta2{Float32, "beta2"};
  Tensor g{Float32, N, Local, "g"};
  Tensor w{Float32, N, Replicated, "w"}, m{Float32, N, Replicated, "m"}, v{Float32, N, Replicated, "v"};
  Stage g1 = AllReduce(Summation, g);
  Stage m1 = Update(m, beta1 * m + (1 - beta1) * g1);
  Stage v1 = Update(v, beta2 * v + (1 - beta2) * g1 * g1);
  Stage m_ = m1 / beta1;
  Stage v_ = v1 / beta2;
  Stage w1 = Update(w, w - lr * (m_ / v_));
};

int main(int argc, char** argv) {
  const std::string c = argc > 1 ? argv[1] : "";
  if (c == "print_unfused" || c == "print_fused" || c == "print_all_fused") {
    AdamParts a;
    Pipeline pl("adam", {a.g, a.w, a.m, a.v, a.lr, a.beta1, a.beta2}, {a.m1, a.v1, a.w1});
    if (c == "print_fused") pl.fuse({a.m1, a.v1, a.m_, a.v_, a.w1});
    if (c == "print_all_fused") pl.fuse({a.g1, a.m1, a.v1, a.m_, a.v_, a.w1});
    pl.print(std::cout);
    return 0;
  }
  if (c == "fuse_skips_consumer") {
    // g1 -> m1 -> m_ ; fusing {g1, m_} while m1 stays outside makes the fused kernel both feed m1 and read it
    AdamParts a;
    Pipeline pl("adam", {a.g, a.w, a.m, a.v, a.lr, a.beta1, a.beta2}, {a.m1, a.v1, a.w1});
    pl.fuse({a.g1, a.m_});
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "fuse_unreachable") {
    AdamParts a;
    Stage stray = a.w * a.lr;
    Pipeline pl("adam", {a.g, a.w, a.m, a.v, a.lr, a.beta1, a.beta2}, {a.m1, a.v1, a.w1});
    pl.fuse({a.m1, stray});
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "allreduce_of_replicated") {
    Variable N(Int32, "N");
    Tensor w(Float32, N, Replicated, "w");
    Stage s = AllReduce(Summation, w);
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "allgather_of_replicated") {
    Variable N(Int32, "N");
    Tensor w(Float32, N, Replicated, "w");
    Stage s = AllGather(w);
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "local_read_without_collective") {
    Variable N(Int32, "N");
    Variable lr(Float32, "lr");
    Tensor g(Float32, N, Local, "g");
    Tensor w(Float32, N, Replicated, "w");
    Stage g1 = AllReduce(Summation, g);
    Stage w1 = Update(w, w - lr * g1 + g);
    Pipeline pl("bad", {g, w, lr}, {w1});
    std::cout << generateHIP(pl, {});
    return 0;
  }
  if (c == "missing_argument") {
    Variable N(Int32, "N");
    Variable lr(Float32, "lr");
    Tensor g(Float32, N, Local, "g");
    Tensor w(Float32, N, Replicated, "w");
    Stage g1 = AllReduce(Summation, g);
    Stage w1 = Update(w, w - lr * g1);
    Pipeline pl("bad", {g, w}, {w1});   // lr not listed
    std::cout << generateHIP(pl, {});
    return 0;
  }
  if (c == "sliced_layouts") {
    // the RS_C_AG shape: slices flow through the pointwise stages and are gathered at the end
    Variable N(Int32, "N");
    Variable lr(Float32, "lr");
    Tensor g(Float32, N, Local, "g");
    Tensor w(Float32, N, Replicated, "w");
    Stage g1 = ReduceScatter(Summation, g);
    Stage w1 = Scatter(w) - lr * g1;
    Stage w2 = Update(w, AllGather(w1));
    Pipeline pl("sgd", {g, w, lr}, {w2});
    pl.print(std::cout);
    return 0;
  }
  if (c == "dims_mismatch_leading") {
    // y has the FIRST dimension of x only: numpy-style broadcast matches trailing dimensions
    Variable B(Int32, "B"), S(Int32, "S"), H(Int32, "H");
    Tensor x(Float32, {B, S, H}, Replicated, "x");
    Tensor y(Float32, B, Replicated, "y");
    Stage s = x + y;
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "dims_mismatch_same_rank") {
    Variable N(Int32, "N"), M(Int32, "M");
    Tensor x(Float32, N, Replicated, "x");
    Tensor y(Float32, M, Replicated, "y");
    Stage s = x * y;
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "dims_mismatch_in_select") {
    Variable N(Int32, "N"), M(Int32, "M");
    Tensor x(Float32, N, Replicated, "x");
    Tensor y(Float32, M, Replicated, "y");
    Stage s = Ite(x > 0, x, y);
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "update_with_more_dims") {
    Variable B(Int32, "B"), H(Int32, "H");
    Tensor x(Float32, {B, H}, Replicated, "x");
    Tensor b(Float32, H, Replicated, "b");
    Stage s = Update(b, x + b);
    std::cout << "not rejected" << std::endl;
    return 0;
  }
  if (c == "broadcast_bias") {
    // a bias over the last dimension added to a [B, S, H] value outside any MatMul: read modulo its element count
    Variable B(Int32, "B"), S(Int32, "S"), H(Int32, "H");
    Variable lr(Float32, "lr");
    Tensor g(Float32, {B, S, H}, Local, "g");
    Tensor x(Float32, {B, S, H}, Replicated, "x");
    Tensor b(Float32, H, Replicated, "b");
    Tensor sh(Float32, {S, H}, Replicated, "sh");
    Stage g1 = AllReduce(Summation, g);
    Stage x1 = Update(x, x - lr * ((g1 + b) * sh));
    Pipeline pl("bc", {g, x, b, sh, lr}, {x1});
    pl.fuse({g1, x1});
    std::cout << generateHIP(pl, {});
    return 0;
  }
  if (c.rfind("mlp_", 0) == 0) {
    // MatMul pipelines are matched against MatMul -> AllReduce|ReduceScatter -> [+bias] -> [Dropout] -> [+residual] -> [AllGather]
    Variable B(Int32, "B"), S(Int32, "S"), H(Int32, "H");
    Tensor w(Float16, {H, H}, Sliced, "w");
    Tensor b(Float16, H, Replicated, "b");
    Tensor b2(Float16, S, Replicated, "b2");
    Tensor in(Float16, {B, S, H}, Sliced_2, "in");
    Tensor r(Float16, {B, S, H}, Replicated, "r");
    Stage layer = MatMul(in, w);
    Stage sum = AllReduce(Summation, layer);
    std::vector<CodeGenVarBounds> bounds = {CodeGenVarBounds(B, {8}), CodeGenVarBounds(S, {1024}), CodeGenVarBounds(H, {3072})};
    if (c == "mlp_scaled_sum") {            // a product where the chain has a sum
      Stage out = Dropout(sum * b, 0.5) + r;
      Pipeline pl("bad", {w, b, in, r}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_two_dropouts") {
      Stage out = Dropout(Dropout(sum + b, 0.5), 0.5) + r;
      Pipeline pl("bad", {w, b, in, r}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_residual_before_dropout") {
      Stage out = Dropout((sum + b) + r, 0.5);
      Pipeline pl("bad", {w, b, in, r}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_no_collective") {
      Stage out = Dropout(layer, 0.5) + r;
      Pipeline pl("bad", {w, b, in, r}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_operands_swapped") {   // b + sum, r + Dropout(.): the same chain
      Stage out = r + Dropout(b + sum, 0.5);
      Pipeline pl("ok", {w, b, in, r}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_mixed_types") {   // a bfloat16 residual under Float16 operands
      Tensor rb(BFloat16, {B, S, H}, Replicated, "rb");
      Stage out = Dropout(sum + b, 0.5) + rb;
      Pipeline pl("bad", {w, b, in, rb}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_bfloat16") {      // the same chain declared in this build's BFloat16
      Tensor wb(BFloat16, {H, H}, Sliced, "wb");
      Tensor bb(BFloat16, H, Replicated, "bb");
      Tensor inb(BFloat16, {B, S, H}, Sliced_2, "inb");
      Tensor rb(BFloat16, {B, S, H}, Replicated, "rb");
      Stage lb = MatMul(inb, wb);
      Stage sb = AllReduce(Summation, lb);
      Stage out = Dropout(sb + bb, 0.5) + rb;
      Pipeline pl("ok", {wb, bb, inb, rb}, {out});
      std::cout << generateHIP(pl, bounds);
    } else if (c == "mlp_no_bias_no_dropout") {
      Stage out = sum + r;
      Pipeline pl("ok", {w, b, in, r}, {out});
      pl.fuse({sum, out});
      std::cout << generateHIP(pl, bounds);
    } else {
      std::cout << "unknown case" << std::endl;
      return 64;
    }
    return 0;
  }
  if (c == "bad_file") {
    AdamParts a;
    Pipeline pl("adam", {a.g, a.w, a.m, a.v, a.lr, a.beta1, a.beta2}, {a.m1, a.v1, a.w1});
    pl.codegen("/nonexistent-dir/x.cu");
    return 0;
  }
  std::cout << "unknown case" << std::endl;
  return 64;
}
