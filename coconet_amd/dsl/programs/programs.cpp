// DSL programs for the benchmark configurations, written against the CoCoNet API.
//   ccn-programs <program> <schedule> [output.hip]
// program: sgd | biasadd | biasstage | clipsgd | reduction | adam | adamf16 | lamb | mlp | mlpepi
// schedule: unfused | fused (adamf16, mlpepi: fused only)
#include <dsl.hpp>
#include <pipeline.hpp>

#include <cstring>

using namespace ACCCDSL;

// w <- w - lr * sum_p g_p   (benchmark configuration 1)
static void sgd(bool fused, const std::string& out) {
  Variable N(Int32, "N");
  Variable lr(Float32, "lr");
  Tensor w(Float32, N, Replicated, "w");
  Tensor g(Float32, N, Local, "g");
  Stage gsum = AllReduce(Summation, g);
  Stage wnew = Update(w, w - lr * gsum);
  Pipeline pl("sgd", {g, w, lr}, {wnew});
  if (fused) pl.fuse({gsum, wnew});
  pl.codegen(out);
}

// SGD on a matrix of weights with a per-column term added to the summed gradient: b has the last dimension only and is
// broadcast over the rows, numpy-style, as the reference's pointwise stages do (src/pipeline.cpp:14-90)
static void biasadd(bool fused, const std::string& out) {
  Variable B(Int32, "B"), H(Int32, "H");
  Variable lr(Float32, "lr");
  Tensor g(Float32, {B, H}, Local, "g");
  Tensor w(Float32, {B, H}, Replicated, "w");
  Tensor b(Float32, H, Replicated, "b");
  Stage gsum = AllReduce(Summation, g);
  Stage wnew = Update(w, w - lr * (gsum + b));
  Pipeline pl("biasadd", {g, w, b, lr}, {wnew});
  if (fused) pl.fuse({gsum, wnew});
  pl.codegen(out);
}

// The same with the per-column term a STAGE value: an Update over [H] (the bias decays first) that a kernel over [B, H]
// reads, broadcast, from the updated tensor's buffer.  Stages of different dimensions do not fuse: unfused only.
static void biasstage(bool fused, const std::string& out) {
  ASSERT(!fused, "biasstage has an unfused schedule only");
  Variable B(Int32, "B"), H(Int32, "H");
  Variable lr(Float32, "lr"), decay(Float32, "decay");
  Tensor g(Float32, {B, H}, Local, "g");
  Tensor w(Float32, {B, H}, Replicated, "w");
  Tensor b(Float32, H, Replicated, "b");
  Stage gsum = AllReduce(Summation, g);
  Stage bnew = Update(b, b * decay);
  Stage wnew = Update(w, w - lr * (gsum + bnew));
  Pipeline pl("biasstage", {g, w, b, lr, decay}, {bnew, wnew});
  pl.codegen(out);
}

// SGD with the summed gradient clipped to [-clip, clip] element by element: exercises Ite and comparisons
static void clipsgd(bool fused, const std::string& out) {
  Variable N(Int32, "N");
  Variable lr(Float32, "lr"), clip(Float32, "clip");
  Tensor w(Float32, N, Replicated, "w");
  Tensor g(Float32, N, Local, "g");
  Stage gsum = AllReduce(Summation, g);
  Stage gc = Ite(gsum > clip, clip, Ite((0 - clip) > gsum, 0 - clip, gsum));
  Stage wnew = Update(w, w - lr * gc);
  Pipeline pl("clipsgd", {g, w, lr, clip}, {wnew});
  if (fused) pl.fuse({gsum, gc, wnew});
  else pl.fuse({gc, wnew});
  pl.codegen(out);
}

// The pipeline behind the reference's examples/test-reduction.cu: a whole-tensor sum feeds the update.
//   S0 = AllReduce(g); S1 = w + S0; S2 = sum(S1); w <- w - S2 * S0     (S2 scaled by `damp` to keep w finite over epochs)
static void reduction(bool fused, const std::string& out) {
  Variable N(Int32, "N");
  Variable damp(Float32, "damp");
  Tensor w(Float32, N, Replicated, "w");
  Tensor g(Float32, N, Local, "g");
  Stage s0 = AllReduce(Summation, g);
  Stage s1 = w + s0;
  Stage s2 = ReduceStage(s1, Summation);
  Stage s3 = Update(w, w - (damp * s2) * s0);
  Pipeline pl("reduction", {g, w, damp}, {s3});
  if (fused) pl.fuse({s0, s1, s2, s3});
  else pl.fuse({s1, s2, s3});
  pl.codegen(out);
}

// bias-corrected Adam (benchmark configuration 2).  The DSL has no pow(), so the caller passes the two bias
// corrections 1-beta^t as scalars; eps as well.
static void adam(bool fused, const std::string& out) {
  Variable N(Int32, "N");
  Variable lr(Float32, "lr"), b1(Float32, "beta1"), b2(Float32, "beta2"), eps(Float32, "eps");
  Variable c1(Float32, "bias1"), c2(Float32, "bias2");
  Tensor g(Float32, N, Local, "g");
  Tensor w(Float32, N, Replicated, "w"), m(Float32, N, Replicated, "m"), v(Float32, N, Replicated, "v");
  Stage gs = AllReduce(Summation, g);
  Stage mn = Update(m, b1 * m + (1 - b1) * gs);
  Stage vn = Update(v, b2 * v + (1 - b2) * gs * gs);
  Stage mhat = mn / c1;
  Stage vhat = vn / c2;
  Stage wn = Update(w, w - lr * mhat / (Sqrt(vhat) + eps));
  Pipeline pl("adam", {g, w, m, v, lr, b1, b2, eps, c1, c2}, {mn, vn, wn});
  if (fused) pl.fuse({gs, mn, vn, mhat, vhat, wn});
  else pl.fuse({mn, vn, mhat, vhat, wn});
  pl.codegen(out);
}

// The pipeline behind the reference's examples/test-adamf16.cu: fp16 gradients, fp32 state, the DSL example's
// "Adam" (divide by beta, no square root) and an fp16 copy of the new weights, all in one kernel.  A Float16 tensor can
// only be reduced inside a fused kernel.
static void adamf16(bool fused, const std::string& out) {
  ASSERT(fused, "adamf16 has a fused schedule only");
  Variable N(Int32, "N");
  Variable lr(Float32, "lr"), b1(Float32, "beta1"), b2(Float32, "beta2");
  Tensor g(Float16, N, Local, "g");
  Tensor w(Float32, N, Replicated, "w"), m(Float32, N, Replicated, "m"), v(Float32, N, Replicated, "v");
  Stage gs = AllReduce(Summation, g);
  Stage vn = Update(v, b2 * v + (1 - b2) * (gs * gs));
  Stage vh = vn / b2;
  Stage mn = Update(m, b1 * m + (1 - b1) * gs);
  Stage mh = mn / b1;
  Stage wn = Update(w, w - (lr * mh) / vh);
  Tensor hw(Float16, N, Replicated, "halfw");            // the fp16 copy of the weights the reference's kernel also writes
  Stage hwn = Update(hw, Cast(Float16, wn));
  Pipeline pl("adamf16", {g, w, hw, m, v, lr, b1, b2}, {mn, vn, wn, hwn});
  pl.fuse({gs, vn, vh, mn, mh, wn, hwn});
  pl.codegen(out);
}

// LAMB with one global trust ratio (the DSL's Norm is over the whole tensor)
static void lamb(bool fused, const std::string& out) {
  Variable N(Int32, "N");
  Variable lr(Float32, "lr"), b1(Float32, "beta1"), b2(Float32, "beta2"), eps(Float32, "eps"), wd(Float32, "wd");
  Variable c1(Float32, "bias1"), c2(Float32, "bias2");
  Tensor g(Float32, N, Local, "g");
  Tensor w(Float32, N, Replicated, "w"), m(Float32, N, Replicated, "m"), v(Float32, N, Replicated, "v");
  Stage gs = AllReduce(Summation, g);
  Stage mn = Update(m, b1 * m + (1 - b1) * gs);
  Stage vn = Update(v, b2 * v + (1 - b2) * gs * gs);
  Stage r = (mn / c1) / (Sqrt(vn / c2) + eps) + wd * w;
  Stage rn = Norm(r);
  Stage wnorm = Norm(w);
  Stage wn = Update(w, w - lr * (wnorm / rn) * r);
  Pipeline pl("lamb", {g, w, m, v, lr, b1, b2, eps, wd, c1, c2}, {wn});
  if (fused) pl.fuse({gs, mn, vn, r, rn, wnorm, wn});
  else pl.fuse({mn, vn, r, rn, wnorm, wn});
  pl.codegen(out);
}

// The model-parallel MLP out-projection at benchmark configuration 5's shape: with 8 ranks, one rank's K-slice is
// X [8192 x 1024] . W [1024 x 8192] in bfloat16, the other 7 ranks' partial products are resident, then bias,
// dropout(0.1), residual.
//   unfused: MatMul, AllReduce and the pointwise part as separate steps      fused: one kernel
static void mlp(bool fused, bool epilogueOnly, const std::string& out) {
  Variable B(Int32, "B"), S(Int32, "S"), H(Int32, "H");
  Tensor w(BFloat16, {H, H}, Sliced, "w");
  Tensor b(BFloat16, H, Replicated, "b");
  Tensor in(BFloat16, {B, S, H}, Sliced_2, "in");
  Tensor r(BFloat16, {B, S, H}, Replicated, "r");
  Stage layer = MatMul(in, w);
  Stage sum = AllReduce(Summation, layer);
  Stage sum2 = sum + b;
  Stage res = Dropout(sum2, 0.1) + r;
  Pipeline pl("mlp", {w, b, in, r}, {res});
  if (epilogueOnly) pl.fuse({sum, sum2, res});          // the sum over ranks joins the pointwise part; the GEMM stays alone
  else if (fused) pl.fuse({layer, sum, sum2, res});
  pl.codegen(out, {CodeGenVarBounds(B, {8}), CodeGenVarBounds(S, {1024}), CodeGenVarBounds(H, {8192})});
}

int main(int argc, char** argv) {
  if (argc < 3) {
    std::cout << "usage: " << argv[0] << " <sgd|biasadd|biasstage|clipsgd|reduction|adam|adamf16|lamb|mlp|mlpepi> <unfused|fused> [output.hip]" << std::endl;
    return 1;
  }
  const std::string prog = argv[1], sched = argv[2];
  const bool fused = sched == "fused";
  if (!fused && sched != "unfused") { std::cout << "Invalid schedule" << std::endl; return 1; }
  const std::string out = argc > 3 ? argv[3] : prog + "-" + sched + ".hip";
  if (prog == "sgd") sgd(fused, out);
  else if (prog == "biasadd") biasadd(fused, out);
  else if (prog == "biasstage") biasstage(fused, out);
  else if (prog == "clipsgd") clipsgd(fused, out);
  else if (prog == "reduction") reduction(fused, out);
  else if (prog == "adam") adam(fused, out);
  else if (prog == "adamf16") adamf16(fused, out);
  else if (prog == "lamb") lamb(fused, out);
  else if (prog == "mlp") mlp(fused, false, out);
  else if (prog == "mlpepi") mlp(fused, true, out);
  else { std::cout << "Invalid program" << std::endl; return 1; }
  return 0;
}
