/*
 * ccn_oracle.h -- CPU oracle for the fused reduce+update path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a scalar C restatement of the host-side checker loops that the reference
 * (parasailteam/coconet) uses to validate its fused all-reduce + optimizer kernels.  It is the
 * checker for the HIP kernels of this repository and the "cpu_baseline" leg of bench.py; the product
 * library (libcoconet_hip.so) never links, loads or calls it.
 *
 * Conventions shared by every routine:
 *   - "P rank-gradient buffers": g[0..P-1] are P arrays of N elements; the all-reduce of the
 *     reference becomes gs[i] = (((g[0][i] + g[1][i]) + g[2][i]) + ... ) in fp32, p ascending.
 *     (MPI_Allreduce in the reference checkers leaves the order open; the oracle fixes it.)
 *   - compile with -O2 -ffp-contract=off: no fused multiply-add may be formed.
 *   - state (w, m, v) is updated in place; g is read-only.
 *
 * Pin status per routine (what independent evidence the tests hold for it):
 *   orc_reduce_f32        closed form on integers, permutation bound            pinned
 *   orc_sgd_f32           examples/test-sgd.cu:17-18; numpy axpy identity       pinned
 *   orc_sgd_axpby_f32     nccl-overlap/samples/single-process-wX.cu:141        pinned (numpy identity)
 *   orc_pseudo_adam_f32   examples/test-adam.cu:14-38; known answer w=-1/P      pinned
 *   orc_dsl_lamb_f32      examples/lamb/lamb.cpp:20-28 stage by stage (src/codegen.cpp:4421-4581 re-executes that way);
 *                         all-ones closed form w1 = 1 - lr, independent float64 numpy restatement           pinned
 *                         (the reference's generated kernel stores 1 into its norms: the norm sum is build-defined)
 *   orc_fused_adam_a3     nccl/.../reduce_kernel.h:36-68 functors; known answer w=-1, half 0xBC00; two steps by hand at
 *                         beta1 != beta2 (the first moment decays with beta2, common_kernel.h:878)          pinned
 *   orc_adam_f32          nccl-overlap/samples/multi-process-adam-scattered.cpp:112-136;
 *                         reference integer fixture, torch.optim.Adam (CPU) cross-check, step-1 closed form   pinned
 *   orc_lamb_f32          same file :402-449; single-segment/w==0 special cases, float64 brute force  pinned
 *                         (mode 2: nccl/.../reduce_kernel.h:391-452; all-ones closed form, float64 brute force;
 *                          the reference sums its norms in fp32 in no fixed order: norm rounding parity unpinned)
 *   orc_lamb_nccl_f16g    nccl/.../common_kernel.h:2438-2535, 2677-2700; equals orc_lamb_f32 mode 2 bit for bit where
 *                         the fp16 sums and squares are exact; numpy float16 restatement of the fp16 chain   pinned
 *                         (rounding of the fp32 norm sums unpinned, as for mode 2)
 *   orc_adam_f16g,        no counterpart in the reference (it has no loss scaling / overflow detection, and no bfloat16):
 *   orc_adam_bf16g        build-defined, pinned by closed forms only; parity with Apex "parity unpinned"
 *   orc_philox4x32_10     Random123 known-answer vectors                         pinned
 *   orc_mlp_outproj       no reference test beyond the all-ones C == K check
 *                         (nccl-overlap/samples/matmul-allreduce-bias-dropout-layernorm.cu:520-526);
 *                         float64 brute force; dropout mask build-defined ("parity unpinned" vs cuRAND)
 *   orc_epilogue_value,   the four dropout forms (src/codegen.cpp:634-640; nccl-overlap/.../reduce_kernel.h:192-213):
 *   orc_mlp_outproj_mode  closed forms at p = 0 and p = 1, complementary survivors at p = 0.3, saturating cases by hand   pinned
 *                         (the uniform draws themselves: "parity unpinned" vs cuRAND)
 *   orc_mlp_outproj_typed the same routine on IEEE-half operands: float64 brute force over numpy's float16 values, numpy's
 *                         float16 cast of the result, the reference's all-ones check                          pinned
 */
#ifndef CCN_ORACLE_H
#define CCN_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Host threads for the element-, segment- and row-parallel loops (default 1, the reference's single-threaded checker);
 * results do not depend on it. */
void orc_set_num_threads(int n);
int  orc_get_num_threads(void);

/* ---- scalar conversions (IEEE binary16 / bfloat16, round-to-nearest-even) ---- */
uint16_t orc_f32_to_f16(float f);
float    orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
float    orc_bf16_to_f32(uint16_t h);
void orc_f32_to_f16_array(const float* src, uint16_t* dst, size_t n);
void orc_f16_to_f32_array(const uint16_t* src, float* dst, size_t n);
void orc_f32_to_bf16_array(const float* src, uint16_t* dst, size_t n);
void orc_bf16_to_f32_array(const uint16_t* src, float* dst, size_t n);

/* ---- the reference's comparators ---- */
int orc_eqFloat_1e3(float u, float v);   /* examples/header.h:52-59 */
int orc_eq_float_1e5(float f1, float f2); /* nccl-overlap/samples/multi-process-adam-scattered.cpp:60-66 */

/* ---- P-way reduce ---- */
void orc_reduce_f32(const float* const* g, int P, size_t N, float* out);

/* ---- SGD ---- */
void orc_sgd_f32(const float* const* g, int P, float* w, size_t N, float lr);
void orc_sgd_axpby_f32(const float* const* g, int P, float* w, size_t N, float alpha, float beta);

/* ---- the DSL example's pseudo-Adam (no sqrt, "bias correction" = divide by beta) ---- */
void orc_pseudo_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                         float lr, float beta1, float beta2);
/* the DSL example's LAMB (examples/lamb/lamb.cpp:20-28), whole-tensor L2 norms; new weights to w_out, w untouched */
void orc_dsl_lamb_f32(const float* const* g, int P, const float* w, float* m, float* v, float* w_out, size_t N,
                      float lr, float beta1, float beta2, float c1, float c2, float eps, int has_eps, float gamma,
                      float* norms_out);

/* ---- the modified-NCCL fused mixed-precision Adam (fp16 ring sum, square in half, beta2 used for m) ---- */
void orc_fused_adam_a3(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* halfw,
                       size_t N, float lr, float beta1, float beta2);

/* ---- bias-corrected Adam; step = epoch+1 >= 1; w <- w - lr * mhat/(sqrt(vhat)+eps) ---- */
void orc_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                  float lr, float beta1, float beta2, float eps, int step);

/* ---- mixed-precision Adam: fp16 gradients, loss-scale removal, overflow flag, fp16 weight copy ---- */
/* returns the overflow flag (0/1) */
uint32_t orc_adam_f16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16,
                       size_t N, float lr, float beta1, float beta2, float eps, int step, float inv_scale);
uint32_t orc_adam_bf16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16,
                        size_t N, float lr, float beta1, float beta2, float eps, int step, float inv_scale);
uint32_t orc_overflow_f16(const uint16_t* const* g, int P, size_t N);

/* ---- LAMB with per-segment norms.  seg_offsets has nseg+1 entries, seg_offsets[nseg] == N.
 *      mode 0: scale = trust ratio W/R;  mode 1 (reference): scale = (W/R)/R;
 *      mode 2: the modified NCCL's global-norm LAMB arithmetic (divide by beta, L2 norms, no eps).
 *      norms_out (optional, 2*nseg doubles): W_b, R_b after the square root. ---- */
void orc_lamb_nccl_f16g(const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v,
                        const size_t* seg_offsets, int nseg, float lr, float beta1, float beta2, float wd,
                        double* norms_out);
void orc_lamb_f32(const float* const* g, int P, float* w, float* m, float* v,
                  const size_t* seg_offsets, int nseg, float lr, float beta1, float beta2,
                  float eps, float wd, int step, int mode, double* norms_out);

/* ---- counter-based RNG ---- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* keep decision for element idx of a dropout with drop probability p_drop (1 = keep) */
int  orc_dropout_keep(uint64_t seed, uint64_t idx, float p_drop);
void orc_dropout_mask(uint64_t seed, uint64_t first_idx, size_t n, float p_drop, uint8_t* keep);

/* ---- model-parallel MLP out-projection, one rank's K-slice:
 *      acc = X[MxK] (bf16) . W[KxN] (bf16), float64 accumulation rounded once to fp32;
 *      s = acc + partial[0] + ... + partial[nPartials-1]  (fp32, ascending);
 *      t = s + bias[col]; d = keep ? t * (1/(1-p)) : 0;  y = d + resid;  out = bf16(y)
 *      out_f32 (optional) receives y before the bf16 rounding. ---- */
/* one element of the epilogue under dropout form `mode` (0 standard, 1-3 the reference's; see ccn_oracle.c) */
float orc_epilogue_value(float s, float b, float r, int kept_inverted, float p_drop, int mode);
/* half != 0 with mode 3: value and bias held as IEEE halves, a rounding to half after each saturating add, as the
 * reference's FuncDropout<half> (nccl-overlap/src/collectives/device/reduce_kernel.h:199-213) */
float orc_epilogue_value_typed(float s, float b, float r, int kept_inverted, float p_drop, int mode, int half);
void orc_mlp_outproj_mode(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                          const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                          int M, int N, int K, float p_drop, uint64_t seed, int mode);
void orc_mlp_outproj(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                     const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                     int M, int N, int K, float p_drop, uint64_t seed);
/* the same with the 16-bit type as an argument: half = 0 bfloat16, 1 IEEE half */
/* the same on a gathered subset of rows: row i of X, partials, resid, out is row row_ids[i] of the whole output (the
 * dropout draw depends on the element's index there); row_ids == NULL: rows 0..M-1 */
void orc_mlp_outproj_rows(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                          const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                          int M, int N, int K, float p_drop, uint64_t seed, int mode, int half, const int64_t* row_ids);
void orc_mlp_outproj_typed(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                           const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                           int M, int N, int K, float p_drop, uint64_t seed, int mode, int half);

#ifdef __cplusplus
}
#endif
#endif
