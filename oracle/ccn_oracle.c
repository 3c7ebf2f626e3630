/*
 * ccn_oracle.c -- CPU oracle (test infrastructure, never shipped in the product library).
 * See ccn_oracle.h for the conventions and for what pins each routine.
 * Build: gcc -O2 -ffp-contract=off -fPIC -shared (see Makefile); -ffp-contract=off is load-bearing.
 */
#include "ccn_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------
 * conversions
 * ---------------------------------------------------------------------------------------------- */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> fp16, round-to-nearest-even; the rounding the reference obtains from __floats2half2_rn
 * (nccl/src/collectives/device/common_kernel.h:655-670). */
uint16_t orc_f32_to_f16(float f) {
  uint32_t x = f2u(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) {                       /* inf / nan */
    if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* >= 65520 rounds to inf */
  if (absx < 0x33000001u) return (uint16_t)sign;                /* <= 2^-25 rounds to zero (tie -> even 0) */
  int32_t e = (int32_t)(absx >> 23) - 127;                      /* unbiased exponent */
  uint32_t mant = (absx & 0x7fffffu) | 0x800000u;               /* 24-bit significand */
  int shift;                                                    /* bits dropped from the significand */
  uint32_t hexp;
  if (e < -14) { shift = 13 + (-14 - e); hexp = 0; }            /* subnormal half */
  else         { shift = 13;             hexp = (uint32_t)(e + 15); }
  uint32_t kept = mant >> shift;
  uint32_t rem  = mant & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept++;
  uint32_t h;
  if (hexp == 0) h = kept;                                      /* may carry into exponent 1: correct */
  else           h = ((hexp - 1) << 10) + kept;                 /* kept includes the hidden bit (0x400) */
  return (uint16_t)(sign | h);
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t m = h & 0x3ffu;
  if (e == 0x1f) return u2f(sign | 0x7f800000u | (m << 13));
  if (e == 0) {
    if (m == 0) return u2f(sign);
    /* subnormal: m * 2^-24 */
    float v = (float)m * 5.9604644775390625e-08f;
    return (sign ? -v : v);
  }
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

uint16_t orc_f32_to_bf16(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);  /* quiet nan */
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

void orc_f32_to_f16_array(const float* s, uint16_t* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_f32_to_f16(s[i]); }
void orc_f16_to_f32_array(const uint16_t* s, float* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_f16_to_f32(s[i]); }
void orc_f32_to_bf16_array(const float* s, uint16_t* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_f32_to_bf16(s[i]); }
void orc_bf16_to_f32_array(const uint16_t* s, float* d, size_t n) { for (size_t i = 0; i < n; i++) d[i] = orc_bf16_to_f32(s[i]); }

/* ------------------------------------------------------------------------------------------------
 * comparators
 * ---------------------------------------------------------------------------------------------- */
/* examples/header.h:52-62  absRelDiff / eqFloat */
int orc_eqFloat_1e3(float u, float v) {
  if (u == 0.0f || v == 0.0f) return u == v;
  return fabsf((u - v) / u) <= 1e-3;
}
/* nccl-overlap/samples/multi-process-adam-scattered.cpp:60-66  eq_float */
int orc_eq_float_1e5(float f1, float f2) {
  if (f1 == 0.0f && f2 == 0.0f) return 1;
  float mx = f1 > f2 ? f1 : f2;
  return fabs((f1 - f2) / mx) <= 1e-5;
}

/* ------------------------------------------------------------------------------------------------
 * reduce / SGD
 * ---------------------------------------------------------------------------------------------- */
static inline float reduce_at(const float* const* g, int P, size_t i) {
  float s = g[0][i];
  for (int p = 1; p < P; p++) s = s + g[p][i];
  return s;
}

/* Host threads for the loops that are independent across elements (or across segments, or rows): 1 = the reference's
 * single-threaded checker; more = the same loops under "omp parallel for" (static schedule, same arithmetic per
 * element, same results), which is how bench.py times the CPU baseline on all cores of the GPU box. */
static int orc_threads = 1;
void orc_set_num_threads(int n) { orc_threads = n > 1 ? n : 1; }
int orc_get_num_threads(void) { return orc_threads; }
#define ORC_PARALLEL_FOR _Pragma("omp parallel for schedule(static) num_threads(orc_threads) if (orc_threads > 1)")

void orc_reduce_f32(const float* const* g, int P, size_t N, float* out) {
  for (size_t i = 0; i < N; i++) out[i] = reduce_at(g, P, i);
}

/* examples/test-sgd.cu:17-18   __S1[i0] = (__w[i0] - (__lr * __S0[i0])) */
void orc_sgd_f32(const float* const* g, int P, float* w, size_t N, float lr) {
  ORC_PARALLEL_FOR
  for (size_t i = 0; i < N; i++) {
    float s0 = reduce_at(g, P, i);
    w[i] = (w[i] - (lr * s0));
  }
}

/* nccl-overlap/samples/single-process-wX.cu:141   new_weight = alpha * w + beta * reduced_grad */
void orc_sgd_axpby_f32(const float* const* g, int P, float* w, size_t N, float alpha, float beta) {
  for (size_t i = 0; i < N; i++) {
    float s0 = reduce_at(g, P, i);
    w[i] = alpha * w[i] + beta * s0;
  }
}

/* ------------------------------------------------------------------------------------------------
 * examples/test-adam.cu:14-38  (the saved checker of the DSL's adam example)
 *   S2 = beta2*v + (1-beta2)*(S0*S0);  S4 = S2/beta2;  S1 = beta1*m + (1-beta1)*S0;  S3 = S1/beta1;
 *   S5 = w - (lr*S3)/S4
 * The DSL program declares m and v as Update targets (examples/adam/adam.cpp:18-23), so S1 and S2
 * are stored back.
 * ---------------------------------------------------------------------------------------------- */
void orc_pseudo_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                         float lr, float beta1, float beta2) {
  for (size_t i = 0; i < N; i++) {
    float S0 = reduce_at(g, P, i);
    float S2 = ((beta2 * v[i]) + ((1 - beta2) * (S0 * S0)));
    float S4 = (S2 / beta2);
    float S1 = ((beta1 * m[i]) + ((1 - beta1) * S0));
    float S3 = (S1 / beta1);
    float S5 = (w[i] - ((lr * S3) / S4));
    v[i] = S2; m[i] = S1; w[i] = S5;
  }
}

/* ------------------------------------------------------------------------------------------------
 * The LAMB of the DSL example, examples/lamb/lamb.cpp:20-28, stage by stage as the reference's generated
 * checker re-executes a pipeline (src/codegen.cpp:4421-4581), every stage value an fp32 array:
 *   g1 = AllReduce(g);  m1 = Update(m, beta1*m + (1.0-beta1)*g1);  v1 = Update(v, beta2*v + (1.0-beta2)*g1*g1);
 *   m_ = m1/(1.0-beta1);  v_ = v1/(1.0-beta2);  r = m_/Sqrt(v_) + gamma*w;
 *   rNorm = Norm(r);  wNorm = Norm(w);  w1 = w - lr*(wNorm/rNorm)*r
 * The constant 1.0 prints as "1" in the reference's kernels ((1 - beta1), float arithmetic); a*b*c is (a*b)*c.
 * Norm is the L2 norm of the WHOLE tensor; the reference's generated kernel never got its accumulation (it stores the
 * constant 1 into the norm), so the sum is build-defined: squares taken in fp32, added in float64 in index order,
 * square root in float64, rounded to fp32.  c1, c2: what m1 and v1 are divided by (1-beta1, 1-beta2 computed in fp32
 * for the example; a caller's bias corrections for programs that pass them).  has_eps adds eps to the square root
 * (the example has none).  w is not written: the new weights go to w_out (the example's w1 is a stage of its own;
 * its RS_C_AG schedules then Update w with it).  norms_out (may be NULL): rNorm, wNorm.
 * ---------------------------------------------------------------------------------------------- */
void orc_dsl_lamb_f32(const float* const* g, int P, const float* w, float* m, float* v, float* w_out, size_t N,
                      float lr, float beta1, float beta2, float c1, float c2, float eps, int has_eps, float gamma,
                      float* norms_out) {
  float* r = (float*)malloc((N ? N : 1) * sizeof(float));
  double r2 = 0.0, w2 = 0.0;
  for (size_t i = 0; i < N; i++) {
    const float g1 = reduce_at(g, P, i);
    const float m1 = ((beta1 * m[i]) + ((1 - beta1) * g1));
    const float v1 = ((beta2 * v[i]) + (((1 - beta2) * g1) * g1));
    m[i] = m1;
    v[i] = v1;
    const float m_ = (m1 / c1);
    const float v_ = (v1 / c2);
    const float root = has_eps ? (sqrtf(v_) + eps) : sqrtf(v_);
    r[i] = ((m_ / root) + (gamma * w[i]));
    { const float x = r[i]; r2 += (double)(x * x); }
    { const float x = w[i]; w2 += (double)(x * x); }
  }
  const float rNorm = (float)sqrt(r2), wNorm = (float)sqrt(w2);
  if (norms_out) { norms_out[0] = rNorm; norms_out[1] = wNorm; }
  for (size_t i = 0; i < N; i++) w_out[i] = (w[i] - ((lr * (wNorm / rNorm)) * r[i]));
  free(r);
}

/* ------------------------------------------------------------------------------------------------
 * The modified NCCL's fused mixed-precision "Adam":
 *   functors  nccl/src/collectives/device/reduce_kernel.h:36-68
 *   call order nccl/src/collectives/device/common_kernel.h:875-887, fp16 store :910-921
 * Faithful to the kernel, including: gradient sum carried in fp16 (__hadd2 chain), the square taken
 * in fp16, and the first moment updated with beta2 in place of beta1 (the kernel invokes the
 * mixedbinOp3 functor through .mixedbinOp1(beta2, ...)).
 * ---------------------------------------------------------------------------------------------- */
static inline uint16_t hadd(uint16_t a, uint16_t b) { return orc_f32_to_f16(orc_f16_to_f32(a) + orc_f16_to_f32(b)); }
static inline uint16_t hmul(uint16_t a, uint16_t b) { return orc_f32_to_f16(orc_f16_to_f32(a) * orc_f16_to_f32(b)); }

void orc_fused_adam_a3(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* halfw,
                       size_t N, float lr, float beta1, float beta2) {
  for (size_t i = 0; i < N; i++) {
    uint16_t S0 = g[0][i];
    for (int p = 1; p < P; p++) S0 = hadd(S0, g[p][i]);
    float S2 = ((v[i] * beta2) + ((orc_f16_to_f32(hmul(S0, S0))) * (1 - beta2)));   /* mixedbinOp1 */
    float S4 = (S2 / beta2);                                                         /* binOp2 */
    float S1 = ((m[i] * beta2) + ((orc_f16_to_f32(S0)) * (1 - beta2)));              /* mixedbinOp3 called with beta2 */
    float S3 = (S1 / beta1);                                                         /* binOp2 with beta1 */
    float S5 = ((S3 * lr) / sqrtf(S4));                                              /* delta */
    v[i] = S2; m[i] = S1;
    float fw = w[i] - S5;                                                            /* weightUpdate */
    w[i] = fw;
    halfw[i] = orc_f32_to_f16(fw);
  }
}

/* ------------------------------------------------------------------------------------------------
 * nccl-overlap/samples/multi-process-adam-scattered.cpp:112-136  (check_epoch_results_adam, T=float)
 *   m  = beta1*old_m + (1-beta1)*gs
 *   v  = beta2*old_v + (1-beta2)*gs*gs                  -- ((1-beta2)*gs)*gs, left to right
 *   m_ = m/(1 - pow(beta1, epoch+1))                     -- pow and the division are double, result float
 *   v_ = v/(1 - pow(beta2, epoch+1))
 *   x  = stepsize * m_ / (sqrt(v_) + epsilon)            -- (stepsize*m_) / (sqrtf(v_)+eps), fp32
 *   w  = w + x
 * The reference passes stepsize = +alpha; the benchmark's "w -= lr*..." is stepsize = -lr, which is the
 * same fp32 result as subtracting (negation is exact).
 * sqrt: the unqualified call resolves to the float overload when the C++ <math.h> wrapper is in
 * scope (it is pulled in by the CUDA runtime header); the device functor computes
 * (float)sqrt((double)v_), which is the same correctly rounded value.
 * ---------------------------------------------------------------------------------------------- */
void orc_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                  float lr, float beta1, float beta2, float eps, int step) {
  const double bc1 = 1 - pow((double)beta1, (double)step);
  const double bc2 = 1 - pow((double)beta2, (double)step);
  const float stepsize = -lr;
  ORC_PARALLEL_FOR
  for (size_t i = 0; i < N; i++) {
    float gs = reduce_at(g, P, i);
    float mi = beta1 * m[i] + (1 - beta1) * gs;
    float vi = beta2 * v[i] + (1 - beta2) * gs * gs;
    float m_ = (float)((double)mi / bc1);
    float v_ = (float)((double)vi / bc2);
    float x = stepsize * m_ / (sqrtf(v_) + eps);
    w[i] = w[i] + x;
    m[i] = mi;
    v[i] = vi;
  }
}

/* ------------------------------------------------------------------------------------------------
 * Mixed-precision Adam with loss-scale removal and overflow detection.  The reference has neither
 * (its only mention of an overflow buffer is the Apex baseline script, experiments/optimbench.py:61-81),
 * so the semantics are defined by this build:
 *   - element i "overflows" when any g[p][i] has fp16 exponent 0x1F (inf or nan);
 *     flag = OR over all elements and ranks;
 *   - gs = sum_p ( float(g[p][i]) * inv_scale ), fp32, p ascending (unscale before the sum);
 *   - an overflowing element leaves w, m, v untouched (the optimizer state is never poisoned);
 *     every other element takes the Adam step of orc_adam_f32;
 *   - w16[i] = fp16_rne(w[i]) is written for every element.
 * ---------------------------------------------------------------------------------------------- */
uint32_t orc_adam_f16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16,
                       size_t N, float lr, float beta1, float beta2, float eps, int step, float inv_scale) {
  const double bc1 = 1 - pow((double)beta1, (double)step);
  const double bc2 = 1 - pow((double)beta2, (double)step);
  const float stepsize = -lr;
  uint32_t flag = 0;
  _Pragma("omp parallel for schedule(static) num_threads(orc_threads) if (orc_threads > 1) reduction(|:flag)")
  for (size_t i = 0; i < N; i++) {
    int bad = 0;
    float gs = 0.0f;
    for (int p = 0; p < P; p++) {
      uint16_t h = g[p][i];
      if ((h & 0x7c00u) == 0x7c00u) bad = 1;
      float t = orc_f16_to_f32(h) * inv_scale;
      gs = (p == 0) ? t : gs + t;
    }
    if (bad) {
      flag = 1;
    } else {
      float mi = beta1 * m[i] + (1 - beta1) * gs;
      float vi = beta2 * v[i] + (1 - beta2) * gs * gs;
      float m_ = (float)((double)mi / bc1);
      float v_ = (float)((double)vi / bc2);
      float x = stepsize * m_ / (sqrtf(v_) + eps);
      w[i] = w[i] + x;
      m[i] = mi;
      v[i] = vi;
    }
    w16[i] = orc_f32_to_f16(w[i]);
  }
  return flag;
}

/* The same step with bfloat16 gradients and a bfloat16 copy of the weights (no counterpart in the reference, which has
 * fp16 only): overflow = exponent 0xFF; conversions round to nearest even. */
uint32_t orc_adam_bf16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16,
                        size_t N, float lr, float beta1, float beta2, float eps, int step, float inv_scale) {
  const double bc1 = 1 - pow((double)beta1, (double)step);
  const double bc2 = 1 - pow((double)beta2, (double)step);
  const float stepsize = -lr;
  uint32_t flag = 0;
  _Pragma("omp parallel for schedule(static) num_threads(orc_threads) if (orc_threads > 1) reduction(|:flag)")
  for (size_t i = 0; i < N; i++) {
    int bad = 0;
    float gs = 0.0f;
    for (int p = 0; p < P; p++) {
      uint16_t h = g[p][i];
      if ((h & 0x7f80u) == 0x7f80u) bad = 1;
      float t = orc_bf16_to_f32(h) * inv_scale;
      gs = (p == 0) ? t : gs + t;
    }
    if (bad) {
      flag = 1;
    } else {
      float mi = beta1 * m[i] + (1 - beta1) * gs;
      float vi = beta2 * v[i] + (1 - beta2) * gs * gs;
      float m_ = (float)((double)mi / bc1);
      float v_ = (float)((double)vi / bc2);
      float x = stepsize * m_ / (sqrtf(v_) + eps);
      w[i] = w[i] + x;
      m[i] = mi;
      v[i] = vi;
    }
    w16[i] = orc_f32_to_bf16(w[i]);
  }
  return flag;
}

uint32_t orc_overflow_f16(const uint16_t* const* g, int P, size_t N) {
  for (int p = 0; p < P; p++)
    for (size_t i = 0; i < N; i++)
      if ((g[p][i] & 0x7c00u) == 0x7c00u) return 1;
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * nccl-overlap/samples/multi-process-adam-scattered.cpp:402-449 (check_epoch_results_lamb, T=float),
 * applied once per segment ("parent buffer"):
 *   first loop : m, v as Adam;  r = m_/(sqrt(v_)+eps) + 1.0f*w;
 *                rNorm += (r*r)/n   (fp32 quotient, double accumulator);  wNorm += w*w (fp32 product)
 *   rNorm = sqrt(rNorm);  wNorm = sqrt(wNorm/n)
 *   second loop: r recomputed from the stored m, v;
 *                scale = (float)( ((wNorm>0) ? (rNorm>0 ? wNorm/rNorm : 1) : 1) / rNorm )
 *                w = w - (stepsize*scale)*r
 * The hard-coded 1.0f is the weight-decay factor wd here (wd = 1.0f reproduces the reference bit for bit).
 * mode 1 keeps the reference's second division by rNorm; mode 0 drops it (textbook trust ratio).
 * ---------------------------------------------------------------------------------------------- */
/* mode 2: the modified NCCL's LAMB (global-norm variant), per segment:
 *   functors nccl/src/collectives/device/reduce_kernel.h:391-452 (binOp1, binOp2, binOp3, binOp4, rOp, delta,
 *   weightUpdate) in the call order of common_kernel.h:2211-2273 (phase 1) and :2687-2726 (phase 2);
 *   norms all_reduce_computation.h:931-978.
 *   v = (v*b2) + ((gs*gs)*(1-b2));  S4 = v/b2;  m = (m*b1) + (gs*(1-b1));  S3 = m/b1;
 *   r = S3/sqrtf(S4) + 1.0f*w;  wNorm = sqrtf(sum w^2), rNorm = sqrtf(sum r^2)   (L2 norms, no division by n)
 *   scale = ((wNorm>0) ? (rNorm>0 ? wNorm/rNorm : 1) : 1)/rNorm  in fp32;  w = w - (lr*scale)*r
 * The kernel accumulates the two sums in fp32 through shuffles and atomics, i.e. in no fixed order; the oracle
 * accumulates in float64 and rounds once, which every fp32 order approximates.  eps and step are not used;
 * wd takes the place of the hard-coded 1.0f. */
static void lamb_nccl_segment(const float* const* g, int P, float* w, float* m, float* v, size_t lo, size_t hi,
                              float lr, float beta1, float beta2, float wd, double* norms_out) {
  double rr = 0.0, ww = 0.0;
  for (size_t i = lo; i < hi; i++) {
    float gs = reduce_at(g, P, i);
    float vi = ((v[i] * beta2) + ((gs * gs) * (1 - beta2)));
    float S4 = (vi / beta2);
    float mi = ((m[i] * beta1) + (gs * (1 - beta1)));
    float S3 = (mi / beta1);
    float r = (S3) / sqrtf(S4) + wd * w[i];
    ww += (double)(w[i] * w[i]);
    rr += (double)(r * r);
    v[i] = vi;
    m[i] = mi;
  }
  const float wNorm = sqrtf((float)ww), rNorm = sqrtf((float)rr);
  if (norms_out) { norms_out[0] = wNorm; norms_out[1] = rNorm; }
  const float scale = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f) / rNorm;
  for (size_t i = lo; i < hi; i++) {
    float r = ((m[i] / beta1)) / sqrtf((v[i] / beta2)) + wd * w[i];
    float delta = (lr * scale) * r;
    w[i] = w[i] - delta;
  }
}

/* The modified NCCL's LAMB with fp16 gradients (its mixed-precision path), per segment:
 *   phase 1 nccl/src/collectives/device/common_kernel.h:2438-2535: gradient sum carried in fp16 (FuncSumHalf chain,
 *   :2460-2472); functors nccl/src/collectives/device/reduce_kernel.h:391-399 mixedbinOp1 (square taken in fp16),
 *   mixedbinOp3 (here with beta1, :2509), binOp2, binOp4, rOp :425-432; phase 2 common_kernel.h:2677-2700 with the
 *   fp16 copy of the new weights (float4ToHalf4, :2695).
 *   S0 = fp16 sum;  v = (v*b2) + (float(S0*S0 in fp16)*(1-b2));  S4 = v/b2;  m = (m*b1) + (float(S0)*(1-b1));  S3 = m/b1;
 *   r = S3/sqrtf(S4) + 1.0f*w;  norms, scale and the update as in lamb_nccl_segment;  halfw = fp16(w).
 * The kernel keeps r in a caller's buffer between the phases; recomputing it from the stored m, v and the old w
 * gives the same bits.  wd takes the place of the hard-coded 1.0f. */
void orc_lamb_nccl_f16g(const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v,
                        const size_t* seg_offsets, int nseg, float lr, float beta1, float beta2, float wd,
                        double* norms_out) {
  ORC_PARALLEL_FOR
  for (int b = 0; b < nseg; b++) {
    const size_t lo = seg_offsets[b], hi = seg_offsets[b + 1];
    double rr = 0.0, ww = 0.0;
    for (size_t i = lo; i < hi; i++) {
      uint16_t S0 = g[0][i];
      for (int p = 1; p < P; p++) S0 = hadd(S0, g[p][i]);
      float vi = ((v[i] * beta2) + ((orc_f16_to_f32(hmul(S0, S0))) * (1 - beta2)));
      float S4 = (vi / beta2);
      float mi = ((m[i] * beta1) + ((orc_f16_to_f32(S0)) * (1 - beta1)));
      float S3 = (mi / beta1);
      float r = (S3) / sqrtf(S4) + wd * w[i];
      ww += (double)(w[i] * w[i]);
      rr += (double)(r * r);
      v[i] = vi;
      m[i] = mi;
    }
    const float wNorm = sqrtf((float)ww), rNorm = sqrtf((float)rr);
    if (norms_out) { norms_out[2 * b] = wNorm; norms_out[2 * b + 1] = rNorm; }
    const float scale = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f) / rNorm;
    for (size_t i = lo; i < hi; i++) {
      float r = ((m[i] / beta1)) / sqrtf((v[i] / beta2)) + wd * w[i];
      float delta = (lr * scale) * r;
      w[i] = w[i] - delta;
      halfw[i] = orc_f32_to_f16(w[i]);
    }
  }
}

void orc_lamb_f32(const float* const* g, int P, float* w, float* m, float* v,
                  const size_t* seg_offsets, int nseg, float lr, float beta1, float beta2,
                  float eps, float wd, int step, int mode, double* norms_out) {
  if (mode == 2) {
    ORC_PARALLEL_FOR
    for (int b = 0; b < nseg; b++)
      lamb_nccl_segment(g, P, w, m, v, seg_offsets[b], seg_offsets[b + 1], lr, beta1, beta2, wd,
                        norms_out ? norms_out + 2 * b : NULL);
    return;
  }
  const double bc1 = 1 - pow((double)beta1, (double)step);
  const double bc2 = 1 - pow((double)beta2, (double)step);
  const float stepsize = lr;
  ORC_PARALLEL_FOR
  for (int b = 0; b < nseg; b++) {
    const size_t lo = seg_offsets[b], hi = seg_offsets[b + 1];
    const uint64_t n = (uint64_t)(hi - lo);
    double rNorm = 0.0, wNorm = 0.0;
    for (size_t i = lo; i < hi; i++) {
      float gs = reduce_at(g, P, i);
      float mi = beta1 * m[i] + (1 - beta1) * gs;
      float vi = beta2 * v[i] + (1 - beta2) * gs * gs;
      float m_ = (float)((double)mi / bc1);
      float v_ = (float)((double)vi / bc2);
      float r = m_ / (sqrtf(v_) + eps) + wd * w[i];
      rNorm += (r * r) / (float)n;
      wNorm += (w[i] * w[i]);
      v[i] = vi;
      m[i] = mi;
    }
    rNorm = sqrt(rNorm);
    wNorm = sqrt(wNorm / (double)n);
    if (norms_out) { norms_out[2 * b] = wNorm; norms_out[2 * b + 1] = rNorm; }
    double ratio = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f);
    float scale = (float)(mode == 1 ? ratio / rNorm : ratio);
    for (size_t i = lo; i < hi; i++) {
      float m_ = (float)((double)m[i] / bc1);
      float v_ = (float)((double)v[i] / bc2);
      float r = m_ / (sqrtf(v_) + eps) + wd * w[i];
      float x = stepsize * scale * r;
      w[i] = w[i] - x;
    }
  }
}

/* ------------------------------------------------------------------------------------------------
 * Philox-4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11)
 * ---------------------------------------------------------------------------------------------- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Dropout mask, build-defined (the reference's mask is curand_init(0,0,0) evaluated identically for
 * every element, src/codegen.cpp:634-640, which is degenerate):
 *   block = idx/4 -> Philox counter (lo, hi, 0, 0), key = (seed lo, seed hi), word = out[idx%4];
 *   u = (word >> 8) * 2^-24 in [0,1);  keep <=> u >= p_drop. */
int orc_dropout_keep(uint64_t seed, uint64_t idx, float p_drop) {
  uint64_t blk = idx >> 2;
  uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), 0u, 0u};
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t out[4];
  orc_philox4x32_10(ctr, key, out);
  float u = (float)(out[idx & 3] >> 8) * 5.9604644775390625e-08f;
  return u >= p_drop;
}

void orc_dropout_mask(uint64_t seed, uint64_t first_idx, size_t n, float p_drop, uint8_t* keep) {
  for (size_t i = 0; i < n; i++) keep[i] = (uint8_t)orc_dropout_keep(seed, first_idx + i, p_drop);
}

/* ------------------------------------------------------------------------------------------------
 * MLP out-projection with fused epilogue.  DSL shape: examples/model-parallel/model-parallel.cpp:18-21
 *   layer = MatMul(in, w); sum = AllReduce(layer); sum2 = sum + b; out = Dropout(sum2, p) + r
 * On one GPU the all-reduce is "own product + (P-1) partial products of the peers".
 * Dropout here is the standard one (drop with probability p, survivors scaled by 1/(1-p)); the
 * reference keeps with probability p and does not rescale (src/codegen.cpp:634-640).
 * ---------------------------------------------------------------------------------------------- */
/* One output element from its sum s (product + partial products), bias b, residual r and keep decision
 * `kept_inverted` (u >= p), under the four dropout forms:
 *   0  standard ("inverted") dropout:                      (u >= p ? (s + b) * 1/(1-p) : 0) + r
 *   1  the reference's emitted expression, src/codegen.cpp:634-640 with examples/model-parallel/model-parallel.cpp:20-21:
 *      (curand_uniform < prob ? (sum + b) : 0) + r          keeps with probability p, no rescale
 *   2  the reference's fused kernel, FuncDropout<T>, nccl-overlap/src/collectives/device/reduce_kernel.h:192-197:
 *      (curand_uniform < p ? val : 0) + biasVal + addTensorVal
 *   3  its half specialisation, :199-213: __hadd2_sat(__hadd2_sat(v, biasVal), addTensorVal), sat = clamp to [0, 1] */
static float sat01(float x) { return x > 0.0f ? (x < 1.0f ? x : 1.0f) : 0.0f; }
float orc_epilogue_value(float s, float b, float r, int kept_inverted, float p_drop, int mode) {
  if (mode == 0) {
    const float scale = 1.0f / (1.0f - p_drop);
    const float t = s + b;
    const float d = kept_inverted ? t * scale : 0.0f;
    return d + r;
  }
  const int kept = !kept_inverted;   /* u < p */
  if (mode == 1) {
    const float t = s + b;
    return (kept ? t : 0.0f) + r;
  }
  const float v = kept ? s : 0.0f;
  if (mode == 2) return (v + b) + r;
  return sat01(sat01(v + b) + r);
}

/* The same with the operand type known.  For IEEE half and the saturating form, the reference's half specialisation
 * (reduce_kernel.h:199-213) holds the value and the bias as halves and rounds to half after EACH of its two
 * __hadd2_sat; an fp32 sum of two halves rounded to half is the correctly rounded half sum (24 >= 2*11+2 bits), so the
 * roundings are restated with the fp32 add followed by a conversion. */
static float f16_round(float x) { return orc_f16_to_f32(orc_f32_to_f16(x)); }
float orc_epilogue_value_typed(float s, float b, float r, int kept_inverted, float p_drop, int mode, int half) {
  if (!(half && mode == 3)) return orc_epilogue_value(s, b, r, kept_inverted, p_drop, mode);
  const float v = !kept_inverted ? f16_round(s) : 0.0f;
  const float t = f16_round(sat01(v + f16_round(b)));
  return f16_round(sat01(t + r));
}

/* half = 0: X, W, resid and out are bfloat16; half = 1: IEEE half (the type the reference's model-parallel example
 * declares, examples/model-parallel/model-parallel.cpp:10-15).  Same arithmetic between the conversions. */
void orc_mlp_outproj_rows(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                          const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                          int M, int N, int K, float p_drop, uint64_t seed, int mode, int half, const int64_t* row_ids) {
  /* Row i of X, partials, resid and out is row row_ids[i] of the whole output (i itself without a table): the dropout
   * draw of an element depends on its index in the whole output.  The product of a row is accumulated in float64 in
   * ascending k for every column (k outer, j inner: the same sum per element as a k-innermost loop, read along W's rows). */
  ORC_PARALLEL_FOR
  for (int i = 0; i < M; i++) {
    double* acc = (double*)malloc((size_t)N * sizeof(double));
    for (int j = 0; j < N; j++) acc[j] = 0.0;
    for (int k = 0; k < K; k++) {
      const uint16_t xb = X[(size_t)i * K + k];
      const double x = half ? (double)orc_f16_to_f32(xb) : (double)orc_bf16_to_f32(xb);
      const uint16_t* wrow = W + (size_t)k * N;
      if (half) for (int j = 0; j < N; j++) acc[j] += x * (double)orc_f16_to_f32(wrow[j]);
      else for (int j = 0; j < N; j++) acc[j] += x * (double)orc_bf16_to_f32(wrow[j]);
    }
    const uint64_t row = row_ids ? (uint64_t)row_ids[i] : (uint64_t)i;
    for (int j = 0; j < N; j++) {
      float s = (float)acc[j];
      size_t idx = (size_t)i * N + j;
      for (int q = 0; q < nPartials; q++) s = s + partials[q][idx];
      const int kept_inverted = orc_dropout_keep(seed, row * (uint64_t)N + (uint64_t)j, p_drop);   /* u >= p; p = 0: always */
      const float r = !resid ? 0.0f : (half ? orc_f16_to_f32(resid[idx]) : orc_bf16_to_f32(resid[idx]));
      float y = orc_epilogue_value_typed(s, bias[j], r, kept_inverted, p_drop, mode, half);
      if (out_f32) out_f32[idx] = y;
      if (out) out[idx] = half ? orc_f32_to_f16(y) : orc_f32_to_bf16(y);
    }
    free(acc);
  }
}

void orc_mlp_outproj_typed(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                           const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                           int M, int N, int K, float p_drop, uint64_t seed, int mode, int half) {
  orc_mlp_outproj_rows(X, W, partials, nPartials, bias, resid, out, out_f32, M, N, K, p_drop, seed, mode, half, NULL);
}

void orc_mlp_outproj_mode(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                          const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                          int M, int N, int K, float p_drop, uint64_t seed, int mode) {
  orc_mlp_outproj_typed(X, W, partials, nPartials, bias, resid, out, out_f32, M, N, K, p_drop, seed, mode, 0);
}

void orc_mlp_outproj(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                     const float* bias, const uint16_t* resid, uint16_t* out, float* out_f32,
                     int M, int N, int K, float p_drop, uint64_t seed) {
  orc_mlp_outproj_mode(X, W, partials, nPartials, bias, resid, out, out_f32, M, N, K, p_drop, seed, 0);
}
