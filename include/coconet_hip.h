/*
 * coconet_hip.h -- C ABI of libcoconet_hip.so: the MI355X (gfx950) backend for CoCoNet's fused
 * "reduce P rank-gradient buffers + optimizer update" kernels and the model-parallel GEMM epilogue.
 *
 * Boundary.  In the reference, generated programs reach this functionality through entry points of a
 * modified NCCL (AllReduce_pipe, ncclAllReduceScatteredAdam, ...) and through emitted CUDA kernels.
 * On one GPU the collective degenerates to a local multi-operand reduce, so each entry point here takes
 * a host table of P device pointers (one gradient buffer per simulated rank) instead of a communicator.
 *
 * Conventions
 *   - plain C types only; every pointer named g/w/m/v/... is a DEVICE pointer unless marked "host".
 *   - `g` is a HOST array of P device pointers; it is read during the call and may be freed afterwards.
 *   - gradient buffers are read-only (the reference clobbers them; callers must not rely on that).
 *   - w, m, v are updated in place.
 *   - calls are asynchronous: work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     null stream); the caller synchronises.  No entry point calls exit(); errors are returned.
 *   - return value: 0 on success, a negative CCN_E* code otherwise (ccn_strerror() names it).
 *   - gradient sum order is fixed: ((g[0]+g[1])+g[2])+... in fp32, no fused multiply-add anywhere.
 *   - thread-compatible: concurrent calls on different streams are allowed; ccn_init is idempotent.
 */
#ifndef COCONET_HIP_H
#define COCONET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CCN_OK        0
#define CCN_EINVAL  (-22)  /* null pointer, N == 0 where not allowed, P out of range, bad mode, misaligned bf16/fp16 buffer */
#define CCN_ENOMEM  (-12)  /* hipMalloc failed */
#define CCN_ENODEV  (-19)  /* no such device / not a gfx950 device */
#define CCN_EHIP     (-5)  /* any other HIP runtime error (ccn_last_hip_error() gives the hipError_t) */
#define CCN_ERANGE  (-34)  /* size beyond what the kernel supports */

#define CCN_MAX_RANKS 16   /* 1 <= P <= CCN_MAX_RANKS */

#define CCN_LAMB_TRUST_RATIO 0  /* scale = W/R                         (textbook)                      */
#define CCN_LAMB_REFERENCE   1  /* scale = (W/R)/R  as the reference's kernel and checker compute it   */
#define CCN_LAMB_NCCL_GLOBAL 2  /* the modified NCCL's global-norm LAMB: m/beta1, v/beta2 in place of bias correction,
                                   r = S3/sqrtf(S4) + wd*w, L2 norms, scale = (W/R)/R in fp32; eps and step unused
                                   (nccl/src/collectives/device/reduce_kernel.h:391-452, common_kernel.h:2211-2273,
                                   2687-2726).  One segment covering [0,N) reproduces its single global norm. */

/* ---- runtime glue: what the generated driver needs instead of cudaMalloc / events
 *      (reference: emitted main(), src/codegen.cpp:4583-4784; examples/header.h:36-53) ---- */
int  ccn_version(void);
int  ccn_init(int device);                       /* hipSetDevice + device query; idempotent */
int  ccn_device_info(int* cu_count, size_t* hbm_bytes, char* arch, size_t arch_len);
int  ccn_malloc(void** p, size_t bytes);
int  ccn_free(void* p);
int  ccn_memcpy_h2d(void* dst, const void* src_host, size_t bytes, void* stream);
int  ccn_memcpy_d2h(void* dst_host, const void* src, size_t bytes, void* stream);
int  ccn_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream);
int  ccn_fill_f32(float* dst, float value, size_t n, void* stream);    /* memset_value, examples/header.h:85-101 */
int  ccn_stream_create(void** stream);
int  ccn_stream_destroy(void* stream);
int  ccn_stream_sync(void* stream);
int  ccn_event_create(void** ev);
int  ccn_event_destroy(void* ev);
int  ccn_event_record(void* ev, void* stream);
int  ccn_stream_wait_event(void* stream, void* ev);   /* work queued on `stream` after this call starts after `ev` (the
                                                         cudaStreamWaitEvent of the overlapped schedules' two streams) */
int  ccn_event_elapsed_ms(void* start, void* stop, float* ms);        /* synchronises on `stop` */
int  ccn_last_hip_error(void);
const char* ccn_strerror(int code);

/* ---- replaying a recorded sequence of calls.  The generated main() launches every epoch's kernels from the host
 *      (epoch loop, src/codegen.cpp:4690-4720); at small sizes (config 1: a 3 us kernel) the launches, not the kernels,
 *      set the pace.  Between ccn_graph_begin and ccn_graph_end the update entry points called on `stream` (a stream from
 *      ccn_stream_create, not the null stream) are recorded instead of run; ccn_graph_launch replays the recording.
 *      Recorded calls keep the arguments they were made with (pointers, sizes, and `step`, which is evaluated on the
 *      host: a recording of Adam or LAMB steps replays the same bias corrections).  Not recordable: ccn_malloc/free,
 *      the memcpy and sync calls, ccn_lamb_plan_create/norms, the first ccn_lamb_f32 call of a plan for a given
 *      rank count (it queries occupancy; make one call before recording), and a *_scattered call whose buffer
 *      pointers differ from the previous call's (it refreshes the plan's device table and waits for the copy). ---- */
typedef struct ccn_graph ccn_graph;
int  ccn_graph_begin(void* stream);
int  ccn_graph_end(void* stream, ccn_graph** graph);
int  ccn_graph_launch(ccn_graph* graph, void* stream);
int  ccn_graph_destroy(ccn_graph* graph);

/* ---- plain P-way reduce: out[i] = sum_p g[p][i].
 *      Replaces the stock ncclAllReduce of the unfused schedules (src/codegen.cpp:4146-4189;
 *      device loop nccl/src/collectives/device/common_kernel.h:1310-1427 ReduceOrCopyMulti).
 *      `out` may alias g[0] (in-place, as the reference's all-reduce). ---- */
int  ccn_reduce_f32(const float* const* g, int P, float* out, size_t N, void* stream);

/* ---- SGD: w <- w - lr * sum_p g[p].
 *      Replaces AllReduce_pipe(lr, g, w, SZ, ...) of the sgd example (examples/test-sgd.cu:3;
 *      checker :17-18) and the emitted kernel of examples/sgd/sgd.cpp:14-15. ---- */
int  ccn_sgd_f32(const float* const* g, int P, float* w, size_t N, float lr, void* stream);

/* ---- SGD, axpby form: w <- alpha*w + beta*sum_p g[p].
 *      Replaces ncclAllReduce2 / the SGD branch of ReduceCopy128bMulti
 *      (nccl-overlap/src/collectives/device/common_kernel.h:969-986; checker
 *      nccl-overlap/samples/single-process-wX.cu:141). ---- */
int  ccn_sgd_axpby_f32(const float* const* g, int P, float* w, size_t N, float alpha, float beta, void* stream);

/* ---- the adam example as the DSL states it (no sqrt, divides by beta instead of bias correction):
 *      v <- beta2*v + (1-beta2)*gs*gs; m <- beta1*m + (1-beta1)*gs; w <- w - (lr*(m/beta1))/(v/beta2).
 *      Replaces AllReduce_pipe(lr,beta1,beta2,g,w,m,v,SZ,...) of examples/test-adam.cu:3 (checker :14-38). ---- */
int  ccn_pseudo_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                         float lr, float beta1, float beta2, void* stream);

/* ---- bias-corrected Adam, fp32:  step >= 1 is the 1-based step number t (the reference passes epoch = t-1).
 *      m <- b1*m + (1-b1)*gs;  v <- b2*v + (1-b2)*gs*gs;  w <- w - lr * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps)
 *      Replaces ncclAllReduceScatteredAdam / ncclAllReduceAdam
 *      (nccl-overlap/src/collectives/all_reduce.cc:47-60, :142-155; device math
 *      nccl-overlap/src/collectives/device/common_kernel.h:905-968; checker
 *      nccl-overlap/samples/multi-process-adam-scattered.cpp:112-136).  The reference's stepsize
 *      alpha corresponds to -lr and its hard-coded epsilon 1e-6 to `eps`. ---- */
int  ccn_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N,
                  float lr, float beta1, float beta2, float eps, int step, void* stream);

/* ---- the same SGD and Adam steps over scattered buffers: gradients and weights stay in nbuff separate buffers (one
 *      per parameter tensor, counts[b] elements each), the moments in single arrays of sum(counts) elements that
 *      follow the buffers' concatenation.  This is the layout ncclAllReduceScatteredAdam takes
 *      (nccl-overlap/src/nccl.h.in:216-218; caller nccl-overlap/samples/multi-process-adam-scattered.cpp:334-337).
 *      g is a host array of P*nbuff device pointers, rank-major (g[p*nbuff + b]); w a host array of nbuff device
 *      pointers.  The plan keeps a device copy of the pointers and refreshes it, with one stream synchronisation,
 *      only when they change; calls on one plan must be ordered (same stream). ---- */
typedef struct ccn_scatter_plan ccn_scatter_plan;
int  ccn_scatter_plan_create(const size_t* counts, int nbuff, ccn_scatter_plan** plan);
int  ccn_scatter_plan_destroy(ccn_scatter_plan* plan);
int  ccn_sgd_f32_scattered(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, float lr, void* stream);
int  ccn_adam_f32_scattered(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, float* m, float* v,
                            float lr, float beta1, float beta2, float eps, int step, void* stream);

/* ---- mixed-precision Adam: fp16 gradients carrying a loss scale, fp32 master state, fp16 weight copy.
 *      gs = sum_p float(g[p][i])*inv_scale.  overflow_flag (device, one uint32) is SET by the call:
 *      1 if any g[p][i] is inf/nan, else 0.  Elements whose gradients overflow keep w, m, v unchanged;
 *      all other elements take the Adam step above; w16[i] = fp16(w[i]) is written for every element.
 *      Takes the place of the mixed-precision AllReduce_pipe(lr,b1,b2,(half*)g,w,(half*)halfw,m,v,count,...)
 *      (nccl/src/nccl.h.in:212; nccl/src/collectives/device/common_kernel.h:830-1172), which has no
 *      loss scaling or overflow detection; those semantics are defined by this library. ---- */
int  ccn_adam_f16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16, size_t N,
                   float lr, float beta1, float beta2, float eps, int step, float inv_scale,
                   uint32_t* overflow_flag, void* stream);
/* The same step with bfloat16 gradients and a bfloat16 copy of the weights (overflow = exponent 0xFF).  No counterpart in
 * the reference, whose mixed-precision path is fp16 only; same contract as ccn_adam_f16g otherwise. */
int  ccn_adam_bf16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16,
                    size_t N, float lr, float beta1, float beta2, float eps, int step, float inv_scale,
                    uint32_t* overflow_flag, void* stream);

/* ---- overflow pre-check for callers that want all-or-nothing steps: *overflow_flag <- any(!isfinite(g)). ---- */
int  ccn_overflow_check_f16(const uint16_t* const* g, int P, size_t N, uint32_t* overflow_flag, void* stream);

/* ---- the modified NCCL's fused mixed-precision Adam exactly as its kernel computes it (fp16 gradient sum,
 *      square taken in fp16, first moment decayed with beta2, no eps):
 *      nccl/src/collectives/device/reduce_kernel.h:36-68, common_kernel.h:875-921.
 *      Same signature shape as AllReduce_pipe (nccl/src/nccl.h.in:212). ---- */
int  ccn_fused_adam_ref_f16g(const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v,
                             size_t N, float lr, float beta1, float beta2, void* stream);

/* ---- LAMB with per-segment ("per-layer", the reference's "parent buffer") norms; two passes.
 *      A plan owns the device-side segment tables and the norm partials for one segmentation of [0,N).
 *      seg_offsets: HOST array of nseg+1 ascending element offsets, seg_offsets[0]==0, last == N.
 *      pass 1: m,v update; r = mhat/(sqrt(vhat)+eps) + wd*w; per-segment sum w^2, sum r^2 in float64
 *      finalize: W_b = sqrt(sum w^2 / n_b), R_b = sqrt(sum r^2 / n_b), scale_b (see CCN_LAMB_*)
 *      pass 2: w <- w - (lr*scale_b)*r   (r recomputed from m, v, w; no r buffer is needed)
 *      Replaces ncclAllReduceScatteredLAMB (nccl-overlap/src/collectives/all_reduce.cc:61-76; kernel
 *      nccl-overlap/src/collectives/device/all_reduce_scattered.h:107-262; checker
 *      nccl-overlap/samples/multi-process-adam-scattered.cpp:402-449).  wd = 1.0f is the reference. ---- */
typedef struct ccn_lamb_plan ccn_lamb_plan;
int  ccn_lamb_plan_create(const size_t* seg_offsets, int nseg, ccn_lamb_plan** plan);
int  ccn_lamb_plan_destroy(ccn_lamb_plan* plan);
int  ccn_lamb_f32(ccn_lamb_plan* plan, const float* const* g, int P, float* w, float* m, float* v,
                  float lr, float beta1, float beta2, float eps, float wd, int step, int mode, void* stream);
/* The same step with every segment's gradients and weights in a buffer of their own (the segments of the plan are the
 * buffers; moments stay in single arrays over the concatenation), as ncclAllReduceScatteredLAMB takes them
 * (nccl-overlap/src/nccl.h.in:219-221).  g: host array of P*nseg device pointers, rank-major; w: host array of nseg
 * device pointers.  The plan keeps a device copy of the pointers, refreshed (one stream synchronisation) when they change. */
/* A plan whose norm segments are made of several buffers each: the reference cuts every parameter tensor ("parent
 * buffer") into small buffers of at most maxBuffSize elements, passes one gradient / weight pointer per small buffer and
 * maps them back with buffIdToParentBufferId; the norms are per parent (nccl-overlap/src/nccl.h.in:219-221, sample
 * nccl-overlap/samples/multi-process-adam-scattered.cpp:505-517, 671-674).  buf_sizes[i]: elements of buffer i;
 * buf_parent[i]: its parent, starting at 0 and never decreasing or skipping (the buffers of a parent are consecutive,
 * as the sample builds them).  The plan then has buf_parent[nbuf-1]+1 segments; ccn_lamb_f32_scattered on it takes
 * P*nbuf gradient pointers (rank-major) and nbuf weight pointers, the moments are single arrays over the concatenation
 * of the buffers, and ccn_lamb_plan_norms returns the parents' norms.  The flat call works on such a plan as well. */
int  ccn_lamb_plan_create_parented(const size_t* buf_sizes, const size_t* buf_parent, int nbuf, ccn_lamb_plan** plan);
int  ccn_lamb_f32_scattered(ccn_lamb_plan* plan, const float* const* g, int P, float* const* w, float* m, float* v,
                            float lr, float beta1, float beta2, float eps, float wd, int step, int mode, void* stream);
/* The modified NCCL's mixed-precision LAMB: fp16 gradients (their sum carried in fp16, the square taken in fp16), fp32
 * w, m, v, and an fp16 copy of the new weights in halfw; arithmetic of CCN_LAMB_NCCL_GLOBAL otherwise (per segment,
 * wd in place of the hard-coded 1.0f, no eps, no step).  g: HOST array of P device pointers to fp16 bit patterns.
 * Replaces AllReduce_pipe(lr, beta1, beta2, (half*)g, w, halfw, m, v, r, ...) of nccl/src/nccl.h.in:211-216 for the
 * LAMB build (phase 1 nccl/src/collectives/device/common_kernel.h:2438-2535, phase 2 :2657-2700); the caller's r
 * buffer is not needed: r stays on chip, or phase 2 recomputes it from the stored m and v.  A plan whose segments all fit
 * on chip runs the one-tile kernel, as for fp32 gradients; any other plan runs the two-pass kernels over all its
 * segments (a second tile table is then made on the first call, which therefore allocates and cannot be recorded). */
int  ccn_lamb_nccl_f16g(ccn_lamb_plan* plan, const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v,
                        float lr, float beta1, float beta2, float wd, void* stream);
/* The two-pass step of ccn_lamb_f32 for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  It takes no plan: the tile sums, norms,
 * scales and index tables a plan would own live in a static device array inside the library (about 4.2 MiB, held by every
 * GPU the library runs on until the process ends), and the call makes no hipMalloc, hipFree or other allocating call.
 * Segments are uniform: N / seg_len segments of seg_len elements each; seg_len must be a multiple of 1024 and divide N
 * (CCN_EINVAL otherwise).  Limits: N <= CCN_LAMB_STATIC_MAX_N and N / seg_len <= CCN_LAMB_STATIC_MAX_SEGS, beyond which
 * the call returns CCN_ERANGE and does nothing.  norms: DEVICE array of 2 * (N / seg_len) doubles receiving W_b, R_b, or
 * NULL.  Same arithmetic, kernels and results as ccn_lamb_f32 on a plan whose segments take the two-pass path.
 * All calls on one GPU share the one array: calls that overlap in time on the same GPU (two streams, two threads)
 * race; order them.  ccn_init looks the array's address up; without ccn_init the first call on a device does. */
#define CCN_LAMB_STATIC_MAX_N    ((size_t)1 << 28)
#define CCN_LAMB_STATIC_MAX_SEGS 4096
int  ccn_lamb_f32_static(const float* const* g, int P, float* w, float* m, float* v, size_t N, size_t seg_len,
                         float lr, float beta1, float beta2, float eps, float wd, int step, int mode,
                         double* norms, void* stream);
/* copies W_b, R_b of the last LAMB step on this plan to a HOST array of 2*nseg doubles (synchronises) */
int  ccn_lamb_plan_norms(ccn_lamb_plan* plan, double* norms_host, void* stream);
/* Tuning and diagnostics of a plan (no counterpart in the reference; results do not depend on any of them beyond the
 * association of the float64 norm sums).  Takes effect from the next step on.  value >= 0.
 *   CCN_LAMB_KNOB_SPIN_LIMIT  how long a tile of the on-chip kernel waits for its segment's scale before it leaves its
 *                             update to the trailing kernel (default 32768 polls; 0: every tile is finished by the
 *                             trailing kernel, what a GPU shared with other work degrades to)
 *   CCN_LAMB_KNOB_TWO_PASS    non-zero: every segment takes the two streaming passes, also those short enough to stay on
 *                             chip (the first step after setting it makes a second tile table: it allocates)
 *   CCN_LAMB_KNOB_WITHHOLD    diagnostic: non-zero makes the on-chip kernel compute its scales but never announce them,
 *                             as if a tile sum had not arrived in time, so that the trailing kernel adds every segment up */
#define CCN_LAMB_KNOB_SPIN_LIMIT 0
#define CCN_LAMB_KNOB_TWO_PASS   1
#define CCN_LAMB_KNOB_WITHHOLD   2
int  ccn_lamb_plan_tune(ccn_lamb_plan* plan, int knob, long value);

/* ---- model-parallel MLP out-projection, one rank's K-slice, epilogue fused into the GEMM write-back:
 *      out = bf16( dropout( X[MxK].W[KxN] + sum_q partials[q] + bias[col] ) + resid )
 *      X, W, resid, out: bf16 bit patterns, row-major; partials: HOST array of nPartials device pointers to
 *      fp32 [MxN]; bias fp32 [N]; resid may be NULL.  Dropout: element idx=row*N+col is dropped when
 *      u(seed, idx) < p_drop, survivors are scaled by 1/(1-p_drop); u comes from Philox-4x32-10 with
 *      counter (idx/4, 0) and key seed, word idx%4, u = (word>>8)*2^-24.
 *      Shapes: any M and K; N a multiple of 4 (CCN_ERANGE otherwise).  Whole 128x128x64 tiles with N and K up to 2^21
 *      run on the matrix cores; any other shape takes a vector-ALU kernel that is an order of magnitude slower (the
 *      reference's cuBLAS call takes any shape too).  fp32 arrays 16-byte aligned, bf16 arrays 8-byte aligned (X, W: 16).
 *      Replaces MatMul + AllReduce + (sum+b) + Dropout + r of examples/model-parallel/model-parallel.cpp:18-21
 *      (emitted cublasGemmEx src/codegen.cpp:1058-1136; fused epilogue
 *      nccl-overlap/src/collectives/device/common_kernel.h:1037-1057, reduce_kernel.h:192-213). ---- */
int  ccn_mlp_outproj_bf16(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                          const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K,
                          float p_drop, uint64_t seed, void* stream);

/* ---- standalone epilogue on an fp32 [MxN] product already in memory (the unfused schedule):
 *      out = bf16( dropout( acc + sum_q partials[q] + bias[col] ) + resid ).
 *      Replaces ncclAllReduceDropoutBiasLayernorm (nccl-overlap/src/collectives/all_reduce.cc:78-90). ---- */
int  ccn_bias_dropout_residual(const float* acc, const float* const* partials, int nPartials, const float* bias,
                               const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                               void* stream);

/* ---- the same two calls with the dropout semantics as an argument.  With s = X.W + sum_q partials[q] (or acc + ...),
 *      b = bias[col], r = resid and u the element's uniform draw (the Philox stream above: the reference draws from
 *      cuRAND, whose stream is not reproducible here):
 *        CCN_DROPOUT_INVERTED      out = (u >= p ? (s + b)/(1-p) : 0) + r      what the two calls above compute; p in [0,1)
 *        CCN_DROPOUT_REF_DSL       out = (u <  p ? (s + b) : 0) + r            the reference's emitted expression for
 *                                  Dropout(sum + b, p) + r: keeps with probability p, no rescale (src/codegen.cpp:634-640)
 *        CCN_DROPOUT_REF_NCCL      out = ((u < p ? s : 0) + b) + r             the reference's fused kernel, FuncDropout<T>
 *                                  (nccl-overlap/src/collectives/device/reduce_kernel.h:192-197, common_kernel.h:1037-1057)
 *        CCN_DROPOUT_REF_NCCL_SAT  out = sat(sat((u < p ? s : 0) + b) + r), sat = clamp to [0,1], as its half
 *                                  specialisation adds with __hadd2_sat (reduce_kernel.h:199-213).  The IEEE-half entry
 *                                  points (_f16_ex) also reproduce its roundings: s and b rounded to half, a rounding
 *                                  to half after each add.  The bfloat16 ones (no counterpart there) add in fp32 and
 *                                  round once.
 *      The reference's forms take p in [0,1]: p = 0 keeps nothing, p = 1 everything.
 *      first_row (epilogue call): row of the whole output that row 0 of this call is, for calls that cover a band of
 *      rows each (one rank's slice): the mask of an element depends on its index in the whole output only. ---- */
#define CCN_DROPOUT_INVERTED     0
#define CCN_DROPOUT_REF_DSL      1
#define CCN_DROPOUT_REF_NCCL     2
#define CCN_DROPOUT_REF_NCCL_SAT 3
int  ccn_mlp_outproj_bf16_ex(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                             const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K,
                             float p_drop, uint64_t seed, int dropout_mode, void* stream);
int  ccn_bias_dropout_residual_ex(const float* acc, const float* const* partials, int nPartials, const float* bias,
                                  const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                                  int dropout_mode, size_t first_row, void* stream);

/* ---- the product alone: C[MxN] (fp32, row-major) = X[MxK].W[KxN], bf16 operands, fp32 accumulation on the matrix
 *      cores.  Replaces the emitted cublasGemmEx call of the unfused schedules (matMulK, src/codegen.cpp:1058-1136);
 *      any shape with N a multiple of 4, as for the fused call. ---- */
int  ccn_matmul_bf16_f32(const uint16_t* X, const uint16_t* W, float* C, int M, int N, int K, void* stream);

/* ---- the same three calls with X, W, resid and out in IEEE half instead of bfloat16: the element type the reference's
 *      model-parallel example declares (Float16, examples/model-parallel/model-parallel.cpp:10-15; its cublasGemmEx
 *      multiplies CUDA_R_16F operands, src/codegen.cpp:1058-1136).  Products are accumulated in fp32 on the matrix
 *      cores (v_mfma_f32_32x32x16_f16), where the reference accumulates in half. ---- */
int  ccn_mlp_outproj_f16_ex(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                            const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K,
                            float p_drop, uint64_t seed, int dropout_mode, void* stream);
int  ccn_bias_dropout_residual_f16_ex(const float* acc, const float* const* partials, int nPartials, const float* bias,
                                      const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                                      int dropout_mode, size_t first_row, void* stream);
int  ccn_matmul_f16_f32(const uint16_t* X, const uint16_t* W, float* C, int M, int N, int K, void* stream);

/* ---- the product alone with C in the operands' 16-bit type, as the emitted cublasGemmEx call writes it (its C type is
 *      the output stage's element type, CUDA_R_16F in the reference's example: src/codegen.cpp:1114-1131,
 *      examples/model-parallel/model-parallel.cpp:13-18).  Accumulated in fp32 on the matrix cores and rounded to
 *      nearest even once, where the reference accumulates in half: every element equals the fp32 call's, rounded.
 *      C 8-byte aligned; shapes as for the fp32 calls. ---- */
int  ccn_matmul_bf16(const uint16_t* X, const uint16_t* W, uint16_t* C, int M, int N, int K, void* stream);
int  ccn_matmul_f16(const uint16_t* X, const uint16_t* W, uint16_t* C, int M, int N, int K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* COCONET_HIP_H */
