// Runtime part of programs emitted by the HIP code-generation target.
//
// The code generator writes, per fused group of pipeline stages, a small "body" struct holding the user's
// expressions as straight-line per-element code.  Everything that decides performance is hand-written here and
// shared by all generated programs: the streaming kernel (16-byte packs, every load of a thread issued before the
// first use, P-way gradient fold in ascending rank order, capped workgroup residency), the workgroup reductions
// for norms, and the launch logic.  Generated programs talk to the device only through the C ABI of
// libcoconet_hip (memory, events, the stock reduce) and hipLaunchKernelGGL for their own kernels.
#ifndef CCN_CODEGEN_RT_HPP
#define CCN_CODEGEN_RT_HPP

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

#include "coconet_hip.h"

#define CCNCHECK(cmd)                                                                              \
  do {                                                                                             \
    int _rc = (cmd);                                                                               \
    if (_rc != CCN_OK) {                                                                           \
      printf("Failed, coconet_hip error %s:%d '%s'\n", __FILE__, __LINE__, ccn_strerror(_rc));     \
      exit(EXIT_FAILURE);                                                                          \
    }                                                                                              \
  } while (0)

#define HIPCHECK(cmd)                                                                              \
  do {                                                                                             \
    hipError_t _e = (cmd);                                                                         \
    if (_e != hipSuccess) {                                                                        \
      printf("Failed: HIP error %s:%d '%s'\n", __FILE__, __LINE__, hipGetErrorString(_e));         \
      exit(EXIT_FAILURE);                                                                          \
    }                                                                                              \
  } while (0)

#define DIVUP(x, y) (((x) + (y)-1) / (y))

namespace ccn_gen {

constexpr int kBlock = 256;
constexpr int kWave = 64;
constexpr int kMaxRanks = CCN_MAX_RANKS;

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int N> struct Vals { float d[N]; };

template <int VEC> __device__ __forceinline__ Vals<VEC> load_vals(const float* p) {
  Vals<VEC> r;
  if constexpr (VEC == 1) {
    r.d[0] = __builtin_nontemporal_load(p);
  } else {
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    r.d[0] = x[0]; r.d[1] = x[1]; r.d[2] = x[2]; r.d[3] = x[3];
  }
  return r;
}
// fp16 gradients (stored as raw 16-bit patterns): widened to fp32 on load, four at a time from one 8-byte access.
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
__host__ __device__ inline float f16_bits_to_f32(uint16_t h) {
  _Float16 x;
  memcpy(&x, &h, 2);
  return (float)x;
}
template <int VEC> __device__ __forceinline__ Vals<VEC> load_vals(const uint16_t* p) {
  Vals<VEC> r;
  if constexpr (VEC == 1) {
    r.d[0] = f16_bits_to_f32(__builtin_nontemporal_load(p));
  } else {
    const u32x2 x = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    r.d[0] = f16_bits_to_f32((uint16_t)(x[0] & 0xffffu)); r.d[1] = f16_bits_to_f32((uint16_t)(x[0] >> 16));
    r.d[2] = f16_bits_to_f32((uint16_t)(x[1] & 0xffffu)); r.d[3] = f16_bits_to_f32((uint16_t)(x[1] >> 16));
  }
  return r;
}
__device__ __forceinline__ float load_one(const float* p) { return *p; }
__device__ __forceinline__ float load_one(const uint16_t* p) { return f16_bits_to_f32(*p); }

__host__ __device__ inline uint16_t f32_to_f16_bits(float f) {
  const _Float16 x = (_Float16)f;
  uint16_t h;
  memcpy(&h, &x, 2);
  return h;
}
template <int VEC> __device__ __forceinline__ void store_vals(uint16_t* p, const Vals<VEC>& v) {
  if constexpr (VEC == 1) {
    __builtin_nontemporal_store(f32_to_f16_bits(v.d[0]), p);
  } else {
    u32x2 x;
    x[0] = (unsigned)f32_to_f16_bits(v.d[0]) | ((unsigned)f32_to_f16_bits(v.d[1]) << 16);
    x[1] = (unsigned)f32_to_f16_bits(v.d[2]) | ((unsigned)f32_to_f16_bits(v.d[3]) << 16);
    __builtin_nontemporal_store(x, reinterpret_cast<u32x2*>(p));
  }
}
template <int VEC> __device__ __forceinline__ void store_vals(float* p, const Vals<VEC>& v) {
  if constexpr (VEC == 1) {
    __builtin_nontemporal_store(v.d[0], p);
  } else {
    f32x4 x;
    x[0] = v.d[0]; x[1] = v.d[1]; x[2] = v.d[2]; x[3] = v.d[3];
    __builtin_nontemporal_store(x, reinterpret_cast<f32x4*>(p));
  }
}

// ---- counter-based dropout mask: Philox-4x32-10 on (seed, element index / 4), word index % 4 ---------------------
__host__ __device__ inline void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1, uint32_t out[4]) {
  uint32_t c2 = 0, c3 = 0;
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
__host__ __device__ inline bool dropout_keep(uint64_t seed, uint64_t idx, float p_drop) {
  uint32_t w[4];
  const uint64_t blk = idx >> 2;
  philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)seed, (uint32_t)(seed >> 32), w);
  const float u = (float)(w[idx & 3] >> 8) * 5.9604644775390625e-08f;
  return u >= p_drop;
}
// Dropout as the emitted expressions use it: drop with probability p, scale survivors by 1/(1-p).
__host__ __device__ inline float dropout(float x, float p_drop, uint64_t seed, uint64_t idx) {
  return dropout_keep(seed, idx, p_drop) ? x * (1.0f / (1.0f - p_drop)) : 0.0f;
}

// The reference's form of the same stage (src/codegen.cpp:634-640): keep with probability p, no rescale.
__host__ __device__ inline float dropout_ref(float x, float p_keep, uint64_t seed, uint64_t idx) {
  return !dropout_keep(seed, idx, p_keep) ? x : 0.0f;   // kept where u < p
}
// One output element of the MLP epilogue from the sum s over the ranks' products, bias b and residual r, under dropout
// form `mode` (CCN_DROPOUT_* of coconet_hip.h); host mirror of the library's epilogue for the emitted self-check.
// half: the operands are IEEE half; the saturating form then rounds to half after each add, as the library does.
inline float epilogue_value(float s, float b, float r, float p, uint64_t seed, uint64_t idx, int mode, bool half = false) {
  auto sat = [](float x) { return x > 0.0f ? (x < 1.0f ? x : 1.0f) : 0.0f; };
  auto h16 = [](float x) { return f16_bits_to_f32(f32_to_f16_bits(x)); };
  if (mode == CCN_DROPOUT_INVERTED) {
    const float t = s + b;
    const float d = p > 0.0f ? dropout(t, p, seed, idx) : t;
    return d + r;
  }
  const bool kept = !dropout_keep(seed, idx, p);
  if (mode == CCN_DROPOUT_REF_DSL) {
    const float t = s + b;
    return (kept ? t : 0.0f) + r;
  }
  const float d = kept ? s : 0.0f;
  if (mode == CCN_DROPOUT_REF_NCCL_SAT && half) return sat(h16(sat(h16(d) + h16(b))) + r);
  return mode == CCN_DROPOUT_REF_NCCL_SAT ? sat(sat(d + b) + r) : (d + b) + r;
}

// ---- reductions ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, kWave);
  return x;
}
// Sum over a workgroup of BS threads (BS = kWave: one wavefront, no LDS); valid in thread 0.
template <int BS = kBlock> __device__ __forceinline__ double block_sum(double x, double* lds) {
  x = wave_sum(x);
  if constexpr (BS == kWave) return x;
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = x;
  __syncthreads();
  double r = 0.0;
  if (threadIdx.x == 0)
    for (int k = 0; k < BS / kWave; k++) r += lds[k];
  __syncthreads();
  return r;
}

// ---- kernel arguments ---------------------------------------------------------------------------------------------
// A generated Body declares:
//   NIN        plain fp32 input arrays, read at the element index
//   NOUT       output arrays (an in-place update lists the array under both); fp32, except those whose bit is set
//   OUT_F16    in this mask: they hold fp16 (the body has already rounded the value to fp16, the store narrows it)
//   HAS_RED    the body's first operand is the sum over rank buffers (the lowered AllReduce / ReduceScatter)
//   RedT       element type of those buffers: float, or uint16_t holding fp16 bits (widened, then summed in fp32)
//   NACC       sums of squares the body accumulates (inputs of Norm stages), float64
//   NNORM      finished norms the body reads
//   struct Scalars
//   static void apply(float red, const float* in, float* out, const Scalars&, double* acc, const float* norms, uint64_t idx)
template <class Body> struct KernelArgs {
  const typename Body::RedT* red[kMaxRanks];
  int nranks;
  const float* in[Body::NIN > 0 ? Body::NIN : 1];
  void* out[Body::NOUT > 0 ? Body::NOUT : 1];
  double* partials;      // NACC values per workgroup
  const float* norms;    // NNORM values
  size_t n;
  size_t idx_base;       // index of element 0 in the whole tensor (a launch over one rank's slice starts at its offset):
                         // what index-dependent expressions (the dropout mask) see is idx_base + the element's position
  typename Body::Scalars s;
};

// One pack of VEC elements per thread and no loop: a workgroup issues every load of its tile at once and leaves.
// BS = kWave (single-wavefront workgroups) for kernels that walk many arrays, kBlock for copy-like ones.
template <class Body, int P, int VEC, int BS>
__global__ __launch_bounds__(BS) void fused_pointwise_kernel(const KernelArgs<Body> a) {
  constexpr int NINX = Body::NIN > 0 ? Body::NIN : 1;
  constexpr int NOUTX = Body::NOUT > 0 ? Body::NOUT : 1;
  constexpr int NACCX = Body::NACC > 0 ? Body::NACC : 1;
  constexpr int PX = P > 0 ? P : kMaxRanks;
  __shared__ double lds[kBlock / kWave];
  const size_t nvec = a.n / VEC;
  double acc[NACCX];
#pragma unroll
  for (int k = 0; k < NACCX; k++) acc[k] = 0.0;
  float nrm[Body::NNORM > 0 ? Body::NNORM : 1];
#pragma unroll
  for (int k = 0; k < Body::NNORM; k++) nrm[k] = a.norms[k];

  const size_t i = (size_t)blockIdx.x * BS + threadIdx.x;
  if (i < nvec) {
    const size_t e0 = i * VEC;
    Vals<VEC> rv[PX];
    Vals<VEC> iv[NINX];
    if constexpr (Body::HAS_RED) {   // P = 0: the first nranks of kMaxRanks, a wave-uniform choice
#pragma unroll
      for (int p = 0; p < PX; p++) {
        if (P > 0 || p < a.nranks) rv[p] = load_vals<VEC>(a.red[p] + e0);
      }
    }
#pragma unroll
    for (int k = 0; k < Body::NIN; k++) iv[k] = load_vals<VEC>(a.in[k] + e0);
    Vals<VEC> red;
    if constexpr (Body::HAS_RED) {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        float s = rv[0].d[e];
#pragma unroll
        for (int p = 1; p < PX; p++) {
          if (P > 0 || p < a.nranks) s = s + rv[p].d[e];
        }
        red.d[e] = s;
      }
    }
    Vals<VEC> ov[NOUTX];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float in1[NINX], out1[NOUTX];
#pragma unroll
      for (int k = 0; k < Body::NIN; k++) in1[k] = iv[k].d[e];
      Body::apply(Body::HAS_RED ? red.d[e] : 0.0f, in1, out1, a.s, acc, nrm, (uint64_t)(a.idx_base + e0 + e));
#pragma unroll
      for (int k = 0; k < Body::NOUT; k++) ov[k].d[e] = out1[k];
    }
#pragma unroll
    for (int k = 0; k < Body::NOUT; k++) {
      if ((Body::OUT_F16 >> k) & 1u) store_vals<VEC>(static_cast<uint16_t*>(a.out[k]) + e0, ov[k]);
      else store_vals<VEC>(static_cast<float*>(a.out[k]) + e0, ov[k]);
    }
  }

  if constexpr (VEC > 1) {   // the last n % VEC elements, scalar, by the first lanes of workgroup 0
    const size_t rem = a.n - nvec * VEC;
    if (blockIdx.x == 0 && threadIdx.x < rem) {
      const size_t i = nvec * VEC + threadIdx.x;
      float red = 0.0f;
      if constexpr (Body::HAS_RED) {
        red = load_one(a.red[0] + i);
        for (int p = 1; p < a.nranks; p++) red = red + load_one(a.red[p] + i);
      }
      float in1[NINX], out1[NOUTX];
      for (int k = 0; k < Body::NIN; k++) in1[k] = a.in[k][i];
      Body::apply(red, in1, out1, a.s, acc, nrm, (uint64_t)(a.idx_base + i));
      for (int k = 0; k < Body::NOUT; k++) {
        if ((Body::OUT_F16 >> k) & 1u) static_cast<uint16_t*>(a.out[k])[i] = f32_to_f16_bits(out1[k]);
        else static_cast<float*>(a.out[k])[i] = out1[k];
      }
    }
  }

  if constexpr (Body::NACC > 0) {
#pragma unroll
    for (int k = 0; k < Body::NACC; k++) {
      const double s = block_sum<BS>(acc[k], lds);
      if (threadIdx.x == 0) a.partials[(size_t)blockIdx.x * Body::NACC + k] = s;
    }
  }
}

// First level of the norm reduction for large launches: workgroup b adds rows [b*rows, (b+1)*rows) of the partial
// sums, thread t taking rows t, t+256, ... in ascending order, into row b of `out`.  Fixed order: deterministic.
__global__ __launch_bounds__(kBlock) void fold_partials_kernel(const double* partials, unsigned nblocks, unsigned rows, int nacc,
                                                               double* out) {
  __shared__ double lds[kBlock / kWave];
  const size_t lo = (size_t)blockIdx.x * rows;
  const size_t hi = lo + rows < nblocks ? lo + rows : nblocks;
  for (int k = 0; k < nacc; k++) {
    double s = 0.0;
    for (size_t b = lo + threadIdx.x; b < hi; b += kBlock) s += partials[b * nacc + k];
    const double t = block_sum(s, lds);
    if (threadIdx.x == 0) out[(size_t)blockIdx.x * nacc + k] = t;
  }
}

// norms[k] = the sum over workgroups of partials[b*nacc + k], or its square root where bit k of sqrt_mask is set;
// one workgroup, fixed order: deterministic.
__global__ __launch_bounds__(kBlock) void finalize_norms_kernel(const double* partials, unsigned nblocks, int nacc,
                                                                unsigned sqrt_mask, float* norms) {
  __shared__ double lds[kBlock / kWave];
  for (int k = 0; k < nacc; k++) {
    double s = 0.0;
    for (unsigned b = threadIdx.x; b < nblocks; b += kBlock) s += partials[(size_t)b * nacc + k];
    const double t = block_sum(s, lds);
    if (threadIdx.x == 0) norms[k] = (float)(((sqrt_mask >> k) & 1u) ? sqrt(t) : t);
  }
}

// ---- host side ------------------------------------------------------------------------------------------------------
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Launch shape for a kernel whose threads load `loads` and store `stores` 16-byte packs, from measurements on MI355X
// at 2^28 elements: single-wavefront workgroups, and fewer of them per CU the more loads a thread has in flight
// (26 up to 2 loads, 20 up to 4, 11 or 12 up to 7, 7 up to 10, 6 up to 13, 8 beyond: from 8 loads on one fewer than the
// library's kernels of the same shape, whose double-precision bias correction keeps a wavefront busy for longer), the
// cap expressed as unused dynamic LDS.  Scalar (unaligned) launches keep 256 threads.
struct LaunchShape {
  int block;
  unsigned lds;
};
inline LaunchShape shape_for(int loads, int stores, int vec, bool has_sums = false, int grad_bytes = 4) {
  LaunchShape sh{kBlock, 0};
  if (vec == 1) return sh;
  // wavefronts per CU by 16-byte loads per thread, measured at N = 2^28: 2 -> 26, 3-4 -> 20, 5-7 -> 11-13 (the library's
  // table: by the number of stores and the width of the gradient loads; the fp16-gradient Adam program: 1.753 ms per
  // epoch at 11, 1.776 at 12, 1.795 at 13), 8-10 -> 7, 11-13 -> 6
  const int mid = stores <= 1 ? (loads == 7 ? 11 : 13) : (grad_bytes == 2 ? (loads == 7 ? 11 : 12) : (loads <= 6 ? 11 : 12));
  const int waves = loads <= 2 ? 26 : (loads <= 4 ? 20 : (loads <= 7 ? mid : (loads <= 10 ? 7 : (loads <= 13 ? 6 : 8))));
  sh.block = kWave;
  sh.lds = ((160u * 1024u / (unsigned)waves) / 1024u) * 1024u;
  if (has_sums) {   // float64 sums and a workgroup reduction: four 256-thread workgroups per CU hide them better
    sh.block = kBlock;   // (emitted LAMB at N = 2^28, P = 8: 3.02 ms per epoch against 3.07 ms with the shape above)
    sh.lds = 40u * 1024u;
  }
  return sh;
}

inline unsigned grid_for(size_t n, int vec, int block) {
  size_t need = DIVUP(n / vec > 0 ? n / vec : 1, (size_t)block);
  return (unsigned)(need < 0x7fffffffull ? need : 0x7fffffffull);
}

template <class Body, int VEC> unsigned launch_vec(const KernelArgs<Body>& a, hipStream_t s) {
  // 16-byte loads per thread: an fp16 gradient pack is half of one
  const int red_loads = Body::HAS_RED ? (a.nranks * (int)sizeof(typename Body::RedT) + 3) / 4 : 0;
  const LaunchShape sh = shape_for(red_loads + Body::NIN, Body::NOUT, VEC, Body::NACC > 0, Body::HAS_RED ? (int)sizeof(typename Body::RedT) : 4);
  const unsigned grid = grid_for(a.n, VEC, sh.block);
  const int P = Body::HAS_RED ? a.nranks : 1;
  auto go = [&](auto ptag) {
    constexpr int PP = decltype(ptag)::value;
    if (sh.block == kWave)
      hipLaunchKernelGGL((fused_pointwise_kernel<Body, PP, VEC, kWave>), dim3(grid), dim3(kWave), sh.lds, s, a);
    else
      hipLaunchKernelGGL((fused_pointwise_kernel<Body, PP, VEC, kBlock>), dim3(grid), dim3(kBlock), sh.lds, s, a);
  };
  switch (P) {
#define CCN_GEN_CASE(K) case K: go(std::integral_constant<int, K>{}); break;
    CCN_GEN_CASE(1) CCN_GEN_CASE(2) CCN_GEN_CASE(3) CCN_GEN_CASE(4) CCN_GEN_CASE(5) CCN_GEN_CASE(6) CCN_GEN_CASE(7)
    CCN_GEN_CASE(8)
#undef CCN_GEN_CASE
    default: go(std::integral_constant<int, 0>{}); break;
  }
  HIPCHECK(hipGetLastError());
  return grid;
}

// An upper bound on the workgroups launch() uses for n elements, whatever the shape (the partials array holds NACC
// values per workgroup): scalar launches have 256 threads, vector launches at least 64 threads of 4 elements.
// (launched slice by slice, every rank's launch rounds up on its own: kMaxRanks more)
inline unsigned blocks_for(size_t n) { return grid_for(n, 1, kBlock) + (unsigned)kMaxRanks; }

// Launches the kernel and returns the number of workgroups used: that many rows of NACC partial sums are written.
template <class Body> unsigned launch(const KernelArgs<Body>& a, void* stream) {
  if (a.n == 0) return 0;
  bool al = true;
  if (Body::HAS_RED)   // a pack of four is 16 bytes of fp32 or 8 bytes of fp16
    for (int p = 0; p < a.nranks; p++) al = al && ((uintptr_t)a.red[p] & (4 * sizeof(typename Body::RedT) - 1)) == 0;
  for (int k = 0; k < Body::NIN; k++) al = al && aligned16(a.in[k]);
  for (int k = 0; k < Body::NOUT; k++)   // a pack of four is 16 bytes of fp32 or 8 bytes of fp16
    al = al && ((uintptr_t)a.out[k] & (((Body::OUT_F16 >> k) & 1u) ? 7u : 15u)) == 0;
  if (al) return launch_vec<Body, 4>(a, (hipStream_t)stream);
  return launch_vec<Body, 1>(a, (hipStream_t)stream);
}

// Rows of the scratch area behind the partial sums that finalize_norms folds large launches into.
constexpr unsigned kFoldRows = 8192;
// Doubles to allocate for the partial sums of launches over up to n elements (8 accumulators at most).
inline size_t partials_doubles(size_t n) { return ((size_t)blocks_for(n) + kFoldRows) * 8; }

// norms[k] = the sum of the nblocks partial sums of accumulator k, or its square root.  A single workgroup would take 2 ms to read
// the 2^20 rows of a 2^28-element launch, so beyond 4096 rows a first level folds them, 4096 or more rows per
// workgroup, into the scratch rows at partials + blocks_for(n) * 8.
inline void finalize_norms(const double* partials, double* scratch, unsigned nblocks, int nacc, unsigned sqrt_mask,
                           float* norms, void* stream) {
  if (nblocks > 4096) {
    unsigned rows = (nblocks + kFoldRows - 1) / kFoldRows;
    if (rows < 4096) rows = 4096;
    const unsigned folded = (nblocks + rows - 1) / rows;
    hipLaunchKernelGGL(fold_partials_kernel, dim3(folded), dim3(kBlock), 0, (hipStream_t)stream, partials, nblocks, rows, nacc,
                       scratch);
    HIPCHECK(hipGetLastError());
    partials = scratch;
    nblocks = folded;
  }
  hipLaunchKernelGGL(finalize_norms_kernel, dim3(1), dim3(kBlock), 0, (hipStream_t)stream, partials, nblocks, nacc, sqrt_mask,
                     norms);
  HIPCHECK(hipGetLastError());
}

// ---- input generation and checking (host) ----------------------------------------------------------------------------
// The reference fills inputs with cuRAND uniform(0,1), seed 1234 (examples/header.h:64-76); cuRAND is not
// available, so a splitmix64 stream with the same seed and range takes its place.
inline float uniform01(uint64_t seed, uint64_t i) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * (i + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (float)((z >> 40) + 1) * 5.9604644775390625e-08f;   // (0, 1]
}

inline void fill_uniform(float* dev, size_t n, uint64_t seed, std::vector<float>* keep = nullptr) {
  std::vector<float> h(n);
  for (size_t i = 0; i < n; i++) h[i] = uniform01(seed, i);
  CCNCHECK(ccn_memcpy_h2d(dev, h.data(), n * sizeof(float), nullptr));
  CCNCHECK(ccn_stream_sync(nullptr));
  if (keep) keep->swap(h);
}

// fp16 inputs: the same uniform stream rounded to fp16 (round to nearest even); `keep` receives the rounded values
// widened back to fp32, which is what the kernels see.
inline void fill_uniform_f16(uint16_t* dev, size_t n, uint64_t seed, std::vector<float>* keep = nullptr) {
  std::vector<uint16_t> h(n);
  std::vector<float> wide(keep ? n : 0);
  for (size_t i = 0; i < n; i++) {
    const _Float16 x = (_Float16)uniform01(seed, i);
    memcpy(&h[i], &x, 2);
    if (keep) wide[i] = (float)x;
  }
  CCNCHECK(ccn_memcpy_h2d(dev, h.data(), n * sizeof(uint16_t), nullptr));
  CCNCHECK(ccn_stream_sync(nullptr));
  if (keep) keep->swap(wide);
}

// relative comparison in the spirit of the reference's eqFloat (examples/header.h:55-62), with a tighter bound:
// the emitted kernels round exactly like the emitted host loops except for the association of norm sums.
inline bool eqFloat(float ref, float got, float tol = 1e-5f) {
  if (ref == got) return true;
  if (std::isnan(ref) || std::isnan(got)) return std::isnan(ref) && std::isnan(got);
  const float den = std::fabs(ref) > 1e-30f ? std::fabs(ref) : 1e-30f;
  return std::fabs(ref - got) / den <= tol;
}

// Host half of the comparison: reports the first element that differs by more than tol (relative).
inline bool compare_host(const char* what, const std::vector<float>& ref, const std::vector<float>& got, float tol) {
  for (size_t i = 0; i < ref.size(); i++) {
    if (!eqFloat(ref[i], got[i], tol)) {
      printf("Mismatch in %s at %zu : ref '%.9g', computed '%.9g'\n", what, i, ref[i], got[i]);
      return false;
    }
  }
  return true;
}

inline bool compare(const char* what, const std::vector<float>& ref, const float* dev, size_t n, float tol = 1e-5f) {
  std::vector<float> got(n);
  CCNCHECK(ccn_memcpy_d2h(got.data(), dev, n * sizeof(float), nullptr));
  return compare_host(what, ref, got, tol);
}

// fp16 outputs: widened and compared like fp32 ones
inline bool compare(const char* what, const std::vector<float>& ref, const uint16_t* dev, size_t n, float tol = 1e-5f) {
  std::vector<uint16_t> got(n);
  CCNCHECK(ccn_memcpy_d2h(got.data(), dev, n * sizeof(uint16_t), nullptr));
  std::vector<float> wide(n);
  for (size_t i = 0; i < n; i++) wide[i] = f16_bits_to_f32(got[i]);
  return compare_host(what, ref, wide, tol);
}

// ---- options of the emitted main(), all from the environment ---------------------------------------------------------
inline size_t env_size(const char* name, size_t dflt) {
  const char* e = getenv(name);
  if (!e || !*e) return dflt;
  char* end = nullptr;
  const unsigned long long x = strtoull(e, &end, 10);
  return end && *end == 0 ? (size_t)x : dflt;
}
// The sizes a dimension variable takes: the one value of the environment variable when it is set, else the defaults.
inline std::vector<size_t> env_sizes(const char* name, std::vector<size_t> dflt) {
  const size_t x = env_size(name, 0);
  return x ? std::vector<size_t>{x} : dflt;
}
inline float env_float(const char* name, float dflt) {
  const char* e = getenv(name);
  if (!e || !*e) return dflt;
  char* end = nullptr;
  const float x = strtof(e, &end);
  return end && *end == 0 ? x : dflt;
}
// Writes n elements of a device array to <prefix>.<name>.<n>.f32 (fp16 arrays widened), raw little-endian floats.
inline void dump_host(const char* prefix, const char* name, const std::vector<float>& h) {
  char path[1024];
  snprintf(path, sizeof(path), "%s.%s.%zu.f32", prefix, name, h.size());
  FILE* f = fopen(path, "wb");
  if (!f || fwrite(h.data(), sizeof(float), h.size(), f) != h.size()) {
    printf("Error writing %s\n", path);
    exit(EXIT_FAILURE);
  }
  fclose(f);
}
inline void dump(const char* prefix, const char* name, const float* dev, size_t n) {
  std::vector<float> h(n);
  CCNCHECK(ccn_memcpy_d2h(h.data(), dev, n * sizeof(float), nullptr));
  dump_host(prefix, name, h);
}
inline void dump(const char* prefix, const char* name, const uint16_t* dev, size_t n) {
  std::vector<uint16_t> h(n);
  CCNCHECK(ccn_memcpy_d2h(h.data(), dev, n * sizeof(uint16_t), nullptr));
  std::vector<float> wide(n);
  for (size_t i = 0; i < n; i++) wide[i] = f16_bits_to_f32(h[i]);
  dump_host(prefix, name, wide);
}
// Corrupts element i of a device array (adds one part in a thousand, or 1 to a zero): what the comparison must catch.
inline void perturb(float* dev, size_t i) {
  float x;
  CCNCHECK(ccn_memcpy_d2h(&x, dev + i, sizeof(float), nullptr));
  x = x != 0.0f ? x * 1.001f : 1.0f;
  CCNCHECK(ccn_memcpy_h2d(dev + i, &x, sizeof(float), nullptr));
  CCNCHECK(ccn_stream_sync(nullptr));
}

// ---- bf16 on the host (round-to-nearest-even), for programs that feed the MFMA GEMM ---------------------------------
inline uint16_t f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}
inline float bf16_to_f32(uint16_t h) {
  const uint32_t x = (uint32_t)h << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

}  // namespace ccn_gen

#endif
