// Shared device/host helpers of libcoconet_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <new>
#include "coconet_hip.h"

namespace ccn {

constexpr int kBlock = 256;        // 4 wavefronts of 64 lanes
constexpr int kWave = 64;
constexpr size_t kLdsPerCu = 160 * 1024;   // LDS bytes of one gfx950 compute unit

// ---- host-side error plumbing -----------------------------------------------------------------------------------
extern thread_local int g_last_hip_error;
int hip_fail(hipError_t e);                        // records e, returns the CCN_E* code for it
#define CCN_HIP(expr)                                                      \
  do {                                                                     \
    hipError_t _e = (expr);                                                \
    if (_e != hipSuccess) return ::ccn::hip_fail(_e);                      \
  } while (0)

// Runs a host-side body that may allocate host memory (std::vector, std::unordered_map) and turns what it could throw
// into an error code: no exception leaves an extern "C" entry point.
template <class Body>
int guarded(Body&& body) noexcept {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return CCN_ENOMEM;
  } catch (...) {
    return CCN_EINVAL;
  }
}

struct DeviceInfo {
  int device = -1;
  int cu_count = 0;
  size_t hbm_bytes = 0;
  char arch[64] = {0};
};
int current_device_info(const DeviceInfo** out);   // lazily initialises the current device

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---- packs: N elements of T held in registers and moved with 16-byte memory instructions ---------------------------
// (N == 1: one scalar access).  Addresses must be 16-byte aligned when N > 1.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T, int N> struct Pack {
  T d[N];
};

// A pack moves as one scalar (N == 1), one 8-byte piece, or whole 16-byte pieces.
template <typename T, int N> struct PackIo {
  static constexpr int kBytes = N * (int)sizeof(T);
  static_assert(N == 1 || kBytes == 8 || kBytes % 16 == 0, "unsupported pack size");
  template <bool NT> static __device__ __forceinline__ Pack<T, N> load(const T* p) {
    Pack<T, N> r;
    if constexpr (N == 1) {
      r.d[0] = NT ? __builtin_nontemporal_load(p) : *p;
    } else if constexpr (kBytes == 8) {
      const u32x2 x = NT ? __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p)) : *reinterpret_cast<const u32x2*>(p);
      __builtin_memcpy(r.d, &x, 8);
    } else {
#pragma unroll
      for (int c = 0; c < kBytes / 16; c++) {
        const u32x4 x = NT ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p) + c)
                           : *(reinterpret_cast<const u32x4*>(p) + c);
        __builtin_memcpy(reinterpret_cast<char*>(r.d) + 16 * c, &x, 16);
      }
    }
    return r;
  }
  template <bool NT> static __device__ __forceinline__ void store(T* p, const Pack<T, N>& v) {
    if constexpr (N == 1) {
      if constexpr (NT) __builtin_nontemporal_store(v.d[0], p); else *p = v.d[0];
    } else if constexpr (kBytes == 8) {
      u32x2 x;
      __builtin_memcpy(&x, v.d, 8);
      if constexpr (NT) __builtin_nontemporal_store(x, reinterpret_cast<u32x2*>(p)); else *reinterpret_cast<u32x2*>(p) = x;
    } else {
#pragma unroll
      for (int c = 0; c < kBytes / 16; c++) {
        u32x4 x;
        __builtin_memcpy(&x, reinterpret_cast<const char*>(v.d) + 16 * c, 16);
        if constexpr (NT) __builtin_nontemporal_store(x, reinterpret_cast<u32x4*>(p) + c);
        else *(reinterpret_cast<u32x4*>(p) + c) = x;
      }
    }
  }
};

// Streaming (nontemporal) accesses: gradients, partial sums and the optimizer state are touched once per step,
// and a step streams gigabytes past them, so nothing here is worth keeping in the caches.
template <typename T, int N> __device__ __forceinline__ Pack<T, N> load_stream(const T* p) {
  return PackIo<T, N>::template load<true>(p);
}
template <typename T, int N> __device__ __forceinline__ Pack<T, N> load_keep(const T* p) {
  return PackIo<T, N>::template load<false>(p);
}
template <typename T, int N> __device__ __forceinline__ void store_stream(T* p, const Pack<T, N>& v) {
  PackIo<T, N>::template store<true>(p, v);
}
template <typename T, int N> __device__ __forceinline__ void store_pack(T* p, const Pack<T, N>& v) {
  PackIo<T, N>::template store<false>(p, v);
}

// ---- table of P source pointers, passed by value in the kernel argument segment ----------------------------------
template <typename T, int CAP> struct SrcTable { const T* p[CAP]; };

// ---- wavefront / workgroup reductions (64-wide) -------------------------------------------------------------------
__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, kWave);
  return x;   // valid in lane 0
}

// Sum of `x` over a kBlock-thread workgroup; result valid in thread 0.  lds must hold kBlock/kWave doubles.
__device__ __forceinline__ double block_sum(double x, double* lds) {
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  x = wave_sum(x);
  if (lane == 0) lds[wv] = x;
  __syncthreads();
  double r = 0.0;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < kBlock / kWave; k++) r += lds[k];
  }
  __syncthreads();
  return r;
}

// ---- half / bfloat16 scalars -----------------------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  _Float16 x = __builtin_bit_cast(_Float16, h);
  return (float)x;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {   // round-to-nearest-even
  _Float16 x = (_Float16)f;
  return __builtin_bit_cast(uint16_t, x);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
// round-to-nearest-even, quiet nan; the rounded word with the bfloat16 in its upper half (selects, no branch: the
// epilogues convert four values per quad and stay one basic block)
__device__ __forceinline__ uint32_t f32_to_bf16_hi(float f) {
  const uint32_t x = __float_as_uint(f);
  const uint32_t r = x + 0x7fffu + ((x >> 16) & 1u);
  return f != f ? (x | 0x00400000u) : r;
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(f32_to_bf16_hi(f) >> 16); }

// ---- Philox-4x32-10, and the dropout keep decision built on it -----------------------------------------------------
struct Philox4 { uint32_t x, y, z, w; };
__host__ __device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                          uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return Philox4{c0, c1, c2, c3};
}
__host__ __device__ __forceinline__ bool keep_from_word(uint32_t word, float p_drop) {
  const float u = (float)(word >> 8) * 5.9604644775390625e-08f;
  return u >= p_drop;
}
// The same decision on integers: u = k * 2^-24 with k = word >> 8 is exact, so u >= p  <=>  k >= ceil(p * 2^24)
// (p * 2^24 is exact in double).  The host computes the threshold once per launch; 2^24 (p = 1) means "never".
inline uint32_t keep_threshold(float p_drop) {
  const double t = (double)p_drop * 16777216.0;
  const double c = (double)(uint64_t)t;
  return (uint32_t)(c < t ? c + 1.0 : c);
}
__device__ __forceinline__ bool keep_from_threshold(uint32_t word, uint32_t thr) { return (word >> 8) >= thr; }

// ---- launch geometry for streaming kernels ----------------------------------------------------------------------------
// Number of workgroups for a grid-stride kernel whose workgroup consumes `tile` units per iteration
// (a few workgroups per CU; used by the small helper kernels).
unsigned stream_grid(size_t units, size_t tile);

// Geometry of the fused reduce+update kernels: one workgroup per tile, no loop, and a cap on the wavefronts resident
// per CU, enforced by requesting dynamic LDS that the kernel never touches.  HBM sustains the most bandwidth when the
// number of address streams times the wavefronts in flight stays moderate.  Measured on MI355X for the 14-stream
// kernel (8 gradients, w/m/v in, w/m/v out; N = 2^28): full occupancy 72-75% of peak; 8 wavefronts per CU as two
// 256-thread workgroups 82%; 7 wavefronts per CU as single-wavefront workgroups 85%; 4 wavefronts 63-70%.  A 2-stream
// copy wants all the occupancy it can get.
struct StreamShape { int block; unsigned lds_bytes; };
// Shape for a kernel whose threads each load `load_bytes` and store `store_bytes`, one pack per array; `grad_bytes` is
// the element size of the gradient arrays (narrow elements mean more load instructions for the same bytes);
// `starts_alike`: most of the arrays start at the same offset within 64 KiB, so a thread's loads meet on one HBM channel.
StreamShape stream_shape(int load_bytes, int store_bytes, int grad_bytes = 4, bool starts_alike = false);
// Dynamic LDS request that keeps at most `per_cu` workgroups on a CU (0 = no request).
unsigned lds_for_residency(int per_cu);

// Looks up, once per device and with that device current, the device address of the static scratch array behind
// ccn_lamb_f32_static, so that the entry point itself never has to (it may run under stream capture).
int lamb_static_setup();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace ccn
