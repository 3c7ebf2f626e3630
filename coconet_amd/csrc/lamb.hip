// LAMB with per-segment trust ratio.  The update of a segment needs the segment's two norms, which need every element
// of the segment first, so each element is visited twice.  A plan sorts the segments into two groups:
//
// resident segments (short enough for the chip to hold between the visits: half the tiles the GPU runs at once, 3 M
//   elements at the default shape) go through lamb_oneshot_kernel, one tile per workgroup.  A workgroup runs pass 1
//   on its tile (P-way gradient reduce, m/v update, r, the tile's float64 sums of w^2 and r^2), keeps r in registers
//   and the old w in LDS, waits until the workgroup that finished the segment's last tile has published the scale,
//   and writes w from what it kept: 56 bytes per element instead of 68.  No sum is an atomic accumulation: tile sums
//   are stored one by one and added in a fixed order, so results do not depend on scheduling.
// the other segments take two streaming passes with a finalize kernel between them:
//   pass 1   one workgroup per tile of kLambTile elements, one 4-element pack per thread
//   finalize one workgroup per segment: fixed-order sum of the segment's tile pairs, norms, scale
//   pass 2   one workgroup per tile: r recomputed from the stored m, v and the old w; w updated
// Arithmetic follows nccl-overlap/samples/multi-process-adam-scattered.cpp:402-449 statement by statement.
#include "ccn_common.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <type_traits>
#include <vector>

namespace ccn {

constexpr int kLambTile = kBlock * 4;   // 1024 elements: one float4 per thread

struct LambTile {
  uint64_t start;   // first element
  uint32_t count;   // elements in the tile (<= kLambTile)
  uint32_t seg;     // segment the tile belongs to
  float nf;         // (float) element count of that segment
  uint32_t buf;     // buffer the tile lies in: index into the pointer tables of the scattered layout (== seg unless a
                    // segment is made of several buffers)
  uint32_t pad[2];
};
static_assert(sizeof(LambTile) == 32, "tile record is 32 bytes");

// Segments of one common length that is a multiple of the tile need no table: tile -> segment by division.
struct LambLayout {
  const LambTile* tiles;    // used when seg_len == 0
  uint64_t seg_len;         // common segment length, or 0 for a ragged layout
  float seg_len_f;
  uint32_t tile;            // elements per full tile
  // Scattered buffers (one gradient / weight buffer per segment, moments still in single arrays): device tables of the
  // segments' pointers, each already moved back by the segment's first element index, so that "pointer + global element
  // index" addresses the segment's elements exactly as it does for flat arrays.  Null for flat arrays.
  const float* const* gtab;   // [P][nbuf], rank-major
  float* const* wtab;         // [nbuf]
  uint32_t nbuf;              // buffers (== segments unless a segment is made of several buffers)
};

// Gradient table and weight pointer to use for the elements of buffer `buf`.
// SCAT is a compile-time choice so that the flat kernels carry none of this.
template <int P, bool SCAT>
__device__ __forceinline__ void lamb_buffers_of(const LambLayout& L, const SrcTable<float, (P ? P : CCN_MAX_RANKS)>& g_flat,
                                                float* w_flat, int nP, uint32_t buf,
                                                SrcTable<float, (P ? P : CCN_MAX_RANKS)>& g, float*& w) {
  if constexpr (!SCAT) {
    g = g_flat;
    w = w_flat;
    return;
  }
  constexpr int PX = P > 0 ? P : CCN_MAX_RANKS;
#pragma unroll
  for (int p = 0; p < PX; p++) g.p[p] = (P > 0 || p < nP) ? L.gtab[(size_t)p * L.nbuf + buf] : nullptr;
  w = L.wtab[buf];
}
template <bool SCAT>
__device__ __forceinline__ float* lamb_weights_of(const LambLayout& L, float* w_flat, uint32_t buf) {
  if constexpr (SCAT) return L.wtab[buf];
  return w_flat;
}

__device__ __forceinline__ LambTile lamb_tile_of(const LambLayout& L, unsigned b) {
  if (L.seg_len != 0) {
    LambTile t;
    t.start = (uint64_t)b * L.tile;
    t.count = L.tile;
    t.seg = (uint32_t)(t.start / L.seg_len);
    t.buf = t.seg;
    t.nf = L.seg_len_f;
    return t;
  }
  return L.tiles[b];
}

struct LambPrm {
  float b1, omb1, b2, omb2, eps, wd, lr;
  int mode;
  double bc1, bc2;
};

__device__ __forceinline__ float lamb_r(float mi, float vi, float w, const LambPrm& k) {
  if (k.mode == CCN_LAMB_NCCL_GLOBAL) return ((mi / k.b1)) / sqrtf((vi / k.b2)) + k.wd * w;
  const float m_ = (float)((double)mi / k.bc1);
  const float v_ = (float)((double)vi / k.bc2);
  return m_ / (sqrtf(v_) + k.eps) + k.wd * w;
}

// One pack of VEC elements starting at element e0.
// Everything pass 1 reads for one pack of VEC elements.
// G = float, or uint16_t for fp16 gradients (the modified NCCL's mixed-precision LAMB, CCN_LAMB_NCCL_GLOBAL only).
template <int P, int VEC, class G = float>
struct LambIn {
  Pack<G, VEC> g[P > 0 ? P : CCN_MAX_RANKS];
  Pack<float, VEC> w, m, v;
};

// Issues the pack's loads, all of them before anything waits (P = 0: the first nP of CCN_MAX_RANKS, wave-uniform).
template <int P, int VEC, class G = float>
__device__ __forceinline__ void lamb_pass1_load(LambIn<P, VEC, G>& in, const SrcTable<G, (P ? P : CCN_MAX_RANKS)>& g, int nP,
                                                const float* w, const float* m, const float* v, size_t e0) {
  constexpr int PX = P > 0 ? P : CCN_MAX_RANKS;
#pragma unroll
  for (int p = 0; p < PX; p++) {
    if (P > 0 || p < nP) in.g[p] = load_stream<G, VEC>(g.p[p] + e0);
  }
  in.w = load_stream<float, VEC>(w + e0);   // w is read again by pass 2, 12 GB later
  in.m = load_stream<float, VEC>(m + e0);
  in.v = load_stream<float, VEC>(v + e0);
}

template <int P, int VEC, class G = float>
__device__ __forceinline__ void lamb_pass1_math(const LambIn<P, VEC, G>& in, int nP, float* m, float* v, size_t e0, float nf,
                                                const LambPrm& k, double& accW, double& accR, Pack<float, VEC>& r_out,
                                                Pack<float, VEC>& w_out) {
  constexpr int PX = P > 0 ? P : CCN_MAX_RANKS;
  Pack<float, VEC> mv, vv;
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    float ge, gsq;   // the gradient sum and its square
    if constexpr (std::is_same<G, uint16_t>::value) {
      // nccl/src/collectives/device/common_kernel.h:2460-2472 and reduce_kernel.h:391-399: the sum is carried in fp16
      // and the square is taken in fp16
      uint16_t S0 = in.g[0].d[e];
#pragma unroll
      for (int p = 1; p < PX; p++) {
        if (P > 0 || p < nP) S0 = f32_to_f16_bits(f16_bits_to_f32(S0) + f16_bits_to_f32(in.g[p].d[e]));
      }
      ge = f16_bits_to_f32(S0);
      gsq = f16_bits_to_f32(f32_to_f16_bits(ge * ge));
    } else {
      ge = in.g[0].d[e];
#pragma unroll
      for (int p = 1; p < PX; p++) {
        if (P > 0 || p < nP) ge = ge + in.g[p].d[e];
      }
      gsq = ge * ge;
    }
    const float we = in.w.d[e];
    float mi, vi;
    if (std::is_same<G, uint16_t>::value || k.mode == CCN_LAMB_NCCL_GLOBAL) {
      vi = ((in.v.d[e] * k.b2) + (gsq * k.omb2));
      mi = ((in.m.d[e] * k.b1) + (ge * k.omb1));
    } else {
      mi = k.b1 * in.m.d[e] + k.omb1 * ge;
      vi = k.b2 * in.v.d[e] + k.omb2 * ge * ge;
    }
    const float r = lamb_r(mi, vi, we, k);
    accR += k.mode == CCN_LAMB_NCCL_GLOBAL ? (double)(r * r) : (double)((r * r) / nf);
    accW += (double)(we * we);
    mv.d[e] = mi;
    vv.d[e] = vi;
    r_out.d[e] = r;
    w_out.d[e] = we;
  }
  store_stream<float, VEC>(m + e0, mv);
  store_stream<float, VEC>(v + e0, vv);
}

// One pack of VEC elements starting at element e0.
template <int P, int VEC, class G = float>
__device__ __forceinline__ void lamb_pass1_pack(const SrcTable<G, (P ? P : CCN_MAX_RANKS)>& g, int nP, const float* w,
                                                float* m, float* v, size_t e0, float nf, const LambPrm& k, double& accW,
                                                double& accR, Pack<float, VEC>& r_out, Pack<float, VEC>& w_out) {
  LambIn<P, VEC, G> in;
  lamb_pass1_load<P, VEC, G>(in, g, nP, w, m, v, e0);
  lamb_pass1_math<P, VEC, G>(in, nP, m, v, e0, nf, k, accW, accR, r_out, w_out);
}

template <int P, bool SCAT>
__global__ __launch_bounds__(kBlock) void lamb_pass1_kernel(const SrcTable<float, (P ? P : CCN_MAX_RANKS)> g, const int nP,
                                                            const float* w, float* m, float* v, const LambLayout lay,
                                                            double* __restrict__ partials, const int vec_ok,
                                                            const LambPrm k) {
  __shared__ double lds[2 * kBlock / kWave];
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  SrcTable<float, (P ? P : CCN_MAX_RANKS)> gt;
  float* wt;
  lamb_buffers_of<P, SCAT>(lay, g, const_cast<float*>(w), nP, t.buf, gt, wt);
  double accW = 0.0, accR = 0.0;
  const uint32_t j0 = threadIdx.x * 4;          // this thread's elements of the tile: [j0, j0+4) clipped to count
  if (j0 < t.count) {
    if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
      Pack<float, 4> r4, w4;
      lamb_pass1_pack<P, 4>(gt, nP, wt, m, v, t.start + j0, t.nf, k, accW, accR, r4, w4);
    } else {
      const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
      Pack<float, 1> r1, w1;
      for (uint32_t j = j0; j < j1; j++) lamb_pass1_pack<P, 1>(gt, nP, wt, m, v, t.start + j, t.nf, k, accW, accR, r1, w1);
    }
  }
  const double sW = block_sum(accW, lds);
  const double sR = block_sum(accR, lds + kBlock / kWave);
  if (threadIdx.x == 0) {
    partials[2 * (size_t)blockIdx.x] = sW;
    partials[2 * (size_t)blockIdx.x + 1] = sR;
  }
}

// Pass 1 for fp16 gradients in flat arrays (the two-pass path only).
template <int P>
__global__ __launch_bounds__(kBlock) void lamb_pass1_f16g_kernel(const SrcTable<uint16_t, (P ? P : CCN_MAX_RANKS)> g, const int nP,
                                                                 const float* w, float* m, float* v, const LambLayout lay,
                                                                 double* __restrict__ partials, const int vec_ok,
                                                                 const LambPrm k) {
  __shared__ double lds[2 * kBlock / kWave];
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  double accW = 0.0, accR = 0.0;
  const uint32_t j0 = threadIdx.x * 4;
  if (j0 < t.count) {
    if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
      Pack<float, 4> r4, w4;
      lamb_pass1_pack<P, 4, uint16_t>(g, nP, w, m, v, t.start + j0, t.nf, k, accW, accR, r4, w4);
    } else {
      const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
      Pack<float, 1> r1, w1;
      for (uint32_t j = j0; j < j1; j++) lamb_pass1_pack<P, 1, uint16_t>(g, nP, w, m, v, t.start + j, t.nf, k, accW, accR, r1, w1);
    }
  }
  const double sW = block_sum(accW, lds);
  const double sR = block_sum(accR, lds + kBlock / kWave);
  if (threadIdx.x == 0) {
    partials[2 * (size_t)blockIdx.x] = sW;
    partials[2 * (size_t)blockIdx.x + 1] = sR;
  }
}

// ---- communication between workgroups of one launch ---------------------------------------------------------------------
// Device-scope release/acquire fences write back and invalidate the XCD's whole L2; with one per tile they serialise
// the kernel (measured: 7 to 40 ms for a 2.8 ms step).  The few words that workgroups exchange therefore go through
// relaxed device-scope atomics only.  On gfx942/gfx950 those carry the sc1 cache policy: stores are written through to
// where the XCDs are coherent, loads and read-modify-writes are performed there, none of them is served from an XCD's
// own L2, so a single word written this way is seen by every later device-scope atomic load of it, from any XCD, without
// cache maintenance.  What relaxed atomics do not give is order BETWEEN words, and the protocol is built not to need it:
//   tile sums      every slot is set to a sentinel by the kernel that precedes the launch; a tile replaces it with its
//                  sum (one 64-bit atomic store per sum); whoever adds a segment's sums up re-reads a slot that still
//                  holds the sentinel, a bounded number of times, and gives the segment up if it stays: a sum that is
//                  not there yet is waited for or left to the trailing kernel, never read as something else;
//   arrival counts only elect the workgroup that adds a segment up (a read-modify-write: exactly one sees the last count);
//   scale + ready  travel in ONE 64-bit word, zero until set;
//   everything else crosses a kernel boundary (the deferred list, the stored m and v, the norms for the host).
// The tile still waits for its stores' acknowledgement (vmcnt = 0) before it counts itself in, so that the elected
// workgroup normally finds every sum in place; that wait is a courtesy to the reader, not what correctness rests on.
constexpr unsigned long long kNoSumYet = ~0ull;   // a NaN pattern no arithmetic produces; real sums are canonicalised away from it
__device__ __forceinline__ unsigned long long sum_bits(double x) {
  const unsigned long long b = (unsigned long long)__double_as_longlong(x);
  return b == kNoSumYet ? 0x7ff8000000000000ull : b;
}
__device__ __forceinline__ unsigned long long peek_u64(const double* p) {
  return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// All vector-memory operations this wavefront has issued are acknowledged before anything after this is issued.
__device__ __forceinline__ void drain_vector_memory() {
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0); expcnt and lgkmcnt left at their maxima
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

// Sum of `x` over a BS-thread workgroup (BS = 64: one wavefront, no LDS); result valid in thread 0.
// lds must hold BS / kWave doubles.
template <int BS>
__device__ __forceinline__ double group_sum(double x, double* lds) {
  static_assert(BS % kWave == 0 && BS <= kBlock, "whole wavefronts, at most kBlock threads");
  x = wave_sum(x);
  if constexpr (BS == kWave) {
    return x;
  } else {
    const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
    if (lane == 0) lds[wv] = x;
    __syncthreads();
    double r = 0.0;
    if (threadIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < BS / kWave; i++) r += lds[i];
    }
    __syncthreads();
    return r;
  }
}

// Norms and scale of segment b from its tiles' partial sums [lo, hi).  Thread t adds tiles lo+t, lo+t+BS, ... in
// ascending order, then the fixed shuffle/LDS tree: the result does not depend on scheduling.
// SHARED: the partial sums are published by other workgroups of this launch: a slot that still holds the sentinel is
// read again up to `patience` times; if one stays empty, nothing is written and *complete is false (thread 0).
// Returns the scale (valid in thread 0).
template <int BS, bool SHARED>
__device__ __forceinline__ float lamb_finalize_segment(const double* partials, uint32_t lo, uint32_t hi, uint64_t seg_len,
                                                      int b, double* norms, float* scale, int mode, double* lds,
                                                      uint32_t patience = 0, bool* complete = nullptr) {
  double aW = 0.0, aR = 0.0;
  double missing = 0.0;   // counts slots that stayed empty (summed over the workgroup like the sums themselves)
  for (uint32_t t = lo + threadIdx.x; t < hi; t += BS) {
    if constexpr (SHARED) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        unsigned long long bits = peek_u64(partials + 2 * (size_t)t + h);
        for (uint32_t tries = 0; bits == kNoSumYet && tries < patience; tries++) {
          __builtin_amdgcn_s_sleep(8);
          bits = peek_u64(partials + 2 * (size_t)t + h);
        }
        if (bits == kNoSumYet) missing += 1.0;
        else if (h == 0) aW += __longlong_as_double((long long)bits);
        else aR += __longlong_as_double((long long)bits);
      }
    } else {
      aW += partials[2 * (size_t)t];
      aR += partials[2 * (size_t)t + 1];
    }
  }
  const double sW = group_sum<BS>(aW, lds);
  const double sR = group_sum<BS>(aR, lds + kBlock / kWave);
  bool ok = true;
  if constexpr (SHARED) {
    const double gaps = group_sum<BS>(missing, lds);
    ok = gaps == 0.0;
    if (complete && threadIdx.x == 0) *complete = ok;
  }
  float sc = 0.0f;
  if (threadIdx.x == 0 && ok && mode == CCN_LAMB_NCCL_GLOBAL) {
    const float wNorm = sqrtf((float)sW), rNorm = sqrtf((float)sR);
    norms[2 * b] = wNorm;
    norms[2 * b + 1] = rNorm;
    sc = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f) / rNorm;
    scale[b] = sc;
  } else if (threadIdx.x == 0 && ok) {
    const double rNorm = sqrt(sR);
    const double wNorm = sqrt(sW / (double)seg_len);
    const double ratio = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f);
    norms[2 * b] = wNorm;
    norms[2 * b + 1] = rNorm;
    sc = (float)(mode == CCN_LAMB_REFERENCE ? ratio / rNorm : ratio);
    scale[b] = sc;
  }
  return sc;
}

// One workgroup per segment that has tiles in this table.
__global__ __launch_bounds__(kBlock) void lamb_finalize_kernel(const double* __restrict__ partials,
                                                               const uint32_t* __restrict__ seg_tile_begin,
                                                               const uint64_t* __restrict__ seg_len,
                                                               double* __restrict__ norms, float* __restrict__ scale,
                                                               const int mode) {
  __shared__ double lds[2 * kBlock / kWave];
  const int b = blockIdx.x;
  const uint32_t lo = seg_tile_begin[b], hi = seg_tile_begin[b + 1];
  if (lo == hi) return;   // the segment is handled by the resident kernel
  lamb_finalize_segment<kBlock, false>(partials, lo, hi, seg_len[b], b, norms, scale, mode, lds);
}

// First level for long segments: workgroup q adds the tile pairs [group_begin[q], group_begin[q+1]), all of one
// segment, in the same fixed order as above, into pair q of `folded`; the finalize kernel then runs over those.
constexpr uint32_t kLambFold = 4096;   // tiles per group
__global__ __launch_bounds__(kBlock) void lamb_fold_kernel(const double* __restrict__ partials,
                                                           const uint32_t* __restrict__ group_begin,
                                                           double* __restrict__ folded) {
  __shared__ double lds[2 * kBlock / kWave];
  const uint32_t lo = group_begin[blockIdx.x], hi = group_begin[blockIdx.x + 1];
  double aW = 0.0, aR = 0.0;
  for (uint32_t t = lo + threadIdx.x; t < hi; t += kBlock) {
    aW += partials[2 * (size_t)t];
    aR += partials[2 * (size_t)t + 1];
  }
  const double sW = block_sum(aW, lds);
  const double sR = block_sum(aR, lds + kBlock / kWave);
  if (threadIdx.x == 0) {
    folded[2 * (size_t)blockIdx.x] = sW;
    folded[2 * (size_t)blockIdx.x + 1] = sR;
  }
}

// HALF: also writes the fp16 copy of the new weights (nccl/src/collectives/device/common_kernel.h:2695).
template <int VEC, bool HALF = false>
__device__ __forceinline__ void lamb_pass2_pack(float* w, const float* m, const float* v, size_t e0, float step_scale,
                                                const LambPrm& k, uint16_t* halfw = nullptr) {
  Pack<float, VEC> wv = load_stream<float, VEC>(w + e0);
  const Pack<float, VEC> mv = load_stream<float, VEC>(m + e0);
  const Pack<float, VEC> vv = load_stream<float, VEC>(v + e0);
  Pack<uint16_t, VEC> hv;
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    const float we = wv.d[e];
    const float r = lamb_r(mv.d[e], vv.d[e], we, k);
    const float x = step_scale * r;
    wv.d[e] = we - x;
    hv.d[e] = HALF ? f32_to_f16_bits(wv.d[e]) : (uint16_t)0;
  }
  store_stream<float, VEC>(w + e0, wv);
  if constexpr (HALF) store_stream<uint16_t, VEC>(halfw + e0, hv);
}

template <bool SCAT>
__global__ __launch_bounds__(kBlock) void lamb_pass2_kernel(float* w, const float* m, const float* v, const LambLayout lay,
                                                            const float* __restrict__ scale, const int vec_ok,
                                                            const LambPrm k) {
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  float* const wt = lamb_weights_of<SCAT>(lay, w, t.buf);
  const float step_scale = k.lr * scale[t.seg];   // stepsize * scale, then times r
  const uint32_t j0 = threadIdx.x * 4;
  if (j0 >= t.count) return;
  if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
    lamb_pass2_pack<4>(wt, m, v, t.start + j0, step_scale, k);
  } else {
    const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
    for (uint32_t j = j0; j < j1; j++) lamb_pass2_pack<1>(wt, m, v, t.start + j, step_scale, k);
  }
}

__global__ __launch_bounds__(kBlock) void lamb_pass2_f16w_kernel(float* w, uint16_t* halfw, const float* m, const float* v,
                                                                 const LambLayout lay, const float* __restrict__ scale,
                                                                 const int vec_ok, const LambPrm k) {
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  const float step_scale = k.lr * scale[t.seg];
  const uint32_t j0 = threadIdx.x * 4;
  if (j0 >= t.count) return;
  if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
    lamb_pass2_pack<4, true>(w, m, v, t.start + j0, step_scale, k, halfw);
  } else {
    const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
    for (uint32_t j = j0; j < j1; j++) lamb_pass2_pack<1, true>(w, m, v, t.start + j, step_scale, k, halfw);
  }
}

// ---- segments that stay on chip: shared state of the one-tile kernel ------------------------------------------------------
constexpr int kOneshotSub = 8;       // packs per thread per tile
constexpr int kOneshotBlock = 256;   // threads per workgroup: a tile is 256 * 4 * 8 = 8192 elements
// Arrival counters.  Device-scope atomics on one address are served one after the other (some 15 ns each, measured),
// so a segment's tiles count into kResFan counters, each on a cache line of its own, and the tile that completes one
// of them counts into the segment's top counter.
constexpr int kResFan = 8;
constexpr int kResCntLine = 16;                              // uint32 per 64-byte line
constexpr int kResCntStride = (kResFan + 1) * kResCntLine;   // uint32 per segment: top counter, then the fan

struct LambResident {
  uint32_t* cnt;                    // [nseg * kResCntStride] arrival counters (zero at kernel start)
  unsigned long long* ready;        // [nseg] (1 << 32 | scale bits) once the segment's scale is known (zero at kernel start)
  const uint32_t* seg_tile_begin;   // [nseg+1] resident-tile numbering
  uint32_t* deferred;               // [ntiles]
  uint32_t* ndeferred;              // zero at kernel start
  uint32_t ntiles;
  uint32_t spin_limit;
  uint32_t withhold;                // diagnostic: scales are computed but never announced, as if their sums had not arrived
};

// Runs before every launch of the one-tile kernel: counters and ready words to zero, every tile-sum slot to "no sum yet".
__global__ void lamb_reset_kernel(uint32_t* cnt, unsigned long long* ready, int nseg, uint32_t* ndeferred, double* partials,
                                  uint32_t ntiles) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if ((uint32_t)i < 2 * ntiles) reinterpret_cast<unsigned long long*>(partials)[i] = kNoSumYet;
  if (i < nseg) {
    ready[i] = 0;
#pragma unroll
    for (int f = 0; f <= kResFan; f++) cnt[(size_t)i * kResCntStride + f * kResCntLine] = 0;
  }
  if (i == 0) *ndeferred = 0;
}

// ---- one tile per workgroup ----------------------------------------------------------------------------------------------
// Workgroup b runs pass 1 on tile b (SUB packs per thread), keeps the tile's r in registers and its old w in LDS, counts
// itself in, waits (within the spin limit) for the segment's scale and writes w.  The workgroup that finishes a segment's
// last tile adds the segment's tile sums up and publishes the scale.  Workgroups are dispatched in tile order, so the
// tiles a waiting workgroup depends on are already running.  Every wait is bounded: a tile whose segment is not ready
// within the spin limit goes onto a deferred list, and a trailing kernel finishes it from the stored m and v (w is still
// the old one), so the result is the same whatever the scheduling and every workgroup exits.
// G = uint16_t: fp16 gradients and an fp16 copy of the new weights in halfw (flat arrays only).
template <int P, int BS, int SUB, bool SCAT, class G = float>
__global__ __launch_bounds__(BS) __attribute__((amdgpu_waves_per_eu(3, 3))) void lamb_oneshot_kernel(const SrcTable<G, (P ? P : CCN_MAX_RANKS)> g, const int nP,
                                                          float* w, uint16_t* halfw, float* m, float* v, const LambLayout lay,
                                                          double* partials, const uint64_t* __restrict__ seg_len,
                                                          double* norms, float* scale, const LambResident rs,
                                                          const int vec_ok, const LambPrm k) {
  extern __shared__ __align__(16) unsigned char smem[];
  Pack<float, 4>* wpark = reinterpret_cast<Pack<float, 4>*>(smem);
  double* red = reinterpret_cast<double*>(smem + (size_t)SUB * BS * sizeof(Pack<float, 4>));
  uint32_t* bc = reinterpret_cast<uint32_t*>(red + 2 * kBlock / kWave);   // [0] last tile of its segment, [1] ready, [2] scale
  const unsigned tile = blockIdx.x;
  const LambTile t = lamb_tile_of(lay, tile);
  constexpr bool kHalf = std::is_same<G, uint16_t>::value;
  static_assert(!(kHalf && SCAT), "fp16 gradients come in flat arrays");
  SrcTable<G, (P ? P : CCN_MAX_RANKS)> gt;
  float* wt;
  if constexpr (SCAT) {
    lamb_buffers_of<P, SCAT>(lay, g, w, nP, t.buf, gt, wt);
  } else {
    gt = g;
    wt = w;
  }
  Pack<float, 4> rpark[SUB];
  double accW = 0.0, accR = 0.0;
  const bool fast = P > 0 && vec_ok && (t.start & 3u) == 0 && t.count == (uint32_t)(BS * 4 * SUB);
  if (fast) {
    LambIn<P, 4, G> cur;
    lamb_pass1_load<P, 4, G>(cur, gt, nP, wt, m, v, t.start + threadIdx.x * 4);
#pragma unroll
    for (int u = 0; u < SUB; u++) {
      const size_t e0 = t.start + (size_t)(u * BS + threadIdx.x) * 4;
      LambIn<P, 4, G> nxt;
      if (u + 1 < SUB) lamb_pass1_load<P, 4, G>(nxt, gt, nP, wt, m, v, e0 + BS * 4);
      Pack<float, 4> w4;
      lamb_pass1_math<P, 4, G>(cur, nP, m, v, e0, t.nf, k, accW, accR, rpark[u], w4);
      wpark[u * BS + threadIdx.x] = w4;
      if (u + 1 < SUB) cur = nxt;
    }
  } else {
#pragma unroll
    for (int u = 0; u < SUB; u++) {
      const uint32_t j0 = (u * BS + threadIdx.x) * 4;
      Pack<float, 4> r4 = {}, w4 = {};
      if (j0 < t.count) {
        if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
          lamb_pass1_pack<P, 4, G>(gt, nP, wt, m, v, t.start + j0, t.nf, k, accW, accR, r4, w4);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (j0 + e < t.count) {
              Pack<float, 1> r1, w1;
              lamb_pass1_pack<P, 1, G>(gt, nP, wt, m, v, t.start + j0 + e, t.nf, k, accW, accR, r1, w1);
              r4.d[e] = r1.d[0];
              w4.d[e] = w1.d[0];
            }
          }
        }
      }
      rpark[u] = r4;
      wpark[u * BS + threadIdx.x] = w4;
    }
  }
  const double sW = group_sum<BS>(accW, red);
  const double sR = group_sum<BS>(accR, red + kBlock / kWave);
  if (threadIdx.x == 0) {
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(partials) + 2 * (size_t)tile, sum_bits(sW), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(partials) + 2 * (size_t)tile + 1, sum_bits(sR), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    drain_vector_memory();   // the sums are in place before the count says so
    const uint32_t seg_lo = rs.seg_tile_begin[t.seg];
    const uint32_t seg_tiles = rs.seg_tile_begin[t.seg + 1] - seg_lo;
    const uint32_t f = (tile - seg_lo) % kResFan;
    const uint32_t fan_target = (seg_tiles - f + kResFan - 1) / kResFan;
    const uint32_t arrived = __hip_atomic_fetch_add(&rs.cnt[(size_t)t.seg * kResCntStride + (1 + f) * kResCntLine], 1u,
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
    uint32_t last = 0;
    if (arrived == fan_target) {
      const uint32_t fans = seg_tiles < (uint32_t)kResFan ? seg_tiles : (uint32_t)kResFan;
      last = __hip_atomic_fetch_add(&rs.cnt[(size_t)t.seg * kResCntStride], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 ==
             fans;
    }
    bc[0] = last;
  }
  __syncthreads();
  if (bc[0]) {
    bool complete = false;
    const float sc = lamb_finalize_segment<BS, true>(partials, rs.seg_tile_begin[t.seg], rs.seg_tile_begin[t.seg + 1],
                                                     seg_len[t.seg], (int)t.seg, norms, scale, k.mode, red, rs.spin_limit, &complete);
    if (threadIdx.x == 0 && complete && !rs.withhold)   // otherwise the trailing kernel adds the segment up
      __hip_atomic_store(&rs.ready[t.seg], (1ull << 32) | __float_as_uint(sc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (threadIdx.x == 0) {
    uint32_t budget = rs.spin_limit / 4;
    unsigned long long word;
    while (((word = __hip_atomic_load(&rs.ready[t.seg], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) >> 32) == 0) {
      if (budget == 0) break;
      budget--;
      __builtin_amdgcn_s_sleep(32);
    }
    if ((word >> 32) == 0) {
      const uint32_t at = __hip_atomic_fetch_add(rs.ndeferred, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      rs.deferred[at] = tile;
    }
    bc[1] = (uint32_t)(word >> 32);
    bc[2] = (uint32_t)word;
  }
  __syncthreads();
  if (!bc[1]) return;
  const float step_scale = k.lr * __uint_as_float(bc[2]);
#pragma unroll
  for (int u = 0; u < SUB; u++) {
    const uint32_t j0 = (u * BS + threadIdx.x) * 4;
    if (j0 >= t.count) continue;
    Pack<float, 4> wv = wpark[u * BS + threadIdx.x];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float x = step_scale * rpark[u].d[e];
      wv.d[e] = wv.d[e] - x;
    }
    if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
      store_stream<float, 4>(wt + t.start + j0, wv);
      if constexpr (kHalf) {
        Pack<uint16_t, 4> hv;
#pragma unroll
        for (int e = 0; e < 4; e++) hv.d[e] = f32_to_f16_bits(wv.d[e]);
        store_stream<uint16_t, 4>(halfw + t.start + j0, hv);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if (j0 + e < t.count) {
          wt[t.start + j0 + e] = wv.d[e];
          if constexpr (kHalf) halfw[t.start + j0 + e] = f32_to_f16_bits(wv.d[e]);
        }
      }
    }
  }
}

// Finishes the deferred tiles: pass 2 from the stored m and v, as the two-pass path does.  A tile is deferred because its
// segment's scale had not been announced when its patience ran out; if it never was (the workgroup that added the segment
// up found a sum missing), the segment is added up here, where every sum of the previous kernel is in place: every
// workgroup that needs the scale computes the same value in the same fixed order and writes the same norms.
template <int BS, int SUB, bool SCAT, bool HALF = false>
__global__ __launch_bounds__(BS) void lamb_deferred_kernel(float* w, uint16_t* halfw, const float* m, const float* v, const LambLayout lay,
                                                           float* __restrict__ scale, const unsigned long long* __restrict__ ready,
                                                           const double* __restrict__ partials,
                                                           const uint32_t* __restrict__ seg_tile_begin,
                                                           const uint64_t* __restrict__ seg_len, double* norms,
                                                           const uint32_t* __restrict__ deferred,
                                                           const uint32_t* __restrict__ ndeferred, const int vec_ok,
                                                           const LambPrm k) {
  __shared__ double red[2 * kBlock / kWave];
  __shared__ float late_scale;
  const uint32_t n = *ndeferred;
  for (uint32_t i = blockIdx.x; i < n; i += gridDim.x) {
    const LambTile t = lamb_tile_of(lay, deferred[i]);
    float* const wt = lamb_weights_of<SCAT>(lay, w, t.buf);
    const unsigned long long word = ready[t.seg];
    float sc;
    if (word >> 32) {
      sc = __uint_as_float((uint32_t)word);
    } else {
      const float mine = lamb_finalize_segment<BS, false>(partials, seg_tile_begin[t.seg], seg_tile_begin[t.seg + 1], seg_len[t.seg],
                                                          (int)t.seg, norms, scale, k.mode, red);
      if (threadIdx.x == 0) late_scale = mine;
      __syncthreads();
      sc = late_scale;
      __syncthreads();
    }
    const float step_scale = k.lr * sc;
    for (int u = 0; u < SUB; u++) {
      const uint32_t j0 = (u * BS + threadIdx.x) * 4;
      if (j0 >= t.count) continue;
      if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
        lamb_pass2_pack<4, HALF>(wt, m, v, t.start + j0, step_scale, k, halfw);
      } else {
        const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
        for (uint32_t j = j0; j < j1; j++) lamb_pass2_pack<1, HALF>(wt, m, v, t.start + j, step_scale, k, halfw);
      }
    }
  }
}

// ---- the two-pass step without a plan, for callers that cannot allocate ------------------------------------------------
// Everything a plan would hold in allocated device memory (tile sums, group sums, norms, scales and the small index
// tables of the finalize kernels) lives in one file-scope device array instead.  Every GPU the library runs on holds its
// own copy of the array at its own address until the process ends; host code never uses the array's name as an address
// (on the host it is a stand-in, not device memory) but the pointer hipGetSymbolAddress returns for the current device.
constexpr size_t kStaticMaxTiles = (size_t)1 << 18;                       // N <= 2^28 elements in tiles of kLambTile
constexpr size_t kStaticMaxSegs = CCN_LAMB_STATIC_MAX_SEGS;
constexpr size_t kStaticMaxGroups = kStaticMaxTiles / kLambFold + 64;      // groups only exist when segments are long
static_assert(kStaticMaxTiles * kLambTile == CCN_LAMB_STATIC_MAX_N, "header and kernel limits agree");

struct LambStaticScratch {
  double partials[2 * kStaticMaxTiles];
  double folded[2 * kStaticMaxGroups];
  double norms[2 * kStaticMaxSegs];
  uint64_t seg_len[kStaticMaxSegs];
  float scale[kStaticMaxSegs];
  uint32_t seg_begin[kStaticMaxSegs + 1];      // first tile (or first group, when sums go through groups) of a segment
  uint32_t group_begin[kStaticMaxGroups + 1];  // first tile of a group
};
static __device__ __align__(256) unsigned char scratch[sizeof(LambStaticScratch)];

// Fills the index tables for nseg segments of tps tiles each.  gps = 0: the finalize kernel reads tile sums, seg_begin
// counts tiles.  gps > 0: segment sums go through gps groups of at most kLambFold tiles, seg_begin counts groups.
__global__ void lamb_static_tables_kernel(LambStaticScratch* sc, const uint32_t nseg, const uint32_t tps, const uint32_t gps,
                                          const uint64_t seg_len) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nseg) sc->seg_len[i] = seg_len;
  if (i <= nseg) sc->seg_begin[i] = gps ? i * gps : i * tps;
  if (gps && i <= nseg * gps) {
    const uint32_t b = i / gps, q = i % gps;
    sc->group_begin[i] = i == nseg * gps ? nseg * tps : b * tps + q * kLambFold;
  }
}

}  // namespace ccn

using namespace ccn;

struct ccn_lamb_plan {
  int device = -1;
  int nseg = 0;
  size_t N = 0;
  // common per-segment state
  uint64_t* seg_len = nullptr;
  double* norms = nullptr;
  float* scale = nullptr;
  // two-pass part: tiles of kLambTile elements of the segments too long to stay on chip
  size_t ntiles = 0;
  uint64_t uniform_seg_len = 0;   // non-zero: all segments have this length and it is a multiple of the tile
  LambTile* tiles = nullptr;
  uint32_t* seg_tile_begin = nullptr;
  double* partials = nullptr;
  uint32_t ngroups = 0;                 // non-zero: some segment has more than kLambFold tiles, sums go through groups
  uint32_t* group_begin = nullptr;      // [ngroups+1] tile index where each group starts
  uint32_t* seg_group_begin = nullptr;  // [nseg+1]
  double* folded = nullptr;             // [2*ngroups]
  // on-chip part: tiles of kOneshotBlock * 4 * kOneshotSub elements of the other segments
  unsigned res_lds = 0;
  uint32_t res_ntiles = 0;
  uint64_t res_uniform_seg_len = 0;
  uint32_t spin_limit = 0;        // bound of the one-tile kernel's waits (CCN_LAMB_KNOB_SPIN_LIMIT)
  uint32_t withhold = 0;          // CCN_LAMB_KNOB_WITHHOLD: diagnostic, see LambResident
  bool force_two_pass = false;    // CCN_LAMB_KNOB_TWO_PASS: every step runs on the two-pass twin
  LambTile* rtiles = nullptr;
  uint32_t* seg_rtile_begin = nullptr;
  double* rpartials = nullptr;
  uint32_t* sync = nullptr;       // cnt[nseg], ndeferred
  unsigned long long* ready = nullptr;
  uint32_t* deferred = nullptr;
  // scattered buffers: the segments' gradient and weight pointers, moved back by the segment's first element index
  std::vector<uint64_t> seg_start;
  int nbuf = 0;                         // buffers of the scattered layout (== nseg unless segments are made of several)
  std::vector<uint64_t> buf_start;
  const void** ptr_dev = nullptr;       // [CCN_MAX_RANKS * nbuf] gradients, rank-major, then [nbuf] weights; made on first use
  const void** ptr_pinned = nullptr;
  std::vector<const void*> ptr_shadow;  // what the device table holds
  int ptr_ranks = 0;
  // a plan over the same segments with every segment on the two-pass path (fp16 gradients with segments too long to
  // stay on chip; CCN_LAMB_KNOB_TWO_PASS); made on first use
  ccn_lamb_plan* two_pass_twin = nullptr;
};

namespace {

// Calls body(integral_constant<P>) with the rank count as a compile-time constant (0 = 9..CCN_MAX_RANKS, looped).
template <class Body>
void with_rank_count(int P, Body body) {
  switch (P) {
#define CCN_CASE(K) case K: body(std::integral_constant<int, K>{}); break;
    CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
    default: body(std::integral_constant<int, 0>{}); break;
  }
}

// Workgroups of the one-tile kernel for P ranks that one CU holds at once with `lds` bytes of LDS each (0 on error).
int oneshot_occupancy(int P, unsigned lds) {
  int occ = 0;
  with_rank_count(P, [&](auto ptag) {
    auto* fn = lamb_oneshot_kernel<decltype(ptag)::value, kOneshotBlock, kOneshotSub, false>;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, fn, kOneshotBlock, lds) != hipSuccess) {
      (void)hipGetLastError();
      occ = 0;
    }
  });
  return occ;
}

// Cuts segment b into tiles of `tile` elements appended to `out`.
// Tiles of the elements [begin, end) of buffer `buf`, which belongs to segment `seg` of seg_n elements.
void cut_buffer(std::vector<LambTile>& out, uint64_t begin, uint64_t end, uint64_t tile, uint32_t seg, uint64_t seg_n,
                uint32_t buf) {
  for (uint64_t at = begin; at < end; at += tile) {
    LambTile t{};
    t.start = at;
    t.count = (uint32_t)((end - at) < tile ? (end - at) : tile);
    t.seg = seg;
    t.nf = (float)seg_n;
    t.buf = buf;
    out.push_back(t);
  }
}

}  // namespace

extern "C" {

int ccn_lamb_plan_destroy(ccn_lamb_plan* plan) {
  if (!plan) return CCN_OK;
  int rc = CCN_OK;
  void* bufs[] = {plan->tiles,  plan->seg_tile_begin,  plan->seg_len,   plan->partials, plan->norms,   plan->scale,
                  plan->rtiles, plan->seg_rtile_begin, plan->rpartials, plan->sync,     plan->deferred, plan->ready,
                  plan->group_begin, plan->seg_group_begin, plan->folded, (void*)plan->ptr_dev};
  for (void* b : bufs) {
    if (b && hipFree(b) != hipSuccess) rc = CCN_EHIP;
  }
  if (plan->ptr_pinned && hipHostFree(plan->ptr_pinned) != hipSuccess) rc = CCN_EHIP;
  if (plan->two_pass_twin && ccn_lamb_plan_destroy(plan->two_pass_twin) != CCN_OK) rc = CCN_EHIP;
  delete plan;
  return rc;
}

// buf_offsets (nbuf + 1 entries) cuts [0, N) into the buffers of the scattered layout; every segment boundary is a buffer
// boundary.  Null: one buffer per segment.
static int lamb_plan_create(const size_t* seg_offsets, int nseg, bool two_pass_only, ccn_lamb_plan** out,
                            const size_t* buf_offsets = nullptr, int nbuf = 0) {
  for (int b = 0; b < nseg; b++) {
    if (seg_offsets[b + 1] <= seg_offsets[b]) return CCN_EINVAL;   // empty or descending segment
  }
  if (!buf_offsets) {
    buf_offsets = seg_offsets;
    nbuf = nseg;
  }
  const bool parented = nbuf != nseg;
  {
    if (nbuf < nseg || buf_offsets[0] != 0 || buf_offsets[nbuf] != seg_offsets[nseg]) return CCN_EINVAL;
    int b = 0;
    for (int q = 0; q < nbuf; q++) {
      if (buf_offsets[q + 1] <= buf_offsets[q]) return CCN_EINVAL;        // empty buffer
      if (buf_offsets[q] == seg_offsets[b + 1]) b++;                      // the next segment starts with this buffer
      if (buf_offsets[q + 1] > seg_offsets[b + 1]) return CCN_EINVAL;     // a buffer may not straddle two segments
    }
  }
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;

  // Shape of the one-tile kernel: registers, not LDS, decide how many of its workgroups share a CU.
  const bool resident_wanted = !two_pass_only;
  const uint64_t res_tile = (uint64_t)kOneshotBlock * 4 * kOneshotSub;
  // the parked w packs, the reduction scratch, three flags
  const size_t res_need = (size_t)kOneshotBlock * kOneshotSub * 16 + 2 * (kBlock / kWave) * sizeof(double) + 16;
  const unsigned res_lds = (unsigned)((res_need + 1023) & ~(size_t)1023);
  const int occ = resident_wanted ? oneshot_occupancy(8, res_lds) : 0;
  const bool resident_ok = occ > 0;
  // Tiles a segment may have to stay on chip: half of what the GPU runs at once of the one-tile workgroups (a segment's
  // waiting tiles must leave room for the ones that complete it).
  const uint64_t res_cap_tiles = (uint64_t)di->cu_count * (uint64_t)(occ > 0 ? occ : 0) / 2;

  std::vector<LambTile> tiles, rtiles;
  std::vector<uint32_t> begin((size_t)nseg + 1), rbegin((size_t)nseg + 1);
  std::vector<uint64_t> len((size_t)nseg);
  bool all_two_pass = true, all_resident = true;
  int q = 0;   // first buffer of segment b
  for (int b = 0; b < nseg; b++) {
    begin[b] = (uint32_t)tiles.size();
    rbegin[b] = (uint32_t)rtiles.size();
    const uint64_t n = seg_offsets[b + 1] - seg_offsets[b];
    len[b] = n;
    int q_end = q;
    uint64_t res_tiles = 0;   // tiles never cross a buffer boundary: every buffer rounds up on its own
    while (q_end < nbuf && buf_offsets[q_end] < seg_offsets[b + 1]) {
      res_tiles += (buf_offsets[q_end + 1] - buf_offsets[q_end] + res_tile - 1) / res_tile;
      q_end++;
    }
    const bool resident = resident_wanted && resident_ok && res_tiles <= res_cap_tiles;
    for (; q < q_end; q++)
      cut_buffer(resident ? rtiles : tiles, buf_offsets[q], buf_offsets[q + 1], resident ? res_tile : (uint64_t)kLambTile,
                 (uint32_t)b, n, (uint32_t)q);
    if (resident) all_two_pass = false;
    else all_resident = false;
    if (tiles.size() > 0x7fffffffu || rtiles.size() > 0x7fffffffu) return CCN_ERANGE;
  }
  begin[nseg] = (uint32_t)tiles.size();
  rbegin[nseg] = (uint32_t)rtiles.size();
  uint64_t uniform = parented ? 0 : len[0];   // tile -> segment by division only when a buffer is a segment
  for (int b = 1; b < nseg; b++) if (len[b] != uniform) uniform = 0;

  // groups of at most kLambFold tiles for the two-pass segments, if any of them is longer than that
  std::vector<uint32_t> group_begin, seg_group_begin;
  bool need_groups = false;
  for (int b = 0; b < nseg; b++) need_groups = need_groups || begin[b + 1] - begin[b] > kLambFold;
  if (need_groups) {
    for (int b = 0; b < nseg; b++) {
      seg_group_begin.push_back((uint32_t)group_begin.size());
      for (uint32_t t = begin[b]; t < begin[b + 1]; t += kLambFold) group_begin.push_back(t);
    }
    seg_group_begin.push_back((uint32_t)group_begin.size());
    group_begin.push_back(begin[nseg]);
  }

  ccn_lamb_plan* p = new (std::nothrow) ccn_lamb_plan();
  if (!p) return CCN_ENOMEM;
  struct Owner {   // frees the half-built plan on every early exit, a throwing std::vector included
    ccn_lamb_plan* p;
    ~Owner() { if (p) ccn_lamb_plan_destroy(p); }
  } owner{p};
  p->device = di->device;
  p->nseg = nseg;
  p->N = seg_offsets[nseg];
  p->seg_start.assign(seg_offsets, seg_offsets + nseg);
  p->nbuf = nbuf;
  p->buf_start.assign(buf_offsets, buf_offsets + nbuf);
  p->ntiles = tiles.size();
  p->uniform_seg_len = (all_two_pass && uniform % kLambTile == 0) ? uniform : 0;
  p->res_ntiles = (uint32_t)rtiles.size();
  p->res_uniform_seg_len = (all_resident && uniform % res_tile == 0) ? uniform : 0;
  p->res_lds = res_lds;
  p->spin_limit = 1u << 15;
  hipError_t e = hipSuccess;
  auto alloc = [&](void** ptr, size_t bytes) { if (e == hipSuccess) e = hipMalloc(ptr, bytes ? bytes : 16); };
  auto upload = [&](void* dst, const void* src, size_t bytes) {
    if (e == hipSuccess && bytes) e = hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice);
  };
  alloc((void**)&p->tiles, tiles.size() * sizeof(LambTile));
  alloc((void**)&p->seg_tile_begin, begin.size() * sizeof(uint32_t));
  alloc((void**)&p->seg_len, len.size() * sizeof(uint64_t));
  alloc((void**)&p->partials, 2 * tiles.size() * sizeof(double));
  alloc((void**)&p->norms, 2 * (size_t)nseg * sizeof(double));
  alloc((void**)&p->scale, (size_t)nseg * sizeof(float));
  alloc((void**)&p->rtiles, rtiles.size() * sizeof(LambTile));
  alloc((void**)&p->seg_rtile_begin, rbegin.size() * sizeof(uint32_t));
  alloc((void**)&p->rpartials, 2 * rtiles.size() * sizeof(double));
  alloc((void**)&p->sync, ((size_t)nseg * kResCntStride + 1) * sizeof(uint32_t));
  alloc((void**)&p->ready, (size_t)nseg * sizeof(unsigned long long));
  alloc((void**)&p->deferred, rtiles.size() * sizeof(uint32_t));
  upload(p->tiles, tiles.data(), tiles.size() * sizeof(LambTile));
  upload(p->seg_tile_begin, begin.data(), begin.size() * sizeof(uint32_t));
  upload(p->seg_len, len.data(), len.size() * sizeof(uint64_t));
  if (need_groups) {
    p->ngroups = (uint32_t)group_begin.size() - 1;
    alloc((void**)&p->group_begin, group_begin.size() * sizeof(uint32_t));
    alloc((void**)&p->seg_group_begin, seg_group_begin.size() * sizeof(uint32_t));
    alloc((void**)&p->folded, 2 * (size_t)p->ngroups * sizeof(double));
    upload(p->group_begin, group_begin.data(), group_begin.size() * sizeof(uint32_t));
    upload(p->seg_group_begin, seg_group_begin.data(), seg_group_begin.size() * sizeof(uint32_t));
  }
  upload(p->rtiles, rtiles.data(), rtiles.size() * sizeof(LambTile));
  upload(p->seg_rtile_begin, rbegin.data(), rbegin.size() * sizeof(uint32_t));
  if (e != hipSuccess) return hip_fail(e);
  owner.p = nullptr;
  *out = p;
  return CCN_OK;
}

int ccn_lamb_plan_create(const size_t* seg_offsets, int nseg, ccn_lamb_plan** out) {
  if (!out) return CCN_EINVAL;
  *out = nullptr;
  if (!seg_offsets || nseg < 1 || seg_offsets[0] != 0) return CCN_EINVAL;
  return guarded([&] { return lamb_plan_create(seg_offsets, nseg, false, out); });
}

int ccn_lamb_plan_create_parented(const size_t* buf_sizes, const size_t* buf_parent, int nbuf, ccn_lamb_plan** out) {
  if (!out) return CCN_EINVAL;
  *out = nullptr;
  if (!buf_sizes || !buf_parent || nbuf < 1 || buf_parent[0] != 0) return CCN_EINVAL;
  return guarded([&] {
    std::vector<size_t> boffs((size_t)nbuf + 1, 0), soffs(1, 0);
    for (int q = 0; q < nbuf; q++) {
      if (buf_sizes[q] == 0) return (int)CCN_EINVAL;
      if (q > 0 && buf_parent[q] != buf_parent[q - 1]) {
        if (buf_parent[q] != buf_parent[q - 1] + 1) return (int)CCN_EINVAL;   // parents in order, none skipped
        soffs.push_back(boffs[q]);
      }
      boffs[q + 1] = boffs[q] + buf_sizes[q];
    }
    soffs.push_back(boffs[nbuf]);
    if (soffs.size() - 1 > 0x7fffffffu) return (int)CCN_ERANGE;
    return lamb_plan_create(soffs.data(), (int)(soffs.size() - 1), false, out, boffs.data(), nbuf);
  });
}

}  // extern "C"

namespace {

// A plan over the same segments and buffers with every segment on the two-pass path, made on first use.
int make_two_pass_twin(ccn_lamb_plan* plan) {
  if (plan->two_pass_twin) return CCN_OK;
  std::vector<size_t> offs(plan->seg_start.begin(), plan->seg_start.end()), boffs(plan->buf_start.begin(), plan->buf_start.end());
  offs.push_back(plan->N);
  boffs.push_back(plan->N);
  return lamb_plan_create(offs.data(), plan->nseg, true, &plan->two_pass_twin, boffs.data(), plan->nbuf);
}

int lamb_step(ccn_lamb_plan* plan, const float* const* g, int P, float* w_flat, float* const* w_seg, float* m, float* v, float lr,
              float beta1, float beta2, float eps, float wd, int step, int mode, void* stream);

// Brings the plan's device table of per-buffer pointers in line with the caller's; copies (and waits for the copy, so
// that the staging buffer can be reused) only when they have changed since the last call.  Returns whether every
// pointer, moved back by its buffer's first element index, is 16-byte aligned.
int sync_segment_pointers(ccn_lamb_plan* plan, const float* const* g, int P, float* const* w, hipStream_t s, bool* aligned) {
  const size_t ns = (size_t)plan->nbuf, words = (size_t)(CCN_MAX_RANKS + 1) * ns;
  if (!plan->ptr_dev) {
    CCN_HIP(hipMalloc((void**)&plan->ptr_dev, words * sizeof(void*)));
    CCN_HIP(hipHostMalloc((void**)&plan->ptr_pinned, words * sizeof(void*), hipHostMallocDefault));
  }
  std::vector<const void*> want(words, nullptr);
  bool al = true;
  auto moved = [&](const float* base, size_t buf) {
    const float* q = base - plan->buf_start[buf];
    al = al && aligned16(q);
    return (const void*)q;
  };
  for (int p = 0; p < P; p++)
    for (size_t b = 0; b < ns; b++) want[(size_t)p * ns + b] = moved(g[(size_t)p * ns + b], b);
  for (size_t b = 0; b < ns; b++) want[(size_t)CCN_MAX_RANKS * ns + b] = moved(w[b], b);
  *aligned = al;
  if (plan->ptr_ranks == P && plan->ptr_shadow == want) return CCN_OK;
  plan->ptr_shadow.swap(want);
  plan->ptr_ranks = P;
  std::memcpy(plan->ptr_pinned, plan->ptr_shadow.data(), words * sizeof(void*));
  CCN_HIP(hipMemcpyAsync(plan->ptr_dev, plan->ptr_pinned, words * sizeof(void*), hipMemcpyHostToDevice, s));
  CCN_HIP(hipStreamSynchronize(s));
  return CCN_OK;
}

// One step.  Flat arrays: g holds P pointers, w_flat the weights, w_seg is null.  Scattered buffers: g holds P * nbuf
// pointers (rank-major), w_seg nbuf pointers, w_flat is null.
int lamb_step(ccn_lamb_plan* plan, const float* const* g, int P, float* w_flat, float* const* w_seg, float* m, float* v, float lr,
              float beta1, float beta2, float eps, float wd, int step, int mode, void* stream) {
  const bool scattered = w_seg != nullptr;
  if (!plan || !g || (!w_flat && !w_seg) || !m || !v || P < 1 || P > CCN_MAX_RANKS || step < 1) return CCN_EINVAL;
  if (mode != CCN_LAMB_TRUST_RATIO && mode != CCN_LAMB_REFERENCE && mode != CCN_LAMB_NCCL_GLOBAL) return CCN_EINVAL;
  const size_t ng = scattered ? (size_t)P * (size_t)plan->nbuf : (size_t)P;
  for (size_t i = 0; i < ng; i++) if (!g[i]) return CCN_EINVAL;
  if (scattered)
    for (int b = 0; b < plan->nbuf; b++) if (!w_seg[b]) return CCN_EINVAL;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  if (di->device != plan->device) return CCN_EINVAL;
  if (plan->force_two_pass && (plan->res_ntiles || plan->two_pass_twin)) {
    rc = make_two_pass_twin(plan);
    if (rc != CCN_OK) return rc;
    rc = lamb_step(plan->two_pass_twin, g, P, w_flat, w_seg, m, v, lr, beta1, beta2, eps, wd, step, mode, stream);
    if (rc != CCN_OK) return rc;
    // the norms land in the caller's plan, where ccn_lamb_plan_norms reads them
    CCN_HIP(hipMemcpyAsync(plan->norms, plan->two_pass_twin->norms, 2 * (size_t)plan->nseg * sizeof(double),
                           hipMemcpyDeviceToDevice, as_stream(stream)));
    return CCN_OK;
  }
  float* const w = w_flat;   // null for scattered buffers: the kernels then take every weight pointer from the table

  LambPrm k;
  k.b1 = beta1;
  k.omb1 = 1 - beta1;
  k.b2 = beta2;
  k.omb2 = 1 - beta2;
  k.eps = eps;
  k.wd = wd;
  k.lr = lr;
  k.mode = mode;
  k.bc1 = 1 - std::pow((double)beta1, (double)step);
  k.bc2 = 1 - std::pow((double)beta2, (double)step);

  hipStream_t s = as_stream(stream);
  bool al = aligned16(m) && aligned16(v);
  if (scattered) {
    bool tal = true;
    rc = sync_segment_pointers(plan, g, P, w_seg, s, &tal);
    if (rc != CCN_OK) return rc;
    al = al && tal;
  } else {
    al = al && aligned16(w);
    for (int p = 0; p < P; p++) al = al && aligned16(g[p]);
  }
  const int vec_ok = al ? 1 : 0;
  const dim3 block(kBlock);
  const float* const* gtab = scattered ? reinterpret_cast<const float* const*>(plan->ptr_dev) : nullptr;
  float* const* wtab =
      scattered ? reinterpret_cast<float* const*>(const_cast<void**>(plan->ptr_dev) + (size_t)CCN_MAX_RANKS * plan->nbuf) : nullptr;

  auto with_ranks = [&](auto body) { with_rank_count(P, body); };
  auto table = [&](auto ptag) {   // the flat arrays' gradient pointers; unused (null) for scattered buffers
    constexpr int PP = decltype(ptag)::value;
    SrcTable<float, (PP ? PP : CCN_MAX_RANKS)> tbl;
    for (int p = 0; p < (PP ? PP : CCN_MAX_RANKS); p++) tbl.p[p] = scattered ? nullptr : g[p < P ? p : 0];
    return tbl;
  };

  if (plan->res_ntiles) {
    LambLayout lay;
    lay.tiles = plan->rtiles;
    lay.seg_len = plan->res_uniform_seg_len;
    lay.seg_len_f = (float)plan->res_uniform_seg_len;
    lay.tile = (uint32_t)(kOneshotBlock * 4 * kOneshotSub);
    lay.gtab = gtab;
    lay.wtab = wtab;
    lay.nbuf = (uint32_t)plan->nbuf;
    LambResident rs;
    rs.cnt = plan->sync;
    rs.ndeferred = plan->sync + (size_t)plan->nseg * kResCntStride;
    rs.ready = plan->ready;
    rs.seg_tile_begin = plan->seg_rtile_begin;
    rs.deferred = plan->deferred;
    rs.ntiles = plan->res_ntiles;
    rs.spin_limit = plan->spin_limit;
    rs.withhold = plan->withhold;
    {
      const size_t items = 2 * (size_t)plan->res_ntiles > (size_t)plan->nseg ? 2 * (size_t)plan->res_ntiles : (size_t)plan->nseg;
      hipLaunchKernelGGL(lamb_reset_kernel, dim3((unsigned)((items + kBlock - 1) / kBlock)), block, 0, s, rs.cnt, rs.ready, plan->nseg,
                         rs.ndeferred, plan->rpartials, plan->res_ntiles);
    }
    CCN_HIP(hipGetLastError());
    with_ranks([&](auto ptag) {
      constexpr int PP = decltype(ptag)::value;
      const auto tbl = table(ptag);
      hipLaunchKernelGGL((scattered ? lamb_oneshot_kernel<PP, kOneshotBlock, kOneshotSub, true> : lamb_oneshot_kernel<PP, kOneshotBlock, kOneshotSub, false>),
                         dim3(plan->res_ntiles), dim3(kOneshotBlock), plan->res_lds, s, tbl, P, w, (uint16_t*)nullptr, m, v, lay, plan->rpartials,
                         (const uint64_t*)plan->seg_len, plan->norms, plan->scale, rs, vec_ok, k);
    });
    CCN_HIP(hipGetLastError());
    const unsigned dg = plan->res_ntiles < 1024u ? plan->res_ntiles : 1024u;
    hipLaunchKernelGGL((scattered ? lamb_deferred_kernel<kOneshotBlock, kOneshotSub, true> : lamb_deferred_kernel<kOneshotBlock, kOneshotSub, false>),
                       dim3(dg), dim3(kOneshotBlock), 0, s, w, (uint16_t*)nullptr, (const float*)m, (const float*)v, lay, plan->scale,
                       (const unsigned long long*)plan->ready, (const double*)plan->rpartials, (const uint32_t*)plan->seg_rtile_begin,
                       (const uint64_t*)plan->seg_len, plan->norms, (const uint32_t*)plan->deferred, (const uint32_t*)rs.ndeferred,
                       vec_ok, k);
    CCN_HIP(hipGetLastError());
  }

  if (plan->ntiles) {
    const dim3 grid((unsigned)plan->ntiles);
    LambLayout lay;
    lay.tiles = plan->tiles;
    lay.seg_len = vec_ok ? plan->uniform_seg_len : 0;
    lay.seg_len_f = (float)plan->uniform_seg_len;
    lay.tile = kLambTile;
    lay.gtab = gtab;
    lay.wtab = wtab;
    lay.nbuf = (uint32_t)plan->nbuf;
    // Residency caps measured for N = 2^28, P = 8: pass 1 is fastest at 4 workgroups per CU (its float64 sums and the
    // workgroup reduction need more wavefronts to hide than the plain Adam kernel), pass 2 uncapped.
    const unsigned lds1 = lds_for_residency(P >= 2 ? 4 : 0);
    const unsigned lds2 = 0;
    with_ranks([&](auto ptag) {
      constexpr int PP = decltype(ptag)::value;
      hipLaunchKernelGGL((scattered ? lamb_pass1_kernel<PP, true> : lamb_pass1_kernel<PP, false>), grid, block, lds1, s,
                         table(ptag), P, (const float*)w, m, v, lay,
                         plan->partials, vec_ok, k);
    });
    CCN_HIP(hipGetLastError());
    const double* sums = plan->partials;
    const uint32_t* seg_begin = plan->seg_tile_begin;
    if (plan->ngroups) {
      hipLaunchKernelGGL(lamb_fold_kernel, dim3(plan->ngroups), block, 0, s, (const double*)plan->partials,
                         (const uint32_t*)plan->group_begin, plan->folded);
      CCN_HIP(hipGetLastError());
      sums = plan->folded;
      seg_begin = plan->seg_group_begin;
    }
    hipLaunchKernelGGL(lamb_finalize_kernel, dim3((unsigned)plan->nseg), block, 0, s, sums, seg_begin,
                       (const uint64_t*)plan->seg_len, plan->norms, plan->scale, mode);
    CCN_HIP(hipGetLastError());
    hipLaunchKernelGGL((scattered ? lamb_pass2_kernel<true> : lamb_pass2_kernel<false>), grid, block, lds2, s, w,
                       (const float*)m, (const float*)v, lay,
                       (const float*)plan->scale, vec_ok, k);
    CCN_HIP(hipGetLastError());
  }
  return CCN_OK;
}

// One step of the modified NCCL's mixed-precision LAMB: fp16 gradients in flat arrays, fp32 w, m, v, fp16 copy of w.
int lamb_step_f16g(ccn_lamb_plan* plan, const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v, float lr,
                   float beta1, float beta2, float wd, void* stream) {
  if (!plan || !g || !w || !halfw || !m || !v || P < 1 || P > CCN_MAX_RANKS) return CCN_EINVAL;
  for (int p = 0; p < P; p++) if (!g[p]) return CCN_EINVAL;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  if (di->device != plan->device) return CCN_EINVAL;
  LambPrm k;
  k.b1 = beta1;
  k.omb1 = 1 - beta1;
  k.b2 = beta2;
  k.omb2 = 1 - beta2;
  k.eps = 0.0f;
  k.wd = wd;
  k.lr = lr;
  k.mode = CCN_LAMB_NCCL_GLOBAL;
  k.bc1 = k.bc2 = 1.0;
  bool al = aligned16(w) && aligned16(m) && aligned16(v) && (reinterpret_cast<uintptr_t>(halfw) & 7u) == 0;
  for (int p = 0; p < P; p++) al = al && (reinterpret_cast<uintptr_t>(g[p]) & 7u) == 0;
  const int vec_ok = al ? 1 : 0;
  hipStream_t s = as_stream(stream);
  const dim3 block(kBlock);

  // Every segment short enough to stay on chip: the one-tile kernel, as for fp32 gradients.
  if (!plan->force_two_pass && plan->ntiles == 0 && plan->res_ntiles) {
    LambLayout lay;
    lay.tiles = plan->rtiles;
    lay.seg_len = plan->res_uniform_seg_len;
    lay.seg_len_f = (float)plan->res_uniform_seg_len;
    lay.tile = (uint32_t)(kOneshotBlock * 4 * kOneshotSub);
    lay.gtab = nullptr;
    lay.wtab = nullptr;
    lay.nbuf = (uint32_t)plan->nbuf;
    LambResident rs;
    rs.cnt = plan->sync;
    rs.ndeferred = plan->sync + (size_t)plan->nseg * kResCntStride;
    rs.ready = plan->ready;
    rs.seg_tile_begin = plan->seg_rtile_begin;
    rs.deferred = plan->deferred;
    rs.ntiles = plan->res_ntiles;
    rs.spin_limit = plan->spin_limit;
    rs.withhold = plan->withhold;
    {
      const size_t items = 2 * (size_t)plan->res_ntiles > (size_t)plan->nseg ? 2 * (size_t)plan->res_ntiles : (size_t)plan->nseg;
      hipLaunchKernelGGL(lamb_reset_kernel, dim3((unsigned)((items + kBlock - 1) / kBlock)), block, 0, s, rs.cnt, rs.ready, plan->nseg,
                         rs.ndeferred, plan->rpartials, plan->res_ntiles);
    }
    CCN_HIP(hipGetLastError());
    with_rank_count(P, [&](auto ptag) {
      constexpr int PP = decltype(ptag)::value;
      SrcTable<uint16_t, (PP ? PP : CCN_MAX_RANKS)> tbl;
      for (int p = 0; p < (PP ? PP : CCN_MAX_RANKS); p++) tbl.p[p] = g[p < P ? p : 0];
      hipLaunchKernelGGL((lamb_oneshot_kernel<PP, kOneshotBlock, kOneshotSub, false, uint16_t>), dim3(plan->res_ntiles),
                         dim3(kOneshotBlock), plan->res_lds, s, tbl, P, w, halfw, m, v, lay, plan->rpartials,
                         (const uint64_t*)plan->seg_len, plan->norms, plan->scale, rs, vec_ok, k);
    });
    CCN_HIP(hipGetLastError());
    const unsigned dg = plan->res_ntiles < 1024u ? plan->res_ntiles : 1024u;
    hipLaunchKernelGGL((lamb_deferred_kernel<kOneshotBlock, kOneshotSub, false, true>), dim3(dg), dim3(kOneshotBlock), 0, s, w,
                       halfw, (const float*)m, (const float*)v, lay, plan->scale, (const unsigned long long*)plan->ready,
                       (const double*)plan->rpartials, (const uint32_t*)plan->seg_rtile_begin, (const uint64_t*)plan->seg_len,
                       plan->norms, (const uint32_t*)plan->deferred, (const uint32_t*)rs.ndeferred, vec_ok, k);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }

  rc = make_two_pass_twin(plan);
  if (rc != CCN_OK) return rc;
  ccn_lamb_plan* tp = plan->two_pass_twin;
  const dim3 grid((unsigned)tp->ntiles);
  LambLayout lay;
  lay.tiles = tp->tiles;
  lay.seg_len = vec_ok ? tp->uniform_seg_len : 0;
  lay.seg_len_f = (float)tp->uniform_seg_len;
  lay.tile = kLambTile;
  lay.gtab = nullptr;
  lay.wtab = nullptr;
  lay.nbuf = (uint32_t)tp->nbuf;
  with_rank_count(P, [&](auto ptag) {
    constexpr int PP = decltype(ptag)::value;
    SrcTable<uint16_t, (PP ? PP : CCN_MAX_RANKS)> tbl;
    for (int p = 0; p < (PP ? PP : CCN_MAX_RANKS); p++) tbl.p[p] = g[p < P ? p : 0];
    // residency cap measured at N = 2^28, P = 8: 5 workgroups per CU 2.29 ms per step, 4: 2.41, 6: 2.32, uncapped: 2.35
    hipLaunchKernelGGL((lamb_pass1_f16g_kernel<PP>), grid, block, lds_for_residency(P >= 2 ? 5 : 0), s, tbl, P, (const float*)w, m,
                       v, lay, tp->partials, vec_ok, k);
  });
  CCN_HIP(hipGetLastError());
  const double* sums = tp->partials;
  const uint32_t* seg_begin = tp->seg_tile_begin;
  if (tp->ngroups) {
    hipLaunchKernelGGL(lamb_fold_kernel, dim3(tp->ngroups), block, 0, s, (const double*)tp->partials,
                       (const uint32_t*)tp->group_begin, tp->folded);
    CCN_HIP(hipGetLastError());
    sums = tp->folded;
    seg_begin = tp->seg_group_begin;
  }
  // the norms and scales land in the caller's plan, where ccn_lamb_plan_norms reads them
  hipLaunchKernelGGL(lamb_finalize_kernel, dim3((unsigned)tp->nseg), block, 0, s, sums, seg_begin, (const uint64_t*)tp->seg_len,
                     plan->norms, plan->scale, k.mode);
  CCN_HIP(hipGetLastError());
  hipLaunchKernelGGL(lamb_pass2_f16w_kernel, grid, block, 0, s, w, halfw, (const float*)m, (const float*)v, lay,
                     (const float*)plan->scale, vec_ok, k);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

}  // namespace

namespace ccn {

// Device address of `scratch` on each device, asked for once per device with that device current.
namespace {
constexpr int kStaticMaxDevices = 16;
LambStaticScratch* g_static_ptr[kStaticMaxDevices];
int g_static_rc[kStaticMaxDevices];
std::once_flag g_static_once[kStaticMaxDevices];
}  // namespace

int lamb_static_setup(LambStaticScratch** out) {
  int dev = -1;
  CCN_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kStaticMaxDevices) return CCN_ENODEV;
  std::call_once(g_static_once[dev], [dev] {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    g_static_rc[dev] = e == hipSuccess ? (ptr ? CCN_OK : CCN_EHIP) : hip_fail(e);
    g_static_ptr[dev] = static_cast<LambStaticScratch*>(ptr);
  });
  if (g_static_rc[dev] != CCN_OK) return g_static_rc[dev];
  if (out) *out = g_static_ptr[dev];
  return CCN_OK;
}

int lamb_static_setup() { return lamb_static_setup(nullptr); }

}  // namespace ccn

extern "C" {

int ccn_lamb_f32(ccn_lamb_plan* plan, const float* const* g, int P, float* w, float* m, float* v, float lr, float beta1,
                 float beta2, float eps, float wd, int step, int mode, void* stream) {
  if (!w) return CCN_EINVAL;
  return guarded([&] { return lamb_step(plan, g, P, w, nullptr, m, v, lr, beta1, beta2, eps, wd, step, mode, stream); });
}

int ccn_lamb_f32_scattered(ccn_lamb_plan* plan, const float* const* g, int P, float* const* w, float* m, float* v, float lr,
                           float beta1, float beta2, float eps, float wd, int step, int mode, void* stream) {
  if (!w) return CCN_EINVAL;
  return guarded([&] { return lamb_step(plan, g, P, nullptr, w, m, v, lr, beta1, beta2, eps, wd, step, mode, stream); });
}

int ccn_lamb_nccl_f16g(ccn_lamb_plan* plan, const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v,
                       float lr, float beta1, float beta2, float wd, void* stream) {
  return guarded([&] { return lamb_step_f16g(plan, g, P, w, halfw, m, v, lr, beta1, beta2, wd, stream); });
}

int ccn_lamb_f32_static(const float* const* g, int P, float* w, float* m, float* v, size_t N, size_t seg_len, float lr,
                        float beta1, float beta2, float eps, float wd, int step, int mode, double* norms, void* stream) {
  if (!g || !w || !m || !v || P < 1 || P > CCN_MAX_RANKS || step < 1 || N == 0 || seg_len == 0) return CCN_EINVAL;
  if (mode != CCN_LAMB_TRUST_RATIO && mode != CCN_LAMB_REFERENCE && mode != CCN_LAMB_NCCL_GLOBAL) return CCN_EINVAL;
  for (int p = 0; p < P; p++) if (!g[p]) return CCN_EINVAL;
  if (seg_len % kLambTile || N % seg_len) return CCN_EINVAL;   // whole tiles per segment, whole segments
  if (N > CCN_LAMB_STATIC_MAX_N || N / seg_len > CCN_LAMB_STATIC_MAX_SEGS) return CCN_ERANGE;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  LambStaticScratch* sc = nullptr;
  rc = lamb_static_setup(&sc);
  if (rc != CCN_OK) return rc;

  LambPrm k;
  k.b1 = beta1;
  k.omb1 = 1 - beta1;
  k.b2 = beta2;
  k.omb2 = 1 - beta2;
  k.eps = eps;
  k.wd = wd;
  k.lr = lr;
  k.mode = mode;
  k.bc1 = 1 - std::pow((double)beta1, (double)step);
  k.bc2 = 1 - std::pow((double)beta2, (double)step);

  const uint32_t nseg = (uint32_t)(N / seg_len), tps = (uint32_t)(seg_len / kLambTile), ntiles = nseg * tps;
  const uint32_t gps = tps > kLambFold ? (tps + kLambFold - 1) / kLambFold : 0;   // the plan's rule for going through groups
  bool al = aligned16(w) && aligned16(m) && aligned16(v);
  for (int p = 0; p < P; p++) al = al && aligned16(g[p]);
  const int vec_ok = al ? 1 : 0;
  LambLayout lay;
  lay.tiles = nullptr;
  lay.seg_len = seg_len;
  lay.seg_len_f = (float)seg_len;
  lay.tile = kLambTile;
  lay.gtab = nullptr;
  lay.wtab = nullptr;
  lay.nbuf = nseg;
  hipStream_t s = as_stream(stream);
  const dim3 block(kBlock), grid(ntiles);
  double* const norms_dst = norms ? norms : sc->norms;

  const uint32_t entries = (gps ? nseg * gps : nseg) + 1;
  hipLaunchKernelGGL(lamb_static_tables_kernel, dim3((entries + kBlock - 1) / kBlock), block, 0, s, sc, nseg, tps, gps,
                     (uint64_t)seg_len);
  CCN_HIP(hipGetLastError());
  with_rank_count(P, [&](auto ptag) {
    constexpr int PP = decltype(ptag)::value;
    SrcTable<float, (PP ? PP : CCN_MAX_RANKS)> tbl;
    for (int p = 0; p < (PP ? PP : CCN_MAX_RANKS); p++) tbl.p[p] = g[p < P ? p : 0];
    hipLaunchKernelGGL((lamb_pass1_kernel<PP, false>), grid, block, lds_for_residency(P >= 2 ? 4 : 0), s, tbl, P, (const float*)w, m,
                       v, lay, sc->partials, vec_ok, k);
  });
  CCN_HIP(hipGetLastError());
  const double* sums = sc->partials;
  if (gps) {
    hipLaunchKernelGGL(lamb_fold_kernel, dim3(nseg * gps), block, 0, s, (const double*)sc->partials,
                       (const uint32_t*)sc->group_begin, sc->folded);
    CCN_HIP(hipGetLastError());
    sums = sc->folded;
  }
  hipLaunchKernelGGL(lamb_finalize_kernel, dim3(nseg), block, 0, s, sums, (const uint32_t*)sc->seg_begin,
                     (const uint64_t*)sc->seg_len, norms_dst, sc->scale, mode);
  CCN_HIP(hipGetLastError());
  hipLaunchKernelGGL((lamb_pass2_kernel<false>), grid, block, 0, s, w, (const float*)m, (const float*)v, lay,
                     (const float*)sc->scale, vec_ok, k);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

int ccn_lamb_plan_tune(ccn_lamb_plan* plan, int knob, long value) {
  if (!plan || value < 0) return CCN_EINVAL;
  switch (knob) {
    case CCN_LAMB_KNOB_SPIN_LIMIT:
      if (value > 0x7fffffffL) return CCN_ERANGE;
      plan->spin_limit = (uint32_t)value;
      return CCN_OK;
    case CCN_LAMB_KNOB_TWO_PASS: plan->force_two_pass = value != 0; return CCN_OK;
    case CCN_LAMB_KNOB_WITHHOLD: plan->withhold = value != 0 ? 1u : 0u; return CCN_OK;
    default: return CCN_EINVAL;
  }
}

int ccn_lamb_plan_norms(ccn_lamb_plan* plan, double* norms_host, void* stream) {
  if (!plan || !norms_host) return CCN_EINVAL;
  hipStream_t s = as_stream(stream);
  CCN_HIP(hipMemcpyAsync(norms_host, plan->norms, 2 * (size_t)plan->nseg * sizeof(double), hipMemcpyDeviceToHost, s));
  CCN_HIP(hipStreamSynchronize(s));
  return CCN_OK;
}

}  // extern "C"
