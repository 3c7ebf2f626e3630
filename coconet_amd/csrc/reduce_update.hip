// Fused "reduce P rank-gradient buffers + optimizer update" kernels for gfx950.
//
// One streaming skeleton (fused_stream_kernel) is instantiated with a math policy per optimizer.
// The skeleton owns the memory behaviour: 128-bit loads of every operand, all loads of a tile issued
// before the first use, one tile per workgroup, in-place 128-bit stores.  The policy owns the
// arithmetic, written operation by operation in the order of the reference's checker loops so that
// every fp32 rounding happens where the checker's does (the library is compiled with
// -ffp-contract=off; division and square root are the correctly rounded ones).
#include "ccn_common.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

namespace ccn {

template <int NS> struct StateTable { float* p[NS > 0 ? NS : 1]; };

// ------------------------------------------------------------------------------------------------------------------
// Math policies.
//   G        storage type of one gradient element (float, or uint16_t holding fp16 bits)
//   NS       number of fp32 state arrays, read and rewritten in place (order: w, m, v)
//   OUT16    one extra uint16 output per element          OUTF   one extra fp32 output per element
//   FLAG     the kernel ORs a "bad element seen" bit into *flag
//   Acc      running gradient sum;  first()/next() fold the P ranks in ascending order
//   apply()  consumes the sum and the state of one element; returns true if the element was "bad"
// ------------------------------------------------------------------------------------------------------------------
struct SumF32 {
  using G = float;
  using Acc = float;
  static constexpr int PACK_BYTES = 16;
  template <class Prm> static __device__ __forceinline__ Acc first(G x, const Prm&) { return x; }
  template <class Prm> static __device__ __forceinline__ void next(Acc& a, G x, const Prm&) { a = a + x; }
};

struct ReduceMath : SumF32 {
  static constexpr int NS = 0, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = true, FLAG = false;
  struct Prm {};
  static __device__ __forceinline__ bool apply(Acc gs, float*, uint16_t&, float& of, const Prm&) {
    of = gs;
    return false;
  }
};

// examples/test-sgd.cu:17-18
struct SgdMath : SumF32 {
  static constexpr int NS = 1, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = false, FLAG = false;
  struct Prm { float lr; };
  static __device__ __forceinline__ bool apply(Acc gs, float* st, uint16_t&, float&, const Prm& k) {
    st[0] = (st[0] - (k.lr * gs));
    return false;
  }
};

// nccl-overlap/samples/single-process-wX.cu:141
struct AxpbyMath : SumF32 {
  static constexpr int NS = 1, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = false, FLAG = false;
  struct Prm { float alpha, beta; };
  static __device__ __forceinline__ bool apply(Acc gs, float* st, uint16_t&, float&, const Prm& k) {
    st[0] = k.alpha * st[0] + k.beta * gs;
    return false;
  }
};

// examples/test-adam.cu:14-38
struct PseudoAdamMath : SumF32 {
  static constexpr int NS = 3, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = false, FLAG = false;
  struct Prm { float lr, b1, omb1, b2, omb2; };
  static __device__ __forceinline__ bool apply(Acc S0, float* st, uint16_t&, float&, const Prm& k) {
    const float S2 = ((k.b2 * st[2]) + (k.omb2 * (S0 * S0)));
    const float S4 = (S2 / k.b2);
    const float S1 = ((k.b1 * st[1]) + (k.omb1 * S0));
    const float S3 = (S1 / k.b1);
    st[0] = (st[0] - ((k.lr * S3) / S4));
    st[1] = S1;
    st[2] = S2;
    return false;
  }
};

// nccl-overlap/samples/multi-process-adam-scattered.cpp:112-136
struct AdamPrm {
  float b1, omb1, b2, omb2, eps, stepsize, inv_scale;
  double bc1, bc2;   // 1 - beta^t, evaluated in double on the host like the checker's pow()
};
__device__ __forceinline__ void adam_step(float gs, float* st, const AdamPrm& k) {
  const float mi = k.b1 * st[1] + k.omb1 * gs;
  const float vi = k.b2 * st[2] + k.omb2 * gs * gs;
  const float m_ = (float)((double)mi / k.bc1);
  const float v_ = (float)((double)vi / k.bc2);
  const float x = k.stepsize * m_ / (sqrtf(v_) + k.eps);
  st[0] = st[0] + x;
  st[1] = mi;
  st[2] = vi;
}

struct AdamMath : SumF32 {
  static constexpr int NS = 3, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = false, FLAG = false;
  using Prm = AdamPrm;
  static __device__ __forceinline__ bool apply(Acc gs, float* st, uint16_t&, float&, const Prm& k) {
    adam_step(gs, st, k);
    return false;
  }
};

// 16-bit gradients with a loss scale.  BF16 = false: IEEE half, overflow = exponent 0x1F; BF16 = true: bfloat16,
// overflow = exponent 0xFF.  The 16-bit copy of the weights is written in the same format.
template <bool BF16> struct Half16 {
  static __device__ __forceinline__ float widen(uint16_t h) { return BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h); }
  static __device__ __forceinline__ uint16_t narrow(float f) { return BF16 ? f32_to_bf16_bits(f) : f32_to_f16_bits(f); }
  static __device__ __forceinline__ bool non_finite(uint16_t h) {
    return BF16 ? (h & 0x7f80u) == 0x7f80u : (h & 0x7c00u) == 0x7c00u;
  }
};
template <bool BF16> struct Adam16MathT {
  using G = uint16_t;
  using H = Half16<BF16>;
  static constexpr int PACK_BYTES = 8;   // 16-bit gradients move as 8-byte packs: measured 6 points of HBM peak faster than 16-byte packs
  struct Acc { float s; bool bad; };
  static constexpr int NS = 3, UNROLL = 1;
  static constexpr bool OUT16 = true, OUTF = false, FLAG = true;
  using Prm = AdamPrm;
  static __device__ __forceinline__ Acc first(G h, const Prm& k) { return Acc{H::widen(h) * k.inv_scale, H::non_finite(h)}; }
  static __device__ __forceinline__ void next(Acc& a, G h, const Prm& k) {
    a.s = a.s + H::widen(h) * k.inv_scale;
    a.bad = a.bad | H::non_finite(h);
  }
  static __device__ __forceinline__ bool apply(Acc a, float* st, uint16_t& o16, float&, const Prm& k) {
    if (!a.bad) adam_step(a.s, st, k);
    o16 = H::narrow(st[0]);
    return a.bad;
  }
};
using Adam16Math = Adam16MathT<false>;
using AdamBf16Math = Adam16MathT<true>;

struct Overflow16Math {
  using G = uint16_t;
  static constexpr int PACK_BYTES = 8;   // fp16 gradients move as 8-byte packs: measured 6 points of HBM peak faster than 16-byte packs
  using Acc = bool;
  static constexpr int NS = 0, UNROLL = 1;
  static constexpr bool OUT16 = false, OUTF = false, FLAG = true;
  struct Prm {};
  static __device__ __forceinline__ Acc first(G h, const Prm&) { return (h & 0x7c00u) == 0x7c00u; }
  static __device__ __forceinline__ void next(Acc& a, G h, const Prm&) { a = a | ((h & 0x7c00u) == 0x7c00u); }
  static __device__ __forceinline__ bool apply(Acc a, float*, uint16_t&, float&, const Prm&) { return a; }
};

// nccl/src/collectives/device/reduce_kernel.h:36-68 in the call order of common_kernel.h:875-921
struct FusedAdamRefMath {
  using G = uint16_t;
  static constexpr int PACK_BYTES = 8;   // fp16 gradients move as 8-byte packs: measured 6 points of HBM peak faster than 16-byte packs
  using Acc = uint16_t;   // the ring carries the running sum in fp16
  static constexpr int NS = 3, UNROLL = 1;
  static constexpr bool OUT16 = true, OUTF = false, FLAG = false;
  struct Prm { float lr, b1, b2, omb2; };
  static __device__ __forceinline__ Acc first(G h, const Prm&) { return h; }
  static __device__ __forceinline__ void next(Acc& a, G h, const Prm&) {
    a = f32_to_f16_bits(f16_bits_to_f32(a) + f16_bits_to_f32(h));
  }
  static __device__ __forceinline__ bool apply(Acc S0, float* st, uint16_t& o16, float&, const Prm& k) {
    const float s0f = f16_bits_to_f32(S0);
    const float sq = f16_bits_to_f32(f32_to_f16_bits(s0f * s0f));           // S0*S0 evaluated in half
    const float S2 = ((st[2] * k.b2) + (sq * k.omb2));
    const float S4 = (S2 / k.b2);
    const float S1 = ((st[1] * k.b2) + (s0f * k.omb2));                      // beta2 on the first moment, as the kernel
    const float S3 = (S1 / k.b1);
    const float S5 = ((S3 * k.lr) / sqrtf(S4));
    st[2] = S2;
    st[1] = S1;
    st[0] = st[0] - S5;
    o16 = f32_to_f16_bits(st[0]);
    return false;
  }
};

// ------------------------------------------------------------------------------------------------------------------
// The streaming skeleton.  P > 0: rank count known at compile time.  P == 0: rank count nP (9..16) read at run
// time; the loads of ranks >= nP are skipped by wavefront-uniform branches.  Either way all loads of a thread
// are in flight together before the first use.
// VEC elements per thread per access; n counts elements.  Elements [ (n/VEC)*VEC, n ) are finished
// by the first lanes of workgroup 0 with scalar accesses.
// ------------------------------------------------------------------------------------------------------------------
template <class M, int P>
__device__ __forceinline__ void one_element(const SrcTable<typename M::G, (P ? P : CCN_MAX_RANKS)>& g, int nP,
                                            const StateTable<M::NS>& st, uint16_t* out16, float* outf, size_t i,
                                            const typename M::Prm& prm, bool& bad) {
  const int np = P ? P : nP;
  typename M::Acc a = M::first(g.p[0][i], prm);
  for (int p = 1; p < np; p++) M::next(a, g.p[p][i], prm);
  float s[M::NS > 0 ? M::NS : 1];
#pragma unroll
  for (int k = 0; k < M::NS; k++) s[k] = st.p[k][i];
  uint16_t o16 = 0;
  float of = 0.f;
  bad |= M::apply(a, s, o16, of, prm);
#pragma unroll
  for (int k = 0; k < M::NS; k++) st.p[k][i] = s[k];
  if constexpr (M::OUT16) out16[i] = o16;
  if constexpr (M::OUTF) outf[i] = of;
}

template <class M, int P, int VEC, int UNROLL, int BS>
__global__ __launch_bounds__(BS) void fused_stream_kernel(
    const SrcTable<typename M::G, (P ? P : CCN_MAX_RANKS)> g, const int nP, const StateTable<M::NS> st,
    uint16_t* out16, float* outf, uint32_t* flag, const size_t n, const typename M::Prm prm) {
  using G = typename M::G;
  constexpr int NSX = M::NS > 0 ? M::NS : 1;
  constexpr int PX = P > 0 ? P : CCN_MAX_RANKS;   // P == 0: rank count nP (9..16) known at run time only
  const size_t nvec = n / VEC;
  bool bad = false;
  // One tile per workgroup, no loop: wavefronts here live for a single pack per array, so every instruction
  // ahead of the first load is exposed latency (a grid-stride loop's bookkeeping costs ~3% of bandwidth).
  // The y dimension of the grid only comes into play beyond 2^30 tiles.
  const size_t blk = (size_t)blockIdx.x + (size_t)blockIdx.y * gridDim.x;
  const size_t t0 = blk * ((size_t)BS * UNROLL);
  {
    Pack<G, VEC> gv[UNROLL][PX];
    Pack<float, VEC> sv[UNROLL][NSX];
    typename M::Acc acc[UNROLL][VEC];
    // ---- issue every load of the tile -------------------------------------------------------------------------
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const size_t e0 = (t0 + (size_t)u * BS + threadIdx.x) * VEC;   // first element of this thread's pack
      if (e0 < nvec * VEC) {
#pragma unroll
        for (int p = 0; p < PX; p++)
          if (P > 0 || p < nP) gv[u][p] = load_stream<G, VEC>(g.p[p] + e0);
#pragma unroll
        for (int k = 0; k < M::NS; k++) sv[u][k] = load_stream<float, VEC>(st.p[k] + e0);
      }
    }
    // ---- fold, update, store ---------------------------------------------------------------------------------
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const size_t e0 = (t0 + (size_t)u * BS + threadIdx.x) * VEC;
      if (e0 < nvec * VEC) {
        Pack<uint16_t, VEC> o16v;
        Pack<float, VEC> ofv;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          acc[u][e] = M::first(gv[u][0].d[e], prm);
#pragma unroll
          for (int p = 1; p < PX; p++)
            if (P > 0 || p < nP) M::next(acc[u][e], gv[u][p].d[e], prm);
          float s[NSX];
#pragma unroll
          for (int k = 0; k < M::NS; k++) s[k] = sv[u][k].d[e];
          uint16_t o16 = 0;
          float of = 0.f;
          bad |= M::apply(acc[u][e], s, o16, of, prm);
#pragma unroll
          for (int k = 0; k < M::NS; k++) sv[u][k].d[e] = s[k];
          o16v.d[e] = o16;
          ofv.d[e] = of;
        }
#pragma unroll
        for (int k = 0; k < M::NS; k++) store_stream<float, VEC>(st.p[k] + e0, sv[u][k]);
        if constexpr (M::OUT16) store_stream<uint16_t, VEC>(out16 + e0, o16v);
        if constexpr (M::OUTF) store_stream<float, VEC>(outf + e0, ofv);
      }
    }
  }

  if constexpr (VEC > 1) {
    const size_t rem = n - nvec * VEC;
    if (blk == 0 && threadIdx.x < rem) one_element<M, P>(g, nP, st, out16, outf, nvec * VEC + threadIdx.x, prm, bad);
  }

  if constexpr (M::FLAG) {
    // one atomic per wavefront that saw a bad element (none in the common case)
    if (__ballot(bad) != 0ull && (threadIdx.x & (kWave - 1)) == 0) atomicOr(flag, 1u);
  }
}

__global__ void set_u32_kernel(uint32_t* p, uint32_t v) { *p = v; }

__global__ __launch_bounds__(kBlock) void fill_f32_kernel(float* __restrict__ dst, float value, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) dst[i] = value;
}

// ------------------------------------------------------------------------------------------------------------------
// Scattered layout: gradients and weights live in nbuff separate buffers (one per parameter tensor), the moments in
// single arrays that follow the buffers' concatenation, as ncclAllReduceScatteredAdam takes them
// (nccl-overlap/src/nccl.h.in:216-218).  A plan cuts every buffer into tiles of kScatTile elements, numbered
// through all buffers; one single-wavefront workgroup per tile finds its buffer, reads the buffer's pointers from a
// device table (rank-major gradient pointers, then the weight pointers), then streams exactly like
// fused_stream_kernel.  State array 0 of the policy (w) is scattered, the others (m, v) are contiguous.
//
// Finding the buffer costs no trip to HBM: a per-tile record would be read once per launch and so always miss the
// caches, doubling the time a wavefront waits before it can issue its loads.  Instead one word per group of 32 tiles
// names the buffer that holds the group's first tile (a 64-byte line of those words serves 512 consecutive
// workgroups, so it is in L2 for all but the first), and the per-buffer records (first tile, first element), which
// stay cached, are scanned forward from there: no step at all unless a buffer ends inside the group.  The pointers of
// the group's buffer are fetched together with its record, and again only if the scan moved on.
// ------------------------------------------------------------------------------------------------------------------
constexpr int kScatTile = kWave * 4;   // 256 elements: one 4-element pack per lane
constexpr int kScatCoarseShift = 5;    // one coarse word per 32 tiles

struct ScatBuf {
  uint64_t goff;        // first element of the buffer in the concatenation (index into the moment arrays)
  uint32_t tile_begin;  // number of its first tile
  uint32_t pad;
};                      // entry nbuff holds the totals, so that [b + 1] always ends buffer b

template <class M, int P>
__global__ __launch_bounds__(kWave) void scattered_stream_kernel(const uint32_t* __restrict__ coarse,
                                                                 const ScatBuf* __restrict__ bufs,
                                                                 const float* const* __restrict__ gtab,
                                                                 float* const* __restrict__ wtab, const int nP,
                                                                 const uint32_t nbuff, const StateTable<M::NS> moments,
                                                                 const typename M::Prm prm) {
  static_assert(M::NS >= 1 && !M::OUT16 && !M::OUTF && !M::FLAG, "fp32 policies with w as state 0");
  constexpr int PX = P > 0 ? P : CCN_MAX_RANKS;
  const uint32_t tile = blockIdx.x + blockIdx.y * gridDim.x;
  uint32_t buf = coarse[tile >> kScatCoarseShift];
  ScatBuf r0 = bufs[buf], r1 = bufs[buf + 1];
  const float* gp[PX];
  float* wp;
  auto fetch_pointers = [&]() {
#pragma unroll
    for (int p = 0; p < PX; p++)
      if (P > 0 || p < nP) gp[p] = gtab[(size_t)p * nbuff + buf];
    wp = wtab[buf];
  };
  fetch_pointers();
  if (r1.tile_begin <= tile) {
    do {   // ends: entry nbuff holds the tile count, above every tile number
      buf++;
      r0 = r1;
      r1 = bufs[buf + 1];
    } while (r1.tile_begin <= tile);
    fetch_pointers();
  }
  struct { uint64_t off, goff; uint32_t count; } t;
  t.off = (uint64_t)(tile - r0.tile_begin) * kScatTile;
  t.goff = r0.goff + t.off;
  const uint64_t left = (r1.goff - r0.goff) - t.off;
  t.count = left < (uint64_t)kScatTile ? (uint32_t)left : (uint32_t)kScatTile;
  uintptr_t bits = 0;
#pragma unroll
  for (int p = 0; p < PX; p++) {
    if (P > 0 || p < nP) {
      gp[p] += t.off;
      bits |= reinterpret_cast<uintptr_t>(gp[p]);
    }
  }
  float* sp[M::NS];
  sp[0] = wp + t.off;
#pragma unroll
  for (int k = 1; k < M::NS; k++) sp[k] = moments.p[k] + t.goff;
#pragma unroll
  for (int k = 0; k < M::NS; k++) bits |= reinterpret_cast<uintptr_t>(sp[k]);
  const uint32_t j0 = threadIdx.x * 4;
  if (j0 >= t.count) return;
  if ((bits & 15u) == 0 && j0 + 4 <= t.count) {
    Pack<float, 4> gv[PX], sv[M::NS];
#pragma unroll
    for (int p = 0; p < PX; p++)
      if (P > 0 || p < nP) gv[p] = load_stream<float, 4>(gp[p] + j0);
#pragma unroll
    for (int k = 0; k < M::NS; k++) sv[k] = load_stream<float, 4>(sp[k] + j0);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      typename M::Acc a = M::first(gv[0].d[e], prm);
#pragma unroll
      for (int p = 1; p < PX; p++)
        if (P > 0 || p < nP) M::next(a, gv[p].d[e], prm);
      float s[M::NS];
#pragma unroll
      for (int k = 0; k < M::NS; k++) s[k] = sv[k].d[e];
      uint16_t o16 = 0;
      float of = 0.f;
      (void)M::apply(a, s, o16, of, prm);
#pragma unroll
      for (int k = 0; k < M::NS; k++) sv[k].d[e] = s[k];
    }
#pragma unroll
    for (int k = 0; k < M::NS; k++) store_stream<float, 4>(sp[k] + j0, sv[k]);
  } else {
    const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
    for (uint32_t j = j0; j < j1; j++) {
      typename M::Acc a = M::first(gp[0][j], prm);
      for (int p = 1; p < (P ? P : nP); p++) M::next(a, gp[p][j], prm);
      float s[M::NS];
#pragma unroll
      for (int k = 0; k < M::NS; k++) s[k] = sp[k][j];
      uint16_t o16 = 0;
      float of = 0.f;
      (void)M::apply(a, s, o16, of, prm);
#pragma unroll
      for (int k = 0; k < M::NS; k++) sp[k][j] = s[k];
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Host side: validation, alignment-based choice of the access width, dispatch on P.
// ------------------------------------------------------------------------------------------------------------------
template <class M, int P, int VEC, int UNROLL>
static int launch_one(const typename M::G* const* g, int nP, const StateTable<M::NS>& st, uint16_t* out16, float* outf,
                      uint32_t* flag, size_t n, const typename M::Prm& prm, hipStream_t s) {
  SrcTable<typename M::G, (P ? P : CCN_MAX_RANKS)> tbl;
  for (int p = 0; p < (P ? P : CCN_MAX_RANKS); p++) tbl.p[p] = g[p < nP ? p : 0];
  const size_t nvec = n / VEC;
  const int load_bytes = VEC * (nP * (int)sizeof(typename M::G) + M::NS * 4);
  const int store_bytes = VEC * (M::NS * 4 + (M::OUT16 ? 2 : 0) + (M::OUTF ? 4 : 0));
  // do the arrays start alike?  (more than half of them in the same 4 KiB step of a 64 KiB period: plain allocations of
  // equal size do, the library's allocator staggers them)
  int slots[16] = {0};
  for (int p = 0; p < nP; p++) slots[(reinterpret_cast<uintptr_t>(g[p]) >> 12) & 15]++;
  for (int k = 0; k < M::NS; k++) slots[(reinterpret_cast<uintptr_t>(st.p[k]) >> 12) & 15]++;
  int most = 0;
  for (int k = 0; k < 16; k++) most = slots[k] > most ? slots[k] : most;
  const bool alike = 2 * most > nP + M::NS;
  const StreamShape sh = stream_shape(load_bytes, store_bytes, (int)sizeof(typename M::G), alike);
  size_t tiles = (nvec + (size_t)sh.block * UNROLL - 1) / ((size_t)sh.block * UNROLL);
  if (tiles < 1) tiles = 1;                                     // the n % VEC tail still needs workgroup 0
  const size_t gx = tiles < 0x40000000ull ? tiles : 0x40000000ull;
  const dim3 grid((unsigned)gx, (unsigned)((tiles + gx - 1) / gx));
  if (sh.block == 64)
    hipLaunchKernelGGL((fused_stream_kernel<M, P, VEC, UNROLL, 64>), grid, dim3(64), sh.lds_bytes, s, tbl, nP, st, out16,
                       outf, flag, n, prm);
  else
    hipLaunchKernelGGL((fused_stream_kernel<M, P, VEC, UNROLL, 256>), grid, dim3(256), sh.lds_bytes, s, tbl, nP, st,
                       out16, outf, flag, n, prm);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

template <class M, int VEC, int UNROLL>
static int launch_p(const typename M::G* const* g, int P, const StateTable<M::NS>& st, uint16_t* out16, float* outf,
                    uint32_t* flag, size_t n, const typename M::Prm& prm, hipStream_t s) {
  switch (P) {
#define CCN_CASE(K) case K: return launch_one<M, K, VEC, UNROLL>(g, P, st, out16, outf, flag, n, prm, s);
    CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
    default: return launch_one<M, 0, VEC, UNROLL>(g, P, st, out16, outf, flag, n, prm, s);
  }
}

template <class M>
static int launch(const typename M::G* const* g, int P, float* const* state, uint16_t* out16, float* outf,
                  uint32_t* flag, size_t n, const typename M::Prm& prm, void* stream) {
  if (!g || P < 1 || P > CCN_MAX_RANKS) return CCN_EINVAL;
  for (int p = 0; p < P; p++) if (!g[p]) return CCN_EINVAL;
  StateTable<M::NS> st;
  st.p[0] = nullptr;
  for (int k = 0; k < M::NS; k++) {
    if (!state[k]) return CCN_EINVAL;
    st.p[k] = state[k];
  }
  if (M::OUT16 && !out16) return CCN_EINVAL;
  if (M::OUTF && !outf) return CCN_EINVAL;
  if (M::FLAG && !flag) return CCN_EINVAL;
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (M::FLAG) {
    hipLaunchKernelGGL(set_u32_kernel, dim3(1), dim3(1), 0, s, flag, 0u);
    CCN_HIP(hipGetLastError());
  }
  if (n == 0) return CCN_OK;

  bool al = true;
  for (int p = 0; p < P; p++) al = al && aligned16(g[p]);
  for (int k = 0; k < M::NS; k++) al = al && aligned16(state[k]);
  if (M::OUT16) al = al && aligned16(out16);
  if (M::OUTF) al = al && aligned16(outf);
  constexpr int VEC = M::PACK_BYTES / (int)sizeof(typename M::G);
  if (al) return launch_p<M, VEC, M::UNROLL>(g, P, st, out16, outf, flag, n, prm, s);
  return launch_p<M, 1, 4>(g, P, st, out16, outf, flag, n, prm, s);
}

static AdamPrm make_adam_prm(float lr, float beta1, float beta2, float eps, int step, float inv_scale) {
  AdamPrm k;
  k.b1 = beta1;
  k.omb1 = 1 - beta1;
  k.b2 = beta2;
  k.omb2 = 1 - beta2;
  k.eps = eps;
  k.stepsize = -lr;
  k.inv_scale = inv_scale;
  k.bc1 = 1 - std::pow((double)beta1, (double)step);
  k.bc2 = 1 - std::pow((double)beta2, (double)step);
  return k;
}

}  // namespace ccn

using namespace ccn;

struct ccn_scatter_plan {
  int device = -1;
  uint32_t nbuff = 0;
  size_t total = 0;
  size_t ntiles = 0;
  uint32_t* coarse = nullptr;          // [ceil(ntiles / 2^kScatCoarseShift)] buffer of the group's first tile
  ScatBuf* bufs = nullptr;             // [nbuff + 1]
  const void** table_dev = nullptr;    // [CCN_MAX_RANKS * nbuff] gradient pointers, rank-major, then [nbuff] weight pointers
  const void** table_pinned = nullptr; // staging copy in pinned host memory
  std::vector<const void*> shadow;     // what the device table holds
  int shadow_ranks = 0;
};

namespace {

// Brings the device pointer table in line with the caller's pointers; copies (and waits for the copy, so that the
// staging buffer can be reused) only when they have changed since the last call.
int sync_pointer_table(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, hipStream_t s) {
  const size_t nb = plan->nbuff, words = (size_t)(CCN_MAX_RANKS + 1) * nb;
  bool same = plan->shadow_ranks == P && plan->shadow.size() == words;
  for (int p = 0; same && p < P; p++)
    for (size_t b = 0; b < nb; b++) same = same && plan->shadow[(size_t)p * nb + b] == g[(size_t)p * nb + b];
  for (size_t b = 0; same && b < nb; b++) same = same && plan->shadow[(size_t)CCN_MAX_RANKS * nb + b] == w[b];
  if (same) return CCN_OK;
  plan->shadow.assign(words, nullptr);
  for (int p = 0; p < P; p++)
    for (size_t b = 0; b < nb; b++) plan->shadow[(size_t)p * nb + b] = g[(size_t)p * nb + b];
  for (size_t b = 0; b < nb; b++) plan->shadow[(size_t)CCN_MAX_RANKS * nb + b] = w[b];
  plan->shadow_ranks = P;
  std::memcpy(plan->table_pinned, plan->shadow.data(), words * sizeof(void*));
  CCN_HIP(hipMemcpyAsync(plan->table_dev, plan->table_pinned, words * sizeof(void*), hipMemcpyHostToDevice, s));
  CCN_HIP(hipStreamSynchronize(s));
  return CCN_OK;
}

template <class M>
int launch_scattered(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, float* const* moments,
                     const typename M::Prm& prm, void* stream) {
  if (!plan || !g || !w || P < 1 || P > CCN_MAX_RANKS) return CCN_EINVAL;
  for (size_t i = 0; i < (size_t)P * plan->nbuff; i++) if (!g[i]) return CCN_EINVAL;
  for (size_t b = 0; b < plan->nbuff; b++) if (!w[b]) return CCN_EINVAL;
  StateTable<M::NS> st;
  st.p[0] = nullptr;
  for (int k = 1; k < M::NS; k++) {
    if (!moments || !moments[k - 1]) return CCN_EINVAL;
    st.p[k] = moments[k - 1];
  }
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  if (di->device != plan->device) return CCN_EINVAL;
  hipStream_t s = as_stream(stream);
  rc = sync_pointer_table(plan, g, P, w, s);
  if (rc != CCN_OK) return rc;
  const float* const* gtab = reinterpret_cast<const float* const*>(plan->table_dev);
  float* const* wtab = reinterpret_cast<float* const*>(const_cast<void**>(plan->table_dev) + (size_t)CCN_MAX_RANKS * plan->nbuff);
  // A wavefront here first finds its buffer and reads the buffer's pointers, and only then its data: two short round
  // trips (cache hits) more than the flat kernels.  Measured at P = 8: 8 to 10 wavefronts per CU give 78 % of HBM peak,
  // 7 give 76 %, 13 give 77 %.
  const unsigned lds = lds_for_residency(8);
  const size_t gx = plan->ntiles < 0x40000000ull ? plan->ntiles : 0x40000000ull;
  const dim3 grid((unsigned)gx, (unsigned)((plan->ntiles + gx - 1) / gx));
  if (grid.x * (size_t)grid.y != plan->ntiles) return CCN_ERANGE;   // the kernel has no bounds check on the tile index
  switch (P) {
#define CCN_CASE(K) \
  case K: hipLaunchKernelGGL((scattered_stream_kernel<M, K>), grid, dim3(kWave), lds, s, (const uint32_t*)plan->coarse, \
                             (const ScatBuf*)plan->bufs, gtab, \
                             wtab, P, plan->nbuff, st, prm); break;
    CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
    default:
      hipLaunchKernelGGL((scattered_stream_kernel<M, 0>), grid, dim3(kWave), lds, s, (const uint32_t*)plan->coarse,
                         (const ScatBuf*)plan->bufs, gtab, wtab, P, plan->nbuff, st, prm);
  }
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

}  // namespace

extern "C" {

int ccn_fill_f32(float* dst, float value, size_t n, void* stream) {
  if (n == 0) return CCN_OK;
  if (!dst) return CCN_EINVAL;
  const unsigned grid = stream_grid(n, kBlock);
  hipLaunchKernelGGL(fill_f32_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), dst, value, n);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

int ccn_reduce_f32(const float* const* g, int P, float* out, size_t N, void* stream) {
  return launch<ReduceMath>(g, P, nullptr, nullptr, out, nullptr, N, ReduceMath::Prm{}, stream);
}

int ccn_sgd_f32(const float* const* g, int P, float* w, size_t N, float lr, void* stream) {
  float* st[1] = {w};
  return launch<SgdMath>(g, P, st, nullptr, nullptr, nullptr, N, SgdMath::Prm{lr}, stream);
}

int ccn_sgd_axpby_f32(const float* const* g, int P, float* w, size_t N, float alpha, float beta, void* stream) {
  float* st[1] = {w};
  return launch<AxpbyMath>(g, P, st, nullptr, nullptr, nullptr, N, AxpbyMath::Prm{alpha, beta}, stream);
}

int ccn_pseudo_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N, float lr, float beta1,
                        float beta2, void* stream) {
  float* st[3] = {w, m, v};
  PseudoAdamMath::Prm k{lr, beta1, 1 - beta1, beta2, 1 - beta2};
  return launch<PseudoAdamMath>(g, P, st, nullptr, nullptr, nullptr, N, k, stream);
}

int ccn_adam_f32(const float* const* g, int P, float* w, float* m, float* v, size_t N, float lr, float beta1,
                 float beta2, float eps, int step, void* stream) {
  if (step < 1) return CCN_EINVAL;
  float* st[3] = {w, m, v};
  return launch<AdamMath>(g, P, st, nullptr, nullptr, nullptr, N, make_adam_prm(lr, beta1, beta2, eps, step, 1.0f), stream);
}

int ccn_adam_f16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16, size_t N, float lr,
                  float beta1, float beta2, float eps, int step, float inv_scale, uint32_t* overflow_flag, void* stream) {
  if (step < 1) return CCN_EINVAL;
  float* st[3] = {w, m, v};
  return launch<Adam16Math>(g, P, st, w16, nullptr, overflow_flag, N, make_adam_prm(lr, beta1, beta2, eps, step, inv_scale),
                            stream);
}

int ccn_adam_bf16g(const uint16_t* const* g, int P, float* w, float* m, float* v, uint16_t* w16, size_t N, float lr,
                   float beta1, float beta2, float eps, int step, float inv_scale, uint32_t* overflow_flag, void* stream) {
  if (step < 1) return CCN_EINVAL;
  float* st[3] = {w, m, v};
  return launch<AdamBf16Math>(g, P, st, w16, nullptr, overflow_flag, N, make_adam_prm(lr, beta1, beta2, eps, step, inv_scale),
                              stream);
}

int ccn_overflow_check_f16(const uint16_t* const* g, int P, size_t N, uint32_t* overflow_flag, void* stream) {
  return launch<Overflow16Math>(g, P, nullptr, nullptr, nullptr, overflow_flag, N, Overflow16Math::Prm{}, stream);
}

int ccn_fused_adam_ref_f16g(const uint16_t* const* g, int P, float* w, uint16_t* halfw, float* m, float* v, size_t N,
                            float lr, float beta1, float beta2, void* stream) {
  float* st[3] = {w, m, v};
  FusedAdamRefMath::Prm k{lr, beta1, beta2, 1 - beta2};
  return launch<FusedAdamRefMath>(g, P, st, halfw, nullptr, nullptr, N, k, stream);
}

int ccn_scatter_plan_destroy(ccn_scatter_plan* plan) {
  if (!plan) return CCN_OK;
  int rc = CCN_OK;
  if (plan->coarse && hipFree(plan->coarse) != hipSuccess) rc = CCN_EHIP;
  if (plan->bufs && hipFree(plan->bufs) != hipSuccess) rc = CCN_EHIP;
  if (plan->table_dev && hipFree(plan->table_dev) != hipSuccess) rc = CCN_EHIP;
  if (plan->table_pinned && hipHostFree(plan->table_pinned) != hipSuccess) rc = CCN_EHIP;
  delete plan;
  return rc;
}

static int scatter_plan_create(const size_t* counts, int nbuff, ccn_scatter_plan** out) {
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  std::vector<ScatBuf> bufs((size_t)nbuff + 1);
  std::vector<uint32_t> coarse;
  size_t total = 0, ntiles = 0;
  for (int b = 0; b < nbuff; b++) {
    if (counts[b] == 0) return CCN_EINVAL;
    const size_t nt = (counts[b] + kScatTile - 1) / kScatTile;
    if (ntiles + nt >= 0xffffffffull) return CCN_ERANGE;          // tile numbers are 32-bit
    bufs[b] = ScatBuf{(uint64_t)total, (uint32_t)ntiles, 0u};
    // every group of tiles whose first tile falls into this buffer
    for (size_t grp = (ntiles + (1u << kScatCoarseShift) - 1) >> kScatCoarseShift; (grp << kScatCoarseShift) < ntiles + nt; grp++)
      coarse.push_back((uint32_t)b);
    total += counts[b];
    ntiles += nt;
  }
  bufs[nbuff] = ScatBuf{(uint64_t)total, (uint32_t)ntiles, 0u};
  ccn_scatter_plan* p = new (std::nothrow) ccn_scatter_plan();
  if (!p) return CCN_ENOMEM;
  p->device = di->device;
  p->nbuff = (uint32_t)nbuff;
  p->total = total;
  p->ntiles = ntiles;
  const size_t words = (size_t)(CCN_MAX_RANKS + 1) * (size_t)nbuff;
  hipError_t e = hipMalloc((void**)&p->coarse, coarse.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = hipMalloc((void**)&p->bufs, bufs.size() * sizeof(ScatBuf));
  if (e == hipSuccess) e = hipMalloc((void**)&p->table_dev, words * sizeof(void*));
  if (e == hipSuccess) e = hipHostMalloc((void**)&p->table_pinned, words * sizeof(void*), hipHostMallocDefault);
  if (e == hipSuccess) e = hipMemcpy(p->coarse, coarse.data(), coarse.size() * sizeof(uint32_t), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(p->bufs, bufs.data(), bufs.size() * sizeof(ScatBuf), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    ccn_scatter_plan_destroy(p);
    return hip_fail(e);
  }
  *out = p;
  return CCN_OK;
}

int ccn_scatter_plan_create(const size_t* counts, int nbuff, ccn_scatter_plan** out) {
  if (!out) return CCN_EINVAL;
  *out = nullptr;
  if (!counts || nbuff < 1) return CCN_EINVAL;
  return guarded([&] { return scatter_plan_create(counts, nbuff, out); });
}

int ccn_sgd_f32_scattered(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, float lr, void* stream) {
  return guarded([&] { return launch_scattered<SgdMath>(plan, g, P, w, nullptr, SgdMath::Prm{lr}, stream); });
}

int ccn_adam_f32_scattered(ccn_scatter_plan* plan, const float* const* g, int P, float* const* w, float* m, float* v,
                           float lr, float beta1, float beta2, float eps, int step, void* stream) {
  if (step < 1) return CCN_EINVAL;
  float* mom[2] = {m, v};
  const AdamPrm prm = make_adam_prm(lr, beta1, beta2, eps, step, 1.0f);
  return guarded([&] { return launch_scattered<AdamMath>(plan, g, P, w, mom, prm, stream); });
}

}  // extern "C"
