// LAMB with per-segment trust ratio: two streaming passes and a tiny finalize kernel, no atomics.
//
// A plan cuts [0,N) into tiles of at most kLambTile elements that never straddle a segment boundary.
//   pass 1   one workgroup per tile, one 4-element pack per thread: P-way gradient reduce, m/v update, r, and the
//            tile's sums of w^2 and r^2 in float64 (lane values -> wavefront shuffle reduction -> LDS -> one pair
//            per tile)
//   finalize one workgroup per segment: fixed-order sum of the segment's tile pairs, norms, scale
//   pass 2   one workgroup per tile: r recomputed from the stored m, v and the old w; w updated
// Both passes use the launch shape of the other fused kernels (one pack per thread, capped residency).
// Arithmetic follows nccl-overlap/samples/multi-process-adam-scattered.cpp:402-449 statement by statement.
#include "ccn_common.hpp"

#include <cmath>
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
  uint32_t pad[3];
};
static_assert(sizeof(LambTile) == 32, "tile record is 32 bytes");

// Segments of one common length that is a multiple of the tile need no table: tile -> segment by division.
struct LambLayout {
  const LambTile* tiles;    // used when seg_len == 0
  uint64_t seg_len;         // common segment length, or 0 for a ragged layout
  float seg_len_f;
};

__device__ __forceinline__ LambTile lamb_tile_of(const LambLayout& L, unsigned b) {
  if (L.seg_len != 0) {
    LambTile t;
    t.start = (uint64_t)b * kLambTile;
    t.count = kLambTile;
    t.seg = (uint32_t)(t.start / L.seg_len);
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
template <int P, int VEC>
__device__ __forceinline__ void lamb_pass1_pack(const SrcTable<float, (P ? P : CCN_MAX_RANKS)>& g, int nP, const float* w,
                                                float* m, float* v, size_t e0, float nf, const LambPrm& k, double& accW,
                                                double& accR) {
  const int np = P ? P : nP;
  constexpr int PX = P > 0 ? P : 1;
  Pack<float, VEC> gv[PX];
  if constexpr (P > 0) {
#pragma unroll
    for (int p = 0; p < P; p++) gv[p] = load_stream<float, VEC>(g.p[p] + e0);
  }
  const Pack<float, VEC> wv = load_stream<float, VEC>(w + e0);   // w is read again by pass 2, 12 GB later
  Pack<float, VEC> mv = load_stream<float, VEC>(m + e0);
  Pack<float, VEC> vv = load_stream<float, VEC>(v + e0);
  Pack<float, VEC> gs;
  if constexpr (P > 0) {
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float a = gv[0].d[e];
#pragma unroll
      for (int p = 1; p < P; p++) a = a + gv[p].d[e];
      gs.d[e] = a;
    }
  } else {
    gs = load_stream<float, VEC>(g.p[0] + e0);
    for (int p = 1; p < np; p++) {
      const Pack<float, VEC> x = load_stream<float, VEC>(g.p[p] + e0);
#pragma unroll
      for (int e = 0; e < VEC; e++) gs.d[e] = gs.d[e] + x.d[e];
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    const float ge = gs.d[e];
    const float we = wv.d[e];
    float mi, vi;
    if (k.mode == CCN_LAMB_NCCL_GLOBAL) {
      vi = ((vv.d[e] * k.b2) + ((ge * ge) * k.omb2));
      mi = ((mv.d[e] * k.b1) + (ge * k.omb1));
    } else {
      mi = k.b1 * mv.d[e] + k.omb1 * ge;
      vi = k.b2 * vv.d[e] + k.omb2 * ge * ge;
    }
    const float r = lamb_r(mi, vi, we, k);
    accR += k.mode == CCN_LAMB_NCCL_GLOBAL ? (double)(r * r) : (double)((r * r) / nf);
    accW += (double)(we * we);
    mv.d[e] = mi;
    vv.d[e] = vi;
  }
  store_stream<float, VEC>(m + e0, mv);
  store_stream<float, VEC>(v + e0, vv);
}

template <int P>
__global__ __launch_bounds__(kBlock) void lamb_pass1_kernel(const SrcTable<float, (P ? P : CCN_MAX_RANKS)> g, const int nP,
                                                            const float* w, float* m, float* v, const LambLayout lay,
                                                            double* __restrict__ partials, const int vec_ok,
                                                            const LambPrm k) {
  __shared__ double lds[2 * kBlock / kWave];
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  double accW = 0.0, accR = 0.0;
  const uint32_t j0 = threadIdx.x * 4;          // this thread's elements of the tile: [j0, j0+4) clipped to count
  if (j0 < t.count) {
    if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
      lamb_pass1_pack<P, 4>(g, nP, w, m, v, t.start + j0, t.nf, k, accW, accR);
    } else {
      const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
      for (uint32_t j = j0; j < j1; j++) lamb_pass1_pack<P, 1>(g, nP, w, m, v, t.start + j, t.nf, k, accW, accR);
    }
  }
  const double sW = block_sum(accW, lds);
  const double sR = block_sum(accR, lds + kBlock / kWave);
  if (threadIdx.x == 0) {
    partials[2 * (size_t)blockIdx.x] = sW;
    partials[2 * (size_t)blockIdx.x + 1] = sR;
  }
}

// One workgroup per segment.  Thread t adds tiles t, t+256, ... in ascending order, then the fixed
// shuffle/LDS tree: the result does not depend on scheduling.
__global__ __launch_bounds__(kBlock) void lamb_finalize_kernel(const double* __restrict__ partials,
                                                               const uint32_t* __restrict__ seg_tile_begin,
                                                               const uint64_t* __restrict__ seg_len,
                                                               double* __restrict__ norms, float* __restrict__ scale,
                                                               const int mode) {
  __shared__ double lds[2 * kBlock / kWave];
  const int b = blockIdx.x;
  const uint32_t lo = seg_tile_begin[b], hi = seg_tile_begin[b + 1];
  double aW = 0.0, aR = 0.0;
  for (uint32_t t = lo + threadIdx.x; t < hi; t += kBlock) {
    aW += partials[2 * (size_t)t];
    aR += partials[2 * (size_t)t + 1];
  }
  const double sW = block_sum(aW, lds);
  const double sR = block_sum(aR, lds + kBlock / kWave);
  if (threadIdx.x == 0 && mode == CCN_LAMB_NCCL_GLOBAL) {
    const float wNorm = sqrtf((float)sW), rNorm = sqrtf((float)sR);
    norms[2 * b] = wNorm;
    norms[2 * b + 1] = rNorm;
    scale[b] = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f) / rNorm;
  } else if (threadIdx.x == 0) {
    const double rNorm = sqrt(sR);
    const double wNorm = sqrt(sW / (double)seg_len[b]);
    const double ratio = ((wNorm > 0) ? (rNorm > 0 ? wNorm / rNorm : 1.0f) : 1.0f);
    norms[2 * b] = wNorm;
    norms[2 * b + 1] = rNorm;
    scale[b] = (float)(mode == CCN_LAMB_REFERENCE ? ratio / rNorm : ratio);
  }
}

template <int VEC>
__device__ __forceinline__ void lamb_pass2_pack(float* w, const float* m, const float* v, size_t e0, float step_scale,
                                                const LambPrm& k) {
  Pack<float, VEC> wv = load_stream<float, VEC>(w + e0);
  const Pack<float, VEC> mv = load_stream<float, VEC>(m + e0);
  const Pack<float, VEC> vv = load_stream<float, VEC>(v + e0);
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    const float we = wv.d[e];
    const float r = lamb_r(mv.d[e], vv.d[e], we, k);
    const float x = step_scale * r;
    wv.d[e] = we - x;
  }
  store_stream<float, VEC>(w + e0, wv);
}

__global__ __launch_bounds__(kBlock) void lamb_pass2_kernel(float* w, const float* m, const float* v, const LambLayout lay,
                                                            const float* __restrict__ scale, const int vec_ok,
                                                            const LambPrm k) {
  const LambTile t = lamb_tile_of(lay, blockIdx.x);
  const float step_scale = k.lr * scale[t.seg];   // stepsize * scale, then times r
  const uint32_t j0 = threadIdx.x * 4;
  if (j0 >= t.count) return;
  if (vec_ok && (t.start & 3u) == 0 && j0 + 4 <= t.count) {
    lamb_pass2_pack<4>(w, m, v, t.start + j0, step_scale, k);
  } else {
    const uint32_t j1 = j0 + 4 < t.count ? j0 + 4 : t.count;
    for (uint32_t j = j0; j < j1; j++) lamb_pass2_pack<1>(w, m, v, t.start + j, step_scale, k);
  }
}

}  // namespace ccn

using namespace ccn;

struct ccn_lamb_plan {
  int device = -1;
  int nseg = 0;
  size_t N = 0;
  size_t ntiles = 0;
  uint64_t uniform_seg_len = 0;   // non-zero: all segments have this length and it is a multiple of the tile
  LambTile* tiles = nullptr;
  uint32_t* seg_tile_begin = nullptr;
  uint64_t* seg_len = nullptr;
  double* partials = nullptr;
  double* norms = nullptr;
  float* scale = nullptr;
};

extern "C" {

int ccn_lamb_plan_destroy(ccn_lamb_plan* plan) {
  if (!plan) return CCN_OK;
  int rc = CCN_OK;
  void* bufs[] = {plan->tiles, plan->seg_tile_begin, plan->seg_len, plan->partials, plan->norms, plan->scale};
  for (void* b : bufs) {
    if (b && hipFree(b) != hipSuccess) rc = CCN_EHIP;
  }
  delete plan;
  return rc;
}

int ccn_lamb_plan_create(const size_t* seg_offsets, int nseg, ccn_lamb_plan** out) {
  if (!out) return CCN_EINVAL;
  *out = nullptr;
  if (!seg_offsets || nseg < 1 || seg_offsets[0] != 0) return CCN_EINVAL;
  for (int b = 0; b < nseg; b++) {
    if (seg_offsets[b + 1] <= seg_offsets[b]) return CCN_EINVAL;   // empty or descending segment
  }
  const DeviceInfo* di = nullptr;
  int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;

  std::vector<LambTile> tiles;
  std::vector<uint32_t> begin((size_t)nseg + 1);
  std::vector<uint64_t> len((size_t)nseg);
  for (int b = 0; b < nseg; b++) {
    begin[b] = (uint32_t)tiles.size();
    const uint64_t n = seg_offsets[b + 1] - seg_offsets[b];
    len[b] = n;
    for (uint64_t off = 0; off < n; off += kLambTile) {
      LambTile t{};
      t.start = seg_offsets[b] + off;
      t.count = (uint32_t)((n - off) < (uint64_t)kLambTile ? (n - off) : (uint64_t)kLambTile);
      t.seg = (uint32_t)b;
      t.nf = (float)n;
      tiles.push_back(t);
    }
    if (tiles.size() > 0x7fffffffu) return CCN_ERANGE;
  }
  begin[nseg] = (uint32_t)tiles.size();
  uint64_t uniform = len[0];
  for (int b = 1; b < nseg; b++) if (len[b] != uniform) uniform = 0;
  if (uniform % kLambTile) uniform = 0;

  ccn_lamb_plan* p = new (std::nothrow) ccn_lamb_plan();
  if (!p) return CCN_ENOMEM;
  p->device = di->device;
  p->nseg = nseg;
  p->N = seg_offsets[nseg];
  p->ntiles = tiles.size();
  p->uniform_seg_len = uniform;
  hipError_t e = hipSuccess;
  auto alloc = [&](void** ptr, size_t bytes) { if (e == hipSuccess) e = hipMalloc(ptr, bytes); };
  alloc((void**)&p->tiles, tiles.size() * sizeof(LambTile));
  alloc((void**)&p->seg_tile_begin, begin.size() * sizeof(uint32_t));
  alloc((void**)&p->seg_len, len.size() * sizeof(uint64_t));
  alloc((void**)&p->partials, 2 * tiles.size() * sizeof(double));
  alloc((void**)&p->norms, 2 * (size_t)nseg * sizeof(double));
  alloc((void**)&p->scale, (size_t)nseg * sizeof(float));
  if (e == hipSuccess) e = hipMemcpy(p->tiles, tiles.data(), tiles.size() * sizeof(LambTile), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(p->seg_tile_begin, begin.data(), begin.size() * sizeof(uint32_t), hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(p->seg_len, len.data(), len.size() * sizeof(uint64_t), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    ccn_lamb_plan_destroy(p);
    return hip_fail(e);
  }
  *out = p;
  return CCN_OK;
}

int ccn_lamb_f32(ccn_lamb_plan* plan, const float* const* g, int P, float* w, float* m, float* v, float lr, float beta1,
                 float beta2, float eps, float wd, int step, int mode, void* stream) {
  if (!plan || !g || !w || !m || !v || P < 1 || P > CCN_MAX_RANKS || step < 1) return CCN_EINVAL;
  if (mode != CCN_LAMB_TRUST_RATIO && mode != CCN_LAMB_REFERENCE && mode != CCN_LAMB_NCCL_GLOBAL) return CCN_EINVAL;
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
  k.eps = eps;
  k.wd = wd;
  k.lr = lr;
  k.mode = mode;
  k.bc1 = 1 - std::pow((double)beta1, (double)step);
  k.bc2 = 1 - std::pow((double)beta2, (double)step);

  bool al = aligned16(w) && aligned16(m) && aligned16(v);
  for (int p = 0; p < P; p++) al = al && aligned16(g[p]);
  const int vec_ok = al ? 1 : 0;
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)plan->ntiles), block(kBlock);
  LambLayout lay;
  lay.tiles = plan->tiles;
  lay.seg_len = vec_ok ? plan->uniform_seg_len : 0;
  lay.seg_len_f = (float)plan->uniform_seg_len;
  // Residency caps measured for config 4 (N = 2^28, P = 8): pass 1 is fastest at 4 workgroups per CU (its float64
  // sums and the workgroup reduction need more wavefronts to hide than the plain Adam kernel), pass 2 uncapped.
  const unsigned lds1 = stream_launch(1, 1, P >= 2 ? 4 : 0).lds_bytes;
  const unsigned lds2 = 0;
  auto pass1 = [&](auto ptag) {
    constexpr int PP = decltype(ptag)::value;
    SrcTable<float, (PP ? PP : CCN_MAX_RANKS)> tbl;
    for (int p = 0; p < (PP ? PP : CCN_MAX_RANKS); p++) tbl.p[p] = g[p < P ? p : 0];
    hipLaunchKernelGGL((lamb_pass1_kernel<PP>), grid, block, lds1, s, tbl, P, (const float*)w, m, v, lay, plan->partials,
                       vec_ok, k);
  };
  switch (P) {
#define CCN_CASE(K) case K: pass1(std::integral_constant<int, K>{}); break;
    CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
    default: pass1(std::integral_constant<int, 0>{}); break;
  }
  CCN_HIP(hipGetLastError());
  hipLaunchKernelGGL(lamb_finalize_kernel, dim3((unsigned)plan->nseg), block, 0, s, (const double*)plan->partials,
                     (const uint32_t*)plan->seg_tile_begin, (const uint64_t*)plan->seg_len, plan->norms, plan->scale, mode);
  CCN_HIP(hipGetLastError());
  hipLaunchKernelGGL(lamb_pass2_kernel, grid, block, lds2, s, w, (const float*)m, (const float*)v, lay,
                     (const float*)plan->scale, vec_ok, k);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

int ccn_lamb_plan_norms(ccn_lamb_plan* plan, double* norms_host, void* stream) {
  if (!plan || !norms_host) return CCN_EINVAL;
  hipStream_t s = as_stream(stream);
  CCN_HIP(hipMemcpyAsync(norms_host, plan->norms, 2 * (size_t)plan->nseg * sizeof(double), hipMemcpyDeviceToHost, s));
  CCN_HIP(hipStreamSynchronize(s));
  return CCN_OK;
}

}  // extern "C"
