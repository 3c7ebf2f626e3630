// Model-parallel MLP out-projection for gfx950: bf16 MFMA GEMM with the all-reduce partial sum, bias,
// dropout and residual fused into the tile write-back, plus the same epilogue as a standalone kernel.
//
// GEMM tiling: a 256-thread workgroup owns a 128(m) x 128(n) tile of C and walks K in steps of 64.
// The four wavefronts form a 2x2 grid; each owns 64x64 as 2x2 v_mfma_f32_32x32x16_bf16 blocks.
// The MFMA computes C^T blocks (rows = n from W, columns = m from X) so that every lane ends up with
// four CONSECUTIVE n of one row m in its accumulator quads: the epilogue then moves 16-byte pieces of
// the fp32 partial buffers and 8-byte pieces of the bf16 residual/output.
// W is [K x N] row-major (n contiguous) while the MFMA wants k contiguous per lane, so the W tile is
// transposed in registers on its way into LDS.  LDS rows are 128 bytes (64 k) with the eight 16-byte
// chunks XOR-swizzled by (row%8)^((row/8)%8): conflict-free for the 8-byte transposed writes and the
// 16-byte fragment reads.
#include "ccn_common.hpp"

#include <type_traits>

namespace ccn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 64;

struct EpiPrm {
  float p_drop, keep_scale;
  uint32_t seed_lo, seed_hi;
  int apply_dropout;
  int mode;   // CCN_DROPOUT_*
};

// The 16-bit operands, residual and output are bfloat16 (F16 = false) or IEEE half (F16 = true: the type the reference's
// model-parallel example declares); accumulation is fp32 either way.
template <bool F16> __device__ __forceinline__ float half_in(uint16_t h) { return F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h); }
template <bool F16> __device__ __forceinline__ uint16_t half_out(float f) { return F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f); }

// Epilogue for four consecutive columns n..n+3 (n % 4 == 0) of row m, in two steps so that the loads of one quad can be
// in flight while the previous one is finished.  NP, the number of partial buffers (0..8), is a compile-time constant:
// all of a quad's loads are issued together (a run-time loop over the buffers measured 20 % slower at 6 partials).
template <int NP> struct EpiIn {
  f32x4 pv[NP > 0 ? NP : 1];
  u32x2 rv;
};
template <int NP>
__device__ __forceinline__ void epilogue_load(EpiIn<NP>& in, const SrcTable<float, 8>& parts,
                                              const uint16_t* __restrict__ resid, size_t idx) {
#pragma unroll
  for (int q = 0; q < NP; q++) in.pv[q] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(parts.p[q] + idx));
  in.rv = u32x2{0u, 0u};
  if (resid) in.rv = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(resid + idx));
}
// [0, 1] clamp of the reference's __hadd2_sat (NaN gives 0)
__device__ __forceinline__ float sat01(float x) { return x > 0.0f ? (x < 1.0f ? x : 1.0f) : 0.0f; }

// idx: where the quad lies in memory; mask_idx: its element index in the whole [M x N] output, which the mask is drawn
// from (the two differ when a call covers a band of rows of a larger output).
// REF: one of the reference's dropout forms (k.mode says which); false: standard dropout, the form the kernels are
// tuned for, compiled without the others.
template <int NP, bool REF, bool F16 = false>
__device__ __forceinline__ void epilogue_finish(f32x4 acc, const EpiIn<NP>& in, const float* __restrict__ bias,
                                                uint16_t* __restrict__ out, size_t idx, size_t n, const EpiPrm& k,
                                                size_t mask_idx) {
  const f32x4 bv = *reinterpret_cast<const f32x4*>(bias + n);
  f32x4 s = acc;
#pragma unroll
  for (int q = 0; q < NP; q++) s = s + in.pv[q];
  const float r0 = half_in<F16>((uint16_t)(in.rv[0] & 0xffffu)), r1 = half_in<F16>((uint16_t)(in.rv[0] >> 16));
  const float r2 = half_in<F16>((uint16_t)(in.rv[1] & 0xffffu)), r3 = half_in<F16>((uint16_t)(in.rv[1] >> 16));
  float y0, y1, y2, y3;
  if constexpr (!REF) {
    // drop with probability p, survivors scaled by 1/(1-p)
    const f32x4 t = s + bv;
    f32x4 d = t;
    if (k.apply_dropout) {
      const uint64_t blk = (uint64_t)mask_idx >> 2;
      const Philox4 r = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), 0u, 0u, k.seed_lo, k.seed_hi);
      d[0] = keep_from_word(r.x, k.p_drop) ? t[0] * k.keep_scale : 0.0f;
      d[1] = keep_from_word(r.y, k.p_drop) ? t[1] * k.keep_scale : 0.0f;
      d[2] = keep_from_word(r.z, k.p_drop) ? t[2] * k.keep_scale : 0.0f;
      d[3] = keep_from_word(r.w, k.p_drop) ? t[3] * k.keep_scale : 0.0f;
    }
    y0 = d[0] + r0; y1 = d[1] + r1; y2 = d[2] + r2; y3 = d[3] + r3;
  } else {
    const uint64_t blk = (uint64_t)mask_idx >> 2;
    const Philox4 r = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), 0u, 0u, k.seed_lo, k.seed_hi);
    // kept where u < p: the complement of keep_from_word's u >= p
    const bool kp[4] = {!keep_from_word(r.x, k.p_drop), !keep_from_word(r.y, k.p_drop), !keep_from_word(r.z, k.p_drop),
                        !keep_from_word(r.w, k.p_drop)};
    const float rs[4] = {r0, r1, r2, r3};
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (k.mode == CCN_DROPOUT_REF_DSL) {
        // the reference's emitted expression (src/codegen.cpp:634-640): (u < p ? (sum + bias) : 0) + residual
        const float t = s[e] + bv[e];
        y[e] = (kp[e] ? t : 0.0f) + rs[e];
      } else {
        // the reference's fused kernel (nccl-overlap/src/collectives/device/reduce_kernel.h:192-213):
        // ((u < p ? sum : 0) + bias) + residual; its half specialisation adds with saturation to [0, 1]
        const float d = kp[e] ? s[e] : 0.0f;
        y[e] = k.mode == CCN_DROPOUT_REF_NCCL_SAT ? sat01(sat01(d + bv[e]) + rs[e]) : (d + bv[e]) + rs[e];
      }
    }
    y0 = y[0]; y1 = y[1]; y2 = y[2]; y3 = y[3];
  }
  u32x2 o;
  o[0] = (uint32_t)half_out<F16>(y0) | ((uint32_t)half_out<F16>(y1) << 16);
  o[1] = (uint32_t)half_out<F16>(y2) | ((uint32_t)half_out<F16>(y3) << 16);
  __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(out + idx));
}

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 7); }

// PLAIN: the product alone, written as fp32 [M x N] through `out` (no partial buffers, bias, dropout or residual).
// REF: the epilogue applies one of the reference's dropout forms.
template <int NP, bool PLAIN = false, bool REF = false, bool F16 = false>
__global__ __launch_bounds__(kBlock) void mlp_outproj_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W,
                                                             const SrcTable<float, 8> parts,
                                                             const float* __restrict__ bias,
                                                             const uint16_t* __restrict__ resid, uint16_t* __restrict__ out,
                                                             const int N, const int K, const EpiPrm ep) {
  // main loop: X tile [m][k] and transposed W tile [n][k], 16 KiB each, chunk-swizzled.
  // epilogue: half of the fp32 C tile, 64 rows x (128 + 4 pad) floats, to turn the MFMA register layout
  // into whole 512-byte row segments per wavefront.
  constexpr int kCStride = BN + 4;
  constexpr int kLdsBytes = (BM / 2) * kCStride * 4 > 2 * BM * BK * 2 ? (BM / 2) * kCStride * 4 : 2 * BM * BK * 2;
  __shared__ __attribute__((aligned(16))) uint8_t lds_all[kLdsBytes];
  uint8_t* const lds_x = lds_all;
  uint8_t* const lds_w = lds_all + BM * BK * 2;
  float* const lds_c = reinterpret_cast<float*>(lds_all);

  // ---- workgroup -> tile: along a tile row first.  Workgroups that run at the same time then cover whole rows of
  //      the partial buffers between them (measured: the epilogue streams reach 75-79 % of HBM peak this way, 62-66 %
  //      when neighbours in time are neighbours in a tile column), and since workgroups are dealt round-robin to the
  //      8 XCDs, an XCD only ever touches the W panels of every 8th tile column: with N/BN a multiple of 8 they stay
  //      in its L2 (8 panels of 2*K*BN bytes), while an X panel is shared by the XCD's 8 tiles of a row.
  const int tilesN = N / BN;
  const int tm = blockIdx.x / tilesN, tn = blockIdx.x % tilesN;
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging assignments
  const int xr = t >> 3, xc = t & 7;          // X: rows xr + 32*j, 16-byte chunk xc
  const int wg = t & 15, wq = t >> 4;         // W: k rows wq*4 + j, columns wg*8..+7
  u32x4 xreg[4], wreg[4];

  auto load_tile = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      xreg[j] = *reinterpret_cast<const u32x4*>(X + (m0 + xr + 32 * j) * (size_t)K + k0 + xc * 8);
      wreg[j] = *reinterpret_cast<const u32x4*>(W + (size_t)(k0 + wq * 4 + j) * N + n0 + wg * 8);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int row = xr + 32 * j;
      *reinterpret_cast<u32x4*>(lds_x + row * 128 + ((xc ^ swz(row)) << 4)) = xreg[j];
    }
    // transpose 4(k) x 8(n) -> 8 rows of 4 k
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const uint32_t a0 = wreg[0][q], a1 = wreg[1][q], a2 = wreg[2][q], a3 = wreg[3][q];
      u32x2 lo, hi;   // lo: column 2q, hi: column 2q+1; each k0..k3
      lo[0] = (a0 & 0xffffu) | (a1 << 16);
      lo[1] = (a2 & 0xffffu) | (a3 << 16);
      hi[0] = (a0 >> 16) | (a1 & 0xffff0000u);
      hi[1] = (a2 >> 16) | (a3 & 0xffff0000u);
      const int r0 = wg * 8 + 2 * q, r1 = r0 + 1;
      *reinterpret_cast<u32x2*>(lds_w + r0 * 128 + (((wq >> 1) ^ swz(r0)) << 4) + ((wq & 1) << 3)) = lo;
      *reinterpret_cast<u32x2*>(lds_w + r1 * 128 + (((wq >> 1) ^ swz(r1)) << 4) + ((wq & 1) << 3)) = hi;
    }
  };

  f32x16 acc[2][2];   // [bn][bm]
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

  const int nk = K / BK;
  load_tile(0);
  store_tile();
  __syncthreads();
  for (int kt = 0; kt < nk; kt++) {
    if (kt + 1 < nk) load_tile((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      const int c = ks * 2 + (lane >> 5);
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int bn = 0; bn < 2; bn++) {
        const int row = wn * 64 + bn * 32 + (lane & 31);
        fa[bn] = *reinterpret_cast<const bf16x8*>(lds_w + row * 128 + ((c ^ swz(row)) << 4));
      }
#pragma unroll
      for (int bm = 0; bm < 2; bm++) {
        const int row = wm * 64 + bm * 32 + (lane & 31);
        fb[bm] = *reinterpret_cast<const bf16x8*>(lds_x + row * 128 + ((c ^ swz(row)) << 4));
      }
#pragma unroll
      for (int bn = 0; bn < 2; bn++)
#pragma unroll
        for (int bm = 0; bm < 2; bm++)
          if constexpr (F16)
            acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[bn]), __builtin_bit_cast(f16x8, fb[bm]),
                                                                 acc[bn][bm], 0, 0, 0);
          else
            acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[bn], fb[bm], acc[bn][bm], 0, 0, 0);
    }
    __syncthreads();
    if (kt + 1 < nk) {
      store_tile();
      __syncthreads();
    }
  }

  // ---- epilogue.  Accumulator register 4*i4+e of block (bn,bm) is C[m][n+e] with
  //      n = wn*64 + bn*32 + i4*8 + (lane/32)*4,  m = wm*64 + bm*32 + lane%32  (tile-local).
  //      Read straight from HBM in that layout, a wavefront instruction would touch 32 rows x 32 bytes of every
  //      partial buffer; going through LDS makes it 2 rows x 512 contiguous bytes.
  for (int half = 0; half < 2; half++) {
    __syncthreads();   // main-loop tiles (half 0) or the previous half's C rows are no longer needed
    if (wm == half) {
#pragma unroll
      for (int bm = 0; bm < 2; bm++) {
        const int row = bm * 32 + (lane & 31);
#pragma unroll
        for (int bn = 0; bn < 2; bn++) {
#pragma unroll
          for (int i4 = 0; i4 < 4; i4++) {
            const int col = wn * 64 + bn * 32 + i4 * 8 + (lane >> 5) * 4;
            f32x4 a;
            a[0] = acc[bn][bm][i4 * 4 + 0];
            a[1] = acc[bn][bm][i4 * 4 + 1];
            a[2] = acc[bn][bm][i4 * 4 + 2];
            a[3] = acc[bn][bm][i4 * 4 + 3];
            *reinterpret_cast<f32x4*>(lds_c + row * kCStride + col) = a;
          }
        }
      }
    }
    __syncthreads();
    constexpr int kIters = (BM / 2) * (BN / 4) / kBlock;
    // the loads of quad it+1 are issued before quad it is finished
    auto index_of = [&](int it) {
      const int q = it * kBlock + t;
      return (m0 + half * 64 + q / (BN / 4)) * (size_t)N + n0 + (q % (BN / 4)) * 4;
    };
    if constexpr (PLAIN) {
      float* const outc = reinterpret_cast<float*>(out);
#pragma unroll
      for (int it = 0; it < kIters; it++) {
        const int q = it * kBlock + t;
        const int row = q / (BN / 4), colq = q % (BN / 4);
        *reinterpret_cast<f32x4*>(outc + index_of(it)) = *reinterpret_cast<const f32x4*>(lds_c + row * kCStride + colq * 4);
      }
    } else {
      EpiIn<NP> cur;
      epilogue_load<NP>(cur, parts, resid, index_of(0));
#pragma unroll
      for (int it = 0; it < kIters; it++) {
        EpiIn<NP> nxt;
        if (it + 1 < kIters) epilogue_load<NP>(nxt, parts, resid, index_of(it + 1));
        const int q = it * kBlock + t;
        const int row = q / (BN / 4), colq = q % (BN / 4);
        const f32x4 a = *reinterpret_cast<const f32x4*>(lds_c + row * kCStride + colq * 4);
        epilogue_finish<NP, REF, F16>(a, cur, bias, out, index_of(it), n0 + colq * 4, ep, index_of(it));
        if (it + 1 < kIters) cur = nxt;
      }
    }
  }
}

// Standalone epilogue over an fp32 product in memory: one quad per thread, no loop, the launch shape of the other
// streaming kernels (the y dimension of the grid only comes into play beyond 2^30 workgroups).
template <int NP, int BS, bool REF, bool F16 = false>
__global__ __launch_bounds__(BS) void bias_dropout_residual_kernel(const float* __restrict__ acc, const SrcTable<float, 8> parts,
                                                                   const float* __restrict__ bias,
                                                                   const uint16_t* __restrict__ resid,
                                                                   uint16_t* __restrict__ out, const size_t total,
                                                                   const size_t N, const size_t mask_base, const EpiPrm ep) {
  const size_t q = ((size_t)blockIdx.x + (size_t)blockIdx.y * gridDim.x) * BS + threadIdx.x;
  if (q >= total) return;
  const size_t idx = q * 4;              // rows are contiguous: element index of the quad
  EpiIn<NP> in;
  const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(acc + idx));
  epilogue_load<NP>(in, parts, resid, idx);
  epilogue_finish<NP, REF, F16>(a, in, bias, out, idx, idx % N, ep, mask_base + idx);
}

// Shapes that are not whole 128 x 128 x 64 tiles (any M and K; N a multiple of 4, which keeps a quad of columns inside a
// row and the rows of the fp32 operands 16-byte aligned): 64 x 64 output tiles, 32-deep steps staged through LDS as fp32
// with the out-of-range part filled with zeros, 4 x 4 outputs per thread accumulated in fp32 in ascending k on the
// vector ALUs.  Slower than the matrix-core kernel by an order of magnitude, and meant for the odd shape only; the
// epilogue is the same code.  nP is a run-time count here: the partial sums are added to the product in buffer order
// before the shared epilogue sees it, which is the order the fixed-count epilogue uses.
constexpr int GT = 64, GK = 32;
template <bool PLAIN, bool REF, bool F16 = false>
__global__ __launch_bounds__(kBlock) void outproj_any_shape_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W,
                                                                   const SrcTable<float, 8> parts, const int nP,
                                                                   const float* __restrict__ bias,
                                                                   const uint16_t* __restrict__ resid, uint16_t* __restrict__ out,
                                                                   const int M, const int N, const int K, const EpiPrm ep) {
  __shared__ float xs[GT][GK + 1];
  __shared__ __align__(16) float ws[GK][GT];
  const int tiles_n = (N + GT - 1) / GT;
  const int m0 = (int)(blockIdx.x / tiles_n) * GT, n0 = (int)(blockIdx.x % tiles_n) * GT;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += GK) {
    // X tile: 64 rows x 32 k, 8 elements per thread (rows need not be aligned: K is arbitrary)
#pragma unroll
    for (int i = 0; i < (GT * GK) / kBlock; i++) {
      const int e = i * kBlock + threadIdx.x, r = e / GK, c = e % GK;
      const int m = m0 + r, k = k0 + c;
      xs[r][c] = (m < M && k < K) ? half_in<F16>(X[(size_t)m * K + k]) : 0.0f;
    }
    // W tile: 32 k x 64 n in quads of columns (N % 4 == 0: a quad is inside the row or outside it, and 8-byte aligned)
#pragma unroll
    for (int i = 0; i < (GK * GT / 4) / kBlock; i++) {
      const int e = i * kBlock + threadIdx.x, r = e / (GT / 4), c = (e % (GT / 4)) * 4;
      const int k = k0 + r, n = n0 + c;
      f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      if (k < K && n < N) {
        const u32x2 b = *reinterpret_cast<const u32x2*>(W + (size_t)k * N + n);
        v[0] = half_in<F16>((uint16_t)(b[0] & 0xffffu));
        v[1] = half_in<F16>((uint16_t)(b[0] >> 16));
        v[2] = half_in<F16>((uint16_t)(b[1] & 0xffffu));
        v[3] = half_in<F16>((uint16_t)(b[1] >> 16));
      }
      *reinterpret_cast<f32x4*>(&ws[r][c]) = v;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < GK; kk++) {
      const f32x4 b = *reinterpret_cast<const f32x4*>(&ws[kk][tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float a = xs[ty * 4 + i][kk];
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = acc[i][j] + a * b[j];
      }
    }
    __syncthreads();
  }
  const int n = n0 + tx * 4;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    const size_t idx = (size_t)m * N + n;
    f32x4 sum = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
    if constexpr (PLAIN) {
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(out) + idx) = sum;
    } else {
      for (int q = 0; q < nP; q++) sum = sum + __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(parts.p[q] + idx));
      EpiIn<0> in;
      epilogue_load<0>(in, parts, resid, idx);
      epilogue_finish<0, REF, F16>(sum, in, bias, out, idx, (size_t)n, ep, idx);
    }
  }
}

static inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

static int make_epi(float p_drop, uint64_t seed, int mode, EpiPrm* ep) {
  if (mode < CCN_DROPOUT_INVERTED || mode > CCN_DROPOUT_REF_NCCL_SAT) return CCN_EINVAL;
  // inverted dropout rescales by 1/(1-p): p < 1.  The reference's forms keep with probability p: p = 1 keeps everything.
  if (!(p_drop >= 0.0f) || !(mode == CCN_DROPOUT_INVERTED ? p_drop < 1.0f : p_drop <= 1.0f)) return CCN_EINVAL;
  ep->p_drop = p_drop;
  ep->keep_scale = mode == CCN_DROPOUT_INVERTED ? 1.0f / (1.0f - p_drop) : 1.0f;
  ep->seed_lo = (uint32_t)seed;
  ep->seed_hi = (uint32_t)(seed >> 32);
  // p = 0 drops nothing when dropping with probability p, and everything when keeping with probability p
  ep->apply_dropout = (mode != CCN_DROPOUT_INVERTED || p_drop > 0.0f) ? 1 : 0;
  ep->mode = mode;
  return CCN_OK;
}

}  // namespace ccn

using namespace ccn;

namespace {

template <bool F16>
int outproj_launch(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials, const float* bias,
                   const uint16_t* resid, uint16_t* out, int M, int N, int K, float p_drop, uint64_t seed, int mode,
                   void* stream) {
  if (!X || !W || !bias || !out || nPartials < 0 || nPartials > 8 || (nPartials > 0 && !partials)) return CCN_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0) return CCN_EINVAL;
  if (N % 4) return CCN_ERANGE;   // a quad of columns never straddles two rows
  SrcTable<float, 8> tbl;
  for (int q = 0; q < 8; q++) {
    tbl.p[q] = q < nPartials ? partials[q] : nullptr;
    if (q < nPartials && (!partials[q] || !aligned16(partials[q]))) return CCN_EINVAL;
  }
  if (!aligned16(X) || !aligned16(W) || !aligned16(bias) || !aligned16(out) || (resid && !aligned16(resid))) return CCN_EINVAL;
  EpiPrm ep;
  int rc = make_epi(p_drop, seed, mode, &ep);
  if (rc != CCN_OK) return rc;
  const DeviceInfo* di = nullptr;
  rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (M % BM || N % BN || K % BK) {   // not whole tiles of the matrix-core kernel
    const size_t tiles = (size_t)((M + GT - 1) / GT) * (size_t)((N + GT - 1) / GT);
    if (tiles > 0x7fffffffull) return CCN_ERANGE;
    if (mode == CCN_DROPOUT_INVERTED)
      hipLaunchKernelGGL((outproj_any_shape_kernel<false, false, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, s, X, W, tbl, nPartials,
                         bias, resid, out, M, N, K, ep);
    else
      hipLaunchKernelGGL((outproj_any_shape_kernel<false, true, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, s, X, W, tbl, nPartials,
                         bias, resid, out, M, N, K, ep);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }
  const dim3 grid((unsigned)((M / BM) * (N / BN))), block(kBlock);
  switch (nPartials) {
#define CCN_CASE(Q)                                                                                                          \
  case Q:                                                                                                                    \
    if (mode == CCN_DROPOUT_INVERTED) hipLaunchKernelGGL((mlp_outproj_kernel<Q, false, false, F16>), grid, block, 0, s, X, W, tbl, bias, resid, out, N, K, ep); \
    else hipLaunchKernelGGL((mlp_outproj_kernel<Q, false, true, F16>), grid, block, 0, s, X, W, tbl, bias, resid, out, N, K, ep); \
    break;
    CCN_CASE(0) CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
  }
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

template <bool F16>
int epilogue_launch(const float* acc, const float* const* partials, int nPartials, const float* bias, const uint16_t* resid,
                    uint16_t* out, int M, int N, float p_drop, uint64_t seed, int mode, size_t first_row, void* stream) {
  if (!acc || !bias || !out || nPartials < 0 || nPartials > 8 || (nPartials > 0 && !partials)) return CCN_EINVAL;
  if (M <= 0 || N <= 0) return CCN_EINVAL;
  if (N % 4) return CCN_ERANGE;
  SrcTable<float, 8> tbl;
  for (int q = 0; q < 8; q++) {
    tbl.p[q] = q < nPartials ? partials[q] : nullptr;
    if (q < nPartials && (!partials[q] || !aligned16(partials[q]))) return CCN_EINVAL;
  }
  // fp32 operands move 16 bytes at a time, the bf16 ones 8 (a band of rows of a larger output may start on any quad)
  if (!aligned16(acc) || !aligned16(bias) || !aligned8(out) || (resid && !aligned8(resid))) return CCN_EINVAL;
  EpiPrm ep;
  int rc = make_epi(p_drop, seed, mode, &ep);
  if (rc != CCN_OK) return rc;
  const DeviceInfo* di = nullptr;
  rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  const size_t total = (size_t)M * (size_t)(N / 4);
  StreamShape sh = stream_shape((1 + nPartials) * 16 + (resid ? 8 : 0), 8);
  // The Philox rounds keep a wavefront busy long after its loads have landed, so more wavefronts are needed to keep
  // loads in flight than the streaming kernels' table gives: 13 per CU measured best with dropout on (84 % of HBM
  // peak at 7 partials against 75 % with 8 per CU).
  if (ep.apply_dropout && sh.block == kWave) sh.lds_bytes = lds_for_residency(nPartials >= 6 ? 13 : 14);
  size_t wgs = (total + (size_t)sh.block - 1) / (size_t)sh.block;
  const size_t gx = wgs < 0x40000000ull ? wgs : 0x40000000ull;
  const dim3 grid((unsigned)gx, (unsigned)((wgs + gx - 1) / gx));
  hipStream_t s = as_stream(stream);
  const size_t mask_base = first_row * (size_t)N;
  auto go = [&](auto qtag) {
    constexpr int Q = decltype(qtag)::value;
    auto launch = [&](auto bstag, auto reftag) {
      constexpr int BS = decltype(bstag)::value;
      hipLaunchKernelGGL((bias_dropout_residual_kernel<Q, BS, decltype(reftag)::value, F16>), grid, dim3(BS), sh.lds_bytes, s, acc, tbl, bias,
                         resid, out, total, (size_t)N, mask_base, ep);
    };
    const bool ref = mode != CCN_DROPOUT_INVERTED;
    if (sh.block == kWave) {
      if (ref) launch(std::integral_constant<int, kWave>{}, std::true_type{});
      else launch(std::integral_constant<int, kWave>{}, std::false_type{});
    } else {
      if (ref) launch(std::integral_constant<int, kBlock>{}, std::true_type{});
      else launch(std::integral_constant<int, kBlock>{}, std::false_type{});
    }
  };
  switch (nPartials) {
#define CCN_CASE(Q) case Q: go(std::integral_constant<int, Q>{}); break;
    CCN_CASE(0) CCN_CASE(1) CCN_CASE(2) CCN_CASE(3) CCN_CASE(4) CCN_CASE(5) CCN_CASE(6) CCN_CASE(7) CCN_CASE(8)
#undef CCN_CASE
  }
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

template <bool F16>
int matmul_launch(const uint16_t* X, const uint16_t* W, float* C, int M, int N, int K, void* stream) {
  if (!X || !W || !C) return CCN_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0) return CCN_EINVAL;
  if (N % 4) return CCN_ERANGE;
  if (!aligned16(X) || !aligned16(W) || !aligned16(C)) return CCN_EINVAL;
  const DeviceInfo* di = nullptr;
  const int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  SrcTable<float, 8> tbl;
  for (int q = 0; q < 8; q++) tbl.p[q] = nullptr;
  EpiPrm ep{};
  if (M % BM || N % BN || K % BK) {
    const size_t tiles = (size_t)((M + GT - 1) / GT) * (size_t)((N + GT - 1) / GT);
    if (tiles > 0x7fffffffull) return CCN_ERANGE;
    hipLaunchKernelGGL((outproj_any_shape_kernel<true, false, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, as_stream(stream), X, W,
                       tbl, 0, (const float*)nullptr, (const uint16_t*)nullptr, reinterpret_cast<uint16_t*>(C), M, N, K, ep);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }
  const dim3 grid((unsigned)((M / BM) * (N / BN))), block(kBlock);
  hipLaunchKernelGGL((mlp_outproj_kernel<0, true, false, F16>), grid, block, 0, as_stream(stream), X, W, tbl, (const float*)nullptr,
                     (const uint16_t*)nullptr, reinterpret_cast<uint16_t*>(C), N, K, ep);
  CCN_HIP(hipGetLastError());
  return CCN_OK;
}

}  // namespace

extern "C" {

int ccn_mlp_outproj_bf16(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                         const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K, float p_drop,
                         uint64_t seed, void* stream) {
  return outproj_launch<false>(X, W, partials, nPartials, bias, resid, out, M, N, K, p_drop, seed, CCN_DROPOUT_INVERTED, stream);
}

int ccn_mlp_outproj_bf16_ex(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                            const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K, float p_drop,
                            uint64_t seed, int dropout_mode, void* stream) {
  return outproj_launch<false>(X, W, partials, nPartials, bias, resid, out, M, N, K, p_drop, seed, dropout_mode, stream);
}

int ccn_bias_dropout_residual(const float* acc, const float* const* partials, int nPartials, const float* bias,
                              const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                              void* stream) {
  return epilogue_launch<false>(acc, partials, nPartials, bias, resid, out, M, N, p_drop, seed, CCN_DROPOUT_INVERTED, 0, stream);
}

int ccn_bias_dropout_residual_ex(const float* acc, const float* const* partials, int nPartials, const float* bias,
                                 const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                                 int dropout_mode, size_t first_row, void* stream) {
  return epilogue_launch<false>(acc, partials, nPartials, bias, resid, out, M, N, p_drop, seed, dropout_mode, first_row, stream);
}

int ccn_matmul_bf16_f32(const uint16_t* X, const uint16_t* W, float* C, int M, int N, int K, void* stream) {
  return matmul_launch<false>(X, W, C, M, N, K, stream);
}

int ccn_mlp_outproj_f16_ex(const uint16_t* X, const uint16_t* W, const float* const* partials, int nPartials,
                           const float* bias, const uint16_t* resid, uint16_t* out, int M, int N, int K, float p_drop,
                           uint64_t seed, int dropout_mode, void* stream) {
  return outproj_launch<true>(X, W, partials, nPartials, bias, resid, out, M, N, K, p_drop, seed, dropout_mode, stream);
}

int ccn_bias_dropout_residual_f16_ex(const float* acc, const float* const* partials, int nPartials, const float* bias,
                                     const uint16_t* resid, uint16_t* out, int M, int N, float p_drop, uint64_t seed,
                                     int dropout_mode, size_t first_row, void* stream) {
  return epilogue_launch<true>(acc, partials, nPartials, bias, resid, out, M, N, p_drop, seed, dropout_mode, first_row, stream);
}

int ccn_matmul_f16_f32(const uint16_t* X, const uint16_t* W, float* C, int M, int N, int K, void* stream) {
  return matmul_launch<true>(X, W, C, M, N, K, stream);
}

}  // extern "C"
