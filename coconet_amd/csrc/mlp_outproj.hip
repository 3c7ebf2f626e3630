// Model-parallel MLP out-projection for gfx950: bf16 MFMA GEMM with the all-reduce partial sum, bias,
// dropout and residual fused into the tile write-back, plus the same epilogue as a standalone kernel.
//
// GEMM tiling: a 256-thread workgroup owns a 128(m) x 128(n) tile of C and walks K in steps of 64.
// Wavefront w owns the 32 tile rows 8j + 2w, 8j + 2w + 1 (j = 0..15) over all 128 columns, as four
// v_mfma_f32_32x32x16_bf16 blocks.  The MFMA computes C^T blocks (rows = n from W, columns = m from X)
// so that every lane ends up with four CONSECUTIVE n of one row m in its accumulator quads.
// X tile in LDS: rows of 128 bytes (64 k), the eight 16-byte chunks XOR-swizzled by (row%8)^((row/8)%8): conflict-free
// for the 16-byte fragment reads with the rows a wavefront owns (they differ in row/8).
// W is [K x N] row-major (n contiguous) while the MFMA wants k contiguous per lane.  The W tile goes into LDS as it
// lies in memory (64 rows of 256 bytes, the sixteen 16-byte chunks of row k XOR-swizzled by 4*(k%4)) and comes back
// transposed through gfx950's ds_read_b64_tr_b16: within 16 lanes, lane j receives element j%4 of the four 8-byte
// pieces addressed by lanes j/4, j/4+4, j/4+8, j/4+12, so a 4(k) x 16(n) block arrives as 4 consecutive k per lane;
// with the swizzle the 32 lanes of half a wavefront touch all 64 banks once.
#include "ccn_common.hpp"

#include <type_traits>

namespace ccn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 64;
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;

struct EpiPrm {
  float p_drop, keep_scale;
  uint32_t thr;   // keep_threshold(p_drop): an element survives standard dropout when (word >> 8) >= thr
  uint32_t seed_lo, seed_hi;
  int apply_dropout;
  int mode;   // CCN_DROPOUT_*
};

// The 16-bit operands, residual and output are bfloat16 (F16 = false) or IEEE half (F16 = true: the type the reference's
// model-parallel example declares); accumulation is fp32 either way.
template <bool F16> __device__ __forceinline__ float half_in(uint16_t h) { return F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h); }
template <bool F16> __device__ __forceinline__ uint16_t half_out(float f) { return F16 ? f32_to_f16_bits(f) : f32_to_bf16_bits(f); }
template <bool F16> __device__ __forceinline__ u32x2 pack_quad(f32x4 v) {
  return u32x2{(uint32_t)half_out<F16>(v[0]) | ((uint32_t)half_out<F16>(v[1]) << 16),
               (uint32_t)half_out<F16>(v[2]) | ((uint32_t)half_out<F16>(v[3]) << 16)};
}

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
__device__ __forceinline__ float f16_round(float x) { return f16_bits_to_f32(f32_to_f16_bits(x)); }

// Two 16-bit halves into one word: the upper halves of lo and hi (lo in bits 0-15)
__device__ __forceinline__ uint32_t pack_upper_halves(uint32_t lo, uint32_t hi) { return __builtin_amdgcn_perm(hi, lo, 0x07060302u); }

// The quad's four draws as a mask: bit e is set where u >= p for element e (the element survives standard dropout; the
// reference's forms keep the complement).  Without dropout every bit is set and nothing is drawn.
// mask_idx: the quad's element index in the whole [M x N] output, which the mask is drawn from.
template <bool REF>
__device__ __forceinline__ uint32_t draw_quad(const EpiPrm& k, size_t mask_idx) {
  if (!REF && !k.apply_dropout) return 0xfu;
  const uint64_t blk = (uint64_t)mask_idx >> 2;   // the Philox counter: one block of four words per quad
  const Philox4 r = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), 0u, 0u, k.seed_lo, k.seed_hi);
  return (keep_from_threshold(r.x, k.thr) ? 1u : 0u) | (keep_from_threshold(r.y, k.thr) ? 2u : 0u) |
         (keep_from_threshold(r.z, k.thr) ? 4u : 0u) | (keep_from_threshold(r.w, k.thr) ? 8u : 0u);
}
// The four finished 16-bit outputs of a quad.  ge: draw_quad's mask for this quad; bv: the bias of its four columns.
// REF: one of the reference's dropout forms (k.mode says which); false: standard dropout, the form the kernels are
// tuned for, compiled without the others.
template <int NP, bool REF, bool F16 = false>
__device__ __forceinline__ u32x2 epilogue_quad(f32x4 acc, const EpiIn<NP>& in, const f32x4 bv, const EpiPrm& k, uint32_t ge) {
  f32x4 s = acc;
#pragma unroll
  for (int q = 0; q < NP; q++) s = s + in.pv[q];
  const float rs[4] = {half_in<F16>((uint16_t)(in.rv[0] & 0xffffu)), half_in<F16>((uint16_t)(in.rv[0] >> 16)),
                       half_in<F16>((uint16_t)(in.rv[1] & 0xffffu)), half_in<F16>((uint16_t)(in.rv[1] >> 16))};
  float y[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const bool g = (ge >> e) & 1u;
    if constexpr (!REF) {
      // drop with probability p, survivors scaled by 1/(1-p) (keep_scale is 1 without dropout)
      const float t = s[e] + bv[e];
      y[e] = (g ? t * k.keep_scale : 0.0f) + rs[e];
    } else if (k.mode == CCN_DROPOUT_REF_DSL) {
      // the reference's emitted expression (src/codegen.cpp:634-640): (u < p ? (sum + bias) : 0) + residual
      const float t = s[e] + bv[e];
      y[e] = (!g ? t : 0.0f) + rs[e];
    } else {
      // the reference's fused kernel (nccl-overlap/src/collectives/device/reduce_kernel.h:192-213):
      // ((u < p ? sum : 0) + bias) + residual; its half specialisation adds with saturation to [0, 1]
      // (value and bias are halves there and each __hadd2_sat rounds to half: restated for IEEE-half operands; an fp32
      // sum of two halves converted to half is the correctly rounded half sum)
      const float d = !g ? s[e] : 0.0f;
      if (k.mode != CCN_DROPOUT_REF_NCCL_SAT) y[e] = (d + bv[e]) + rs[e];
      else if constexpr (F16) y[e] = sat01(f16_round(sat01(f16_round(d) + f16_round(bv[e]))) + rs[e]);
      else y[e] = sat01(sat01(d + bv[e]) + rs[e]);
    }
  }
  u32x2 o;
  if constexpr (F16) {
    o[0] = (uint32_t)half_out<F16>(y[0]) | ((uint32_t)half_out<F16>(y[1]) << 16);
    o[1] = (uint32_t)half_out<F16>(y[2]) | ((uint32_t)half_out<F16>(y[3]) << 16);
  } else {
    o[0] = pack_upper_halves(f32_to_bf16_hi(y[0]), f32_to_bf16_hi(y[1]));
    o[1] = pack_upper_halves(f32_to_bf16_hi(y[2]), f32_to_bf16_hi(y[3]));
  }
  return o;
}
// The same with the quad addressed by its element index idx in `out` and its first column n.
template <int NP, bool REF, bool F16 = false>
__device__ __forceinline__ void epilogue_finish(f32x4 acc, const EpiIn<NP>& in, const float* __restrict__ bias,
                                                uint16_t* __restrict__ out, size_t idx, size_t n, const EpiPrm& k,
                                                size_t mask_idx) {
  const u32x2 o = epilogue_quad<NP, REF, F16>(acc, in, *reinterpret_cast<const f32x4*>(bias + n), k, draw_quad<REF>(k, mask_idx));
  __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(out + idx));
}

// Buffer addressing: a workgroup-uniform base (a resource descriptor in scalar registers, no bounds: the host checks the
// offsets), a uniform scalar offset and one 32-bit offset per lane.  The addresses of a tile walk then cost scalar
// adds where 64-bit flat addresses cost a vector register pair and a 64-bit vector add per access.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t buffer_at(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7ffffffc, 0x00020000);
}
constexpr int kAuxNt = 2;   // the nontemporal bit of a gfx950 buffer instruction's cache policy
// The matrix-core kernel reaches 128 rows of N fp32 and 128 rows of K 16-bit elements from one descriptor: both must stay
// inside the 2 GiB a descriptor spans.  Larger row lengths take the any-shape kernel.
constexpr int kMaxRowLen = 1 << 21;

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 7); }

// PLAIN: the product alone through `out` (no partial buffers, bias, dropout or residual): 1 writes fp32 [M x N], 2 rounds
// to the operands' 16-bit type (round to nearest even).
// REF: the epilogue applies one of the reference's dropout forms.
// The rows are dealt to the wavefronts (see the top of the file) so that the epilogue needs no workgroup barrier: after
// the main loop a wavefront turns its own accumulators into rows through a private piece of LDS (16 rows at a time) and
// walks its 16 row pairs.  At step j the four wavefronts of the workgroup together touch 8 adjacent rows x 512 bytes of
// every partial buffer; the operands of step j+1 are requested before step j is finished, step 0's under the last MFMA
// step.  Three workgroups share a CU (168 registers, 33 KiB of LDS).
template <int NP, int PLAIN = 0, bool REF = false, bool F16 = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(3, 3)))
void mlp_outproj_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, const SrcTable<float, 8> parts,
                        const float* __restrict__ bias, const uint16_t* __restrict__ resid, uint16_t* __restrict__ out,
                        const int N, const int K, const EpiPrm ep) {
  constexpr int kCStride = BN + 4;
  constexpr int kWaveRows = 16;   // rows of C a wavefront has in LDS at a time
  constexpr int kCBytes = (kBlock / kWave) * kWaveRows * kCStride * 4;
  constexpr int kTileBytes = 2 * BM * BK * 2;                 // one K-step of X and W^T
  constexpr int kLdsBytes = kCBytes > kTileBytes ? kCBytes : kTileBytes;
  __shared__ __attribute__((aligned(16))) uint8_t lds_all[kLdsBytes];
  uint8_t* const lds_x = lds_all;
  uint8_t* const lds_w = lds_all + BM * BK * 2;

  const int tilesN = N / BN;
  const int tm = blockIdx.x / tilesN, tn = blockIdx.x % tilesN;
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int li = lane & 31, lh = lane >> 5;
  const int rho = 8 * (li >> 1) + 2 * wave + (li & 1);   // tile row behind this lane's accumulator column

  // Addresses are a workgroup-uniform 64-bit base, kept in scalar registers and advanced by scalar adds, plus a 32-bit
  // byte offset per lane that never changes (the host checks that the offsets fit): no vector address arithmetic.
  const int xr = t >> 3, xc = t & 7;          // X: rows xr + 32*j, 16-byte chunk xc
  const int wg = t & 15, wq = t >> 4;         // W: k rows wq*4 + j, columns wg*8..+7
  struct Staged { u32x4 x[4], w[4]; };
  uint32_t xoff[4], woff[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    xoff[j] = (uint32_t)(((xr + 32 * j) * K + xc * 8) * 2);
    woff[j] = (uint32_t)(((wq * 4 + j) * N + wg * 8) * 2);
  }
  const rsrc_t x_rs = buffer_at(X + m0 * (size_t)K);   // the tile's 128 rows of X
  const uint16_t* const wbase = W + n0;

  auto load_tile = [&](Staged& r, int k0) {
    const rsrc_t w_rs = buffer_at(wbase + (size_t)k0 * N);   // the 64 rows of W of this K-step
#pragma unroll
    for (int j = 0; j < 4; j++) {
      r.x[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(x_rs, xoff[j], (uint32_t)k0 * 2u, 0));
      r.w[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(w_rs, woff[j], 0, 0));
    }
  };
  auto store_tile = [&](const Staged& r) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int row = xr + 32 * j;
      *reinterpret_cast<u32x4*>(lds_x + row * 128 + ((xc ^ swz(row)) << 4)) = r.x[j];
    }
    // W as it lies in memory: row k = wq*4 + j of 256 bytes, the 16-byte chunk wg at position wg ^ 4*(k%4)
#pragma unroll
    for (int j = 0; j < 4; j++)
      *reinterpret_cast<u32x4*>(lds_w + ((wq * 4 + j) * 16 + (wg ^ (4 * j))) * 16) = r.w[j];
  };

  f32x16 acc[4];   // [bn]: register 4*i4+e is C[rho][bn*32 + i4*8 + lh*4 + e]
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[a][i] = 0.0f;

  // One K-step: four rounds of 16 k, each one X fragment against four W fragments: 16 MFMAs.  The W fragment of MFMA
  // i+2 (and the X fragment of the next round) is read from LDS before MFMA i is issued, so that an MFMA does not wait
  // for the read just before it; two fragments ahead is what the register budget of three workgroups per CU allows.
  const int a16 = lane & 15, g2 = (lane >> 4) & 1;
  const int waddr = ((lh * 8 + (a16 >> 2)) * 16 + ((2 * g2 + ((a16 >> 1) & 1)) ^ (4 * (a16 >> 2)))) * 16 + 8 * (a16 & 1);
  auto read_w = [&](int i) {
    // fragment i%4 (32 columns), round i/4: k = 16*(i/4) + 8*lh + 0..7 in two transposing reads of 4 k each
    const uint8_t* p = lds_w + (waddr ^ ((i & 3) * 64)) + (i >> 2) * 4096;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 1024));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto read_x = [&](int ks) {
    const int c = ks * 2 + lh;
    return *reinterpret_cast<const bf16x8*>(lds_x + rho * 128 + ((c ^ swz(rho)) << 4));
  };
  auto mfma_step = [&]() {
    constexpr int kAhead = 2;
    bf16x8 fa[kAhead + 1], fb[2];
    fb[0] = read_x(0);
#pragma unroll
    for (int i = 0; i < kAhead; i++) fa[i] = read_w(i);
    constexpr int kWReads = 2;   // LDS instructions per W fragment
    __builtin_amdgcn_sched_group_barrier(0x100, 1 + kAhead * kWReads, 0);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      int reads = 0;
      if (i + kAhead < 16) { fa[(i + kAhead) % (kAhead + 1)] = read_w(i + kAhead); reads += kWReads; }
      if ((i & 3) == 4 - kAhead && (i >> 2) + 1 < 4) { fb[((i >> 2) + 1) & 1] = read_x((i >> 2) + 1); reads++; }
      if (reads == 3) __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
      if (reads == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      if (reads == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      const bf16x8 a = fa[i % (kAhead + 1)], b = fb[(i >> 2) & 1];
      if constexpr (F16)
        acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc[i & 3], 0, 0, 0);
      else
        acc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i & 3], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  };

  // the walk of the epilogue: at step j this lane has row 8j + 2*wave + lane/32, columns 4*(lane%32)..+3
  const int sc = li * 4;
  const size_t tile0 = m0 * (size_t)N + n0;                                  // first element of the tile (uniform)
  const uint32_t eoff = (uint32_t)((2 * wave + lh) * N + sc);                // this lane's element within a step
  const uint32_t estep = 8u * (uint32_t)N;                                   // elements from one step to the next
  rsrc_t p_rs[NP > 0 ? NP : 1];
#pragma unroll
  for (int q = 0; q < (PLAIN ? 0 : NP); q++) p_rs[q] = buffer_at(parts.p[q] + tile0);
  const rsrc_t r_rs = buffer_at(resid ? resid + tile0 : nullptr);
  const rsrc_t o_rs = buffer_at(PLAIN == 1 ? static_cast<void*>(reinterpret_cast<float*>(out) + tile0) : static_cast<void*>(out + tile0));
  auto load_step = [&](EpiIn<PLAIN ? 0 : NP>& in, int j) {
#pragma unroll
    for (int q = 0; q < (PLAIN ? 0 : NP); q++)
      in.pv[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(p_rs[q], eoff * 4u, (uint32_t)j * estep * 4u, kAuxNt));
    in.rv = u32x2{0u, 0u};
    if (resid) in.rv = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r_rs, eoff * 2u, (uint32_t)j * estep * 2u, kAuxNt));
  };
  EpiIn<PLAIN ? 0 : NP> cur;

  // main loop: the tile of step kt+1 travels from memory to registers while step kt is multiplied
  const int nk = K / BK;
  Staged st;
  load_tile(st, 0);
  store_tile(st);
  if (nk > 1) load_tile(st, BK);
  __syncthreads();
  for (int kt = 0; kt + 1 < nk; kt++) {
    mfma_step();
    __syncthreads();
    store_tile(st);
    // the next tile's loads go out as soon as the staging registers are free, ahead of the barrier and the MFMA step
    // (the sched_barrier keeps the scheduler from sinking them to their use)
    if (kt + 2 < nk) load_tile(st, (kt + 2) * BK);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
  }
  if constexpr (!PLAIN) load_step(cur, 0);
  mfma_step();
  __syncthreads();   // every wavefront is done with the operand tiles: LDS becomes four private C pieces

  float* const cw = reinterpret_cast<float*>(lds_all) + wave * (kWaveRows * kCStride);
  f32x4 bv = {0.0f, 0.0f, 0.0f, 0.0f};
  if constexpr (!PLAIN) bv = *reinterpret_cast<const f32x4*>(bias + n0 + sc);
#pragma unroll
  for (int half = 0; half < 2; half++) {
    if ((li >> 4) == half) {
      const int r16 = li & 15;
#pragma unroll
      for (int bn = 0; bn < 4; bn++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          f32x4 v;
          v[0] = acc[bn][i4 * 4 + 0];
          v[1] = acc[bn][i4 * 4 + 1];
          v[2] = acc[bn][i4 * 4 + 2];
          v[3] = acc[bn][i4 * 4 + 3];
          *reinterpret_cast<f32x4*>(cw + r16 * kCStride + bn * 32 + i4 * 8 + lh * 4) = v;
        }
    }
    __builtin_amdgcn_wave_barrier();   // a wavefront's LDS operations complete in order: no wait between its writes and reads
#pragma unroll
    for (int jj = 0; jj < 8; jj++) {
      const int j = half * 8 + jj;
      const f32x4 v = *reinterpret_cast<const f32x4*>(cw + (2 * jj + lh) * kCStride + sc);
      if constexpr (PLAIN == 1) {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), o_rs, eoff * 4u, (uint32_t)j * estep * 4u, 0);
      } else if constexpr (PLAIN == 2) {
        __builtin_amdgcn_raw_buffer_store_b64(pack_quad<F16>(v), o_rs, eoff * 2u, (uint32_t)j * estep * 2u, 0);
      } else {
        const uint32_t ge = draw_quad<REF>(ep, tile0 + (size_t)j * estep + eoff);
        EpiIn<NP> nxt;
        if (j + 1 < 16) load_step(nxt, j + 1);
        const u32x2 o = epilogue_quad<NP, REF, F16>(v, cur, bv, ep, ge);
        __builtin_amdgcn_raw_buffer_store_b64(o, o_rs, eoff * 2u, (uint32_t)j * estep * 2u, kAuxNt);
        if (j + 1 < 16) cur = nxt;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// ---- the plain product on large tiles ------------------------------------------------------------------------------------
// C[M x N] (fp32) = X . W alone is bound by the matrix cores, and a 128 x 128 tile moves too many operand bytes per MFMA
// to keep them busy.  For whole multiples of 256 rows and columns: a 256-thread workgroup owns a 256(m) x 256(n) tile,
// ONE wavefront per SIMD, each 128 x 128 as sixteen 32 x 32 blocks (256 accumulator registers, which the compiler keeps
// in the accumulation half of the register file); per 16-k round a wavefront reads four X and four W fragments from
// LDS for sixteen MFMAs.  (Two wavefronts per SIMD of 128 x 64 each do not share the matrix core evenly: the older one
// is served first and then waits at every barrier for the younger one, which runs the rest alone at three quarters of
// the rate.)  One workgroup per CU.
// The operands travel global memory -> LDS directly (no staging registers, no LDS store instructions) into a ring of
// four stages of 32 k (X: 256 rows of 64 bytes, chunks swizzled by (row/4)%4; W as it lies in memory, 32 rows of 512
// bytes, chunks swizzled by 4*(k%4), read back through ds_read_b64_tr_b16).  A wavefront requests one KiB every fourth
// MFMA, all the time: wavefronts asking for a whole step at once stand in the queue of the CU's address path instead
// of issuing MFMAs.  A request is waited for three steps after it was made.
// Workgroups are numbered so that the 32 an XCD runs at a time form a block of 4 x 8 tiles: their X and W panels are
// shared inside that XCD's L2.  The accumulators leave through wavefront-private pieces of LDS as whole 512-byte rows.
constexpr int TM = 256, TN = 256;
constexpr int kBigBlock = 256;
constexpr int kBigK = 32;                            // k per stage
constexpr int kBigStage = (TM + TN) * kBigK * 2;     // one step of X and W: 32 KiB
constexpr int kBigStages = 4;
constexpr int kBigLds = kBigStages * kBigStage;

template <bool F16, bool C16>
__global__ __launch_bounds__(kBigBlock) __attribute__((amdgpu_waves_per_eu(1, 1)))
void matmul_tile256_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ W, void* __restrict__ Cout, const int N,
                           const int K, const int tilesM, const int tilesN) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_big[];
  // tile of this workgroup: blocks of 4 x 8 tiles dealt to the XCDs (workgroup b runs on XCD b % 8) when the grid divides
  int tm, tn;
  {
    const int b = blockIdx.x;
    if (tilesM % 4 == 0 && tilesN % 8 == 0 && ((tilesM / 4) * (tilesN / 8)) % 8 == 0) {
      const int xcd = b & 7, s_ = b >> 3, blk = (s_ >> 5) * 8 + xcd, j = s_ & 31;
      const int bcols = tilesN / 8;
      tm = (blk / bcols) * 4 + (j >> 3);
      tn = (blk % bcols) * 8 + (j & 7);
    } else {
      tm = b / tilesN;
      tn = b % tilesN;
    }
  }
  const size_t m0 = (size_t)tm * TM, n0 = (size_t)tn * TN;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);   // a scalar: it goes into descriptors
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lh = lane >> 5;

  // A direct-to-LDS load fills 1 KiB, lane L its 16 bytes at position L, so the swizzles are applied on the global side:
  // lane L fetches the chunk that belongs at L.  Per stage wavefront w brings the X rows 16*(w + 4j).. (16 rows of 64
  // bytes) and the W rows 2*(w + 4j).. (2 rows of 512 bytes), j = 0..3.  X: position (row, slot) holds memory chunk
  // slot ^ (row/4)%4; W: position (k, slot) holds chunk slot ^ 4*(k%4).
  const uint32_t xvoff = (uint32_t)(((lane >> 2) * K + 8 * ((lane & 3) ^ ((lane >> 4) & 3))) * 2);
  const uint32_t wvoff = (uint32_t)(((lane >> 5) * N + 8 * ((lane & 31) ^ (4 * (2 * (wave & 1) + (lane >> 5))))) * 2);
  // The loads are written as assembly: the compiler orders every LDS read after a direct-to-LDS load it can see behind a
  // wait for ALL outstanding loads, which would put the memory latency into every step.  Here the only reads of a
  // stage follow the wait and barrier below, so the waits are placed by hand.  (m0, which names the LDS destination, is
  // a reserved register: the compiler sets it right before its own uses and keeps nothing in it across a statement.)
  auto words = [](const void* base) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    return u32x4{(uint32_t)a, (uint32_t)(a >> 32), 0x7ffffffcu, 0x00020000u};   // no stride, no bounds, as buffer_at()
  };
  auto load_to_lds = [](u32x4 rs, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rs), "s"(soff) : "memory");
  };
  const u32x4 x_rs = words(X + m0 * (size_t)K);
  const uint16_t* const wbase = W + n0;
  typedef __attribute__((address_space(3))) void* lds_void_ptr;
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((lds_void_ptr)lds_big) + (uint32_t)wave * 1024u;
  const int nk = K / kBigK;
  // request j (0..3) of the X / W operands of step `kt` (past the end: the last step's again, unused), into stage `stage`
  const uint32_t xs0 = (uint32_t)(16 * wave * K * 2), xsj = (uint32_t)(64 * K * 2);
  const uint32_t ws0 = (uint32_t)(2 * wave * N * 2), wsj = (uint32_t)(8 * N * 2);
  auto request_x = [&](int stage, int kt, int j) {
    const uint32_t kc = (uint32_t)(kt < nk ? kt : nk - 1);
    load_to_lds(x_rs, lds0 + stage * kBigStage + j * 4096, xvoff, xs0 + j * xsj + kc * (kBigK * 2));
  };
  auto request_w = [&](int stage, int kt, int j) {
    const uint32_t kc = (uint32_t)(kt < nk ? kt : nk - 1);
    // the step goes into the descriptor's 64-bit base: W may be larger than the 2 GiB a descriptor spans
    load_to_lds(words(wbase + (size_t)kc * kBigK * N), lds0 + stage * kBigStage + TM * kBigK * 2 + j * 4096, wvoff, ws0 + j * wsj);
  };
  // fragment addresses: X rows 128*wm + 32*bm + li, chunk 2*ks + lh; W fragment bn of this wavefront's 128 columns
  int xaddr[4];
#pragma unroll
  for (int bm = 0; bm < 4; bm++) xaddr[bm] = (128 * wm + 32 * bm + li) * 64;   // + ((2*ks + lh) ^ swizzle) * 16
  const int xsw = (li >> 2) & 3;   // (row/4) % 4: the rows of a fragment start at a multiple of 32
  const int a16 = lane & 15, g2 = (lane >> 4) & 1;
  const int waddr = ((lh * 8 + (a16 >> 2)) * 32 + ((16 * wn + 2 * g2 + ((a16 >> 1) & 1)) ^ (4 * (a16 >> 2)))) * 16 + 8 * (a16 & 1);
  auto read_x = [&](int buf, int bm, int ks) {
    return *reinterpret_cast<const s16x8*>(lds_big + buf * kBigStage + xaddr[bm] + (((2 * ks + lh) ^ xsw) << 4));
  };
  auto read_w = [&](int buf, int bn, int ks) {
    const uint8_t* p = lds_big + buf * kBigStage + TM * kBigK * 2 + (waddr ^ (bn * 64)) + ks * (16 * 512);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * 512));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  f32x16 acc[4][4];   // [bn][bm]: register 4*i4+e is C[128*wm + 32*bm + li][128*wn + 32*bn + 8*i4 + 4*lh + e]
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

  // A round of 16 k: four W and four X fragments for sixteen MFMAs, in two alternating fragment sets.  A round multiplies
  // from set `set` while the eight fragments of the NEXT round are read into the other set from (stage rbuf, round rks)
  // in the order the next round's MFMAs need them; after every fourth MFMA the round makes one request for step `lkt`
  // (requests 2*half.. of X, then of W).  Every piece is pinned in place: the order IS the schedule.
  s16x8 fw[2][4], fx[2][4];
  auto mfma = [&](int set, int bm, int bn) {
    if constexpr (F16)
      acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fw[set][bn]), __builtin_bit_cast(f16x8, fx[set][bm]), acc[bn][bm], 0, 0, 0);
    else
      acc[bn][bm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fw[set][bn]), __builtin_bit_cast(bf16x8, fx[set][bm]), acc[bn][bm], 0, 0, 0);
  };
  auto pin = [] { __builtin_amdgcn_sched_barrier(0); };
  auto round = [&](int set, int rbuf, int rks, int lstage, int lkt, int half) {
    const int o = set ^ 1;
    fw[o][0] = read_w(rbuf, 0, rks); mfma(set, 0, 0); pin();
    fx[o][0] = read_x(rbuf, 0, rks); mfma(set, 0, 1); pin();
    fw[o][1] = read_w(rbuf, 1, rks); mfma(set, 0, 2); pin();
    mfma(set, 0, 3); pin();
    request_x(lstage, lkt, 2 * half); pin();
    fw[o][2] = read_w(rbuf, 2, rks); mfma(set, 1, 0); pin();
    fw[o][3] = read_w(rbuf, 3, rks); mfma(set, 1, 1); pin();
    fx[o][1] = read_x(rbuf, 1, rks); mfma(set, 1, 2); pin();
    mfma(set, 1, 3); pin();
    request_x(lstage, lkt, 2 * half + 1); pin();
    fx[o][2] = read_x(rbuf, 2, rks); mfma(set, 2, 0); pin();
    mfma(set, 2, 1); pin();
    mfma(set, 2, 2); pin();
    mfma(set, 2, 3); pin();
    request_w(lstage, lkt, 2 * half); pin();
    fx[o][3] = read_x(rbuf, 3, rks); mfma(set, 3, 0); pin();
    mfma(set, 3, 1); pin();
    mfma(set, 3, 2); pin();
    mfma(set, 3, 3); pin();
    request_w(lstage, lkt, 2 * half + 1); pin();
  };

  // Main loop: step kt multiplies 32 k from stage kt%4 (four steps per trip, so that every LDS address is a constant).
  //   round 0   MFMAs; reads round 1's fragments; second half of the requests for step kt+3
  //   barrier   every wavefront waits for its own requests for step kt+1 (the sixteen newer ones stay in flight) and
  //             for its LDS reads, then for the others: stage (kt+1)%4 is complete, nobody reads stage kt%4 any more
  //   round 1   MFMAs; reads round 0 of step kt+1; first half of the requests for step kt+4, into stage kt%4
  auto step = [&](int st, int kt) {
    round(0, st, 1, (st + 3) & 3, kt + 3, 1);
    __builtin_amdgcn_s_waitcnt(0x4070);   // vmcnt(16) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    pin();
    round(1, (st + 1) & 3, 0, st, kt + 4, 0);
  };
#pragma unroll
  for (int st = 0; st < 3; st++) {
    request_x(st, st, 0); request_x(st, st, 1); request_w(st, st, 0); request_w(st, st, 1);
    request_x(st, st, 2); request_x(st, st, 3); request_w(st, st, 2); request_w(st, st, 3);
  }
  request_x(3, 3, 0); request_x(3, 3, 1); request_w(3, 3, 0); request_w(3, 3, 1);
  __builtin_amdgcn_s_waitcnt(0x4074);   // vmcnt(20) lgkmcnt(0): the requests for step 0 have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int bn = 0; bn < 4; bn++) fw[0][bn] = read_w(0, bn, 0);
#pragma unroll
  for (int bm = 0; bm < 4; bm++) fx[0][bm] = read_x(0, bm, 0);
  int kt = 0;
  for (; kt + 4 <= nk; kt += 4) {
    step(0, kt);
    step(1, kt + 1);
    step(2, kt + 2);
    step(3, kt + 3);
  }
  if (kt < nk) {   // K is a multiple of 64: two steps are left
    step(0, kt);
    step(1, kt + 1);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0): the last reads of LDS and the last (unused) loads into it are done
  __builtin_amdgcn_s_barrier();         // ... everywhere, before the stages become C pieces
  constexpr int kCS = 128 + 4;   // floats per row of a piece: 32 rows x 128 columns at a time
  float* const cw = reinterpret_cast<float*>(lds_big) + wave * (32 * kCS);
  const size_t c0 = (m0 + 128 * wm) * (size_t)N + n0 + 128 * wn;
  const rsrc_t c_rs = C16 ? buffer_at(static_cast<uint16_t*>(Cout) + c0) : buffer_at(static_cast<float*>(Cout) + c0);
  const int r2 = lane >> 5, c32 = lane & 31, r4 = lane >> 4, c16 = lane & 15;
#pragma unroll
  for (int bm = 0; bm < 4; bm++) {
#pragma unroll
    for (int bn = 0; bn < 4; bn++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        f32x4 v;
        v[0] = acc[bn][bm][i4 * 4 + 0];
        v[1] = acc[bn][bm][i4 * 4 + 1];
        v[2] = acc[bn][bm][i4 * 4 + 2];
        v[3] = acc[bn][bm][i4 * 4 + 3];
        *reinterpret_cast<f32x4*>(cw + li * kCS + bn * 32 + i4 * 8 + lh * 4) = v;
      }
    __builtin_amdgcn_wave_barrier();   // a wavefront's LDS operations complete in order
    if constexpr (C16) {   // 8 columns per lane: four rows of 256 bytes per instruction
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        const float* src = cw + (4 * jj + r4) * kCS + 8 * c16;
        const u32x2 lo = pack_quad<F16>(*reinterpret_cast<const f32x4*>(src)), hi = pack_quad<F16>(*reinterpret_cast<const f32x4*>(src + 4));
        const uint32_t off = (uint32_t)(((32 * bm + 4 * jj + r4) * N + 8 * c16) * 2);
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{lo[0], lo[1], hi[0], hi[1]}, c_rs, off, 0, 0);
      }
    } else {
#pragma unroll
      for (int jj = 0; jj < 16; jj++) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(cw + (2 * jj + r2) * kCS + 4 * c32);
        const uint32_t off = (uint32_t)(((32 * bm + 2 * jj + r2) * N + 4 * c32) * 4);
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), c_rs, off, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
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
template <int PLAIN, bool REF, bool F16 = false>
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
    if constexpr (PLAIN == 1) {
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(out) + idx) = sum;
    } else if constexpr (PLAIN == 2) {
      *reinterpret_cast<u32x2*>(out + idx) = pack_quad<F16>(sum);
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
  ep->thr = keep_threshold(p_drop);
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
  // the 16-bit residual and output move 8 bytes at a time (a tile starts on a multiple of 4 columns)
  if (!aligned16(X) || !aligned16(W) || !aligned16(bias) || !aligned8(out) || (resid && !aligned8(resid))) return CCN_EINVAL;
  EpiPrm ep;
  int rc = make_epi(p_drop, seed, mode, &ep);
  if (rc != CCN_OK) return rc;
  const DeviceInfo* di = nullptr;
  rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (M % BM || N % BN || K % BK || N > kMaxRowLen || K > kMaxRowLen) {   // not whole tiles of the matrix-core kernel
    const size_t tiles = (size_t)((M + GT - 1) / GT) * (size_t)((N + GT - 1) / GT);
    if (tiles > 0x7fffffffull) return CCN_ERANGE;
    if (mode == CCN_DROPOUT_INVERTED)
      hipLaunchKernelGGL((outproj_any_shape_kernel<0, false, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, s, X, W, tbl, nPartials,
                         bias, resid, out, M, N, K, ep);
    else
      hipLaunchKernelGGL((outproj_any_shape_kernel<0, true, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, s, X, W, tbl, nPartials,
                         bias, resid, out, M, N, K, ep);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }
  const dim3 grid((unsigned)((M / BM) * (N / BN))), block(kBlock);
  switch (nPartials) {
#define CCN_CASE(Q)                                                                                                          \
  case Q:                                                                                                                    \
    if (mode == CCN_DROPOUT_INVERTED) hipLaunchKernelGGL((mlp_outproj_kernel<Q, 0, false, F16>), grid, block, 0, s, X, W, tbl, bias, resid, out, N, K, ep); \
    else hipLaunchKernelGGL((mlp_outproj_kernel<Q, 0, true, F16>), grid, block, 0, s, X, W, tbl, bias, resid, out, N, K, ep); \
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

template <bool F16, bool C16>
int matmul_launch(const uint16_t* X, const uint16_t* W, void* C, int M, int N, int K, void* stream) {
  if (!X || !W || !C) return CCN_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0) return CCN_EINVAL;
  if (N % 4) return CCN_ERANGE;
  if (!aligned16(X) || !aligned16(W) || !(C16 ? aligned8(C) : aligned16(C))) return CCN_EINVAL;
  const DeviceInfo* di = nullptr;
  const int rc = current_device_info(&di);
  if (rc != CCN_OK) return rc;
  SrcTable<float, 8> tbl;
  for (int q = 0; q < 8; q++) tbl.p[q] = nullptr;
  EpiPrm ep{};
  constexpr int kPlain = C16 ? 2 : 1;
  if (M % BM || N % BN || K % BK || N > kMaxRowLen || K > kMaxRowLen) {
    const size_t tiles = (size_t)((M + GT - 1) / GT) * (size_t)((N + GT - 1) / GT);
    if (tiles > 0x7fffffffull) return CCN_ERANGE;
    hipLaunchKernelGGL((outproj_any_shape_kernel<kPlain, false, F16>), dim3((unsigned)tiles), dim3(kBlock), 0, as_stream(stream), X, W,
                       tbl, 0, (const float*)nullptr, (const uint16_t*)nullptr, static_cast<uint16_t*>(C), M, N, K, ep);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }
  // Whole large tiles, and enough of them to occupy at least half of the CUs (one workgroup per CU): the matrix-core-bound
  // kernel.  Smaller products are faster on four times as many 128 x 128 tiles (16 / 64 large tiles at K = 1024: 13.5
  // against 21.4 us / 17.6 against 24.9 us; 128: 26.6 against 27.6; 256: 52.0 against 37.8).
  if (M % TM == 0 && N % TN == 0 && (size_t)128 * (size_t)N * 4 < 0x7fffffffull && aligned16(C) &&   // it stores 16 bytes per lane
      2 * (size_t)(M / TM) * (size_t)(N / TN) >= (size_t)di->cu_count) {
    static const hipError_t attr = hipFuncSetAttribute((const void*)matmul_tile256_kernel<F16, C16>,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kBigLds);
    if (attr != hipSuccess) return hip_fail(attr);
    const int tilesM = M / TM, tilesN = N / TN;
    hipLaunchKernelGGL((matmul_tile256_kernel<F16, C16>), dim3((unsigned)(tilesM * tilesN)), dim3(kBigBlock), kBigLds, as_stream(stream),
                       X, W, C, N, K, tilesM, tilesN);
    CCN_HIP(hipGetLastError());
    return CCN_OK;
  }
  const dim3 grid((unsigned)((M / BM) * (N / BN))), block(kBlock);
  hipLaunchKernelGGL((mlp_outproj_kernel<0, kPlain, false, F16>), grid, block, 0, as_stream(stream), X, W, tbl, (const float*)nullptr,
                     (const uint16_t*)nullptr, static_cast<uint16_t*>(C), N, K, ep);
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
  return matmul_launch<false, false>(X, W, C, M, N, K, stream);
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
  return matmul_launch<true, false>(X, W, C, M, N, K, stream);
}

int ccn_matmul_bf16(const uint16_t* X, const uint16_t* W, uint16_t* C, int M, int N, int K, void* stream) {
  return matmul_launch<false, true>(X, W, C, M, N, K, stream);
}

int ccn_matmul_f16(const uint16_t* X, const uint16_t* W, uint16_t* C, int M, int N, int K, void* stream) {
  return matmul_launch<true, true>(X, W, C, M, N, K, stream);
}

}  // extern "C"
