// to_mx quantize casts for gfx950: bf16 -> e4m3fn codes + E8M0 scales, blocks of 32.
//
// All three kernels are HBM-streaming: one coalesced read of the bf16 tensor, one write of
// the codes (1 B/elem) and of the scales (1/32 B/elem).  Algorithmic traffic is
// 3.03125 B/elem for a single direction and 4.0625 B/elem for the fused row+column cast.
#include "mx_common.h"

namespace mx {

// ------------------------------------------------------------------------------------
// dim0: blocks run along the contiguous dimension.  A lane owns 8 consecutive elements
// (one 16-byte load); the 4 lanes of a DPP quad own one block and share its amax through
// two quad_perm exchanges.  Each workgroup streams 1024 consecutive 16-byte chunks.
// ------------------------------------------------------------------------------------
constexpr int kDim0Threads = 256;
constexpr int kDim0Unroll = 4;

template <int MODE, int ORDER>
__global__ __launch_bounds__(kDim0Threads) void cast_dim0_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, uint32_t cpr /* 16B chunks per row */,
    int64_t total_chunks, uint8_t* __restrict__ codes, uint8_t* __restrict__ scales,
    int64_t nblk, int64_t ks_n) {
  const int64_t base = (int64_t)blockIdx.x * (kDim0Threads * kDim0Unroll) + threadIdx.x;
  u32x4 v[kDim0Unroll];
  int64_t row[kDim0Unroll];
  uint32_t col[kDim0Unroll];
  bool ok[kDim0Unroll];
#pragma unroll
  for (int k = 0; k < kDim0Unroll; ++k) {
    const int64_t c = base + (int64_t)k * kDim0Threads;
    ok[k] = c < total_chunks;
    const int64_t cc = ok[k] ? c : 0;
    if (total_chunks <= 0xFFFFFFFFll) {  // 32-bit divide when the index fits
      const uint32_t r32 = (uint32_t)cc / cpr;
      row[k] = r32;
      col[k] = (uint32_t)cc - r32 * cpr;
    } else {
      row[k] = cc / cpr;
      col[k] = (uint32_t)(cc - row[k] * cpr);
    }
    v[k] = u32x4{0, 0, 0, 0};
    if (ok[k])
      v[k] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>(x + row[k] * ldx + (int64_t)col[k] * 8));
  }
#pragma unroll
  for (int k = 0; k < kDim0Unroll; ++k) {
    const u32x4 w = v[k];
    uint32_t m = pk_max_u16(pk_max_u16(w.x & 0x7FFF7FFFu, w.y & 0x7FFF7FFFu),
                            pk_max_u16(w.z & 0x7FFF7FFFu, w.w & 0x7FFF7FFFu));
    m = max(m & 0xFFFFu, m >> 16);
    m = max(m, dpp<kQuadXor1>(m));
    m = max(m, dpp<kQuadXor2>(m));
    const uint32_t sb = scale_byte<MODE>(m);
    const float mult = scale_multiplier<MODE>(sb);
    u32x2 out;
    if (sb != 255) {
      out.x = cvt2<true>(w.y, mult, cvt2<false>(w.x, mult, 0));
      out.y = cvt2<true>(w.w, mult, cvt2<false>(w.z, mult, 0));
    } else {
      out.x = nan_block_codes2(w.x) | (nan_block_codes2(w.y) << 16);
      out.y = nan_block_codes2(w.z) | (nan_block_codes2(w.w) << 16);
    }
    if (ok[k]) {
      __builtin_nontemporal_store(
          out, reinterpret_cast<u32x2*>(codes + (row[k] * cpr + col[k]) * 8));
      if ((threadIdx.x & 3) == 0) {
        const int64_t blk = col[k] >> 2;
        const int64_t off = (ORDER == MX_SCALES_MFMA) ? mfma_scale_offset(row[k], blk, ks_n)
                                                       : row[k] * nblk + blk;
        scales[off] = (uint8_t)sb;
      }
    }
  }
}

// ------------------------------------------------------------------------------------
// dim1: blocks run down the rows; codes and scales are written transposed.
// Tile = 128 rows x 128 columns per 256-thread workgroup.  Wave w owns row-block w of the
// tile, lane l owns columns 2l, 2l+1: every load instruction reads one 256-byte row
// segment, each thread keeps its 32x2 values in registers, the column amax is thread-local,
// and the codes go through LDS so that the transposed tile leaves as 128-byte rows.
// ------------------------------------------------------------------------------------
constexpr int kT = 128;          // tile edge
constexpr int kPitch = kT + 16;  // LDS row pitch of the transposed code tile (bytes)

template <int MODE>
__device__ __forceinline__ void quantize_column_pair(const uint32_t (&v)[32], uint32_t (&ca)[8],
                                                     uint32_t (&cb)[8], uint32_t& sa,
                                                     uint32_t& sb) {
  uint32_t m = 0;
#pragma unroll
  for (int k = 0; k < 32; ++k) m = pk_max_u16(m, v[k] & 0x7FFF7FFFu);
  sa = scale_byte<MODE>(m & 0xFFFFu);
  sb = scale_byte<MODE>(m >> 16);
  const float ma = scale_multiplier<MODE>(sa), mb = scale_multiplier<MODE>(sb);
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const uint32_t w0 = v[4 * q], w1 = v[4 * q + 1], w2 = v[4 * q + 2], w3 = v[4 * q + 3];
    if (sa != 255) {
      uint32_t c = cvt2f<false>(__uint_as_float(w0 << 16) * ma, __uint_as_float(w1 << 16) * ma, 0);
      ca[q] = cvt2f<true>(__uint_as_float(w2 << 16) * ma, __uint_as_float(w3 << 16) * ma, c);
    } else {
      ca[q] = nan_block_code(w0 & 0xFFFFu) | (nan_block_code(w1 & 0xFFFFu) << 8) |
              (nan_block_code(w2 & 0xFFFFu) << 16) | (nan_block_code(w3 & 0xFFFFu) << 24);
    }
    if (sb != 255) {
      uint32_t c = cvt2f<false>(__uint_as_float(w0 & 0xFFFF0000u) * mb,
                                __uint_as_float(w1 & 0xFFFF0000u) * mb, 0);
      cb[q] = cvt2f<true>(__uint_as_float(w2 & 0xFFFF0000u) * mb,
                          __uint_as_float(w3 & 0xFFFF0000u) * mb, c);
    } else {
      cb[q] = nan_block_code(w0 >> 16) | (nan_block_code(w1 >> 16) << 8) |
              (nan_block_code(w2 >> 16) << 16) | (nan_block_code(w3 >> 16) << 24);
    }
  }
}

// Write the staged transposed tile: 128 out-rows x 128 B of codes, plus its scales.
template <int ORDER>
__device__ __forceinline__ void store_transposed_tile(const uint8_t* lds_codes,
                                                      const uint8_t* lds_scales, int64_t r0,
                                                      int64_t c0, int64_t rows, int64_t cols,
                                                      uint8_t* __restrict__ codes_t,
                                                      uint8_t* __restrict__ scales_t,
                                                      int64_t nblk_t, int64_t ks_n_t) {
  const int tid = threadIdx.x;
  const int seg = tid & 7;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int o = p * 32 + (tid >> 3);
    if (c0 + o < cols && r0 + seg * 16 < rows) {
      const u32x4 q = *reinterpret_cast<const u32x4*>(lds_codes + o * kPitch + seg * 16);
      __builtin_nontemporal_store(
          q, reinterpret_cast<u32x4*>(codes_t + (c0 + o) * rows + r0 + seg * 16));
    }
  }
  if (tid < kT) {
    const uint32_t s4 = *reinterpret_cast<const uint32_t*>(lds_scales + tid * 4);
    if (ORDER == MX_SCALES_MFMA) {
      // the 512 staged bytes are two complete 256-byte (128-row, 64-deep K step) groups
      const int64_t ks = (r0 >> 6) + (tid >> 6);
      if (ks < ks_n_t)
        *reinterpret_cast<uint32_t*>(scales_t + (((c0 >> 7) * ks_n_t + ks) << 8) +
                                     (tid & 63) * 4) = s4;
    } else if (c0 + tid < cols) {
      const int64_t b0 = r0 >> 5;
      uint8_t* dst = scales_t + (c0 + tid) * nblk_t + b0;
      if ((nblk_t & 3) == 0 && b0 + 4 <= nblk_t) {
        *reinterpret_cast<uint32_t*>(dst) = s4;
      } else {
        for (int w = 0; w < 4 && b0 + w < nblk_t; ++w) dst[w] = (uint8_t)(s4 >> (8 * w));
      }
    }
  }
}

template <int MODE, int ORDER>
__global__ __launch_bounds__(256) void cast_dim1_kernel(const uint16_t* __restrict__ x,
                                                        int64_t rows, int64_t cols, int64_t ldx,
                                                        uint8_t* __restrict__ codes_t,
                                                        uint8_t* __restrict__ scales_t,
                                                        int64_t nblk_t, int64_t ks_n_t,
                                                        int64_t x_bstride, int64_t st_bstride) {
  __shared__ __attribute__((aligned(16))) uint8_t lds_codes[kT * kPitch];
  __shared__ __attribute__((aligned(16))) uint8_t lds_scales[kT * 4];
  x += blockIdx.z * x_bstride;  // batch of independent [rows, cols] matrices
  codes_t += blockIdx.z * rows * cols;
  scales_t += blockIdx.z * st_bstride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t r0 = (int64_t)blockIdx.y * kT, c0 = (int64_t)blockIdx.x * kT;
  const int64_t rb = r0 + wave * 32;
  const int64_t c = c0 + 2 * lane;
  const bool live = rb < rows && c < cols;

  uint32_t v[32];
  const uint16_t* src = x + rb * ldx + c;
#pragma unroll
  for (int k = 0; k < 32; ++k)
    v[k] = live ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src + k * ldx)) : 0u;

  uint32_t ca[8], cb[8], sa, sb;
  quantize_column_pair<MODE>(v, ca, cb, sa, sb);

  uint4* da = reinterpret_cast<uint4*>(lds_codes + (2 * lane) * kPitch + wave * 32);
  uint4* db = reinterpret_cast<uint4*>(lds_codes + (2 * lane + 1) * kPitch + wave * 32);
  da[0] = make_uint4(ca[0], ca[1], ca[2], ca[3]);
  da[1] = make_uint4(ca[4], ca[5], ca[6], ca[7]);
  db[0] = make_uint4(cb[0], cb[1], cb[2], cb[3]);
  db[1] = make_uint4(cb[4], cb[5], cb[6], cb[7]);
  if (!live) sa = sb = 0;
  if (ORDER == MX_SCALES_MFMA) {
    const int ca_ = 2 * lane, cb_ = 2 * lane + 1;
    lds_scales[(wave >> 1) * 256 + (((wave & 1) << 5) + (ca_ & 31)) * 4 + (ca_ >> 5)] = (uint8_t)sa;
    lds_scales[(wave >> 1) * 256 + (((wave & 1) << 5) + (cb_ & 31)) * 4 + (cb_ >> 5)] = (uint8_t)sb;
  } else {
    lds_scales[(2 * lane) * 4 + wave] = (uint8_t)sa;
    lds_scales[(2 * lane + 1) * 4 + wave] = (uint8_t)sb;
  }
  __syncthreads();
  store_transposed_tile<ORDER>(lds_codes, lds_scales, r0, c0, rows, cols, codes_t, scales_t,
                               nblk_t, ks_n_t);
}

// ------------------------------------------------------------------------------------
// Fused dim0 + dim1 from one read.  Same tile and thread ownership as cast_dim1_kernel;
// the row-wise amax of a 32-column block is the max over the 16 lanes that own it,
// exchanged with 4 DPP steps inside a 16-lane row.
// ------------------------------------------------------------------------------------
constexpr int kRowXor1 = 0xB1;   // quad_perm [1,0,3,2]
constexpr int kRowXor2 = 0x4E;   // quad_perm [2,3,0,1]
constexpr int kRowHalfMirror = 0x141;  // row_half_mirror: lane i <-> 7-i inside 8 lanes
constexpr int kRowMirror = 0x140;      // row_mirror: lane i <-> 15-i inside 16 lanes

template <int MODE, int ORDER>
__global__ __launch_bounds__(256) void cast_dim0_dim1_kernel(
    const uint16_t* __restrict__ x, int64_t rows, int64_t cols, int64_t ldx,
    uint8_t* __restrict__ codes, uint8_t* __restrict__ scales, int64_t nblk, int64_t ks_n,
    uint8_t* __restrict__ codes_t, uint8_t* __restrict__ scales_t, int64_t nblk_t,
    int64_t ks_n_t, int64_t x_bstride, int64_t s_bstride, int64_t st_bstride) {
  __shared__ __attribute__((aligned(16))) uint8_t lds_codes[kT * kPitch];
  __shared__ __attribute__((aligned(16))) uint8_t lds_scales[kT * 4];
  x += blockIdx.z * x_bstride;  // batch of independent [rows, cols] matrices
  codes += blockIdx.z * rows * cols;
  scales += blockIdx.z * s_bstride;
  codes_t += blockIdx.z * rows * cols;
  scales_t += blockIdx.z * st_bstride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t r0 = (int64_t)blockIdx.y * kT, c0 = (int64_t)blockIdx.x * kT;
  const int64_t rb = r0 + wave * 32;
  const int64_t c = c0 + 2 * lane;
  const bool live = rb < rows && c < cols;

  uint32_t v[32];
  const uint16_t* src = x + rb * ldx + c;
#pragma unroll
  for (int k = 0; k < 32; ++k)
    v[k] = live ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(src + k * ldx)) : 0u;

  // ---- row-wise (dim0) part: one 2-byte store per lane per row, 128 B per wave-row
#pragma unroll
  for (int k = 0; k < 32; ++k) {
    const uint32_t w = v[k] & 0x7FFF7FFFu;
    uint32_t m = max(w & 0xFFFFu, w >> 16);
    m = max(m, dpp<kRowXor1>(m));
    m = max(m, dpp<kRowXor2>(m));
    m = max(m, dpp<kRowHalfMirror>(m));
    m = max(m, dpp<kRowMirror>(m));
    const uint32_t sb = scale_byte<MODE>(m);
    const float mult = scale_multiplier<MODE>(sb);
    const uint32_t code2 = (sb != 255) ? cvt2<false>(v[k], mult, 0) : nan_block_codes2(v[k]);
    if (live) {
      const int64_t r = rb + k;
      *reinterpret_cast<uint16_t*>(codes + r * cols + c) = (uint16_t)code2;
      if ((lane & 15) == 0) {
        const int64_t blk = c >> 5;
        const int64_t off =
            (ORDER == MX_SCALES_MFMA) ? mfma_scale_offset(r, blk, ks_n) : r * nblk + blk;
        scales[off] = (uint8_t)sb;
      }
    }
  }

  // ---- column-wise (dim1) part
  uint32_t ca[8], cb[8], sa, sb;
  quantize_column_pair<MODE>(v, ca, cb, sa, sb);
  uint4* da = reinterpret_cast<uint4*>(lds_codes + (2 * lane) * kPitch + wave * 32);
  uint4* db = reinterpret_cast<uint4*>(lds_codes + (2 * lane + 1) * kPitch + wave * 32);
  da[0] = make_uint4(ca[0], ca[1], ca[2], ca[3]);
  da[1] = make_uint4(ca[4], ca[5], ca[6], ca[7]);
  db[0] = make_uint4(cb[0], cb[1], cb[2], cb[3]);
  db[1] = make_uint4(cb[4], cb[5], cb[6], cb[7]);
  if (!live) sa = sb = 0;
  if (ORDER == MX_SCALES_MFMA) {
    const int ca_ = 2 * lane, cb_ = 2 * lane + 1;
    lds_scales[(wave >> 1) * 256 + (((wave & 1) << 5) + (ca_ & 31)) * 4 + (ca_ >> 5)] = (uint8_t)sa;
    lds_scales[(wave >> 1) * 256 + (((wave & 1) << 5) + (cb_ & 31)) * 4 + (cb_ >> 5)] = (uint8_t)sb;
  } else {
    lds_scales[(2 * lane) * 4 + wave] = (uint8_t)sa;
    lds_scales[(2 * lane + 1) * 4 + wave] = (uint8_t)sb;
  }
  __syncthreads();
  store_transposed_tile<ORDER>(lds_codes, lds_scales, r0, c0, rows, cols, codes_t, scales_t,
                               nblk_t, ks_n_t);
}

// ------------------------------------------------------------------------------------
// Tile kernel with 16-byte loads: row-wise, column-wise or both casts of one tile.
// Workgroup tile = 32*WAVES rows x 128 columns.  Wave w owns rows [32w, 32w+32); lane l owns
// columns 8(l&15)..+8 of the eight rows 8(l>>4)+k, so one load instruction fetches four
// 256-byte row segments and a lane keeps an 8x8 patch in 32 registers.
//   row-wise:    the 4 lanes of a DPP quad share a 32-column block (two quad_perm steps);
//                codes leave as 8-byte stores (128 B per row segment).
//   column-wise: the patch gives 8 per-column maxima, completed over the 4 lane groups with
//                two lane exchanges; a column's 8 codes are one 8-byte LDS write into the
//                transposed tile, which leaves as 32*WAVES-byte rows.
// All scale bytes of the tile are staged in LDS in their final order and leave as dwords
// (whole 256-byte groups in MFMA order, padding entries included as zeros).
// ------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t lane_xor(uint32_t v, int lane, int mask) {
  return (uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, (int)v);
}

// Scale byte and narrowing factor of a block whose amax is finite (bits < 0x7F80): the
// general formulas without the NaN / byte-254 cases, which cannot occur here.
template <int MODE>
__device__ __forceinline__ void finite_scale(uint32_t amax_bits, uint32_t& sb, float& mult) {
  const uint32_t e = (MODE == MX_SCALE_RCEIL ? amax_bits + 0x1Fu : amax_bits) >> 7;
  sb = max(e, 8u) - 8u;
  uint32_t bits = (254u - sb) << 23;
  if (sb == 0) bits = (MODE == MX_SCALE_FLOOR) ? 0x7E800000u : 0x3F800000u;
  mult = __uint_as_float(bits);
}

// Two scaled floats -> two codes.  With RCEIL scales of a finite block every |value| is at
// most 448 already, so the clamp is only needed for FLOOR scales.
template <int MODE, bool HIGH>
__device__ __forceinline__ uint32_t cvt2_finite(float lo, float hi, uint32_t old) {
  if (MODE == MX_SCALE_FLOOR) {
    lo = __builtin_amdgcn_fmed3f(lo, -448.0f, 448.0f);
    hi = __builtin_amdgcn_fmed3f(hi, -448.0f, 448.0f);
  }
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, (int)old, HIGH);
}

typedef float v2f_t __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// Quantize one lane's 8x8 patch.  FINITE = no Inf / NaN anywhere in the wave's patches: the
// straight-line path; otherwise the general path with per-block NaN handling and clamps.
template <int MODE, int ORDER, bool ROW, bool COL, int WAVES, bool FINITE>
__device__ __forceinline__ void quantize_patch(u32x4 (&v)[8], const uint32_t (&mr)[8],
                                               const uint32_t (&mc)[4], uint8_t* codes_row,
                                               int64_t cols, int rows_left, bool col_ok,
                                               uint8_t* lds_codes, uint8_t* lds_st,
                                               uint8_t* lds_sr, int wave, int lane, int rl0) {
  constexpr int PITCH = 32 * WAVES + 16;
  const int g = lane >> 4, q = lane & 15;
  if (ROW) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const u32x4 w = v[k];
      uint32_t sb;
      float mult;
      u32x2 out;
      if (FINITE) {
        finite_scale<MODE>(mr[k], sb, mult);
        out.x = cvt2_finite<MODE, true>(bf16_lo(w.y) * mult, bf16_hi(w.y) * mult,
                                        cvt2_finite<MODE, false>(bf16_lo(w.x) * mult,
                                                                 bf16_hi(w.x) * mult, 0));
        out.y = cvt2_finite<MODE, true>(bf16_lo(w.w) * mult, bf16_hi(w.w) * mult,
                                        cvt2_finite<MODE, false>(bf16_lo(w.z) * mult,
                                                                 bf16_hi(w.z) * mult, 0));
      } else {
        sb = scale_byte<MODE>(mr[k]);
        mult = scale_multiplier<MODE>(sb);
        if (sb != 255) {
          out.x = cvt2<true>(w.y, mult, cvt2<false>(w.x, mult, 0));
          out.y = cvt2<true>(w.w, mult, cvt2<false>(w.z, mult, 0));
        } else {
          out.x = nan_block_codes2(w.x) | (nan_block_codes2(w.y) << 16);
          out.y = nan_block_codes2(w.z) | (nan_block_codes2(w.w) << 16);
        }
      }
      if (col_ok && k < rows_left)
        __builtin_nontemporal_store(out, reinterpret_cast<u32x2*>(codes_row + k * cols));
      if ((lane & 3) == 0) {  // rows / columns beyond the matrix were loaded as zeros: byte 0
        const int rl = rl0 + k, bl = q >> 2;
        if (ORDER == MX_SCALES_MFMA)
          lds_sr[(((rl >> 7) * 2 + (bl >> 1)) << 8) + ((((bl & 1) << 5) + (rl & 31)) << 2) +
                 ((rl & 127) >> 5)] = (uint8_t)sb;
        else
          lds_sr[rl * 4 + bl] = (uint8_t)sb;
      }
    }
  }
  if (COL) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t amax = (j & 1) ? (mc[j >> 1] >> 16) : (mc[j >> 1] & 0xFFFFu);
      uint32_t sb;
      float mu;
      u32x2 d;
      if (FINITE) {
        finite_scale<MODE>(amax, sb, mu);
        float f[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
          f[k] = ((j & 1) ? bf16_hi(v[k][j >> 1]) : bf16_lo(v[k][j >> 1])) * mu;
        d.x = cvt2_finite<MODE, true>(f[2], f[3], cvt2_finite<MODE, false>(f[0], f[1], 0));
        d.y = cvt2_finite<MODE, true>(f[6], f[7], cvt2_finite<MODE, false>(f[4], f[5], 0));
      } else {
        sb = scale_byte<MODE>(amax);
        mu = scale_multiplier<MODE>(sb);
        uint32_t e[8];
#pragma unroll
        for (int k = 0; k < 8; ++k)
          e[k] = (j & 1) ? (v[k][j >> 1] >> 16) : (v[k][j >> 1] & 0xFFFFu);
        if (sb != 255) {
          float f[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) f[k] = __uint_as_float(e[k] << 16) * mu;
          d.x = cvt2f<true>(f[2], f[3], cvt2f<false>(f[0], f[1], 0));
          d.y = cvt2f<true>(f[6], f[7], cvt2f<false>(f[4], f[5], 0));
        } else {
          d.x = nan_block_code(e[0]) | (nan_block_code(e[1]) << 8) |
                (nan_block_code(e[2]) << 16) | (nan_block_code(e[3]) << 24);
          d.y = nan_block_code(e[4]) | (nan_block_code(e[5]) << 8) |
                (nan_block_code(e[6]) << 16) | (nan_block_code(e[7]) << 24);
        }
      }
      const int cl = 8 * q + j;
      *reinterpret_cast<u32x2*>(lds_codes + cl * PITCH + wave * 32 + 8 * g) = d;
      if (g == 0) {
        if (ORDER == MX_SCALES_MFMA)
          lds_st[((wave >> 1) << 8) + ((((wave & 1) << 5) + (cl & 31)) << 2) + (cl >> 5)] =
              (uint8_t)sb;
        else
          lds_st[cl * WAVES + wave] = (uint8_t)sb;
      }
    }
  }
}

// Tiles are walked in blocks of BX x BY tiles, down the rows first inside a block, so that
// workgroups running together cover compact regions of the input and of the transposed
// output.  Measured best: wide, flat blocks for the row-wise cast (long contiguous reads and
// writes), narrow, tall ones as soon as the transposed output is written.
#ifndef MX_CAST_ROW_BX
#define MX_CAST_ROW_BX 32
#define MX_CAST_ROW_BY 2
#endif
#ifndef MX_CAST_COL_BX
#define MX_CAST_COL_BX 2
#define MX_CAST_COL_BY 32
#endif
template <bool COL>
struct TileWalk {
  static constexpr uint32_t BX = COL ? MX_CAST_COL_BX : MX_CAST_ROW_BX;
  static constexpr uint32_t BY = COL ? MX_CAST_COL_BY : MX_CAST_ROW_BY;
};

// SwiGLU gate in front of the cast: g = bf16(bf16(silu(a)) * b) per element, each step rounded
// to bf16 like the unfused bf16 tensor ops.  silu follows the float32 formula a / (1 + exp(-a))
// with a correctly rounded quotient (hardware reciprocal plus one Newton step on the
// remainder): the bf16 result equals torch's GPU silu for every one of the 65536 bf16 inputs.
__device__ __forceinline__ float silu_f32(float a) {
  // the hardware reciprocal flushes a denormal result: a denominator beyond 2^100 (a below -69)
  // is scaled into range first; an infinite one gives a * 0 as the float32 division would
  const float d = 1.0f + __expf(-a);
  const float sc = d > 0x1p100f ? 0x1p-32f : 1.0f;
  const float ds = d * sc, r = __builtin_amdgcn_rcpf(ds);
  const float q = a * r;
  const float e = __builtin_fmaf(-q, ds, a);  // NaN for a = +inf, +0 for a = -0: keep q then
  const float q2 = __builtin_islessgreater(e, 0.0f) ? __builtin_fmaf(e, r, q) : q;
  return d == __builtin_inff() ? a * 0.0f : q2 * sc;
}
__device__ __forceinline__ uint32_t swiglu2(uint32_t a2, uint32_t b2) {
  const float s_lo = silu_f32(bf16_lo(a2)), s_hi = silu_f32(bf16_hi(a2));
  const uint32_t s2 = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{s_lo, s_hi}, v2bf_t));
  const float g_lo = bf16_lo(s2) * bf16_lo(b2), g_hi = bf16_hi(s2) * bf16_hi(b2);
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{g_lo, g_hi}, v2bf_t));
}

// Backward of g = silu(a) * b under bf16 autograd, tensor op by tensor op:
//   d/db = bf16(dg * bf16(silu(a)))
//   d/da = silu_backward(bf16(dg * b), a) = bf16(t * s * (1 + a * (1 - s))),  s = 1 / (1 + exp(-a))
// with the float32 formula of the unfused silu backward op.  silu(a) = a / (1 + exp(-a)) shares
// the denominator: a * s corrected by one Newton step on the remainder is the correctly rounded
// quotient (the remainder is NaN or zero for infinite a, an infinite denominator and a = -0:
// the uncorrected product is the answer there).
__device__ __forceinline__ void swiglu_bwd_f32(float dg, float a, float b, float& da, float& db) {
  // exp as the library computes it (the fast hardware path moves a few results in a million by
  // one bf16 step); 1 / d = hardware reciprocal, scaled into its range, plus one Newton step
  const float d = 1.0f + expf(-a);
  const float sc = d > 0x1p100f ? 0x1p-32f : 1.0f;
  const float ds = d * sc, r0 = __builtin_amdgcn_rcpf(ds);
  const float s = d == __builtin_inff() ? 0.0f : __builtin_fmaf(__builtin_fmaf(-r0, ds, 1.0f), r0, r0) * sc;
  const float q = a * s;
  const float rem = __builtin_fmaf(-q, d, a);
  const float silu = __builtin_islessgreater(rem, 0.0f) ? __builtin_fmaf(rem, s, q) : q;
  const uint32_t sb = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{silu, dg * b}, v2bf_t));
  db = dg * bf16_lo(sb);
  const float t = bf16_hi(sb);
  da = t * s * (1.0f + a * (1.0f - s));
}
__device__ __forceinline__ void swiglu_bwd2(uint32_t dg2, uint32_t a2, uint32_t b2, uint32_t& da2,
                                            uint32_t& db2) {
  float da_lo, da_hi, db_lo, db_hi;
  swiglu_bwd_f32(bf16_lo(dg2), bf16_lo(a2), bf16_lo(b2), da_lo, db_lo);
  swiglu_bwd_f32(bf16_hi(dg2), bf16_hi(a2), bf16_hi(b2), da_hi, db_hi);
  da2 = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{da_lo, da_hi}, v2bf_t));
  db2 = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{db_lo, db_hi}, v2bf_t));
}

// 8 rows x 16 bytes of a bf16 matrix per lane; rows past `rows_left` and lanes past the last
// column read as zero.
__device__ __forceinline__ void load_patch(u32x4 (&v)[8], const uint16_t* src, int64_t ld,
                                           bool col_ok, int rows_left) {
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    v[k] = u32x4{0, 0, 0, 0};
    if (col_ok && k < rows_left)
      v[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + k * ld));
  }
}

// Second half of the tile kernel: block maxima, quantization and the stores of one 8 x 8 patch
// per lane.  Ends with every wave past its reads of the shared staging buffers only after the
// caller's next barrier.
template <int MODE, int ORDER, bool ROW, bool COL, int WAVES>
__device__ __forceinline__ void emit_tile(
    u32x4 (&v)[8], uint8_t* __restrict__ codes, uint8_t* __restrict__ scales,
    uint8_t* __restrict__ codes_t, uint8_t* __restrict__ scales_t, uint8_t* lds_codes,
    uint8_t* lds_st, uint8_t* lds_sr, int64_t rows, int64_t cols, int64_t nblk, int64_t ks_n,
    int64_t nblk_t, int64_t ks_n_t, int64_t r0, int64_t c0, int64_t c, int rl0, int rows_left,
    bool col_ok, int tid, int wave, int lane, int64_t ldc, int64_t ldct) {
  // ldc / ldct: bytes between rows of the row-wise / column-wise codes (>= cols / rows)
  constexpr int TR = 32 * WAVES, TC = 128, PITCH = TR + 16;
  // block maxima first: they also tell whether the wave holds any Inf / NaN
  uint32_t mr[8] = {0, 0, 0, 0, 0, 0, 0, 0}, mc[4] = {0, 0, 0, 0};
  uint32_t top = 0;
  if (ROW) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const u32x4 w = v[k];
      uint32_t m = pk_max_u16(pk_max_u16(w.x & 0x7FFF7FFFu, w.y & 0x7FFF7FFFu),
                              pk_max_u16(w.z & 0x7FFF7FFFu, w.w & 0x7FFF7FFFu));
      m = max(m & 0xFFFFu, m >> 16);
      m = max(m, dpp<kQuadXor1>(m));
      m = max(m, dpp<kQuadXor2>(m));
      mr[k] = m;
      top = max(top, m);
    }
  }
  if (COL) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      mc[0] = pk_max_u16(mc[0], v[k].x & 0x7FFF7FFFu);
      mc[1] = pk_max_u16(mc[1], v[k].y & 0x7FFF7FFFu);
      mc[2] = pk_max_u16(mc[2], v[k].z & 0x7FFF7FFFu);
      mc[3] = pk_max_u16(mc[3], v[k].w & 0x7FFF7FFFu);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mc[i] = pk_max_u16(mc[i], lane_xor(mc[i], lane, 16));
      mc[i] = pk_max_u16(mc[i], lane_xor(mc[i], lane, 32));
    }
    if (!ROW) {
      const uint32_t t = pk_max_u16(pk_max_u16(mc[0], mc[1]), pk_max_u16(mc[2], mc[3]));
      top = max(t & 0xFFFFu, t >> 16);
    }
  }
  uint8_t* codes_row = ROW ? codes + (r0 + rl0) * ldc + c : nullptr;
  if (__builtin_amdgcn_ballot_w64(top >= 0x7F80u) == 0)
    quantize_patch<MODE, ORDER, ROW, COL, WAVES, true>(v, mr, mc, codes_row, ldc, rows_left,
                                                       col_ok, lds_codes, lds_st, lds_sr, wave,
                                                       lane, rl0);
  else
    quantize_patch<MODE, ORDER, ROW, COL, WAVES, false>(v, mr, mc, codes_row, ldc, rows_left,
                                                        col_ok, lds_codes, lds_st, lds_sr, wave,
                                                        lane, rl0);
  __syncthreads();

  if (ROW && tid < TR) {
    const uint32_t s4 = *reinterpret_cast<const uint32_t*>(lds_sr + tid * 4);
    if (ORDER == MX_SCALES_MFMA) {
      const int grp = tid >> 6;
      const int64_t rt = (r0 >> 7) + (grp >> 1), ks = (c0 >> 6) + (grp & 1);
      if (rt * 128 < rows && ks < ks_n)
        *reinterpret_cast<uint32_t*>(scales + ((rt * ks_n + ks) << 8) + (tid & 63) * 4) = s4;
    } else if (r0 + tid < rows) {
      const int64_t b0 = c0 >> 5;
      uint8_t* dst = scales + (r0 + tid) * nblk + b0;
      if ((nblk & 3) == 0) {
        if (b0 < nblk) *reinterpret_cast<uint32_t*>(dst) = s4;
      } else {
        for (int w = 0; w < 4 && b0 + w < nblk; ++w) dst[w] = (uint8_t)(s4 >> (8 * w));
      }
    }
  }
  if (COL) {
    constexpr int SEGS = TR / 16;  // 16-byte pieces of one transposed row
    const int seg = tid % SEGS;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int o = p * 32 + tid / SEGS;
      if (c0 + o < cols && r0 + seg * 16 < rows) {
        const u32x4 t = *reinterpret_cast<const u32x4*>(lds_codes + o * PITCH + seg * 16);
#ifdef MX_ABL_COL_UNTRANSPOSED  // timing ablation: the column-wise codes go out as rows of the input
        __builtin_nontemporal_store(
            t, reinterpret_cast<u32x4*>(codes_t + (r0 + o) * cols + c0 + seg * 16));
#else
        __builtin_nontemporal_store(
            t, reinterpret_cast<u32x4*>(codes_t + (c0 + o) * ldct + r0 + seg * 16));
#endif
      }
    }
    if (ORDER == MX_SCALES_MFMA) {
      if (tid < TR) {  // WAVES/2 complete 256-byte groups
        const int64_t ks = (r0 >> 6) + (tid >> 6);
        if (ks < ks_n_t)
          *reinterpret_cast<uint32_t*>(scales_t + (((c0 >> 7) * ks_n_t + ks) << 8) +
                                       (tid & 63) * 4) =
              *reinterpret_cast<const uint32_t*>(lds_st + tid * 4);
      }
    } else if (tid < TC && c0 + tid < cols) {
      const int64_t b0 = r0 >> 5;
      uint8_t* dst = scales_t + (c0 + tid) * nblk_t + b0;
      if ((nblk_t & 3) == 0 && b0 + WAVES <= nblk_t) {
#pragma unroll
        for (int w = 0; w < WAVES / 4; ++w)
          reinterpret_cast<uint32_t*>(dst)[w] =
              *reinterpret_cast<const uint32_t*>(lds_st + tid * WAVES + 4 * w);
      } else {
        for (int w = 0; w < WAVES && b0 + w < nblk_t; ++w) dst[w] = lds_st[tid * WAVES + w];
      }
    }
  }
}

// As load_patch, with the source row of output row r taken from row_idx[r]; an index outside
// [0, src_rows) (the padding slots of a token-group layout hold -1) reads as a row of zeros.
// With row_scale, every element of output row r is multiplied by row_scale[r] in float32 and
// rounded back to bf16 first (the routing-score multiply in front of the experts).
__device__ __forceinline__ uint32_t scale2(uint32_t w, float s) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f_t{bf16_lo(w) * s, bf16_hi(w) * s}, v2bf_t));
}
__device__ __forceinline__ void load_patch_rows(u32x4 (&v)[8], const uint16_t* x, int64_t ld,
                                                int64_t c, const int64_t* row_idx, int64_t src_rows,
                                                const float* row_scale, bool col_ok, int rows_left) {
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    v[k] = u32x4{0, 0, 0, 0};
    if (col_ok && k < rows_left) {
      const int64_t r = row_idx[k];
      if (r >= 0 && r < src_rows) {
        v[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + r * ld + c));
        if (row_scale) {
          const float s = row_scale[k];
          v[k] = u32x4{scale2(v[k].x, s), scale2(v[k].y, s), scale2(v[k].z, s), scale2(v[k].w, s)};
        }
      }
    }
  }
}

// Operands of the tile kernel's variants beyond the plain cast.
struct TileExtras {
  const uint16_t* x3 = nullptr;  // GATE 1, 2: second gate input b; GATE 3: norm weight [cols]
  int64_t ldx3 = 0;
  uint16_t* g_out = nullptr;     // GATE 1: g; GATE 2: stacked da, db (optional)
  const uint16_t* x4 = nullptr;  // GATE 2: dg
  int64_t ldx4 = 0;
  const int64_t* row_idx = nullptr;  // GATHER: source row of every output row
  int64_t src_rows = 0;
  uint32_t batch = 1;  // stacked independent matrices
  const float* row_scale = nullptr;  // GATHER: optional multiplier of every output row; GATE 3: rstd
  int64_t ldc = 0, ldct = 0;  // bytes between rows of the row-wise / column-wise codes (0: dense)
};

// The gate-backward variant is bound by vector ALU work: four workgroups per CU (128 VGPRs).
template <int MODE, int ORDER, bool ROW, bool COL, int WAVES, int GATE, bool GATHER>
__global__ __launch_bounds__(64 * WAVES, GATE == 2 ? 4 : 1) void cast_tile_kernel(
    const uint16_t* __restrict__ x, int64_t rows, int64_t cols, int64_t ldx,
    uint8_t* __restrict__ codes, uint8_t* __restrict__ scales, int64_t nblk, int64_t ks_n,
    uint8_t* __restrict__ codes_t, uint8_t* __restrict__ scales_t, int64_t nblk_t,
    int64_t ks_n_t, int64_t x_bstride, int64_t s_bstride, int64_t st_bstride, uint32_t gx,
    uint32_t gy, TileExtras ex) {
  const uint16_t* __restrict__ x3 = ex.x3;
  const uint16_t* __restrict__ x4 = ex.x4;
  uint16_t* __restrict__ g_out = ex.g_out;
  const int64_t ldx3 = ex.ldx3, ldx4 = ex.ldx4;
  constexpr int TR = 32 * WAVES, TC = 128, PITCH = TR + 16;
  __shared__ __attribute__((aligned(16))) uint8_t lds_codes[COL ? TC * PITCH : 16];
  __shared__ __attribute__((aligned(16))) uint8_t lds_st[COL ? TC * WAVES : 16];
  __shared__ __attribute__((aligned(16))) uint8_t lds_sr[ROW ? TR * 4 : 16];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, q = lane & 15;
  const int rl0 = wave * 32 + 8 * g;  // first tile-local row of this lane

  // a batch of independent [rows, cols] matrices is walked as one stack of gy * batch tile rows
  constexpr uint32_t BX = TileWalk<COL>::BX, BY = TileWalk<COL>::BY;
  const uint32_t gy_all = gy * ex.batch;
  const uint32_t spr = (gx + BX - 1) / BX;
  const uint32_t sup = blockIdx.x / (BX * BY), in = blockIdx.x % (BX * BY);
  const uint32_t bx = (sup % spr) * BX + in / BY;
  const uint32_t by_all = (sup / spr) * BY + in % BY;
  if (bx >= gx || by_all >= gy_all) return;
  const uint32_t bz = by_all / gy, by = by_all - bz * gy;
  const int64_t ldc = ex.ldc ? ex.ldc : cols, ldct = ex.ldct ? ex.ldct : rows;
  x += bz * x_bstride;
  if (ROW) {
    codes += bz * rows * ldc;
    scales += bz * s_bstride;
  }
  if (COL) {
    codes_t += bz * cols * ldct;
    scales_t += bz * st_bstride;
  }

  const int64_t r0 = (int64_t)by * TR, c0 = (int64_t)bx * TC;
  const int64_t c = c0 + 8 * q;
  const bool col_ok = c < cols;
  const int64_t left64 = rows - (r0 + rl0);
  const int rows_left = left64 > 8 ? 8 : (left64 < 0 ? 0 : (int)left64);

  u32x4 v[8];
  if constexpr (GATHER)
    load_patch_rows(v, x, ldx, c, ex.row_idx + r0 + rl0, ex.src_rows,
                    ex.row_scale ? ex.row_scale + r0 + rl0 : nullptr, col_ok, rows_left);
  else
    load_patch(v, x + (r0 + rl0) * ldx + c, ldx, col_ok, rows_left);
  if constexpr (GATE == 1) {  // x = gate input a, x3 = b: quantize g = silu(a) * b
    u32x4 b[8];
    load_patch(b, x3 + (r0 + rl0) * ldx3 + c, ldx3, col_ok, rows_left);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      v[k] = u32x4{swiglu2(v[k].x, b[k].x), swiglu2(v[k].y, b[k].y), swiglu2(v[k].z, b[k].z),
                   swiglu2(v[k].w, b[k].w)};
      if (g_out && col_ok && k < rows_left)
        *reinterpret_cast<u32x4*>(g_out + (r0 + rl0 + k) * cols + c) = v[k];
    }
  }
  if constexpr (GATE == 3) {
    // RMSNorm in front of the cast: y = bf16(w[c] * (rstd[r] * x)), x3 = the norm weight [cols],
    // row_scale = rstd [rows]
    u32x4 wv = u32x4{0, 0, 0, 0};
    if (col_ok) wv = *reinterpret_cast<const u32x4*>(x3 + c);
    const float w8[8] = {bf16_lo(wv.x), bf16_hi(wv.x), bf16_lo(wv.y), bf16_hi(wv.y),
                         bf16_lo(wv.z), bf16_hi(wv.z), bf16_lo(wv.w), bf16_hi(wv.w)};
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (col_ok && k < rows_left) {
        const float rs = ex.row_scale[r0 + rl0 + k];
        const uint32_t d[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(
                     v2f_t{w8[2 * e] * (rs * bf16_lo(d[e])), w8[2 * e + 1] * (rs * bf16_hi(d[e]))}, v2bf_t));
        v[k] = u32x4{o[0], o[1], o[2], o[3]};
        if (g_out) *reinterpret_cast<u32x4*>(g_out + (r0 + rl0 + k) * cols + c) = v[k];
      }
    }
  }
  if constexpr (GATE == 2) {
    // backward of the gate: x = a, x3 = b, x4 = dg; two stacked outputs, d/da then d/db
    u32x4 w[8];
    {
      u32x4 b[8], dg[8];
      load_patch(b, x3 + (r0 + rl0) * ldx3 + c, ldx3, col_ok, rows_left);
      load_patch(dg, x4 + (r0 + rl0) * ldx4 + c, ldx4, col_ok, rows_left);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        uint32_t da[4], db[4];
        swiglu_bwd2(dg[k].x, v[k].x, b[k].x, da[0], db[0]);
        swiglu_bwd2(dg[k].y, v[k].y, b[k].y, da[1], db[1]);
        swiglu_bwd2(dg[k].z, v[k].z, b[k].z, da[2], db[2]);
        swiglu_bwd2(dg[k].w, v[k].w, b[k].w, da[3], db[3]);
        w[k] = u32x4{da[0], da[1], da[2], da[3]};
        v[k] = u32x4{db[0], db[1], db[2], db[3]};
        if (g_out && col_ok && k < rows_left) {
          *reinterpret_cast<u32x4*>(g_out + (r0 + rl0 + k) * cols + c) = w[k];
          *reinterpret_cast<u32x4*>(g_out + (rows + r0 + rl0 + k) * cols + c) = v[k];
        }
      }
    }
    emit_tile<MODE, ORDER, ROW, COL, WAVES>(w, codes, scales, codes_t, scales_t, lds_codes, lds_st,
                                            lds_sr, rows, cols, nblk, ks_n, nblk_t, ks_n_t, r0, c0,
                                            c, rl0, rows_left, col_ok, tid, wave, lane, ldc, ldct);
    __syncthreads();  // the staging buffers are reused by the second output
    if (ROW) {
      codes += rows * ldc;
      scales += s_bstride;
    }
    if (COL) {
      codes_t += cols * ldct;
      scales_t += st_bstride;
    }
  }
  emit_tile<MODE, ORDER, ROW, COL, WAVES>(v, codes, scales, codes_t, scales_t, lds_codes, lds_st,
                                          lds_sr, rows, cols, nblk, ks_n, nblk_t, ks_n_t, r0, c0, c,
                                          rl0, rows_left, col_ok, tid, wave, lane, ldc, ldct);
}

// ------------------------------------------------------------------------------------
// Scale re-layout (pure byte permutation) and its inverse.
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void scale_layout_kernel(const uint8_t* __restrict__ in,
                                                           int64_t rows, int64_t nblk,
                                                           int64_t ks_n, int64_t out_dwords,
                                                           uint32_t* __restrict__ out) {
  const int64_t d = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one dword = (rt, ks, lane)
  if (d >= out_dwords) return;
  const int lane = (int)(d & 63);
  const int64_t g = d >> 6;
  const int64_t ks = g % ks_n, rt = g / ks_n;
  const int64_t blk = ks * 2 + (lane >> 5);
  uint32_t w = 0;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int64_t r = rt * 128 + t * 32 + (lane & 31);
    if (r < rows && blk < nblk) w |= (uint32_t)in[r * nblk + blk] << (8 * t);
  }
  out[d] = w;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, int64_t n,
                                                       uint32_t value) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = value;
}

__global__ __launch_bounds__(256) void scale_unlayout_kernel(const uint8_t* __restrict__ laid,
                                                             int64_t rows, int64_t nblk,
                                                             int64_t ks_n,
                                                             uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * nblk) return;
  const int64_t r = i / nblk, b = i - r * nblk;
  out[i] = laid[mfma_scale_offset(r, b, ks_n)];
}

}  // namespace mx

// ------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------
using namespace mx;

#define MX_DISPATCH_MODE_ORDER(KERNEL, ...)                                                     \
  do {                                                                                          \
    if (scale_mode == MX_SCALE_FLOOR && scale_order == MX_SCALES_ROWMAJOR)                      \
      hipLaunchKernelGGL((KERNEL<MX_SCALE_FLOOR, MX_SCALES_ROWMAJOR>), grid, block, 0, st,      \
                         __VA_ARGS__);                                                          \
    else if (scale_mode == MX_SCALE_FLOOR)                                                      \
      hipLaunchKernelGGL((KERNEL<MX_SCALE_FLOOR, MX_SCALES_MFMA>), grid, block, 0, st,          \
                         __VA_ARGS__);                                                          \
    else if (scale_order == MX_SCALES_ROWMAJOR)                                                 \
      hipLaunchKernelGGL((KERNEL<MX_SCALE_RCEIL, MX_SCALES_ROWMAJOR>), grid, block, 0, st,      \
                         __VA_ARGS__);                                                          \
    else                                                                                        \
      hipLaunchKernelGGL((KERNEL<MX_SCALE_RCEIL, MX_SCALES_MFMA>), grid, block, 0, st,          \
                         __VA_ARGS__);                                                          \
  } while (0)

#ifndef MX_CAST_WAVES
#define MX_CAST_WAVES 4
#endif
#define MX_DISPATCH_TILE(ROW, COL, GATE, GATHER, ...)                                                         \
  do {                                                                                           \
    if (scale_mode == MX_SCALE_FLOOR && scale_order == MX_SCALES_ROWMAJOR)                       \
      hipLaunchKernelGGL(                                                                        \
          (cast_tile_kernel<MX_SCALE_FLOOR, MX_SCALES_ROWMAJOR, ROW, COL, MX_CAST_WAVES, GATE, GATHER>), grid, \
          block, 0, st, __VA_ARGS__);                                                            \
    else if (scale_mode == MX_SCALE_FLOOR)                                                       \
      hipLaunchKernelGGL(                                                                        \
          (cast_tile_kernel<MX_SCALE_FLOOR, MX_SCALES_MFMA, ROW, COL, MX_CAST_WAVES, GATE, GATHER>), grid,     \
          block, 0, st, __VA_ARGS__);                                                            \
    else if (scale_order == MX_SCALES_ROWMAJOR)                                                  \
      hipLaunchKernelGGL(                                                                        \
          (cast_tile_kernel<MX_SCALE_RCEIL, MX_SCALES_ROWMAJOR, ROW, COL, MX_CAST_WAVES, GATE, GATHER>), grid, \
          block, 0, st, __VA_ARGS__);                                                            \
    else                                                                                         \
      hipLaunchKernelGGL(                                                                        \
          (cast_tile_kernel<MX_SCALE_RCEIL, MX_SCALES_MFMA, ROW, COL, MX_CAST_WAVES, GATE, GATHER>), grid,     \
          block, 0, st, __VA_ARGS__);                                                            \
  } while (0)

// The tile kernel loads 16 bytes (8 columns) per lane.
static inline bool tile_ok(const void* x, int64_t cols, int64_t ldx) {
  return ((uintptr_t)x & 15) == 0 && (ldx & 7) == 0 && (cols & 7) == 0;
}
constexpr int kTileRows = 32 * MX_CAST_WAVES;
static inline int64_t tile_grid_x(int64_t gx, int64_t gy, bool col) {
  const int64_t bx = col ? TileWalk<true>::BX : TileWalk<false>::BX;
  const int64_t by = col ? TileWalk<true>::BY : TileWalk<false>::BY;
  return ((gx + bx - 1) / bx) * ((gy + by - 1) / by) * (bx * by);
}
static inline dim3 tile_grid(int64_t gx, int64_t gy, int64_t batch, bool col) {
  return dim3((unsigned)tile_grid_x(gx, gy * batch, col));
}
static inline TileExtras tile_batch(int64_t batch) {
  TileExtras ex;
  ex.batch = (uint32_t)batch;
  return ex;
}

static inline bool bad_enums(int scale_mode, int scale_order) {
  return (scale_mode != MX_SCALE_FLOOR && scale_mode != MX_SCALE_RCEIL) ||
         (scale_order != MX_SCALES_ROWMAJOR && scale_order != MX_SCALES_MFMA);
}
static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
// The row-wise kernels write one scale byte per block and never touch the padding of an
// MFMA-order buffer; when the matrix does not fill whole (128-row, 2-block) groups the buffer
// is cleared first so the padding reads as 2^-127 and never as NaN.  (A fill kernel, not a
// memset node, so the call stays safe under stream capture.)
static inline void clear_mfma_padding(uint8_t* scales, int64_t rows, int64_t nblk, int order,
                                      hipStream_t st) {
  if (order != MX_SCALES_MFMA || ((rows & 127) == 0 && (nblk & 1) == 0)) return;
  const int64_t n = mfma_scale_bytes(rows, nblk) / 4;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                     (uint32_t*)scales, n, 0u);
}

extern "C" int mx_cast_dim0(const void* x, int64_t rows, int64_t cols, int64_t ldx,
                            uint8_t* codes, uint8_t* scales, int scale_mode, int scale_order,
                            void* stream) {
  if (rows < 0 || cols < 0 || ldx < cols || bad_enums(scale_mode, scale_order))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (!x || !codes || !scales) return MX_ERR_INVALID_ARG;
  if (cols % 32 || ldx % 8 || ((uintptr_t)x & 15) || ((uintptr_t)codes & 7))
    return MX_ERR_ALIGNMENT;
  const int64_t cpr = cols / 8;
  if (cpr > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  const int64_t total = rows * cpr;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t per_block = kDim0Threads * kDim0Unroll;
  const int64_t nblocks = (total + per_block - 1) / per_block;
  if (nblocks > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  dim3 grid((unsigned)nblocks), block(kDim0Threads);
  hipStream_t st = (hipStream_t)stream;
  if (scale_order == MX_SCALES_MFMA && ((uintptr_t)scales & 3)) return MX_ERR_ALIGNMENT;
  const int64_t tgx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  if (scale_order == MX_SCALES_MFMA && tile_grid_x(tgx, tgy, false) <= 0x7FFFFFFF) {
    // scattered scale bytes cost more than the tiled read: stage them through LDS
    dim3 grid = tile_grid(tgx, tgy, 1, false), block(64 * MX_CAST_WAVES);
    MX_DISPATCH_TILE(true, false, 0, false, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk,
                     ks_n, (uint8_t*)nullptr, (uint8_t*)nullptr, (int64_t)0, (int64_t)0, (int64_t)0,
                     (int64_t)0, (int64_t)0, (uint32_t)tgx, (uint32_t)tgy, TileExtras{});
    return launch_status();
  }
  clear_mfma_padding(scales, rows, nblk, scale_order, st);
  MX_DISPATCH_MODE_ORDER(cast_dim0_kernel, (const uint16_t*)x, ldx, (uint32_t)cpr, total, codes,
                         scales, nblk, ks_n);
  return launch_status();
}

static inline int64_t scale_bytes(int64_t rows, int64_t nblk, int order) {
  return order == MX_SCALES_MFMA ? mfma_scale_bytes(rows, nblk) : rows * nblk;
}

extern "C" int mx_cast_dim1_batched(const void* x, int64_t batch, int64_t rows, int64_t cols,
                                    int64_t ldx, uint8_t* codes_t, uint8_t* scales_t,
                                    int scale_mode, int scale_order, void* stream) {
  if (batch < 0 || rows < 0 || cols < 0 || ldx < cols || bad_enums(scale_mode, scale_order))
    return MX_ERR_INVALID_ARG;
  if (batch == 0 || rows == 0 || cols == 0) return MX_OK;
  if (!x || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 2 || ldx % 2 || ((uintptr_t)x & 3) || ((uintptr_t)codes_t & 15) ||
      ((uintptr_t)scales_t & 3))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t st_b = scale_bytes(cols, nblk_t, scale_order);
  if (batch > 1 && ((rows * cols) % 16 || st_b % 4)) return MX_ERR_ALIGNMENT;
  const int64_t gx = (cols + kT - 1) / kT, gy = (rows + kT - 1) / kT;
  if (gy > 65535 || batch > 65535 || gx > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int64_t tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_ok(x, cols, ldx) && tile_grid_x(gx, tgy * batch, true) <= 0x7FFFFFFF) {
    dim3 grid = tile_grid(gx, tgy, batch, true), block(64 * MX_CAST_WAVES);
    MX_DISPATCH_TILE(false, true, 0, false, (const uint16_t*)x, rows, cols, ldx, (uint8_t*)nullptr,
                     (uint8_t*)nullptr, (int64_t)0, (int64_t)0, codes_t, scales_t, nblk_t, ks_n_t,
                     rows * ldx, (int64_t)0, st_b, (uint32_t)gx, (uint32_t)tgy,
                     tile_batch(batch));
    return launch_status();
  }
  dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch), block(256);
  MX_DISPATCH_MODE_ORDER(cast_dim1_kernel, (const uint16_t*)x, rows, cols, ldx, codes_t,
                         scales_t, nblk_t, ks_n_t, rows * ldx, st_b);
  return launch_status();
}

extern "C" int mx_cast_dim1(const void* x, int64_t rows, int64_t cols, int64_t ldx,
                            uint8_t* codes_t, uint8_t* scales_t, int scale_mode,
                            int scale_order, void* stream) {
  return mx_cast_dim1_batched(x, 1, rows, cols, ldx, codes_t, scales_t, scale_mode,
                              scale_order, stream);
}

extern "C" int mx_cast_dim0_dim1_batched(const void* x, int64_t batch, int64_t rows,
                                         int64_t cols, int64_t ldx, uint8_t* codes,
                                         uint8_t* scales, uint8_t* codes_t, uint8_t* scales_t,
                                         int scale_mode, int scale_order, void* stream) {
  if (batch < 0 || rows < 0 || cols < 0 || ldx < cols || bad_enums(scale_mode, scale_order))
    return MX_ERR_INVALID_ARG;
  if (batch == 0 || rows == 0 || cols == 0) return MX_OK;
  if (!x || !codes || !scales || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 32 || ldx % 2 || ((uintptr_t)x & 3) || ((uintptr_t)codes & 1) ||
      ((uintptr_t)codes_t & 15) || ((uintptr_t)scales_t & 3))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t s_b = scale_bytes(rows, nblk, scale_order);
  const int64_t st_b = scale_bytes(cols, nblk_t, scale_order);
  const int64_t gx = (cols + kT - 1) / kT, gy = (rows + kT - 1) / kT;
  if (gy > 65535 || batch > 65535 || gx > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  if (scale_order == MX_SCALES_MFMA && ((uintptr_t)scales & 3)) return MX_ERR_ALIGNMENT;
  const int64_t tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_ok(x, cols, ldx) && ((uintptr_t)codes & 7) == 0 && ((uintptr_t)scales & 3) == 0 &&
      tile_grid_x(gx, tgy * batch, true) <= 0x7FFFFFFF) {
    dim3 grid = tile_grid(gx, tgy, batch, true), block(64 * MX_CAST_WAVES);
    MX_DISPATCH_TILE(true, true, 0, false, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk,
                     ks_n, codes_t, scales_t, nblk_t, ks_n_t, rows * ldx, s_b, st_b, (uint32_t)gx,
                     (uint32_t)tgy, tile_batch(batch));
    return launch_status();
  }
  dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch), block(256);
  if (scale_order == MX_SCALES_MFMA && ((rows & 127) || (nblk & 1))) {
    // padding of every batch entry's row-wise scale block must read as zero
    const int64_t n = batch * s_b / 4;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (uint32_t*)scales, n, 0u);
  }
  MX_DISPATCH_MODE_ORDER(cast_dim0_dim1_kernel, (const uint16_t*)x, rows, cols, ldx, codes,
                         scales, nblk, ks_n, codes_t, scales_t, nblk_t, ks_n_t, rows * ldx, s_b,
                         st_b);
  return launch_status();
}

// The fused cast with a row pitch for each of its code outputs (scales are laid out as ever): rows of
// codes that start at different positions within a 4 KB span of addresses spread the lines a GEMM
// fetches together (the same K block of many rows) over the channels of the L2.
extern "C" int mx_cast_dim0_dim1_ld(const void* x, int64_t rows, int64_t cols, int64_t ldx,
                                    uint8_t* codes, int64_t ld_codes, uint8_t* scales,
                                    uint8_t* codes_t, int64_t ld_codes_t, uint8_t* scales_t,
                                    int scale_mode, int scale_order, void* stream) {
  if (rows < 0 || cols < 0 || ldx < cols || ld_codes < cols || ld_codes_t < rows || bad_enums(scale_mode, scale_order))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (ld_codes == cols && ld_codes_t == rows)
    return mx_cast_dim0_dim1_batched(x, 1, rows, cols, ldx, codes, scales, codes_t, scales_t, scale_mode,
                                     scale_order, stream);
  if (!x || !codes || !scales || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 32 || ld_codes % 16 || ld_codes_t % 16 || ((uintptr_t)codes & 15) ||
      ((uintptr_t)codes_t & 15) || ((uintptr_t)scales & 3) || ((uintptr_t)scales_t & 3))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t gx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  // only the tile kernel knows pitches: inputs it does not take are the caller's dense cast
  if (!tile_ok(x, cols, ldx) || tile_grid_x(gx, tgy, true) > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid = tile_grid(gx, tgy, 1, true), block(64 * MX_CAST_WAVES);
  TileExtras ex = tile_batch(1);
  ex.ldc = ld_codes;
  ex.ldct = ld_codes_t;
  MX_DISPATCH_TILE(true, true, 0, false, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk, ks_n,
                   codes_t, scales_t, nblk_t, ks_n_t, rows * ldx, scale_bytes(rows, nblk, scale_order),
                   scale_bytes(cols, nblk_t, scale_order), (uint32_t)gx, (uint32_t)tgy, ex);
  return launch_status();
}

extern "C" int mx_cast_dim0_dim1(const void* x, int64_t rows, int64_t cols, int64_t ldx,
                                 uint8_t* codes, uint8_t* scales, uint8_t* codes_t,
                                 uint8_t* scales_t, int scale_mode, int scale_order,
                                 void* stream) {
  return mx_cast_dim0_dim1_batched(x, 1, rows, cols, ldx, codes, scales, codes_t, scales_t,
                                   scale_mode, scale_order, stream);
}

extern "C" int64_t mx_scales_mfma_bytes(int64_t rows, int64_t nblk) {
  if (rows < 0 || nblk < 0) return -1;
  return mfma_scale_bytes(rows, nblk);
}

extern "C" int mx_scale_layout(const uint8_t* scales, int64_t rows, int64_t nblk, uint8_t* out,
                               void* stream) {
  if (rows < 0 || nblk < 0) return MX_ERR_INVALID_ARG;
  if (rows == 0 || nblk == 0) return MX_OK;
  if (!scales || !out) return MX_ERR_INVALID_ARG;
  if ((uintptr_t)out & 3) return MX_ERR_ALIGNMENT;
  const int64_t ks_n = (nblk + 1) / 2;
  const int64_t dwords = mx_scales_mfma_bytes(rows, nblk) / 4;
  hipLaunchKernelGGL(scale_layout_kernel, dim3((unsigned)((dwords + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, scales, rows, nblk, ks_n, dwords, (uint32_t*)out);
  return launch_status();
}

extern "C" int mx_scale_unlayout(const uint8_t* laid, int64_t rows, int64_t nblk, uint8_t* out,
                                 void* stream) {
  if (rows < 0 || nblk < 0) return MX_ERR_INVALID_ARG;
  if (rows == 0 || nblk == 0) return MX_OK;
  if (!laid || !out) return MX_ERR_INVALID_ARG;
  const int64_t ks_n = (nblk + 1) / 2;
  const int64_t n = rows * nblk;
  hipLaunchKernelGGL(scale_unlayout_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, laid, rows, nblk, ks_n, out);
  return launch_status();
}

extern "C" int mx_cast_rows_gathered(const void* x, const int64_t* row_index,
                                     const float* row_scale, int64_t src_rows,
                                     int64_t rows, int64_t cols, int64_t ldx, uint8_t* codes,
                                     uint8_t* scales, uint8_t* codes_t, uint8_t* scales_t,
                                     int scale_mode, int scale_order, void* stream) {
  if (rows < 0 || cols < 0 || src_rows < 0 || ldx < cols || bad_enums(scale_mode, scale_order))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (!x || !row_index || !codes || !scales || (!codes_t) != (!scales_t)) return MX_ERR_INVALID_ARG;
  if (cols % 32 || ldx % 8 || ((uintptr_t)x & 15) || ((uintptr_t)codes & 7) ||
      ((uintptr_t)scales & 3) || ((uintptr_t)row_index & 7) || ((uintptr_t)row_scale & 3))
    return MX_ERR_ALIGNMENT;
  if (codes_t && (rows % 32 || ((uintptr_t)codes_t & 15) || ((uintptr_t)scales_t & 3)))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t gx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_grid_x(gx, tgy, codes_t != nullptr) > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid = tile_grid(gx, tgy, 1, codes_t != nullptr), block(64 * MX_CAST_WAVES);
  TileExtras ex;
  ex.row_idx = row_index;
  ex.src_rows = src_rows;
  ex.row_scale = row_scale;
  if (codes_t)
    MX_DISPATCH_TILE(true, true, 0, true, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk,
                     ks_n, codes_t, scales_t, nblk_t, ks_n_t, (int64_t)0, (int64_t)0, (int64_t)0,
                     (uint32_t)gx, (uint32_t)tgy, ex);
  else
    MX_DISPATCH_TILE(true, false, 0, true, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk,
                     ks_n, (uint8_t*)nullptr, (uint8_t*)nullptr, (int64_t)0, (int64_t)0, (int64_t)0,
                     (int64_t)0, (int64_t)0, (uint32_t)gx, (uint32_t)tgy, ex);
  return launch_status();
}

namespace mx {
// rstd[r] = 1 / sqrt(mean_c x[r, c]^2 + eps) in float32; one wave per row, lanes stride over
// 8-column chunks, butterfly over the 64 lanes.
__global__ __launch_bounds__(256) void rms_rstd_kernel(const uint16_t* __restrict__ x, int64_t rows,
                                                       int64_t cols, int64_t ldx, float eps,
                                                       float* __restrict__ rstd) {
  const int lane = threadIdx.x & 63;
  const int64_t r = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  if (r >= rows) return;
  const uint16_t* row = x + r * ldx;
  float acc = 0.f;
  for (int64_t c = lane * 8; c < cols; c += 64 * 8) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(row + c);
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = bf16_lo(d[e]), hi = bf16_hi(d[e]);
      acc = __builtin_fmaf(lo, lo, acc);
      acc = __builtin_fmaf(hi, hi, acc);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) rstd[r] = rsqrtf(acc / (float)cols + eps);
}
}  // namespace mx

// A code pitch of 0 stands for dense rows; a pitch must keep every row 16-byte aligned.
static inline bool bad_pitches(int64_t ld_codes, int64_t cols, int64_t ld_codes_t, int64_t rows) {
  return (ld_codes && ld_codes < cols) || (ld_codes_t && ld_codes_t < rows);
}
static inline bool misaligned_pitches(int64_t ld_codes, int64_t ld_codes_t, const void* codes) {
  return (ld_codes % 16) || (ld_codes_t % 16) || ((ld_codes || ld_codes_t) && ((uintptr_t)codes & 15));
}

extern "C" int mx_rmsnorm_cast_dim0_dim1_ld(const void* x, const void* weight, float eps, int64_t rows,
                                            int64_t cols, int64_t ldx, float* rstd, void* y,
                                            uint8_t* codes, int64_t ld_codes, uint8_t* scales,
                                            uint8_t* codes_t, int64_t ld_codes_t, uint8_t* scales_t,
                                            int scale_mode, int scale_order, void* stream) {
  if (rows < 0 || cols < 0 || ldx < cols || bad_enums(scale_mode, scale_order) ||
      bad_pitches(ld_codes, cols, ld_codes_t, rows))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (misaligned_pitches(ld_codes, ld_codes_t, codes)) return MX_ERR_ALIGNMENT;
  if (!x || !weight || !rstd || !codes || !scales || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 32 || ldx % 8 || ((uintptr_t)x & 15) || ((uintptr_t)weight & 15) ||
      ((uintptr_t)y & 15) || ((uintptr_t)rstd & 3) || ((uintptr_t)codes & 7) ||
      ((uintptr_t)codes_t & 15) || ((uintptr_t)scales & 3) || ((uintptr_t)scales_t & 3))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t gx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_grid_x(gx, tgy, true) > 0x7FFFFFFF || (rows + 3) / 4 > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(rms_rstd_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st,
                     (const uint16_t*)x, rows, cols, ldx, eps, rstd);
  dim3 grid = tile_grid(gx, tgy, 1, true), block(64 * MX_CAST_WAVES);
  TileExtras ex;
  ex.x3 = (const uint16_t*)weight;
  ex.g_out = (uint16_t*)y;
  ex.row_scale = rstd;
  ex.ldc = ld_codes;
  ex.ldct = ld_codes_t;
  MX_DISPATCH_TILE(true, true, 3, false, (const uint16_t*)x, rows, cols, ldx, codes, scales, nblk, ks_n,
                   codes_t, scales_t, nblk_t, ks_n_t, (int64_t)0, (int64_t)0, (int64_t)0,
                   (uint32_t)gx, (uint32_t)tgy, ex);
  return launch_status();
}

extern "C" int mx_rmsnorm_cast_dim0_dim1(const void* x, const void* weight, float eps, int64_t rows,
                                         int64_t cols, int64_t ldx, float* rstd, void* y,
                                         uint8_t* codes, uint8_t* scales, uint8_t* codes_t,
                                         uint8_t* scales_t, int scale_mode, int scale_order,
                                         void* stream) {
  return mx_rmsnorm_cast_dim0_dim1_ld(x, weight, eps, rows, cols, ldx, rstd, y, codes, 0, scales, codes_t, 0,
                                      scales_t, scale_mode, scale_order, stream);
}

extern "C" int mx_swiglu_cast_dim0_dim1_ld(const void* a, const void* b, int64_t rows, int64_t cols,
                                           int64_t lda, int64_t ldb, uint8_t* codes, int64_t ld_codes,
                                           uint8_t* scales, uint8_t* codes_t, int64_t ld_codes_t,
                                           uint8_t* scales_t, void* g, int scale_mode,
                                           int scale_order, void* stream) {
  if (rows < 0 || cols < 0 || lda < cols || ldb < cols || bad_enums(scale_mode, scale_order) ||
      bad_pitches(ld_codes, cols, ld_codes_t, rows))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (misaligned_pitches(ld_codes, ld_codes_t, codes)) return MX_ERR_ALIGNMENT;
  if (!a || !b || !codes || !scales || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 32 || lda % 8 || ldb % 8 || ((uintptr_t)a & 15) || ((uintptr_t)b & 15) ||
      ((uintptr_t)codes & 7) || ((uintptr_t)codes_t & 15) || ((uintptr_t)scales & 3) ||
      ((uintptr_t)scales_t & 3) || ((uintptr_t)g & 15))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  const int64_t gx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_grid_x(gx, tgy, true) > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid = tile_grid(gx, tgy, 1, true), block(64 * MX_CAST_WAVES);
  TileExtras ex{(const uint16_t*)b, ldb, (uint16_t*)g, nullptr, 0, nullptr, 0};
  ex.ldc = ld_codes;
  ex.ldct = ld_codes_t;
  MX_DISPATCH_TILE(true, true, 1, false, (const uint16_t*)a, rows, cols, lda, codes, scales, nblk, ks_n,
                   codes_t, scales_t, nblk_t, ks_n_t, (int64_t)0, (int64_t)0, (int64_t)0,
                   (uint32_t)gx, (uint32_t)tgy, ex);
  return launch_status();
}

extern "C" int mx_swiglu_cast_dim0_dim1(const void* a, const void* b, int64_t rows, int64_t cols,
                                        int64_t lda, int64_t ldb, uint8_t* codes, uint8_t* scales,
                                        uint8_t* codes_t, uint8_t* scales_t, void* g,
                                        int scale_mode, int scale_order, void* stream) {
  return mx_swiglu_cast_dim0_dim1_ld(a, b, rows, cols, lda, ldb, codes, 0, scales, codes_t, 0, scales_t, g,
                                     scale_mode, scale_order, stream);
}

extern "C" int mx_swiglu_bwd_cast_dim0_dim1_ld(const void* dg, const void* a, const void* b,
                                               int64_t rows, int64_t cols, int64_t lddg, int64_t lda,
                                               int64_t ldb, uint8_t* codes, int64_t ld_codes,
                                               uint8_t* scales, uint8_t* codes_t, int64_t ld_codes_t,
                                               uint8_t* scales_t, void* dab, int scale_mode,
                                               int scale_order, void* stream) {
  if (rows < 0 || cols < 0 || lddg < cols || lda < cols || ldb < cols ||
      bad_enums(scale_mode, scale_order) || bad_pitches(ld_codes, cols, ld_codes_t, rows))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (misaligned_pitches(ld_codes, ld_codes_t, codes)) return MX_ERR_ALIGNMENT;
  if (!dg || !a || !b || !codes || !scales || !codes_t || !scales_t) return MX_ERR_INVALID_ARG;
  if (rows % 32 || cols % 32 || lddg % 8 || lda % 8 || ldb % 8 || ((uintptr_t)dg & 15) ||
      ((uintptr_t)a & 15) || ((uintptr_t)b & 15) || ((uintptr_t)codes & 7) ||
      ((uintptr_t)codes_t & 15) || ((uintptr_t)scales & 3) || ((uintptr_t)scales_t & 3) ||
      ((uintptr_t)dab & 15))
    return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t nblk_t = rows / 32, ks_n_t = (nblk_t + 1) / 2;
  // the second output follows the first: one matrix of codes and one scale buffer further on
  const int64_t s_b = scale_bytes(rows, nblk, scale_order);
  const int64_t st_b = scale_bytes(cols, nblk_t, scale_order);
  const int64_t gx = (cols + kT - 1) / kT, tgy = (rows + kTileRows - 1) / kTileRows;
  if (tile_grid_x(gx, tgy, true) > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid = tile_grid(gx, tgy, 1, true), block(64 * MX_CAST_WAVES);
  TileExtras ex{(const uint16_t*)b, ldb, (uint16_t*)dab, (const uint16_t*)dg, lddg, nullptr, 0};
  ex.ldc = ld_codes;
  ex.ldct = ld_codes_t;
  MX_DISPATCH_TILE(true, true, 2, false, (const uint16_t*)a, rows, cols, lda, codes, scales, nblk, ks_n,
                   codes_t, scales_t, nblk_t, ks_n_t, (int64_t)0, s_b, st_b, (uint32_t)gx,
                   (uint32_t)tgy, ex);
  return launch_status();
}

extern "C" int mx_swiglu_bwd_cast_dim0_dim1(const void* dg, const void* a, const void* b,
                                            int64_t rows, int64_t cols, int64_t lddg, int64_t lda,
                                            int64_t ldb, uint8_t* codes, uint8_t* scales,
                                            uint8_t* codes_t, uint8_t* scales_t, void* dab,
                                            int scale_mode, int scale_order, void* stream) {
  return mx_swiglu_bwd_cast_dim0_dim1_ld(dg, a, b, rows, cols, lddg, lda, ldb, codes, 0, scales, codes_t, 0,
                                         scales_t, dab, scale_mode, scale_order, stream);
}
