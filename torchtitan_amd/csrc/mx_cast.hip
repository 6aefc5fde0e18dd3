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
  dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch), block(256);
  hipStream_t st = (hipStream_t)stream;
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
  dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (scale_order == MX_SCALES_MFMA && ((uintptr_t)scales & 3)) return MX_ERR_ALIGNMENT;
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
