// One workgroup's MXFP8 "NT" GEMM tile on gfx950: D[BM,BN] = deq(A)[BM,K] * deq(B)[BN,K]^T.
//
// 256 threads = 4 waves in a 2x2 grid, each wave owns a (BM/2)x(BN/2) patch made of 16x16
// accumulators fed by v_mfma_scale_f32_16x16x128_f8f6f4: per lane 2 x 16 K bytes of one row
// plus the E8M0 scale of one 32-element MX block, so the block scaling is done by the matrix
// core and the products are exact.
//
// Data movement per 128-deep K step:
//   * codes: buffer_load_dwordx4 ... lds (global -> LDS without touching VGPRs), two LDS
//     stages, one barrier per step.  A load instruction moves 8 rows x 128 B; inside LDS the
//     16-byte chunk c of row r sits at chunk position c ^ ((r & 2) | ((r & 8) >> 1)) so every
//     16-lane pass of a fragment read hits 16 different bank groups.
//   * scales: straight from global into VGPRs, either two dwords per lane per 128 rows from a
//     buffer in MFMA order, or one byte per lane per 16 rows from a row-major matrix.
//   * out-of-range rows and K tails read as zero through the buffer descriptor's bounds.
#pragma once

#include <type_traits>

#include "mx_common.h"

namespace mx {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void_t;

constexpr int kBK = 128;

template <int I, int End, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < End) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, End>(f);
  }
}

// One GEMM operand as the tile sees it.
struct Operand {
  const uint8_t* codes;    // first row of this tile, column 0
  int64_t ld;              // row stride in bytes (= elements)
  int64_t rows_valid;      // rows of the tile that exist (may exceed the tile height)
  const uint8_t* scales;   // MFMA order: group of the tile's first 128 rows, K-step 0
                           // row-major:  scale of (tile's first row, block 0)
  int64_t scale_stride;    // MFMA order: 64-deep K-steps per 128-row group; row-major: nblk
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0x7FFFFFFFll ? 0x7FFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// two floats -> two bf16 (round to nearest even) in one dword: v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{lo, hi}, v2bf));
}

template <int BM, int BN, bool A_ROWMAJOR, bool B_ROWMAJOR>
struct GemmTile {
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static constexpr int A_BYTES = BM * kBK, B_BYTES = BN * kBK, STAGE = A_BYTES + B_BYTES;
  static constexpr int A_UNITS = BM / 32, B_UNITS = BN / 32;  // 1 KB load units per wave
  static constexpr int SA = A_ROWMAJOR ? TM : 2;  // scale registers per step (MFMA order:
  static constexpr int SB = B_ROWMAJOR ? TN : 2;  // one dword for even, one for odd sub-tiles)
  static constexpr int kLdsBytes = 2 * STAGE;
  static_assert((WM == 64 || WM == 128) && (WN == 64 || WN == 128), "wave tile is 64 or 128");

  // k_begin/k_end: contraction range in elements (multiples of 32); for MFMA-order scales
  // k_begin must be 0.  d points at the tile's first output element.
  __device__ __forceinline__ static void run(uint8_t* smem, const Operand& A, const Operand& B, int64_t k_begin,
                             int64_t k_end, uint16_t* __restrict__ d, int64_t ldd) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 15, lj = lane >> 4;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(A.codes, A.rows_valid * A.ld);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(B.codes, B.rows_valid * B.ld);

    // global -> LDS: lane l of a load unit (8 rows) fetches row l/8 and the logical chunk that
    // belongs at physical chunk l%8 of that row: c = (l%8) ^ swz(row), swz(r) = (r&2) | ((r&8)>>1)
    const uint32_t lrow = lane >> 3;
    const uint32_t chunk_even = (lane & 7) ^ (lrow & 2);  // even units; odd units flip bit 2
    const uint32_t va_even = lrow * (uint32_t)A.ld + chunk_even * 16;
    const uint32_t va_odd = lrow * (uint32_t)A.ld + (chunk_even ^ 4) * 16;
    const uint32_t vb_even = lrow * (uint32_t)B.ld + chunk_even * 16;
    const uint32_t vb_odd = lrow * (uint32_t)B.ld + (chunk_even ^ 4) * 16;

    // LDS -> VGPR.  Operand layout of the 16x16x128 f8 MFMA (measured on gfx950): lane
    // (li, lj) holds row li, K bytes [16*lj, 16*lj+16) in its first four registers and
    // [64+16*lj, 64+16*lj+16) in the last four, i.e. 16-byte chunks lj and lj+4; the scale
    // of K-block b (bytes [32b, 32b+32)) is taken from lane group b.
    // The swizzle makes ds_read_b128 conflict-free: the LDS serves a b128 read in four passes
    // of 16 lanes, and (measured) the lanes of a pass are {0-3, 12-15, 20-23, 24-27} and
    // {4-11, 16-19, 28-31} of each half-wave, not 16 consecutive lanes.
    const uint32_t sw = (li & 2) | ((li & 8) >> 1);
    const uint32_t fa0 = (wm * WM + li) * kBK + ((lj ^ sw) << 4);
    const uint32_t fa1 = (wm * WM + li) * kBK + (((lj + 4) ^ sw) << 4);
    const uint32_t fb0 = A_BYTES + (wn * WN + li) * kBK + ((lj ^ sw) << 4);
    const uint32_t fb1 = A_BYTES + (wn * WN + li) * kBK + (((lj + 4) ^ sw) << 4);

    v4f acc[TM][TN];
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
      for (int n = 0; n < TN; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    const int64_t nsteps = (k_end - k_begin + kBK - 1) / kBK;

    auto issue_loads = [&](int stage, int64_t k0) {
      // K tail: lanes whose 16-byte chunk starts at or beyond k_end read out of range (zero)
      const bool tail = k0 + kBK > k_end;
      const uint32_t kk = (uint32_t)k0;
      uint8_t* sbase = smem + stage * STAGE;
#pragma unroll
      for (int q = 0; q < A_UNITS; ++q) {
        const int unit = wave * A_UNITS + q;
        uint32_t v = (q & 1) ? va_odd : va_even;
        if (tail) {
          const uint32_t c = (q & 1) ? (chunk_even ^ 4) : chunk_even;
          if (k0 + c * 16 >= k_end) v = 0x80000000u;
        }
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_a, (lds_void_t*)(sbase + unit * 1024), 16, v,
            (uint32_t)(unit * 8) * (uint32_t)A.ld + kk, 0, 0);
      }
#pragma unroll
      for (int q = 0; q < B_UNITS; ++q) {
        const int unit = wave * B_UNITS + q;
        uint32_t v = (q & 1) ? vb_odd : vb_even;
        if (tail) {
          const uint32_t c = (q & 1) ? (chunk_even ^ 4) : chunk_even;
          if (k0 + c * 16 >= k_end) v = 0x80000000u;
        }
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrc_b, (lds_void_t*)(sbase + A_BYTES + unit * 1024), 16, v,
            (uint32_t)(unit * 8) * (uint32_t)B.ld + kk, 0, 0);
      }
    };

    // scale fetch for the K step starting at k0: buffer loads with a per-lane offset that is
    // fixed for the whole kernel and a scalar offset per (group, step); rows or 64-row groups
    // past the end of the operand read as zero through the descriptor's bounds
    const __amdgpu_buffer_rsrc_t rsrc_sa = make_rsrc(
        A.scales, A_ROWMAJOR ? A.rows_valid * A.scale_stride
                             : ((A.rows_valid + 127) >> 7) * A.scale_stride * 256);
    const __amdgpu_buffer_rsrc_t rsrc_sb = make_rsrc(
        B.scales, B_ROWMAJOR ? B.rows_valid * B.scale_stride
                             : ((B.rows_valid + 127) >> 7) * B.scale_stride * 256);
    // MFMA order (groups of 128 rows x 2 blocks, lane = 32 * (block & 1) + (row & 31), byte =
    // (row & 127) / 32): lane (li, lj) of 16-row sub-tile m needs row m*16 + li, block lj of
    // the 128-deep step, i.e. group step 2*ks + (lj >> 1), lane 32*(lj & 1) + 16*(m & 1) + li,
    // byte (m >> 1) -- one dword for the even sub-tiles and one for the odd ones.
    const uint32_t v_mfma = (uint32_t)(((lj & 1) * 32 + li) * 4 + (lj >> 1) * 256);
    const uint32_t vsa = A_ROWMAJOR ? (uint32_t)li * (uint32_t)A.scale_stride + lj : v_mfma;
    const uint32_t vsb = B_ROWMAJOR ? (uint32_t)li * (uint32_t)B.scale_stride + lj : v_mfma;
    const uint32_t sa_stride = (uint32_t)A.scale_stride, sb_stride = (uint32_t)B.scale_stride;
    // a 64-row wave tile sits in one half of its 128-row group: bring its bytes down
    const uint32_t sh_a = (WM == 64) ? 16u * wm : 0u, sh_b = (WN == 64) ? 16u * wn : 0u;

    auto load_scales_a = [&](uint32_t (&s)[SA], int64_t k0) {
      const bool valid = k0 + 32 * lj < k_end;
      if constexpr (A_ROWMAJOR) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
          const uint32_t so = (uint32_t)(wm * WM + m * 16) * sa_stride + (uint32_t)(k0 >> 5);
          const uint32_t b = __builtin_amdgcn_raw_buffer_load_b8(rsrc_sa, valid ? vsa : 0x80000000u, so, 0);
          s[m] = b;
        }
      } else {
        const uint32_t so = ((uint32_t)(wm * WM / 128) * sa_stride + (uint32_t)(k0 >> 6)) * 256;
#pragma unroll
        for (int g = 0; g < 2; ++g)
          s[g] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sa, valid ? vsa + g * 64 : 0x80000000u, so, 0) >> sh_a;
      }
    };
    auto load_scales_b = [&](uint32_t (&s)[SB], int64_t k0) {
      const bool valid = k0 + 32 * lj < k_end;
      if constexpr (B_ROWMAJOR) {
#pragma unroll
        for (int n = 0; n < TN; ++n) {
          const uint32_t so = (uint32_t)(wn * WN + n * 16) * sb_stride + (uint32_t)(k0 >> 5);
          const uint32_t b = __builtin_amdgcn_raw_buffer_load_b8(rsrc_sb, valid ? vsb : 0x80000000u, so, 0);
          s[n] = b;
        }
      } else {
        const uint32_t so = ((uint32_t)(wn * WN / 128) * sb_stride + (uint32_t)(k0 >> 6)) * 256;
#pragma unroll
        for (int g = 0; g < 2; ++g)
          s[g] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sb, valid ? vsb + g * 64 : 0x80000000u, so, 0) >> sh_b;
      }
    };

    uint32_t sa_cur[SA], sb_cur[SB], sa_nxt[SA], sb_nxt[SB];
    load_scales_a(sa_cur, k_begin);
    load_scales_b(sb_cur, k_begin);
    issue_loads(0, k_begin);

    for (int64_t step = 0; step < nsteps; ++step) {
      const int cur = (int)(step & 1);
      const int64_t k0 = k_begin + step * kBK;
      // this wave's loads of stage `cur` have landed; after the barrier everybody's have,
      // and everybody has finished reading stage `cur ^ 1`
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      __syncthreads();
      // Prefetch the next step unconditionally (past k_end every lane is out of range and the
      // loads return zeros), so the loop body stays one basic block.  Scales first: the wait
      // before they are consumed then leaves the code loads in flight.
      load_scales_a(sa_nxt, k0 + kBK);
      load_scales_b(sb_nxt, k0 + kBK);
      issue_loads(cur ^ 1, k0 + kBK);

      const uint8_t* sbase = smem + cur * STAGE;
      v8i af[TM];
#pragma unroll
      for (int m = 0; m < TM; ++m) {
        const v4i lo = *reinterpret_cast<const v4i*>(sbase + fa0 + m * 2048);
        const v4i hi = *reinterpret_cast<const v4i*>(sbase + fa1 + m * 2048);
        af[m] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
      static_for<0, TN>([&](auto n_) {
        constexpr int n = decltype(n_)::value;
        const v4i lo = *reinterpret_cast<const v4i*>(sbase + fb0 + n * 2048);
        const v4i hi = *reinterpret_cast<const v4i*>(sbase + fb1 + n * 2048);
        const v8i bf = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        constexpr int ob = B_ROWMAJOR ? 0 : (n >> 1);
        const uint32_t sbv = sb_cur[B_ROWMAJOR ? n : (n & 1)];
        static_for<0, TM>([&](auto m_) {
          constexpr int m = decltype(m_)::value;
          constexpr int oa = A_ROWMAJOR ? 0 : (m >> 1);
          const uint32_t sav = sa_cur[A_ROWMAJOR ? m : (m & 1)];
          // first MFMA operand = B rows (N), second = A rows (M): the lane then holds four
          // consecutive N of one M row, which stores as 8 contiguous bytes
          acc[m][n] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
              bf, af[m], acc[m][n], 0, 0, ob, (int)sbv, oa, (int)sav);
        });
      });

      // keep the register hand-over behind the MFMAs: moved earlier it would make the wave
      // wait for the next step's loads before it starts computing
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int g = 0; g < SA; ++g) sa_cur[g] = sa_nxt[g];
#pragma unroll
      for (int g = 0; g < SB; ++g) sb_cur[g] = sb_nxt[g];
    }

    // drain the last (out-of-range) prefetch before the wave can retire
    __builtin_amdgcn_s_waitcnt(0x0F70);

    // epilogue: lane holds D[row = m*16 + li][col = n*16 + lj*4 + 0..3]
    const int64_t rows_valid = A.rows_valid, cols_valid = B.rows_valid;
    const bool vec_ok = (ldd & 3) == 0 && ((uintptr_t)d & 7) == 0;
#pragma unroll
    for (int m = 0; m < TM; ++m) {
      const int64_t r = wm * WM + m * 16 + li;
      if (r >= rows_valid) continue;
#pragma unroll
      for (int n = 0; n < TN; ++n) {
        const int64_t c = wn * WN + n * 16 + lj * 4;
        if (c >= cols_valid) continue;
        const v4f a = acc[m][n];
        uint16_t* dst = d + r * ldd + c;
        const u32x2 w = {pack_bf16(a.x, a.y), pack_bf16(a.z, a.w)};
        if (vec_ok && c + 3 < cols_valid) {
          *reinterpret_cast<u32x2*>(dst) = w;
        } else {
          const uint16_t h0 = (uint16_t)w.x, h1 = (uint16_t)(w.x >> 16), h2 = (uint16_t)w.y,
                         h3 = (uint16_t)(w.y >> 16);
          dst[0] = h0;
          if (c + 1 < cols_valid) dst[1] = h1;
          if (c + 2 < cols_valid) dst[2] = h2;
          if (c + 3 < cols_valid) dst[3] = h3;
        }
      }
    }
  }
};

// XCD-aware tile order: workgroup b runs on XCD b % 8, so XCD x is given one contiguous
// run of the tile list, and the list walks 8-tall column-major panels so the 32 tiles an
// XCD has in flight share 8 A panels and 4 B panels in its L2.
__device__ __forceinline__ bool map_tile(int64_t tiles_m, int64_t tiles_n, int64_t& tm,
                                         int64_t& tn) {
  constexpr int64_t kXcd = 8, kGroupM = 8;
  const int64_t nb = tiles_m * tiles_n;
  const int64_t per_xcd = (nb + kXcd - 1) / kXcd;
  const int64_t b = blockIdx.x;
  const int64_t t = (b % kXcd) * per_xcd + b / kXcd;
  if (t >= nb) return false;
  const int64_t width = kGroupM * tiles_n;
  const int64_t group = t / width;
  const int64_t first_m = group * kGroupM;
  const int64_t gsz = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  const int64_t in = t - group * width;
  tm = first_m + in % gsz;
  tn = in / gsz;
  return true;
}

}  // namespace mx
