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
//     16-byte chunk c of row r sits at chunk position c ^ (r & 7) ^ ((r >> 3) & 1) so the 16
//     lanes that read one K-block column of a 16-row sub-tile hit 16 different bank groups.
//   * scales: straight from global into VGPRs, either one dword per lane per 64 rows from a
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
  const uint8_t* scales;   // MFMA order: group of the tile's first 64 rows, K-step 0
                           // row-major:  scale of (tile's first row, block 0)
  int64_t scale_stride;    // MFMA order: ks_n (K-steps per 64-row group); row-major: nblk
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0x7FFFFFFFll ? 0x7FFFFFFFu : (uint32_t)(bytes < 0 ? 0 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <int BM, int BN, bool A_ROWMAJOR, bool B_ROWMAJOR>
struct GemmTile {
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static constexpr int A_BYTES = BM * kBK, B_BYTES = BN * kBK, STAGE = A_BYTES + B_BYTES;
  static constexpr int A_UNITS = BM / 32, B_UNITS = BN / 32;  // 1 KB load units per wave
  static constexpr int SA = A_ROWMAJOR ? TM : TM / 4;          // scale registers per step
  static constexpr int SB = B_ROWMAJOR ? TN : TN / 4;
  static constexpr int kLdsBytes = 2 * STAGE;
  static_assert(WM % 64 == 0 && WN % 64 == 0, "wave tile must be a multiple of 64");

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

    // global -> LDS: lane l of a load unit fetches row l/8, logical chunk (l%8)^(l/8)^(unit&1)
    const uint32_t lrow = lane >> 3;
    const uint32_t chunk_even = (lane & 7) ^ lrow;  // unit parity 0; parity 1 flips bit 0
    const uint32_t va_even = lrow * (uint32_t)A.ld + chunk_even * 16;
    const uint32_t va_odd = lrow * (uint32_t)A.ld + (chunk_even ^ 1) * 16;
    const uint32_t vb_even = lrow * (uint32_t)B.ld + chunk_even * 16;
    const uint32_t vb_odd = lrow * (uint32_t)B.ld + (chunk_even ^ 1) * 16;

    // LDS -> VGPR.  Operand layout of the 16x16x128 f8 MFMA (measured on gfx950): lane
    // (li, lj) holds row li, K bytes [16*lj, 16*lj+16) in its first four registers and
    // [64+16*lj, 64+16*lj+16) in the last four, i.e. 16-byte chunks lj and lj+4; the scale
    // of K-block b (bytes [32b, 32b+32)) is taken from lane group b.
    const uint32_t sw = (li & 7) ^ (li >> 3);
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
          const uint32_t c = (q & 1) ? (chunk_even ^ 1) : chunk_even;
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
          const uint32_t c = (q & 1) ? (chunk_even ^ 1) : chunk_even;
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
                             : ((A.rows_valid + 63) >> 6) * A.scale_stride * 256);
    const __amdgpu_buffer_rsrc_t rsrc_sb = make_rsrc(
        B.scales, B_ROWMAJOR ? B.rows_valid * B.scale_stride
                             : ((B.rows_valid + 63) >> 6) * B.scale_stride * 256);
    const uint32_t vsa = A_ROWMAJOR ? (uint32_t)li * (uint32_t)A.scale_stride + lj : lane * 4;
    const uint32_t vsb = B_ROWMAJOR ? (uint32_t)li * (uint32_t)B.scale_stride + lj : lane * 4;
    const uint32_t sa_stride = (uint32_t)A.scale_stride, sb_stride = (uint32_t)B.scale_stride;

    auto load_scales_a = [&](uint32_t (&s)[SA], int64_t k0) {
      if constexpr (A_ROWMAJOR) {
        const bool valid = k0 + 32 * lj < k_end;
#pragma unroll
        for (int m = 0; m < TM; ++m) {
          const uint32_t so = (uint32_t)(wm * WM + m * 16) * sa_stride + (uint32_t)(k0 >> 5);
          const uint32_t b = __builtin_amdgcn_raw_buffer_load_b8(rsrc_sa, valid ? vsa : 0x80000000u, so, 0);
          s[m] = b;
        }
      } else {
#pragma unroll
        for (int g = 0; g < SA; ++g) {
          const uint32_t so = ((uint32_t)(wm * (WM / 64) + g) * sa_stride + (uint32_t)(k0 >> 7)) * 256;
          s[g] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sa, vsa, so, 0);
        }
      }
    };
    auto load_scales_b = [&](uint32_t (&s)[SB], int64_t k0) {
      if constexpr (B_ROWMAJOR) {
        const bool valid = k0 + 32 * lj < k_end;
#pragma unroll
        for (int n = 0; n < TN; ++n) {
          const uint32_t so = (uint32_t)(wn * WN + n * 16) * sb_stride + (uint32_t)(k0 >> 5);
          const uint32_t b = __builtin_amdgcn_raw_buffer_load_b8(rsrc_sb, valid ? vsb : 0x80000000u, so, 0);
          s[n] = b;
        }
      } else {
#pragma unroll
        for (int g = 0; g < SB; ++g) {
          const uint32_t so = ((uint32_t)(wn * (WN / 64) + g) * sb_stride + (uint32_t)(k0 >> 7)) * 256;
          s[g] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sb, vsb, so, 0);
        }
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
        constexpr int ob = B_ROWMAJOR ? 0 : (n & 3);
        const uint32_t sbv = sb_cur[B_ROWMAJOR ? n : (n >> 2)];
        static_for<0, TM>([&](auto m_) {
          constexpr int m = decltype(m_)::value;
          constexpr int oa = A_ROWMAJOR ? 0 : (m & 3);
          const uint32_t sav = sa_cur[A_ROWMAJOR ? m : (m >> 2)];
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
        const uint16_t h0 = f32_to_bf16_rne(a.x), h1 = f32_to_bf16_rne(a.y),
                       h2 = f32_to_bf16_rne(a.z), h3 = f32_to_bf16_rne(a.w);
        if (vec_ok && c + 3 < cols_valid) {
          u32x2 w = {(uint32_t)h0 | ((uint32_t)h1 << 16), (uint32_t)h2 | ((uint32_t)h3 << 16)};
          *reinterpret_cast<u32x2*>(dst) = w;
        } else {
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
