// MoE grouped MXFP8 GEMMs over variable-size expert groups (device-side offsets, no host
// synchronisation): 2D x 3D for forward / dgrad, 2D x 2D for wgrad.  Both reuse the dense
// workgroup tile; only the tile -> (group, rows, K range) mapping differs.
#include "mx_gemm_tile.h"

namespace mx {

struct G2d3dArgs {
  const uint8_t* a_codes;   // [T, K]
  const uint8_t* a_scales;  // row-major [T, K/32]
  const uint8_t* b_codes;   // [G, N, K]
  const uint8_t* b_scales;  // G MFMA-order blocks for [N, K/32]
  const int32_t* offs;      // [G] inclusive cumulative group sizes
  uint16_t* d;              // [T, N]
  int64_t T, N, K, G, ldd;
  int64_t max_mtiles;
};

template <int BM, int BN>
__global__ __launch_bounds__(256, 1) void grouped_2d3d_kernel(G2d3dArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  using Tile = GemmTile<BM, BN, true, false>;
  const int64_t tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = p.max_mtiles * tiles_n;
  const int64_t per_xcd = (nb + 7) / 8;
  const int64_t b = blockIdx.x;
  const int64_t t = (b % 8) * per_xcd + b / 8;  // XCD x walks one contiguous run of tiles
  if (t >= nb) return;
  const int64_t mt = t / tiles_n, tn = t - mt * tiles_n;

  // which group owns M-tile `mt`: groups are tiled one after another
  int64_t first = 0, lo = 0, hi = 0;
  int64_t g = 0;
  for (; g < p.G; ++g) {
    hi = p.offs[g];
    const int64_t nt = (hi - lo + BM - 1) / BM;
    if (mt < first + nt) break;
    first += nt;
    lo = hi;
  }
  const int64_t col0 = tn * BN;
  if (g == p.G) {
    // past the last group: rows [offs[G-1], T) are padding and come out as zeros
    const int64_t row0 = lo + (mt - first) * BM;
    const int64_t rows = p.T - row0 < BM ? p.T - row0 : BM;
    const int64_t cols = p.N - col0 < BN ? p.N - col0 : BN;
    for (int64_t r = threadIdx.x >> 6; r < rows; r += 4)
      for (int64_t c = threadIdx.x & 63; c < cols; c += 64) p.d[(row0 + r) * p.ldd + col0 + c] = 0;
    return;
  }
  const int64_t row0 = lo + (mt - first) * BM;
  const int64_t nblk = p.K / 32, ks_n = (nblk + 1) / 2;
  const int64_t b_scale_block = ((p.N + 127) / 128) * ks_n * 256;
  Operand A{p.a_codes + row0 * p.K, p.K, hi - row0, p.a_scales + row0 * nblk, nblk};
  Operand B{p.b_codes + (g * p.N + col0) * p.K, p.K, p.N - col0,
            p.b_scales + g * b_scale_block + tn * (BN / 128) * ks_n * 256, ks_n};
  Tile::run(smem, A, B, 0, p.K, p.d + row0 * p.ldd + col0, p.ldd);
}

struct G2d2dArgs {
  const uint8_t* at_codes;   // [N, T]
  const uint8_t* at_scales;  // row-major [N, T/32]
  const uint8_t* bt_codes;   // [K, T]
  const uint8_t* bt_scales;  // row-major [K, T/32]
  const int32_t* offs;
  uint16_t* d;               // [G, N, K]
  int64_t T, N, K, G;
};

template <int BM, int BN>
__global__ __launch_bounds__(256, 1) void grouped_2d2d_kernel(G2d2dArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  using Tile = GemmTile<BM, BN, true, true>;
  const int64_t tiles_m = (p.N + BM - 1) / BM, tiles_n = (p.K + BN - 1) / BN;
  const int64_t per_group = tiles_m * tiles_n;
  const int64_t nb = p.G * per_group;
  const int64_t per_xcd = (nb + 7) / 8;
  const int64_t b = blockIdx.x;
  const int64_t t = (b % 8) * per_xcd + b / 8;
  if (t >= nb) return;
  const int64_t g = t / per_group, in = t - g * per_group;
  const int64_t tm = in % tiles_m, tn = in / tiles_m;
  const int64_t lo = g ? p.offs[g - 1] : 0, hi = p.offs[g];
  const int64_t nblk = p.T / 32;
  if (((lo | hi) & 31) || hi < lo || lo < 0 || hi > p.T) {
    // a group that does not start and end on a 32-token block would share scale blocks with its
    // neighbour: the contract is broken, and the result must not pass for a gradient.  NaN.
    const int64_t row0 = tm * BM, col0 = tn * BN;
    const int64_t rows = p.N - row0 < BM ? p.N - row0 : BM, cols = p.K - col0 < BN ? p.K - col0 : BN;
    uint16_t* out = p.d + g * p.N * p.K + row0 * p.K + col0;
    for (int64_t r = threadIdx.x >> 6; r < rows; r += 4)
      for (int64_t c = threadIdx.x & 63; c < cols; c += 64) out[r * p.K + c] = 0x7FC0;
    return;
  }
  Operand A{p.at_codes + tm * BM * p.T, p.T, p.N - tm * BM, p.at_scales + tm * BM * nblk, nblk};
  Operand B{p.bt_codes + tn * BN * p.T, p.T, p.K - tn * BN, p.bt_scales + tn * BN * nblk, nblk};
  Tile::run(smem, A, B, lo, hi, p.d + g * p.N * p.K + tm * BM * p.K + tn * BN, p.K);
}

template <class Kern, class Args>
static int launch_tile_kernel(Kern kern, std::atomic<bool> (&configured)[kMaxDevices], int lds_bytes,
                              int64_t nb, const Args& p, hipStream_t st) {
  if (!raise_lds_limit(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return MX_ERR_LAUNCH;
  const int64_t grid = (nb + 7) / 8 * 8;
  if (grid > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds_bytes, st, p);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

template <int BM, int BN>
static int launch_2d3d(G2d3dArgs p, hipStream_t st) {
  static std::atomic<bool> configured[kMaxDevices];
  p.max_mtiles = (p.T + BM - 1) / BM + p.G + 1;
  const int64_t nb = p.max_mtiles * ((p.N + BN - 1) / BN);
  return launch_tile_kernel(grouped_2d3d_kernel<BM, BN>, configured,
                            GemmTile<BM, BN, true, false>::kLdsBytes, nb, p, st);
}

template <int BM, int BN>
static int launch_2d2d(const G2d2dArgs& p, hipStream_t st) {
  static std::atomic<bool> configured[kMaxDevices];
  const int64_t nb = p.G * ((p.N + BM - 1) / BM) * ((p.K + BN - 1) / BN);
  return launch_tile_kernel(grouped_2d2d_kernel<BM, BN>, configured,
                            GemmTile<BM, BN, true, true>::kLdsBytes, nb, p, st);
}

}  // namespace mx

using namespace mx;

namespace mx {
int launch_grouped32_2d3d(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                          const uint8_t* b_scales, const int32_t* offs, void* d, int64_t T,
                          int64_t N, int64_t K, int64_t G, int64_t ldd, hipStream_t st);
int launch_grouped32_2d2d(const uint8_t* at_codes, const uint8_t* at_scales,
                          const uint8_t* bt_codes, const uint8_t* bt_scales, const int32_t* offs,
                          void* d, int64_t T, int64_t N, int64_t K, int64_t G, hipStream_t st);
int launch_grouped32_2d3d_pair(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                               const uint8_t* b_scales, const uint8_t* a2_codes,
                               const uint8_t* a2_scales, const uint8_t* b2_codes,
                               const uint8_t* b2_scales, const int32_t* offs, void* d, int64_t T,
                               int64_t N, int64_t K, int64_t G, int64_t ldd, hipStream_t st);
int launch_grouped32_2d3d_rows_out(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                   const uint8_t* b_scales, const uint8_t* a2_codes,
                                   const uint8_t* a2_scales, const uint8_t* b2_codes,
                                   const uint8_t* b2_scales, const int32_t* offs, const int32_t* d_offs,
                                   void* d, int64_t T, int64_t d_rows, int64_t N, int64_t K, int64_t G,
                                   int64_t ldd, hipStream_t st);
int launch_grouped32_2d3d_two_b(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                                const int32_t* offs, void* d, void* d2, int64_t T, int64_t N, int64_t K,
                                int64_t G, int64_t ldd, hipStream_t st);
int launch_grouped32_2d2d_two_a(const uint8_t* at_codes, const uint8_t* at_scales, const uint8_t* at2_codes,
                                const uint8_t* at2_scales, const uint8_t* bt_codes, const uint8_t* bt_scales,
                                const int32_t* offs, void* d, void* d2, int64_t T, int64_t N, int64_t K,
                                int64_t G, hipStream_t st);
}  // namespace mx

// Two grouped products that share an operand, one launch of the persistent kernel (all scales in
// MFMA order); other shapes are the caller's two calls.
extern "C" int mx_grouped_gemm_2d3d_shared_a(const uint8_t* a_codes, const uint8_t* a_scales,
                                             const uint8_t* b_codes, const uint8_t* b_scales,
                                             const uint8_t* b2_codes, const uint8_t* b2_scales,
                                             const int32_t* offs, void* d, void* d2, int64_t T,
                                             int64_t N, int64_t K, int64_t G, int64_t ldd,
                                             void* stream) {
  if (T < 0 || N < 0 || K < 0 || G <= 0 || ldd < N) return MX_ERR_INVALID_ARG;
  if (T == 0 || N == 0) return MX_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !b2_codes || !b2_scales || !offs || !d || !d2)
    return MX_ERR_INVALID_ARG;
  if (K == 0 || K % 128 || N % 8 || ldd % 8 || T % 32) return MX_ERR_ALIGNMENT;
  if (((uintptr_t)a_codes & 15) || ((uintptr_t)b_codes & 15) || ((uintptr_t)b2_codes & 15) ||
      ((uintptr_t)a_scales & 3) || ((uintptr_t)b_scales & 3) || ((uintptr_t)b2_scales & 3) ||
      ((uintptr_t)d & 15) || ((uintptr_t)d2 & 15))
    return MX_ERR_ALIGNMENT;
  if (256 * K > 0x7FFFFFFFll || G > 510 || ldd * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  return launch_grouped32_2d3d_two_b(a_codes, a_scales, b_codes, b_scales, b2_codes, b2_scales, offs, d,
                                     d2, T, N, K, G, ldd, (hipStream_t)stream);
}

extern "C" int mx_grouped_gemm_2d2d_shared_b(const uint8_t* at_codes, const uint8_t* at_scales,
                                             const uint8_t* at2_codes, const uint8_t* at2_scales,
                                             const uint8_t* bt_codes, const uint8_t* bt_scales,
                                             const int32_t* offs, void* d, void* d2, int64_t T,
                                             int64_t N, int64_t K, int64_t G, void* stream) {
  if (T < 0 || N < 0 || K < 0 || G <= 0) return MX_ERR_INVALID_ARG;
  if (N == 0 || K == 0) return MX_OK;
  if (!d || !d2 || !offs || !at_codes || !at_scales || !at2_codes || !at2_scales || !bt_codes || !bt_scales)
    return MX_ERR_INVALID_ARG;
  if (T == 0) return MX_ERR_UNSUPPORTED;  // nothing to contract: the general kernel writes the zeros
  if (T % 128 || K % 8 || ((uintptr_t)d & 15) || ((uintptr_t)d2 & 15) || ((uintptr_t)at_codes & 15) ||
      ((uintptr_t)at2_codes & 15) || ((uintptr_t)bt_codes & 15) || ((uintptr_t)at_scales & 3) ||
      ((uintptr_t)at2_scales & 3) || ((uintptr_t)bt_scales & 3))
    return MX_ERR_ALIGNMENT;
  if (256 * T > 0x7FFFFFFFll || K * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  return launch_grouped32_2d2d_two_a(at_codes, at_scales, at2_codes, at2_scales, bt_codes, bt_scales, offs,
                                     d, d2, T, N, K, G, (hipStream_t)stream);
}

extern "C" int mx_grouped_gemm_2d3d_rows_out(const uint8_t* a_codes, const uint8_t* a_scales,
                                             const uint8_t* b_codes, const uint8_t* b_scales,
                                             const uint8_t* a2_codes, const uint8_t* a2_scales,
                                             const uint8_t* b2_codes, const uint8_t* b2_scales,
                                             const int32_t* offs, const int32_t* out_offs, void* d,
                                             int64_t T, int64_t out_rows, int64_t N, int64_t K,
                                             int64_t G, int64_t ldd, void* stream) {
  if (T < 0 || out_rows < 0 || out_rows > T || N < 0 || K < 0 || G <= 0 || ldd < N)
    return MX_ERR_INVALID_ARG;
  if (out_rows == 0 || N == 0) return MX_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !offs || !out_offs || !d)
    return MX_ERR_INVALID_ARG;
  const bool two = a2_codes || a2_scales || b2_codes || b2_scales;
  if (two && (!a2_codes || !a2_scales || !b2_codes || !b2_scales)) return MX_ERR_INVALID_ARG;
  if (K == 0 || K % 128 || N % 8 || ldd % 8 || T % 32) return MX_ERR_ALIGNMENT;
  if (((uintptr_t)a_codes & 15) || ((uintptr_t)b_codes & 15) || ((uintptr_t)a_scales & 3) ||
      ((uintptr_t)b_scales & 3) || ((uintptr_t)d & 15))
    return MX_ERR_ALIGNMENT;
  if (two && (((uintptr_t)a2_codes & 15) || ((uintptr_t)b2_codes & 15) || ((uintptr_t)a2_scales & 3) ||
              ((uintptr_t)b2_scales & 3)))
    return MX_ERR_ALIGNMENT;
  if (256 * K > 0x7FFFFFFFll || G > 510 || ldd * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  return launch_grouped32_2d3d_rows_out(a_codes, a_scales, b_codes, b_scales, a2_codes, a2_scales,
                                        b2_codes, b2_scales, offs, out_offs, d, T, out_rows, N, K, G,
                                        ldd, (hipStream_t)stream);
}

extern "C" int mx_grouped_gemm_2d3d_pair(const uint8_t* a_codes, const uint8_t* a_scales,
                                         const uint8_t* b_codes, const uint8_t* b_scales,
                                         const uint8_t* a2_codes, const uint8_t* a2_scales,
                                         const uint8_t* b2_codes, const uint8_t* b2_scales,
                                         const int32_t* offs, void* d, int64_t T, int64_t N,
                                         int64_t K, int64_t G, int64_t ldd, void* stream) {
  if (T < 0 || N < 0 || K < 0 || G <= 0 || ldd < N) return MX_ERR_INVALID_ARG;
  if (T == 0 || N == 0) return MX_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !a2_codes || !a2_scales || !b2_codes ||
      !b2_scales || !offs || !d)
    return MX_ERR_INVALID_ARG;
  if (K == 0 || K % 128 || N % 8 || ldd % 8 || T % 32) return MX_ERR_ALIGNMENT;
  if (((uintptr_t)a_codes & 15) || ((uintptr_t)b_codes & 15) || ((uintptr_t)a2_codes & 15) ||
      ((uintptr_t)b2_codes & 15) || ((uintptr_t)a_scales & 3) || ((uintptr_t)b_scales & 3) ||
      ((uintptr_t)a2_scales & 3) || ((uintptr_t)b2_scales & 3) || ((uintptr_t)d & 15))
    return MX_ERR_ALIGNMENT;
  if (256 * K > 0x7FFFFFFFll || G > 510 || ldd * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  return launch_grouped32_2d3d_pair(a_codes, a_scales, b_codes, b_scales, a2_codes, a2_scales,
                                    b2_codes, b2_scales, offs, d, T, N, K, G, ldd,
                                    (hipStream_t)stream);
}

extern "C" int mx_grouped_gemm_2d3d(const uint8_t* a_codes, const uint8_t* a_scales,
                                    const uint8_t* b_codes, const uint8_t* b_scales,
                                    const int32_t* offs, void* d, int64_t T, int64_t N, int64_t K,
                                    int64_t G, int64_t ldd, int a_scale_order, void* stream) {
  if (T < 0 || N < 0 || K < 0 || G <= 0 || ldd < N) return MX_ERR_INVALID_ARG;
  if (a_scale_order != MX_SCALES_ROWMAJOR && a_scale_order != MX_SCALES_MFMA)
    return MX_ERR_INVALID_ARG;
  if (T == 0 || N == 0) return MX_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !offs || !d) return MX_ERR_INVALID_ARG;
  if (K == 0 || K % 32) return MX_ERR_ALIGNMENT;
  if (((uintptr_t)a_codes & 15) || ((uintptr_t)b_codes & 15) || ((uintptr_t)b_scales & 3))
    return MX_ERR_ALIGNMENT;
  if (256 * K > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  if (a_scale_order == MX_SCALES_MFMA) {
    // group ends at multiples of 32 (checked on the device): the persistent kernel (mx_gemm32.hip)
    if (K % 128 || N % 8 || ldd % 8 || ((uintptr_t)d & 15) || ((uintptr_t)a_scales & 3) ||
        T % 32)
      return MX_ERR_ALIGNMENT;
    if (G > 510 || ldd * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
    return launch_grouped32_2d3d(a_codes, a_scales, b_codes, b_scales, offs, d, T, N, K, G, ldd,
                                 st);
  }
  G2d3dArgs p{a_codes, a_scales, b_codes, b_scales, offs, (uint16_t*)d, T, N, K, G, ldd, 0};
  if (T / G < 192 || N <= 128) return launch_2d3d<128, 128>(p, st);
  return launch_2d3d<256, 256>(p, st);
}

extern "C" int mx_grouped_gemm_2d2d(const uint8_t* at_codes, const uint8_t* at_scales,
                                    const uint8_t* bt_codes, const uint8_t* bt_scales,
                                    const int32_t* offs, void* d, int64_t T, int64_t N, int64_t K,
                                    int64_t G, int scale_order, void* stream) {
  if (T < 0 || N < 0 || K < 0 || G <= 0) return MX_ERR_INVALID_ARG;
  if (scale_order != MX_SCALES_ROWMAJOR && scale_order != MX_SCALES_MFMA)
    return MX_ERR_INVALID_ARG;
  if (N == 0 || K == 0) return MX_OK;
  if (!d || !offs) return MX_ERR_INVALID_ARG;
  if (T % 32) return MX_ERR_ALIGNMENT;
  if (T > 0 && (!at_codes || !at_scales || !bt_codes || !bt_scales)) return MX_ERR_INVALID_ARG;
  if (((uintptr_t)at_codes & 15) || ((uintptr_t)bt_codes & 15) || (T % 16))
    return MX_ERR_ALIGNMENT;
  if (256 * T > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  if (scale_order == MX_SCALES_MFMA) {
    if (T % 128 || K % 8 || ((uintptr_t)d & 15) || ((uintptr_t)at_scales & 3) ||
        ((uintptr_t)bt_scales & 3))
      return MX_ERR_ALIGNMENT;
    if (K * 512 > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
    if (T == 0) return MX_ERR_UNSUPPORTED;  // nothing to contract: the general kernel writes the zeros
    return launch_grouped32_2d2d(at_codes, at_scales, bt_codes, bt_scales, offs, d, T, N, K, G, st);
  }
  G2d2dArgs p{at_codes, at_scales, bt_codes, bt_scales, offs, (uint16_t*)d, T, N, K, G};
  if (N <= 128 || K <= 128) return launch_2d2d<128, 128>(p, st);
  return launch_2d2d<256, 256>(p, st);
}
