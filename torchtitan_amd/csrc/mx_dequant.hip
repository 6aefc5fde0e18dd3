// MXFP8 -> bf16: value = e4m3(code) * 2^(scale byte - 127), one scale per 32 codes of a row.
// Receiving side of a weight hand-over in MXFP8 form.  HBM-bound streaming: 1.03 B read and
// 2 B written per element.
#include "mx_common.h"

namespace mx {

constexpr int kDqThreads = 256;

// float32 -> bf16 bits, round to nearest even (results here are exact except below bf16's
// normal range), NaN kept quiet.
__device__ __forceinline__ uint32_t dq_bf16(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// 2^(byte - 127) as a float; byte 0 -> 2^-127 (a float32 denormal), byte 255 -> NaN.
__device__ __forceinline__ float e8m0_value(uint32_t byte) {
  if (byte == 255u) return __uint_as_float(0x7FC00000u);
  return byte == 0u ? __uint_as_float(0x00400000u) : __uint_as_float(byte << 23);
}

template <int ORDER>
__global__ __launch_bounds__(kDqThreads) void dequant_kernel(
    const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales, int64_t rows,
    int64_t cols, int64_t nblk, int64_t ks_n, uint16_t* __restrict__ out, int64_t ldo) {
  const int64_t per_row = cols / 16;  // one lane: 16 codes = half a block
  const int64_t total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * kDqThreads + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * kDqThreads) {
    const int64_t r = i / per_row, c = (i - r * per_row) * 16;
    const int64_t blk = c >> 5;
    const uint32_t sb = scales[ORDER == MX_SCALES_MFMA ? mfma_scale_offset(r, blk, ks_n) : r * nblk + blk];
    const float s = e8m0_value(sb);
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(codes + r * cols + c));
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float f0 = __builtin_amdgcn_cvt_f32_fp8((int)w[e], 0) * s;
      const float f1 = __builtin_amdgcn_cvt_f32_fp8((int)w[e], 1) * s;
      const float f2 = __builtin_amdgcn_cvt_f32_fp8((int)w[e], 2) * s;
      const float f3 = __builtin_amdgcn_cvt_f32_fp8((int)w[e], 3) * s;
      o[2 * e] = dq_bf16(f0) | (dq_bf16(f1) << 16);
      o[2 * e + 1] = dq_bf16(f2) | (dq_bf16(f3) << 16);
    }
    u32x4* dst = reinterpret_cast<u32x4*>(out + r * ldo + c);
    __builtin_nontemporal_store(u32x4{o[0], o[1], o[2], o[3]}, dst);
    __builtin_nontemporal_store(u32x4{o[4], o[5], o[6], o[7]}, dst + 1);
  }
}

}  // namespace mx

using namespace mx;

extern "C" int mx_dequant(const uint8_t* codes, const uint8_t* scales, int64_t rows, int64_t cols,
                          int scale_order, void* out, int64_t ldo, void* stream) {
  if (rows < 0 || cols < 0 || ldo < cols ||
      (scale_order != MX_SCALES_ROWMAJOR && scale_order != MX_SCALES_MFMA))
    return MX_ERR_INVALID_ARG;
  if (rows == 0 || cols == 0) return MX_OK;
  if (!codes || !scales || !out) return MX_ERR_INVALID_ARG;
  if (cols % 32 || ldo % 8 || ((uintptr_t)codes & 15) || ((uintptr_t)out & 15)) return MX_ERR_ALIGNMENT;
  const int64_t nblk = cols / 32, ks_n = (nblk + 1) / 2;
  const int64_t work = rows * (cols / 16);
  int64_t blocks = (work + kDqThreads - 1) / kDqThreads;
  blocks = blocks > 256 * 16 ? 256 * 16 : blocks;
  hipStream_t st = (hipStream_t)stream;
  if (scale_order == MX_SCALES_MFMA)
    hipLaunchKernelGGL((dequant_kernel<MX_SCALES_MFMA>), dim3((unsigned)blocks), dim3(kDqThreads), 0, st,
                       codes, scales, rows, cols, nblk, ks_n, (uint16_t*)out, ldo);
  else
    hipLaunchKernelGGL((dequant_kernel<MX_SCALES_ROWMAJOR>), dim3((unsigned)blocks), dim3(kDqThreads), 0,
                       st, codes, scales, rows, cols, nblk, ks_n, (uint16_t*)out, ldo);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
