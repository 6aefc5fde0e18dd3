// Routed-token side of the MoE layer around the expert GEMMs: the weighted sum that brings the
// top-k expert outputs of a token back together, and the row dot products that give the
// gradient of the routing scores.  HBM-bound row streaming, float32 arithmetic in a fixed order.
#include "mx_common.h"

namespace mx {

constexpr int kMoeThreads = 256;

__device__ __forceinline__ float bf16_bits_f32(uint32_t w_lo16) { return __uint_as_float(w_lo16 << 16); }

// float32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint32_t f32_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// a * b rounded to float32 on its own: the empty asm keeps the compiler from contracting the
// product into the addition that follows (one rounding instead of the stated two).
__device__ __forceinline__ float rounded_product(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return p;
}

// bf16(a + b) of two bf16 values, as a bf16 tensor addition forms it.
__device__ __forceinline__ float bf16_sum(uint32_t a16, uint32_t b16) {
  return bf16_bits_f32(f32_bf16_bits(bf16_bits_f32(a16) + bf16_bits_f32(b16)));
}

// out[t, :] = sum_j w[t, j] * y[pos[t, j], :]   (j = 0 .. k-1 in that order, float32, the product
// and the sum rounded separately; w == nullptr: plain sum).  A position outside [0, y_rows)
// contributes nothing.  With y2, the rows summed are bf16(y + y2) (two matrices of one shape
// that a bf16 addition would have merged first).  One lane per 8 columns, grid-stride over
// (token, column chunk).
__global__ __launch_bounds__(kMoeThreads) void moe_combine_kernel(
    const uint16_t* __restrict__ y, const uint16_t* __restrict__ y2, int64_t y_rows, int64_t ldy,
    const int64_t* __restrict__ pos,
    const float* __restrict__ w, int64_t tokens, int k, int64_t cols, uint16_t* __restrict__ out,
    int64_t ldo) {
  const int64_t chunks = cols / 8;
  const int64_t total = tokens * chunks;
  for (int64_t i = (int64_t)blockIdx.x * kMoeThreads + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * kMoeThreads) {
    const int64_t t = i / chunks, c = (i - t * chunks) * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const int64_t r = pos[t * k + j];
      if (r < 0 || r >= y_rows) continue;
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(y + r * ldy + c));
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};
      float x[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = bf16_bits_f32(d[e] & 0xFFFFu);
        x[2 * e + 1] = bf16_bits_f32(d[e] >> 16);
      }
      if (y2) {
        const u32x4 v2 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(y2 + r * ldy + c));
        const uint32_t d2[4] = {v2.x, v2.y, v2.z, v2.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[2 * e] = bf16_sum(d[e] & 0xFFFFu, d2[e] & 0xFFFFu);
          x[2 * e + 1] = bf16_sum(d[e] >> 16, d2[e] >> 16);
        }
      }
      if (w) {
        const float s = w[t * k + j];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += rounded_product(s, x[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = acc[e] + x[e];
      }
    }
    u32x4 o;
    o.x = f32_bf16_bits(acc[0]) | (f32_bf16_bits(acc[1]) << 16);
    o.y = f32_bf16_bits(acc[2]) | (f32_bf16_bits(acc[3]) << 16);
    o.z = f32_bf16_bits(acc[4]) | (f32_bf16_bits(acc[5]) << 16);
    o.w = f32_bf16_bits(acc[6]) | (f32_bf16_bits(acc[7]) << 16);
    *reinterpret_cast<u32x4*>(out + t * ldo + c) = o;
  }
}

// out[i] = sum_d a[ia[i], d] * b[ib[i], d] in float32; a row index outside its matrix gives 0.
// With a2, a's rows are bf16(a + a2).  One wave per output: lanes stride over 8-column chunks,
// then a butterfly over the 64 lanes.
__global__ __launch_bounds__(kMoeThreads) void moe_row_dot_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ a2, int64_t a_rows, int64_t lda,
    const int64_t* __restrict__ ia,
    const uint16_t* __restrict__ b, int64_t b_rows, int64_t ldb, const int64_t* __restrict__ ib,
    int64_t n, int64_t cols, float* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * kMoeThreads + threadIdx.x) >> 6;
  const int64_t waves = ((int64_t)gridDim.x * kMoeThreads) >> 6;
  for (int64_t i = wave; i < n; i += waves) {
    const int64_t ra = ia[i], rb = ib[i];
    float acc = 0.f;
    if (ra >= 0 && ra < a_rows && rb >= 0 && rb < b_rows) {
      for (int64_t c = lane * 8; c < cols; c += 64 * 8) {
        const u32x4 va = *reinterpret_cast<const u32x4*>(a + ra * lda + c);
        const u32x4 vb = *reinterpret_cast<const u32x4*>(b + rb * ldb + c);
        const uint32_t da[4] = {va.x, va.y, va.z, va.w}, db[4] = {vb.x, vb.y, vb.z, vb.w};
        float xa[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          xa[2 * e] = bf16_bits_f32(da[e] & 0xFFFFu);
          xa[2 * e + 1] = bf16_bits_f32(da[e] >> 16);
        }
        if (a2) {
          const u32x4 v2 = *reinterpret_cast<const u32x4*>(a2 + ra * lda + c);
          const uint32_t d2[4] = {v2.x, v2.y, v2.z, v2.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            xa[2 * e] = bf16_sum(da[e] & 0xFFFFu, d2[e] & 0xFFFFu);
            xa[2 * e + 1] = bf16_sum(da[e] >> 16, d2[e] >> 16);
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc = __builtin_fmaf(xa[2 * e], bf16_bits_f32(db[e] & 0xFFFFu), acc);
          acc = __builtin_fmaf(xa[2 * e + 1], bf16_bits_f32(db[e] >> 16), acc);
        }
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) out[i] = acc;
  }
}

static inline unsigned moe_grid(int64_t work_items) {
  const int64_t blocks = (work_items + kMoeThreads - 1) / kMoeThreads;
  const int64_t cap = 256 * 16;  // 16 workgroups per CU keep every CU streaming
  return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace mx

using namespace mx;

extern "C" int mx_moe_combine(const void* y, const void* y2, int64_t y_rows, int64_t ldy,
                              const int64_t* pos,
                              const float* weights, int64_t tokens, int64_t top_k, int64_t cols,
                              void* out, int64_t ldo, void* stream) {
  if (y_rows < 0 || tokens < 0 || top_k < 0 || top_k > 1024 || cols < 0 || ldy < cols || ldo < cols)
    return MX_ERR_INVALID_ARG;
  if (tokens == 0 || cols == 0) return MX_OK;
  if (!out || (top_k > 0 && (!y || !pos))) return MX_ERR_INVALID_ARG;
  if (cols % 8 || ldy % 8 || ldo % 8 || ((uintptr_t)y & 15) || ((uintptr_t)y2 & 15) ||
      ((uintptr_t)out & 15) || ((uintptr_t)pos & 7) || ((uintptr_t)weights & 3))
    return MX_ERR_ALIGNMENT;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(moe_grid(tokens * (cols / 8))), dim3(kMoeThreads), 0,
                     (hipStream_t)stream, (const uint16_t*)y, (const uint16_t*)y2, y_rows, ldy, pos,
                     weights, tokens,
                     (int)top_k, cols, (uint16_t*)out, ldo);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

extern "C" int mx_moe_row_dot(const void* a, const void* a2, int64_t a_rows, int64_t lda,
                              const int64_t* ia,
                              const void* b, int64_t b_rows, int64_t ldb, const int64_t* ib,
                              int64_t n, int64_t cols, float* out, void* stream) {
  if (a_rows < 0 || b_rows < 0 || n < 0 || cols < 0 || lda < cols || ldb < cols)
    return MX_ERR_INVALID_ARG;
  if (n == 0) return MX_OK;
  if (!a || !b || !ia || !ib || !out) return MX_ERR_INVALID_ARG;
  if (cols % 8 || lda % 8 || ldb % 8 || ((uintptr_t)a & 15) || ((uintptr_t)a2 & 15) ||
      ((uintptr_t)b & 15) ||
      ((uintptr_t)ia & 7) || ((uintptr_t)ib & 7) || ((uintptr_t)out & 3))
    return MX_ERR_ALIGNMENT;
  hipLaunchKernelGGL(moe_row_dot_kernel, dim3(moe_grid(n * 64)), dim3(kMoeThreads), 0,
                     (hipStream_t)stream, (const uint16_t*)a, (const uint16_t*)a2, a_rows, lda, ia,
                     (const uint16_t*)b,
                     b_rows, ldb, ib, n, cols, out);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
