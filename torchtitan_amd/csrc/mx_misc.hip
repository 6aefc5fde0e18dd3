// Library identification and status strings.
#include "mx_common.h"

extern "C" int mx_version(void) { return 101; }

extern "C" const char* mx_status_string(int status) {
  switch (status) {
    case MX_OK: return "ok";
    case MX_ERR_INVALID_ARG: return "invalid argument";
    case MX_ERR_ALIGNMENT: return "dimension or pointer not aligned to what the kernel needs";
    case MX_ERR_LAUNCH: return "kernel launch failed";
    case MX_ERR_UNSUPPORTED: return "shape not supported";
    case MX_ERR_SCRATCH_TOO_SMALL:
      return "the split of this shape needs more than the library's built-in scratch array holds";
    default: return "unknown status";
  }
}

// ---- HBM yardsticks (include/mxfp8_debug.h) --------------------------------------------------
// The plainest streaming kernels there are, 16 bytes per lane, every lane of a wave next to its
// neighbour, nontemporal like the casts' accesses: what this chip's memory system gives a kernel
// that does nothing but move bytes.  bench.py times them next to the casts.
namespace mx {
typedef uint32_t y_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void stream_copy_kernel(const y_u32x4* __restrict__ src,
                                                          y_u32x4* __restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}
__global__ __launch_bounds__(256) void stream_read_kernel(const y_u32x4* __restrict__ src, int64_t n,
                                                          y_u32x4* __restrict__ sink) {
  const int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
  y_u32x4 acc = {0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < 4; ++k)
    if (i + k * 256 < n) {
      const y_u32x4 v = __builtin_nontemporal_load(src + i + k * 256);
      acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
    }
  // never true for the patterns bench.py fills the buffer with: keeps the loads alive
  if (acc.x == 0x12345678u && acc.y == 0x9ABCDEF1u && acc.z == 0x0F1E2D3Cu) *sink = acc;
}
// a row-wise cast's traffic without the cast: 16 bytes read and 8 bytes written per lane
typedef uint32_t y_u32x2 __attribute__((ext_vector_type(2)));
__global__ __launch_bounds__(256) void stream_2to1_kernel(const y_u32x4* __restrict__ src,
                                                          y_u32x2* __restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    const y_u32x4 v = __builtin_nontemporal_load(src + i);
    __builtin_nontemporal_store(y_u32x2{v.x ^ v.z, v.y ^ v.w}, dst + i);
  }
}
__global__ __launch_bounds__(256) void stream_write_kernel(y_u32x4* __restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) __builtin_nontemporal_store(y_u32x4{(uint32_t)i, 1u, 2u, 3u}, dst + i);
}
// Matrix-pipe yardstick: nothing but independent scaled fp8 MFMAs on operands held in registers
// (no LDS, no memory traffic after the first loads), one wave per SIMD.  What a launch of it
// sustains is what the power limit leaves of the matrix peak for the given operand bits.
typedef int y_v8i __attribute__((ext_vector_type(8)));
typedef float y_v16f __attribute__((ext_vector_type(16)));
typedef float y_v4f __attribute__((ext_vector_type(4)));

// The same 64 MFMAs per iteration (8 x 8 sub-tiles of 16x16x128) in a fixed order, as assembly so
// that the order is what runs.  HOLD = how many MFMAs in a row share one operand fragment:
//   8: sub-tile row i meets all eight columns in a row (a[i] stays, b changes)
//   4: the order of the GEMM's K loop: four quarters a0 x b0, a1 x b0, a1 x b1, a0 x b1 over halves
//      of four fragments, the held operand changing sides from quarter to quarter
//   1: along diagonals, both fragments change with every MFMA
template <int HOLD>
__global__ __launch_bounds__(256) void mfma_order_kernel(const y_v8i* __restrict__ src, float* __restrict__ dst,
                                                         int iters) {
  const int lane = threadIdx.x;
  y_v8i a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[i * 256 + lane];
    b[i] = src[(8 + i) * 256 + lane];
  }
  const int sc = 0x7f7f7f7f;
  y_v4f acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = y_v4f{0.f, 0.f, 0.f, 0.f};
  auto one = [&](int i, int j) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel:[0,0,0] op_sel_hi:[0,0,0]"
                 : "+a"(acc[i][j])
                 : "v"(b[j]), "v"(a[i]), "v"(sc));
  };
  for (int it = 0; it < iters; ++it) {
    if constexpr (HOLD == 8) {
#pragma unroll
      for (int k = 0; k < 64; ++k) one(k >> 3, k & 7);
    } else if constexpr (HOLD == 4) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ah = (q == 1 || q == 2) ? 1 : 0, bh = q >= 2 ? 1 : 0;
        const bool amajor = q == 0 || q == 3;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          const int tm = amajor ? k >> 2 : k & 3, tn = amajor ? k & 3 : k >> 2;
          one(4 * ah + tm, 4 * bh + tn);
        }
      }
    } else {
#pragma unroll
      for (int k = 0; k < 64; ++k) one(k & 7, ((k & 7) + (k >> 3)) & 7);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  dst[blockIdx.x * 256 + lane] = s;
}

template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_only_kernel(const y_v8i* __restrict__ src, float* __restrict__ dst,
                                                        int iters) {
  const int lane = threadIdx.x;
  constexpr int kF = SHAPE == 32 ? 4 : 8;  // fragments per operand: 16 or 64 accumulator tiles, 256 registers
  y_v8i a[kF], b[kF];
#pragma unroll
  for (int i = 0; i < kF; ++i) {
    a[i] = src[i * 256 + lane];
    b[i] = src[(kF + i) * 256 + lane];
  }
  const int sc = 0x7f7f7f7f;  // E8M0 127 = 1.0 in every scale byte
  float s = 0.f;
  if constexpr (SHAPE == 32) {
    y_v16f acc[kF][kF];
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
      for (int j = 0; j < kF; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < kF; ++i)
#pragma unroll
        for (int j = 0; j < kF; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, sc, 0, sc);
    }
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
      for (int j = 0; j < kF; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  } else {
    y_v4f acc[kF][kF];
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
      for (int j = 0; j < kF; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < kF; ++i)
#pragma unroll
        for (int j = 0; j < kF; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, sc, 0, sc);
    }
#pragma unroll
    for (int i = 0; i < kF; ++i)
#pragma unroll
      for (int j = 0; j < kF; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  }
  dst[blockIdx.x * 256 + lane] = s;
}
}  // namespace mx

extern "C" int mx_debug_mfma_only(int shape, const void* operands, void* out, int workgroups, int iters,
                                  void* stream) {
  if (shape == 1601 || shape == 1604 || shape == 1608) {  // 16x16x128 in a fixed order, see mfma_order_kernel
    if (!operands || !out || workgroups <= 0 || iters <= 0 || ((uintptr_t)operands & 31)) return MX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const dim3 g((unsigned)workgroups), b(256);
    if (shape == 1601)
      hipLaunchKernelGGL(mx::mfma_order_kernel<1>, g, b, 0, st, (const mx::y_v8i*)operands, (float*)out, iters);
    else if (shape == 1604)
      hipLaunchKernelGGL(mx::mfma_order_kernel<4>, g, b, 0, st, (const mx::y_v8i*)operands, (float*)out, iters);
    else
      hipLaunchKernelGGL(mx::mfma_order_kernel<8>, g, b, 0, st, (const mx::y_v8i*)operands, (float*)out, iters);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
  }
  if ((shape != 16 && shape != 32) || !operands || !out || workgroups <= 0 || iters <= 0 ||
      ((uintptr_t)operands & 31))
    return MX_ERR_INVALID_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (shape == 32)
    hipLaunchKernelGGL(mx::mfma_only_kernel<32>, dim3((unsigned)workgroups), dim3(256), 0, st,
                       (const mx::y_v8i*)operands, (float*)out, iters);
  else
    hipLaunchKernelGGL(mx::mfma_only_kernel<16>, dim3((unsigned)workgroups), dim3(256), 0, st,
                       (const mx::y_v8i*)operands, (float*)out, iters);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

extern "C" int mx_debug_stream(int kind, const void* src, void* dst, int64_t bytes, void* stream) {
  if (bytes <= 0 || bytes % 16 || kind < 0 || kind > 3) return MX_ERR_INVALID_ARG;
  if ((kind != 2 && (!src || ((uintptr_t)src & 15))) || !dst || ((uintptr_t)dst & 15)) return MX_ERR_INVALID_ARG;
  const int64_t n = bytes / 16;
  hipStream_t st = (hipStream_t)stream;
  if (kind == 0)
    hipLaunchKernelGGL(mx::stream_copy_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const mx::y_u32x4*)src, (mx::y_u32x4*)dst, n);
  else if (kind == 1)
    hipLaunchKernelGGL(mx::stream_read_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, st,
                       (const mx::y_u32x4*)src, n, (mx::y_u32x4*)dst);
  else if (kind == 3)
    hipLaunchKernelGGL(mx::stream_2to1_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (const mx::y_u32x4*)src, (mx::y_u32x2*)dst, n);
  else
    hipLaunchKernelGGL(mx::stream_write_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                       (mx::y_u32x4*)dst, n);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
