// Shared device helpers for the gfx950 MXFP8 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "mxfp8.h"

namespace mx {

constexpr int kBlock = 32;  // elements per E8M0 scale

typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  us2 x = __builtin_bit_cast(us2, a), y = __builtin_bit_cast(us2, b);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(x, y));
}

// Lane exchange inside a quad / row through DPP (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ uint32_t dpp(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}
constexpr int kQuadXor1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int kQuadXor2 = 0x4E;  // quad_perm:[2,3,0,1]

// E8M0 byte from the bf16 bit pattern of the block's max magnitude (sign bit clear).
//   FLOOR: floor(log2 amax) - 8          RCEIL: ceil(log2(amax / 448))
// both read off the exponent / mantissa fields, clamped to [0, 254]; amax == 0 -> 0,
// NaN -> 255.
template <int MODE>
__device__ __forceinline__ uint32_t scale_byte(uint32_t amax_bits) {
  int expf = (int)(amax_bits >> 7);
  int b = expf - 8;
  if (MODE == MX_SCALE_RCEIL) b += ((amax_bits & 0x7F) > 0x60) ? 1 : 0;
  b = b < 0 ? 0 : (b > 254 ? 254 : b);
  if (amax_bits == 0) b = 0;
  if (amax_bits > 0x7F80) b = 255;
  return (uint32_t)b;
}

// float factor 2^(127 - byte) applied before narrowing; byte 0 -> 2^126 (FLOOR) or 1
// (RCEIL); byte 255 (NaN block) -> 0.
template <int MODE>
__device__ __forceinline__ float scale_multiplier(uint32_t byte) {
  uint32_t bits = (254u - byte) << 23;
  if (byte == 0) bits = (MODE == MX_SCALE_FLOOR) ? 0x7E800000u : 0x3F800000u;
  if (byte >= 254) bits = (byte == 254) ? 0x00400000u : 0u;
  return __uint_as_float(bits);
}

// Two bf16 (packed in one dword) -> two saturating e4m3 codes in the low or high half of
// `old`.  v_med3_f32 clamps to +-448 so the narrowing never overflows; the hardware convert
// rounds to nearest even, subnormals included.
template <bool HIGH>
__device__ __forceinline__ uint32_t cvt2(uint32_t w, float mult, uint32_t old) {
  float lo = __uint_as_float(w << 16) * mult;
  float hi = __uint_as_float(w & 0xFFFF0000u) * mult;
  lo = __builtin_amdgcn_fmed3f(lo, -448.0f, 448.0f);
  hi = __builtin_amdgcn_fmed3f(hi, -448.0f, 448.0f);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, (int)old, HIGH);
}

// Two floats -> two codes (same contract as cvt2, inputs already scaled).
template <bool HIGH>
__device__ __forceinline__ uint32_t cvt2f(float lo, float hi, uint32_t old) {
  lo = __builtin_amdgcn_fmed3f(lo, -448.0f, 448.0f);
  hi = __builtin_amdgcn_fmed3f(hi, -448.0f, 448.0f);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, (int)old, HIGH);
}

// Code of one bf16 lane inside a block whose amax is NaN: NaN lanes keep NaN (0x7F) with
// their sign, every other lane becomes a signed zero.
__device__ __forceinline__ uint32_t nan_block_code(uint32_t bf16_bits) {
  uint32_t sign = (bf16_bits >> 8) & 0x80u;
  return ((bf16_bits & 0x7FFFu) > 0x7F80u ? 0x7Fu : 0u) | sign;
}
__device__ __forceinline__ uint32_t nan_block_codes2(uint32_t w) {
  return nan_block_code(w & 0xFFFFu) | (nan_block_code(w >> 16) << 8);
}

// Byte offset of scale (row, blk) in MX_SCALES_MFMA order; ks_n = ceil(nblk / 2).
// Groups of 128 rows x 2 blocks (one 64-deep K step) are 256 contiguous bytes: for lane l and
// byte t the entry is row = 32 t + (l & 31), block = l >> 5 -- one dword per lane carries the
// scales that a 32x32x64 MFMA lane needs for four 32-row sub-tiles (a 16x16x128 MFMA lane: for
// four 16-row sub-tiles 32 rows apart).
__device__ __host__ __forceinline__ int64_t mfma_scale_offset(int64_t row, int64_t blk,
                                                              int64_t ks_n) {
  return (((row >> 7) * ks_n + (blk >> 1)) << 8) + ((((blk & 1) << 5) + (row & 31)) << 2) +
         ((row & 127) >> 5);
}
__device__ __host__ __forceinline__ int64_t mfma_scale_bytes(int64_t rows, int64_t nblk) {
  return ((rows + 127) >> 7) * ((nblk + 1) >> 1) * 256;
}

// ---- per-device host state -------------------------------------------------------------------
// A process may drive several GPUs, from several threads: whatever the host side remembers about
// "the device" (its CU count, whether a kernel's dynamic-LDS limit has been raised there) is kept
// per device ordinal in atomics.  Two threads that race on the first call both do the same
// idempotent set-up.
constexpr int kMaxDevices = 64;

// Ordinal of the calling thread's current device, -1 if it cannot be asked or is out of range.
inline int current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
  return dev;
}

// Compute units of the current device (0: unknown).
inline int current_device_cus() {
  static std::atomic<int> cus[kMaxDevices];
  const int dev = current_device();
  if (dev < 0) return 0;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Raises a kernel's dynamic-LDS limit once per device.  `done` is the kernel's own table
// (a function-local static of the launcher, one per template instance).
inline bool raise_lds_limit(const void* kernel, int bytes, std::atomic<bool> (&done)[kMaxDevices]) {
  const int dev = current_device();
  if (dev < 0) return false;
  if (!done[dev].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    done[dev].store(true, std::memory_order_release);
  }
  return true;
}

}  // namespace mx
