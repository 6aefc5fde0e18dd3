// Per-token log-probabilities of chosen tokens from bf16 logits, and their backward: the hot
// op of the policy-gradient loss around the model.  HBM-bound row streaming: the forward reads
// each logit once (online log-sum-exp in float32), the backward reads it once more and writes
// the bf16 gradient; no float32 copy of the logits and no [rows, vocab] log-softmax exist.
#include "mx_common.h"

namespace mx {

constexpr int kLpThreads = 256;

__device__ __forceinline__ float lp_bf16(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

// (max, sum of exp(x - max)) of two partial results.
__device__ __forceinline__ void lse_merge(float& m, float& s, float m2, float s2) {
  const float mm = fmaxf(m, m2);
  // exp(-inf - (-inf)) would be NaN: an empty partial result contributes nothing
  const float a = m == -__builtin_inff() ? 0.f : s * __expf(m - mm);
  const float b = m2 == -__builtin_inff() ? 0.f : s2 * __expf(m2 - mm);
  m = mm;
  s = a + b;
}

// One workgroup per row: lse[r] = log sum_v exp(x[r, v]); lp[r] = x[r, target[r]] - lse[r]
// (NaN if the target is outside [0, vocab)).
__global__ __launch_bounds__(kLpThreads) void token_logprob_fwd_kernel(
    const uint16_t* __restrict__ logits, int64_t ld, int64_t vocab, const int64_t* __restrict__ target,
    float* __restrict__ lp, float* __restrict__ lse) {
  __shared__ float sm[kLpThreads / 64], ss[kLpThreads / 64];
  const int64_t r = blockIdx.x;
  const uint16_t* row = logits + r * ld;
  const int tid = threadIdx.x;
  float m = -__builtin_inff(), s = 0.f;
  const int64_t chunks = vocab / 8;
  for (int64_t c = tid; c < chunks; c += kLpThreads) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + c * 8));
    const float x[8] = {lp_bf16(v.x & 0xFFFFu), lp_bf16(v.x >> 16), lp_bf16(v.y & 0xFFFFu), lp_bf16(v.y >> 16),
                        lp_bf16(v.z & 0xFFFFu), lp_bf16(v.z >> 16), lp_bf16(v.w & 0xFFFFu), lp_bf16(v.w >> 16)};
    float cm = x[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) cm = fmaxf(cm, x[e]);
    if (cm > m) {  // rescale the running sum to the new maximum
      s = m == -__builtin_inff() ? 0.f : s * __expf(m - cm);
      m = cm;
    }
    if (m != -__builtin_inff()) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s += __expf(x[e] - m);
    }
  }
  for (int64_t i = chunks * 8 + tid; i < vocab; i += kLpThreads) lse_merge(m, s, lp_bf16(row[i]), 1.f);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) lse_merge(m, s, __shfl_xor(m, off, 64), __shfl_xor(s, off, 64));
  if ((tid & 63) == 0) {
    sm[tid >> 6] = m;
    ss[tid >> 6] = s;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < kLpThreads / 64; ++w) lse_merge(m, s, sm[w], ss[w]);
    const float l = m + __logf(s);
    const int64_t t = target[r];
    lse[r] = l;
    lp[r] = (t >= 0 && t < vocab) ? lp_bf16(row[t]) - l : __builtin_nanf("");
  }
}

// dlogits[r, v] = g[r] * ((v == target[r]) - exp(x[r, v] - lse[r])) rounded to bf16.
__global__ __launch_bounds__(kLpThreads) void token_logprob_bwd_kernel(
    const uint16_t* __restrict__ logits, int64_t ld, int64_t vocab, const int64_t* __restrict__ target,
    const float* __restrict__ lse, const float* __restrict__ g, uint16_t* __restrict__ dlogits,
    int64_t ldd) {
  const int64_t r = blockIdx.y;
  const uint16_t* row = logits + r * ld;
  uint16_t* drow = dlogits + r * ldd;
  const float l = lse[r], gr = g[r];
  const int64_t t = target[r];
  const int64_t chunks = vocab / 8;
  auto grad = [&](float x, int64_t v) {
    const float p = __expf(x - l);
    const float d = gr * ((v == t ? 1.f : 0.f) - p);
    const uint32_t u = __float_as_uint(d);
    return (u & 0x7FFFFFFFu) > 0x7F800000u ? ((u >> 16) | 0x40u) : ((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
  };
  for (int64_t c = (int64_t)blockIdx.x * kLpThreads + threadIdx.x; c < chunks;
       c += (int64_t)gridDim.x * kLpThreads) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row + c * 8));
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      o[e] = grad(lp_bf16(w[e] & 0xFFFFu), c * 8 + 2 * e) | (grad(lp_bf16(w[e] >> 16), c * 8 + 2 * e + 1) << 16);
    __builtin_nontemporal_store(u32x4{o[0], o[1], o[2], o[3]}, reinterpret_cast<u32x4*>(drow + c * 8));
  }
  if (blockIdx.x == 0)
    for (int64_t i = chunks * 8 + threadIdx.x; i < vocab; i += kLpThreads)
      drow[i] = (uint16_t)grad(lp_bf16(row[i]), i);
}

}  // namespace mx

using namespace mx;

extern "C" int mx_token_logprob_fwd(const void* logits, int64_t rows, int64_t vocab, int64_t ld,
                                    const int64_t* target, float* logprob, float* lse, void* stream) {
  if (rows < 0 || vocab <= 0 || ld < vocab) return MX_ERR_INVALID_ARG;
  if (rows == 0) return MX_OK;
  if (!logits || !target || !logprob || !lse) return MX_ERR_INVALID_ARG;
  if (ld % 8 || ((uintptr_t)logits & 15) || ((uintptr_t)target & 7) || ((uintptr_t)logprob & 3) ||
      ((uintptr_t)lse & 3))
    return MX_ERR_ALIGNMENT;
  if (rows > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(token_logprob_fwd_kernel, dim3((unsigned)rows), dim3(kLpThreads), 0,
                     (hipStream_t)stream, (const uint16_t*)logits, ld, vocab, target, logprob, lse);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

extern "C" int mx_token_logprob_bwd(const void* logits, int64_t rows, int64_t vocab, int64_t ld,
                                    const int64_t* target, const float* lse, const float* grad_logprob,
                                    void* dlogits, int64_t ldd, void* stream) {
  if (rows < 0 || vocab <= 0 || ld < vocab || ldd < vocab) return MX_ERR_INVALID_ARG;
  if (rows == 0) return MX_OK;
  if (!logits || !target || !lse || !grad_logprob || !dlogits) return MX_ERR_INVALID_ARG;
  if (ld % 8 || ldd % 8 || ((uintptr_t)logits & 15) || ((uintptr_t)dlogits & 15) ||
      ((uintptr_t)target & 7) || ((uintptr_t)lse & 3) || ((uintptr_t)grad_logprob & 3))
    return MX_ERR_ALIGNMENT;
  if (rows > 65535) return MX_ERR_UNSUPPORTED;  // one grid row per token row
  const int64_t chunks = vocab / 8;
  int64_t gx = (chunks + kLpThreads - 1) / kLpThreads;
  gx = gx < 1 ? 1 : (gx > 64 ? 64 : gx);
  hipLaunchKernelGGL(token_logprob_bwd_kernel, dim3((unsigned)gx, (unsigned)rows), dim3(kLpThreads), 0,
                     (hipStream_t)stream, (const uint16_t*)logits, ld, vocab, target, lse, grad_logprob,
                     (uint16_t*)dlogits, ldd);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}
