// Dense MXFP8 GEMM entry point: D[M,N] = deq(A)[M,K] * deq(B)[N,K]^T (bf16 out).
#include <mutex>

#include "mx_gemm_tile.h"

namespace mx {

struct DenseArgs {
  const uint8_t* a_codes;
  const uint8_t* a_scales;
  const uint8_t* b_codes;
  const uint8_t* b_scales;
  uint16_t* d;
  int64_t M, N, K, ldd;
  int64_t ldk;  // bytes between operand rows (>= K)
};

template <int BM, int BN>
__global__ __launch_bounds__(256, 1) void gemm_nt_kernel(DenseArgs p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  using Tile = GemmTile<BM, BN, false, false>;
  const int64_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int64_t tm, tn;
  if (!map_tile(tiles_m, tiles_n, tm, tn)) return;
  const int64_t ks_n = (p.K / 32 + 1) / 2;
  Operand A{p.a_codes + tm * BM * p.ldk, p.ldk, p.M - tm * BM,
            p.a_scales + tm * (BM / 128) * ks_n * 256, ks_n};
  Operand B{p.b_codes + tn * BN * p.ldk, p.ldk, p.N - tn * BN,
            p.b_scales + tn * (BN / 128) * ks_n * 256, ks_n};
  Tile::run(smem, A, B, 0, p.K, p.d + tm * BM * p.ldd + tn * BN, p.ldd);
}

template <int BM, int BN>
static int launch_dense(const DenseArgs& p, hipStream_t st) {
  using Tile = GemmTile<BM, BN, false, false>;
  auto kern = gemm_nt_kernel<BM, BN>;
  static std::atomic<bool> configured[kMaxDevices];  // a per-function, per-device setting
  if (!raise_lds_limit(reinterpret_cast<const void*>(kern), Tile::kLdsBytes, configured)) return MX_ERR_LAUNCH;
  const int64_t nb = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  const int64_t grid = (nb + 7) / 8 * 8;
  if (grid > 0x7FFFFFFF) return MX_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), Tile::kLdsBytes, st, p);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

}  // namespace mx

using namespace mx;

namespace mx {
int launch_gemm_nt32(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                     const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                     int64_t ldk, int64_t ldd, hipStream_t st);
}
namespace mx {
int splitk_slices(int64_t M, int64_t N, int64_t K);
int launch_gemm_nt32_splitk(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                            const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                            int64_t ldk, int64_t ldd, int slices, void* workspace, hipStream_t st);
}
// Test hooks (include/mxfp8_debug.h), process-wide.
// 0: pick by shape; 1 / 2: the 16x16x128 tile kernel with 256x256 / 128x128 tiles for every
// shape; 3: the persistent kernel wherever it is legal (comparison runs and tests)
static std::atomic<int> force_kernel{0};
extern "C" void mx_debug_force_kernel(int which) { force_kernel = which; }
namespace mx { void set_debug_grid(int g); }
extern "C" void mx_debug_set_grid(int g) { mx::set_debug_grid(g); }
#ifdef MX_TIMING_BUILD
namespace mx { void set_debug_prof(uint64_t* buf); }
// device buffer of 256*4*8 uint64 receiving per-wave cycle counts; nullptr switches timing off
extern "C" void mx_debug_set_prof(void* buf) { mx::set_debug_prof((uint64_t*)buf); }
#endif

static int check_dense(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                       const uint8_t* b_scales, const void* d, int64_t M, int64_t N, int64_t K,
                       int64_t ldd) {
  if (M < 0 || N < 0 || K < 0 || ldd < N) return MX_ERR_INVALID_ARG;
  if (M == 0 || N == 0) return MX_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !d) return MX_ERR_INVALID_ARG;
  if (K % 32 || K == 0) return MX_ERR_ALIGNMENT;  // K == 0 would need a zero fill: not a linear
  if (((uintptr_t)a_codes & 15) || ((uintptr_t)b_codes & 15) || ((uintptr_t)a_scales & 3) ||
      ((uintptr_t)b_scales & 3) || ((uintptr_t)d & 1) || (K % 16))
    return MX_ERR_ALIGNMENT;
  if (256 * K > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  return MX_OK;
}

// What the persistent kernel (mx_gemm32.hip) needs beyond the general checks.
static bool persistent_ok(const void* d, int64_t N, int64_t K, int64_t ldd, int64_t ldk = 0) {
  if (ldk == 0) ldk = K;
  return !(K % 128 || ldk % 128 || (uint64_t)ldk * 256 > 0x7FFFFFFFull || N % 8 || ldd % 8 || ((uintptr_t)d & 15) ||
           (uint64_t)ldd * 512 > 0x7FFFFFFFull);
}

// mx_gemm_nt with operand rows `ldk` bytes apart (ldk >= K, a multiple of 16).
static int gemm_nt_pitched(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                           const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K, int64_t ldk,
                           int64_t ldd, void* stream) {
  const int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  if (ldk < K) return MX_ERR_INVALID_ARG;
  if (ldk % 16) return MX_ERR_ALIGNMENT;
  if (256 * ldk > 0x7FFFFFFFll) return MX_ERR_UNSUPPORTED;
  DenseArgs p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, ldk};
  hipStream_t st = (hipStream_t)stream;
  if (M <= 128 || N <= 128 || force_kernel == 2) return launch_dense<128, 128>(p, st);
  // Few 256x256 tiles leave most CUs of the persistent kernel idle when the contraction is not
  // split: up to 3/8 of the CUs' worth of tiles, four times as many 128x128 tiles finish sooner
  // (measured: 64 tiles 58 vs 71 us at K = 8192; 128 tiles 46 vs 43 us).
  int num_cus = current_device_cus();
  if (num_cus == 0) num_cus = 256;
  const int64_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256);
  if (force_kernel == 0 && tiles256 * 8 <= (int64_t)num_cus * 3) return launch_dense<128, 128>(p, st);
  if (force_kernel == 1 || !persistent_ok(d, N, K, ldd, ldk)) return launch_dense<256, 256>(p, st);
  return launch_gemm_nt32(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldk, ldd, st);
}

extern "C" int mx_gemm_nt(const uint8_t* a_codes, const uint8_t* a_scales,
                          const uint8_t* b_codes, const uint8_t* b_scales, void* d, int64_t M,
                          int64_t N, int64_t K, int64_t ldd, void* stream) {
  return gemm_nt_pitched(a_codes, a_scales, b_codes, b_scales, d, M, N, K, K, ldd, stream);
}

namespace mx {
int launch_gemm_nt32_pair(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                          const uint8_t* b_scales, const uint8_t* a2_codes, const uint8_t* a2_scales,
                          const uint8_t* b2_codes, const uint8_t* b2_scales, void* d, int64_t M,
                          int64_t N, int64_t K, int64_t ldk, int64_t ldd, hipStream_t st);
}

// The forms over two operand sets exist for the persistent kernel only, dense rows (ldk == K) or
// pitched: other shapes are the caller's two GEMMs (and an add).
extern "C" int mx_gemm_nt_pair_ld(const uint8_t* a_codes, const uint8_t* a_scales,
                                  const uint8_t* b_codes, const uint8_t* b_scales,
                                  const uint8_t* a2_codes, const uint8_t* a2_scales,
                                  const uint8_t* b2_codes, const uint8_t* b2_scales, void* d,
                                  int64_t M, int64_t N, int64_t K, int64_t ldk, int64_t ldd,
                                  void* stream) {
  int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc == MX_OK) rc = check_dense(a2_codes, a2_scales, b2_codes, b2_scales, d, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  if (ldk < K) return MX_ERR_INVALID_ARG;
  if (M <= 128 || N <= 128 || !persistent_ok(d, N, K, ldd, ldk) || force_kernel == 1 || force_kernel == 2)
    return MX_ERR_UNSUPPORTED;
  return launch_gemm_nt32_pair(a_codes, a_scales, b_codes, b_scales, a2_codes, a2_scales, b2_codes,
                               b2_scales, d, M, N, K, ldk, ldd, (hipStream_t)stream);
}

extern "C" int mx_gemm_nt_pair(const uint8_t* a_codes, const uint8_t* a_scales,
                               const uint8_t* b_codes, const uint8_t* b_scales,
                               const uint8_t* a2_codes, const uint8_t* a2_scales,
                               const uint8_t* b2_codes, const uint8_t* b2_scales, void* d,
                               int64_t M, int64_t N, int64_t K, int64_t ldd, void* stream) {
  return mx_gemm_nt_pair_ld(a_codes, a_scales, b_codes, b_scales, a2_codes, a2_scales, b2_codes, b2_scales, d,
                            M, N, K, K, ldd, stream);
}

namespace mx {
int launch_gemm_nt32_two_b(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                           const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk, int64_t ldd,
                           hipStream_t st);
int launch_gemm_nt32_two_a(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* a2_codes,
                           const uint8_t* a2_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk, int64_t ldd,
                           hipStream_t st);
}

// Two products that share an operand, one launch of the persistent kernel; other shapes are the
// caller's two mx_gemm_nt calls.
extern "C" int mx_gemm_nt_shared_a_ld(const uint8_t* a_codes, const uint8_t* a_scales,
                                      const uint8_t* b_codes, const uint8_t* b_scales,
                                      const uint8_t* b2_codes, const uint8_t* b2_scales, void* d,
                                      void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk,
                                      int64_t ldd, void* stream) {
  int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc == MX_OK) rc = check_dense(a_codes, a_scales, b2_codes, b2_scales, d2, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  if (ldk < K) return MX_ERR_INVALID_ARG;
  if (M <= 128 || N <= 128 || !persistent_ok(d, N, K, ldd, ldk) || !persistent_ok(d2, N, K, ldd, ldk) ||
      force_kernel == 1 || force_kernel == 2)
    return MX_ERR_UNSUPPORTED;
  return launch_gemm_nt32_two_b(a_codes, a_scales, b_codes, b_scales, b2_codes, b2_scales, d, d2, M, N,
                                K, ldk, ldd, (hipStream_t)stream);
}

extern "C" int mx_gemm_nt_shared_a(const uint8_t* a_codes, const uint8_t* a_scales,
                                   const uint8_t* b_codes, const uint8_t* b_scales,
                                   const uint8_t* b2_codes, const uint8_t* b2_scales, void* d,
                                   void* d2, int64_t M, int64_t N, int64_t K, int64_t ldd,
                                   void* stream) {
  return mx_gemm_nt_shared_a_ld(a_codes, a_scales, b_codes, b_scales, b2_codes, b2_scales, d, d2, M, N, K, K,
                                ldd, stream);
}

extern "C" int mx_gemm_nt_shared_b_ld(const uint8_t* a_codes, const uint8_t* a_scales,
                                      const uint8_t* a2_codes, const uint8_t* a2_scales,
                                      const uint8_t* b_codes, const uint8_t* b_scales, void* d,
                                      void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk,
                                      int64_t ldd, void* stream) {
  int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc == MX_OK) rc = check_dense(a2_codes, a2_scales, b_codes, b_scales, d2, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  if (ldk < K) return MX_ERR_INVALID_ARG;
  if (M <= 128 || N <= 128 || !persistent_ok(d, N, K, ldd, ldk) || !persistent_ok(d2, N, K, ldd, ldk) ||
      force_kernel == 1 || force_kernel == 2)
    return MX_ERR_UNSUPPORTED;
  return launch_gemm_nt32_two_a(a_codes, a_scales, a2_codes, a2_scales, b_codes, b_scales, d, d2, M, N,
                                K, ldk, ldd, (hipStream_t)stream);
}

extern "C" int mx_gemm_nt_shared_b(const uint8_t* a_codes, const uint8_t* a_scales,
                                   const uint8_t* a2_codes, const uint8_t* a2_scales,
                                   const uint8_t* b_codes, const uint8_t* b_scales, void* d,
                                   void* d2, int64_t M, int64_t N, int64_t K, int64_t ldd,
                                   void* stream) {
  return mx_gemm_nt_shared_b_ld(a_codes, a_scales, a2_codes, a2_scales, b_codes, b_scales, d, d2, M, N, K, K,
                                ldd, stream);
}

extern "C" int64_t mx_gemm_nt_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 128 || N <= 128 || K <= 0 || N % 8 || (uint64_t)N * 1024 > 0x7FFFFFFFull) return 0;
  const int s = splitk_slices(M, N, K);
  return s > 1 ? (int64_t)s * M * N * 4 : 0;
}

extern "C" int mx_gemm_nt_ld(const uint8_t* a_codes, const uint8_t* a_scales,
                             const uint8_t* b_codes, const uint8_t* b_scales, void* d, int64_t M,
                             int64_t N, int64_t K, int64_t ldk, int64_t ldd, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  const int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  if (ldk < K) return MX_ERR_INVALID_ARG;
  const int64_t need = force_kernel == 0 ? mx_gemm_nt_workspace_bytes(M, N, K) : 0;
  if (need == 0 || !workspace || workspace_bytes < need || ((uintptr_t)workspace & 15) ||
      !persistent_ok(d, N, K, ldd, ldk))
    return gemm_nt_pitched(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldk, ldd, stream);
  return launch_gemm_nt32_splitk(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldk, ldd,
                                 (int)(need / (M * N * 4)), workspace, (hipStream_t)stream);
}

extern "C" int mx_gemm_nt_ws(const uint8_t* a_codes, const uint8_t* a_scales,
                             const uint8_t* b_codes, const uint8_t* b_scales, void* d, int64_t M,
                             int64_t N, int64_t K, int64_t ldd, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  return mx_gemm_nt_ld(a_codes, a_scales, b_codes, b_scales, d, M, N, K, K, ldd, workspace, workspace_bytes,
                       stream);
}

// ---- the split GEMM for callers that cannot allocate -------------------------------------------
// The float32 partial tiles of the split along K live in a file-scope device array instead of a
// caller-provided workspace.  Every GPU holds its own copy of the array at its own address until
// the process ends; the address is looked up once per device and is what the kernels receive.
constexpr int64_t kScratchBytes = 64ll << 20;
static __device__ __align__(256) uint8_t scratch[kScratchBytes];

static void* scratch_ptr[kMaxDevices];  // device address of `scratch` per GPU, nullptr: not looked up yet
static std::mutex scratch_mutex;

// Device address of this GPU's scratch array (nullptr: the lookup failed).
static void* scratch_of_current_device() {
  const int dev = current_device();
  if (dev < 0) return nullptr;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    scratch_ptr[dev] = ptr;
  }
  return scratch_ptr[dev];
}

extern "C" int64_t mx_gemm_nt_static_max_bytes(void) { return kScratchBytes; }

extern "C" int mx_gemm_nt_static(const uint8_t* a_codes, const uint8_t* a_scales,
                                 const uint8_t* b_codes, const uint8_t* b_scales, void* d,
                                 int64_t M, int64_t N, int64_t K, int64_t ldd, void* stream) {
  const int rc = check_dense(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd);
  if (rc != MX_OK || M == 0 || N == 0) return rc;
  // the size check stands on the shape alone, whatever the test hooks say
  const int64_t need = mx_gemm_nt_workspace_bytes(M, N, K);
  if (need > kScratchBytes && persistent_ok(d, N, K, ldd)) return MX_ERR_SCRATCH_TOO_SMALL;
  if (need == 0 || force_kernel != 0 || !persistent_ok(d, N, K, ldd))  // not split: no scratch involved
    return mx_gemm_nt(a_codes, a_scales, b_codes, b_scales, d, M, N, K, ldd, stream);
  void* ws = scratch_of_current_device();
  if (!ws) return MX_ERR_LAUNCH;
  return launch_gemm_nt32_splitk(a_codes, a_scales, b_codes, b_scales, d, M, N, K, K, ldd,
                                 (int)(need / (M * N * 4)), ws, (hipStream_t)stream);
}
