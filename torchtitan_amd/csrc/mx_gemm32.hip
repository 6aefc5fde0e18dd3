// Dense MXFP8 GEMM for large shapes: persistent 256x256 tiles on v_mfma_scale_f32_32x32x64_f8f6f4.
//
//   D[M,N] (bf16) = deq(A)[M,K] * deq(B)[N,K]^T, fp32 accumulate.
//
// One workgroup (4 waves, 2x2, 128x128 each = 256 accumulator registers per lane) per CU walks
// a list of output tiles; the K loop of all its tiles is one flat stream of 64-deep steps, so
// the loads of the next tile's first steps are already in flight while a tile is written out.
//
// Per step and per CU: 32 KB of codes + 1 KB of scales go global -> LDS with
// buffer_load ... lds into a ring of NSTAGE stages (issued NSTAGE steps ahead), 64 KB of
// fragments go LDS -> VGPR (double-buffered in registers, read one step ahead, conflict-free
// under the b128 pass grouping), and 16 MFMAs per wave (1024 MFMA cycles) consume them.
// One barrier per step.
//
// Operand layout of the 32x32x64 f8 MFMA (measured): lane (i = l & 31, j = l >> 5) holds row i,
// K bytes [16j, 16j+16) in registers 0-3 and [32+16j, 32+16j+16) in registers 4-7; the scale
// of 32-element block b is taken from lane group b.  With the first operand = B rows and the
// second = A rows, a lane ends up with D[row = l & 31][col = 8q + 4j + 0..3], q = 0..3.
#include "mx_gemm_tile.h"

namespace mx {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kT32 = 256;                       // tile edge (M and N)
constexpr int kK32 = 64;                        // K per step
constexpr int kCodes32 = 2 * kT32 * kK32;       // 32 KB: A rows then B rows, 64 B per row
constexpr int kStage32 = kCodes32 + 1024;       // + 4 x 256 B of scales (A group 0,1, B group 0,1)
constexpr int kVmPerStep = 9;                   // VM instructions per wave per step (8 + 1)

struct Dense32Args {
  const uint8_t* a_codes;
  const uint8_t* a_scales;
  const uint8_t* b_codes;
  const uint8_t* b_scales;
  uint16_t* d;
  int64_t M, N, K, ldd;
  uint64_t* prof;  // timing build only: per wave {vmcnt wait, barrier wait, step body} cycles
};

// Tile order: 8-tall column-major panels, so tiles that run together share A and B panels.
// 32-bit arithmetic: the tile count of any supported shape is far below 2^31.
__device__ __forceinline__ void tile_coords(uint32_t t, uint32_t tiles_m, uint32_t tiles_n,
                                            uint32_t& tm, uint32_t& tn) {
  constexpr uint32_t kGroupM = 8;
  const uint32_t width = kGroupM * tiles_n;
  const uint32_t group = t / width;
  const uint32_t first_m = group * kGroupM;
  const uint32_t gsz = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  const uint32_t in = t - group * width;
  tn = in / gsz;
  tm = first_m + (in - tn * gsz);
}

struct Frags32 {
  v8i a[4];
  v8i b[4];
  uint32_t sa, sb;
};

template <int NSTAGE, bool PROF>
__global__ __launch_bounds__(256, 1) void gemm_nt32_kernel(Dense32Args p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lj = lane >> 5;

  // ---- this workgroup's tile list: XCD x (= blockIdx % 8) owns one contiguous run of tiles,
  //      its workgroups take them round-robin, so the XCD's CUs work on neighbouring tiles
  const uint32_t tiles_m = (uint32_t)((p.M + kT32 - 1) / kT32), tiles_n = (uint32_t)((p.N + kT32 - 1) / kT32);
  const uint32_t nb = tiles_m * tiles_n;
  const uint32_t wgs_per_xcd = gridDim.x / 8;
  const uint32_t xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
  const uint32_t per_xcd = (nb + 7) / 8;
  const uint32_t t_lo = xcd * per_xcd + idx;
  const uint32_t t_hi = (xcd + 1) * per_xcd < nb ? (xcd + 1) * per_xcd : nb;
  const uint32_t n_my = t_lo < t_hi ? (t_hi - t_lo + wgs_per_xcd - 1) / wgs_per_xcd : 0;
  if (n_my == 0) return;
  const uint32_t K = (uint32_t)p.K;          // a multiple of 128 for this kernel
  const uint32_t nsteps = K / kK32;          // even, >= 2
  const uint32_t ks_n = nsteps;              // 64-deep steps per 128-row scale group

  // ---- per-lane constants
  // global -> LDS: a load unit is 16 rows x 64 B; lane l fetches row l/4 and the logical chunk
  // that belongs at physical chunk l%4: c = (l%4) ^ ((row >> 3) & 3)
  const uint32_t c_even = (lane & 3) ^ (lane >> 5);  // units 0,2 of a wave; units 1,3 flip bit 1
  const uint32_t v_even = (uint32_t)(lane >> 2) * K + c_even * 16;
  const uint32_t v_odd = (uint32_t)(lane >> 2) * K + (c_even ^ 2) * 16;
  // LDS -> VGPR: lane (li, lj) reads chunks lj and 2+lj of row li of each 32-row sub-tile
  const uint32_t sw = (li >> 3) & 3;
  const uint32_t fa0 = (wm * 128 + li) * kK32 + ((lj ^ sw) << 4);
  const uint32_t fa1 = (wm * 128 + li) * kK32 + (((2 + lj) ^ sw) << 4);
  const uint32_t fb0 = kT32 * kK32 + (wn * 128 + li) * kK32 + ((lj ^ sw) << 4);
  const uint32_t fb1 = kT32 * kK32 + (wn * 128 + li) * kK32 + (((2 + lj) ^ sw) << 4);
  const uint32_t fsa = kCodes32 + wm * 256 + lane * 4;
  const uint32_t fsb = kCodes32 + 512 + wn * 256 + lane * 4;

  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t*)smem;  // LDS byte address of the ring

  // ---- loader stream (runs NSTAGE steps ahead of the compute stream)
  uint32_t ld_tile = 0, ld_ks = 0;
  int ld_stage = 0;
  __amdgpu_buffer_rsrc_t ra, rb, rs;  // codes of A, codes of B, scales this wave copies
  auto loader_open_tile = [&]() {
    if (ld_tile < n_my) {
      uint32_t tm, tn;
      tile_coords(t_lo + ld_tile * wgs_per_xcd, tiles_m, tiles_n, tm, tn);
      const int64_t rows_a = p.M - (int64_t)tm * kT32, rows_b = p.N - (int64_t)tn * kT32;
      ra = make_rsrc(p.a_codes + (int64_t)tm * kT32 * K, rows_a * K);
      rb = make_rsrc(p.b_codes + (int64_t)tn * kT32 * K, rows_b * K);
      // wave 0,1 copy A's two 128-row scale groups, wave 2,3 copy B's
      const int64_t rows = wave < 2 ? rows_a : rows_b;
      const uint8_t* sbase = wave < 2 ? p.a_scales + (int64_t)(tm * 2 + wave) * ks_n * 256
                                      : p.b_scales + (int64_t)(tn * 2 + wave - 2) * ks_n * 256;
      const int64_t groups_left = ((rows + 127) >> 7) - (wave & 1);
      rs = make_rsrc(sbase, groups_left > 0 ? (int64_t)ks_n * 256 : 0);
    } else {  // past the last tile: every lane reads out of range (zeros, no traffic)
      ra = make_rsrc(p.a_codes, 0);
      rb = ra;
      rs = ra;
    }
  };
  auto issue_step = [&]() {
    const uint32_t k0 = ld_ks * kK32;
    const uint32_t sbase = lds_base + ld_stage * kStage32;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int unit = wave * 4 + q;
      const uint32_t v = (q & 1) ? v_odd : v_even;
      const uint32_t so = (uint32_t)(unit * 16) * K + k0;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void_t*)(uintptr_t)(sbase + unit * 1024), 16, v, so, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rb, (lds_void_t*)(uintptr_t)(sbase + kT32 * kK32 + unit * 1024), 16, v, so, 0, 0);
    }
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void_t*)(uintptr_t)(sbase + kCodes32 + wave * 256), 4,
                                             (uint32_t)lane * 4, ld_ks * 256, 0, 0);
    if (++ld_ks == nsteps) {
      ld_ks = 0;
      ++ld_tile;
      loader_open_tile();
    }
    if (++ld_stage == NSTAGE) ld_stage = 0;
  };

  // Fragment reads are issued as inline assembly: the compiler cannot tell which ring stage a
  // ds_read touches, so for reads it can see it waits until every global->LDS copy in flight
  // has landed (vmcnt(0)) and the prefetch distance collapses.  The reads are therefore
  // invisible to its wait-count tracking; `pin_frags` (after the explicit lgkmcnt(0) at the top
  // of the next step) is what the MFMAs depend on.
  auto lds_b128 = [&](uint32_t addr, auto off_) -> v4i {
    constexpr int off = decltype(off_)::value;
    v4i v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(off));
    return v;
  };
  auto read_frags = [&](Frags32& f, int stage) {
    const uint32_t sbase = lds_base + stage * kStage32;
    const uint32_t pa0 = sbase + fa0, pa1 = sbase + fa1, pb0 = sbase + fb0, pb1 = sbase + fb1;
    static_for<0, 4>([&](auto m_) {
      constexpr int m = decltype(m_)::value;
      const v4i lo = lds_b128(pa0, std::integral_constant<int, m * 2048>{});
      const v4i hi = lds_b128(pa1, std::integral_constant<int, m * 2048>{});
      f.a[m] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    });
    static_for<0, 4>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      const v4i lo = lds_b128(pb0, std::integral_constant<int, n * 2048>{});
      const v4i hi = lds_b128(pb1, std::integral_constant<int, n * 2048>{});
      f.b[n] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    });
    asm volatile("ds_read_b32 %0, %1" : "=v"(f.sa) : "v"(sbase + fsa));
    asm volatile("ds_read_b32 %0, %1" : "=v"(f.sb) : "v"(sbase + fsb));
  };
  auto pin_frags = [&](Frags32& f) {
#pragma unroll
    for (int m = 0; m < 4; ++m) asm volatile("" : "+v"(f.a[m]));
#pragma unroll
    for (int n = 0; n < 4; ++n) asm volatile("" : "+v"(f.b[n]));
    asm volatile("" : "+v"(f.sa), "+v"(f.sb));
  };

  // ---- compute stream
  v16f acc[4][4];
  int c_stage = 0;
  uint64_t prof_vm = 0, prof_bar = 0, prof_body = 0, prof_last = 0, prof_epi = 0, prof_issue = 0, prof_read = 0;

  auto mfma_step = [&](const Frags32& f, auto first_) {
    constexpr bool kFirst = decltype(first_)::value;  // first step of a tile starts from zero
    static_for<0, 4>([&](auto n_) {
      constexpr int n = decltype(n_)::value;
      static_for<0, 4>([&](auto m_) {
        constexpr int m = decltype(m_)::value;
        if constexpr (kFirst) {
          acc[m][n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              f.b[n], f.a[m], v16f{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, 0, 0, n,
              (int)f.sb, m, (int)f.sa);
        } else {
          acc[m][n] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              f.b[n], f.a[m], acc[m][n], 0, 0, n, (int)f.sb, m, (int)f.sa);
        }
      });
    });
  };

  // One step: `cur` holds the fragments of step g (read during step g-1), `nxt` receives g+1.
  // The first step of a tile follows the previous tile's output stores, which sit in the same
  // counter as the loads, so it waits for everything outstanding.
  auto step = [&](Frags32& cur, Frags32& nxt, auto first_) {
    constexpr bool kFirst = decltype(first_)::value;
    // stage c_stage is free once every wave holds its fragments of this step in registers;
    // stage c_stage+1 must have landed for everyone before it is read
    // (waits written as assembly: the compiler rewrites the immediates of s_waitcnt builtins
    // from its own, here too pessimistic, model of what is outstanding)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    pin_frags(cur);
    uint64_t t0 = 0, t1 = 0;
    if constexpr (PROF) {
      t0 = __builtin_readcyclecounter();
      prof_body += t0 - prof_last;
    }
    if constexpr (kFirst) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
      // groups in flight: g+1 .. g+NSTAGE-1; all but the first may stay outstanding
      static_assert(NSTAGE == 4 && kVmPerStep == 9, "update the immediate below");
      asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
    }
    if constexpr (PROF) {
      t1 = __builtin_readcyclecounter();
      prof_vm += t1 - t0;
    }
    __builtin_amdgcn_s_barrier();
    if constexpr (PROF) {
      prof_last = __builtin_readcyclecounter();
      prof_bar += prof_last - t1;
    }
    issue_step();  // step g+NSTAGE into the stage just freed
    const int next_stage = c_stage + 1 == NSTAGE ? 0 : c_stage + 1;
    if constexpr (PROF) {
      const uint64_t t3 = __builtin_readcyclecounter();
      prof_issue += t3 - prof_last;
      read_frags(nxt, next_stage);
      const uint64_t t4 = __builtin_readcyclecounter();
      prof_read += t4 - t3;
    } else {
      read_frags(nxt, next_stage);
    }
    mfma_step(cur, first_);
    c_stage = next_stage;
  };

  // Output: a lane holds, per 32x32 sub-tile, row li and columns 8q + 4lj + 0..3.  The two
  // lanes of a row (lj = 0, 1) trade halves with v_permlane32_swap so that each stores 8
  // consecutive bf16 (16 bytes); ordinary (cached) stores let L2 merge the pieces of a line.
  // Buffer stores: one descriptor per tile bounds the rows, one 32-bit offset per lane and
  // sub-tile row, immediates for the columns -- no 64-bit address arithmetic, no branches.
  // Requires N % 8 == 0 and ldd % 8 == 0 (checked on the host).
  auto epilogue = [&](uint32_t tile) {
    uint32_t tm, tn;
    tile_coords(t_lo + tile * wgs_per_xcd, tiles_m, tiles_n, tm, tn);
    const int64_t rows_valid = p.M - (int64_t)tm * kT32;
    const uint32_t cols_valid = (uint32_t)(p.N - (int64_t)tn * kT32);
    const uint32_t ldd_b = (uint32_t)p.ldd * 2;
    const __amdgpu_buffer_rsrc_t rd =
        make_rsrc(p.d + (int64_t)tm * kT32 * p.ldd + (int64_t)tn * kT32, rows_valid * ldd_b);
    // byte offset of (row wm*128 + li, column wn*128 + lj*8); out of range if the column is
    const uint32_t col0 = wn * 128 + lj * 8;
    const uint32_t v0 = (wm * 128 + li) * ldd_b + col0 * 2;
    static_for<0, 4>([&](auto m_) {
      constexpr int m = decltype(m_)::value;
      static_for<0, 4>([&](auto n_) {
        constexpr int n = decltype(n_)::value;
        const v16f a = acc[m][n];
        static_for<0, 2>([&](auto h_) {
          constexpr int h = decltype(h_)::value;
          const uint32_t x0 = pack_bf16(a[8 * h + 0], a[8 * h + 1]), y0 = pack_bf16(a[8 * h + 2], a[8 * h + 3]);
          const uint32_t x1 = pack_bf16(a[8 * h + 4], a[8 * h + 5]), y1 = pack_bf16(a[8 * h + 6], a[8 * h + 7]);
          const u32x2 sx = __builtin_amdgcn_permlane32_swap(x0, x1, false, false);
          const u32x2 sy = __builtin_amdgcn_permlane32_swap(y0, y1, false, false);
          const u32x4 w = {sx.x, sy.x, sx.y, sy.y};
          const uint32_t v = (col0 + n * 32 + h * 16 < cols_valid) ? v0 : 0x80000000u;
          __builtin_amdgcn_raw_buffer_store_b128(w, rd, v + (n * 32 + h * 16) * 2, m * 32 * ldd_b, 0);
        });
      });
    });
  };

  // ---- prologue: fill the ring, fetch the first fragments
  loader_open_tile();
#pragma unroll
  for (int s = 0; s < NSTAGE; ++s) issue_step();
  asm volatile("s_waitcnt vmcnt(27)" ::: "memory");  // (NSTAGE - 1) groups may stay in flight
  __builtin_amdgcn_s_barrier();
  Frags32 f0, f1;
  read_frags(f0, 0);
  if constexpr (PROF) prof_last = __builtin_readcyclecounter();

  // ---- tiles; at the top of every tile f0 holds the fragments of its step 0 (nsteps is even)
  const uint32_t pairs = nsteps / 2 - 1;
  for (uint32_t tile = 0; tile < n_my; ++tile) {
    step(f0, f1, std::true_type{});
    step(f1, f0, std::false_type{});
    for (uint32_t i = 0; i < pairs; ++i) {
      step(f0, f1, std::false_type{});
      step(f1, f0, std::false_type{});
    }
    if constexpr (PROF) {
      const uint64_t e0 = __builtin_readcyclecounter();
      prof_body += e0 - prof_last;
      epilogue(tile);
      prof_last = __builtin_readcyclecounter();
      prof_epi += prof_last - e0;
    } else {
      epilogue(tile);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the over-issued prefetches before retiring
  if constexpr (PROF) {
    if (lane == 0) {
      uint64_t* o = p.prof + (blockIdx.x * 4 + wave) * 8;
      o[0] = prof_vm;
      o[1] = prof_bar;
      o[2] = prof_body;
      o[3] = prof_epi;
      o[4] = prof_issue;
      o[5] = prof_read;
    }
  }
}

static int debug_grid = 0;
static uint64_t* debug_prof = nullptr;  // > 0: number of persistent workgroups (experiments only)

template <int NSTAGE, bool PROF>
static int launch_dense32(const Dense32Args& p, hipStream_t st) {
  auto kern = gemm_nt32_kernel<NSTAGE, PROF>;
  constexpr int lds = NSTAGE * kStage32;
  static int num_cus = 0;
  if (num_cus == 0) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return MX_ERR_LAUNCH;
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return MX_ERR_LAUNCH;
    num_cus = n;
  }
  const int64_t nb = ((p.M + kT32 - 1) / kT32) * ((p.N + kT32 - 1) / kT32);
  int64_t grid = (num_cus / 8) * 8;  // one persistent workgroup per CU, a multiple of the 8 XCDs
  if (grid < 8) grid = 8;
  const int64_t need = (nb + 7) / 8 * 8;
  if (need < grid) grid = need;
  if (debug_grid > 0) grid = (debug_grid + 7) / 8 * 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, p);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

void set_debug_grid(int g) { debug_grid = g; }
void set_debug_prof(uint64_t* buf) { debug_prof = buf; }

int launch_gemm_nt32(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                     const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                     int64_t ldd, hipStream_t st) {
  Dense32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, debug_prof};
  if (debug_prof) return launch_dense32<4, true>(p, st);
  return launch_dense32<4, false>(p, st);
}

}  // namespace mx
