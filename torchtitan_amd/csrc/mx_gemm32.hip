// MXFP8 GEMM for large shapes, dense and grouped: persistent 256x256 tiles on the scaled fp8
// MFMA v_mfma_scale_f32_16x16x128_f8f6f4.
//
//   D[M,N] (bf16) = deq(A)[M,K] * deq(B)[N,K]^T, fp32 accumulate.
//
// One workgroup (4 waves, 2x2, 128x128 each = 256 accumulator registers per lane) per CU walks
// a list of output tiles; the K loops of all its tiles form one flat stream of 128-deep
// blocks, so the loads of the next tile's first blocks are already in flight while a tile is
// written out.
//
// Global -> LDS moves whole 128-byte rows (buffer_load_dwordx4 ... lds, 8 rows per instruction:
// full cache lines, which the texture path delivers about twice as fast as 64-byte pieces), so
// the ring holds two 128-deep blocks of 64 KB codes + 2 KB scales.  Two barriers per block: one
// releases the ring block whose last fragments have just been read (its refill starts there,
// spread thinly because the copy path is the scarce resource), one makes sure the next block
// has landed.
//
// Which MFMA.  The 16x16x128 and the 32x32x64 form both do 2048 flop per cycle and SIMD and read
// the same operand bytes per flop; the 16x16x128 one reads and writes a quarter of the
// accumulator registers per instruction.  Under the chip's power limit that is worth 9 % of
// sustained rate on the same operand bits with nothing else running, and was worth 6-10 % of
// shader clock inside this kernel against 2-3 % more cycles when the K loop moved to it (64 MFMA
// slots of 32 cycles per block leave less room behind each MFMA for the block's LDS reads and
// copies than 32 slots of 64 cycles).
//   A block is 64 MFMAs, one per 16x16 sub-tile, in four quarters over four fragment sets (two
//   64-row halves of A, two of B) that are refilled in place as soon as their last MFMA has been
//   issued; see block_steps for the slot plan.  Operand layout (measured): lane (i = l & 15,
//   j = l >> 4) holds row i, K bytes [16j, 16j+16) in registers 0-3 and [64+16j, 64+16j+16) in
//   registers 4-7; the scale of 32-element block b is taken from lane group b.  With the first
//   operand = B rows and the second = A rows, a lane ends up with D[row = l & 15][col = 4j + 0..3].
// Fragment reads are conflict-free under the b128 pass grouping.
//
// MX_ABL_NO_DMA / MX_ABL_NO_READ / MX_ABL_STORE_ROWS / MX_ABL_NO_EPILOGUE (never defined in the
// product build) drop the copies, the fragment reads, part of the output stores or the whole
// epilogue from the steady state, to time what is left; MX_ABL_SAME_PANEL makes all dense tiles
// read the same twelve operand panels (MX_ABL_SAME_A / MX_ABL_SAME_B: the same A / B panels only), so
// that every read beyond the L2 finds its line in the memory-side cache; MX_ABL_ROW_PAD=n reads the
// rows of a tile n bytes further apart than they lie (what a padded row pitch would do to the
// spread of a block's lines over the cache channels); MX_ABL_TR_READ issues every fragment read as
// two ds_read_b64_tr_b8 (what a K loop over operands stored K-strided would issue); MX_ABL_DMA_OOB
// issues every copy with all lanes out of range (the instructions and their LDS writes stay, the
// fetches go).  Results are then meaningless.
#include "mx_gemm_tile.h"

namespace mx {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kT32 = 256;                        // tile edge (M and N)
constexpr int kK32 = 64;                         // K per compute step
constexpr int kKB = 128;                         // K per ring block (= one cache line per row)
constexpr int kOperand32 = kT32 * kKB;           // 32 KB: 256 rows x 128 B
constexpr int kCodes32 = 2 * kOperand32;         // A rows then B rows
constexpr int kBlock32 = kCodes32 + 3072;        // + scales: groups A0, A1, B0, B1, A2 (+ 512 unused) x 2 steps x 256 B
constexpr int kRing32 = 2 * kBlock32;            // 134 KB
constexpr int kPatch32 = 6656;                   // per wave: 4608 B output patch + 2 KB of records / tables
constexpr int kPatchUsed = 4608;
constexpr uint32_t kRecordsPerPatch = (kPatch32 - kPatchUsed) / 64;
constexpr uint32_t kMaxTileRecords = 3 * kRecordsPerPatch;  // grouped modes: tile records a workgroup keeps in LDS
static_assert(kRing32 + 4 * kPatch32 == 160 * 1024, "the kernel's LDS map fills the CU's 160 KB");

// What a launch works on.  One kernel serves three problems that differ only in how a linear
// tile number maps to operand rows, K range and output address:
//   kDense        D[M,N] = A[M,K] B[N,K]^T
//   kGrouped2d3d  rows of A in groups (inclusive ends offs[g], all multiples of 32), group g
//                 against B[g][N,K]; rows from offs[G-1] to M are written as zeros
//   kGrouped2d2d  D[g][M,N] = A[M, lo_g:hi_g] B[N, lo_g:hi_g]^T, K = row length of A and B
//   kSplitK       as kGrouped2d2d with G equal slices of the K blocks worked out in the kernel
//                 and float32 output: D[g][M,N] are partial sums for a reduction pass
enum Gemm32Mode { kDense = 0, kGrouped2d3d = 1, kGrouped2d2d = 2, kSplitK = 3 };
struct Gemm32Args {
  const uint8_t* a_codes;
  const uint8_t* a_scales;
  const uint8_t* b_codes;
  const uint8_t* b_scales;
  uint16_t* d;
  int64_t M, N, K, ldd;
  const int32_t* offs;  // grouped modes: inclusive cumulative group sizes, on the device
  int64_t G;
  int32_t tn0, tn_cnt;  // grouped modes: this launch covers tile columns [tn0, tn0 + tn_cnt)
  uint64_t* prof;  // timing build only: per wave {vmcnt wait, barrier wait, step body} cycles
  // PAIR kernels: a second operand set of the same shapes; D = A B^T + A2 B2^T in one pass, every
  // output tile running the K blocks of the first set and then those of the second before it is
  // written out (dx = da W1 + db W3 of a SwiGLU block's backward)
  const uint8_t* a2_codes = nullptr;
  const uint8_t* a2_scales = nullptr;
  const uint8_t* b2_codes = nullptr;
  const uint8_t* b2_scales = nullptr;
  // Two products that share one operand in one launch (not with PAIR).  kTwoB: D = A B^T and
  // D2 = A B2^T, the tile columns of the second product numbered behind those of the first
  // (h1 = x W1^T and h3 = x W3^T of a SwiGLU block: every A panel is fetched for both).  kTwoA:
  // D = A B^T and D2 = A2 B^T, the tile rows of the second behind those of the first (the weight
  // gradients dW1 = d(h1)^T x and dW3 = d(h3)^T x).
  int32_t two = 0;
  uint16_t* d2 = nullptr;
  // kDense, kSplitK: bytes between the rows of A and of B (both operands' rows are K bytes long
  // and may lie further apart, by a multiple of 128); 0 = K
  int64_t ldk = 0;
  // kGrouped2d3d: output rows without the groups' padding.  Group g's first d_offs[g] -
  // d_offs[g-1] rows are written to rows [d_offs[g-1], d_offs[g]) of D (inclusive ends, on the
  // device), the rest of its rows nowhere; rows [d_offs[G-1], d_rows) of D are written as zeros
  // as far as A has rows behind its last group.  nullptr: D has A's rows.
  const int32_t* d_offs = nullptr;
  int64_t d_rows = 0;
};
enum Gemm32Two { kTwoNone = 0, kTwoB = 1, kTwoA = 2 };

// Where one 256x256 tile lives.
struct Tile32 {
  const uint8_t *a, *b;    // first operand row of the tile, at the first K byte of its range
  const uint8_t *sa, *sb;  // scales of the tile's first 128-row group at its first 64-deep step
  uint16_t* d;
  int64_t rows_a, rows_b;  // valid rows from the tile's origin (may exceed 256; <= 0: none)
  int32_t rows_d;          // Gemm32Args::d_offs given: rows of the tile that D has (0..256)
  uint32_t koff;           // first K byte of the range inside an operand row (kGrouped2d2d)
  uint32_t nblocks;        // 128-deep K blocks, at least 1
  bool empty;              // no K range (an empty group, rows behind the last group, or poison):
                           // one block of out-of-range reads, i.e. zeros, stands in for it
  bool poison;             // grouped modes: the group ends break the alignment contract
  uint32_t rot;            // kGrouped2d3d: 32-row blocks between the tile's first row and the start of
                           // its 128-row scale group (0..3): the A scale bytes are turned by as much
  uint32_t head, tail;     // kGrouped2d2d: the K range starts `head` 32-deep blocks into its first
                           // 128-deep block and ends `tail` of them into its last (0: at its end)
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

// LDS accesses the compiler must not see (see the fragment reads in the kernel)
template <int OFF>
__device__ __forceinline__ void lds_write_b128_hidden(uint32_t addr, v4i v) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ v4i lds_read_b128_hidden(uint32_t addr) {
  v4i v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
__device__ __forceinline__ v4i pin(v4i v) {
  asm volatile("" : "+v"(v));
  return v;
}

// One scaled MFMA, C = 0 (FIRST) or accumulate.  Written as assembly: left as builtins, the
// compiler gathers all MFMAs of a tile's first block behind the block's copies, reads and
// barriers instead of leaving them interleaved.  op_sel / op_sel_hi pick the scale byte of the
// lane's scale dword: NB for the first operand, MB for the second.
template <int NB, int MB, bool FIRST>
__device__ __forceinline__ void mfma16_asm(v4f& c, const v8i& b, const v8i& a, uint32_t sb,
                                           uint32_t sa) {
  if constexpr (FIRST)
    asm volatile(
        "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0]"
        : "=a"(c)
        : "v"(b), "v"(a), "v"(sb), "v"(sa), "n"(NB & 1), "n"(MB & 1), "n"(NB >> 1), "n"(MB >> 1));
  else
    asm volatile(
        "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%6,0] op_sel_hi:[%7,%8,0]"
        : "+a"(c)
        : "v"(b), "v"(a), "v"(sb), "v"(sa), "n"(NB & 1), "n"(MB & 1), "n"(NB >> 1), "n"(MB >> 1));
}

// One accumulator register into a VGPR, where the caller says (as assembly: the compiler's own
// copies out of the accumulator file are all placed at the top of the epilogue).
template <int E, class V>
__device__ __forceinline__ float acc_read(const V& c) {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(c[E]));
  return x;
}

// Fragment sets of four 16-row sub-tiles each, whole 128-deep blocks (a[h][t] =
// sub-tile 4h + t of the wave's 128 rows of A, b[h][t] likewise for B), the scale dwords of the
// block being computed (one for the even and one for the odd sub-tiles) and those of the next.
struct Frags16 {
  v8i a[2][4];
  v8i b[2][4];
  uint32_t sa[2], sb[2];
  uint32_t san[2], sbn[2];
  uint32_t sa_hi[2];  // kGrouped2d3d: as san, of the next 128-row group (see next_scales)
};

template <int MODE, bool PROF, bool PAIR = false>
__global__ __launch_bounds__(256, 1) void gemm_nt32_kernel(Gemm32Args p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 15, lj = lane >> 4;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t*)smem;  // LDS byte address of the ring
  const uint32_t K = (uint32_t)p.K;  // bytes per operand row; a multiple of 128 for this kernel
#ifndef MX_ABL_ROW_PAD  // timing ablation: the rows of a tile are read this many bytes further apart than they lie
#define MX_ABL_ROW_PAD 0
#endif
  // Kp: bytes from one operand row to the next.  A pitch that is not a multiple of 4 KB spreads the
  // lines a block's copies fetch together (one K block of 512 rows) over the channels of the L2.
  const uint32_t Kp = ((MODE == kDense || MODE == kSplitK) && p.ldk ? (uint32_t)p.ldk : K) + MX_ABL_ROW_PAD;
  const int64_t Kt = (MODE == kDense || MODE == kSplitK) && p.ldk ? p.ldk : p.K;  // ... as the tile origins use it
  const uint32_t ks_n = K / kK32;    // 64-deep steps per 128-row scale group
  // tile rows / columns of one product, and of the launch (p.two: the second product's tile
  // columns or rows come behind the first's; grouped launches cover columns [tn0, tn0 + tn_cnt))
  const uint32_t tiles_n1 = (uint32_t)((p.N + kT32 - 1) / kT32), tiles_m1 = (uint32_t)((p.M + kT32 - 1) / kT32);
  const uint32_t tiles_n = MODE == kDense ? (p.two == kTwoB ? 2 * tiles_n1 : tiles_n1) : (uint32_t)p.tn_cnt;
  const uint32_t tiles_m = p.two == kTwoA ? 2 * tiles_m1 : tiles_m1;
  const uint32_t tn0 = MODE == kDense ? 0u : (uint32_t)p.tn0;
  const uint32_t G = (uint32_t)p.G;

  // ---- tile count.  kGrouped2d3d: group g has ceil(rows_g / 256) x tiles_n tiles; the first
  //      tile number of every group (G + 2 entries, the last group being the zero rows behind
  //      offs[G-1]) is kept in the 2 KB that wave 0's output patch leaves unused.
  bool poison = false;
  bool dealt = false;  // kGrouped2d2d: tiles dealt by length (below) instead of in tile order
  constexpr uint32_t kMaxDealt = (kPatch32 - kPatchUsed) / 4;  // two uint16 per group in wave 0's spare patch LDS
  constexpr uint32_t kMinDealt = 32;   // fewer groups than that cannot be spread evenly over 8 XCDs
  uint32_t nb;
  // "any thread saw a bad group end", through a word of wave 1's spare patch bytes (the
  // kernel's whole 160 KB are dynamic LDS: a library reduction would ask for more)
  auto any_bad = [&](int bad) -> bool {
    uint32_t* flag = reinterpret_cast<uint32_t*>(smem + kRing32 + kPatch32 + kPatchUsed);
    if (tid == 0) *flag = 0;
    __syncthreads();
    if (bad) atomicOr(flag, 1u);
    __syncthreads();
    return *flag != 0;
  };
  if constexpr (MODE == kDense) {
    nb = tiles_m * tiles_n;
  } else if constexpr (MODE == kSplitK) {
    nb = G * tiles_m * tiles_n;
  } else if constexpr (MODE == kGrouped2d2d) {
    nb = G * tiles_m * tiles_n;
    // group lengths in K blocks, kept for the dealing below (up to kMaxDealt groups)
    uint16_t* g_blocks = reinterpret_cast<uint16_t*>(smem + kRing32 + kPatchUsed);
    int bad = 0;
    for (uint32_t g = tid; g < G; g += 256) {
      const int32_t hi = p.offs[g], lo = g ? p.offs[g - 1] : 0;
      bad |= (hi & 31) | (hi < lo) | (hi > (int64_t)K) | (lo < 0);
      if (G <= kMaxDealt && G >= kMinDealt) {
        const int64_t len = hi > lo ? (((int64_t)hi + 127) >> 7) - (lo >> 7) : 0;
        g_blocks[g] = (uint16_t)(len > 0xFFFF ? 0xFFFF : len);
      }
    }
    poison = any_bad(bad);
    dealt = !poison && G <= kMaxDealt && G >= kMinDealt;
    if (dealt) {
      // position of every group in the order of falling length (ties by index): G^2 / 256
      // comparisons per thread, far below one tile's worth of time
      uint16_t* g_sorted = g_blocks + kMaxDealt;
      for (uint32_t g = tid; g < G; g += 256) {
        const uint32_t mine = g_blocks[g];
        uint32_t rank = 0;
        for (uint32_t h = 0; h < G; ++h) {
          const uint32_t o = g_blocks[h];
          rank += (o > mine) | ((o == mine) & (h < g));
        }
        g_sorted[rank] = (uint16_t)g;
      }
      __syncthreads();
    }
  } else {
    uint32_t* first = reinterpret_cast<uint32_t*>(smem + kRing32 + kPatchUsed);
    int bad = 0;
    for (uint32_t g = tid; g <= G; g += 256) {
      const int64_t lo = g ? p.offs[g - 1] : 0, hi = g < G ? (int64_t)p.offs[g] : p.M;
      bad |= (g < G && (hi & 31)) | (hi < lo) | (hi > p.M) | (lo < 0);
      const int64_t rows = hi > lo ? hi - lo : 0;
      first[g + 1] = (uint32_t)((rows + kT32 - 1) / kT32) * tiles_n;
    }
    poison = any_bad(bad);
    if (tid < 64) {  // inclusive prefix sum of first[1 .. G+1] by wave 0, 10 entries per lane
      uint32_t sum = 0;
      for (uint32_t g = 1 + (uint32_t)tid * 10; g < 11 + (uint32_t)tid * 10 && g <= G + 1; ++g) sum += first[g];
      uint32_t incl = sum;
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(incl, d);
        if (tid >= d) incl += o;
      }
      uint32_t run = incl - sum;
      for (uint32_t g = 1 + (uint32_t)tid * 10; g < 11 + (uint32_t)tid * 10 && g <= G + 1; ++g) {
        run += first[g];
        first[g] = run;
      }
      if (tid == 0) first[0] = 0;
    }
    __syncthreads();
    nb = first[G + 1];
    if (poison) nb = tiles_m * tiles_n;  // then: NaN over all of D
  }

  // ---- this workgroup's tile list: XCD x (= blockIdx % 8) owns one contiguous run of tiles,
  //      its workgroups take them round-robin, so the XCD's CUs work on neighbouring tiles
  const uint32_t wgs_per_xcd = gridDim.x / 8;
  const uint32_t xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
  const uint32_t per_xcd = (nb + 7) / 8;
  const uint32_t t_lo = xcd * per_xcd + idx;
  const uint32_t t_hi = (xcd + 1) * per_xcd < nb ? (xcd + 1) * per_xcd : nb;
  uint32_t n_my = t_lo < t_hi ? (t_hi - t_lo + wgs_per_xcd - 1) / wgs_per_xcd : 0;
  // kGrouped2d2d with uneven groups: a tile's time goes with its group's length, so tiles taken
  // in tile order leave the workgroups with sums that differ by a fifth and more.  Instead the
  // groups, in order of falling length, are dealt to the XCDs back and forth (j-th group of XCD
  // x = position 8j + x or 8j + 7 - x), which keeps the tiles of a group, and their operand
  // panels, inside one L2; and the tiles of an XCD's groups, still in that order, are dealt to
  // its workgroups back and forth in the same way: every workgroup gets one tile from each band
  // of neighbouring lengths.
  auto snake = [](uint32_t band, uint32_t k, uint32_t width) -> uint32_t {
    return (band & 1) ? width - 1 - k : k;
  };
  const uint32_t per_g2 = tiles_m * tiles_n;  // tiles of one group
  if (MODE == kGrouped2d2d && dealt) {
    const uint32_t full = G / 8, rest = G % 8;
    const uint32_t groups_x = full + (snake(full, xcd, 8) < rest ? 1 : 0);
    const uint32_t tiles_x = groups_x * per_g2;
    const uint32_t bands = tiles_x / wgs_per_xcd, tail = tiles_x % wgs_per_xcd;
    n_my = bands + (snake(bands, idx, wgs_per_xcd) < tail ? 1 : 0);
  }
  if (n_my == 0) return;
  if (PAIR) n_my *= 2;  // from here on n_my counts segments: two per output tile
  if (MODE != kDense && n_my > kMaxTileRecords) {
    // More tiles than records: the host splits launches so that this cannot happen.  Should it
    // ever, the tiles that have a record are written as NaN rather than left as they were.
    n_my = kMaxTileRecords;
    poison = true;
  }

  // Tile number -> operands.
  auto describe = [&](uint32_t t, uint32_t seg) -> Tile32 {
    Tile32 r;
    r.poison = poison;
    r.koff = 0;
    r.empty = false;
    r.rows_d = 0;
    r.rot = 0;
    r.head = 0;
    r.tail = 0;
    const uint8_t* a_codes = (PAIR && seg) ? p.a2_codes : p.a_codes;
    const uint8_t* a_scales = (PAIR && seg) ? p.a2_scales : p.a_scales;
    const uint8_t* b_codes = (PAIR && seg) ? p.b2_codes : p.b_codes;
    const uint8_t* b_scales = (PAIR && seg) ? p.b2_scales : p.b_scales;
    uint16_t* d_base = p.d;
    // p.two: a tile column / row of the second product becomes that product's own, with its
    // operand and output in place of the first's
    auto second_product = [&](uint32_t& tm, uint32_t& tn) {
      if constexpr (!PAIR && (MODE == kDense || MODE == kGrouped2d3d || MODE == kGrouped2d2d)) {
        if (p.two == kTwoB && tn >= tiles_n1) {
          tn -= tiles_n1;
          b_codes = p.b2_codes;
          b_scales = p.b2_scales;
          d_base = p.d2;
        }
        if (p.two == kTwoA && tm >= tiles_m1) {
          tm -= tiles_m1;
          a_codes = p.a2_codes;
          a_scales = p.a2_scales;
          d_base = p.d2;
        }
      }
    };
    uint32_t tm, tn;
    if (MODE == kDense || (MODE == kGrouped2d3d && poison)) {
      tile_coords(t, tiles_m, tiles_n, tm, tn);
      tn += tn0;
      second_product(tm, tn);
#if defined(MX_ABL_SAME_PANEL)  // timing ablation: every 8 x 4 round reads the same twelve operand panels
      r.a = a_codes + (int64_t)(tm & 7) * kT32 * K;
      r.b = b_codes + (int64_t)(tn & 3) * kT32 * K;
#elif defined(MX_ABL_SAME_A)  // ... the same eight A panels only
      r.a = a_codes + (int64_t)(tm & 7) * kT32 * K;
      r.b = b_codes + (int64_t)tn * kT32 * K;
#elif defined(MX_ABL_SAME_B)  // ... the same four B panels only
      r.a = a_codes + (int64_t)tm * kT32 * K;
      r.b = b_codes + (int64_t)(tn & 3) * kT32 * K;
#else
      r.a = a_codes + (int64_t)tm * kT32 * Kt;
      r.b = b_codes + (int64_t)tn * kT32 * Kt;
#endif
      r.sa = a_scales + (int64_t)(tm * 2) * ks_n * 256;
      r.sb = b_scales + (int64_t)(tn * 2) * ks_n * 256;
      r.d = d_base + (int64_t)tm * kT32 * p.ldd + (int64_t)tn * kT32;
      r.rows_a = p.M - (int64_t)tm * kT32;
      r.rows_b = p.N - (int64_t)tn * kT32;
      if (MODE == kGrouped2d3d && p.d_offs) {
        const int64_t left = p.d_rows - (int64_t)tm * kT32;
        r.rows_d = (int32_t)(left < 0 ? 0 : (left > kT32 ? kT32 : left));
      }
      r.nblocks = poison ? 1 : K / kKB;
      r.empty = poison;
    } else if (MODE == kGrouped2d3d) {
      const uint32_t* first = reinterpret_cast<const uint32_t*>(smem + kRing32 + kPatchUsed);
      uint32_t g = 0, hi_g = G + 1;  // first[g] <= t < first[g + 1]
      while (hi_g - g > 1) {
        const uint32_t mid = (g + hi_g) >> 1;
        if (first[mid] <= t) g = mid; else hi_g = mid;
      }
      const int64_t lo = g ? p.offs[g - 1] : 0, hi = g < G ? (int64_t)p.offs[g] : p.M;
      const uint32_t tiles_mg = (uint32_t)((hi - lo + kT32 - 1) / kT32);
      tile_coords(t - first[g], tiles_mg, tiles_n, tm, tn);
      tn += tn0;
      second_product(tm, tn);
      const int64_t row0 = lo + (int64_t)tm * kT32;
      const uint32_t gb = g < G ? g : 0;  // the zero rows have no expert: any valid address
      r.a = a_codes + row0 * K;
      r.b = b_codes + ((int64_t)gb * p.N + (int64_t)tn * kT32) * K;
      r.sa = a_scales + (row0 >> 7) * ks_n * 256;
      r.rot = (uint32_t)(row0 >> 5) & 3;
      r.sb = b_scales + ((int64_t)gb * ((p.N + 127) >> 7) + tn * 2) * ks_n * 256;
      r.d = d_base + row0 * p.ldd + (int64_t)tn * kT32;
      r.rows_a = hi - row0;
      r.rows_b = p.N - (int64_t)tn * kT32;
      if (p.d_offs) {  // the group's rows in D, both ends kept inside D whatever the array holds
        int64_t lo_d = g ? p.d_offs[g - 1] : 0, hi_d = g < G ? (int64_t)p.d_offs[g] : p.d_rows;
        lo_d = lo_d < 0 ? 0 : (lo_d > p.d_rows ? p.d_rows : lo_d);
        hi_d = hi_d < lo_d ? lo_d : (hi_d > p.d_rows ? p.d_rows : hi_d);
        const int64_t left = hi_d - lo_d - (int64_t)tm * kT32;
        r.rows_d = (int32_t)(left < 0 ? 0 : (left > kT32 ? kT32 : left));
        r.d = d_base + (lo_d + (int64_t)tm * kT32) * p.ldd + (int64_t)tn * kT32;
      }
      r.nblocks = g < G ? K / kKB : 1;
      r.empty = g >= G;
    } else if (MODE == kSplitK) {
      // slice g of the K blocks: ceil(blocks / G) each, the host picks G so that none is empty
      const uint32_t per_g = tiles_m * tiles_n;
      const uint32_t g = t / per_g;
      tile_coords(t - g * per_g, tiles_m, tiles_n, tm, tn);
      const uint32_t blocks = K / kKB, per = (blocks + G - 1) / G;
      const uint32_t b_lo = g * per, b_hi = b_lo + per < blocks ? b_lo + per : blocks;
      const uint32_t lo = b_lo * kKB;
      r.a = a_codes + (int64_t)tm * kT32 * Kt + lo;
      r.b = b_codes + (int64_t)tn * kT32 * Kt + lo;
      r.sa = a_scales + ((int64_t)(tm * 2) * ks_n + (lo >> 6)) * 256;
      r.sb = b_scales + ((int64_t)(tn * 2) * ks_n + (lo >> 6)) * 256;
      float* part = reinterpret_cast<float*>(p.d) +
                    ((int64_t)g * p.M + (int64_t)tm * kT32) * p.ldd + (int64_t)tn * kT32;
      r.d = reinterpret_cast<uint16_t*>(part);
      r.rows_a = p.M - (int64_t)tm * kT32;
      r.rows_b = p.N - (int64_t)tn * kT32;
      r.koff = lo;
      r.nblocks = b_hi - b_lo;
    } else {
      const uint32_t per_g = tiles_m * tiles_n;
      uint32_t g = t / per_g, in_g = t - g * per_g;
      if (dealt) {  // t counts this workgroup's tiles: the i-th tile it was dealt
        const uint16_t* g_sorted = reinterpret_cast<const uint16_t*>(smem + kRing32 + kPatchUsed) + kMaxDealt;
        const uint32_t q = wgs_per_xcd * t + snake(t, idx, wgs_per_xcd);  // place in the XCD's tile list
        const uint32_t j = q / per_g;
        in_g = q - j * per_g;
        g = g_sorted[8 * j + snake(j, xcd, 8)];
      }
      tile_coords(in_g, tiles_m, tiles_n, tm, tn);
      tn += tn0;
      second_product(tm, tn);
      const int64_t lo = poison ? 0 : (g ? p.offs[g - 1] : 0), hi = poison ? 0 : p.offs[g];
      // the K blocks keep to multiples of 128 (whole cache lines per operand row: a copy that
      // straddles two lines costs the texture path twice); a range that starts or ends inside
      // a block has the 32-deep blocks outside it masked (head, tail)
      const int64_t lo128 = lo & ~(int64_t)127;
      r.a = a_codes + (int64_t)tm * kT32 * K + lo128;
      r.b = b_codes + (int64_t)tn * kT32 * K + lo128;
      r.sa = a_scales + ((int64_t)(tm * 2) * ks_n + (lo128 >> 6)) * 256;
      r.sb = b_scales + ((int64_t)(tn * 2) * ks_n + (lo128 >> 6)) * 256;
      r.d = d_base + ((int64_t)g * p.M + (int64_t)tm * kT32) * p.ldd + (int64_t)tn * kT32;
      r.rows_a = p.M - (int64_t)tm * kT32;
      r.rows_b = p.N - (int64_t)tn * kT32;
      r.koff = (uint32_t)lo128;
      r.nblocks = hi > lo ? (uint32_t)(((hi + 127) >> 7) - (lo >> 7)) : 0;
      r.head = (uint32_t)(lo >> 5) & 3;
      r.tail = (uint32_t)(hi >> 5) & 3;
      if (r.nblocks == 0) {
        r.nblocks = 1;
        r.empty = true;
      }
    }
    return r;
  };

  // Grouped modes: the map needs loads of the group ends and a search, far too slow for the
  // in-order instruction stream of the MFMA waves.  Every thread works out one of this
  // workgroup's tiles up front and leaves a 64-byte record in the spare 2 KB behind the
  // output patches of waves 1-3 (32 records each; the host splits launches so that a
  // workgroup never has more than kMaxRecords tiles).
  auto record_offset = [&](uint32_t i) -> uint32_t {
    return kRing32 + (1 + i / kRecordsPerPatch) * kPatch32 + kPatchUsed + (i % kRecordsPerPatch) * 64;
  };
  if constexpr (MODE != kDense) {
    for (uint32_t i = tid; i < n_my; i += 256) {
      const uint32_t ti = PAIR ? i >> 1 : i;  // PAIR: records 2t and 2t+1 are the two segments of tile t
      const Tile32 t = describe((MODE == kGrouped2d2d && dealt) ? ti : t_lo + ti * wgs_per_xcd, PAIR ? i & 1 : 0);
      uint64_t* q = reinterpret_cast<uint64_t*>(smem + record_offset(i));
      q[0] = (uint64_t)(uintptr_t)t.a;
      q[1] = (uint64_t)(uintptr_t)t.b;
      q[2] = (uint64_t)(uintptr_t)t.sa;
      q[3] = (uint64_t)(uintptr_t)t.sb;
      q[4] = (uint64_t)(uintptr_t)t.d;
      int32_t* w = reinterpret_cast<int32_t*>(q + 5);
      w[0] = (int32_t)(t.rows_a > 0x7FFFFFFF ? 0x7FFFFFFF : t.rows_a);
      w[1] = (int32_t)(t.rows_b > 0x7FFFFFFF ? 0x7FFFFFFF : t.rows_b);
      w[2] = (int32_t)t.nblocks;
      w[3] = (int32_t)t.koff;
      w[4] = t.empty ? 1 : 0;
      w[5] = (int32_t)(t.rot | (t.tail << 8) | (t.head << 16) | ((uint32_t)t.rows_d << 20));
    }
    __syncthreads();
  }
  // this workgroup's i-th tile (records are read so that the compiler's wait-count model
  // does not see an LDS read, see the fragment reads; every lane reads the same 64 bytes)
  auto get_tile = [&](uint32_t i) -> Tile32 {
    if constexpr (MODE == kDense) {
      return describe(t_lo + (PAIR ? i >> 1 : i) * wgs_per_xcd, PAIR ? i & 1 : 0);
    } else {
      const uint32_t addr = lds_base + record_offset(i);
      v4i r0, r1, r2, r3;
      asm volatile(
          "ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:16\n\tds_read_b128 %2, %4 offset:32\n\t"
          "ds_read_b128 %3, %4 offset:48\n\ts_waitcnt lgkmcnt(0)"
          : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
          : "v"(addr)
          : "memory");
      auto u64 = [](int lo, int hi) -> uint64_t {
        return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(lo) |
               ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(hi) << 32);
      };
      Tile32 t;
      t.a = (const uint8_t*)(uintptr_t)u64(r0.x, r0.y);
      t.b = (const uint8_t*)(uintptr_t)u64(r0.z, r0.w);
      t.sa = (const uint8_t*)(uintptr_t)u64(r1.x, r1.y);
      t.sb = (const uint8_t*)(uintptr_t)u64(r1.z, r1.w);
      t.d = (uint16_t*)(uintptr_t)u64(r2.x, r2.y);
      t.rows_a = __builtin_amdgcn_readfirstlane(r2.z);
      t.rows_b = __builtin_amdgcn_readfirstlane(r2.w);
      t.nblocks = (uint32_t)__builtin_amdgcn_readfirstlane(r3.x);
      t.koff = (uint32_t)__builtin_amdgcn_readfirstlane(r3.y);
      t.empty = __builtin_amdgcn_readfirstlane(r3.z) != 0;
      const uint32_t rt = (uint32_t)__builtin_amdgcn_readfirstlane(r3.w);
      t.rot = rt & 3;
      t.tail = (rt >> 8) & 3;
      t.head = (rt >> 16) & 3;
      t.rows_d = (int32_t)(rt >> 20);
      t.poison = poison;
      return t;
    }
  };

  // ---- per-lane constants
  // global -> LDS: a load unit is 8 rows x 128 B; lane l fetches row l/8 and the logical 16-byte
  // chunk that belongs at physical chunk l%8 of that row:
  // c = (l%8) ^ ((row & 2) | ((row & 8) >> 1)), see the fragment reads
  const uint32_t c_even = (lane & 7) ^ ((lane >> 3) & 2);
  const uint32_t v_even = (uint32_t)(lane >> 3) * Kp + c_even * 16;
  // (odd units: v_even ^ 64 -- K is a multiple of 128, so bit 6 belongs to the chunk alone)
  // LDS -> VGPR: lane (li = l & 15, lj = l >> 4) of a 16-row sub-tile reads chunks lj and lj + 4 of
  // row li (K bytes [16 lj, +16) and [64 + 16 lj, +16)); physical chunk = logical ^ sw with
  // sw = (row & 2) | ((row & 8) >> 1), which spreads the 16 lanes of every b128 pass (lanes
  // {0-3, 12-15, 20-23, 24-27} and {4-11, 16-19, 28-31} of a half-wave) over all bank groups;
  // the second chunk is address ^ 64.  Scales: sub-tile m needs row 16m + li, 32-deep block lj,
  // i.e. 64-deep step lj >> 1, lane 32 (lj & 1) + 16 (m & 1) + li of the 128-row group, byte
  // m >> 1: one dword for the even sub-tiles, the one 64 bytes on for the odd ones.
  const uint32_t sw = (li & 2) | ((li & 8) >> 1);
  const uint32_t lane4 = (uint32_t)(lj >> 1) * 256 + (uint32_t)((lj & 1) * 32 + li) * 4;
  const uint32_t fa0 = (wm * 128 + li) * kKB + ((lj ^ sw) << 4);
  const uint32_t fb_delta = kOperand32 + (wn - wm) * 128 * kKB;
  // scale copy: lanes 0-31 fetch one 128-row group's 512 bytes of a block, lanes 32-63 the next
  // group's; wave 1 (kGrouped2d3d: a third group of A) has its upper lanes read nothing
  const uint32_t v_scale = (MODE == kGrouped2d3d && wave == 1)
                               ? (lane < 32 ? (uint32_t)lane * 16 : 0x80000000u)
                               : (uint32_t)(lane >> 5) * ks_n * 256 + (lane & 31) * 16;
  // scale groups of a ring block: A0, A1, B0, B1, A2 (512 bytes each, then 512 unused)
  const uint32_t scale_dst = kCodes32 + ((MODE == kGrouped2d3d && wave == 1) ? 2048u : (uint32_t)(wave >> 1) * 1024u);
  const uint32_t fsa_s = kCodes32 + wm * 512, fsb_s = kCodes32 + 1024 + wn * 512;
  const uint32_t fsa_hi_s = kCodes32 + (wm == 0 ? 512 : 2048);

  // ---- loader stream: fills ring block `ld_slot` with K block `ld_kb` of tile `ld_tile`
  uint32_t ld_tile = 0, ld_kb = 0, ld_nb = 1;
  int ld_slot = 0;
  __amdgpu_buffer_rsrc_t ra, rb, rs;  // codes of A, codes of B, scales this wave copies
  // kGrouped2d3d: a group may start at any multiple of 32 rows, the scales come in 128-row groups
  // of the whole matrix: a tile that starts `rot` 32-row blocks into a group fetches three groups
  // and turns the bytes of every scale dword by `rot` (next_scales).  The rotation belongs to
  // the tile whose block sits in a ring slot.
  uint32_t ld_rot = 0, slot_rot0 = 0, slot_rot1 = 0;
  // kGrouped2d2d: a K range may start and end at any multiple of 32.  Its first and last
  // 128-deep blocks send the chunks outside the range out of range, so that zeros land in the
  // ring instead of the neighbouring groups' codes and scales.
  uint32_t ld_head = 0, ld_tail = 0;
  uint32_t cur_v_even = v_even, cur_v_odd = v_even ^ 64, cur_v_scale = v_scale;
  auto set_block_offsets = [&]() {
    if constexpr (MODE == kGrouped2d2d) {
      // 32-deep blocks [first, lim) of this 128-deep block are fetched
      const uint32_t first = ld_kb == 0 ? ld_head : 0;
      const uint32_t lim = (ld_tail != 0 && ld_kb + 1 == ld_nb) ? ld_tail : 4;
      auto inside = [&](uint32_t blk) { return blk >= first && blk < lim; };
      cur_v_even = inside(c_even >> 1) ? v_even : 0x80000000u;
      cur_v_odd = inside((c_even ^ 4) >> 1) ? (v_even ^ 64) : 0x80000000u;
      cur_v_scale = inside((uint32_t)(lane & 31) >> 3) ? v_scale : 0x80000000u;
    }
  };
  auto loader_open_tile = [&]() {
    if (ld_tile < n_my) {
      const Tile32 t = get_tile(ld_tile);
      ld_nb = t.nblocks;
      ld_rot = t.rot;
      ld_head = t.head;
      ld_tail = t.tail;
      // (kGrouped2d2d: the range stops at the end of the operand rows, not of the K range;
      //  the K range is exact because nblocks is.)  A tile without a K range reads nothing:
      // its one block arrives as zeros, scales included.
      const bool none = MODE != kDense && t.empty;
      ra = make_rsrc(t.a, none ? 0 : t.rows_a * (int64_t)Kp - t.koff);
      rb = make_rsrc(t.b, none ? 0 : t.rows_b * (int64_t)Kp - t.koff);
      // wave 0 copies the scales of A's two 128-row groups, wave 2 those of B's (one copy per
      // block each: lanes 0-31 fetch group 0, lanes 32-63 group 1); a group beyond the operand
      // is cut off by the range and arrives as zeros
      // (kGrouped2d3d: rows counted from the start of the first scale group; wave 1 copies a
      // third group of A when the tile's rows reach into it)
      const int64_t rows = wave < 2 ? (t.rows_a > 0 ? t.rows_a + 32 * (int64_t)t.rot : 0) : t.rows_b;
      const uint8_t* sbase = wave < 2 ? t.sa : t.sb;
      if (MODE == kGrouped2d3d && wave == 1)
        rs = make_rsrc(sbase + (int64_t)ks_n * 512, (none || rows <= 256) ? 0 : (int64_t)ld_nb * 512);
      else
        rs = make_rsrc(sbase, none ? 0
                                   : rows > 128 ? (int64_t)ks_n * 256 + (int64_t)ld_nb * 512
                                                : (rows > 0 ? (int64_t)ld_nb * 512 : 0));
    } else {  // past the last tile: every lane reads out of range (zeros, no traffic)
      ld_nb = 1;
      ld_rot = 0;
      ld_head = 0;
      ld_tail = 0;
      ra = make_rsrc(p.a_codes, 0);
      rb = ra;
      rs = ra;
    }
    set_block_offsets();
  };
#ifndef MX_LOAD_AUX  // cache policy bits of the operand copies (0: default)
#define MX_LOAD_AUX 0
#endif
  // The 17 copies of a block are issued one at a time, between MFMAs (see block_steps):
  // piece 0..15 = unit pairs (A unit, B unit alternating), 16 = scales, then advance.
  auto issue_piece = [&](auto i_) {
    constexpr int i = decltype(i_)::value;
#ifdef MX_ABL_DMA_OOB  // timing ablation: every copy is issued with all lanes out of range (zeros land in LDS, nothing is fetched)
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.a_codes, 0), rb = ra, rs = ra;
#endif

    const uint32_t sbase = lds_base + ld_slot * kBlock32;
    if constexpr (i < 16) {
      constexpr int q = i >> 1;
      const int unit = wave * 8 + q;
      const uint32_t v = MODE == kGrouped2d2d ? ((q & 1) ? cur_v_odd : cur_v_even)
                                              : ((q & 1) ? (v_even ^ 64) : v_even);
      const uint32_t so = (uint32_t)(unit * 8) * Kp + ld_kb * kKB;
      if constexpr ((i & 1) == 0)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_void_t*)(uintptr_t)(sbase + unit * 1024), 16, v, so, 0, MX_LOAD_AUX);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rb, (lds_void_t*)(uintptr_t)(sbase + kOperand32 + unit * 1024), 16, v, so, 0, MX_LOAD_AUX);
    } else {
      // scales: a group's two 64-deep steps are 512 contiguous bytes, the two groups land behind
      // one another, which is the order the fragment reads expect.  Waves 0 and 2 copy A's and
      // B's; waves 1 and 3 copy the same bytes to the same place once more (kGrouped2d3d: wave 1
      // the third group of A instead): every wave then runs the same instructions, where a
      // branch around the copy costs the two waves that take it more than the copy itself
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rs, (lds_void_t*)(uintptr_t)(sbase + scale_dst), 16,
          MODE == kGrouped2d2d ? cur_v_scale : v_scale, ld_kb * 512, 0, 0);
    }
  };
  auto issue_advance = [&]() {
    if constexpr (MODE == kGrouped2d3d) {
      if (ld_slot) slot_rot1 = ld_rot; else slot_rot0 = ld_rot;
    }
    if (++ld_kb == ld_nb) {
      ld_kb = 0;
      ++ld_tile;
      loader_open_tile();
    } else {
      set_block_offsets();
    }
    ld_slot ^= 1;
  };
  auto issue_block = [&]() {
    static_for<0, 17>([&](auto i_) { issue_piece(i_); });
    issue_advance();
  };

  // Fragment reads are issued as inline assembly: the compiler cannot tell which ring block a
  // ds_read touches, so for reads it can see it waits until every global->LDS copy in flight
  // has landed (vmcnt(0)) and the prefetch distance collapses.  The reads are therefore
  // invisible to its wait-count tracking; `pin_set` / `landed` (after an explicit lgkmcnt wait)
  // are what the MFMAs depend on.
#ifdef MX_ABL_TR_READ
  constexpr int kReadsPerPiece = 2;
#else
  constexpr int kReadsPerPiece = 1;
#endif
  auto lds_b128 = [&](uint32_t addr, auto off_) -> v4i {
    constexpr int off = decltype(off_)::value;
    v4i v;
#ifdef MX_ABL_TR_READ  // timing ablation: the 16 bytes come as two transposing 8-byte reads
    typedef int v2i_t __attribute__((ext_vector_type(2)));
    v2i_t lo, hi;
    const uint32_t first = addr + ((lane & 16) >> 1);  // each 32-lane pass still covers all banks
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(lo) : "v"(first), "n"(off));
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(first ^ 8u), "n"(off));
    v = v4i{lo.x, lo.y, hi.x, hi.y};
#else
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(off));
#endif
    return v;
  };
  // ---- fragment sets, scale dwords
  // one b128 read of a fragment set: i = 2t + (0: K bytes [16 lj, +16), 1: [64 + 16 lj, +16)) of
  // sub-tile 4h + t
  auto read_set_piece = [&](v8i (&set)[4], uint32_t sbase, uint32_t delta, auto h_, auto i_) {
    constexpr int h = decltype(h_)::value, i = decltype(i_)::value;
    constexpr int t = i >> 1;
    constexpr bool hi = i & 1;
    const uint32_t base = (fa0 ^ (hi ? 64u : 0u)) + delta;
    const v4i v = lds_b128(sbase + base, std::integral_constant<int, (4 * h + t) * 2048>{});
    v8i& dst = set[t];
    if constexpr (hi) {
      dst[4] = v.x; dst[5] = v.y; dst[6] = v.z; dst[7] = v.w;
    } else {
      dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    }
  };
  // the scale dwords of a block, into the "next" registers: piece 0, 1 = A even / odd
  // sub-tiles, 2, 3 = B, 4, 5 = A of the next 128-row group (kGrouped2d3d)
  constexpr int kScalePieces = MODE == kGrouped2d3d ? 6 : 4;
  auto read_scale_piece = [&](Frags16& f, uint32_t sbase, auto i_) {
    constexpr int i = decltype(i_)::value;
    constexpr int e = i & 1;
    if constexpr (i < 2) {
      const uint32_t ps = sbase + fsa_s + lane4 + e * 64;
      asm volatile("ds_read_b32 %0, %1" : "=v"(f.san[e]) : "v"(ps));
    } else if constexpr (i < 4) {
      const uint32_t ps = sbase + fsb_s + lane4 + e * 64;
      asm volatile("ds_read_b32 %0, %1" : "=v"(f.sbn[e]) : "v"(ps));
    } else {
      const uint32_t ps = sbase + fsa_hi_s + lane4 + e * 64;
      asm volatile("ds_read_b32 %0, %1" : "=v"(f.sa_hi[e]) : "v"(ps));
    }
  };
  auto pin_set = [&](v8i (&set)[4]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("" : "+v"(set[t]));
  };
  // The next block's scales become the current ones, once their reads have landed.
  // kGrouped2d3d: byte k of an A scale dword becomes the scale of the tile's k-th 32-row block,
  // which is byte (rot + k) of the eight bytes that two neighbouring 128-row groups hold for
  // this lane
  auto next_scales = [&](Frags16& f, int slot) {
    asm volatile("" : "+v"(f.san[0]), "+v"(f.san[1]), "+v"(f.sbn[0]), "+v"(f.sbn[1]));
    if constexpr (MODE == kGrouped2d3d) {
      asm volatile("" : "+v"(f.sa_hi[0]), "+v"(f.sa_hi[1]));
      const uint32_t rot = slot ? slot_rot1 : slot_rot0;
      f.sa[0] = __builtin_amdgcn_alignbyte(f.sa_hi[0], f.san[0], rot);
      f.sa[1] = __builtin_amdgcn_alignbyte(f.sa_hi[1], f.san[1], rot);
    } else {
      f.sa[0] = f.san[0];
      f.sa[1] = f.san[1];
    }
    f.sb[0] = f.sbn[0];
    f.sb[1] = f.sbn[1];
  };
  // ---- compute stream
  v4f acc[8][8];
  int c_slot = 0;  // ring block holding the K block being computed
  uint64_t prof_vm = 0, prof_bar = 0, prof_body = 0, prof_last = 0, prof_epi = 0;
  uint64_t prof_e_stage = 0, prof_e_wait = 0, prof_e_store = 0;

// Output stores carry the nontemporal policy bit: written once, never re-read by this kernel,
// and without it the output lines displace operand panels in L2 and the copies of the next
// tile's first blocks queue behind the draining stores.
#ifndef MX_STORE_AUX
#define MX_STORE_AUX 2
#endif
#ifndef MX_RELEASE16
#define MX_RELEASE16 12
#endif
  // A K block is 64 MFMAs, one per 16x16 sub-tile, in four quarters of 16 (512 MFMA cycles each)
  // over the fragment sets a[0], a[1] (rows 0-63, 64-127 of the wave) and b[0], b[1], in an
  // order that needs every set for two quarters in a row (slots 0-63 = the block's MFMAs):
  //   quarter 0: a[0] x b[0], a[0]'s sub-tiles one after the other.  Read meanwhile, from this
  //              block: the last sub-tile of a[0] (slots 0, 1; used from slot 12) and b[1]
  //              (2-9).  Once every wave has done so (barrier in front of slot kRelease) the
  //              ring block is free and the copies of block b+2 start, one every third slot
  //              (the copy unit takes about 20 cycles per copy for each of the four waves)
  //   quarter 1: a[1] x b[0]
  //   quarter 2: a[1] x b[1].  Block b+1 must have landed (wait, barrier); its b[0] and scales
  //              are read
  //   quarter 3: a[0] x b[1], a[0]'s sub-tiles one after the other.  a[1] takes block b+1's data,
  //              and so does a sub-tile of a[0] as soon as an MFMA of the next sub-tile has been
  //              issued (slots 52/53, 56/57, 60/61)
  // A register is read from LDS between the last MFMA that uses its old contents and its first
  // use; LDS reads return in order, so "the reads issued up to some point have landed" is
  // s_waitcnt lgkmcnt(number of reads issued since).  An MFMA occupies the matrix pipe for 32
  // cycles and the wave's issue for about half of that: what is issued behind it has to fit
  // the other half, so copies and reads are spread over the slots as evenly as the rules above
  // allow.
  constexpr int kRelease = MX_RELEASE16;          // slot in front of which the ring block is released
  constexpr int kFirstCopy = kRelease + 1;        // copy j goes behind the MFMA of slot kFirstCopy + 3j
  constexpr int kCopiesA = (32 - kFirstCopy + 2) / 3;  // copies issued in quarters 0 and 1
  static_assert(kRelease >= 12 && kFirstCopy + 3 * 16 < 64, "seventeen copies, three slots apart");
  auto copy_at = [&](auto slot_) {  // slot 0..63 of the block
#ifndef MX_ABL_NO_DMA
    constexpr int sl = decltype(slot_)::value;
    if constexpr (sl >= kFirstCopy && (sl - kFirstCopy) % 3 == 0 && (sl - kFirstCopy) / 3 < 17)
      issue_piece(std::integral_constant<int, (sl - kFirstCopy) / 3>{});
#endif
  };
  // quarter: 16 MFMAs of a[ah] x b[bh]; AMAJOR: a's sub-tiles one after the other (else b's);
  // side(slot, false) runs in front of a slot's MFMA, side(slot, true) behind it
  auto quarter = [&](Frags16& f, auto first_, auto ah_, auto bh_, auto amajor_, auto&& side) {
    constexpr bool kFirst = decltype(first_)::value;
    constexpr int ah = decltype(ah_)::value, bh = decltype(bh_)::value;
    constexpr bool kAMajor = decltype(amajor_)::value;
    static_for<0, 16>([&](auto i_) {
      constexpr int i = decltype(i_)::value;
      constexpr int tm = kAMajor ? i >> 2 : i & 3, tn = kAMajor ? i & 3 : i >> 2;
      constexpr int m = 4 * ah + tm, n = 4 * bh + tn;
      side(i_, std::false_type{});
      mfma16_asm<(n >> 1), (m >> 1), kFirst>(acc[m][n], f.b[bh][tn], f.a[ah][tm], f.sb[n & 1], f.sa[m & 1]);
      side(i_, std::true_type{});
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto landed = [&](auto n_, v8i& frag) {  // all LDS reads but the n youngest have landed
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsPerPiece * decltype(n_)::value > 15 ? 15 : kReadsPerPiece * decltype(n_)::value) : "memory");
    asm volatile("" : "+v"(frag));
  };
  auto block_steps = [&](Frags16& f, auto first_) {
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    const uint32_t s_cur = lds_base + c_slot * kBlock32, s_nxt = lds_base + (c_slot ^ 1) * kBlock32;
    // quarter 0.  In flight on entry, oldest first: the last two reads of a[1], a[0][1], the
    // other last two reads of a[1], a[0][2] (see quarter 3)
    quarter(f, first_, H0{}, H0{}, std::true_type{}, [&](auto i_, auto after_) {
      constexpr int i = decltype(i_)::value;
      if constexpr (!decltype(after_)::value) {
        if constexpr (i == 4) landed(std::integral_constant<int, 4 + 4>{}, f.a[0][1]);
        if constexpr (i == 8) landed(std::integral_constant<int, 8>{}, f.a[0][2]);
        if constexpr (i == kRelease) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's reads of the block are done
          asm volatile("" : "+v"(f.a[0][3]));
          uint64_t t0 = 0;
          if constexpr (PROF) t0 = __builtin_readcyclecounter();
          __builtin_amdgcn_s_barrier();
          if constexpr (PROF) {
            const uint64_t t1 = __builtin_readcyclecounter();
            prof_bar += t1 - t0;
            prof_last += t1 - t0;  // keep the barrier out of the body figure
          }
        }
      } else {
#ifndef MX_ABL_NO_READ
        if constexpr (i < 2) read_set_piece(f.a[0], s_cur, 0u, H0{}, std::integral_constant<int, 6 + i>{});
        else if constexpr (i < 10) read_set_piece(f.b[1], s_cur, fb_delta, H1{}, std::integral_constant<int, i - 2>{});
#endif
        copy_at(i_);
      }
    });
    pin_set(f.a[1]);
    pin_set(f.b[1]);
    // quarter 1
    quarter(f, first_, H1{}, H0{}, std::false_type{}, [&](auto i_, auto after_) {
      if constexpr (decltype(after_)::value) copy_at(std::integral_constant<int, 16 + decltype(i_)::value>{});
    });
    uint64_t t0 = 0, t1 = 0;
    if constexpr (PROF) {
      t0 = __builtin_readcyclecounter();
      prof_body += t0 - prof_last;
    }
    // block b+1 (and any output stores): everything but the copies issued so far in this block
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kCopiesA) : "memory");
    if constexpr (PROF) {
      t1 = __builtin_readcyclecounter();
      prof_vm += t1 - t0;
    }
    __builtin_amdgcn_s_barrier();
    if constexpr (PROF) {
      prof_last = __builtin_readcyclecounter();
      prof_bar += prof_last - t1;
    }
    // quarter 2: b[0] of block b+1 and its first three scale dwords, in the slots without a copy
    quarter(f, first_, H1{}, H1{}, std::false_type{}, [&](auto i_, auto after_) {
      constexpr int i = decltype(i_)::value, sl = 32 + i;
      if constexpr (decltype(after_)::value) {
        copy_at(std::integral_constant<int, sl>{});
#ifndef MX_ABL_NO_READ
        constexpr bool has_copy = sl >= kFirstCopy && (sl - kFirstCopy) % 3 == 0;
        // free slots of the quarter before this one
        constexpr int before = i - (sl - kFirstCopy + 2) / 3 + (32 - kFirstCopy + 2) / 3;
        if constexpr (!has_copy) {
          if constexpr (before < 8) read_set_piece(f.b[0], s_nxt, fb_delta, H0{}, std::integral_constant<int, before>{});
          else if constexpr (before < 11) read_scale_piece(f, s_nxt, std::integral_constant<int, before - 8>{});
        }
#endif
      }
    });
    // quarter 3, reads by slot: a[1] 0 (+ the fourth scale dword), 1, 2, 3 (+ the two dwords of
    // the next scale group, kGrouped2d3d), a[0][0], a[1] 4, 5, a[0][1], a[1] 6, 7, a[0][2]
    quarter(f, first_, H0{}, H1{}, std::true_type{}, [&](auto i_, auto after_) {
      constexpr int i = decltype(i_)::value;
      if constexpr (decltype(after_)::value) {
        copy_at(std::integral_constant<int, 48 + i>{});
#ifndef MX_ABL_NO_READ
        if constexpr (i < 4) {
          read_set_piece(f.a[1], s_nxt, 0u, H1{}, i_);
          if constexpr (i == 0) read_scale_piece(f, s_nxt, std::integral_constant<int, 3>{});
          if constexpr (kScalePieces == 6 && i >= 2) read_scale_piece(f, s_nxt, std::integral_constant<int, i + 2>{});
        } else if constexpr (i < 14) {
          constexpr int k = i - 4;  // 0, 1: a[0][0]; 2, 3: a[1] 4, 5; 4, 5: a[0][1]; 6, 7: a[1] 6, 7; 8, 9: a[0][2]
          if constexpr ((k & 3) < 2) read_set_piece(f.a[0], s_nxt, 0u, H0{}, std::integral_constant<int, 2 * (k >> 2) + (k & 1)>{});
          else read_set_piece(f.a[1], s_nxt, 0u, H1{}, std::integral_constant<int, 4 + 2 * (k >> 2) + (k & 1)>{});
        }
#endif
      }
    });
    c_slot ^= 1;
    // the next block's first MFMAs need its b[0], its scales and the first sub-tile of its
    // a[0]: everything but the eight reads issued since
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsPerPiece * 8 > 15 ? 15 : kReadsPerPiece * 8) : "memory");
    pin_set(f.b[0]);
    asm volatile("" : "+v"(f.a[0][0]));
    next_scales(f, c_slot);
    issue_advance();
  };

  // Output: a lane holds, per 16x16 sub-tile, row li and columns 4lj + 0..3.  Lanes of
  // neighbouring lane groups trade halves with v_permlane16_swap so that each owns 8 consecutive
  // bf16 of a row; a 32-row x 64-column piece is then turned around in this wave's private LDS
  // patch (the 26 KB the ring leaves free) so that 8 lanes store one full 128-byte line of a row
  // -- stores that scatter 32-byte pieces over many rows back up the write path.
  // Buffer stores: one descriptor per tile bounds the rows, a 32-bit offset per lane, scalar
  // offsets per piece.  Requires N % 8 == 0 and ldd % 8 == 0 (checked on the host).
  // (LDS accesses as assembly, for the reason given at the fragment reads.)
  constexpr int kPatchPitch = 144;  // bytes per staged row: 128 + 16, keeps b128 accesses spread
  const uint32_t patch = lds_base + kRing32 + wave * kPatch32;
  const uint32_t nan_mask = (MODE != kDense && poison) ? 0x7FC07FC0u : 0u;
  auto epilogue = [&](const Tile32& t) {
    // The epilogue's per-lane addresses are worked out here, from a lane number the compiler
    // cannot see through, every time: kept across the K loop instead they push its register
    // file over the edge, and a spilled register's reload waits for every copy and store in
    // flight (s_waitcnt vmcnt(0)) at exactly the two places where those should keep running.
    uint32_t lane_e = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane_e));
    // + (m & 1) * 16 rows + (second sub-tile pair of the piece) * 64
    const uint32_t patch_w = patch + (lane_e & 15) * kPatchPitch + ((lane_e >> 4) & 1) * 32 + (lane_e >> 5) * 16;
    const uint32_t patch_r = patch + (lane_e >> 3) * kPatchPitch + (lane_e & 7) * 16;  // + pass*8 rows
    const int64_t rows_valid = (MODE == kGrouped2d3d && p.d_offs) ? (int64_t)t.rows_d : t.rows_a;
    const uint32_t cols_valid = (uint32_t)(t.rows_b < kT32 ? t.rows_b : kT32);
    if constexpr (MODE == kSplitK) {
      // float32 partial sums straight from the accumulators: a lane stores 16 bytes of row li
      // per sub-tile and q; short pieces, but the partial tiles are few and are read back at once
      const uint32_t ld_b = (uint32_t)p.ldd * 4;
      const __amdgpu_buffer_rsrc_t rp = make_rsrc(t.d, rows_valid * ld_b);
      const uint32_t row_b = (wm * 128 + li) * ld_b;
      // (a lane holds row 16m + li, columns 16n + 4lj + 0..3 of sub-tile (m, n))
      static_for<0, 64>([&](auto i_) {
        constexpr int m = decltype(i_)::value >> 3, n = decltype(i_)::value & 7;
        const uint32_t col = wn * 128 + n * 16 + 4 * lj;
        const uint32_t v = col < cols_valid ? row_b + col * 4 : 0x80000000u;
        const u32x4 w = {__float_as_uint(acc_read<0>(acc[m][n])), __float_as_uint(acc_read<1>(acc[m][n])),
                         __float_as_uint(acc_read<2>(acc[m][n])), __float_as_uint(acc_read<3>(acc[m][n]))};
        __builtin_amdgcn_raw_buffer_store_b128(w, rp, v, m * 16 * ld_b, MX_STORE_AUX);
      });
      return;
    }
    const uint32_t ldd_b = (uint32_t)p.ldd * 2;
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(t.d, rows_valid * ldd_b);
    // lane's place in a stored piece: row (lane >> 3) + 8*pass, columns (lane & 7)*8 .. +7
    const uint32_t colp = wn * 128 + (lane_e & 7) * 8;
    const uint32_t vrow = (wm * 128 + (lane_e >> 3)) * ldd_b + colp * 2;
    // Pieces p = 0..7: 32 rows (sub-tile row m = p/2) x 64 columns (sub-tiles n = 2(p%2), +1).
    // A wave's LDS instructions execute in order, so a piece's reads may follow its writes
    // without a wait, and the next piece's writes may follow those reads: the only waits are
    // for the read data, with the next piece's conversion and writes already under way.
    // a lane holds row 16m + li, columns 16n + 4lj + 0..3 of sub-tile (m, n).  Part k of
    // piece p covers 16 rows x 32 columns: sub-tiles (m, n) and (m, n + 1), m = 2(p / 2) + k / 2,
    // n = 4(p % 2) + 2(k % 2).  v_permlane16_swap trades the halves of two neighbouring lane
    // groups: the even groups end up with 8 consecutive columns of sub-tile n, the odd ones with
    // 8 of sub-tile n + 1.
    auto stage_part = [&](auto p_, auto k_) {
      constexpr int mp = decltype(p_)::value >> 1, np = decltype(p_)::value & 1, k = decltype(k_)::value;
      constexpr int m = 2 * mp + (k >> 1), n = 4 * np + 2 * (k & 1);
      const v4f& c0 = acc[m][n];
      const v4f& c1 = acc[m][n + 1];
      const float a[8] = {acc_read<0>(c0), acc_read<1>(c0), acc_read<2>(c0), acc_read<3>(c0),
                          acc_read<0>(c1), acc_read<1>(c1), acc_read<2>(c1), acc_read<3>(c1)};
      uint32_t x0 = pack_bf16(a[0], a[1]), y0 = pack_bf16(a[2], a[3]);
      uint32_t x1 = pack_bf16(a[4], a[5]), y1 = pack_bf16(a[6], a[7]);
      if constexpr (MODE != kDense) {  // a broken group contract must not pass unnoticed: NaN
        x0 |= nan_mask;
        y0 |= nan_mask;
        x1 |= nan_mask;
        y1 |= nan_mask;
      }
      const u32x2 sx = __builtin_amdgcn_permlane16_swap(x0, x1, false, false);
      const u32x2 sy = __builtin_amdgcn_permlane16_swap(y0, y1, false, false);
      const v4i w = {(int)sx.x, (int)sy.x, (int)sx.y, (int)sy.y};
      lds_write_b128_hidden<(m & 1) * 16 * kPatchPitch + (k & 1) * 64>(patch_w, w);
      __builtin_amdgcn_sched_barrier(0);
    };
    v4i r[2][4];
    static_for<0, 4>([&](auto k_) { stage_part(std::integral_constant<int, 0>{}, k_); });
    static_for<0, 8>([&](auto p_) {
      constexpr int pc = decltype(p_)::value, m = pc >> 1, np = pc & 1;
      uint64_t e0 = 0;
      if constexpr (PROF) e0 = __builtin_readcyclecounter();
      static_for<0, 4>([&](auto q_) {
        constexpr int q = decltype(q_)::value;
        r[pc & 1][q] = lds_read_b128_hidden<q * 8 * kPatchPitch>(patch_r);
      });
      const uint32_t v = (colp + np * 64 < cols_valid) ? vrow + np * 128 : 0x80000000u;
      // the next piece's conversion runs between this piece's stores, which drain at the
      // write path's pace
      static_for<0, 4>([&](auto q_) {
        constexpr int q = decltype(q_)::value;
        if constexpr (pc < 7) stage_part(std::integral_constant<int, pc + 1>{}, q_);
        if constexpr (q == 0) {
          // the four reads are done once at most the one younger write is outstanding
          if constexpr (pc < 7) asm volatile("s_waitcnt lgkmcnt(1)" ::: "memory");
          else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        const v4i rq = pin(r[pc & 1][q]);
        const u32x4 w = {(uint32_t)rq.x, (uint32_t)rq.y, (uint32_t)rq.z, (uint32_t)rq.w};
#ifdef MX_ABL_STORE_ROWS  // timing ablation: only sub-tile rows below this many are written
        if constexpr (m < MX_ABL_STORE_ROWS)
#endif
        __builtin_amdgcn_raw_buffer_store_b128(w, rd, v, (m * 32 + q * 8) * ldd_b, MX_STORE_AUX);
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (PROF) prof_e_stage += __builtin_readcyclecounter() - e0;
    });
  };

  uint64_t prof_t0 = 0;
  if constexpr (PROF) prof_t0 = __builtin_readcyclecounter();
  // ---- prologue: fill the ring, fetch the first fragments
  loader_open_tile();
  issue_block();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  issue_block();  // block 1: in flight when the first step starts
  Frags16 f;
  {
    using Z = std::integral_constant<int, 0>;
    using O = std::integral_constant<int, 1>;
    static_for<0, 8>([&](auto i_) { read_set_piece(f.a[0], lds_base, 0u, Z{}, i_); });
    static_for<0, 8>([&](auto i_) { read_set_piece(f.a[1], lds_base, 0u, O{}, i_); });
    static_for<0, 8>([&](auto i_) { read_set_piece(f.b[0], lds_base, fb_delta, Z{}, i_); });
    static_for<0, kScalePieces>([&](auto i_) { read_scale_piece(f, lds_base, i_); });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    pin_set(f.a[0]);
    pin_set(f.a[1]);
    pin_set(f.b[0]);
    next_scales(f, 0);
  }
  if constexpr (PROF) prof_last = __builtin_readcyclecounter();

  // ---- tiles; at the top of every tile f0 holds the fragments of its first half block (the
  // last step of a tile has already read them from the next tile's first block, which the
  // loader fetched like any other block).
  for (uint32_t tile = 0; tile < n_my; tile += PAIR ? 2 : 1) {
    const Tile32 t = get_tile(tile);
    {
      // PAIR: the loader walks both segments of the tile one after the other (same K for both);
      // for the compute stream they are one run of blocks
      const uint32_t nblocks = PAIR ? 2 * t.nblocks : t.nblocks;
      block_steps(f, std::true_type{});
      // two blocks per trip: a taken branch stalls the lone wave of a SIMD for longer than the
      // 32 cycles its last MFMA covers, and the trip's end has two of them
      uint32_t i = 1;
      for (; i + 2 <= nblocks; i += 2) {
        block_steps(f, std::false_type{});
        block_steps(f, std::false_type{});
      }
      if (i < nblocks) block_steps(f, std::false_type{});
      // the next tile's first fragments, read in the last quarter, become ordinary values
      // before anything else runs
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      pin_set(f.a[0]);
      pin_set(f.a[1]);
      if constexpr (PROF) {
        const uint64_t e0 = __builtin_readcyclecounter();
        prof_body += e0 - prof_last;
        epilogue(t);
        prof_last = __builtin_readcyclecounter();
        prof_epi += prof_last - e0;
      } else {
#ifndef MX_ABL_NO_EPILOGUE
        epilogue(t);
#else
        (void)t;  // timing ablation: the MFMAs are volatile assembly and stay
#endif
      }
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
      o[4] = prof_e_stage;
      o[5] = prof_e_wait;
      o[6] = prof_e_store;
      o[7] = __builtin_readcyclecounter() - prof_t0;
    }
  }
}

// Test hook, process-wide: > 0 = number of persistent workgroups (also lowers how many tiles one
// grouped launch covers, which is what the tests use it for); 0 = one per CU.
static std::atomic<int> debug_grid{0};
#ifdef MX_TIMING_BUILD
static uint64_t* debug_prof = nullptr;  // device buffer for the per-wave cycle counts, or nullptr
#else
static constexpr uint64_t* debug_prof = nullptr;
#endif

// One persistent workgroup per CU of the current device, a multiple of the 8 XCDs (0: the device
// cannot be queried).
static int64_t persistent_grid() {
  const int num_cus = current_device_cus();
  if (num_cus == 0) return 0;
  int64_t grid = (num_cus / 8) * 8;
  if (grid < 8) grid = 8;
  if (debug_grid > 0) grid = (debug_grid + 7) / 8 * 8;
  return grid;
}

template <int MODE, bool PROF, bool PAIR = false>
static int launch32(const Gemm32Args& p, int64_t nb, hipStream_t st) {
  auto kern = gemm_nt32_kernel<MODE, PROF, PAIR>;
  constexpr int lds = kRing32 + 4 * kPatch32;  // ring + one output patch per wave = all 160 KB
  static std::atomic<bool> configured[kMaxDevices];
  if (!raise_lds_limit(reinterpret_cast<const void*>(kern), lds, configured)) return MX_ERR_LAUNCH;
  int64_t grid = persistent_grid();
  if (grid == 0) return MX_ERR_LAUNCH;
  const int64_t need = (nb + 7) / 8 * 8;  // nb: the tile count, or an upper bound of it
  if (need < grid && debug_grid <= 0) grid = need;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), lds, st, p);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

void set_debug_grid(int g) { debug_grid = g; }
#ifdef MX_TIMING_BUILD
void set_debug_prof(uint64_t* buf) { debug_prof = buf; }
#endif

int launch_gemm_nt32(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                     const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                     int64_t ldk, int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, nullptr, 0, 0, 0, debug_prof};
  p.ldk = ldk;
  const int64_t nb = ((M + kT32 - 1) / kT32) * ((N + kT32 - 1) / kT32);
#ifdef MX_TIMING_BUILD
  if (debug_prof) return launch32<kDense, true>(p, nb, st);
#endif
  return launch32<kDense, false>(p, nb, st);
}

// ---- split along K for shapes whose 256x256 tiles do not fill the CUs ----------------------
// Sum of the S float32 partial matrices [S][M][N], in slice order, rounded once to bf16.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int S,
                                                            int64_t M, int64_t N,
                                                            uint16_t* __restrict__ d, int64_t ldd) {
  const int64_t per_row = N / 8, i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * per_row) return;
  const int64_t r = i / per_row, c = (i - r * per_row) * 8;
  const float* src = part + r * N + c;
  float acc[8];
  {
    const v4f lo = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src));
    const v4f hi = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(src) + 1);
    acc[0] = lo.x; acc[1] = lo.y; acc[2] = lo.z; acc[3] = lo.w;
    acc[4] = hi.x; acc[5] = hi.y; acc[6] = hi.z; acc[7] = hi.w;
  }
  for (int s = 1; s < S; ++s) {
    const float* q = src + (int64_t)s * M * N;
    const v4f lo = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(q));
    const v4f hi = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(q) + 1);
    acc[0] += lo.x; acc[1] += lo.y; acc[2] += lo.z; acc[3] += lo.w;
    acc[4] += hi.x; acc[5] += hi.y; acc[6] += hi.z; acc[7] += hi.w;
  }
  const u32x4 w = {pack_bf16(acc[0], acc[1]), pack_bf16(acc[2], acc[3]), pack_bf16(acc[4], acc[5]),
                   pack_bf16(acc[6], acc[7])};
  *reinterpret_cast<u32x4*>(d + r * ldd + c) = w;
}

// Number of K slices for a dense shape on the persistent kernel (1: no split), from a cost model
// in microseconds fitted to measurements on MI355X:
//   one 128-deep block of a 256x256 tile takes a CU 1.6 us with the whole chip busy (about 10 %
//   less with idle CUs: the clock is power-bound);
//   unsplit, up to 3/8 of the CUs' worth of tiles go to the 128x128-tile kernel, 1.3 PFLOP/s
//   times the share of the CUs its tiles cover;
//   split, S slices run ceil(tiles * S / CUs) rounds of blocks / S each, then the float32
//   partial tiles make a round trip through memory (8 bytes per element and slice at 3 TB/s)
//   plus a second launch.
// The split is taken when the model promises at least a fifth less time: a 2048 x 2048 weight
// gradient over 147 456 tokens 1265 -> 559 us, over 32 768 tokens 198 -> 154 us; over 16 384
// tokens it stays unsplit (105 vs 110 us).
int splitk_slices(int64_t M, int64_t N, int64_t K) {
  const int64_t grid = persistent_grid();
  if (grid == 0 || K % kKB) return 1;
  const int64_t tiles = ((M + kT32 - 1) / kT32) * ((N + kT32 - 1) / kT32), blocks = K / kKB;
  if (tiles >= 2 * grid) return 1;
  const double block_us = 1.6, flops = 2.0 * (double)M * (double)N * (double)K;
  double plain;
  if (tiles * 8 <= grid * 3) {
    const double share = 4.0 * tiles / grid;
    plain = flops / (1.3e9 * (share < 1.0 ? share : 1.0));  // 1.3e9 flop per microsecond
  } else {
    plain = (double)((tiles + grid - 1) / grid) * blocks * block_us * (tiles < grid ? 0.9 : 1.0);
  }
  int best = 1;
  double best_us = plain;
  for (int s = 2; s <= 8; ++s) {
    const int64_t per = (blocks + s - 1) / s;
    if (per < 16 || (int64_t)(s - 1) * per >= blocks) continue;
    const double us = (double)((tiles * s + grid - 1) / grid) * per * block_us +
                      (double)s * M * N * 8.0 / 3.0e6 + 8.0;
    if (us < best_us) {
      best = s;
      best_us = us;
    }
  }
  return best_us <= 0.8 * plain ? best : 1;
}

// D = sum over slices, through `workspace` (S * M * N floats).
int launch_gemm_nt32_splitk(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                            const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                            int64_t ldk, int64_t ldd, int slices, void* workspace, hipStream_t st) {
  const int64_t tiles_n = (N + kT32 - 1) / kT32, tiles = ((M + kT32 - 1) / kT32) * tiles_n;
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)workspace, M, N, K, N, nullptr,
               slices, 0, (int32_t)tiles_n, nullptr};
  p.ldk = ldk;
  const int rc = launch32<kSplitK, false>(p, tiles * slices, st);
  if (rc != MX_OK) return rc;
  const int64_t threads = M * (N / 8);
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st,
                     (const float*)workspace, slices, M, N, (uint16_t*)d, ldd);
  return hipGetLastError() == hipSuccess ? MX_OK : MX_ERR_LAUNCH;
}

// Grouped forms with every group end a multiple of 32 and all scales in MFMA order
// (a_scales over the whole [T, K/32] matrix, b_scales one block per expert).  A workgroup keeps
// a record per tile in LDS, at most kMaxRecords of them: larger problems are cut into several
// launches over ranges of tile columns.
constexpr int64_t kMaxRecords = kMaxTileRecords;

template <int MODE, bool PAIR = false>
static int launch_grouped32(Gemm32Args p, int64_t tiles_per_column, int64_t tiles_n, hipStream_t st) {
  const int64_t grid = persistent_grid();
  if (grid == 0) return MX_ERR_LAUNCH;
  // tiles of one launch <= grid * kMaxRecords - slack for the rounding of the per-XCD runs
  // (PAIR: two records per tile)
  int64_t cols = (grid * (kMaxRecords / (PAIR ? 2 : 1)) - 8 * (grid / 8)) / tiles_per_column;
  if (cols < 1) return MX_ERR_UNSUPPORTED;
  if (cols > tiles_n) cols = tiles_n;
  for (int64_t tn0 = 0; tn0 < tiles_n; tn0 += cols) {
    p.tn0 = (int32_t)tn0;
    p.tn_cnt = (int32_t)(tiles_n - tn0 < cols ? tiles_n - tn0 : cols);
    const int64_t nb = tiles_per_column * p.tn_cnt;
    int rc;
    if constexpr (PAIR)
      rc = launch32<MODE, false, true>(p, nb, st);
    else {
#ifdef MX_TIMING_BUILD
      rc = p.prof ? launch32<MODE, true>(p, nb, st) : launch32<MODE, false>(p, nb, st);
#else
      rc = launch32<MODE, false>(p, nb, st);
#endif
    }
    if (rc != MX_OK) return rc;
  }
  return MX_OK;
}

int launch_grouped32_2d3d(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                          const uint8_t* b_scales, const int32_t* offs, void* d, int64_t T,
                          int64_t N, int64_t K, int64_t G, int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, T, N, K, ldd, offs, G, 0, 0, debug_prof};
  // an upper bound of the tile rows: every group may add one partly filled tile
  return launch_grouped32<kGrouped2d3d>(p, (T + kT32 - 1) / kT32 + G + 1, (N + kT32 - 1) / kT32, st);
}

// D = A B^T and D2 = A B2^T in one launch (same shapes), dense and grouped 2D x 3D.
int launch_gemm_nt32_two_b(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                           const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk, int64_t ldd,
                           hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, nullptr, 0, 0, 0, nullptr};
  p.b2_codes = b2_codes;
  p.b2_scales = b2_scales;
  p.two = kTwoB;
  p.d2 = (uint16_t*)d2;
  p.ldk = ldk;
  return launch32<kDense, false>(p, ((M + kT32 - 1) / kT32) * 2 * ((N + kT32 - 1) / kT32), st);
}
int launch_grouped32_2d3d_two_b(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                                const int32_t* offs, void* d, void* d2, int64_t T, int64_t N, int64_t K,
                                int64_t G, int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, T, N, K, ldd, offs, G, 0, 0, nullptr};
  p.b2_codes = b2_codes;
  p.b2_scales = b2_scales;
  p.two = kTwoB;
  p.d2 = (uint16_t*)d2;
  return launch_grouped32<kGrouped2d3d>(p, (T + kT32 - 1) / kT32 + G + 1, 2 * ((N + kT32 - 1) / kT32), st);
}
// D = A B^T and D2 = A2 B^T in one launch (same shapes), dense and grouped 2D x 2D.
int launch_gemm_nt32_two_a(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* a2_codes,
                           const uint8_t* a2_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk, int64_t ldd,
                           hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, nullptr, 0, 0, 0, nullptr};
  p.a2_codes = a2_codes;
  p.a2_scales = a2_scales;
  p.two = kTwoA;
  p.d2 = (uint16_t*)d2;
  p.ldk = ldk;
  return launch32<kDense, false>(p, 2 * ((M + kT32 - 1) / kT32) * ((N + kT32 - 1) / kT32), st);
}
int launch_grouped32_2d2d_two_a(const uint8_t* at_codes, const uint8_t* at_scales, const uint8_t* at2_codes,
                                const uint8_t* at2_scales, const uint8_t* bt_codes, const uint8_t* bt_scales,
                                const int32_t* offs, void* d, void* d2, int64_t T, int64_t N, int64_t K,
                                int64_t G, hipStream_t st) {
  Gemm32Args p{at_codes, at_scales, bt_codes, bt_scales, (uint16_t*)d, N, K, T, K, offs, G, 0, 0, nullptr};
  p.a2_codes = at2_codes;
  p.a2_scales = at2_scales;
  p.two = kTwoA;
  p.d2 = (uint16_t*)d2;
  return launch_grouped32<kGrouped2d2d>(p, (G + 7) / 8 * 8 * 2 * ((N + kT32 - 1) / kT32), (K + kT32 - 1) / kT32, st);
}

// D = A B^T + A2 B2^T (dense) and its grouped 2D x 3D form: both operand sets of the same shapes.
int launch_gemm_nt32_pair(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                          const uint8_t* b_scales, const uint8_t* a2_codes, const uint8_t* a2_scales,
                          const uint8_t* b2_codes, const uint8_t* b2_scales, void* d, int64_t M,
                          int64_t N, int64_t K, int64_t ldk, int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, M, N, K, ldd, nullptr, 0, 0, 0, nullptr,
               a2_codes, a2_scales, b2_codes, b2_scales};
  p.ldk = ldk;
  const int64_t nb = ((M + kT32 - 1) / kT32) * ((N + kT32 - 1) / kT32);
  return launch32<kDense, false, true>(p, nb, st);
}

int launch_grouped32_2d3d_pair(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                               const uint8_t* b_scales, const uint8_t* a2_codes,
                               const uint8_t* a2_scales, const uint8_t* b2_codes,
                               const uint8_t* b2_scales, const int32_t* offs, void* d, int64_t T,
                               int64_t N, int64_t K, int64_t G, int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, T, N, K, ldd, offs, G, 0, 0, nullptr,
               a2_codes, a2_scales, b2_codes, b2_scales};
  return launch_grouped32<kGrouped2d3d, true>(p, (T + kT32 - 1) / kT32 + G + 1, (N + kT32 - 1) / kT32, st);
}

// Grouped 2D x 3D (one product, or with a2_codes the sum of two) whose output leaves the groups'
// padding out: see Gemm32Args::d_offs.
int launch_grouped32_2d3d_rows_out(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                   const uint8_t* b_scales, const uint8_t* a2_codes,
                                   const uint8_t* a2_scales, const uint8_t* b2_codes,
                                   const uint8_t* b2_scales, const int32_t* offs, const int32_t* d_offs,
                                   void* d, int64_t T, int64_t d_rows, int64_t N, int64_t K, int64_t G,
                                   int64_t ldd, hipStream_t st) {
  Gemm32Args p{a_codes, a_scales, b_codes, b_scales, (uint16_t*)d, T, N, K, ldd, offs, G, 0, 0, nullptr,
               a2_codes, a2_scales, b2_codes, b2_scales};
  p.d_offs = d_offs;
  p.d_rows = d_rows;
  const int64_t tile_rows = (T + kT32 - 1) / kT32 + G + 1, tiles_n = (N + kT32 - 1) / kT32;
  if (a2_codes) return launch_grouped32<kGrouped2d3d, true>(p, tile_rows, tiles_n, st);
  return launch_grouped32<kGrouped2d3d>(p, tile_rows, tiles_n, st);
}

// D[g][N, K] = A^T[N, lo:hi] B^T[K, lo:hi]^T; operand rows are T long.
int launch_grouped32_2d2d(const uint8_t* at_codes, const uint8_t* at_scales,
                          const uint8_t* bt_codes, const uint8_t* bt_scales, const int32_t* offs,
                          void* d, int64_t T, int64_t N, int64_t K, int64_t G, hipStream_t st) {
  Gemm32Args p{at_codes, at_scales, bt_codes, bt_scales, (uint16_t*)d, N, K, T, K, offs, G, 0, 0, debug_prof};
  // tiles per column counted with G rounded up to the 8 XCDs: the kernel deals whole groups to
  // XCDs, and the busiest XCD's share must fit its workgroups' records
  return launch_grouped32<kGrouped2d2d>(p, (G + 7) / 8 * 8 * ((N + kT32 - 1) / kT32), (K + kT32 - 1) / kT32, st);
}

}  // namespace mx
