/*
 * C ABI of the MI355X (gfx950) MXFP8 linear path.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream (as void*), launches
 * asynchronously on that stream, allocates nothing, never synchronises, and returns an
 * mx_status_t (0 = ok).  No exceptions cross this boundary.  Calls may come from several host
 * threads and for several GPUs (each call works on the calling thread's current device): the
 * library keeps no mutable state of its own beyond per-device set-up flags, which are atomic.
 * Concurrent calls must use distinct output buffers; mx_gemm_nt_static has its own rule (below).
 *
 * The reference has no native interface for this path: its converter hands the arithmetic
 * to an external Python library.  Each declaration cites the reference statement that the
 * entry point stands in for.
 *
 * Data formats (OCP Microscaling v1.0, "MXFP8"):
 *   codes   uint8  e4m3fn (S EEEE MMM, bias 7, max 448, 0x7F/0xFF NaN), saturating RNE
 *   scales  uint8  E8M0, byte b = 2^(b-127), 255 = NaN; one per 32 consecutive elements
 *   hp      bf16   (uint16 bit patterns), row-major
 */
#ifndef MXFP8_H_
#define MXFP8_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  MX_OK = 0,
  MX_ERR_INVALID_ARG = 1,   /* null pointer, negative size, bad enum */
  MX_ERR_ALIGNMENT = 2,     /* a dimension is not a multiple of what the kernel needs */
  MX_ERR_LAUNCH = 3,        /* hipLaunchKernel reported an error */
  MX_ERR_UNSUPPORTED = 4,   /* shape outside what this build handles */
  MX_ERR_SCRATCH_TOO_SMALL = 5 /* mx_gemm_nt_static: the split needs more than the built-in scratch */
} mx_status_t;

/* How the E8M0 scale is derived from the block's max |x| (amax = (1+m) 2^E):
 *   FLOOR  s = E - 8                         (OCP MX v1.0 section 6.3; may saturate codes)
 *   RCEIL  s = ceil(log2(amax / 448))        (recipe "mxfp8_rceil",
 *                                             torchtitan/components/quantization/mx.py:37-42)
 */
typedef enum { MX_SCALE_FLOOR = 0, MX_SCALE_RCEIL = 1 } mx_scale_mode_t;

/* Where a cast writes its scale bytes:
 *   ROWMAJOR  [rows, nblk]
 *   MFMA      [ceil(rows/128), ceil(nblk/2), 64, 4]: for row group rt, 64-deep K step ks,
 *             lane l, byte t the entry is scale[rt*128 + t*32 + (l & 31)][ks*2 + (l >> 5)]
 *             (zero beyond the matrix) -- one dword per lane feeds four 32-row sub-tiles of
 *             v_mfma_scale_f32_32x32x64_f8f6f4, or four 16-row sub-tiles 32 rows apart of
 *             v_mfma_scale_f32_16x16x128_f8f6f4; the order mx_gemm_nt reads.
 */
typedef enum { MX_SCALES_ROWMAJOR = 0, MX_SCALES_MFMA = 1 } mx_scale_order_t;

/* Library/ABI version (major*100 + minor). */
int mx_version(void);
const char* mx_status_string(int status);

/* Bytes of a scale buffer in MX_SCALES_MFMA order for a [rows, nblk] scale matrix. */
int64_t mx_scales_mfma_bytes(int64_t rows, int64_t nblk);

/* Row-wise to_mx: x bf16 [rows, cols] (row stride ldx elements) ->
 * codes u8 [rows, cols] (dense) and scales for blocks of 32 along `cols`.
 * Requires cols % 32 == 0.  Stands in for the cast of the activation / weight along the
 * contraction dim that the converted F.linear performs
 * (torchtitan/components/quantization/mx.py:27-31,119-125; docs/mxfp8.md:35). */
int mx_cast_dim0(const void* x, int64_t rows, int64_t cols, int64_t ldx, uint8_t* codes,
                 uint8_t* scales, int scale_mode, int scale_order, void* stream);

/* Column-wise to_mx: x bf16 [rows, cols] -> codes u8 [cols, rows] (transposed, dense) and
 * scales [cols, rows/32] for blocks of 32 down the rows.  Requires rows % 32 == 0 and
 * cols % 2 == 0.  Equals mx_cast_dim0 of the transposed tensor.  Feeds dgrad / wgrad
 * operands (docs/mxfp8.md:61; torchtitan/models/common/moe/utils.py:47-52). */
int mx_cast_dim1(const void* x, int64_t rows, int64_t cols, int64_t ldx, uint8_t* codes_t,
                 uint8_t* scales_t, int scale_mode, int scale_order, void* stream);

/* Both casts from one read of x.  Requires rows % 32 == 0 and cols % 32 == 0. */
int mx_cast_dim0_dim1(const void* x, int64_t rows, int64_t cols, int64_t ldx, uint8_t* codes,
                      uint8_t* scales, uint8_t* codes_t, uint8_t* scales_t, int scale_mode,
                      int scale_order, void* stream);

/* mx_cast_dim0_dim1 with a row pitch for each code matrix: row r of the row-wise codes starts at
 * codes + r * ld_codes (ld_codes >= cols), row c of the column-wise codes at
 * codes_t + c * ld_codes_t (ld_codes_t >= rows); both multiples of 16, the bytes between the
 * rows are left alone.  Scales as ever.  Why: codes whose rows lie a multiple of 4 KB apart put
 * the lines a GEMM fetches together (one K block of many rows) on few channels of the L2; a
 * pitch of row length + 128 spreads them.  Inputs the tile kernel does not take (x not 16-byte
 * aligned, cols % 8, ldx % 8) return MX_ERR_UNSUPPORTED: the caller then casts densely.  Same
 * reference anchors as mx_cast_dim0 / mx_cast_dim1. */
int mx_cast_dim0_dim1_ld(const void* x, int64_t rows, int64_t cols, int64_t ldx, uint8_t* codes,
                         int64_t ld_codes, uint8_t* scales, uint8_t* codes_t, int64_t ld_codes_t,
                         uint8_t* scales_t, int scale_mode, int scale_order, void* stream);

/* Batched forms for 3-D expert weights x [batch, rows, cols] (dense, matrix stride rows*ldx):
 * every matrix is cast on its own; outputs are [batch, cols, rows] codes (and [batch, rows,
 * cols] for the fused form) with one scale block per matrix, each laid out as for the
 * unbatched call.  Same alignment rules; with batch > 1 also rows*cols % 16 == 0.
 * (3-D expert parameters: torchtitan/models/common/moe/moe.py:90-92.) */
int mx_cast_dim1_batched(const void* x, int64_t batch, int64_t rows, int64_t cols, int64_t ldx,
                         uint8_t* codes_t, uint8_t* scales_t, int scale_mode, int scale_order,
                         void* stream);
int mx_cast_dim0_dim1_batched(const void* x, int64_t batch, int64_t rows, int64_t cols,
                              int64_t ldx, uint8_t* codes, uint8_t* scales, uint8_t* codes_t,
                              uint8_t* scales_t, int scale_mode, int scale_order, void* stream);

/* Cast of gathered rows: output row r is row row_index[r] of x (bf16 [src_rows, cols], row
 * stride ldx); an index outside [0, src_rows) gives a row of zeros (the padding slots of an
 * aligned token-group layout hold -1).  With row_scale (float32 [rows], may be NULL) row r is
 * first multiplied by row_scale[r] in float32 and rounded to bf16: the routing-score multiply
 * `(routed_input.float() * top_scores).to(dtype)` of torchtitan/models/common/moe/moe.py:519-527.  Row-wise cast always; the column-wise cast too unless
 * codes_t and scales_t are both NULL (then `rows` need not be a multiple of 32).  Outputs as
 * mx_cast_dim0_dim1 for a [rows, cols] matrix.  Requires cols % 32 == 0, ldx % 8 == 0, x 16-byte
 * aligned.  Stands in for the token permutation `x[permuted_indices, :]` in front of the grouped
 * GEMMs (torchtitan/models/common/moe/utils.py:65-89) followed by the cast of its result. */
int mx_cast_rows_gathered(const void* x, const int64_t* row_index, const float* row_scale,
                          int64_t src_rows, int64_t rows, int64_t cols, int64_t ldx,
                          uint8_t* codes, uint8_t* scales, uint8_t* codes_t, uint8_t* scales_t,
                          int scale_mode, int scale_order, void* stream);

/* Routing plan of an MoE layer, one launch, no host round trip.  counts int32 [experts] (pairs
 * per expert), order int64 [pairs] (the (token, choice) pair = token * top_k + choice at every
 * position of the expert-sorted order: `token_indices_experts_sorted` of
 * torchtitan/models/common/moe/moe.py:355-362), scores float32 [pairs] by pair (may be NULL).
 * Every expert's group is padded to a multiple of `alignment` rows (at least one multiple, as in
 * moe/kernels.py:183-191).  Outputs: m_offsets int32 [experts] inclusive padded group ends;
 * src_row int64 [max_len] token of every padded row, -1 for padding and for rows behind the last
 * group; row_score float32 [max_len] that pair's score (0 for padding); pos int64 [pairs] padded
 * row of every pair (entries of pairs that no count covers are left untouched).
 * max_len >= sum of the padded sizes is the caller's static bound. */
int mx_moe_route_plan(const int32_t* counts, int64_t experts, const int64_t* order,
                      const float* scores, int64_t pairs, int64_t top_k, int64_t max_len,
                      int64_t alignment, int32_t* m_offsets, int64_t* src_row, float* row_score,
                      int64_t* pos, void* stream);

/* Combine of the routed expert outputs: out[t, :] = sum_j weights[t, j] * y[pos[t, j], :] for
 * j = 0 .. top_k-1 in that order, in float32 (product and sum rounded separately), result
 * rounded to bf16; weights == NULL gives the plain sum.  y: bf16 [y_rows, cols] (row stride
 * ldy), pos: int64 [tokens, top_k] rows of y (outside [0, y_rows): contributes nothing), out:
 * bf16 [tokens, cols] (row stride ldo).  cols % 8 == 0, 16-byte aligned rows.  With y2 (same
 * shape and stride as y, may be NULL) the rows summed are bf16(y + y2): the bf16 addition of two
 * partial gradients (dx from w1 and from w3) without a pass of its own.
 * Stands in for the un-sort scatter and the score-weighted sum over top_k of
 * torchtitan/models/common/moe/moe.py:535-555, and (with y = the gradient of the routed input)
 * for the backward of the token gather `x[token_indices // top_k]` (moe.py:519). */
int mx_moe_combine(const void* y, const void* y2, int64_t y_rows, int64_t ldy, const int64_t* pos,
                   const float* weights, int64_t tokens, int64_t top_k, int64_t cols, void* out,
                   int64_t ldo, void* stream);

/* Row dot products out[i] = sum_d a[ia[i], d] * b[ib[i], d] in float32 over bf16 matrices
 * a [a_rows, cols], b [b_rows, cols]; an index outside its matrix gives 0; with a2 (a's shape,
 * may be NULL) a's rows are bf16(a + a2).  The gradient of the
 * routing scores on either side of the experts (backward of moe.py:521-527 and :541-551). */
int mx_moe_row_dot(const void* a, const void* a2, int64_t a_rows, int64_t lda, const int64_t* ia, const void* b,
                   int64_t b_rows, int64_t ldb, const int64_t* ib, int64_t n, int64_t cols,
                   float* out, void* stream);

/* SwiGLU gate fused into the cast: g = silu(a) * b elementwise over bf16 [rows, cols] (row strides
 * lda, ldb), each step rounded to bf16 as the unfused tensor ops round it, then both casts of g
 * as mx_cast_dim0_dim1 produces them -- g itself never travels through HBM unless `g` is given
 * (bf16 [rows, cols] dense, may be NULL).  silu is a / (1 + exp(-a)) in float32 with a
 * correctly rounded quotient: its bf16 value equals the GPU tensor op's for every bf16 input.
 * Requires rows % 32 == 0, cols % 32 == 0, lda % 8 == 0, ldb % 8 == 0, 16-byte aligned inputs.
 * Stands in for the activation between the two halves of the feed-forward and the casts that
 * feed w2 (torchtitan/models/common/feed_forward.py:61-62; models/common/moe/moe.py:68-73). */
int mx_swiglu_cast_dim0_dim1(const void* a, const void* b, int64_t rows, int64_t cols,
                             int64_t lda, int64_t ldb, uint8_t* codes, uint8_t* scales,
                             uint8_t* codes_t, uint8_t* scales_t, void* g, int scale_mode,
                             int scale_order, void* stream);

/* RMSNorm fused in front of the casts: rstd[r] = 1 / sqrt(mean_c x[r, c]^2 + eps) (float32, also
 * an output: the norm's backward needs it), y[r, c] = bf16(weight[c] * (rstd[r] * x[r, c])) in
 * float32, then both casts of y as mx_cast_dim0_dim1 produces them.  x bf16 [rows, cols] (row
 * stride ldx), weight bf16 [cols], y bf16 [rows, cols] dense or NULL (then the normalised
 * activation never reaches memory).  rows % 32 == 0, cols % 32 == 0, ldx % 8 == 0, 16-byte aligned.
 * Stands in for the RMSNorm in front of wq / wk / wv and of w1 / w3
 * (torchtitan/models/common/rmsnorm.py:14-50) followed by the cast of its output. */
int mx_rmsnorm_cast_dim0_dim1(const void* x, const void* weight, float eps, int64_t rows,
                              int64_t cols, int64_t ldx, float* rstd, void* y, uint8_t* codes,
                              uint8_t* scales, uint8_t* codes_t, uint8_t* scales_t, int scale_mode,
                              int scale_order, void* stream);

/* Backward of that gate fused into the casts that feed the dgrad and wgrad GEMMs of w1 and w3:
 * from dg, a, b (bf16 [rows, cols], row strides lddg, lda, ldb) forms, as bf16 autograd does
 * tensor op by tensor op,
 *     da = silu_backward(bf16(dg * b), a),   db = bf16(dg * bf16(silu(a)))
 * and writes both casts of each.  Every output holds da's part followed by db's part:
 * codes [2, rows, cols], codes_t [2, cols, rows], scales and scales_t two buffers of the size a
 * single cast would use, back to back.  `dab` (bf16 [2, rows, cols], may be NULL) receives da and
 * db themselves.  Same shape and alignment rules as mx_swiglu_cast_dim0_dim1.
 * Stands in for the autograd nodes of feed_forward.py:61-62 (mul, silu) and the casts of their
 * results under the converted w1 / w3. */
int mx_swiglu_bwd_cast_dim0_dim1(const void* dg, const void* a, const void* b, int64_t rows,
                                 int64_t cols, int64_t lddg, int64_t lda, int64_t ldb,
                                 uint8_t* codes, uint8_t* scales, uint8_t* codes_t,
                                 uint8_t* scales_t, void* dab, int scale_mode, int scale_order,
                                 void* stream);

/* The three casts above with a row pitch for their codes, as mx_cast_dim0_dim1_ld has it:
 * rows of `codes` ld_codes bytes apart (>= cols), rows of `codes_t` ld_codes_t bytes apart
 * (>= rows), both multiples of 16 with 16-byte aligned buffers; 0 stands for dense rows.  The
 * two halves of the backward cast's outputs lie rows * ld_codes and cols * ld_codes_t bytes
 * apart.  Scales, every other argument and the results are those of the dense forms, which
 * forward here.  (The pitched operands of the fused SwiGLU block's GEMMs: see mx_gemm_nt_ld.) */
int mx_swiglu_cast_dim0_dim1_ld(const void* a, const void* b, int64_t rows, int64_t cols,
                                int64_t lda, int64_t ldb, uint8_t* codes, int64_t ld_codes,
                                uint8_t* scales, uint8_t* codes_t, int64_t ld_codes_t,
                                uint8_t* scales_t, void* g, int scale_mode, int scale_order,
                                void* stream);
int mx_rmsnorm_cast_dim0_dim1_ld(const void* x, const void* weight, float eps, int64_t rows,
                                 int64_t cols, int64_t ldx, float* rstd, void* y, uint8_t* codes,
                                 int64_t ld_codes, uint8_t* scales, uint8_t* codes_t,
                                 int64_t ld_codes_t, uint8_t* scales_t, int scale_mode,
                                 int scale_order, void* stream);
int mx_swiglu_bwd_cast_dim0_dim1_ld(const void* dg, const void* a, const void* b, int64_t rows,
                                    int64_t cols, int64_t lddg, int64_t lda, int64_t ldb,
                                    uint8_t* codes, int64_t ld_codes, uint8_t* scales,
                                    uint8_t* codes_t, int64_t ld_codes_t, uint8_t* scales_t,
                                    void* dab, int scale_mode, int scale_order, void* stream);

/* MXFP8 -> bf16: out[r, c] = e4m3(codes[r, c]) * 2^(scale of row r, block c / 32 - 127) rounded
 * to bf16 (exact above bf16's subnormal range); a scale byte 255 gives NaN.  codes uint8
 * [rows, cols] dense (16-byte aligned, cols % 32 == 0), scales in either order, out bf16
 * [rows, cols] with row stride ldo (% 8).  The receiving side of a weight hand-over in MXFP8
 * form (in place of the bf16 state dict of
 * torchtitan/experiments/rl/unified/actors/trainer.py:226-239 -> generator.py:307-335). */
int mx_dequant(const uint8_t* codes, const uint8_t* scales, int64_t rows, int64_t cols,
               int scale_order, void* out, int64_t ldo, void* stream);

/* Log-probabilities of chosen tokens: logprob[r] = x[r, target[r]] - lse[r],
 * lse[r] = log sum_v exp(x[r, v]) in float32 over bf16 logits x [rows, vocab] (row stride ld,
 * ld % 8 == 0, 16-byte aligned); target int64 [rows] (outside [0, vocab): NaN).  One read of
 * the logits.  Stands in for `.to(float32)`, `F.log_softmax` and `gather` on the policy's
 * logits (torchtitan/experiments/rl/unified/actors/utils.py:37-50). */
int mx_token_logprob_fwd(const void* logits, int64_t rows, int64_t vocab, int64_t ld,
                         const int64_t* target, float* logprob, float* lse, void* stream);
/* Its backward: dlogits[r, v] = grad_logprob[r] * ((v == target[r]) - exp(x[r, v] - lse[r]))
 * rounded to bf16 (dlogits bf16 [rows, vocab], row stride ldd); rows <= 65535 per call. */
int mx_token_logprob_bwd(const void* logits, int64_t rows, int64_t vocab, int64_t ld,
                         const int64_t* target, const float* lse, const float* grad_logprob,
                         void* dlogits, int64_t ldd, void* stream);

/* Re-order a row-major [rows, nblk] scale matrix into MX_SCALES_MFMA order
 * (the "blocked layout" step the reference leaves to torch._scaled_mm, docs/mxfp8.md:36). */
int mx_scale_layout(const uint8_t* scales, int64_t rows, int64_t nblk, uint8_t* out, void* stream);
/* Inverse permutation. */
int mx_scale_unlayout(const uint8_t* laid, int64_t rows, int64_t nblk, uint8_t* out, void* stream);

/* D[M,N] (bf16, row stride ldd) = deq(A)[M,K] * deq(B)[N,K]^T, fp32 accumulate.
 * a_codes [M,K], b_codes [N,K] row-major dense; a_scales / b_scales in MX_SCALES_MFMA order
 * for [M, K/32] and [N, K/32].  Requires K % 32 == 0.  One primitive serves forward
 * (X along K, W along K), dgrad (dY along N, W^T along N) and wgrad (dY^T along M, X^T along
 * M) -- the F.linear on a converted weight and its autograd
 * (torchtitan/components/quantization/mx.py:27-31; torchtitan/models/common/feed_forward.py:61-62). */
int mx_gemm_nt(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
               const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K, int64_t ldd,
               void* stream);

/* The same GEMM for a caller that can lend scratch memory: shapes with few 256x256 output
 * tiles and a long contraction (the wgrad of a small weight over many tokens,
 * dW[N,K] = dY^T X with M in the tens of thousands) are then split along the contraction over
 * several workgroups per tile, float32 partial sums in `workspace`, one reduction pass.
 * mx_gemm_nt_workspace_bytes: bytes with which the shape would be split on the current device
 * (0: mx_gemm_nt_ws runs exactly what mx_gemm_nt runs).  workspace: device memory, 16-byte
 * aligned, contents undefined before and after; with less than the stated size (or NULL) the
 * call falls back to mx_gemm_nt.  Results differ from mx_gemm_nt's only by the order of the
 * float32 summation.  Same reference anchor as mx_gemm_nt. */
int64_t mx_gemm_nt_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mx_gemm_nt_ws(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                  const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K, int64_t ldd,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* mx_gemm_nt / mx_gemm_nt_ws for operands whose rows lie `ldk` >= K bytes apart (a multiple of 16;
 * of 128 for the persistent kernel), e.g. the codes mx_cast_dim0_dim1_ld writes.  workspace may be
 * NULL (then as mx_gemm_nt).  Same reference anchor as mx_gemm_nt. */
int mx_gemm_nt_ld(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                  const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K, int64_t ldk,
                  int64_t ldd, void* workspace, int64_t workspace_bytes, void* stream);

/* mx_gemm_nt_ws for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * float32 partial sums of the split live in a device array built into the library
 * (mx_gemm_nt_static_max_bytes() = 64 MiB, held on every GPU the library runs on until the process
 * ends) instead of a caller's workspace; the call allocates nothing, on the host or the device.
 * Runs the kernels mx_gemm_nt_ws runs with a workspace of mx_gemm_nt_workspace_bytes(M, N, K), so
 * the results are bit-identical to that call's; shapes that are not split run what mx_gemm_nt
 * runs.  A shape whose split needs more than the array holds returns MX_ERR_SCRATCH_TOO_SMALL and
 * launches nothing (to know beforehand: mx_gemm_nt_workspace_bytes(M, N, K) against
 * mx_gemm_nt_static_max_bytes(); such a shape runs through mx_gemm_nt unsplit, or through
 * mx_gemm_nt_ws with memory of the caller's).  The first call on a GPU looks up that GPU's copy
 * of the array and raises the kernel's LDS limit, neither of which belongs into a graph capture:
 * make one call per GPU (any shape) before capturing.  All calls on one GPU share that GPU's array: calls that overlap in time on
 * the same GPU (two streams, two threads) race on it.  Nothing in the array needs clearing between
 * calls: every partial tile is written in full before the reduction reads it. */
int64_t mx_gemm_nt_static_max_bytes(void);
int mx_gemm_nt_static(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                      const uint8_t* b_scales, void* d, int64_t M, int64_t N, int64_t K,
                      int64_t ldd, void* stream);

/* D = deq(A) deq(B)^T + deq(A2) deq(B2)^T in one pass, both operand sets of the shapes of
 * mx_gemm_nt: every output tile accumulates the products of the first set and then of the second
 * before it is rounded once to bf16 and written.  The input gradient of a SwiGLU block,
 * dx = d(h1) W1 + d(h3) W3 (autograd of torchtitan/models/common/feed_forward.py:61-62), as one
 * GEMM instead of two and a bf16 add.  Shapes the persistent kernel does not take (M or N <= 128,
 * K % 128, N % 8, ldd % 8, D not 16-byte aligned) return MX_ERR_UNSUPPORTED: the caller then
 * runs two mx_gemm_nt calls and adds. */
int mx_gemm_nt_pair(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                    const uint8_t* b_scales, const uint8_t* a2_codes, const uint8_t* a2_scales,
                    const uint8_t* b2_codes, const uint8_t* b2_scales, void* d, int64_t M,
                    int64_t N, int64_t K, int64_t ldd, void* stream);

/* Two products that share an operand, in one launch of the persistent kernel: the output tiles
 * of the second product are numbered behind those of the first, so the panels of the shared
 * operand are fetched once for both, and the launch's fixed cost is paid once.
 *   mx_gemm_nt_shared_a:  D = deq(A) deq(B)^T  and  D2 = deq(A) deq(B2)^T   (B, B2 [N,K]; D, D2 [M,N])
 *     h1 = x W1^T and h3 = x W3^T of a SwiGLU block (torchtitan/models/common/feed_forward.py:61-62)
 *   mx_gemm_nt_shared_b:  D = deq(A) deq(B)^T  and  D2 = deq(A2) deq(B)^T   (A, A2 [M,K])
 *     the weight gradients dW1 = d(h1)^T x and dW3 = d(h3)^T x of the same block (its autograd)
 * Every tile is computed exactly as by mx_gemm_nt: results are bit-identical to two calls.
 * Both outputs share ldd.  Shapes the persistent kernel does not take (as for mx_gemm_nt_pair)
 * return MX_ERR_UNSUPPORTED: the caller then runs two mx_gemm_nt calls. */
int mx_gemm_nt_shared_a(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                        const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                        void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldd,
                        void* stream);
int mx_gemm_nt_shared_b(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* a2_codes,
                        const uint8_t* a2_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                        void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldd,
                        void* stream);

/* mx_gemm_nt_pair / _shared_a / _shared_b on operands whose rows lie ldk bytes apart (every code
 * matrix of the call with the same pitch, ldk >= K and a multiple of 128, as for mx_gemm_nt_ld);
 * the dense forms forward here with ldk = K.  Same results. */
int mx_gemm_nt_pair_ld(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                       const uint8_t* b_scales, const uint8_t* a2_codes, const uint8_t* a2_scales,
                       const uint8_t* b2_codes, const uint8_t* b2_scales, void* d, int64_t M,
                       int64_t N, int64_t K, int64_t ldk, int64_t ldd, void* stream);
int mx_gemm_nt_shared_a_ld(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                           const uint8_t* b_scales, const uint8_t* b2_codes, const uint8_t* b2_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk,
                           int64_t ldd, void* stream);
int mx_gemm_nt_shared_b_ld(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* a2_codes,
                           const uint8_t* a2_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                           void* d, void* d2, int64_t M, int64_t N, int64_t K, int64_t ldk,
                           int64_t ldd, void* stream);

/* Grouped GEMM, 2D x 3D: for group g with rows [offs[g-1], offs[g]) of A:
 * D[rows, :] = deq(A[rows, :]) * deq(B[g])^T.  a_codes [T,K]; b_codes [G,N,K];
 * b_scales G consecutive MFMA-order blocks, each for [N, K/32].
 * offs int32 [G] inclusive cumulative sizes on the device; rows >= offs[G-1] are written as
 * zeros.  a_scale_order says how a_scales is laid out:
 *   MX_SCALES_ROWMAJOR  [T, K/32]; groups may end anywhere (tile kernel);
 *   MX_SCALES_MFMA      MFMA order over the whole [T, K/32] matrix; every group must end at a
 *                       multiple of 32 rows (the alignment of the reference's padded token
 *                       groups, torchtitan/components/quantization/__init__.py:36),
 *                       T % 32 == 0, K % 128 == 0, N % 8 == 0, G <= 510: the
 *                       persistent kernel (several times faster).  The group ends live on the
 *                       device, so they are checked there: a violation fills D with NaN.
 * Stands in for torch._grouped_mm(x, w^T, offs) in forward and dgrad
 * (torchtitan/models/common/moe/moe.py:59-76). */
int mx_grouped_gemm_2d3d(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                         const uint8_t* b_scales, const int32_t* offs, void* d, int64_t T,
                         int64_t N, int64_t K, int64_t G, int64_t ldd, int a_scale_order,
                         void* stream);

/* The grouped 2D x 3D GEMM over two operand sets of the same shapes, summed per output tile as
 * in mx_gemm_nt_pair: the expert block's input gradient d(h1) W1[g] + d(h3) W3[g]
 * (autograd of torchtitan/models/common/moe/moe.py:59-76) as one grouped GEMM.  MFMA-order
 * scales and the contract of the MX_SCALES_MFMA form above only. */
int mx_grouped_gemm_2d3d_pair(const uint8_t* a_codes, const uint8_t* a_scales,
                              const uint8_t* b_codes, const uint8_t* b_scales,
                              const uint8_t* a2_codes, const uint8_t* a2_scales,
                              const uint8_t* b2_codes, const uint8_t* b2_scales,
                              const int32_t* offs, void* d, int64_t T, int64_t N, int64_t K,
                              int64_t G, int64_t ldd, void* stream);

/* The grouped 2D x 3D GEMM (one product, or with a2_codes .. b2_scales non-null the sum of two as
 * mx_grouped_gemm_2d3d_pair) over operands whose groups are padded to multiples of 32 rows, with
 * the padding left out of the output: the first out_offs[g] - out_offs[g-1] rows of group g are
 * written to rows [out_offs[g-1], out_offs[g]) of d [out_rows, ldd] (out_offs: int32 [G]
 * inclusive ends, on the device); rows from out_offs[G-1] on are written as zeros as far as A
 * has rows behind its last group (out_rows - out_offs[G-1] <= T - offs[G-1] is the caller's
 * side of the contract; whatever the arrays hold, no row outside d is written).  Takes the
 * place of the grouped GEMM followed by the gather that moves the rows back
 * (`_unpermute`, torchtitan/models/common/moe/utils.py:85-89, called at :116).  MFMA-order scales
 * and the contract of the MX_SCALES_MFMA form of mx_grouped_gemm_2d3d only; out_rows <= T. */
int mx_grouped_gemm_2d3d_rows_out(const uint8_t* a_codes, const uint8_t* a_scales,
                                  const uint8_t* b_codes, const uint8_t* b_scales,
                                  const uint8_t* a2_codes, const uint8_t* a2_scales,
                                  const uint8_t* b2_codes, const uint8_t* b2_scales,
                                  const int32_t* offs, const int32_t* out_offs, void* d, int64_t T,
                                  int64_t out_rows, int64_t N, int64_t K, int64_t G, int64_t ldd,
                                  void* stream);

/* Grouped GEMM, 2D x 2D (wgrad): D[g][N,K] = deq(A^T[:, rows_g]) * deq(B^T[:, rows_g])^T,
 * contracting over the tokens of group g.  at_codes [N,T] and bt_codes [K,T] are the
 * column-wise casts; scale_order says how both scale buffers are laid out:
 *   MX_SCALES_ROWMAJOR  [N, T/32] and [K, T/32]; every group size a multiple of 32
 *                       (torchtitan/models/common/moe/utils.py:47-52);
 *   MX_SCALES_MFMA      MFMA order; every group must end at a multiple of 32 tokens,
 *                       T % 128 == 0, K % 8 == 0: the persistent kernel; checked on the
 *                       device, a violation fills D with NaN.
 * Empty groups give zeros.  d is [G,N,K] bf16 dense. */
int mx_grouped_gemm_2d2d(const uint8_t* at_codes, const uint8_t* at_scales,
                         const uint8_t* bt_codes, const uint8_t* bt_scales, const int32_t* offs,
                         void* d, int64_t T, int64_t N, int64_t K, int64_t G, int scale_order,
                         void* stream);

/* The grouped forms of mx_gemm_nt_shared_a / _shared_b, MFMA-order scales and the contracts of
 * the MX_SCALES_MFMA forms above only:
 *   mx_grouped_gemm_2d3d_shared_a:  D = A x B[g]^T and D2 = A x B2[g]^T per group -- the experts'
 *     h1 and h3 from one pass over the routed tokens (torchtitan/models/common/moe/moe.py:68-73)
 *   mx_grouped_gemm_2d2d_shared_b:  D[g] = A^T B^T' and D2[g] = A2^T B^T' over the tokens of group g
 *     -- dW1 and dW3 of the experts from one pass over the column-wise form of the routed tokens
 * Bit-identical to two calls of the plain forms. */
int mx_grouped_gemm_2d3d_shared_a(const uint8_t* a_codes, const uint8_t* a_scales,
                                  const uint8_t* b_codes, const uint8_t* b_scales,
                                  const uint8_t* b2_codes, const uint8_t* b2_scales,
                                  const int32_t* offs, void* d, void* d2, int64_t T, int64_t N,
                                  int64_t K, int64_t G, int64_t ldd, void* stream);
int mx_grouped_gemm_2d2d_shared_b(const uint8_t* at_codes, const uint8_t* at_scales,
                                  const uint8_t* at2_codes, const uint8_t* at2_scales,
                                  const uint8_t* bt_codes, const uint8_t* bt_scales,
                                  const int32_t* offs, void* d, void* d2, int64_t T, int64_t N,
                                  int64_t K, int64_t G, void* stream);

/* Token-group padding: from per-(rank, expert) counts build
 *   m_sizes[e]   = round_up(max(sum_r counts[r*E+e], alignment), alignment)   int32 [E]
 *   m_offsets    = inclusive cumsum(m_sizes)                                  int32 [E]
 *   perm[max_len]: perm[write_off[e] + j] = start[r*E+e] + j, -1 in padding   int64
 * One launch, no host synchronisation.  Stands in for generate_permute_indices and its
 * Triton fill kernel (torchtitan/models/common/moe/kernels.py:16-63,145-218).
 * Requires experts_per_rank * num_ranks <= 4096. */
int mx_group_offsets_pad(const int32_t* counts, int64_t experts_per_rank, int64_t num_ranks,
                         int64_t max_len, int64_t alignment, int64_t* perm, int32_t* m_sizes,
                         int32_t* m_offsets, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MXFP8_H_ */
