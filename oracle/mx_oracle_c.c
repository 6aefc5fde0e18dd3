/*
 * CPU restatement (plain C) of the to_mx casts of the MXFP8 linear path.  TEST INFRASTRUCTURE
 * ONLY: built by oracle/Makefile into oracle/libmx_oracle.so and loaded by tests and by the
 * benchmark's CPU-baseline leg; the product never calls it.
 *
 * A second, independent statement of the same definition as oracle/mx_oracle.py (OCP MX v1.0
 * block format; reference call site torchtitan/components/quantization/mx.py:100-125, block
 * size torchtitan/components/quantization/__init__.py:36): the narrowing here is done by
 * value comparison against the table of e4m3 magnitudes rather than by bit manipulation, so
 * a slip in either one shows up as a disagreement between the two.
 *
 * Pinned / unpinned corners: see the header of oracle/mx_oracle.py.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define MX_BLOCK 32

static float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* magnitude table of the 127 finite e4m3fn codes 0x00..0x7E */
static double e4m3_mag(int code) {
  int e = (code >> 3) & 0xF, m = code & 7;
  return e == 0 ? m * ldexp(1.0, -9) : (1.0 + m / 8.0) * ldexp(1.0, e - 7);
}

/* saturating round-to-nearest-even onto the e4m3 grid, by search over the value table */
static uint8_t e4m3_from_double(double y, int negative) {
  uint8_t sign = negative ? 0x80 : 0;
  if (isnan(y)) return 0x7F | sign;
  double a = fabs(y);
  if (a >= 448.0) return 0x7E | sign;
  int lo = 0, hi = 0x7E; /* largest code with magnitude <= a */
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (e4m3_mag(mid) <= a) lo = mid; else hi = mid - 1;
  }
  if (lo == 0x7E) return 0x7E | sign;
  double below = e4m3_mag(lo), above = e4m3_mag(lo + 1);
  double dl = a - below, du = above - a;
  int code = dl < du ? lo : (dl > du ? lo + 1 : ((lo & 1) ? lo + 1 : lo));
  return (uint8_t)code | sign;
}

static int scale_byte(uint16_t amax_bits, int mode) {
  if (amax_bits > 0x7F80) return 255;
  if (amax_bits == 0) return 0;
  int expf = amax_bits >> 7, man = amax_bits & 0x7F;
  int s = expf - 127 - 8 + ((mode == 1 && man > 0x60) ? 1 : 0);
  if (s < -127) s = -127;
  if (s > 127) s = 127;
  return s + 127;
}

/* one block of 32 values with element stride `stride` -> 32 codes (stride 1) + scale byte */
static void cast_block(const uint16_t* x, int64_t stride, int mode, uint8_t* codes, uint8_t* scale) {
  uint16_t amax = 0;
  for (int k = 0; k < MX_BLOCK; ++k) {
    uint16_t a = x[k * stride] & 0x7FFF;
    if (a > amax) amax = a;
  }
  int sb = scale_byte(amax, mode);
  *scale = (uint8_t)sb;
  for (int k = 0; k < MX_BLOCK; ++k) {
    uint16_t b = x[k * stride];
    int neg = b >> 15;
    if (sb == 255) {
      codes[k] = (uint8_t)(((b & 0x7FFF) > 0x7F80 ? 0x7F : 0) | (neg ? 0x80 : 0));
      continue;
    }
    double v = (double)bf16_to_f32(b);
    double y;
    if (sb == 0) y = (mode == 0) ? ldexp(v, 126) : v;
    else y = ldexp(v, 127 - sb);
    /* float32 evaluation of the product: flush what float32 cannot hold exactly is not
       needed, a power-of-two factor is exact unless the result is below the e4m3 grid */
    codes[k] = e4m3_from_double(y, neg);
  }
}

/* x bf16 [rows, cols] row-major -> codes [rows, cols], scales [rows, cols/32] */
void mxo_cast_dim0(const uint16_t* x, int64_t rows, int64_t cols, int mode, uint8_t* codes, uint8_t* scales) {
  int64_t nblk = cols / MX_BLOCK;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t b = 0; b < nblk; ++b)
      cast_block(x + r * cols + b * MX_BLOCK, 1, mode, codes + r * cols + b * MX_BLOCK, scales + r * nblk + b);
}

/* x bf16 [rows, cols] -> codes [cols, rows], scales [cols, rows/32] (blocks down the rows) */
void mxo_cast_dim1(const uint16_t* x, int64_t rows, int64_t cols, int mode, uint8_t* codes_t, uint8_t* scales_t) {
  int64_t nblk = rows / MX_BLOCK;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < cols; ++c)
    for (int64_t b = 0; b < nblk; ++b)
      cast_block(x + b * MX_BLOCK * cols + c, cols, mode, codes_t + c * rows + b * MX_BLOCK, scales_t + c * nblk + b);
}

/* float32 value of every element: code value * 2^(scale-127), blocks along the last dim */
void mxo_dequant(const uint8_t* codes, const uint8_t* scales, int64_t rows, int64_t cols, float* out) {
  int64_t nblk = cols / MX_BLOCK;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t b = 0; b < nblk; ++b) {
      int sb = scales[r * nblk + b];
      for (int k = 0; k < MX_BLOCK; ++k) {
        uint8_t c = codes[r * cols + b * MX_BLOCK + k];
        double v = ((c & 0x7F) == 0x7F || sb == 255) ? NAN : ldexp(e4m3_mag(c & 0x7F), sb - 127);
        out[r * cols + b * MX_BLOCK + k] = (float)((c & 0x80) ? -v : v);
      }
    }
}
