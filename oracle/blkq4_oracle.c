/*
 * CPU oracle for the blockwise-4-bit weight quantizer, its prepacked layouts and the
 * dequantize-then-GEMM result.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is a scalar restatement of the reference algorithm used only to
 * check the HIP kernels (tests, the smoke check and the CPU-baseline leg of the benchmark).  No
 * product code path may call it.
 *
 * Every function names the reference lines it restates (paths relative to the reference tree).
 *
 * Conventions (reference: test/blkq4_fp16_gemm_sm80.h:24-36):
 *   W is the logical [K, N] weight matrix, K = rows = in_features, N = columns = out_features.
 *   The fp16 source holds element (k, n) at src[k + n * ld]  (torch weight[n][k], ld = in_features).
 *   Column-wise blocking: a block is [bs, 1] (bs consecutive k of one n); meta shape [K/bs, N].
 *   Row-wise blocking:    a block is [1, bs] (bs consecutive n of one k); meta shape [K, N/bs].
 *
 * Pinning status of each function:
 *   oracle_quantize          pinned by the reference's round-trip known-answer construction
 *                            (test/blkq4_fp16_quant_sm80_test.cu:53-186) and closed-form edge cases.
 *                            One detail is PARITY UNPINNED: whether `v * reciprocal_scale + zp`
 *                            (src/mickey/blk_q4/f16_quant_sm80.cuh:296,307) was contracted to an FMA
 *                            by nvcc in a shipped binary.  Source plus nvcc's default (-fmad=true)
 *                            say yes, so `fused != 0` is the default everywhere; the reference's own
 *                            vectors are insensitive to the choice.
 *   oracle_prepack_*_sm80    pinned by the host reference prepack functions
 *                            (test/blkq4_fp16_gemm_sm80.h:39-226) and the digests of the reference's
 *                            known-answer vectors held in tests/golden/.
 *   oracle_dequantize        pinned by test/blkq4_fp16_gemm_sm80_test.cu:309-328 (exact on the
 *                            known-answer data, so any mistake in indexing shows as a mismatch).
 *   bf16 (`bf16 != 0` in the `_t` variants): the reference has no bf16 path and no vectors for one
 *                            (src/blkq4_f16_gemm_sm80.cu:53 rejects the type), so these are the fp16
 *                            functions with the 16-bit conversions exchanged.  The conversions are
 *                            pinned exhaustively (all 65536 patterns up, round trip, and the rounding
 *                            of every float between neighbouring bf16 values against numpy arithmetic);
 *                            the quantizer by the same round-trip construction as fp16 on data exact
 *                            in bf16; dequantize and GEMM against float64 numpy.
 *   oracle_gemm              textbook fp32-accumulate GEMM with one round-to-nearest fp16 conversion
 *                            (test/blkq4_fp16_gemm_sm80_test.cu:54-107,445-459); checked against a
 *                            float64 numpy matmul.
 */

#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------------------------------------
 * IEEE binary16 <-> binary32, software, round-to-nearest-even (what CUDA's half(float) and
 * cutlass::half_t(float) do).
 * ------------------------------------------------------------------------------------------- */

static inline float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline uint16_t f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
  }
  if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* below half of the smallest subnormal (2^-25) -> zero */
    return sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;
  uint32_t base;
  if (e < -14) { /* subnormal result: value = man * 2^(e-23); unit = 2^-24 */
    shift = -e - 1; /* 13 + (-14 - e) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  uint32_t r = base + q; /* mantissa carry propagates into the exponent correctly */
  if (rem > half || (rem == half && (r & 1u))) {
    ++r;
  }
  return (uint16_t)(sign | r);
}

ORACLE_API float oracle_h2f(uint16_t h) { return h2f(h); }
ORACLE_API uint16_t oracle_f2h(float f) { return f2h(f); }

/* bfloat16 (the upper half of a binary32) <-> binary32, round-to-nearest-even.  The `_t` variants of the
 * functions below take `bf16 != 0` to run the same algorithm on that 16-bit type instead of binary16. */
static inline float b2f(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline uint16_t f2b(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u); /* quiet NaN */
  x += 0x7fffu + ((x >> 16) & 1u); /* ties to even; a carry out of the mantissa rounds up to the next exponent / inf */
  return (uint16_t)(x >> 16);
}

ORACLE_API float oracle_b2f(uint16_t b) { return b2f(b); }
ORACLE_API uint16_t oracle_f2b(float f) { return f2b(f); }

static inline float e2f(uint16_t v, int bf16) { return bf16 ? b2f(v) : h2f(v); }
static inline uint16_t f2e(float f, int bf16) { return bf16 ? f2b(f) : f2h(f); }

/* ---------------------------------------------------------------------------------------------
 * Size query.  Reference: src/blkq4_f16_gemm_sm80.cu:155-203 (blkq4_quant_size_sm80_T) and
 * src/mickey/blk_q4/f16_quant_sm80.cuh:191-198.
 * Returns 0 and the two element counts, or a negative code:
 *   -1 empty, -2 bad block size, -3 rows not quantizable, -4 columns not quantizable.
 * ------------------------------------------------------------------------------------------- */
ORACLE_API int oracle_quant_size(int block_size, int column_wise, int rows, int columns,
                                 int64_t* quant_weights_size, int64_t* quant_meta_size) {
  *quant_weights_size = 0;
  *quant_meta_size = 0;
  if (block_size != 16 && block_size != 32 && block_size != 64) return -2;
  if (rows == 0 || columns == 0) return -1;
  const int krow = column_wise ? block_size : 1;
  const int kcol = column_wise ? 1 : block_size;
  const int64_t meta_rows = rows / krow;
  const int64_t meta_cols = columns / kcol;
  if ((rows % 64) != 0 || meta_rows == 0 || (rows % meta_rows) != 0) return -3;
  if ((columns % 32) != 0 || meta_cols == 0 || (columns % meta_cols) != 0) return -4;
  *quant_weights_size = (int64_t)(rows / 2) * columns;
  *quant_meta_size = meta_rows * meta_cols;
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Quantizer arithmetic.  Reference: src/mickey/blk_q4/f16_quant_sm80.cuh
 *   range2scalezp :96-122, range2scale :124-135, clamp :137-141, dev_quantize_blk :225-315.
 * ------------------------------------------------------------------------------------------- */

/* :96-122 -- asymmetric: rectify the range to include 0, scale in fp32, zero-point from the
 * unrounded fp32 scale, roundf (half away from zero), then the scale is rounded to fp16. */
static void range2scalezp(float mn, float mx, uint16_t* scale, uint8_t* zp, int bf16) {
  mn = fminf(mn, 0.0f);
  mx = fmaxf(mx, 0.0f);
  volatile float scale_f = (mx - mn) / 15.0f; /* volatile: forbid excess precision / reassociation */
  float zero_point_fp = mn;
  if (scale_f != 0.0f) {
    volatile float t = mn / scale_f;
    zero_point_fp = 0.f - t;
  }
  if (zero_point_fp < 0.0f) {
    *zp = 0;
  } else if (zero_point_fp > 15.0f) {
    *zp = 15;
  } else {
    *zp = (uint8_t)roundf(zero_point_fp);
  }
  *scale = f2e(scale_f, bf16);
}

/* :124-135 -- symmetric: the extreme value (ties go to min) divided by -8. */
static void range2scale(float mn, float mx, uint16_t* scale, int bf16) {
  float m = fabsf(mx) > fabsf(mn) ? mx : mn;
  *scale = f2e(m / -8.0f, bf16);
}

/* :286-313 -- one element. */
static inline uint8_t quantize_one(float v, float reciprocal_scale, uint8_t zp, int fused) {
  float t;
  if (fused) {
    t = fmaf(v, reciprocal_scale, (float)zp);
  } else {
    volatile float p = v * reciprocal_scale;
    t = p + (float)zp;
  }
  float r = roundf(t);
  r = fmaxf(0.0f, fminf(15.0f, r));
  return (uint8_t)r;
}

/*
 * Canonical quantized form ("output of block_quantize", :317-332):
 *   weights  uint8[K/2, N] column-major: byte n*(K/2) + k/2 = q(k,n) | q(k+1,n) << 4  (:312)
 *   scales   fp16 column-major [K/kRow, N/kCol]: index meta_col*(K/kRow) + meta_row    (:277,290)
 *   zps      uint8, same indexing; NULL selects the symmetric quantizer (implicit zp 8, :292)
 */
ORACLE_API int oracle_quantize_t(int block_size, int column_wise, int rows, int columns, int ld,
                                 const uint16_t* src, uint8_t* canon_w, uint16_t* canon_scales,
                                 uint8_t* canon_zps, int fused, int bf16) {
  int64_t wsz, msz;
  int err = oracle_quant_size(block_size, column_wise, rows, columns, &wsz, &msz);
  if (err) return err;
  const int krow = column_wise ? block_size : 1;
  const int kcol = column_wise ? 1 : block_size;
  const int meta_rows = rows / krow;
  const int meta_cols = columns / kcol;

  /* pass 1: range -> scale (and zero-point) per block (:261-284) */
#pragma omp parallel for schedule(static)
  for (int mc = 0; mc < meta_cols; ++mc) {
    for (int mr = 0; mr < meta_rows; ++mr) {
      float mn = FLT_MAX;
      float mx = -FLT_MAX;
      for (int i = mr * krow; i < (mr + 1) * krow; ++i) {
        for (int j = mc * kcol; j < (mc + 1) * kcol; ++j) {
          const float v = e2f(src[(size_t)i + (size_t)j * ld], bf16);
          if (v < mn) mn = v;
          if (v > mx) mx = v;
        }
      }
      const size_t meta_idx = (size_t)mc * meta_rows + mr;
      if (canon_zps == NULL) {
        range2scale(mn, mx, &canon_scales[meta_idx], bf16);
      } else {
        range2scalezp(mn, mx, &canon_scales[meta_idx], &canon_zps[meta_idx], bf16);
      }
    }
  }

  /* pass 2: quantize with the fp16-rounded scale read back (:286-313) */
#pragma omp parallel for schedule(static)
  for (int j = 0; j < columns; ++j) {
    const int meta_c = j / kcol;
    for (int i = 0; i < rows; i += 2) {
      uint8_t q[2];
      for (int t = 0; t < 2; ++t) {
        const int meta_r = (i + t) / krow;
        const size_t meta_idx = (size_t)meta_c * meta_rows + meta_r;
        const float scale = e2f(canon_scales[meta_idx], bf16);
        const uint8_t zp = canon_zps ? canon_zps[meta_idx] : 8;
        volatile float reciprocal_scale = scale ? 1.0f / scale : 0.0f;
        const float v = e2f(src[(size_t)(i + t) + (size_t)j * ld], bf16);
        q[t] = quantize_one(v, reciprocal_scale, zp, fused);
      }
      canon_w[(size_t)j * (rows / 2) + i / 2] = (uint8_t)((q[0] & 0xf) | (q[1] << 4));
    }
  }
  return 0;
}

ORACLE_API int oracle_quantize(int block_size, int column_wise, int rows, int columns, int ld,
                               const uint16_t* src, uint8_t* canon_w, uint16_t* canon_scales,
                               uint8_t* canon_zps, int fused) {
  return oracle_quantize_t(block_size, column_wise, rows, columns, ld, src, canon_w, canon_scales, canon_zps, fused, 0);
}

/* ---------------------------------------------------------------------------------------------
 * sm80 prepacked weight layout.  Reference: f16_quant_sm80.cuh:362-417 and the host restatement
 * test/blkq4_fp16_gemm_sm80.h:39-86.  In: canonical uint8[K/2, N] col-major.  Out: uint8[K, N/2]
 * col-major (byte pc*K + pr), same byte count.
 * ------------------------------------------------------------------------------------------- */
ORACLE_API int oracle_prepack_weights_sm80(int rows, int columns, const uint8_t* canon_w,
                                           uint8_t* packed_w) {
  if ((rows % 16) != 0 || (columns % 16) != 0) return -1;
  const size_t ld_in = (size_t)rows / 2; /* canonical column stride */
  const size_t ld_out = (size_t)rows;    /* packed column stride */
  for (int col_dtile = 0; col_dtile < columns / 16; ++col_dtile) {
    for (int row_dtile = 0; row_dtile < rows / 16; ++row_dtile) {
      /* an 8x16 byte tile (16x16 weights) becomes a 16x8 byte tile */
      const size_t in_r = (size_t)row_dtile * 8, in_c = (size_t)col_dtile * 16;
      const size_t out_r = (size_t)row_dtile * 16, out_c = (size_t)col_dtile * 8;
      for (int col = 0; col < 8; ++col) {
        for (int row = 0; row < 4; ++row) {
          const uint8_t b0 = canon_w[(in_c + col) * ld_in + in_r + row];         /* t0 (0,0) */
          const uint8_t b1 = canon_w[(in_c + col) * ld_in + in_r + row + 4];     /* t1 (4,0) */
          const uint8_t b2 = canon_w[(in_c + col + 8) * ld_in + in_r + row];     /* t2 (0,8) */
          const uint8_t b3 = canon_w[(in_c + col + 8) * ld_in + in_r + row + 4]; /* t3 (4,8) */
          uint8_t* o = &packed_w[(out_c + col) * ld_out + out_r + (size_t)row * 4];
          o[0] = (uint8_t)((b0 & 0x0f) | ((b1 & 0x0f) << 4));
          o[1] = (uint8_t)((b2 & 0x0f) | ((b3 & 0x0f) << 4));
          o[2] = (uint8_t)(((b0 & 0xf0) >> 4) | (b1 & 0xf0));
          o[3] = (uint8_t)(((b2 & 0xf0) >> 4) | (b3 & 0xf0));
        }
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * sm80 prepacked meta layout.  Reference: f16_quant_sm80.cuh:457-547 and
 * test/blkq4_fp16_gemm_sm80.h:88-226.
 *   column-wise blocking: canonical col-major [K/bs, N]  ->  row-major [K/bs, N] (a transpose)
 *   row-wise blocking   : stays col-major [K, N/bs]; each 16-row group of a column is permuted,
 *                         scales dst[4t+{0,1,2,3}] = src[2t+{0,1,8,9}],
 *                         zps    dst[4t+{0,1,2,3}] = src[2t+{0,8,1,9}].
 * canon_zps / packed_zps may be NULL.
 * ------------------------------------------------------------------------------------------- */
ORACLE_API int oracle_prepack_meta_sm80(int block_size, int column_wise, int rows, int columns,
                                        const uint16_t* canon_scales, const uint8_t* canon_zps,
                                        uint16_t* packed_scales, uint8_t* packed_zps) {
  if ((rows % 16) != 0 || (columns % 16) != 0) return -1;
  const int krow = column_wise ? block_size : 1;
  const int kcol = column_wise ? 1 : block_size;
  const int meta_rows = rows / krow;
  const int meta_cols = columns / kcol;
  if (column_wise) {
    for (int c = 0; c < meta_cols; ++c) {
      for (int r = 0; r < meta_rows; ++r) {
        const size_t s = (size_t)c * meta_rows + r; /* col-major */
        const size_t d = (size_t)r * meta_cols + c; /* row-major */
        packed_scales[d] = canon_scales[s];
        if (canon_zps && packed_zps) packed_zps[d] = canon_zps[s];
      }
    }
  } else {
    if ((meta_rows % 16) != 0) return -1;
    for (int c = 0; c < meta_cols; ++c) {
      for (int row_blk = 0; row_blk < meta_rows; row_blk += 16) {
        const size_t base = (size_t)c * meta_rows + row_blk;
        for (int t = 0; t < 4; ++t) {
          const size_t d = base + (size_t)t * 4;
          const size_t s = base + (size_t)t * 2;
          packed_scales[d + 0] = canon_scales[s + 0];
          packed_scales[d + 1] = canon_scales[s + 1];
          packed_scales[d + 2] = canon_scales[s + 8];
          packed_scales[d + 3] = canon_scales[s + 9];
          if (canon_zps && packed_zps) {
            packed_zps[d + 0] = canon_zps[s + 0];
            packed_zps[d + 1] = canon_zps[s + 8];
            packed_zps[d + 2] = canon_zps[s + 1];
            packed_zps[d + 3] = canon_zps[s + 9];
          }
        }
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Dequantize from the canonical form.  Reference: test/blkq4_fp16_gemm_sm80_test.cu:309-328
 * (and test/blkq4_fp16_quant_sm80_test.cu:165-186): b = fp16( float(scale) * float(q - zp) ),
 * zp = 8 when there are no offsets.  Out: fp16 [K, N] column-major with leading dimension K.
 * ------------------------------------------------------------------------------------------- */
ORACLE_API int oracle_dequantize_t(int block_size, int column_wise, int rows, int columns,
                                   const uint8_t* canon_w, const uint16_t* canon_scales,
                                   const uint8_t* canon_zps, uint16_t* b, int bf16) {
  const int krow = column_wise ? block_size : 1;
  const int kcol = column_wise ? 1 : block_size;
  const int meta_rows = rows / krow;
#pragma omp parallel for schedule(static)
  for (int col = 0; col < columns; ++col) {
    for (int row = 0; row < rows; ++row) {
      const size_t meta_idx = (size_t)(col / kcol) * meta_rows + row / krow;
      const int offset = canon_zps ? canon_zps[meta_idx] : 8;
      const uint8_t byte = canon_w[(size_t)col * (rows / 2) + row / 2];
      const int w = ((row % 2 == 0) ? (byte & 0x0f) : (byte >> 4)) - offset;
      const float scale = e2f(canon_scales[meta_idx], bf16);
      b[(size_t)col * rows + row] = f2e(scale * (float)w, bf16);
    }
  }
  return 0;
}

ORACLE_API int oracle_dequantize(int block_size, int column_wise, int rows, int columns,
                                 const uint8_t* canon_w, const uint16_t* canon_scales,
                                 const uint8_t* canon_zps, uint16_t* b) {
  return oracle_dequantize_t(block_size, column_wise, rows, columns, canon_w, canon_scales, canon_zps, b, 0);
}

/* ---------------------------------------------------------------------------------------------
 * C[M,N] (fp16 row-major) = A[M,K] (fp16 row-major) * B[K,N] (fp16 column-major), fp32 accumulate
 * in ascending k, one round-to-nearest conversion to fp16, alpha = 1, beta = 0.
 * Reference: test/blkq4_fp16_gemm_sm80_test.cu:54-107 (cutlass reference GEMM, multiply_add<float>)
 * and :445-459.  A product of two fp16 values is exact in fp32, so a fused and an unfused
 * multiply-add give the same bits.
 * `af` / `bf` are scratch float copies made once so the inner loop vectorises; the k order of the
 * additions within one output is ascending within each of 8 interleaved partial sums when
 * `strict_order` is 0 (fast, for the CPU baseline) and strictly ascending when it is 1.
 * ------------------------------------------------------------------------------------------- */
ORACLE_API int oracle_gemm_t(int m, int n, int k, const uint16_t* a, const uint16_t* b, uint16_t* c,
                             int strict_order, int bf16) {
  float* af = (float*)malloc((size_t)m * k * sizeof(float));
  float* bf = (float*)malloc((size_t)n * k * sizeof(float));
  if (!af || !bf) {
    free(af);
    free(bf);
    return -1;
  }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)m * k; ++i) af[i] = e2f(a[i], bf16);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n * k; ++i) bf[i] = e2f(b[i], bf16);

#pragma omp parallel for schedule(dynamic, 4) collapse(2)
  for (int j0 = 0; j0 < n; j0 += 8) {
    for (int i = 0; i < m; ++i) {
      const float* ar = af + (size_t)i * k;
      const int jend = j0 + 8 < n ? j0 + 8 : n;
      for (int j = j0; j < jend; ++j) {
        const float* bc = bf + (size_t)j * k;
        float acc;
        if (strict_order) {
          acc = 0.0f;
          for (int kk = 0; kk < k; ++kk) acc = fmaf(ar[kk], bc[kk], acc);
        } else {
          float part[16] = {0};
          int kk = 0;
          for (; kk + 16 <= k; kk += 16) {
#pragma omp simd
            for (int t = 0; t < 16; ++t) part[t] += ar[kk + t] * bc[kk + t];
          }
          acc = 0.0f;
          for (int t = 0; t < 16; ++t) acc += part[t];
          for (; kk < k; ++kk) acc += ar[kk] * bc[kk];
        }
        c[(size_t)i * n + j] = f2e(acc, bf16);
      }
    }
  }
  free(af);
  free(bf);
  return 0;
}

ORACLE_API int oracle_gemm(int m, int n, int k, const uint16_t* a, const uint16_t* b, uint16_t* c,
                           int strict_order) {
  return oracle_gemm_t(m, n, k, a, b, c, strict_order, 0);
}

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
