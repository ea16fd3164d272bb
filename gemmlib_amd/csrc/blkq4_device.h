/*
 * Thin C layer between the host-side API code (plain C++, no HIP headers) and the HIP kernels.
 * Every function validates nothing: arguments have been checked by the caller in blkq4_api.cpp.
 * Each returns 0 or a hipError_t value; blkq4_dev_error_string() turns that into text.
 *
 * Data layout in device memory (K = rows = in_features, N = columns = out_features, bs = block size,
 * blocks run along K):
 *
 *   packed weights  uint8[K/32][N][16]
 *       The 16-byte unit (ks, n) holds the 32 weights k = 32*ks .. 32*ks+31 of column n as four
 *       little-endian 32-bit words; word j holds k0 = 32*ks + 8*j .. +7 and stores weight k0+t in
 *       nibble position (t >> 1) + 4 * (t & 1).  With that order `(w >> 4*i) & 0x000f000f` is the
 *       pair (k0+2i, k0+2i+1) in the low/high 16-bit halves, which is how an MFMA operand register
 *       wants it, and a lane of an MFMA operand owns exactly one word per 16- or 32-deep k step.
 *       Consecutive n are 16 bytes apart, so 32 or 64 lanes reading one unit each issue one
 *       fully coalesced 512 B / 1 KiB request.
 *   scales          fp16 [K/bs][N] row-major   (identical to the reference's packed scales)
 *   zero-points     uint8 [K/bs][N] row-major  (identical to the reference's packed offsets)
 *
 * With blocks along N (column_wise = 0: one k, bs consecutive columns) the packed weights are the
 * same and the meta data keep the reference's packed order for that blocking: column-major
 * [K][N/bs] (element (k, g) in the 16-row group starting at g*K + (k & ~15)), and inside a group of
 * 16 rows the scales of rows (2t, 2t+1, 2t+8, 2t+9) and the zero-points of rows (2t, 2t+8, 2t+1,
 * 2t+9) sit at positions 4t .. 4t+3, t = 0..3.
 */

#pragma once

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
  int block_size;      /* 16, 32 or 64 */
  int column_wise;     /* 1: blocks of bs x 1 (along K); 0: blocks of 1 x bs (along N) */
  int rows;            /* K, multiple of 64 */
  int columns;         /* N, multiple of 32 */
  int ld;              /* leading dimension of the fp16 source, >= rows */
  const void* src;     /* fp16, element (k, n) at src[k + n * ld] */
  void* packed_w;      /* uint8[K/32][N][16] */
  void* scales;        /* fp16 [K/bs][N] */
  void* zero_points;   /* uint8 [K/bs][N] or NULL (symmetric) */
  void* stream;
  int bf16;            /* 1: src and scales are bf16; 0: fp16 */
} blkq4_prepack_args;

typedef struct {
  int block_size;
  int column_wise;          /* as in blkq4_prepack_args */
  int m, n, k;
  const void* a;            /* fp16 [m][k] */
  const void* packed_w;     /* uint8[K/32][N][16] */
  const void* scales;       /* fp16 [K/bs][N]; column_wise = 0: packed [K][N/bs] order described above */
  const void* zero_points;  /* uint8, same shape and order as the scales, or NULL */
  void* c;                  /* fp16 [m][n] */
  const void* bias;         /* fp16 [n] added to every row of c after its rounding to fp16, or NULL */
  void* stream;
} blkq4_gemm_args;

typedef struct {
  int to_sm80; /* 1: native -> sm80, 0: sm80 -> native */
  int rows, columns;
  const void* src;
  void* dst;
  void* stream;
} blkq4_repack_args;

int blkq4_dev_prepack(const blkq4_prepack_args* args);
int blkq4_dev_gemm(const blkq4_gemm_args* args);   /* MFMA tile kernel, every m (made for large m) */
int blkq4_dev_skinny(const blkq4_gemm_args* args); /* weight-streaming kernel, 1 <= m <= 1024 */
int blkq4_dev_gemm_bf16(const blkq4_gemm_args* args);   /* the tile kernel with bf16 a, scales, c and bias */
int blkq4_dev_skinny_bf16(const blkq4_gemm_args* args); /* the same with bf16 a, scales, c and bias */
int blkq4_dev_repack(const blkq4_repack_args* args);
const char* blkq4_dev_error_string(int code);

#ifdef __cplusplus
}
#endif
