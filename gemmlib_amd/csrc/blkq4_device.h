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

/* Which streaming kernel runs and how it is launched: the template parameters of skinny_mfma_kernel
 * (blkq4_skinny.hip) and the launch geometry derived from them.  Filled in by blkq4::choose() (blkq4_choose.h). */
typedef struct {
  int depth, nt, mt, waves, am, split; /* split = waves (the waves split K) or 1 (they do not) */
  int rows_log2, row_groups;
  int refill;          /* workgroups walk over several column groups / waves stream all of K by themselves */
  int cg_stride;       /* column groups a workgroup steps over */
  uint32_t grid;       /* workgroups */
  uint32_t lds_bytes;  /* dynamic LDS */
  uint32_t red_offset; /* where the partial tiles of the sum across waves lie in it */
} blkq4_streaming_plan;

/* Which tile kernel runs: wm x wn computing waves of (32 rt) x (32 nt) outputs, pw producer waves.
 * kw = 4 (with wm = wn = 1): four computing waves share the one (32 rt) x (32 nt) tile and split every 64-deep k tile
 * between them; kw = 1 otherwise.
 * split_k > 1: the last split_tiles tiles of the tile order are computed by split_k workgroups each, which
 * leave fp32 partial tiles in the workspace; the last of them to finish sums them in a fixed order.
 * xcd_rows: 0, or into how many row bands (1, 2, 4 or 8) a round of 256 tiles is cut for the 8 XCDs, each of which then
 * owns one band x (xcd_rows / 8 of the round's columns) -- see xcd_tile_map() in blkq4_choose.h. */
typedef struct {
  int rt, nt, wm, wn, pw;
  int kw;
  int xcd_rows;
  int split_k;            /* 1: no workspace needed */
  int split_tiles;        /* 0 without a split */
  int tiles;              /* all tiles of the problem */
  size_t workspace_bytes; /* arrival counters + partial tiles, 0 without a split */
} blkq4_tile_plan;

/* Which decode kernel runs (blkq4_decode.hip): `rows` activation rows kept (a power of two >= m), `nt` column
 * tiles per workgroup, `waves` waves that split K, `depth` slices requested by each.  Filled in by
 * blkq4::decode_shape() (blkq4_choose.h). */
typedef struct {
  int row;             /* 1: blocks along N */
  int rows, nt, waves, depth;
  uint32_t grid;       /* workgroups */
  uint32_t lds_bytes;  /* dynamic LDS */
} blkq4_decode_plan;

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
  blkq4_streaming_plan streaming; /* read by blkq4_dev_skinny* */
  blkq4_tile_plan tile;           /* read by blkq4_dev_gemm* */
  blkq4_decode_plan decode;       /* read by blkq4_dev_decode* */
  void* workspace;                /* tile.split_k > 1: device memory of workspace_bytes, 256-byte aligned, whose */
  size_t workspace_bytes;         /* first 16 KiB (the arrival counters) are zero between launches */
  int dry_run;                    /* 1: launch nothing, only report the kernel */
  uint64_t* launched_id;          /* if not NULL: receives the identity of the kernel instantiation (blkq4_choose.h) */
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
int blkq4_dev_decode(const blkq4_gemm_args* args);      /* decode kernel: few rows, all of K requested at once, blocks along K */
int blkq4_dev_decode_bf16(const blkq4_gemm_args* args); /* the same with bf16 a, scales, c and bias */
int blkq4_dev_gemv_dot(const blkq4_gemm_args* args);    /* fp16 GEMV on the vector ALU (no MFMA): 1 <= m <= 4, blocks along K */
int blkq4_dev_repack(const blkq4_repack_args* args);
/* The fp16 quantizer's shortened arithmetic against its IEEE definition over the whole domain; counts: four
 * 64-bit counters in device memory (disagreements of asymmetric blocks, symmetric blocks, the rounding; cases). */
int blkq4_dev_quant_selfcheck(void* counts, void* stream);
const char* blkq4_dev_error_string(int code);

/* Workspace of the split tile kernels: the library-owned buffer of (current device, stream, the recording the
 * stream is in, if any), allocated on first use with a fixed size and its counters zeroed; *ptr = NULL (and 0
 * returned) when there is none and none can be made (out of memory, too many buffers handed out, or the stream is
 * hipStreamPerThread). */
size_t blkq4_dev_workspace_capacity(void);
int blkq4_dev_workspace(void* stream, void** ptr);
/* What a split GEMM issued on `stream` now would find: *state = 1 a buffer, 0 room to allocate one, -1 neither (it
 * would run the unsplit plan); buffers handed out so far and the most there can be. */
int blkq4_dev_workspace_info(void* stream, int* state, int* in_use, int* capacity);
/* Frees every buffer (the caller promises that nothing that uses one is running, queued or will be replayed). */
int blkq4_dev_workspace_release(void);
/* The workspace inside the library's device image (nothing is ever allocated): one per device, shared by every
 * stream of that device. */
size_t blkq4_dev_static_workspace_capacity(void);
int blkq4_dev_static_workspace(void** ptr);  /* resolves the buffer's address on the first call per device */

#ifdef __cplusplus
}
#endif
