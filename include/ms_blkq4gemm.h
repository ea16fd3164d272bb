/*
 * Public C ABI of the MI355X (gfx950) blockwise-int4 x fp16 GEMM library.
 *
 * The first three entry points keep the names, argument order, argument meaning and error behaviour
 * of the reference library's public header (reference: include/ms_blkq4gemm.h:41-50, :71-80, :94-100,
 * implemented in src/blkq4_f16_gemm_sm80.cu:319-531) so that a program or extension linked against
 * the reference links against this library unchanged.  The `_sm80` suffix is part of that contract
 * and says nothing about the hardware the code runs on.
 *
 * Conventions shared by all entry points
 *   - every pointer is DEVICE memory owned by the caller unless stated otherwise;
 *   - every `*_size` argument is a size in BYTES; the two outputs of the size query are ELEMENT counts;
 *   - `stream` is a hipStream_t cast to void* (nullptr = the default stream); calls are asynchronous
 *     with respect to that stream and allocate no device memory;
 *   - `error_message` is nullptr or a `std::string*` that receives a message when the call fails;
 *   - the return value is 0 on success and -1 on failure; no exception crosses the boundary;
 *   - the library keeps no global state and may be called from several host threads.
 *
 * The includer provides <cstdint> and <cstddef> (as with the reference header).
 */

#pragma once

#include <cstddef>
#include <cstdint>

extern "C" {

/**
 * C[m,n] (fp16, row-major) = A[m,k] (fp16, row-major) x dequant(W[k,n]), fp32 accumulation, one
 * rounding to fp16.  W, scales and offsets are the buffers `blkq4_fp16_quant_sm80` produced for the
 * same block_size / blocking / shape (or buffers converted with `blkq4_fp16_repack_sm80`).
 *
 * Replaces: reference include/ms_blkq4gemm.h:41-50 (src/blkq4_f16_gemm_sm80.cu:319-429).
 *
 * Sizes must be exact: a_size = m*k*2, weights_size = k*n/2, scales_size = (k/bs)*n*2,
 * offsets_size = (k/bs)*n (or offsets_ptr == nullptr / offsets_size == 0 for symmetric weights with
 * the implicit zero-point 8), output_size = m*n*2.  k must be a multiple of 64 and n a multiple of
 * the block's column extent; A, W and C must be 16-byte aligned.
 */
int blkq4_fp16_gemm_sm80(
  int block_size,
  bool column_wise_blocking,
  int m, int n, int k, void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * The GEMM above with the bias of the linear layer added in its epilogue: every row of C gets
 * bias[0..n) (fp16) added AFTER the sum has been rounded to fp16, in fp32 and rounded to fp16 again,
 * which is bit for bit what the reference module's `output += self.bias` computes with a second
 * kernel (reference: python/ms_blkq4linear.py:26-27).  bias_size = n*2, bias 16-byte aligned;
 * bias_ptr == nullptr or bias_size == 0 means no bias (then identical to blkq4_fp16_gemm_sm80).
 *
 * No counterpart in the reference's C API (its module adds the bias itself); every other argument,
 * check and message as in blkq4_fp16_gemm_sm80.
 */
int blkq4_fp16_gemm_bias_sm80(
  int block_size,
  bool column_wise_blocking,
  int m, int n, int k,
  void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void const* bias_ptr, size_t bias_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * Quantize an fp16 weight matrix blockwise to 4 bits and pack it for the GEMM above.
 * `weights` holds element (row r, column c) at weights[r + c * leadingDimension] (rows = in_features,
 * columns = out_features, i.e. a torch [out, in] contiguous tensor with leadingDimension = in).
 *
 * Replaces: reference include/ms_blkq4gemm.h:71-80 (src/blkq4_f16_gemm_sm80.cu:465-531).
 *
 * Outputs: quant_weights rows*columns/2 bytes; quant_scales one fp16 per block; offsets one uint8
 * (0..15) per block, or nullptr / size 0 to select the symmetric quantizer.  The scale and offset
 * buffers are byte-identical to the reference's for column-wise blocking (row-major [rows/bs, columns]).
 * The weight buffer holds the same nibbles in this library's gfx950 order; `blkq4_fp16_repack_sm80`
 * converts either way without loss.
 */
extern int blkq4_fp16_quant_sm80(
    int block_size,
    bool column_wise_blocking,
    int rows, int columns, int leadingDimension,
    void* stream,
    void const* weights, size_t weights_size,
    void* quant_weights, size_t quant_weights_size,
    void* quant_scales, size_t quant_scales_size,
    void* offsets, size_t offsets_size,
    void* error_message);

/**
 * Element counts of the buffers `blkq4_fp16_quant_sm80` fills: quant_weights_size uint8 elements and
 * quant_meta_size scale elements (and as many offset bytes).  Host-only.
 *
 * Replaces: reference include/ms_blkq4gemm.h:94-100 (src/blkq4_f16_gemm_sm80.cu:431-463).
 */
int blkq4_fp16_quant_size_sm80(
    int block_size,
    bool column_wise_blocking,
    int rows, int columns,
    int64_t& quant_weights_size,
    int64_t& quant_meta_size,
    void* error_message);

/**
 * Convert a packed weight buffer between this library's gfx950 order and the reference's sm80 order
 * (reference: src/mickey/blk_q4/f16_quant_sm80.cuh:362-417).  `to_sm80 != 0` converts gfx950 -> sm80,
 * `to_sm80 == 0` converts sm80 -> gfx950.  Both buffers hold rows*columns/2 bytes and must not
 * overlap.  Scales and offsets need no conversion for column-wise blocking.
 *
 * No counterpart in the reference: it exists so that weights packed by the reference can be loaded
 * here and vice versa, and so that the packing can be compared byte for byte with the reference's.
 */
int blkq4_fp16_repack_sm80(
    int to_sm80,
    int rows, int columns,
    void* stream,
    void const* src, size_t src_size,
    void* dst, size_t dst_size,
    void* error_message);

/**
 * bf16: the quantizer and the GEMM above for bf16 weights, activations, scales, bias and output, the
 * element type the reference's templates anticipate (reference: src/mickey/blk_q4/f16_quant_sm80.cuh:16,
 * src/mickey/cutlass_ext/q4gemm/warp/quantb_mma_tensor_op.h:95-114) and its entry points reject
 * (src/blkq4_f16_gemm_sm80.cu:53) -- so these two have no counterpart in the reference's C API.
 * Same arguments, checks and messages as blkq4_fp16_quant_sm80 and blkq4_fp16_gemm_bias_sm80, every
 * 16-bit buffer holding bf16; buffer sizes from blkq4_fp16_quant_size_sm80.  Arithmetic: the reference
 * quantizer's with the scale rounded to bf16; weight = bf16(scale * (q - offset)) with one rounding; fp32
 * accumulation, one rounding of the output to bf16, then the bias added in fp32 and rounded to bf16.
 * Both blockings.  The packed weights and the offsets are interchangeable with the fp16 entry points';
 * the scales are not.
 */
int blkq4_bf16_quant_sm80(
    int block_size,
    bool column_wise_blocking,
    int rows, int columns, int leadingDimension,
    void* stream,
    void const* weights, size_t weights_size,
    void* quant_weights, size_t quant_weights_size,
    void* quant_scales, size_t quant_scales_size,
    void* offsets, size_t offsets_size,
    void* error_message);
int blkq4_bf16_gemm_sm80(
  int block_size,
  bool column_wise_blocking,
  int m, int n, int k,
  void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void const* bias_ptr, size_t bias_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * blkq4_fp16_gemm_sm80 for callers that cannot allocate device memory: code recorded into a graph by a harness
 * that forbids allocation, tight serving loops.  Same arguments, checks, messages, kernels and result bits as
 * blkq4_fp16_gemm_sm80.  The difference: when the chosen kernel splits tiles over K and needs a workspace for the
 * fp32 partial tiles, that workspace is a buffer inside the library's device image (16 MiB + 16 KiB per GPU, held
 * until the process ends) instead of the per-stream buffer blkq4_fp16_gemm_sm80 allocates on first use.  No
 * hipMalloc, hipFree or other allocating call is made.  A shape whose plan needs more than the buffer holds is
 * rejected with "Workspace of N bytes needed, the allocation-free entry point holds M" (-1); blkq4_fp16_gemm_sm80
 * takes such a shape.  All streams of a GPU share the one buffer: calls that overlap on one GPU race, so issue
 * them on one stream or order them yourself.
 *
 * No counterpart in the reference (whose GEMM needs no workspace): it is for the callers that cannot allocate.
 */
int blkq4_fp16_gemm_noalloc_sm80(
  int block_size,
  bool column_wise_blocking,
  int m, int n, int k,
  void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * The GEMV (1 <= m <= 4, fp16, column_wise_blocking = true) computed without matrix instructions: per-lane fp32
 * partial sums over K with v_dot2_f32_f16, summed across the wave by lane exchanges and across the workgroup's
 * waves through LDS.  Same arguments, checks and messages as blkq4_fp16_gemm_sm80, same dequantized weights, fp32
 * accumulation and single rounding of the output; other shapes are rejected (-1).
 *
 * No counterpart in the reference (whose small-M kernel, src/mickey/blk_q4/f16_gemm_sm80.h:63-72, uses tensor
 * cores too).  blkq4_fp16_gemm_sm80 picks between this form and the MFMA form by shape; this entry point runs this
 * form whatever the shape, so that the two can be measured against each other.
 */
int blkq4_fp16_gemv_valu_sm80(
  int block_size,
  bool column_wise_blocking,
  int m, int n, int k,
  void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * Which kernel a GEMM of this shape runs, without running it.  Host-only.  chosen_id receives the identity of the
 * kernel the library's cost model picks for (m, n, k), launched_id the identity of the kernel instantiation its
 * launcher maps that choice to -- the two are equal unless the library is broken -- and description (if not
 * null, description_size bytes) a line of text such as "tile: 128 x 256, 4 + 4 waves, 258 tiles, the last 2 in
 * 8 parts".  Any of the three may be null.
 *
 * No counterpart in the reference, whose choice is a single `m > 16` (src/blkq4_f16_gemm_sm80.cu:343): it exists
 * so that a test can check, on a machine without a GPU, that the choice and the launchers agree for every shape,
 * and so that a user can ask what a shape gets.
 */
int blkq4_gemm_plan_sm80(
    int block_size,
    bool column_wise_blocking,
    bool bf16,
    bool has_offsets,
    int m, int n, int k,
    uint64_t* chosen_id,
    uint64_t* launched_id,
    char* description, size_t description_size,
    void* error_message);

/**
 * Helpers for callers that cannot construct a C++ std::string (ctypes, cgo, JNI ...): create an
 * error-message object to pass as `error_message`, read it, destroy it.  Host-only; no counterpart
 * in the reference, whose callers are all C++.
 */
void* blkq4_error_message_create(void);
char const* blkq4_error_message_cstr(void* error_message);
void blkq4_error_message_destroy(void* error_message);

}  // extern "C"
