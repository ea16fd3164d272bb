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
 *     with respect to that stream;
 *   - `error_message` is nullptr or a `std::string*` that receives a message when the call fails;
 *   - the return value is 0 on success and -1 on failure; no exception crosses the boundary;
 *   - every entry point may be called from several host threads.
 *
 * Device memory and state.  The quantizer, the layout conversion and the queries allocate nothing and keep
 * nothing.  The GEMM entry points keep ONE kind of state, which the reference's GEMM does not have
 * (src/blkq4_f16_gemm_sm80.cu:38-153 allocates nothing): for some shapes (few tiles and a long K, e.g. m = 256,
 * k = 11008, n = 4096) the fastest plan shares tiles out over several workgroups along K, and those leave fp32
 * partial tiles in a workspace.  The first such call on a stream allocates that workspace with hipMalloc (32 MiB
 * + 16 KiB; it waits for a small kernel on a stream of its own and, while a graph is being recorded, switches the
 * calling thread's capture mode to relaxed around the allocation) and the library keeps it: one buffer per
 * (device, stream handle, recording).  What follows from that:
 *   - calls on different streams, and a recorded graph against eager calls or against another recorded graph,
 *     never share a buffer and may run side by side;
 *   - ONE recorded graph must not run twice at the same time (two executable copies of it launched on two
 *     streams share the recording's buffer and would race);
 *   - at most 16 streams and 16 recordings get a buffer; calls beyond that, calls on hipStreamPerThread and calls
 *     made when the allocation fails run the best plan that needs no workspace (same results to the stated
 *     tolerance, up to a quarter slower on the shapes above).  blkq4_gemm_workspace_info_sm80 tells which of the
 *     two a call would get, blkq4_gemm_workspace_release_sm80 frees the buffers;
 *   - blkq4_fp16_gemm_noalloc_sm80 is the GEMM that never allocates.
 * Shapes whose plan does not split (all of the reference's own `m <= 16` cases, and most others) never touch any
 * of this.
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
 * Self-check of blkq4_fp16_quant_sm80's arithmetic on the GPU it runs on.  The quantizer is bound by its vector
 * instructions, so it computes the reference's two divisions (src/mickey/blk_q4/f16_quant_sm80.cuh:104-112, :294)
 * and its roundf (:110, :298) with shorter instruction sequences than the IEEE ones.  This entry point compares
 * the short forms with the IEEE forms over their WHOLE domain -- every range an fp16 block can have (about 10^9 pairs),
 * every nonzero symmetric extreme, every float in [0, 15] -- and leaves four 64-bit counters in `counts` (device memory,
 * counts_size = 32): disagreements for asymmetric blocks, for symmetric blocks, for the rounding (all three must
 * be 0), and the number of cases looked at.  A few milliseconds; asynchronous like every other call.
 *
 * No counterpart in the reference.
 */
int blkq4_fp16_quant_selfcheck_sm80(void* stream, void* counts, size_t counts_size, void* error_message);

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
 * that forbids allocation, tight serving loops.  Same arguments, checks and messages as blkq4_fp16_gemm_sm80 and
 * every shape it takes.  The difference: when the chosen kernel splits tiles over K and needs a workspace for the
 * fp32 partial tiles, that workspace is a buffer inside the library's device image (16 MiB + 16 KiB per GPU, held
 * until the process ends) instead of a buffer blkq4_fp16_gemm_sm80 allocates on first use, and the plan is made for
 * that size: a shape whose fastest plan needs more (m = 300, n = 28672, k = 4096 wants 30 MiB) runs a smaller
 * split or the unsplit kernel, so its result can differ from blkq4_fp16_gemm_sm80's in the last bit (another
 * order of summation) while shapes whose plan fits give the same bits.  No hipMalloc, hipFree or other allocating
 * call is made.  All streams of a GPU share the one buffer: calls that overlap on one GPU race, so issue them on
 * one stream or order them yourself.  The first call on a device asks the runtime for the buffer's address, which
 * makes it load the library's device image if nothing has yet: call blkq4_fp16_gemm_noalloc_init_sm80 (or this
 * entry point once) on each device before recording a graph.
 *
 * No counterpart in the reference (whose GEMM needs no workspace): it is for the callers that cannot allocate.
 */
int blkq4_fp16_gemm_noalloc_init_sm80(void* error_message);
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
 * cores too).  blkq4_fp16_gemm_sm80 runs this form for no shape (its MFMA kernels are faster on every shape
 * measured); it is reachable by this name only, so that the two forms can be measured against each other.
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
 * blkq4_fp16_gemm_sm80 / blkq4_bf16_gemm_sm80 (bf16 != 0) with the kernel given by the caller instead of the library's
 * cost model.  `plan` is text:
 *   "auto"                                     what the cost model picks (then identical to the entry points above);
 *   "tile RT NT WM WN PW KW PARTS [BANDS]"     the tile kernel: WM x WN computing waves of (32 RT) x (32 NT) outputs, PW
 *                                              producer waves, KW = 4 for the tiles whose waves split the k tile (else
 *                                              1), the tiles of the last round shared out over PARTS workgroups along K;
 *                                              BANDS (optional; 1, 2, 4 or 8): every whole round of 256 tiles is dealt to
 *                                              the 8 XCDs in blocks, BANDS row bands x 8 / BANDS column bands; 0 or
 *                                              absent: every eighth tile of the column-major order per XCD;
 *   "streaming DEPTH NT MT WAVES ROWS SPLIT"   the weight-streaming kernel: slices in flight, column tiles and row tiles
 *                                              (1: up to 16 rows, 2: row groups of 32) per workgroup, waves, rows whole
 *                                              in LDS (1) or staged per slice (2), SPLIT = WAVES or 1;
 *   "decode ROWS NT WAVES DEPTH"               the decode kernel: rows kept, column tiles per workgroup, waves, slices each.
 * The shapes that exist are the ones blkq4_gemm_plan_sm80 can name; any other, or one that does not fit the problem, is
 * refused with -1 before anything is launched.  Same arguments, checks and results (to the stated tolerance; the
 * reference's exact construction stays exact) as the entry points above.
 *
 * No counterpart in the reference, whose choice is a single `m > 16` (src/blkq4_f16_gemm_sm80.cu:343): it exists so
 * that the cost model's choices can be measured against the alternatives on a given machine (`python -m bench_probe.plan_check`).
 */
int blkq4_gemm_with_plan_sm80(
  const char* plan,
  int block_size,
  bool column_wise_blocking,
  bool bf16,
  int m, int n, int k,
  void* stream,
  void const* act_ptr, size_t a_size,
  void const* weights_ptr, size_t weights_size,
  void const* scales_ptr, size_t scales_size,
  void const* offsets_ptr, size_t offsets_size,
  void* output_ptr, size_t output_size,
  void* error_message);

/**
 * The workspaces of the GEMM's split plans (see "Device memory and state" at the top).  Host-side bookkeeping; no
 * kernel is launched.
 *   blkq4_gemm_workspace_info_sm80: *state = 1 when a GEMM issued on `stream` now (in the recording the stream is
 *     in, if any) has a workspace already, 0 when it would allocate one on first need, -1 when it would run the
 *     plan without a workspace (all buffers handed out, or hipStreamPerThread); buffers handed out so far, the
 *     most there can be, and the size of one.  Any of the outputs may be null.
 *   blkq4_gemm_workspace_release_sm80: frees every buffer.  The caller promises that no GEMM of this library is
 *     running or queued and that no graph recorded with one will be launched again.
 *
 * No counterpart in the reference, whose GEMM has no workspace.
 */
int blkq4_gemm_workspace_info_sm80(
    void* stream,
    int* state,
    int* buffers_in_use,
    int* buffers_max,
    size_t* buffer_bytes,
    void* error_message);
int blkq4_gemm_workspace_release_sm80(void* error_message);

/**
 * Helpers for callers that cannot construct a C++ std::string (ctypes, cgo, JNI ...): create an
 * error-message object to pass as `error_message`, read it, destroy it.  Host-only; no counterpart
 * in the reference, whose callers are all C++.
 */
void* blkq4_error_message_create(void);
char const* blkq4_error_message_cstr(void* error_message);
void blkq4_error_message_destroy(void* error_message);

}  // extern "C"
