// Host side of the C ABI: argument validation, error strings, kernel selection.  Plain C++ with no
// HIP headers; device work is reached through the C functions declared in blkq4_device.h.
//
// Behaviour mirrors the reference dispatcher (reference: src/blkq4_f16_gemm_sm80.cu:38-531): same
// checks in the same order, same return codes, same message texts.

#include "ms_blkq4gemm.h"

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

#include "blkq4_choose.h"
#include "blkq4_device.h"

#define BLKQ4_EXPORT __attribute__((visibility("default")))

namespace {

// Every kernel addresses the activations and the packed weights with 32-bit byte offsets.
inline bool too_large(int m, int n, int k) {
  return static_cast<uint64_t>(m) * static_cast<uint64_t>(k) * 2 >= (uint64_t{1} << 32) ||
         static_cast<uint64_t>(k) * static_cast<uint64_t>(n) / 2 >= (uint64_t{1} << 32);
}
constexpr const char* kTooLarge =
    "Kernel execution failed: Error Invalid Problem (activations of m * k * 2 bytes and packed weights of k * n / 2 bytes "
    "must stay below 4 GiB)";

inline void set_error(std::string* err, std::string&& text) {
  if (err) *err = std::move(text);
}

inline bool supported_block_size(int bs) { return bs == 16 || bs == 32 || bs == 64; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// reference: src/blkq4_f16_gemm_sm80.cu:155-203 (blkq4_quant_size_sm80_T)
int quant_size(int block_size, bool column_wise, int rows, int columns, int64_t& w_size,
               int64_t& meta_size, std::string* err) {
  if (rows == 0 || columns == 0) {
    set_error(err, "Empty problem size: " + std::to_string(rows) + "x" + std::to_string(columns));
    return -1;
  }
  const int krow = column_wise ? block_size : 1;
  const int kcol = column_wise ? 1 : block_size;
  const int meta_rows = rows / krow;
  const int meta_cols = columns / kcol;
  // The reference divides by the meta extent (which is zero when the matrix is smaller than one
  // block, a division by zero there); such shapes are reported as not quantizable here.
  // (rows % krow, columns % kcol: a matrix that is no whole number of blocks; the reference's `% meta extent`
  // lets some of those through, e.g. 96 columns in blocks of 64, and its kernels then write out of bounds)
  if (rows < 0 || (rows % 64) != 0 || meta_rows == 0 || (rows % meta_rows) != 0 || (rows % krow) != 0) {
    set_error(err, "Cannot block quantize matrix with rows: " + std::to_string(rows));
    return -1;
  }
  if (columns < 0 || (columns % 32) != 0 || meta_cols == 0 || (columns % meta_cols) != 0 || (columns % kcol) != 0) {
    set_error(err, "Cannot block quantize matrix with columns: " + std::to_string(columns));
    return -1;
  }
  w_size = static_cast<int64_t>(rows / 2) * columns;
  meta_size = static_cast<int64_t>(meta_rows) * meta_cols;
  return 0;
}

int device_failure(int code, std::string* err) {
  set_error(err, std::string("Kernel execution failed: ") + blkq4_dev_error_string(code));
  return -1;
}

}  // namespace

// reference: src/blkq4_f16_gemm_sm80.cu:431-463
extern "C" BLKQ4_EXPORT int blkq4_fp16_quant_size_sm80(int block_size, bool column_wise_blocking,
                                                       int rows, int columns,
                                                       int64_t& quant_weights_size,
                                                       int64_t& quant_meta_size, void* err_msg_ptr) {
  quant_weights_size = 0;
  quant_meta_size = 0;
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (!supported_block_size(block_size)) {
    set_error(err, "Unsupported block size: " + std::to_string(block_size));
    return -1;
  }
  return quant_size(block_size, column_wise_blocking, rows, columns, quant_weights_size,
                    quant_meta_size, err);
}

namespace {

// reference: src/blkq4_f16_gemm_sm80.cu:465-531 and :205-314 (blkq4_quant_sm80_T); bf16: the element type
// the reference's template anticipates (src/mickey/blk_q4/f16_quant_sm80.cuh:16) and its entry points
// reject (src/blkq4_f16_gemm_sm80.cu:53)
int quant_entry(bool bf16, int block_size, bool column_wise_blocking, int rows, int columns, int leadingDimension,
                void* stream, void const* weights, size_t weights_size, void* quant_weights,
                size_t quant_weights_size, void* quant_scales, size_t quant_scales_size, void* offsets,
                size_t offsets_size, void* err_msg_ptr) {
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (!supported_block_size(block_size)) {
    set_error(err, "Unsupported block size: " + std::to_string(block_size));
    return -1;
  }
  const bool has_offsets = offsets != nullptr && offsets_size > 0;

  if (rows == 0 || columns == 0) {
    set_error(err, "Empty problem size: " + std::to_string(rows) + "x" + std::to_string(columns));
    return -1;
  }
  int64_t w_elems = 0, meta_elems = 0;
  if (int e = quant_size(block_size, column_wise_blocking, rows, columns, w_elems, meta_elems, err)) {
    return e;
  }
  // element counts of the caller's buffers, as the reference's spans see them
  const int64_t qw_have = static_cast<int64_t>(quant_weights_size);
  const int64_t sc_have = static_cast<int64_t>(quant_scales_size / 2);
  const int64_t zp_have = static_cast<int64_t>(offsets_size);
  const int64_t w_have = static_cast<int64_t>(weights_size / 2);
  if (qw_have < w_elems) {
    set_error(err, "Unexpected quantized weight tensor size: " + std::to_string(qw_have) +
                       " expected: " + std::to_string(w_elems));
    return -1;
  }
  if (sc_have < meta_elems) {
    set_error(err, "Unexpected scale tensor size: " + std::to_string(sc_have) +
                       " expected: " + std::to_string(meta_elems));
    return -1;
  }
  if (has_offsets && zp_have < meta_elems) {
    set_error(err, "Unexpected offset tensor size: " + std::to_string(zp_have) +
                       " expected: " + std::to_string(meta_elems));
    return -1;
  }
  const int64_t w_need = static_cast<int64_t>(columns) * leadingDimension;
  if (w_have < w_need) {
    set_error(err, "Unexpected weight tensor size: " + std::to_string(w_have) +
                       " expected: " + std::to_string(w_need));
    return -1;
  }
  if (leadingDimension < rows) {
    set_error(err, "Leading dimension " + std::to_string(leadingDimension) +
                       " is smaller than the number of rows: " + std::to_string(rows));
    return -1;
  }
  if (weights == nullptr || quant_weights == nullptr || quant_scales == nullptr) {
    set_error(err, "Null tensor pointer");
    return -1;
  }

  blkq4_prepack_args args{};
  args.block_size = block_size;
  args.column_wise = column_wise_blocking ? 1 : 0;
  args.rows = rows;
  args.columns = columns;
  args.ld = leadingDimension;
  args.src = weights;
  args.packed_w = quant_weights;
  args.scales = quant_scales;
  args.zero_points = has_offsets ? offsets : nullptr;
  args.stream = stream;
  args.bf16 = bf16 ? 1 : 0;
  if (int code = blkq4_dev_prepack(&args)) return device_failure(code, err);
  return 0;
}

}  // namespace

extern "C" BLKQ4_EXPORT int blkq4_fp16_quant_sm80(int block_size, bool column_wise_blocking, int rows,
                                                  int columns, int leadingDimension, void* stream,
                                                  void const* weights, size_t weights_size,
                                                  void* quant_weights, size_t quant_weights_size,
                                                  void* quant_scales, size_t quant_scales_size,
                                                  void* offsets, size_t offsets_size,
                                                  void* err_msg_ptr) {
  return quant_entry(false, block_size, column_wise_blocking, rows, columns, leadingDimension, stream, weights,
                     weights_size, quant_weights, quant_weights_size, quant_scales, quant_scales_size, offsets,
                     offsets_size, err_msg_ptr);
}

// the same quantizer for bf16 weights and scales; sizes as blkq4_fp16_quant_size_sm80 gives them
extern "C" BLKQ4_EXPORT int blkq4_bf16_quant_sm80(int block_size, bool column_wise_blocking, int rows,
                                                  int columns, int leadingDimension, void* stream,
                                                  void const* weights, size_t weights_size,
                                                  void* quant_weights, size_t quant_weights_size,
                                                  void* quant_scales, size_t quant_scales_size,
                                                  void* offsets, size_t offsets_size,
                                                  void* err_msg_ptr) {
  return quant_entry(true, block_size, column_wise_blocking, rows, columns, leadingDimension, stream, weights,
                     weights_size, quant_weights, quant_weights_size, quant_scales, quant_scales_size, offsets,
                     offsets_size, err_msg_ptr);
}

namespace {

int launch_choice(const blkq4::Choice& choice, bool bf16, const blkq4_gemm_args* args) {
  if (choice.family == blkq4::kFamilyDecode) return bf16 ? blkq4_dev_decode_bf16(args) : blkq4_dev_decode(args);
  const bool streaming = choice.family == blkq4::kFamilyStreaming;
  return bf16 ? (streaming ? blkq4_dev_skinny_bf16(args) : blkq4_dev_gemm_bf16(args))
              : (streaming ? blkq4_dev_skinny(args) : blkq4_dev_gemm(args));
}

// A plan given as text (blkq4_gemm_with_plan_sm80): the kernel family and its shape parameters, everything else
// derived the way blkq4::choose() derives it.  Whether such a kernel exists and fits the problem is the launchers'
// check.  Returns false and says why when the text is no plan.
bool parse_plan(const char* text, int block_size, bool column_wise, bool bf16, int m, int n, int k, size_t workspace_capacity,
                blkq4::Choice* c, std::string* why) {
  *c = blkq4::Choice{};
  int v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (text == nullptr || std::strcmp(text, "auto") == 0) {
    *c = blkq4::choose(column_wise, bf16, m, n, k, workspace_capacity, block_size);
    return true;
  }
  if (std::sscanf(text, "tile %d %d %d %d %d %d %d %d", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5], &v[6], &v[7]) >= 7) {
    auto& t = c->t;
    c->family = blkq4::kFamilyTile;
    t.rt = v[0]; t.nt = v[1]; t.wm = v[2]; t.wn = v[3]; t.pw = v[4]; t.kw = v[5];
    t.xcd_rows = v[7];
    if (t.rt < 1 || t.nt < 1 || t.wm < 1 || t.wn < 1 || t.pw < 0 || t.kw < 1 || v[6] < 1 || v[7] < 0 || t.rt * t.wm > 64 || t.nt * t.wn > 64) {
      *why = "tile RT NT WM WN PW KW PARTS [BANDS]: positive numbers (PW may be 0, PARTS 1 means no split, BANDS 0 or absent: "
             "tile order as it is)";
      return false;
    }
    t.tiles = static_cast<int>(blkq4::ceil_div(m, 32 * t.rt * t.wm) * blkq4::ceil_div(n, 32 * t.nt * t.wn));
    t.split_k = v[6];
    if (t.split_k > 1) {
      // the tiles of the last, partly filled round (all of them when there is one round only), as choose() splits
      t.split_tiles = t.tiles % blkq4::kComputeUnits ? t.tiles % blkq4::kComputeUnits : t.tiles;
      t.workspace_bytes = blkq4::tile_workspace_bytes(t);
      if (t.workspace_bytes > workspace_capacity || static_cast<size_t>(t.split_tiles) * sizeof(int) > blkq4::kCounterBytes) {
        *why = "the split needs a workspace of " + std::to_string(t.workspace_bytes) + " bytes, more than there is";
        return false;
      }
    }
    return true;
  }
  if (std::sscanf(text, "streaming %d %d %d %d %d %d", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5]) == 6) {
    if (m > blkq4::kStreamingMaxRows || v[0] < 1 || v[1] < 1 || (v[2] != 1 && v[2] != 2) || v[3] < 1 || v[3] > 16 ||
        (v[4] != blkq4::kRowsWholeInLds && v[4] != blkq4::kRowsPerSlotInLds) || (v[5] != 1 && v[5] != v[3]) ||
        (v[2] == 1 && m > 16)) {
      *why = "streaming DEPTH NT MT WAVES ROWS SPLIT: MT 1 (up to 16 rows) or 2 (row groups of 32), ROWS 1 (whole in LDS) or 2 "
             "(staged per slice), SPLIT = WAVES (the waves split K) or 1; at most 1024 rows";
      return false;
    }
    auto& p = c->s;
    c->family = blkq4::kFamilyStreaming;
    p.depth = v[0]; p.nt = v[1]; p.mt = v[2]; p.waves = v[3]; p.am = v[4]; p.split = v[5];
    if (p.mt == 2) {
      p.rows_log2 = 5;
      p.row_groups = (m + 31) / 32;
    } else {
      p.row_groups = 1;
      while ((1 << p.rows_log2) < m) ++p.rows_log2;
    }
    blkq4::streaming_geometry(&p, !column_wise, n, k);
    return true;
  }
  if (std::sscanf(text, "decode %d %d %d %d", &v[0], &v[1], &v[2], &v[3]) == 4) {
    if (v[0] < 1 || v[0] > blkq4::kDecodeMaxRows || v[1] < 1 || v[1] > 8 || v[2] < 1 || v[2] > 16 || v[3] < 1 || v[3] > 16 ||
        (n % 16) != 0) {
      *why = "decode ROWS NT WAVES DEPTH: rows kept (a power of two, at least m), column tiles per workgroup, waves, slices per wave";
      return false;
    }
    auto& d = c->d;
    c->family = blkq4::kFamilyDecode;
    d.row = column_wise ? 0 : 1;
    d.rows = v[0]; d.nt = v[1]; d.waves = v[2]; d.depth = v[3];
    d.grid = blkq4::decode_grid(n, d.nt);
    d.lds_bytes = static_cast<uint32_t>(blkq4::decode_lds_bytes(d.row != 0, d.rows, d.nt, d.waves, d.depth));
    return true;
  }
  *why = "a plan is \"auto\", \"tile RT NT WM WN PW KW PARTS [BANDS]\", \"streaming DEPTH NT MT WAVES ROWS SPLIT\" or \"decode ROWS NT WAVES DEPTH\"";
  return false;
}

// reference: src/blkq4_f16_gemm_sm80.cu:319-429 and :38-153 (blkq4_gemm_sm80_T); bias_ptr == nullptr or
// bias_size == 0: no bias
int gemm_entry(bool bf16, int block_size, bool column_wise_blocking, int m, int n, int k, void* stream, void const* act_ptr,
               size_t a_size, void const* weights_ptr, size_t weights_size, void const* scales_ptr,
               size_t scales_size, void const* offsets_ptr, size_t offsets_size, void const* bias_ptr,
               size_t bias_size, void* output_ptr, size_t output_size, void* err_msg_ptr,
               bool static_workspace = false, bool valu_gemv = false, const char* plan = nullptr) {
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (!supported_block_size(block_size)) {
    set_error(err, "Unsupported block size: " + std::to_string(block_size));
    return -1;
  }
  const bool has_offsets = offsets_ptr != nullptr && offsets_size > 0;

  if (m <= 0 || n <= 0 || k <= 0) {
    set_error(err, "Empty problem size: " + std::to_string(m) + "x" + std::to_string(n) + "x" +
                       std::to_string(k));
    return -1;
  }
  const int krow = column_wise_blocking ? block_size : 1;
  const int kcol = column_wise_blocking ? 1 : block_size;
  const uint64_t M = static_cast<uint64_t>(m), N = static_cast<uint64_t>(n), K = static_cast<uint64_t>(k);

  if (a_size != M * K * 2) {
    set_error(err, "Unexpected activation tensor size: " + std::to_string(a_size) +
                       " expected: " + std::to_string(M * K * 2));
    return -1;
  }
  if (weights_size != (K / 2) * (N / 2) * 2) {
    set_error(err, "Unexpected weight tensor size: " + std::to_string(weights_size) +
                       " expected: " + std::to_string(K / 2 * N / 2 * 2));
    return -1;
  }
  const uint64_t meta_elems = (K / krow) * (N / kcol);
  if (scales_size != meta_elems * 2) {
    set_error(err, "Unexpected scale tensor size: " + std::to_string(scales_size) +
                       " expected: " + std::to_string(meta_elems * 2));
    return -1;
  }
  if (output_size != M * N * 2) {
    set_error(err, "Unexpected output tensor size: " + std::to_string(output_size) +
                       " expected: " + std::to_string(M * N * 2));
    return -1;
  }
  if (has_offsets && offsets_size != meta_elems) {
    set_error(err, "Unexpected offsets tensor size: " + std::to_string(offsets_size) +
                       " expected: " + std::to_string(meta_elems));
    return -1;
  }
  const bool has_bias = bias_ptr != nullptr && bias_size > 0;
  if (has_bias && bias_size != N * 2) {
    set_error(err, "Unexpected bias tensor size: " + std::to_string(bias_size) +
                       " expected: " + std::to_string(N * 2));
    return -1;
  }
  if (has_bias && !aligned16(bias_ptr)) {
    set_error(err, "Kernel execution failed: Error Misaligned Operand");
    return -1;
  }
  // What the reference kernel's can_implement rejects
  // (src/mickey/cutlass_ext/q4gemm/kernel/quantb_gemm.h:172-255).
  if (!aligned16(act_ptr) || !aligned16(weights_ptr) || (k % 8) != 0) {
    set_error(err, "Kernel execution failed: Error Misaligned Operand");
    return -1;
  }
  // n % 32: the quantize entry point cannot produce buffers for any other n (columns % 32 rule).
  if ((k % 64) != 0 || (k % krow) != 0 || (n % kcol) != 0 || (n % 32) != 0) {
    set_error(err, "Kernel execution failed: Error Invalid Problem");
    return -1;
  }
  // scales and zero-points: 4-byte aligned for every m (the tile kernel copies them four bytes at a time, and
  // which kernel runs depends on m: one rule for all of them)
  if ((reinterpret_cast<uintptr_t>(scales_ptr) & 3u) != 0 ||
      (has_offsets && (reinterpret_cast<uintptr_t>(offsets_ptr) & 3u) != 0) || !aligned16(output_ptr) || (n % 8) != 0) {
    set_error(err, "Kernel execution failed: Error Misaligned Operand");
    return -1;
  }
  // blocks along N: the streaming kernel fetches scales and zero-points 16 bytes at a time
  if (!column_wise_blocking && (!aligned16(scales_ptr) || (has_offsets && !aligned16(offsets_ptr)))) {
    set_error(err, "Kernel execution failed: Error Misaligned Operand");
    return -1;
  }
  if (act_ptr == nullptr || weights_ptr == nullptr || scales_ptr == nullptr || output_ptr == nullptr) {
    set_error(err, "Null tensor pointer");
    return -1;
  }
  if (too_large(m, n, k)) {
    set_error(err, kTooLarge);
    return -1;
  }

  blkq4_gemm_args args{};
  args.block_size = block_size;
  args.column_wise = column_wise_blocking ? 1 : 0;
  args.m = m;
  args.n = n;
  args.k = k;
  args.a = act_ptr;
  args.packed_w = weights_ptr;
  args.scales = scales_ptr;
  args.zero_points = has_offsets ? offsets_ptr : nullptr;
  args.c = output_ptr;
  args.bias = has_bias ? bias_ptr : nullptr;
  args.stream = stream;
  // Which kernel, in which shape (blkq4_choose.h; the reference switches at m > 16,
  // src/blkq4_f16_gemm_sm80.cu:343, f16_gemm_sm80.h:63-72).  A split tile kernel needs a workspace: the
  // library's own for this stream; when there is none to be had (out of memory, too many streams), the plan is
  // made again without one.
  if (valu_gemv) {
    // the GEMV kernel without MFMA, asked for by name
    if (m > 4 || !column_wise_blocking || bf16 || (m == 3 ? 4 : m) * K * 2 > 150 * 1024) {
      set_error(err, "The GEMV without matrix instructions takes fp16, 1 to 4 rows of at most 150 KiB together and blocks along K");
      return -1;
    }
    if (int code = blkq4_dev_gemv_dot(&args)) return device_failure(code, err);
    return 0;
  }
  // The allocation-free entry point plans with what its buffer holds: a shape whose best plan would need more gets
  // a smaller split or the unsplit kernel, never a refusal.
  const size_t capacity = static_workspace ? blkq4_dev_static_workspace_capacity() : blkq4_dev_workspace_capacity();
  blkq4::Choice choice;
  if (plan != nullptr) {
    // a plan given by the caller (blkq4_gemm_with_plan_sm80)
    std::string why;
    if (!parse_plan(plan, block_size, column_wise_blocking, bf16, m, n, k, capacity, &choice, &why)) {
      set_error(err, "Unknown plan: " + why);
      return -1;
    }
  } else {
    choice = blkq4::choose(column_wise_blocking, bf16, m, n, k, capacity, block_size);
  }
  if (choice.family == blkq4::kFamilyTile && choice.t.split_k > 1) {
    void* workspace = nullptr;
    if (static_workspace) {
      if (choice.t.workspace_bytes > capacity) {  // cannot happen: the plan was made for this capacity
        set_error(err, "Workspace of " + std::to_string(choice.t.workspace_bytes) +
                           " bytes needed, the allocation-free entry point holds " + std::to_string(capacity));
        return -1;
      }
      if (int code = blkq4_dev_static_workspace(&workspace)) return device_failure(code, err);
      args.workspace = workspace;
      args.workspace_bytes = capacity;
    } else {
      if (int code = blkq4_dev_workspace(stream, &workspace)) return device_failure(code, err);
      if (workspace == nullptr) {
        if (plan != nullptr && std::strcmp(plan, "auto") != 0) {
          set_error(err, "No workspace for the split the plan asks for (blkq4_gemm_workspace_info_sm80 says why)");
          return -1;
        }
        choice = blkq4::choose(column_wise_blocking, bf16, m, n, k, 0, block_size);
      } else {
        args.workspace = workspace;
        args.workspace_bytes = capacity;
      }
    }
  }
  args.streaming = choice.s;
  args.tile = choice.t;
  args.decode = choice.d;
  if (int code = launch_choice(choice, bf16, &args)) return device_failure(code, err);
  return 0;
}

}  // namespace

extern "C" BLKQ4_EXPORT int blkq4_fp16_gemm_sm80(int block_size, bool column_wise_blocking, int m,
                                                 int n, int k, void* stream, void const* act_ptr,
                                                 size_t a_size, void const* weights_ptr,
                                                 size_t weights_size, void const* scales_ptr,
                                                 size_t scales_size, void const* offsets_ptr,
                                                 size_t offsets_size, void* output_ptr,
                                                 size_t output_size, void* err_msg_ptr) {
  return gemm_entry(false, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr, weights_size,
                    scales_ptr, scales_size, offsets_ptr, offsets_size, nullptr, 0, output_ptr, output_size,
                    err_msg_ptr);
}

// the GEMM with the bias of the linear layer added in its epilogue (reference: python/ms_blkq4linear.py:26-27,
// `output += self.bias` as a second kernel)
extern "C" BLKQ4_EXPORT int blkq4_fp16_gemm_bias_sm80(int block_size, bool column_wise_blocking, int m,
                                                      int n, int k, void* stream, void const* act_ptr,
                                                      size_t a_size, void const* weights_ptr,
                                                      size_t weights_size, void const* scales_ptr,
                                                      size_t scales_size, void const* offsets_ptr,
                                                      size_t offsets_size, void const* bias_ptr,
                                                      size_t bias_size, void* output_ptr,
                                                      size_t output_size, void* err_msg_ptr) {
  return gemm_entry(false, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr, weights_size,
                    scales_ptr, scales_size, offsets_ptr, offsets_size, bias_ptr, bias_size, output_ptr,
                    output_size, err_msg_ptr);
}

// bf16 activations, scales, bias and output (fp32 accumulation, one rounding of the output, then the bias the
// way a tensor library adds two bf16 tensors); bias_ptr == nullptr or bias_size == 0: no bias
extern "C" BLKQ4_EXPORT int blkq4_bf16_gemm_sm80(int block_size, bool column_wise_blocking, int m, int n, int k,
                                                 void* stream, void const* act_ptr, size_t a_size,
                                                 void const* weights_ptr, size_t weights_size,
                                                 void const* scales_ptr, size_t scales_size,
                                                 void const* offsets_ptr, size_t offsets_size,
                                                 void const* bias_ptr, size_t bias_size, void* output_ptr,
                                                 size_t output_size, void* err_msg_ptr) {
  return gemm_entry(true, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr,
                    weights_size, scales_ptr, scales_size, offsets_ptr, offsets_size, bias_ptr, bias_size,
                    output_ptr, output_size, err_msg_ptr);
}

// blkq4_fp16_gemm_sm80 for callers that must not allocate: a split tile kernel's workspace is the buffer inside
// the library's device image, never the library's own per-stream buffer (which is allocated on first use)
extern "C" BLKQ4_EXPORT int blkq4_fp16_gemm_noalloc_sm80(int block_size, bool column_wise_blocking, int m, int n,
                                                         int k, void* stream, void const* act_ptr, size_t a_size,
                                                         void const* weights_ptr, size_t weights_size,
                                                         void const* scales_ptr, size_t scales_size,
                                                         void const* offsets_ptr, size_t offsets_size,
                                                         void* output_ptr, size_t output_size, void* err_msg_ptr) {
  return gemm_entry(false, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr, weights_size,
                    scales_ptr, scales_size, offsets_ptr, offsets_size, nullptr, 0, output_ptr, output_size,
                    err_msg_ptr, /*static_workspace=*/true);
}

// blkq4_fp16_gemm_sm80 for 1 to 4 rows, computed by the kernel that uses no matrix instructions (per-lane fp32
// partial sums, v_dot2_f32_f16, lane exchanges across K): the alternative form of the GEMV, kept callable by name
// so that it can be measured against the form blkq4_fp16_gemm_sm80 picks
extern "C" BLKQ4_EXPORT int blkq4_fp16_gemv_valu_sm80(int block_size, bool column_wise_blocking, int m, int n, int k,
                                                      void* stream, void const* act_ptr, size_t a_size,
                                                      void const* weights_ptr, size_t weights_size,
                                                      void const* scales_ptr, size_t scales_size,
                                                      void const* offsets_ptr, size_t offsets_size,
                                                      void* output_ptr, size_t output_size, void* err_msg_ptr) {
  return gemm_entry(false, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr, weights_size,
                    scales_ptr, scales_size, offsets_ptr, offsets_size, nullptr, 0, output_ptr, output_size,
                    err_msg_ptr, /*static_workspace=*/false, /*valu_gemv=*/true);
}

// Which kernel a GEMM of this shape runs, without running it: the identity of the kernel blkq4::choose() picks
// and the identity of the instantiation the launcher maps that choice to (they must agree), plus a description.
extern "C" BLKQ4_EXPORT int blkq4_gemm_plan_sm80(int block_size, bool column_wise_blocking, bool bf16,
                                                 bool has_offsets, int m, int n, int k, uint64_t* chosen_id,
                                                 uint64_t* launched_id, char* description,
                                                 size_t description_size, void* err_msg_ptr) {
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (!supported_block_size(block_size)) {
    set_error(err, "Unsupported block size: " + std::to_string(block_size));
    return -1;
  }
  const int krow = column_wise_blocking ? block_size : 1;
  const int kcol = column_wise_blocking ? 1 : block_size;
  if (m <= 0 || n <= 0 || k <= 0) {
    set_error(err, "Empty problem size: " + std::to_string(m) + "x" + std::to_string(n) + "x" + std::to_string(k));
    return -1;
  }
  if ((k % 64) != 0 || (k % krow) != 0 || (n % kcol) != 0 || (n % 32) != 0) {
    set_error(err, "Kernel execution failed: Error Invalid Problem");
    return -1;
  }
  if (too_large(m, n, k)) {
    set_error(err, kTooLarge);
    return -1;
  }
  const blkq4::Choice choice = blkq4::choose(column_wise_blocking, bf16, m, n, k, blkq4_dev_workspace_capacity(), block_size);
  blkq4_gemm_args args{};
  args.block_size = block_size;
  args.column_wise = column_wise_blocking ? 1 : 0;
  args.m = m;
  args.n = n;
  args.k = k;
  // addresses that are never used: the launchers only look at their alignment
  void* const dummy = reinterpret_cast<void*>(uintptr_t{1} << 20);
  args.a = args.packed_w = args.scales = dummy;
  args.zero_points = has_offsets ? dummy : nullptr;
  args.c = dummy;
  args.streaming = choice.s;
  args.tile = choice.t;
  args.decode = choice.d;
  args.dry_run = 1;
  uint64_t launched = 0;
  args.launched_id = &launched;
  const bool streaming = choice.family == blkq4::kFamilyStreaming;
  if (int code = launch_choice(choice, bf16, &args)) return device_failure(code, err);
  if (chosen_id != nullptr) *chosen_id = blkq4::choice_id(choice);
  if (launched_id != nullptr) *launched_id = launched;
  if (description != nullptr && description_size > 0) {
    std::string text;
    if (choice.family == blkq4::kFamilyDecode) {
      const auto& d = choice.d;
      text = std::string("decode") + (d.row ? " (blocks along N)" : "") + ": " + std::to_string(d.waves) + " waves splitting K, " + std::to_string(d.depth) +
             " slices requested by each, " + std::to_string(d.nt) + " column tile(s) x " + std::to_string(d.rows) +
             " row(s), " + std::to_string((n / 16 + d.nt - 1) / d.nt) + " workgroups";
    } else if (streaming) {
      const auto& p = choice.s;
      text = "streaming: " + std::to_string(p.waves) + " waves" + (p.split == 1 ? " with column tiles of their own" : " splitting K") +
             ", " + std::to_string(p.nt) + " column tile(s) x " + std::to_string(16 * p.mt) + " rows, " +
             std::to_string(p.depth) + " slices in flight, rows " +
             (p.am == blkq4::kRowsWholeInLds ? "whole in LDS" : "staged per slice") + ", " + std::to_string(p.row_groups) +
             " row group(s), " + std::to_string(p.grid) + " workgroups" + (p.refill ? " (walking)" : "");
    } else {
      const auto& t = choice.t;
      text = "tile: " + std::to_string(32 * t.rt * t.wm) + " x " + std::to_string(32 * t.nt * t.wn) + ", " +
             std::to_string(t.wm * t.wn * t.kw) + " + " + std::to_string(t.pw) + " waves" +
             (t.kw > 1 ? " (the computing waves split the k tile)" : "") + ", " + std::to_string(t.tiles) + " tiles";
      if (t.xcd_rows != 0) {
        const int rows = static_cast<int>(blkq4::ceil_div(m, 32 * t.rt * t.wm)) / t.xcd_rows;
        text += ", blocks of " + std::to_string(rows) + " x " + std::to_string(32 / rows) + " tiles per XCD";
      }
      if (t.split_k > 1) {
        text += ", the last " + std::to_string(t.split_tiles) + " in " + std::to_string(t.split_k) + " parts (workspace " +
                std::to_string(t.workspace_bytes) + " bytes)";
      }
    }
    const size_t len = text.size() < description_size - 1 ? text.size() : description_size - 1;
    text.copy(description, len);
    description[len] = '\0';
  }
  return 0;
}

// Set-up of the allocation-free entry point on the current device: resolves the address of the workspace inside the
// library's device image (which makes the runtime load that image, if it has not yet).
extern "C" BLKQ4_EXPORT int blkq4_fp16_gemm_noalloc_init_sm80(void* err_msg_ptr) {
  void* workspace = nullptr;
  if (int code = blkq4_dev_static_workspace(&workspace)) return device_failure(code, static_cast<std::string*>(err_msg_ptr));
  return 0;
}

// The GEMM with the kernel and its shape given by the caller instead of the cost model (see the header): what the
// model's choices are measured against.
extern "C" BLKQ4_EXPORT int blkq4_gemm_with_plan_sm80(const char* plan, int block_size, bool column_wise_blocking, bool bf16,
                                                      int m, int n, int k, void* stream, void const* act_ptr, size_t a_size,
                                                      void const* weights_ptr, size_t weights_size, void const* scales_ptr,
                                                      size_t scales_size, void const* offsets_ptr, size_t offsets_size,
                                                      void* output_ptr, size_t output_size, void* err_msg_ptr) {
  return gemm_entry(bf16, block_size, column_wise_blocking, m, n, k, stream, act_ptr, a_size, weights_ptr, weights_size,
                    scales_ptr, scales_size, offsets_ptr, offsets_size, nullptr, 0, output_ptr, output_size, err_msg_ptr,
                    /*static_workspace=*/false, /*valu_gemv=*/false, plan != nullptr ? plan : "auto");
}

// What a GEMM whose plan splits tiles would find on `stream` now (see the header).
extern "C" BLKQ4_EXPORT int blkq4_gemm_workspace_info_sm80(void* stream, int* state, int* buffers_in_use,
                                                           int* buffers_max, size_t* buffer_bytes, void* err_msg_ptr) {
  int st = 0, in_use = 0, cap = 0;
  if (int code = blkq4_dev_workspace_info(stream, &st, &in_use, &cap)) {
    return device_failure(code, static_cast<std::string*>(err_msg_ptr));
  }
  if (state != nullptr) *state = st;
  if (buffers_in_use != nullptr) *buffers_in_use = in_use;
  if (buffers_max != nullptr) *buffers_max = cap;
  if (buffer_bytes != nullptr) *buffer_bytes = blkq4_dev_workspace_capacity();
  return 0;
}

extern "C" BLKQ4_EXPORT int blkq4_gemm_workspace_release_sm80(void* err_msg_ptr) {
  if (int code = blkq4_dev_workspace_release()) return device_failure(code, static_cast<std::string*>(err_msg_ptr));
  return 0;
}

// The fp16 quantizer computes its divisions and its rounding with sequences shorter than the IEEE ones; this runs
// the comparison of the two over the whole domain on the current GPU (see the header).
extern "C" BLKQ4_EXPORT int blkq4_fp16_quant_selfcheck_sm80(void* stream, void* counts, size_t counts_size,
                                                            void* err_msg_ptr) {
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (counts == nullptr || counts_size != 4 * sizeof(uint64_t) || (reinterpret_cast<uintptr_t>(counts) & 7u) != 0) {
    set_error(err, "Unexpected counter buffer: four 64-bit counters in device memory, 8-byte aligned, expected");
    return -1;
  }
  if (int code = blkq4_dev_quant_selfcheck(counts, stream)) return device_failure(code, err);
  return 0;
}

extern "C" BLKQ4_EXPORT int blkq4_fp16_repack_sm80(int to_sm80, int rows, int columns, void* stream,
                                                   void const* src, size_t src_size, void* dst,
                                                   size_t dst_size, void* err_msg_ptr) {
  auto* err = static_cast<std::string*>(err_msg_ptr);
  if (rows <= 0 || columns <= 0) {
    set_error(err, "Empty problem size: " + std::to_string(rows) + "x" + std::to_string(columns));
    return -1;
  }
  if ((rows % 64) != 0) {
    set_error(err, "Cannot block quantize matrix with rows: " + std::to_string(rows));
    return -1;
  }
  if ((columns % 32) != 0) {
    set_error(err, "Cannot block quantize matrix with columns: " + std::to_string(columns));
    return -1;
  }
  const uint64_t bytes = static_cast<uint64_t>(rows / 2) * static_cast<uint64_t>(columns);
  if (src_size != bytes || dst_size != bytes) {
    set_error(err, "Unexpected quantized weight tensor size: " +
                       std::to_string(src_size != bytes ? src_size : dst_size) +
                       " expected: " + std::to_string(bytes));
    return -1;
  }
  if (src == nullptr || dst == nullptr) {
    set_error(err, "Null tensor pointer");
    return -1;
  }
  {
    const auto s = reinterpret_cast<uintptr_t>(src), d = reinterpret_cast<uintptr_t>(dst);
    if (s < d + bytes && d < s + bytes) {
      set_error(err, "Source and destination buffers overlap");
      return -1;
    }
    if ((s & 15u) != 0 || (d & 15u) != 0) {
      set_error(err, "Kernel execution failed: Error Misaligned Operand");
      return -1;
    }
  }
  blkq4_repack_args args{};
  args.to_sm80 = to_sm80 ? 1 : 0;
  args.rows = rows;
  args.columns = columns;
  args.src = src;
  args.dst = dst;
  args.stream = stream;
  if (int code = blkq4_dev_repack(&args)) return device_failure(code, err);
  return 0;
}

extern "C" BLKQ4_EXPORT void* blkq4_error_message_create(void) { return new std::string(); }

extern "C" BLKQ4_EXPORT char const* blkq4_error_message_cstr(void* error_message) {
  return error_message ? static_cast<std::string*>(error_message)->c_str() : "";
}

extern "C" BLKQ4_EXPORT void blkq4_error_message_destroy(void* error_message) {
  delete static_cast<std::string*>(error_message);
}
