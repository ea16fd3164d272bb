// PyTorch-ROCm extension `ms_blkq4linear_ext`: tensor checks, allocation and device guard around the
// three C entry points.  Same Python surface as the reference extension
// (reference: python/ms_blkq4linear_ext/ms_blkq4linear.cpp:13-123):
//   quant(block_size, col_wise, has_offsets, weights) -> [q_weights(uint8), q_scales(fp16), q_zp(uint8)]
//   forward(block_size, col_wise, in_features, out_features, input, q_weights, q_scales, q_zp, bias=None) -> Tensor
// Differences on purpose: kernels run on torch's current stream instead of the default stream, a
// scale-only quantization returns an empty uint8 tensor for q_zp (the reference returns an undefined
// tensor that its own forward() cannot take), and bfloat16 weights / inputs are taken too (scales, bias and
// output then are bfloat16), through blkq4_bf16_quant_sm80 / blkq4_bf16_gemm_sm80.

#include <torch/extension.h>

// PyTorch-ROCm tensors carry the device type "cuda"; these are the guard and stream accessors that
// speak that device type while driving HIP.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <string>
#include <vector>

#include "ms_blkq4gemm.h"

namespace {

constexpr size_t kHalfBytes = 2;

std::vector<torch::Tensor> blkq4linear_quant(int64_t block_size, bool col_wise, bool has_offsets,
                                             torch::Tensor weights) {
  const bool bf16 = weights.scalar_type() == torch::kBFloat16;
  TORCH_CHECK(bf16 || weights.scalar_type() == torch::kFloat16,
              "blkq4linear_quant only supports float16 weights");
  TORCH_CHECK(weights.numel() != 0, "blkq4linear_quant only supports non-empty tensors");
  TORCH_CHECK(weights.is_contiguous(), "blkq4linear_quant only supports contiguous tensors");
  TORCH_CHECK(weights.dim() == 2, "blkq4linear_quant only supports 2D tensors");
  TORCH_CHECK(weights.is_cuda(), "blkq4linear_quant only supports CUDA tensors, instead got ",
              weights.device().str());
  const int64_t out_features = weights.size(0);
  const int64_t in_features = weights.size(1);

  std::string err;
  int64_t w_elems = 0, meta_elems = 0;
  int rc = blkq4_fp16_quant_size_sm80(static_cast<int>(block_size), col_wise, static_cast<int>(in_features),
                                      static_cast<int>(out_features), w_elems, meta_elems, &err);
  TORCH_CHECK(rc == 0, err);

  const c10::hip::HIPGuardMasqueradingAsCUDA guard(weights.device());
  const auto bytes = torch::TensorOptions().dtype(torch::kUInt8).device(weights.device());
  torch::Tensor q_weights = torch::empty({w_elems}, bytes);
  torch::Tensor q_scales = torch::empty({meta_elems}, bytes.dtype(weights.scalar_type()));
  torch::Tensor q_zp = torch::empty({has_offsets ? meta_elems : 0}, bytes);

  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(weights.device().index()).stream();
  const auto quant_entry = bf16 ? &blkq4_bf16_quant_sm80 : &blkq4_fp16_quant_sm80;
  rc = quant_entry(static_cast<int>(block_size), col_wise, static_cast<int>(in_features),
                   static_cast<int>(out_features), static_cast<int>(in_features), stream,
                   weights.data_ptr(), weights.numel() * kHalfBytes, q_weights.data_ptr(),
                   static_cast<size_t>(w_elems), q_scales.data_ptr(),
                   static_cast<size_t>(meta_elems) * kHalfBytes,
                   has_offsets ? q_zp.data_ptr() : nullptr,
                   has_offsets ? static_cast<size_t>(meta_elems) : 0, &err);
  TORCH_CHECK(rc == 0, err);
  return {q_weights, q_scales, q_zp};
}

torch::Tensor blkq4linear_forward(int64_t block_size, bool col_wise, int64_t in_features,
                                  int64_t out_features, torch::Tensor input, torch::Tensor q_weights,
                                  torch::Tensor q_scales, torch::Tensor q_zp,
                                  const c10::optional<torch::Tensor>& bias) {
  const bool bf16 = input.scalar_type() == torch::kBFloat16;
  TORCH_CHECK(bf16 || input.scalar_type() == torch::kFloat16, "blkq4linear_forward only supports float16 inputs");
  TORCH_CHECK(q_scales.scalar_type() == input.scalar_type(),
              "blkq4linear_forward: the scales must have the input's element type");
  TORCH_CHECK(input.dim() == 2 && input.size(1) == in_features,
              "Activation shape is not compatible with the weights");
  TORCH_CHECK(input.is_cuda(), "blkq4linear_forward only supports CUDA inputs");
  const auto dev = input.device();
  TORCH_CHECK(q_weights.device() == dev && q_scales.device() == dev && (!q_zp.defined() || q_zp.numel() == 0 || q_zp.device() == dev),
              "blkq4linear_forward requires all tensors on the same device");
  input = input.contiguous();

  const c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  torch::Tensor output = torch::empty({input.size(0), out_features}, input.options());

  const void* zp_ptr = nullptr;
  size_t zp_bytes = 0;
  if (q_zp.defined() && q_zp.numel() > 0) {
    zp_ptr = q_zp.data_ptr();
    zp_bytes = static_cast<size_t>(q_zp.numel());
  }
  // the bias is added in the GEMM's epilogue (the reference module adds it with a second kernel,
  // python/ms_blkq4linear.py:26-27); a bias that is not 16-byte aligned is copied first
  torch::Tensor bias_t;
  const void* bias_ptr = nullptr;
  size_t bias_bytes = 0;
  if (bias.has_value() && bias->defined() && bias->numel() > 0) {
    TORCH_CHECK(bias->scalar_type() == input.scalar_type() && bias->dim() == 1 && bias->size(0) == out_features,
                "blkq4linear_forward: the bias must be a float16 tensor of out_features elements");
    TORCH_CHECK(bias->device() == dev, "blkq4linear_forward requires all tensors on the same device");
    bias_t = bias->contiguous();
    if ((reinterpret_cast<uintptr_t>(bias_t.data_ptr()) & 15u) != 0) bias_t = bias_t.clone();
    bias_ptr = bias_t.data_ptr();
    bias_bytes = bias_t.numel() * kHalfBytes;
  }
  std::string err;
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).stream();
  const auto gemm_entry = bf16 ? &blkq4_bf16_gemm_sm80 : &blkq4_fp16_gemm_bias_sm80;
  const int rc = gemm_entry(
      static_cast<int>(block_size), col_wise, static_cast<int>(input.size(0)), static_cast<int>(out_features),
      static_cast<int>(in_features), stream, input.data_ptr(), input.numel() * kHalfBytes,
      q_weights.data_ptr(), static_cast<size_t>(q_weights.numel()), q_scales.data_ptr(),
      q_scales.numel() * kHalfBytes, zp_ptr, zp_bytes, bias_ptr, bias_bytes, output.data_ptr(),
      output.numel() * kHalfBytes, &err);
  TORCH_CHECK(rc == 0, err);
  return output;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("quant", &blkq4linear_quant, "Quantize float 16 weights");
  m.def("forward", &blkq4linear_forward, "Forward pass for block quantized linear layer", pybind11::arg("block_size"),
        pybind11::arg("col_wise"), pybind11::arg("in_features"), pybind11::arg("out_features"),
        pybind11::arg("input"), pybind11::arg("q_weights"), pybind11::arg("q_scales"), pybind11::arg("q_zp"),
        pybind11::arg("bias") = pybind11::none());
}
