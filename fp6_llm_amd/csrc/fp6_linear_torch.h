// torch::Tensor entry points of the FPx x FP16 linear layer for C++ callers, with the names, argument order and shapes of the
// reference's header (usyd-fsalab/fp6_llm, fp6_llm/csrc/fp6_linear.cuh:50-90).  Defined in torch_binding.cpp (the extension
// _fp6mi_torch, which links libfp6mi.so); the same functions are bound to Python under the reference's six names
// (fp6_llm/csrc/pybind.cpp:8-15).  Where the reference asserts or exits, these throw pybind11::value_error / std::runtime_error.
#ifndef FP6MI_FP6_LINEAR_TORCH_H
#define FP6MI_FP6_LINEAR_TORCH_H

#include <torch/extension.h>

// _in_feats: fp16 [B, IC] on the GPU;  _weights: int32 [OC, IC/32*x], the REFERENCE prepacked layout, on the same GPU;
// _scales: fp16 [OC].  Returns fp16 [B, OC].  (fp6_llm/csrc/fp6_linear.cuh:50-61)
torch::Tensor fp6_linear_forward_cuda(torch::Tensor _in_feats, torch::Tensor _weights, torch::Tensor _scales, int splitK = 1);
torch::Tensor fp_eXmY_linear_forward_cuda(int EXPONENT, int MANTISSA, torch::Tensor _in_feats, torch::Tensor _weights, torch::Tensor _scales,
                                          int splitK = 1);

// raw int32 CPU [OC, IC/32*x] -> the reference's prepacked layout, bit-exact (fp6_llm/csrc/fp6_linear.cuh:67-71)
torch::Tensor weight_matrix_prepacking_cpu(torch::Tensor fp6_tensor);
torch::Tensor weight_matrix_prepacking_fp_eXmY_cpu(int EXPONENT, int MANTISSA, torch::Tensor fpx_tensor);

// RAW weights + fp16 [OC] scales (CPU) -> fp16 [OC, IC], bit-exact (fp6_llm/csrc/fp6_linear.cuh:83-90)
torch::Tensor weight_matrix_dequant_cpu(torch::Tensor fp6_tensor, torch::Tensor fp16_scale);
torch::Tensor weight_matrix_dequant_fp_eXmY_cpu(int EXPONENT, int MANTISSA, torch::Tensor fpx_tensor, torch::Tensor fp16_scale);

#endif
