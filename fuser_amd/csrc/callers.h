// What the reference's expression nodes do around the nvf_cutlass kernels when a fusion is evaluated
// (csrc/ir/composite_nodes.cpp): layout conventions of the graph-level operands, synthesis of the
// stride / problem-size / offset tensors the kernels take, and "validate, else let the caller fall back".
// A caller that used to reach the kernels through ScaledMmaOp / GroupedMmaOp / CutlassNvfp4GroupedMmaOp
// calls these with the graph-level tensors.
#pragma once

#include "nvf_cutlass.h"

namespace nvfuser {
namespace callers {

// ScaledMmaOp::evaluate, kernel branch (csrc/ir/composite_nodes.cpp:1133-1162).
// mat1 [M, K/2] fp4x2, mat2 [K/2, N] fp4x2 as the graph holds it (a transposed view of the [N, K/2]
// weight), scales in the 128x4 layout, alpha fp32.  Runs nvfp4_scaled_mm on (mat1, mat2.t()) when there
// is no bias and no beta and the operands pass validateInputsNvfp4ScaledMm; otherwise returns an
// undefined tensor, which tells the caller to take its own fallback (the reference continues with
// at::_scaled_mm there).
NVF_HOST_API torch::Tensor scaled_mma(const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& scale1,
                                      const torch::Tensor& scale2, const c10::optional<torch::Tensor>& alpha,
                                      const c10::optional<torch::Tensor>& bias, const c10::optional<torch::Tensor>& beta,
                                      at::ScalarType out_dtype);

// The tensors GroupedMmaOp::evaluate derives from the graph-level `offsets` (int32 [G], the END row of
// every group) for the kernel (csrc/ir/composite_nodes.cpp:1435-1452):
// (problem_sizes int32 [G,3] = (rows, n, k), expert_offsets int32 [G] = START rows, ab_strides int64 [G] = k,
//  c_strides int64 [G] = n).
struct GroupedMmaArguments {
  torch::Tensor problem_sizes, expert_offsets, ab_strides, c_strides;
};
NVF_HOST_API GroupedMmaArguments grouped_mma_arguments(const torch::Tensor& offsets, int64_t n, int64_t k);

// GroupedMmaOp::evaluate, kernel branch (csrc/ir/composite_nodes.cpp:1427-1459).
// mat1 [M, K] contiguous, mat2 [G, K, N] whose transpose(-1, -2) is contiguous, offsets as above.
// Returns an undefined tensor when the operands do not have that form (caller falls back).
NVF_HOST_API torch::Tensor grouped_mma(const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& offsets);

// CutlassNvfp4GroupedMmaOp::evaluate (csrc/ir/composite_nodes.cpp:1663-1712).
// mat1 [M, K/2] fp4x2, mat2 [G, K/2, N] fp4x2 (a transposed view of [G, N, K/2]), problem_sizes int32 [G,3],
// expert_offsets = START rows, sf_offsets = start rows of every group's padded scale slab.
NVF_HOST_API torch::Tensor cutlass_nvfp4_grouped_mma(const torch::Tensor& mat1, const torch::Tensor& mat2,
                                                     const torch::Tensor& scale1, const torch::Tensor& scale2,
                                                     const torch::Tensor& alpha, const torch::Tensor& problem_sizes,
                                                     const torch::Tensor& expert_offsets, const torch::Tensor& sf_offsets,
                                                     at::ScalarType out_dtype);

}  // namespace callers
}  // namespace nvfuser
