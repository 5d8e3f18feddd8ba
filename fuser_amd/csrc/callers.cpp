#include "callers.h"

#include "nvf_checks.h"

namespace nvfuser {
namespace callers {

namespace ck = cutlass_kernels;

torch::Tensor scaled_mma(const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& scale1,
                         const torch::Tensor& scale2, const c10::optional<torch::Tensor>& alpha,
                         const c10::optional<torch::Tensor>& bias, const c10::optional<torch::Tensor>& beta,
                         at::ScalarType out_dtype) {
  // the kernel has no bias, no beta and a single (unquantized) result
  if ((bias.has_value() && bias->defined()) || (beta.has_value() && beta->defined())) return torch::Tensor();
  if (mat2.dim() != 2) return torch::Tensor();
  const torch::Tensor weight = mat2.t();  // [N, K/2], the layout nvfp4_scaled_mm expects
  const torch::Tensor a = alpha.has_value() ? *alpha : torch::Tensor();
  try {
    ck::validateInputsNvfp4ScaledMm(mat1, weight, scale1, scale2, a);
  } catch (const std::exception&) {
    return torch::Tensor();
  }
  return ck::nvfp4_scaled_mm(mat1, weight, scale1, scale2, a, out_dtype, /*skip_checks=*/true);
}

GroupedMmaArguments grouped_mma_arguments(const torch::Tensor& offsets, int64_t n, int64_t k) {
  NVF_CHECK(offsets.dim() == 1, "grouped_mma_arguments: offsets must be a 1D tensor of group end rows");
  const auto i32 = offsets.options().dtype(at::kInt);
  const auto i64 = offsets.options().dtype(at::kLong);
  const int64_t groups = offsets.size(0);
  const torch::Tensor ends = offsets.to(at::kInt);
  // start of a group = end of the one before it, 0 for the first
  torch::Tensor starts = at::zeros({groups}, i32);
  if (groups > 1) starts.slice(0, 1, groups).copy_(ends.slice(0, 0, groups - 1));
  GroupedMmaArguments r;
  r.expert_offsets = starts;
  r.ab_strides = at::full({groups}, k, i64);
  r.c_strides = at::full({groups}, n, i64);
  r.problem_sizes = at::empty({groups, 3}, i32);
  r.problem_sizes.select(1, 0).copy_(ends - starts);
  r.problem_sizes.select(1, 1).fill_(n);
  r.problem_sizes.select(1, 2).fill_(k);
  return r;
}

torch::Tensor grouped_mma(const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& offsets) {
  if (mat1.dim() != 2 || mat2.dim() != 3 || !mat1.is_contiguous()) return torch::Tensor();
  const torch::Tensor weight = mat2.transpose(-1, -2);  // [G, N, K]
  if (!weight.is_contiguous()) return torch::Tensor();
  const GroupedMmaArguments args = grouped_mma_arguments(offsets, /*n=*/weight.size(1), /*k=*/mat1.size(-1));
  return ck::grouped_mm(mat1, weight, args.ab_strides, args.c_strides, args.problem_sizes, args.expert_offsets);
}

torch::Tensor cutlass_nvfp4_grouped_mma(const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& scale1,
                                        const torch::Tensor& scale2, const torch::Tensor& alpha,
                                        const torch::Tensor& problem_sizes, const torch::Tensor& expert_offsets,
                                        const torch::Tensor& sf_offsets, at::ScalarType out_dtype) {
  NVF_CHECK(mat1.scalar_type() == at::ScalarType::Float4_e2m1fn_x2 && mat2.scalar_type() == at::ScalarType::Float4_e2m1fn_x2);
  NVF_CHECK(problem_sizes.dim() == 2, "problem_sizes must be a 2D tensor");
  NVF_CHECK(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)");
  NVF_CHECK(mat1.dim() == 2 && mat2.dim() == 3, "cutlass_nvfp4_grouped_mma: mat1 must be 2D and mat2 3D");
  const int64_t groups = problem_sizes.size(0);
  const int64_t k = mat1.size(1) * 2;  // mat1 is packed, two values per byte
  const int64_t n = mat2.size(2);
  const auto i64 = at::TensorOptions().device(mat1.device()).dtype(at::kLong);
  const torch::Tensor ab_strides = at::full({groups}, k, i64);
  const torch::Tensor c_strides = at::full({groups}, n, i64);
  // the kernel takes the weights as [G, N, K/2]
  return ck::nvfp4_scaled_grouped_mm(mat1, mat2.transpose(-1, -2), scale1, scale2, alpha, ab_strides, c_strides,
                                     problem_sizes, expert_offsets, sf_offsets, out_dtype);
}

}  // namespace callers
}  // namespace nvfuser
