// Call sites written the way the reference's own callers use cutlass/nvf_cutlass.h (the pybind lambdas of
// python/python_direct/cutlass.cpp:17-117 and the expression nodes of csrc/ir/composite_nodes.cpp), compiled
// and linked against this build's header and shared objects: every export must exist with the reference's
// name, namespace, argument list and return type.  Run without a GPU it exercises the failure path: CPU
// tensors must be rejected with nvfuser::nvfError carrying the reference's message.
#include <cstdio>
#include <cstring>
#include <functional>
#include <tuple>
#include <type_traits>

#include "callers.h"
#include "nvf_cutlass.h"

namespace ck = nvfuser::cutlass_kernels;

// the address of every export with the exact type the reference declares
static_assert(std::is_same_v<decltype(&ck::nvfp4_scaled_mm),
                             torch::Tensor (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                               const torch::Tensor&, at::ScalarType, bool)>);
static_assert(std::is_same_v<decltype(&ck::mxfp8_scaled_mm),
                             torch::Tensor (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                               const torch::Tensor&, at::ScalarType, bool)>);
static_assert(std::is_same_v<decltype(&ck::nvfp4_scaled_mm_blockscale),
                             std::pair<torch::Tensor, torch::Tensor> (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                                                         const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, bool)>);
static_assert(std::is_same_v<decltype(&ck::validateInputsNvfp4ScaledMm),
                             std::tuple<int64_t, int64_t, int64_t> (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                                                       const torch::Tensor&, const torch::Tensor&, bool)>);
static_assert(std::is_same_v<decltype(&ck::validateInputsMxFp8ScaledMm),
                             std::tuple<int64_t, int64_t, int64_t> (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                                                       const torch::Tensor&, const torch::Tensor&, bool)>);
static_assert(std::is_same_v<decltype(&ck::nvfp4_scaled_grouped_mm),
                             torch::Tensor (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                               const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                               const torch::Tensor&, const torch::Tensor&, const at::ScalarType)>);
static_assert(std::is_same_v<decltype(&ck::grouped_mm),
                             torch::Tensor (*)(const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&,
                                               const torch::Tensor&, const torch::Tensor&)>);
static_assert(std::is_same_v<decltype(&ck::getSMVersion), int (*)()> && std::is_same_v<decltype(&ck::getMultiProcessorCount), int (*)()>);

static int expect_error(const char* what, const char* needle, const std::function<void()>& f) {
  try {
    f();
  } catch (const nvfuser::nvfError& e) {
    if (std::strstr(e.what(), needle)) return 0;
    std::printf("%s: wrong message: %s\n", what, e.what());
    return 1;
  }
  std::printf("%s: no error\n", what);
  return 1;
}

int main() {
  int bad = 0;
  const auto u8 = torch::TensorOptions().dtype(torch::kUInt8);
  torch::Tensor a = torch::zeros({128, 32}, u8).view(at::ScalarType::Float4_e2m1fn_x2);
  torch::Tensor b = torch::zeros({64, 32}, u8).view(at::ScalarType::Float4_e2m1fn_x2);
  torch::Tensor sa = torch::zeros({128, 4}, u8).view(at::ScalarType::Float8_e4m3fn);
  torch::Tensor sb = torch::zeros({128, 4}, u8).view(at::ScalarType::Float8_e4m3fn);
  torch::Tensor alpha = torch::ones({}, torch::kFloat32);
  // the pybind lambda of the dense op: (a, b, scales_a, scales_b, alpha, out_dtype) with skip_checks defaulted
  bad += expect_error("nvfp4_scaled_mm", "CUDA", [&] { ck::nvfp4_scaled_mm(a, b, sa, sb, alpha, at::ScalarType::BFloat16); });
  bad += expect_error("mxfp8_scaled_mm", "CUDA", [&] {
    ck::mxfp8_scaled_mm(a.view(at::ScalarType::Float8_e4m3fn), b.view(at::ScalarType::Float8_e4m3fn), sa.view(at::ScalarType::Float8_e8m0fnu),
                        sb.view(at::ScalarType::Float8_e8m0fnu), alpha, at::ScalarType::Half);
  });
  // ScaledMmaOp: validate, run with skip_checks = true, else fall back (undefined tensor here)
  torch::Tensor fell_back = nvfuser::callers::scaled_mma(a, b.t(), sa, sb, alpha, c10::nullopt, c10::nullopt, at::ScalarType::BFloat16);
  if (fell_back.defined()) { std::printf("scaled_mma ran on CPU tensors\n"); ++bad; }
  // GroupedMmaOp: END offsets -> the kernel's arguments
  const auto args = nvfuser::callers::grouped_mma_arguments(torch::tensor({3, 3, 10}, torch::kInt32), /*n=*/64, /*k=*/32);
  if (args.problem_sizes.size(0) != 3 || args.problem_sizes[2][0].item<int>() != 7 || args.expert_offsets[2].item<int>() != 3) {
    std::printf("grouped_mma_arguments: wrong sizes / offsets\n");
    ++bad;
  }
  bad += expect_error("grouped_mm", "CUDA", [&] {
    ck::grouped_mm(torch::zeros({10, 32}, torch::kBFloat16), torch::zeros({3, 64, 32}, torch::kBFloat16), args.ab_strides, args.c_strides,
                   args.problem_sizes, args.expert_offsets);
  });
  std::printf(bad ? "FAILED\n" : "call sites ok\n");
  return bad;
}
