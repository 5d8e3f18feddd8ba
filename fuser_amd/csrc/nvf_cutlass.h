// at::Tensor entry points of the quantized-GEMM path, same names, namespace, argument order and
// error behaviour as the reference's cutlass/nvf_cutlass.h, implemented on MI355X by forwarding
// raw device pointers to the C ABI of libnvf_hip.so (include/nvf_hip.h).  libtorch is used for
// tensor plumbing only: allocation of the result, the current HIP stream, dtype/shape queries.
#pragma once

#include <torch/torch.h>

#include <exception>
#include <string>
#include <tuple>
#include <utility>

#define NVF_HOST_API __attribute__((visibility("default")))

// Built inside the reference's tree (its csrc/ on the include path), the failed checks throw the reference's own
// nvfuser::nvfError through its own NVF_CHECK / NVF_THROW (csrc/exceptions.h:136-245), so that the program holds one
// definition of the class and catch sites may use msg(), context(), what_without_backtrace().  Built on its own,
// a stand-in with the same name, base class and what() takes its place.
#if defined(__has_include)
#if __has_include(<exceptions.h>) && __has_include(<visibility.h>)
#include <exceptions.h>
#define NVF_HIP_REFERENCE_EXCEPTIONS 1
#endif
#endif

namespace nvfuser {

#ifndef NVF_HIP_REFERENCE_EXCEPTIONS
class NVF_HOST_API nvfError : public std::exception {
 public:
  explicit nvfError(std::string msg) : msg_(std::move(msg)) {}
  const char* what() const noexcept override { return msg_.c_str(); }
  const std::string& msg() const { return msg_; }
  const char* what_without_backtrace() const noexcept { return msg_.c_str(); }

 private:
  std::string msg_;
};
#endif

namespace cutlass_kernels {

// cutlass/nvf_cutlass.h:17-24
inline int64_t ceilDiv(int64_t x, int64_t y) { return (x + y - 1) / y; }
inline int64_t roundUp(int64_t x, int64_t y) { return ceilDiv(x, y) * y; }

// cutlass/cutlass_utils.cpp:13-41
NVF_HOST_API int getSMVersion();             // gfx target number of the current device (950)
NVF_HOST_API int getMultiProcessorCount();   // compute units of the current device

// cutlass/nvf_cutlass.h:44-50.  Returns (m, n, k) with k = 2 * a.size(1); throws nvfError.
NVF_HOST_API std::tuple<int64_t, int64_t, int64_t> validateInputsNvfp4ScaledMm(
    const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
    const torch::Tensor& alpha, bool skip_checks = false);

// cutlass/nvf_cutlass.h:68-75.  out[m,n] = alpha * dequant(a) @ dequant(b)^T, out_dtype Half | BFloat16.
NVF_HOST_API torch::Tensor nvfp4_scaled_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a,
                                           const torch::Tensor& scales_b, const torch::Tensor& alpha,
                                           at::ScalarType out_dtype, bool skip_checks = false);

// cutlass/nvf_cutlass.h:147-154.  The product alpha * dequant(a) @ dequant(b)^T (fp32) quantized again to
// NVFP4 along N: returns (fp4 [m, n/2], e4m3 block scales in the 128x4 layout of [roundUp(m,128), roundUp(n/16,4)]);
// global_normconst is the fp32 global (encode) scale of the output.
NVF_HOST_API std::pair<torch::Tensor, torch::Tensor> nvfp4_scaled_mm_blockscale(
    const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
    const torch::Tensor& alpha, const torch::Tensor& global_normconst, bool skip_checks = false);

// cutlass/nvf_cutlass.h:95-101.  Returns (m, n, k) with k = a.size(1).
NVF_HOST_API std::tuple<int64_t, int64_t, int64_t> validateInputsMxFp8ScaledMm(
    const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
    const torch::Tensor& alpha, bool skip_checks = false);

// cutlass/nvf_cutlass.h:119-126
NVF_HOST_API torch::Tensor mxfp8_scaled_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a,
                                           const torch::Tensor& scales_b, const torch::Tensor& alpha,
                                           at::ScalarType out_dtype, bool skip_checks = false);

// cutlass/nvf_cutlass.h:180-191
NVF_HOST_API torch::Tensor nvfp4_scaled_grouped_mm(const torch::Tensor& a, const torch::Tensor& b,
                                                   const torch::Tensor& a_blockscale, const torch::Tensor& b_blockscales,
                                                   const torch::Tensor& alphas, const torch::Tensor& ab_strides,
                                                   const torch::Tensor& c_strides, const torch::Tensor& problem_sizes,
                                                   const torch::Tensor& expert_offsets, const torch::Tensor& sf_offsets,
                                                   const at::ScalarType out_dtype);

// cutlass/nvf_cutlass.h:211-217
NVF_HOST_API torch::Tensor grouped_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& ab_strides,
                                      const torch::Tensor& c_strides, const torch::Tensor& problem_sizes,
                                      const torch::Tensor& expert_offsets);

}  // namespace cutlass_kernels

// Eager counterparts of the graph ops fd.ops.nv_block_quantize / nv_grouped_block_quantize /
// preprocess_grouped_matmul_input_sf (python/python_direct/ops.cpp:3521-3607, :3179-3212); the
// reference reaches runtime/block_quantization_kernels.cu only through its JIT.
namespace block_quantization {

// -> (quantized, block_scales).  dtype Float4_e2m1fn_x2 (block 16, e4m3 scales, optional 0-dim fp32
// global_scale) or Float8_e4m3fn (block 32, e8m0 scales, no global scale).  With swizzled scales the
// scale tensor has the padded shape (roundUp(M,128), roundUp(K/block,4)) that the GEMM validators expect.
NVF_HOST_API std::pair<torch::Tensor, torch::Tensor> nv_block_quantize(
    const torch::Tensor& input, const c10::optional<torch::Tensor>& global_scale, bool swizzle_block_scales,
    int64_t block_size, at::ScalarType dtype);

// -> (quantized [M, K/2], block_scales [sum roundUp(m_g,128) upper bound M + 127*G, roundUp(K/16,4)])
NVF_HOST_API std::pair<torch::Tensor, torch::Tensor> nv_grouped_block_quantize(
    const torch::Tensor& input, const torch::Tensor& input_offsets, const torch::Tensor& output_offsets,
    const c10::optional<torch::Tensor>& global_scale, int64_t block_size, at::ScalarType dtype);

// nv_grouped_block_quantize of silu(gate) * up (evaluated in the inputs' 16-bit type as the eager chain of
// benchmarks/python/layers_for_inference_benchmark.py:504 does), without materialising the product.
NVF_HOST_API std::pair<torch::Tensor, torch::Tensor> silu_mul_nv_grouped_block_quantize(
    const torch::Tensor& gate, const torch::Tensor& up, const torch::Tensor& input_offsets,
    const torch::Tensor& output_offsets, const c10::optional<torch::Tensor>& global_scale);

// 0-dim fp32 device tensor 448 * 6 / max|tensor| (1.0 if all zero), the global_scale argument of the
// quantizers; compute_nvfp4_global_scale of tests/python/direct/test_narrow_precision.py:138-156 without the
// host round trip.
NVF_HOST_API torch::Tensor compute_nvfp4_global_scale(const torch::Tensor& tensor);

NVF_HOST_API torch::Tensor preprocess_grouped_matmul_input_sf(const torch::Tensor& input,
                                                              const torch::Tensor& input_offsets,
                                                              const torch::Tensor& output_offsets);

}  // namespace block_quantization
}  // namespace nvfuser
