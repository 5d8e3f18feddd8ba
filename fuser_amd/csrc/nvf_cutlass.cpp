// Host side of the quantized-GEMM path: validation with the reference's rules and messages, output
// allocation, current-stream lookup, then one call into the C ABI of libnvf_hip.so.
#include "nvf_cutlass.h"

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "nvf_checks.h"
#include "nvf_hip.h"

namespace nvfuser {
namespace {

void* current_stream(const torch::Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

void check_status(int status, const char* op) {
  if (status != NVF_OK) NVF_THROW(op, ": ", nvf_status_string(status), ": ", nvf_last_error());
}

int to_nvf_dtype(at::ScalarType t) {
  switch (t) {
    case at::ScalarType::Float: return NVF_F32;
    case at::ScalarType::BFloat16: return NVF_BF16;
    case at::ScalarType::Half: return NVF_F16;
    default: return -1;
  }
}

// Shared body of the two dense validators (cutlass/nvf_cutlass.cpp:13-122 and :124-234).
std::tuple<int64_t, int64_t, int64_t> validate_scaled_mm(const torch::Tensor& a, const torch::Tensor& b,
                                                         const torch::Tensor& scales_a, const torch::Tensor& scales_b,
                                                         const torch::Tensor& alpha, bool skip_checks, bool nvfp4) {
  NVF_CHECK(a.dim() == 2, "Operand A must be a matrix.");
  NVF_CHECK(b.dim() == 2, "Operand B must be a matrix.");
  NVF_CHECK(a.sizes()[1] == b.sizes()[1], "A and B shapes cannot be multiplied (", a.sizes()[0], ",", a.sizes()[1],
            " and ", b.sizes()[0], ",", b.sizes()[1], ")");
  const int64_t m = a.sizes()[0];
  const int64_t n = b.sizes()[0];
  const int64_t k = nvfp4 ? a.sizes()[1] * 2 : a.sizes()[1];
  std::tuple<int64_t, int64_t, int64_t> ret = {m, n, k};
  if (skip_checks) return ret;

  for (const torch::Tensor& t : {a, b, scales_a, scales_b, alpha}) {
    NVF_CHECK(t.is_cuda() && t.is_contiguous(), "Input argument must be a CUDA tensor and contiguous.");
  }
  if (nvfp4) {
    NVF_CHECK(a.scalar_type() == at::ScalarType::Float4_e2m1fn_x2, "Expected Float4_e2m1fn_x2 for Operand A.");
    NVF_CHECK(b.scalar_type() == at::ScalarType::Float4_e2m1fn_x2, "Expected Float4_e2m1fn_x2 for Operand B.");
    NVF_CHECK(scales_a.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected FP8_E4M3 for Blockscale scale_a.");
    NVF_CHECK(scales_b.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected FP8_E4M3 for Blockscale scale_b.");
  } else {
    NVF_CHECK(a.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected Float8_e4m3fn for Operand A.");
    NVF_CHECK(b.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected Float8_e4m3fn for Operand B.");
    NVF_CHECK(scales_a.scalar_type() == at::ScalarType::Float8_e8m0fnu, "Expected FP8_e8m0fnu for Blockscale scale_a.");
    NVF_CHECK(scales_b.scalar_type() == at::ScalarType::Float8_e8m0fnu, "Expected FP8_e8m0fnu for Blockscale scale_b.");
  }
  NVF_CHECK(alpha.scalar_type() == at::ScalarType::Float, "Expected FP32 for alpha scalar.");

  const int64_t kAlignment = nvfp4 ? 32 : 16;
  NVF_CHECK_EQ(k % kAlignment, 0, "The K dimension", k, "is not divisible by ", kAlignment);
  NVF_CHECK_EQ(n % kAlignment, 0, "The N dimension", n, "is not divisible by ", kAlignment);

  const int64_t rounded_m = cutlass_kernels::roundUp(m, 128);
  const int64_t rounded_n = cutlass_kernels::roundUp(n, 128);
  const int64_t rounded_k = cutlass_kernels::roundUp(k / (nvfp4 ? 16 : 32), 4);
  NVF_CHECK(scales_a.dim() == 2, "Blockscale scale_a must be a matrix.");
  NVF_CHECK(scales_b.dim() == 2, "Blockscale scale_b must be a matrix.");
  NVF_CHECK(scales_a.sizes()[1] == scales_b.sizes()[1],
            "scale_a and scale_b shapes cannot be multiplied because the inner-most dimensions are not equal.");
  NVF_CHECK(scales_a.sizes()[0] == rounded_m && scales_a.sizes()[1] == rounded_k,
            "scale_a must be padded and swizzled to a shape (", rounded_m, ",", rounded_k, "), but got a shape (",
            scales_a.sizes()[0], ",", scales_a.sizes()[1], ")");
  NVF_CHECK(scales_b.sizes()[0] == rounded_n && scales_b.sizes()[1] == rounded_k,
            "scale_b must be padded and swizzled to a shape (", rounded_n, ",", rounded_k, "), but got a shape (",
            scales_b.sizes()[0], ",", scales_b.sizes()[1], ")");
  return ret;
}

}  // namespace

namespace cutlass_kernels {

int getSMVersion() {
  int v = 0;
  check_status(nvf_get_arch_version(&v), "getSMVersion");
  return v;
}

int getMultiProcessorCount() {
  static int count = [] {
    int c = 0;
    check_status(nvf_get_multiprocessor_count(&c), "getMultiProcessorCount");
    return c;
  }();
  return count;
}

std::tuple<int64_t, int64_t, int64_t> validateInputsNvfp4ScaledMm(const torch::Tensor& a, const torch::Tensor& b,
                                                                 const torch::Tensor& scales_a,
                                                                 const torch::Tensor& scales_b,
                                                                 const torch::Tensor& alpha, bool skip_checks) {
  return validate_scaled_mm(a, b, scales_a, scales_b, alpha, skip_checks, /*nvfp4=*/true);
}

std::tuple<int64_t, int64_t, int64_t> validateInputsMxFp8ScaledMm(const torch::Tensor& a, const torch::Tensor& b,
                                                                 const torch::Tensor& scales_a,
                                                                 const torch::Tensor& scales_b,
                                                                 const torch::Tensor& alpha, bool skip_checks) {
  return validate_scaled_mm(a, b, scales_a, scales_b, alpha, skip_checks, /*nvfp4=*/false);
}

// cutlass/nvfp4_scaled_mm.cu:283-312
torch::Tensor nvfp4_scaled_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a,
                              const torch::Tensor& scales_b, const torch::Tensor& alpha, at::ScalarType out_dtype,
                              bool skip_checks) {
  auto [m, n, k] = validateInputsNvfp4ScaledMm(a, b, scales_a, scales_b, alpha, skip_checks);
  c10::DeviceGuard guard(a.device());
  void* stream = current_stream(a);
  auto options = at::TensorOptions().dtype(out_dtype).device(a.device());
  torch::Tensor output = at::empty({m, n}, options);
  if (out_dtype != at::ScalarType::Half && out_dtype != at::ScalarType::BFloat16) {
    NVF_THROW("Unsupported output data type of nvfp4 scaled_mm.");
  }
  // scratch for the shapes that split K, from torch's stream-ordered allocator (the reference allocates its
  // kernel's workspace in the same place, cutlass/nvfp4_scaled_mm.cu:241-244)
  const int64_t ws_bytes = nvf_nvfp4_scaled_mm_workspace_bytes(m, n, k);
  torch::Tensor workspace;
  if (ws_bytes > 0) workspace = at::empty({ws_bytes}, at::TensorOptions().dtype(at::ScalarType::Byte).device(a.device()));
  check_status(nvf_nvfp4_scaled_mm_ws(a.data_ptr(), b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(),
                                      static_cast<const float*>(alpha.data_ptr()), output.data_ptr(), m, n, k,
                                      to_nvf_dtype(out_dtype), ws_bytes > 0 ? workspace.data_ptr() : nullptr, ws_bytes, stream),
               "nvfp4_scaled_mm");
  return output;
}

// cutlass/nvfp4_scaled_mm_blockscale.cu:332-373
std::pair<torch::Tensor, torch::Tensor> nvfp4_scaled_mm_blockscale(const torch::Tensor& a, const torch::Tensor& b,
                                                                   const torch::Tensor& scales_a, const torch::Tensor& scales_b,
                                                                   const torch::Tensor& alpha,
                                                                   const torch::Tensor& global_normconst, bool skip_checks) {
  auto [m, n, k] = validateInputsNvfp4ScaledMm(a, b, scales_a, scales_b, alpha, skip_checks);
  NVF_CHECK(global_normconst.is_cuda() && global_normconst.scalar_type() == at::ScalarType::Float && global_normconst.numel() == 1,
            "global_normconst must be a single fp32 value on the device.");
  c10::DeviceGuard guard(a.device());
  void* stream = current_stream(a);
  torch::Tensor output = at::empty({m, ceilDiv(n, 2)}, at::TensorOptions().dtype(at::ScalarType::Float4_e2m1fn_x2).device(a.device()));
  // The 128x4 layout needs whole 128-row tiles; for m % 128 == 0 this is the reference's [m, roundUp(n/16, 4)].
  torch::Tensor output_blockscale =
      at::empty({roundUp(m, 128), roundUp(n / 16, 4)}, at::TensorOptions().dtype(at::ScalarType::Float8_e4m3fn).device(a.device()));
  check_status(nvf_nvfp4_scaled_mm_blockscale(a.data_ptr(), b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(),
                                              static_cast<const float*>(alpha.data_ptr()),
                                              static_cast<const float*>(global_normconst.data_ptr()), output.data_ptr(),
                                              output_blockscale.data_ptr(), /*product dump*/ nullptr, m, n, k, stream),
               "nvfp4_scaled_mm_blockscale");
  return {output, output_blockscale};
}

// cutlass/mxfp8_scaled_mm.cu:290-319
torch::Tensor mxfp8_scaled_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a,
                              const torch::Tensor& scales_b, const torch::Tensor& alpha, at::ScalarType out_dtype,
                              bool skip_checks) {
  auto [m, n, k] = validateInputsMxFp8ScaledMm(a, b, scales_a, scales_b, alpha, skip_checks);
  c10::DeviceGuard guard(a.device());
  void* stream = current_stream(a);
  auto options = at::TensorOptions().dtype(out_dtype).device(a.device());
  torch::Tensor output = at::empty({m, n}, options);
  if (out_dtype != at::ScalarType::Half && out_dtype != at::ScalarType::BFloat16) {
    NVF_THROW("Unsupported output data type of mxfp8 scaled_mm.");
  }
  check_status(nvf_mxfp8_scaled_mm(a.data_ptr(), b.data_ptr(), scales_a.data_ptr(), scales_b.data_ptr(),
                                   static_cast<const float*>(alpha.data_ptr()), output.data_ptr(), m, n, k,
                                   to_nvf_dtype(out_dtype), stream),
               "mxfp8_scaled_mm");
  return output;
}

// cutlass/nvfp4_scaled_group_mm.cu:570-688 (validation) and :714-788 (entry)
torch::Tensor nvfp4_scaled_grouped_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& a_blockscale,
                                      const torch::Tensor& b_blockscales, const torch::Tensor& alphas,
                                      const torch::Tensor& ab_strides, const torch::Tensor& c_strides,
                                      const torch::Tensor& problem_sizes, const torch::Tensor& expert_offsets,
                                      const torch::Tensor& sf_offsets, const at::ScalarType out_dtype) {
  NVF_CHECK(a.dim() >= 1 && b.dim() >= 2, "Operands must have rank >= 1 and >= 2.");
  // the reference allocates the result before validating
  NVF_CHECK(a.is_cuda(), "Expected CUDA tensor for Operand A.");
  auto options = at::TensorOptions().dtype(out_dtype).device(a.device());
  torch::Tensor output = at::empty({a.size(0), b.size(1)}, options);

  NVF_CHECK(a.scalar_type() == at::ScalarType::Float4_e2m1fn_x2, "Expected Float4_e2m1fn_x2 for Operand A.");
  NVF_CHECK(b.scalar_type() == at::ScalarType::Float4_e2m1fn_x2, "Expected Float4_e2m1fn_x2 for Operand B.");
  NVF_CHECK(a_blockscale.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected FP8_E4M3 for Blockscale scale_a.");
  NVF_CHECK(b_blockscales.scalar_type() == at::ScalarType::Float8_e4m3fn, "Expected FP8_E4M3 for Blockscale scale_b.");
  NVF_CHECK(alphas.scalar_type() == at::ScalarType::Float, "Expected FP32 for alpha scalar.");
  NVF_CHECK(b.is_cuda(), "Expected CUDA tensor for Operand B.");
  NVF_CHECK(a_blockscale.is_cuda(), "Expected CUDA tensor for Blockscale scale_a.");
  NVF_CHECK(b_blockscales.is_cuda(), "Expected CUDA tensor for Blockscale scale_b.");
  NVF_CHECK(alphas.is_cuda(), "Expected CUDA tensor for alpha scalar.");
  NVF_CHECK(a.is_contiguous(), "Expected contiguous tensor for Operand A.");
  NVF_CHECK(b.is_contiguous(), "Expected contiguous tensor for Operand B.");
  NVF_CHECK(a_blockscale.is_contiguous(), "Expected contiguous tensor for Blockscale scale_a.");
  NVF_CHECK(b_blockscales.is_contiguous(), "Expected contiguous tensor for Blockscale scale_b.");
  NVF_CHECK(alphas.is_contiguous(), "Expected contiguous tensor for alpha scalar.");
  NVF_CHECK(a_blockscale.dim() == 2,
            "Expected a_blockscale to be of shape: [padded_m, k // nvfp4_block_size], observed rank: ",
            a_blockscale.dim());
  NVF_CHECK(b_blockscales.dim() == 3,
            "Expected b_blockscale to be of shape:  [num_experts, n, k // nvfp4_block_size], observed rank: ",
            b_blockscales.dim());
  NVF_CHECK(problem_sizes.dim() == 2, "problem_sizes must be  a 2D tensor");
  NVF_CHECK(problem_sizes.size(1) == 3, "problem_sizes must have the shape (num_experts, 3)");
  NVF_CHECK(problem_sizes.size(0) == expert_offsets.size(0),
            "Number of experts in problem_sizes must match expert_offsets");
  NVF_CHECK(problem_sizes.dtype() == torch::kInt32, "problem_sizes must be int32.");
  NVF_CHECK_EQ(a.dim(), 2, "Expected Operand A to be a 2D tensor.");
  NVF_CHECK_EQ(b.dim(), 3, "Expected Operand B to be a 3D tensor.");
  constexpr int kOperandAlignment = 32;
  NVF_CHECK_EQ(a.size(-1) % kOperandAlignment, 0, "The inner dimension ", a.size(-1),
               " of Operand A is not a multiple of ", kOperandAlignment);
  NVF_CHECK_EQ(b.size(-1) % kOperandAlignment, 0, "The inner dimension ", b.size(-1),
               " of Operand B is not a multiple of ", kOperandAlignment);
  constexpr int kOutputAlignment = 8;
  NVF_CHECK_EQ(b.size(-2) % kOutputAlignment, 0, "The inner dimension ", b.size(-2),
               " of the output tensor is not a multiple of ", kOutputAlignment);
  // Needed by this implementation (the reference reads them on the device without checking).
  NVF_CHECK(expert_offsets.scalar_type() == at::ScalarType::Int && sf_offsets.scalar_type() == at::ScalarType::Int,
            "expert_offsets and sf_offsets must be int32.");
  NVF_CHECK(expert_offsets.is_cuda() && sf_offsets.is_cuda() && problem_sizes.is_cuda(),
            "problem_sizes, expert_offsets and sf_offsets must be CUDA tensors.");
  NVF_CHECK(expert_offsets.is_contiguous() && sf_offsets.is_contiguous() && problem_sizes.is_contiguous(),
            "problem_sizes, expert_offsets and sf_offsets must be contiguous.");
  NVF_CHECK(a.size(1) == b.size(2), "A and B inner dimensions differ (", a.size(1), " vs ", b.size(2), ")");
  (void)ab_strides;  // carry K and N again; the kernel derives them from the shapes
  (void)c_strides;

  const int64_t M = a.size(0), N = b.size(1), K = 2 * b.size(2);
  c10::DeviceGuard guard(a.device());
  void* stream = current_stream(a);
  if (out_dtype != at::ScalarType::Half && out_dtype != at::ScalarType::BFloat16) {
    NVF_THROW("Unsupported output data type of nvfp4 scaled_grouped_mm.");
  }
  check_status(nvf_nvfp4_scaled_grouped_mm(a.data_ptr(), b.data_ptr(), a_blockscale.data_ptr(), b_blockscales.data_ptr(),
                                           static_cast<const float*>(alphas.data_ptr()), output.data_ptr(),
                                           static_cast<const int32_t*>(problem_sizes.data_ptr()),
                                           static_cast<const int32_t*>(expert_offsets.data_ptr()),
                                           static_cast<const int32_t*>(sf_offsets.data_ptr()),
                                           static_cast<int>(problem_sizes.size(0)), M, N, K, to_nvf_dtype(out_dtype),
                                           stream),
               "nvfp4_scaled_grouped_mm");
  return output;
}

// cutlass/group_mm.cu:417-497 (validation) and :518-571 (entry)
torch::Tensor grouped_mm(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& ab_strides,
                         const torch::Tensor& c_strides, const torch::Tensor& problem_sizes,
                         const torch::Tensor& expert_offsets) {
  NVF_CHECK(a.dim() >= 1 && b.dim() >= 2, "Operands must have rank >= 1 and >= 2.");
  NVF_CHECK(a.is_cuda(), "Expected CUDA tensor for Operand A.");
  auto options = at::TensorOptions().dtype(a.scalar_type()).device(a.device());
  torch::Tensor output = at::empty({a.size(0), b.size(1)}, options);

  NVF_CHECK(a.scalar_type() == at::ScalarType::BFloat16 || a.scalar_type() == at::ScalarType::Half,
            "Expected BFloat16 or Half for Operand A.");
  NVF_CHECK(b.scalar_type() == at::ScalarType::BFloat16 || b.scalar_type() == at::ScalarType::Half,
            "Expected BFloat16 or Half for Operand B.");
  NVF_CHECK_EQ(ab_strides.dtype(), at::kLong);
  NVF_CHECK_EQ(c_strides.dtype(), at::kLong);
  NVF_CHECK(b.is_cuda(), "Expected CUDA tensor for Operand B.");
  NVF_CHECK(a.is_contiguous(), "Expected contiguous tensor for Operand A.");
  NVF_CHECK(b.is_contiguous(), "Expected contiguous tensor for Operand B.");
  NVF_CHECK_EQ(a.dim(), 2, "Expected Operand A to be a 2D tensor.");
  NVF_CHECK_EQ(b.dim(), 3, "Expected Operand B to be a 3D tensor.");
  constexpr int kAlignment = 8;
  NVF_CHECK_EQ(a.size(-1) % kAlignment, 0, "The inner dimension ", a.size(-1), " of Operand A is not a multiple of ",
               kAlignment);
  NVF_CHECK_EQ(b.size(-1) % kAlignment, 0, "The inner dimension ", b.size(-1), " of Operand B is not a multiple of ",
               kAlignment);
  NVF_CHECK_EQ(b.size(-2) % kAlignment, 0, "The inner dimension ", b.size(-2),
               " of the output tensor is not a multiple of ", kAlignment);
  NVF_CHECK_EQ(problem_sizes.dim(), 2);
  NVF_CHECK_EQ(problem_sizes.size(1), 3);
  NVF_CHECK_EQ(problem_sizes.size(0), expert_offsets.size(0));
  NVF_CHECK_EQ(problem_sizes.dtype(), at::kInt);
  // Needed by this implementation (the reference reads them on the device without checking).
  NVF_CHECK(a.scalar_type() == b.scalar_type(), "Operands A and B must have the same dtype.");
  NVF_CHECK(expert_offsets.scalar_type() == at::ScalarType::Int, "expert_offsets must be int32.");
  NVF_CHECK(expert_offsets.is_cuda() && problem_sizes.is_cuda(), "problem_sizes and expert_offsets must be CUDA tensors.");
  NVF_CHECK(expert_offsets.is_contiguous() && problem_sizes.is_contiguous(),
            "problem_sizes and expert_offsets must be contiguous.");
  NVF_CHECK(a.size(1) == b.size(2), "A and B inner dimensions differ (", a.size(1), " vs ", b.size(2), ")");

  const int64_t M = a.size(0), N = b.size(1), K = b.size(2);
  c10::DeviceGuard guard(a.device());
  void* stream = current_stream(a);
  check_status(nvf_grouped_mm(a.data_ptr(), b.data_ptr(), output.data_ptr(),
                              static_cast<const int32_t*>(problem_sizes.data_ptr()),
                              static_cast<const int32_t*>(expert_offsets.data_ptr()),
                              static_cast<int>(problem_sizes.size(0)), M, N, K, to_nvf_dtype(a.scalar_type()), stream),
               "grouped_mm");
  return output;
}

}  // namespace cutlass_kernels

namespace block_quantization {

namespace {
void check_quant_input(const torch::Tensor& input, int64_t block) {
  NVF_CHECK(input.is_cuda() && input.is_contiguous(), "Input argument must be a CUDA tensor and contiguous.");
  NVF_CHECK(to_nvf_dtype(input.scalar_type()) >= 0, "Block quantization expects Float, BFloat16 or Half input.");
  NVF_CHECK(input.dim() >= 1, "Block quantization expects an input of rank >= 1.");
  NVF_CHECK_EQ(input.size(-1) % block, 0, "The inner dimension ", input.size(-1),
               " is not divisible by the block size ", block);
}
const float* check_global_scale(const c10::optional<torch::Tensor>& gs, const torch::Tensor& input) {
  if (!gs.has_value() || !gs->defined()) return nullptr;
  NVF_CHECK(gs->dim() == 0 && gs->scalar_type() == at::ScalarType::Float, "Global scale must be a 0-dim fp32 tensor.");
  NVF_CHECK(gs->is_cuda() && gs->device() == input.device(), "Global scale must live on the input's device.");
  return static_cast<const float*>(gs->data_ptr());
}
}  // namespace

std::pair<torch::Tensor, torch::Tensor> nv_block_quantize(const torch::Tensor& input,
                                                          const c10::optional<torch::Tensor>& global_scale,
                                                          bool swizzle_block_scales, int64_t block_size,
                                                          at::ScalarType dtype) {
  const bool fp4 = dtype == at::ScalarType::Float4_e2m1fn_x2;
  const bool fp8 = dtype == at::ScalarType::Float8_e4m3fn;
  NVF_CHECK(fp4 || fp8, "Block quantization supports Float4_e2m1fn(_x2) and Float8_e4m3fn outputs.");
  NVF_CHECK(block_size == (fp4 ? 16 : 32), "Block size must be 16 for nvfp4 and 32 for mxfp8, got ", block_size);
  check_quant_input(input, block_size);
  NVF_CHECK(!(fp8 && global_scale.has_value() && global_scale->defined()), "mxfp8 quantization takes no global scale.");
  const float* gs = check_global_scale(global_scale, input);

  const int64_t cols = input.size(-1);
  const int64_t rows = cols == 0 ? 0 : input.numel() / cols;
  NVF_CHECK(!swizzle_block_scales || input.dim() == 2, "Swizzled block scales need a 2-D input.");
  c10::DeviceGuard guard(input.device());
  void* stream = current_stream(input);

  std::vector<int64_t> qshape(input.sizes().begin(), input.sizes().end());
  if (fp4) qshape.back() = cols / 2;
  torch::Tensor quantized = at::empty(qshape, input.options().dtype(dtype));

  std::vector<int64_t> sshape(input.sizes().begin(), input.sizes().end());
  sshape.back() = cols / block_size;
  if (swizzle_block_scales) sshape = {cutlass_kernels::roundUp(rows, 128), cutlass_kernels::roundUp(cols / block_size, 4)};
  torch::Tensor scales =
      at::empty(sshape, input.options().dtype(fp4 ? at::ScalarType::Float8_e4m3fn : at::ScalarType::Float8_e8m0fnu));

  if (fp4) {
    check_status(nvf_nvfp4_block_quantize(input.data_ptr(), to_nvf_dtype(input.scalar_type()), rows, cols, gs,
                                          swizzle_block_scales ? 1 : 0, quantized.data_ptr(), scales.data_ptr(), stream),
                 "nv_block_quantize");
  } else {
    check_status(nvf_mxfp8_block_quantize(input.data_ptr(), to_nvf_dtype(input.scalar_type()), rows, cols,
                                          swizzle_block_scales ? 1 : 0, quantized.data_ptr(), scales.data_ptr(), stream),
                 "nv_block_quantize");
  }
  return {quantized, scales};
}

std::pair<torch::Tensor, torch::Tensor> nv_grouped_block_quantize(const torch::Tensor& input,
                                                                  const torch::Tensor& input_offsets,
                                                                  const torch::Tensor& output_offsets,
                                                                  const c10::optional<torch::Tensor>& global_scale,
                                                                  int64_t block_size, at::ScalarType dtype) {
  NVF_CHECK(dtype == at::ScalarType::Float4_e2m1fn_x2, "Grouped block quantization produces Float4_e2m1fn(_x2) only.");
  NVF_CHECK(block_size == 16, "Block size must be 16 for nvfp4, got ", block_size);
  check_quant_input(input, block_size);
  NVF_CHECK(input.dim() == 2, "Grouped block quantization only supports 2D input tensors");  // csrc/ops/arith.cpp:2818-2822
  const float* gs = check_global_scale(global_scale, input);
  for (const torch::Tensor& t : {input_offsets, output_offsets}) {
    NVF_CHECK(t.is_cuda() && t.is_contiguous() && t.dim() == 1 && t.scalar_type() == at::ScalarType::Int,
              "Offsets must be contiguous 1-D int32 CUDA tensors.");
  }
  NVF_CHECK_EQ(input_offsets.size(0), output_offsets.size(0), "input_offsets and output_offsets differ in length.");
  const int64_t rows = input.size(0), cols = input.size(1), groups = input_offsets.size(0);
  NVF_CHECK(groups >= 1, "At least one group is required.");

  c10::DeviceGuard guard(input.device());
  void* stream = current_stream(input);
  torch::Tensor quantized = at::empty({rows, cols / 2}, input.options().dtype(dtype));
  // Upper bound of the padded row count, as the reference allocates it (csrc/ops/indexing.cpp:371-432).
  torch::Tensor scales = at::empty({rows + groups * 127, cutlass_kernels::roundUp(cols / 16, 4)},
                                   input.options().dtype(at::ScalarType::Float8_e4m3fn));
  check_status(nvf_nvfp4_grouped_block_quantize(input.data_ptr(), to_nvf_dtype(input.scalar_type()), rows, cols,
                                                static_cast<const int32_t*>(input_offsets.data_ptr()),
                                                static_cast<const int32_t*>(output_offsets.data_ptr()),
                                                static_cast<int>(groups), gs, quantized.data_ptr(), scales.data_ptr(),
                                                stream),
               "nv_grouped_block_quantize");
  return {quantized, scales};
}

std::pair<torch::Tensor, torch::Tensor> silu_mul_nv_grouped_block_quantize(const torch::Tensor& gate, const torch::Tensor& up,
                                                                           const torch::Tensor& input_offsets,
                                                                           const torch::Tensor& output_offsets,
                                                                           const c10::optional<torch::Tensor>& global_scale) {
  check_quant_input(gate, 16);
  check_quant_input(up, 16);
  NVF_CHECK(gate.dim() == 2, "Grouped block quantization only supports 2D input tensors");
  NVF_CHECK(gate.scalar_type() == at::ScalarType::BFloat16 || gate.scalar_type() == at::ScalarType::Half,
            "Expected BFloat16 or Half inputs.");
  NVF_CHECK(up.scalar_type() == gate.scalar_type() && up.sizes() == gate.sizes() && up.device() == gate.device(),
            "gate and up must have the same dtype, shape and device.");
  const float* gs = check_global_scale(global_scale, gate);
  for (const torch::Tensor& t : {input_offsets, output_offsets}) {
    NVF_CHECK(t.is_cuda() && t.is_contiguous() && t.dim() == 1 && t.scalar_type() == at::ScalarType::Int,
              "Offsets must be contiguous 1-D int32 CUDA tensors.");
  }
  NVF_CHECK_EQ(input_offsets.size(0), output_offsets.size(0), "input_offsets and output_offsets differ in length.");
  const int64_t rows = gate.size(0), cols = gate.size(1), groups = input_offsets.size(0);
  NVF_CHECK(groups >= 1, "At least one group is required.");

  c10::DeviceGuard guard(gate.device());
  void* stream = current_stream(gate);
  torch::Tensor quantized = at::empty({rows, cols / 2}, gate.options().dtype(at::ScalarType::Float4_e2m1fn_x2));
  torch::Tensor scales = at::empty({rows + groups * 127, cutlass_kernels::roundUp(cols / 16, 4)},
                                   gate.options().dtype(at::ScalarType::Float8_e4m3fn));
  check_status(nvf_nvfp4_silu_mul_block_quantize(gate.data_ptr(), up.data_ptr(), to_nvf_dtype(gate.scalar_type()), rows, cols,
                                                 static_cast<const int32_t*>(input_offsets.data_ptr()),
                                                 static_cast<const int32_t*>(output_offsets.data_ptr()),
                                                 static_cast<int>(groups), gs, quantized.data_ptr(), scales.data_ptr(), stream),
               "silu_mul_nv_grouped_block_quantize");
  return {quantized, scales};
}

torch::Tensor compute_nvfp4_global_scale(const torch::Tensor& tensor) {
  NVF_CHECK(tensor.is_cuda(), "Expected a CUDA tensor.");
  NVF_CHECK(tensor.is_contiguous(), "Expected a contiguous tensor.");
  const at::ScalarType t = tensor.scalar_type();
  NVF_CHECK(t == at::ScalarType::Float || t == at::ScalarType::BFloat16 || t == at::ScalarType::Half,
            "Expected a Float, BFloat16 or Half tensor.");
  c10::DeviceGuard guard(tensor.device());
  torch::Tensor scale = at::empty({}, tensor.options().dtype(at::ScalarType::Float));
  check_status(nvf_nvfp4_global_scale(tensor.data_ptr(), to_nvf_dtype(t), tensor.numel(), static_cast<float*>(scale.data_ptr()),
                                      current_stream(tensor)),
               "compute_nvfp4_global_scale");
  return scale;
}

torch::Tensor preprocess_grouped_matmul_input_sf(const torch::Tensor& input, const torch::Tensor& input_offsets,
                                                 const torch::Tensor& output_offsets) {
  NVF_CHECK(input.is_cuda() && input.is_contiguous() && input.dim() == 2, "Expected a contiguous 2-D CUDA tensor.");
  for (const torch::Tensor& t : {input_offsets, output_offsets}) {
    NVF_CHECK(t.is_cuda() && t.is_contiguous() && t.dim() == 1 && t.scalar_type() == at::ScalarType::Int,
              "Offsets must be contiguous 1-D int32 CUDA tensors.");
  }
  NVF_CHECK_EQ(input_offsets.size(0), output_offsets.size(0), "input_offsets and output_offsets differ in length.");
  const int64_t rows = input.size(0), cols = input.size(1), groups = input_offsets.size(0);
  NVF_CHECK(groups >= 1, "At least one group is required.");
  const int64_t es = input.element_size();
  NVF_CHECK(es == 1 || es == 2 || es == 4, "Unsupported element size ", es);
  c10::DeviceGuard guard(input.device());
  void* stream = current_stream(input);
  torch::Tensor out = at::empty({rows + groups * 127, cutlass_kernels::roundUp(cols, 4)}, input.options());
  check_status(nvf_preprocess_grouped_matmul_input_sf(input.data_ptr(), static_cast<int>(es), rows, cols,
                                                      static_cast<const int32_t*>(input_offsets.data_ptr()),
                                                      static_cast<const int32_t*>(output_offsets.data_ptr()),
                                                      static_cast<int>(groups), out.data_ptr(), stream),
               "preprocess_grouped_matmul_input_sf");
  return out;
}

}  // namespace block_quantization
}  // namespace nvfuser
