// Python module fuser_amd._C: submodule `nvf_cutlass` with the same six callables and argument
// lists as the reference's nvfuser_direct.nvf_cutlass (python/python_direct/cutlass.cpp:17-117),
// plus eager entry points for the block quantizers.
#include <torch/extension.h>

#include "callers.h"
#include "nvf_cutlass.h"

namespace py = pybind11;
namespace ck = nvfuser::cutlass_kernels;
namespace bq = nvfuser::block_quantization;
namespace cl = nvfuser::callers;

PYBIND11_MODULE(_C, m) {
  m.doc() = "MI355X implementation of nvFuser's quantized-GEMM path";
  py::module_ cutlass = m.def_submodule("nvf_cutlass", "Block-scaled and grouped GEMMs (MI355X).");

  // As in the reference bindings, the dense ops do not expose skip_checks.
  cutlass.def(
      "mxfp8_scaled_mm",
      [](const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
         const torch::Tensor& alpha, at::ScalarType out_dtype) { return ck::mxfp8_scaled_mm(a, b, scales_a, scales_b, alpha, out_dtype); },
      "mxfp8_scaled_mm(a, b, scales_a, scales_b, alpha, out_dtype) -> Tensor");
  cutlass.def(
      "nvfp4_scaled_mm",
      [](const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
         const torch::Tensor& alpha, at::ScalarType out_dtype) { return ck::nvfp4_scaled_mm(a, b, scales_a, scales_b, alpha, out_dtype); },
      "nvfp4_scaled_mm(a, b, scales_a, scales_b, alpha, out_dtype) -> Tensor");
  cutlass.def(
      "nvfp4_scaled_mm_blockscale",
      [](const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& scales_a, const torch::Tensor& scales_b,
         const torch::Tensor& alpha, const torch::Tensor& global_normconst) -> py::tuple {
        auto r = ck::nvfp4_scaled_mm_blockscale(a, b, scales_a, scales_b, alpha, global_normconst);
        return py::make_tuple(r.first, r.second);
      },
      "nvfp4_scaled_mm_blockscale(a, b, scales_a, scales_b, alpha, global_normconst) -> (out_nvfp4, blockscale)");
  cutlass.def("grouped_mm", &ck::grouped_mm,
              "grouped_mm(a, b, ab_strides, c_strides, problem_sizes, expert_offsets) -> Tensor");
  cutlass.def("nvfp4_scaled_grouped_mm", &ck::nvfp4_scaled_grouped_mm,
              "nvfp4_scaled_grouped_mm(a, b, a_blockscale, b_blockscale, alphas, ab_strides, c_strides, "
              "problem_sizes, expert_offsets, sf_offsets, out_dtype) -> Tensor");
  cutlass.def(
      "validate_inputs_nvfp4_scaled_mm",
      [](const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& sa, const torch::Tensor& sb,
         const torch::Tensor& alpha, bool skip_checks) { return ck::validateInputsNvfp4ScaledMm(a, b, sa, sb, alpha, skip_checks); },
      py::arg("a"), py::arg("b"), py::arg("scales_a"), py::arg("scales_b"), py::arg("alpha"), py::arg("skip_checks") = false);
  cutlass.def(
      "validate_inputs_mxfp8_scaled_mm",
      [](const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& sa, const torch::Tensor& sb,
         const torch::Tensor& alpha, bool skip_checks) { return ck::validateInputsMxFp8ScaledMm(a, b, sa, sb, alpha, skip_checks); },
      py::arg("a"), py::arg("b"), py::arg("scales_a"), py::arg("scales_b"), py::arg("alpha"), py::arg("skip_checks") = false);
  cutlass.def("get_sm_version", &ck::getSMVersion);
  cutlass.def("get_multiprocessor_count", &ck::getMultiProcessorCount);

  m.def(
      "nv_block_quantize",
      [](const torch::Tensor& input, const c10::optional<torch::Tensor>& global_scale, bool swizzle_block_scales,
         int64_t block_size, at::ScalarType dtype) {
        auto r = bq::nv_block_quantize(input, global_scale, swizzle_block_scales, block_size, dtype);
        return py::make_tuple(r.first, r.second);
      },
      py::arg("input"), py::arg("global_scale") = py::none(), py::arg("swizzle_block_scales") = false,
      py::arg("block_size") = 16, py::arg("dtype") = at::ScalarType::Float4_e2m1fn_x2);
  m.def(
      "nv_grouped_block_quantize",
      [](const torch::Tensor& input, const torch::Tensor& input_offsets, const torch::Tensor& output_offsets,
         const c10::optional<torch::Tensor>& global_scale, int64_t block_size, at::ScalarType dtype) {
        auto r = bq::nv_grouped_block_quantize(input, input_offsets, output_offsets, global_scale, block_size, dtype);
        return py::make_tuple(r.first, r.second);
      },
      py::arg("input"), py::arg("input_offsets"), py::arg("output_offsets"), py::arg("global_scale") = py::none(),
      py::arg("block_size") = 16, py::arg("dtype") = at::ScalarType::Float4_e2m1fn_x2);
  m.def("preprocess_grouped_matmul_input_sf", &bq::preprocess_grouped_matmul_input_sf, py::arg("input"),
        py::arg("input_offsets"), py::arg("output_offsets"));
  m.def(
      "silu_mul_nv_grouped_block_quantize",
      [](const torch::Tensor& gate, const torch::Tensor& up, const torch::Tensor& input_offsets,
         const torch::Tensor& output_offsets, const c10::optional<torch::Tensor>& global_scale) {
        auto r = bq::silu_mul_nv_grouped_block_quantize(gate, up, input_offsets, output_offsets, global_scale);
        return py::make_tuple(r.first, r.second);
      },
      py::arg("gate"), py::arg("up"), py::arg("input_offsets"), py::arg("output_offsets"), py::arg("global_scale") = py::none());
  m.def("compute_nvfp4_global_scale", &bq::compute_nvfp4_global_scale, py::arg("tensor"));

  // Conventions of the reference's expression nodes around the kernels (csrc/ir/composite_nodes.cpp).
  // A kernel branch that does not apply returns None: the caller falls back.
  py::module_ callers = m.def_submodule("callers", "ScaledMmaOp / GroupedMmaOp / CutlassNvfp4GroupedMmaOp conventions.");
  auto or_none = [](const torch::Tensor& t) -> py::object { return t.defined() ? py::cast(t) : py::none(); };
  callers.def(
      "scaled_mma",
      [or_none](const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& scale1, const torch::Tensor& scale2,
                const c10::optional<torch::Tensor>& alpha, const c10::optional<torch::Tensor>& bias,
                const c10::optional<torch::Tensor>& beta, at::ScalarType out_dtype) {
        return or_none(cl::scaled_mma(mat1, mat2, scale1, scale2, alpha, bias, beta, out_dtype));
      },
      py::arg("mat1"), py::arg("mat2"), py::arg("scale1"), py::arg("scale2"), py::arg("alpha") = py::none(),
      py::arg("bias") = py::none(), py::arg("beta") = py::none(), py::arg("out_dtype") = at::ScalarType::BFloat16);
  callers.def(
      "grouped_mma_arguments",
      [](const torch::Tensor& offsets, int64_t n, int64_t k) {
        auto r = cl::grouped_mma_arguments(offsets, n, k);
        return py::make_tuple(r.problem_sizes, r.expert_offsets, r.ab_strides, r.c_strides);
      },
      py::arg("offsets"), py::arg("n"), py::arg("k"));
  callers.def(
      "grouped_mma",
      [or_none](const torch::Tensor& mat1, const torch::Tensor& mat2, const torch::Tensor& offsets) {
        return or_none(cl::grouped_mma(mat1, mat2, offsets));
      },
      py::arg("mat1"), py::arg("mat2"), py::arg("offsets"));
  callers.def("cutlass_nvfp4_grouped_mma", &cl::cutlass_nvfp4_grouped_mma, py::arg("mat1"), py::arg("mat2"),
              py::arg("scale1"), py::arg("scale2"), py::arg("alpha"), py::arg("problem_sizes"), py::arg("expert_offsets"),
              py::arg("sf_offsets"), py::arg("out_dtype") = at::ScalarType::BFloat16);
}
