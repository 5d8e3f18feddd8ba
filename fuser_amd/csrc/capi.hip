// extern "C" entry points of libnvf_hip.so: argument checks, then the kernel launchers.
// Shape rules follow the reference's validators (cutlass/nvf_cutlass.cpp:13-234,
// cutlass/group_mm.cu:417-497, cutlass/nvfp4_scaled_group_mm.cu:570-688,
// csrc/device_lower/pass/index.cpp:417-432).
#include "nvf_internal.h"

#include <cstring>
#include <string>

namespace nvf {

static thread_local char g_last_error[512] = "";

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return status;
}

static thread_local bool g_plan = false;
static thread_local std::string g_plan_text;

bool plan_mode() { return g_plan; }

bool note_launch(const char* fmt, ...) {
  if (!g_plan) return false;
  char line[256];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(line, sizeof(line), fmt, ap);
  va_end(ap);
  if (!g_plan_text.empty()) g_plan_text += "; ";
  g_plan_text += line;
  return true;
}

int cu_count() {
  static std::atomic<int> cached{0};
  int n = cached.load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (g_plan) return 256;  // a dry run describes the dispatch on a whole MI355X and touches no device
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    return 256;
  cached.store(n, std::memory_order_relaxed);
  return n;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NVF_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return NVF_OK;
}

static bool dtype16(int d) { return d == NVF_BF16 || d == NVF_F16; }
// The GEMM kernels move operands, scales and results in 16-byte pieces.
template <typename... P>
static bool aligned16(P... ptrs) { return ((reinterpret_cast<uintptr_t>(ptrs) | ...) & 15) == 0; }
#define NVF_REQUIRE_ALIGNED16(...) \
  NVF_REQUIRE(aligned16(__VA_ARGS__), NVF_ERR_INVALID_ARGUMENT, "operand, scale and output buffers must be 16-byte aligned")
static bool dtype_in(int d) { return d == NVF_F32 || d == NVF_BF16 || d == NVF_F16; }

}  // namespace nvf

using namespace nvf;

extern "C" {

const char* nvf_status_string(int status) {
  switch (status) {
    case NVF_OK: return "ok";
    case NVF_ERR_INVALID_ARGUMENT: return "invalid argument";
    case NVF_ERR_UNSUPPORTED_SHAPE: return "unsupported shape";
    case NVF_ERR_LAUNCH: return "kernel launch failed";
    case NVF_ERR_NO_DEVICE: return "no usable device";
  }
  return "unknown status";
}

const char* nvf_last_error(void) { return g_last_error; }

int nvf_get_arch_version(int* version) {
  NVF_REQUIRE(version, NVF_ERR_INVALID_ARGUMENT, "version is NULL");
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return fail(NVF_ERR_NO_DEVICE, "hipGetDevice failed");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return fail(NVF_ERR_NO_DEVICE, "hipGetDeviceProperties failed");
  int v = 0;
  if (sscanf(prop.gcnArchName, "gfx%d", &v) != 1) return fail(NVF_ERR_NO_DEVICE, "unexpected arch name %s", prop.gcnArchName);
  *version = v;
  return NVF_OK;
}

int nvf_get_multiprocessor_count(int* count) {
  NVF_REQUIRE(count, NVF_ERR_INVALID_ARGUMENT, "count is NULL");
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return fail(NVF_ERR_NO_DEVICE, "hipGetDevice failed");
  if (hipDeviceGetAttribute(count, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return fail(NVF_ERR_NO_DEVICE, "hipDeviceGetAttribute failed");
  return NVF_OK;
}

int nvf_nvfp4_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, const float* global_scale,
                             int swizzle, void* out_fp4, void* out_scales, void* stream) {
  NVF_REQUIRE(dtype_in(in_dtype), NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
  NVF_REQUIRE(rows >= 0 && cols >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size (%lld, %lld)", (long long)rows, (long long)cols);
  NVF_REQUIRE(cols % 16 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "the inner dimension %lld is not divisible by the block size 16", (long long)cols);
  if (rows == 0 || cols == 0) return NVF_OK;
  NVF_REQUIRE(in && out_fp4 && out_scales, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_nvfp4_quantize(in, in_dtype, rows, cols, global_scale, swizzle ? 1 : 0, nullptr, nullptr, 1, out_fp4,
                               out_scales, static_cast<hipStream_t>(stream));
}

int nvf_nvfp4_grouped_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols,
                                     const int32_t* input_offsets, const int32_t* output_offsets, int groups,
                                     const float* global_scale, void* out_fp4, void* out_scales, void* stream) {
  NVF_REQUIRE(dtype_in(in_dtype), NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
  NVF_REQUIRE(rows >= 0 && cols >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size (%lld, %lld)", (long long)rows, (long long)cols);
  NVF_REQUIRE(groups >= 1, NVF_ERR_INVALID_ARGUMENT, "groups must be >= 1, got %d", groups);
  NVF_REQUIRE(cols % 16 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "the inner dimension %lld is not divisible by the block size 16", (long long)cols);
  if (rows == 0 || cols == 0) return NVF_OK;
  NVF_REQUIRE(in && out_fp4 && out_scales && input_offsets && output_offsets, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_nvfp4_quantize(in, in_dtype, rows, cols, global_scale, 2, input_offsets, output_offsets, groups, out_fp4,
                               out_scales, static_cast<hipStream_t>(stream));
}

int nvf_nvfp4_silu_mul_block_quantize(const void* gate, const void* up, int in_dtype, int64_t rows, int64_t cols,
                                      const int32_t* input_offsets, const int32_t* output_offsets, int groups,
                                      const float* global_scale, void* out_fp4, void* out_scales, void* stream) {
  NVF_REQUIRE(in_dtype == NVF_BF16 || in_dtype == NVF_F16, NVF_ERR_INVALID_ARGUMENT, "inputs must be bf16 or f16, got dtype %d", in_dtype);
  NVF_REQUIRE(rows >= 0 && cols >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size (%lld, %lld)", (long long)rows, (long long)cols);
  NVF_REQUIRE(cols % 16 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "the inner dimension %lld is not divisible by the block size 16", (long long)cols);
  const bool grouped = input_offsets != nullptr;
  if (grouped) NVF_REQUIRE(groups >= 1, NVF_ERR_INVALID_ARGUMENT, "groups must be >= 1, got %d", groups);
  if (rows == 0 || cols == 0) return NVF_OK;
  NVF_REQUIRE(gate && up && out_fp4 && out_scales && (!grouped || output_offsets), NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_nvfp4_silu_mul_quantize(gate, up, in_dtype, rows, cols, global_scale, grouped ? 2 : 1, input_offsets, output_offsets,
                                        grouped ? groups : 1, out_fp4, out_scales, static_cast<hipStream_t>(stream));
}

int nvf_nvfp4_global_scale(const void* in, int in_dtype, int64_t numel, float* out_scale, void* stream) {
  NVF_REQUIRE(dtype_in(in_dtype), NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
  NVF_REQUIRE(numel >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size %lld", (long long)numel);
  NVF_REQUIRE(out_scale && (in || numel == 0), NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_nvfp4_global_scale(in, in_dtype, numel, out_scale, static_cast<hipStream_t>(stream));
}

int nvf_preprocess_grouped_matmul_input_sf(const void* in, int elem_size, int64_t rows, int64_t cols,
                                           const int32_t* input_offsets, const int32_t* output_offsets, int groups,
                                           void* out, void* stream) {
  NVF_REQUIRE(rows >= 0 && cols >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size (%lld, %lld)", (long long)rows, (long long)cols);
  NVF_REQUIRE(groups >= 1, NVF_ERR_INVALID_ARGUMENT, "groups must be >= 1, got %d", groups);
  NVF_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4, NVF_ERR_INVALID_ARGUMENT, "element size %d is not 1, 2 or 4", elem_size);
  if (rows == 0 || cols == 0) return NVF_OK;
  NVF_REQUIRE(in && out && input_offsets && output_offsets, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_preprocess_sf(in, elem_size, rows, cols, input_offsets, output_offsets, groups, out,
                              static_cast<hipStream_t>(stream));
}

int nvf_mxfp8_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, int swizzle, void* out_fp8,
                             void* out_scales, void* stream) {
  NVF_REQUIRE(dtype_in(in_dtype), NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
  NVF_REQUIRE(rows >= 0 && cols >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size (%lld, %lld)", (long long)rows, (long long)cols);
  NVF_REQUIRE(cols % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "the inner dimension %lld is not divisible by the block size 32", (long long)cols);
  if (rows == 0 || cols == 0) return NVF_OK;
  NVF_REQUIRE(in && out_fp8 && out_scales, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_mxfp8_quantize(in, in_dtype, rows, cols, swizzle ? 1 : 0, out_fp8, out_scales,
                               static_cast<hipStream_t>(stream));
}

static int cast_common(int kind, const float* in, int64_t n, uint8_t* out, void* stream) {
  NVF_REQUIRE(n >= 0, NVF_ERR_INVALID_ARGUMENT, "negative count %lld", (long long)n);
  if (n == 0) return NVF_OK;
  NVF_REQUIRE(in && out, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_cast(kind, in, n, out, static_cast<hipStream_t>(stream));
}
int nvf_cast_f32_to_e2m1(const float* in, int64_t n, uint8_t* out, void* stream) { return cast_common(0, in, n, out, stream); }
int nvf_cast_f32_to_e4m3(const float* in, int64_t n, uint8_t* out, void* stream) { return cast_common(1, in, n, out, stream); }
int nvf_cast_f32_to_e8m0(const float* in, int64_t n, uint8_t* out, void* stream) { return cast_common(2, in, n, out, stream); }

// argument checks of nvfp4_scaled_mm shared by its three entry points; *empty is set for a call without output
static int check_nvfp4_scaled_mm(const void* a, const void* b, const void* scales_a, const void* scales_b, const float* alpha, void* out,
                                 int64_t m, int64_t n, int64_t k, int out_dtype, int64_t workspace_bytes, bool* empty) {
  *empty = true;
  NVF_REQUIRE(dtype16(out_dtype), NVF_ERR_INVALID_ARGUMENT, "output dtype must be bf16 or f16, got %d", out_dtype);
  NVF_REQUIRE(m >= 0 && n >= 0 && k >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size");
  NVF_REQUIRE(k % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The K dimension %lld is not divisible by 32", (long long)k);
  NVF_REQUIRE(n % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The N dimension %lld is not divisible by 32", (long long)n);
  NVF_REQUIRE(workspace_bytes >= 0, NVF_ERR_INVALID_ARGUMENT, "negative workspace size");
  if (m == 0 || n == 0) return NVF_OK;
  NVF_REQUIRE(a && b && scales_a && scales_b && alpha && out, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  NVF_REQUIRE_ALIGNED16(a, b, scales_a, scales_b, out);
  *empty = false;
  return NVF_OK;
}

int nvf_nvfp4_scaled_mm_ws(const void* a, const void* b, const void* scales_a, const void* scales_b, const float* alpha,
                           void* out, int64_t m, int64_t n, int64_t k, int out_dtype, void* workspace,
                           int64_t workspace_bytes, void* stream) {
  bool empty;
  if (const int rc = check_nvfp4_scaled_mm(a, b, scales_a, scales_b, alpha, out, m, n, k, out_dtype, workspace_bytes, &empty)) return rc;
  if (empty) return NVF_OK;
  Gemm16Args g{a, b, scales_a, scales_b, alpha, out, nullptr, nullptr, nullptr, 1, m, n, k, out_dtype};
  if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {  // fp32x4 accesses
    g.workspace = workspace;
    g.workspace_bytes = workspace_bytes;
  }
  return launch_gemm16(0, g, static_cast<hipStream_t>(stream));
}

int nvf_nvfp4_scaled_mm(const void* a, const void* b, const void* scales_a, const void* scales_b, const float* alpha,
                        void* out, int64_t m, int64_t n, int64_t k, int out_dtype, void* stream) {
  return nvf_nvfp4_scaled_mm_ws(a, b, scales_a, scales_b, alpha, out, m, n, k, out_dtype, nullptr, 0, stream);
}

int64_t nvf_nvfp4_scaled_mm_workspace_bytes(int64_t m, int64_t n, int64_t k) { return nvfp4_gemm_workspace_bytes(m, n, k); }

int nvf_nvfp4_scaled_mm_static_ws(const void* a, const void* b, const void* scales_a, const void* scales_b, const float* alpha,
                                  void* out, int64_t m, int64_t n, int64_t k, int out_dtype, void* stream) {
  // the arguments first: an invalid call must not touch the device
  bool empty;
  if (const int rc = check_nvfp4_scaled_mm(a, b, scales_a, scales_b, alpha, out, m, n, k, out_dtype, 0, &empty)) return rc;
  if (empty) return NVF_OK;
  const int64_t need = nvfp4_gemm_workspace_bytes(m, n, k);
  NVF_REQUIRE(need <= kStaticScratchBytes, NVF_ERR_UNSUPPORTED_SHAPE,
              "M = %lld, N = %lld, K = %lld needs %lld bytes of scratch memory, the library's static scratch holds %lld: use "
              "nvf_nvfp4_scaled_mm_ws with a workspace of the caller's, or nvf_nvfp4_scaled_mm",
              (long long)m, (long long)n, (long long)k, (long long)need, (long long)kStaticScratchBytes);
  void* ws = nullptr;
  if (need > 0) {
    if (const int rc = static_scratch(&ws)) return rc;
  }
  return nvf_nvfp4_scaled_mm_ws(a, b, scales_a, scales_b, alpha, out, m, n, k, out_dtype, ws, ws ? need : 0, stream);
}

int nvf_nvfp4_scaled_mm_blockscale(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                   const float* alpha, const float* global_normconst, void* out_fp4, void* out_scales,
                                   float* workspace, int64_t m, int64_t n, int64_t k, void* stream) {
  NVF_REQUIRE(m >= 0 && n >= 0 && k >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size");
  NVF_REQUIRE(k % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The K dimension %lld is not divisible by 32", (long long)k);
  NVF_REQUIRE(n % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The N dimension %lld is not divisible by 32", (long long)n);
  if (m == 0 || n == 0) return NVF_OK;
  NVF_REQUIRE(a && b && scales_a && scales_b && alpha && global_normconst && out_fp4 && out_scales, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  NVF_REQUIRE_ALIGNED16(a, b, scales_a, scales_b, out_fp4, out_scales, workspace);
  Gemm16Args g{a, b, scales_a, scales_b, alpha, out_fp4, nullptr, nullptr, nullptr, 1, m, n, k, kDtypeFp4BlockScaled};
  g.out_sf = out_scales;
  g.gnorm = global_normconst;
  const int rc = launch_gemm16(0, g, static_cast<hipStream_t>(stream));
  if (rc != NVF_OK || workspace == nullptr) return rc;
  // the optional dump of the fp32 product: the same kernel once more, with the accumulators written out as they are
  Gemm16Args d{a, b, scales_a, scales_b, alpha, workspace, nullptr, nullptr, nullptr, 1, m, n, k, NVF_F32};
  return launch_gemm16(0, d, static_cast<hipStream_t>(stream));
}

int nvf_mxfp8_scaled_mm(const void* a, const void* b, const void* scales_a, const void* scales_b, const float* alpha,
                        void* out, int64_t m, int64_t n, int64_t k, int out_dtype, void* stream) {
  NVF_REQUIRE(dtype16(out_dtype), NVF_ERR_INVALID_ARGUMENT, "output dtype must be bf16 or f16, got %d", out_dtype);
  NVF_REQUIRE(m >= 0 && n >= 0 && k >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size");
  NVF_REQUIRE(k % 16 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The K dimension %lld is not divisible by 16", (long long)k);
  NVF_REQUIRE(n % 16 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The N dimension %lld is not divisible by 16", (long long)n);
  NVF_REQUIRE(k % 32 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The K dimension %lld is not a whole number of 32-element scale blocks", (long long)k);
  if (m == 0 || n == 0) return NVF_OK;
  NVF_REQUIRE(a && b && scales_a && scales_b && alpha && out, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  NVF_REQUIRE_ALIGNED16(a, b, scales_a, scales_b, out);
  return launch_mxfp8_gemm(a, b, scales_a, scales_b, alpha, out, m, n, k, out_dtype, static_cast<hipStream_t>(stream));
}

int nvf_grouped_mm(const void* a, const void* b, void* out, const int32_t* problem_sizes, const int32_t* expert_offsets,
                   int groups, int64_t m, int64_t n, int64_t k, int ab_dtype, void* stream) {
  NVF_REQUIRE(dtype16(ab_dtype), NVF_ERR_INVALID_ARGUMENT, "Expected BFloat16 or Half operands, got dtype %d", ab_dtype);
  NVF_REQUIRE(m >= 0 && n >= 0 && k >= 0 && groups >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size");
  NVF_REQUIRE(k % 8 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The inner dimension %lld of the operands is not a multiple of 8", (long long)k);
  NVF_REQUIRE(n % 8 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The inner dimension %lld of the output tensor is not a multiple of 8", (long long)n);
  if (m == 0 || n == 0 || groups == 0) return NVF_OK;
  NVF_REQUIRE(a && b && out && problem_sizes && expert_offsets, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  NVF_REQUIRE_ALIGNED16(a, b, out);
  Gemm16Args g{a, b, nullptr, nullptr, nullptr, out, problem_sizes, expert_offsets, nullptr, groups, m, n, k, ab_dtype};
  return launch_gemm16(2, g, static_cast<hipStream_t>(stream));
}

int nvf_nvfp4_scaled_grouped_mm(const void* a, const void* b, const void* a_scales, const void* b_scales,
                                const float* alphas, void* out, const int32_t* problem_sizes,
                                const int32_t* expert_offsets, const int32_t* sf_offsets, int groups, int64_t m,
                                int64_t n, int64_t k, int out_dtype, void* stream) {
  NVF_REQUIRE(dtype16(out_dtype), NVF_ERR_INVALID_ARGUMENT, "output dtype must be bf16 or f16, got %d", out_dtype);
  NVF_REQUIRE(m >= 0 && n >= 0 && k >= 0 && groups >= 0, NVF_ERR_INVALID_ARGUMENT, "negative size");
  NVF_REQUIRE(k % 64 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The packed inner dimension %lld of the operands is not a multiple of 32", (long long)(k / 2));
  NVF_REQUIRE(n % 8 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "The inner dimension %lld of the output tensor is not a multiple of 8", (long long)n);
  NVF_REQUIRE(n % 128 == 0, NVF_ERR_UNSUPPORTED_SHAPE, "N = %lld: every expert's scale slab must be whole 128x4 tiles (N %% 128 == 0)", (long long)n);
  if (m == 0 || n == 0 || groups == 0) return NVF_OK;
  NVF_REQUIRE(a && b && a_scales && b_scales && alphas && out && problem_sizes && expert_offsets && sf_offsets,
              NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  NVF_REQUIRE_ALIGNED16(a, b, a_scales, b_scales, out);
  Gemm16Args g{a, b, a_scales, b_scales, alphas, out, problem_sizes, expert_offsets, sf_offsets, groups, m, n, k, out_dtype};
  return launch_gemm16(1, g, static_cast<hipStream_t>(stream));
}

int nvf_selftest_fast_division(uint32_t* result4, void* stream) {
  NVF_REQUIRE(result4, NVF_ERR_INVALID_ARGUMENT, "NULL buffer");
  return launch_division_selftest(result4, static_cast<hipStream_t>(stream));
}

int nvf_describe_dispatch(const char* op, int64_t m, int64_t n, int64_t k, int groups, int dtype, int64_t workspace_bytes,
                          char* text, int64_t text_bytes) {
  NVF_REQUIRE(op && text && text_bytes > 0, NVF_ERR_INVALID_ARGUMENT, "NULL argument");
  // never dereferenced: in plan mode every launcher returns before it touches the device
  void* const x = reinterpret_cast<void*>(uintptr_t{256});
  const float* const f = static_cast<const float*>(x);
  const int32_t* const i = static_cast<const int32_t*>(x);
  g_plan = true;
  g_plan_text.clear();
  int rc;
  const std::string name(op);
  if (name == "nvfp4_scaled_mm") rc = nvf_nvfp4_scaled_mm_ws(x, x, x, x, f, x, m, n, k, dtype, workspace_bytes > 0 ? x : nullptr, workspace_bytes, nullptr);
  else if (name == "nvfp4_scaled_mm_blockscale") rc = nvf_nvfp4_scaled_mm_blockscale(x, x, x, x, f, f, x, x, workspace_bytes > 0 ? static_cast<float*>(x) : nullptr, m, n, k, nullptr);
  else if (name == "mxfp8_scaled_mm") rc = nvf_mxfp8_scaled_mm(x, x, x, x, f, x, m, n, k, dtype, nullptr);
  else if (name == "grouped_mm") rc = nvf_grouped_mm(x, x, x, i, i, groups, m, n, k, dtype, nullptr);
  else if (name == "nvfp4_scaled_grouped_mm") rc = nvf_nvfp4_scaled_grouped_mm(x, x, x, x, f, x, i, i, i, groups, m, n, k, dtype, nullptr);
  else rc = fail(NVF_ERR_INVALID_ARGUMENT, "unknown op %s", op);
  g_plan = false;
  snprintf(text, (size_t)text_bytes, "%s", g_plan_text.c_str());
  return rc;
}

}  // extern "C"
