// Internal helpers shared by the HIP translation units of libnvf_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "nvf_hip.h"

namespace nvf {

// Records a message for nvf_last_error() and returns `status`.
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Checks the launch that was just issued on the calling thread.
int check_launch(const char* what);

// Dry run of a dispatch (nvf_describe_dispatch): while the calling thread is in plan mode, launchers
// record the kernel they would start and return before any HIP call.  note_launch() returns true in that mode.
bool plan_mode();
bool note_launch(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Compute units of the current device, cached per process (256 when no device can be asked, as in a dry run).
int cu_count();

// Raises a kernel's dynamic LDS limit on the current device, once per device (`done`: one bit per device id;
// the attribute call is idempotent, so two threads that both find the bit clear do no harm).
inline int allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(NVF_ERR_NO_DEVICE, "hipGetDevice failed");
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return NVF_OK;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(NVF_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  done.fetch_or(bit, std::memory_order_release);
  return NVF_OK;
}

inline int64_t ceil_div(int64_t x, int64_t y) { return (x + y - 1) / y; }
inline int64_t round_up(int64_t x, int64_t y) { return ceil_div(x, y) * y; }

#define NVF_REQUIRE(cond, status, ...) \
  do {                                 \
    if (!(cond)) return ::nvf::fail((status), __VA_ARGS__); \
  } while (0)

// ---- launchers implemented in the kernel translation units ----
int launch_nvfp4_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, const float* gs, int layout,
                          const int32_t* in_off, const int32_t* out_off, int groups, void* out_fp4, void* out_sf,
                          hipStream_t stream);
// input = silu(gate) * up evaluated in the inputs' 16-bit type (bf16 / f16 only)
int launch_nvfp4_silu_mul_quantize(const void* gate, const void* up, int in_dtype, int64_t rows, int64_t cols, const float* gs,
                                   int layout, const int32_t* in_off, const int32_t* out_off, int groups, void* out_fp4,
                                   void* out_sf, hipStream_t stream);
// out[0] = 448 * 6 / max|in| (1 if the tensor is all zero)
int launch_nvfp4_global_scale(const void* in, int in_dtype, int64_t n, float* out, hipStream_t stream);
int launch_preprocess_sf(const void* in, int elem_size, int64_t rows, int64_t cols, const int32_t* in_off,
                         const int32_t* out_off, int groups, void* out, hipStream_t stream);
int launch_mxfp8_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, int swizzle, void* out_fp8,
                          void* out_sf, hipStream_t stream);
int launch_cast(int kind, const float* in, int64_t n, uint8_t* out, hipStream_t stream);
int launch_division_selftest(uint32_t* out4, hipStream_t stream);

// op: 0 dense NVFP4, 1 grouped NVFP4, 2 grouped bf16/f16
struct Gemm16Args {
  const void* a;
  const void* b;
  const void* sfa;
  const void* sfb;
  const float* alpha;  // dense: scalar; grouped NVFP4: [groups]; grouped 16-bit: nullptr
  void* out;
  const int32_t* problem_sizes;
  const int32_t* expert_offsets;
  const int32_t* sf_offsets;
  int groups;
  int64_t m, n, k;
  int dtype;  // out dtype (NVFP4 ops) or in/out dtype (grouped_mm)
  void* workspace = nullptr;  // dense NVFP4: optional scratch for a split of K (nvfp4_gemm_workspace_bytes)
  int64_t workspace_bytes = 0;
  // dtype == kDtypeFp4BlockScaled (dense NVFP4 only): out = packed e2m1 [m, n/2], out_sf = its e4m3 scales (128x4
  // layout), gnorm = the result's global scale on the device
  void* out_sf = nullptr;
  const float* gnorm = nullptr;
  int64_t ldc = 0;  // dense NVFP4, 16-bit result: elements between rows of the result (0: n); set by the N cut's launches
};
constexpr int kDtypeFp4BlockScaled = 100;  // internal result type code of launch_gemm16, next to nvf_dtype
int launch_gemm16(int op, const Gemm16Args& args, hipStream_t stream);
// scratch bytes with which the dense NVFP4 GEMM of this shape runs faster (0: none needed)
int64_t nvfp4_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k);
// the library's own scratch array (one per device, no allocation): its size and its address on the current device
constexpr int64_t kStaticScratchBytes = (int64_t)32 << 20;
int static_scratch(void** ptr);
int launch_mxfp8_gemm(const void* a, const void* b, const void* sfa, const void* sfb, const float* alpha, void* out,
                      int64_t m, int64_t n, int64_t k, int out_dtype, hipStream_t stream);

}  // namespace nvf

// ------------------------------------------------------------------------------------------------
// Device-side narrow-float codecs (gfx950).
// ------------------------------------------------------------------------------------------------
#if defined(__HIPCC__)
namespace nvf {

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __float_as_uint(f); }

// 128x4 scale layout: byte offset of (row, col) in a buffer with `padded_cols` columns.
__device__ __forceinline__ int64_t swizzle_128x4(int64_t row, int64_t col, int64_t padded_cols) {
  return (row >> 7) * (padded_cols << 7) + ((col >> 2) << 9) + ((row & 31) << 4) + (((row >> 5) & 3) << 2) + (col & 3);
}

// e4m3fn decode, exact (hardware convert, verified for all 256 codes).
__device__ __forceinline__ float e4m3_to_f32(uint32_t code) { return __builtin_amdgcn_cvt_f32_fp8((int)code, 0); }

// e4m3fn encode, round-to-nearest-even, saturating to +-448, NaN -> 0x7F.
// The hardware convert rounds correctly but turns overflow into NaN, hence the clamp.
__device__ __forceinline__ uint32_t f32_to_e4m3_satfinite(float x) {
  if (x != x) return 0x7fu;
  float c = fminf(fmaxf(x, -448.0f), 448.0f);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xffu;
}

// e2m1 encode of two values into one byte (first value in the low nibble), RNE, saturating to
// +-6.  The hardware convert does exactly that for every non-NaN input; NaN is mapped to +6.
__device__ __forceinline__ uint32_t f32x2_to_e2m1_byte(float lo, float hi) {
  uint32_t r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, lo, hi, 1.0f, 0) & 0xffu;
  if (lo != lo) r = (r & 0xf0u) | 0x07u;
  if (hi != hi) r = (r & 0x0fu) | 0x70u;
  return r;
}

// ue8m0 encode, round toward +inf (smallest power of two >= x), saturating; NaN -> 0xFF;
// zero and negative inputs -> 0.
__device__ __forceinline__ uint32_t f32_to_e8m0_rp(float x) {
  uint32_t b = f32_to_bits(x);
  if (x != x) return 0xffu;
  if ((b >> 31) || b == 0) return 0u;
  uint32_t e = b >> 23, m = b & 0x7fffffu;
  if (e == 255) return 0xfeu;
  if (e == 0) return m > 0x400000u ? 1u : 0u;  // denormal: 2^-127 is e8m0 code 0
  uint32_t r = e + (m != 0);
  return r > 254u ? 254u : r;
}

// true when the 3-instruction divisions below give the result of the true division for this operand: biased
// exponent in [2, 250], or +0 (amax / 6 = 0 exactly; 1 / 0: v_rcp gives +Inf, the correction step NaN, and
// fminf(NaN, FLT_MAX) = FLT_MAX = fminf(+Inf, FLT_MAX))
__device__ __forceinline__ bool fast_div_ok(float v) {
  const uint32_t b = f32_to_bits(v);
  return ((b >> 23) & 0xffu) - 2u <= 248u || b == 0u;
}
__device__ __forceinline__ float fast_div6(float m) {
  const float r6 = 0x1.555556p-3f;  // RN(1/6)
  const float q0 = m * r6;
  return __builtin_fmaf(__builtin_fmaf(-6.0f, q0, m), r6, q0);
}
__device__ __forceinline__ float fast_rcp(float v) {
  const float r0 = __builtin_amdgcn_rcpf(v);
  return __builtin_fmaf(__builtin_fmaf(-v, r0, 1.0f), r0, r0);
}

// NVFP4 block scale from the block's amax m (>= 0 or -inf), in the operation order of
// runtime/block_quantization_kernels.cu:224-239.  Returns the e4m3 code that is stored and sets r, the factor the
// block's values are multiplied with ahead of the e2m1 cast.  gs: encode scale (use_gs), decode = 1.0f / gs.
// Must be called by all lanes of the wavefront: if any `active` lane holds an operand outside the range of the
// 3-instruction divisions, the wavefront redoes the arithmetic with true divisions.
__device__ __forceinline__ uint32_t nvfp4_block_scale(float m, bool use_gs, float gs, float decode, bool active, float& r) {
  float s = fast_div6(m);                 // :224  amax / 6
  if (use_gs) s = s * gs;                 // :226
  s = fminf(s, 3.402823466e+38f);         // :228
  uint32_t q8 = f32_to_e4m3_satfinite(s); // :230
  float sf = e4m3_to_f32(q8);             // :233
  float den = use_gs ? sf * decode : sf;  // :237 / :239
  r = fminf(fast_rcp(den), 3.402823466e+38f);
  if (__builtin_amdgcn_ballot_w64(active && (!fast_div_ok(m) || !fast_div_ok(den))) != 0) {
    s = m / 6.0f;
    if (use_gs) s = s * gs;
    s = fminf(s, 3.402823466e+38f);
    q8 = f32_to_e4m3_satfinite(s);
    sf = e4m3_to_f32(q8);
    den = use_gs ? sf * decode : sf;
    r = fminf(1.0f / den, 3.402823466e+38f);
  }
  return q8;
}

}  // namespace nvf
#endif
