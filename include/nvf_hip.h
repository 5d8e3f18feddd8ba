/*
 * C ABI of libnvf_hip.so: the MI355X (gfx950) kernels behind nvFuser's `nvf_cutlass` ops and
 * the NVFP4 / MXFP8 block quantizers.
 *
 * Plain pointers and sizes only: every pointer is a DEVICE pointer unless stated otherwise,
 * `stream` is a hipStream_t passed as void* (NULL = the default stream), all launches are
 * asynchronous on that stream and no entry point allocates, frees or synchronises.
 * Every function returns NVF_OK (0) or a negative nvf_status; nvf_status_string() names it and
 * nvf_last_error() gives the detailed message of the calling thread's last failure.
 *
 * Data formats (identical to the reference's):
 *   packed fp4   1 byte = 2 e2m1 codes, element 2j in the low nibble      runtime/casts.cu:1081-1088
 *   NVFP4        e2m1 payload + one e4m3 scale per 16 K-elements + fp32   cutlass/nvf_cutlass.h:52-75
 *   MXFP8        e4m3 payload + one e8m0 scale per 32 K-elements          cutlass/nvf_cutlass.h:103-126
 *   128x4 layout scale (r,c) of an [R,C] scale matrix lives at byte
 *                ((r/128)*ceil(C/4) + c/4)*512 + (r%32)*16 + ((r%128)/32)*4 + c%4
 *                of a [roundUp(R,128), roundUp(C,4)] buffer       runtime/block_quantization_kernels.cu:15-57
 */
#ifndef NVF_HIP_H_
#define NVF_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NVF_API __attribute__((visibility("default")))

typedef enum nvf_status {
  NVF_OK = 0,
  NVF_ERR_INVALID_ARGUMENT = -1, /* NULL pointer, negative size, unknown dtype */
  NVF_ERR_UNSUPPORTED_SHAPE = -2, /* alignment rule of the op violated */
  NVF_ERR_LAUNCH = -3,           /* the HIP runtime rejected the launch */
  NVF_ERR_NO_DEVICE = -4         /* no gfx950 device is current */
} nvf_status;

typedef enum nvf_dtype {
  NVF_F32 = 0,
  NVF_BF16 = 1,
  NVF_F16 = 2
} nvf_dtype;

NVF_API const char* nvf_status_string(int status);
NVF_API const char* nvf_last_error(void);

/* cutlass/cutlass_utils.cpp:13-23 getSMVersion -> here the gfx target number (950). */
NVF_API int nvf_get_arch_version(int* version);
/* cutlass/cutlass_utils.cpp:25-41 getMultiProcessorCount -> compute units of the current device. */
NVF_API int nvf_get_multiprocessor_count(int* count);

/* ----------------------------------------------------------------------------------------------
 * Block quantizers
 * -------------------------------------------------------------------------------------------- */

/* runtime/block_quantization_kernels.cu:194-319 bq::block_quantize_to_nvfp4
 * (graph op nv_block_quantize, python/python_direct/ops.cpp:3521-3558).
 *   in            [rows, cols] row-major, in_dtype in {F32,BF16,F16}, cols % 16 == 0
 *   global_scale  device fp32 scalar (the encode scale gs) or NULL
 *   swizzle       0: out_scales is linear [rows, cols/16]
 *                 1: out_scales is the 128x4 layout in [roundUp(rows,128), roundUp(cols/16,4)];
 *                    the padding bytes of every 128x4 tile this call touches are written as 0
 *   out_fp4       [rows, cols/2] bytes
 */
NVF_API int nvf_nvfp4_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols,
                                     const float* global_scale, int swizzle, void* out_fp4,
                                     void* out_scales, void* stream);

/* runtime/block_quantization_kernels.cu:363-413 bq::grouped_block_quantize_to_nvfp4
 * (graph op nv_grouped_block_quantize, python/python_direct/ops.cpp:3559-3607).
 * Row r belongs to the last group g with input_offsets[g] <= r; its scales go to rows
 * output_offsets[g] + (r - input_offsets[g]) of a [>= sum roundUp(m_g,128), roundUp(cols/16,4)]
 * buffer, each group swizzled 128x4 on its own.  input_offsets / output_offsets: int32 [groups].
 */
NVF_API int nvf_nvfp4_grouped_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols,
                                             const int32_t* input_offsets, const int32_t* output_offsets,
                                             int groups, const float* global_scale, void* out_fp4,
                                             void* out_scales, void* stream);

/* The step ahead of nv_grouped_block_quantize in the reference's NVFP4 MoE layer, fused into the quantizer:
 * the input is silu(gate) * up as benchmarks/python/layers_for_inference_benchmark.py:504 computes it on
 * tensors of the inputs' type (silu = x / (1 + exp(-x)) in fp32 rounded to that type, product in fp32 rounded
 * to that type), then quantized exactly as nvf_nvfp4_grouped_block_quantize does.  gate, up: [rows, cols]
 * bf16 or f16.  input_offsets == NULL selects the ungrouped quantizer with the 128x4 scale layout
 * (swizzle = 1 of nvf_nvfp4_block_quantize); output_offsets and groups are then ignored.
 */
NVF_API int nvf_nvfp4_silu_mul_block_quantize(const void* gate, const void* up, int in_dtype, int64_t rows,
                                              int64_t cols, const int32_t* input_offsets,
                                              const int32_t* output_offsets, int groups, const float* global_scale,
                                              void* out_fp4, void* out_scales, void* stream);

/* The step ahead of nv_block_quantize when a global scale is used: compute_nvfp4_global_scale of
 * tests/python/direct/test_narrow_precision.py:138-156 on the device, without its host round trip.
 * out_scale[0] = min(448 * 6 / max|in|, FLT_MAX), 1.0 if the tensor is all zero, NaN if it holds a NaN;
 * in: numel elements of in_dtype (f32, bf16, f16), any alignment of the element type.
 */
NVF_API int nvf_nvfp4_global_scale(const void* in, int in_dtype, int64_t numel, float* out_scale, void* stream);

/* runtime/block_quantization_kernels.cu:321-361 bq::preprocessGroupedMatmulInputSf
 * (graph op preprocess_grouped_matmul_input_sf, python/python_direct/ops.cpp:3179-3212).
 * Pure layout: copies a linear [rows, cols] matrix of elem_size-byte elements (1, 2 or 4) into
 * the per-group padded 128x4 buffer addressed as above with padded_cols = roundUp(cols,4). */
NVF_API int nvf_preprocess_grouped_matmul_input_sf(const void* in, int elem_size, int64_t rows, int64_t cols,
                                                   const int32_t* input_offsets, const int32_t* output_offsets,
                                                   int groups, void* out, void* stream);

/* runtime/block_quantization_kernels.cu:142-186 bq::block_quantize_to_mxfp8
 * (graph op nv_block_quantize with dtype Float8_e4m3fn).  cols % 32 == 0.
 *   out_fp8     [rows, cols] e4m3 bytes
 *   out_scales  e8m0 bytes, linear [rows, cols/32] (swizzle == 0, the reference's only mode) or the
 *               128x4 layout in [roundUp(rows,128), roundUp(cols/32,4)] (swizzle == 1, so that the
 *               output feeds nvf_mxfp8_scaled_mm directly). */
NVF_API int nvf_mxfp8_block_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, int swizzle,
                                     void* out_fp8, void* out_scales, void* stream);

/* runtime/casts.cu:1074-1111, :698-712, :913-927 -- the narrow casts themselves, element-wise on
 * n fp32 values: e2m1 (rn, satfinite; one code per output byte), e4m3 (rn, satfinite), ue8m0 (rp). */
NVF_API int nvf_cast_f32_to_e2m1(const float* in, int64_t n, uint8_t* out, void* stream);
NVF_API int nvf_cast_f32_to_e4m3(const float* in, int64_t n, uint8_t* out, void* stream);
NVF_API int nvf_cast_f32_to_e8m0(const float* in, int64_t n, uint8_t* out, void* stream);

/* ----------------------------------------------------------------------------------------------
 * GEMMs.  out_dtype / ab_dtype in {NVF_BF16, NVF_F16}.  B is always [N, K] with K contiguous
 * ("ColumnMajor" in the reference), so every op computes A * B^T with fp32 accumulation.
 * Operand, scale, result and workspace buffers must be 16-byte aligned (NVF_ERR_INVALID_ARGUMENT
 * otherwise; the reference's TMA descriptors need the same of its tensors).
 * -------------------------------------------------------------------------------------------- */

/* cutlass/nvfp4_scaled_mm.cu:283-312 nvfp4_scaled_mm (shape rules: cutlass/nvf_cutlass.cpp:13-122).
 *   a [m, k/2], b [n, k/2] packed fp4; scales_a / scales_b e4m3 in the 128x4 layout of
 *   [roundUp(m|n,128), roundUp(k/16,4)]; alpha: device fp32 scalar; out [m, n].
 *   k % 32 == 0, n % 32 == 0. */
NVF_API int nvf_nvfp4_scaled_mm(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                const float* alpha, void* out, int64_t m, int64_t n, int64_t k,
                                int out_dtype, void* stream);

/* The same op with scratch memory, as the reference's entry point allocates a workspace for its kernel
 * (cutlass/nvfp4_scaled_mm.cu:241-256).  nvf_nvfp4_scaled_mm_workspace_bytes returns the number of bytes with
 * which this shape runs faster (0 for most shapes: then workspace may be NULL); with at least that many
 * bytes of device memory, shapes with few output tiles and a deep K (decode and small prefill batches) split
 * K over workgroups, keep fp32 partial products in the workspace and add them in a fixed order
 * (deterministic).  With less, the call is nvf_nvfp4_scaled_mm.  The workspace must not be shared with a
 * call that may run at the same time. */
NVF_API int64_t nvf_nvfp4_scaled_mm_workspace_bytes(int64_t m, int64_t n, int64_t k);
NVF_API int nvf_nvfp4_scaled_mm_ws(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                   const float* alpha, void* out, int64_t m, int64_t n, int64_t k, int out_dtype,
                                   void* workspace, int64_t workspace_bytes, void* stream);

/* No counterpart in the reference (its entry point allocates its workspace with torch, cutlass/nvfp4_scaled_mm.cu:241-256).
 * nvf_nvfp4_scaled_mm_ws for callers that cannot allocate -- code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc: the split of K keeps its fp32 partial tiles in a scratch array inside the
 * library (NVF_STATIC_SCRATCH_BYTES per device, held until the process ends) and the call allocates nothing.
 * Results are bit-identical to nvf_nvfp4_scaled_mm_ws with a workspace of nvf_nvfp4_scaled_mm_workspace_bytes.
 * A shape whose split needs more than NVF_STATIC_SCRATCH_BYTES is rejected with NVF_ERR_UNSUPPORTED_SHAPE.
 * Every call on a device shares that device's array: calls that may overlap in time on one device (different
 * streams or threads) race on it and must be serialised by the caller.
 * The first call on a device looks up the array's address and sets kernel attributes (a mutex, hipGetSymbolAddress,
 * hipFuncSetAttribute): make it outside any stream capture; every later call only launches kernels. */
#define NVF_STATIC_SCRATCH_BYTES (32ll << 20)
NVF_API int nvf_nvfp4_scaled_mm_static_ws(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                          const float* alpha, void* out, int64_t m, int64_t n, int64_t k,
                                          int out_dtype, void* stream);

/* cutlass/nvfp4_scaled_mm_blockscale.cu:332-373 nvfp4_scaled_mm_blockscale (decl cutlass/nvf_cutlass.h:147-154).
 *   Operands as nvf_nvfp4_scaled_mm.  The fp32 product alpha * A * B^T is quantized again along n in the GEMM's own
 *   epilogue (one launch, as the reference's fused epilogue :87-93), with the arithmetic of the NVFP4 block
 *   quantizer (block 16, global scale *global_normconst): out_fp4 [m, n/2], out_scales e4m3 in the 128x4 layout of
 *   [roundUp(m,128), roundUp(n/16,4)] (padding bytes of the last tiles written as 0).
 *   workspace: NULL, or m * n floats of device memory that receive the fp32 product the result was quantized from
 *   (a verification aid: it costs a second run of the GEMM). */
NVF_API int nvf_nvfp4_scaled_mm_blockscale(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                           const float* alpha, const float* global_normconst, void* out_fp4,
                                           void* out_scales, float* workspace, int64_t m, int64_t n, int64_t k,
                                           void* stream);

/* cutlass/mxfp8_scaled_mm.cu:290-319 mxfp8_scaled_mm (shape rules: cutlass/nvf_cutlass.cpp:124-234).
 *   a [m, k], b [n, k] e4m3; scales e8m0 in the 128x4 layout of [roundUp(m|n,128), roundUp(k/32,4)].
 *   k % 16 == 0, n % 16 == 0 (as in the reference); this implementation also needs k % 32 == 0. */
NVF_API int nvf_mxfp8_scaled_mm(const void* a, const void* b, const void* scales_a, const void* scales_b,
                                const float* alpha, void* out, int64_t m, int64_t n, int64_t k,
                                int out_dtype, void* stream);

/* cutlass/group_mm.cu:518-571 grouped_mm (+ get_group_gemm_starts :76-105).
 *   a [m, k], b [groups, n, k], out [m, n], all ab_dtype.
 *   problem_sizes int32 [groups, 3] = (m_g, n, k); expert_offsets int32 [groups] = first row of
 *   each group.  Rows covered by no group are left untouched.  k % 8 == 0, n % 8 == 0.
 *   The reference's ab_strides / c_strides tensors carry k and n again and are not needed here. */
NVF_API int nvf_grouped_mm(const void* a, const void* b, void* out, const int32_t* problem_sizes,
                           const int32_t* expert_offsets, int groups, int64_t m, int64_t n, int64_t k,
                           int ab_dtype, void* stream);

/* cutlass/nvfp4_scaled_group_mm.cu:714-788 nvfp4_scaled_grouped_mm (+ get_group_gemm_starts :83-155).
 *   a [m, k/2], b [groups, n, k/2] packed fp4; a_scales e4m3: group g owns rows
 *   [sf_offsets[g], sf_offsets[g] + roundUp(m_g,128)) of a [*, k/16] buffer, 128x4-swizzled on its
 *   own; b_scales [groups, n, k/16] e4m3, each [n, k/16] slab 128x4-swizzled; alphas fp32 [groups].
 *   k % 64 == 0, n % 8 == 0 as in the reference; this implementation also needs n % 128 == 0 for
 *   the per-expert b_scales slabs to be whole 128x4 tiles (the reference's pointer rule implies it). */
NVF_API int nvf_nvfp4_scaled_grouped_mm(const void* a, const void* b, const void* a_scales,
                                        const void* b_scales, const float* alphas, void* out,
                                        const int32_t* problem_sizes, const int32_t* expert_offsets,
                                        const int32_t* sf_offsets, int groups, int64_t m, int64_t n,
                                        int64_t k, int out_dtype, void* stream);

/* No counterpart in the reference: a self-check of the NVFP4 quantizer's arithmetic on the current device.  The
 * quantizer evaluates amax / 6 and 1 / x (runtime/block_quantization_kernels.cu:224, :237-239) as a reciprocal
 * with one fused correction step; this compares both forms with true fp32 division for EVERY fp32 pattern with
 * biased exponent in [2, 250] (the operands for which the quantizer uses them).  result4: 4 device uint32 =
 * { mismatches of 1/x, smallest mismatching bit pattern or 0xffffffff, the same two for x/6 }. */
NVF_API int nvf_selftest_fast_division(uint32_t* result4, void* stream);

/* No counterpart in the reference (its CUTLASS heuristics are not observable either): a dry run of the
 * dispatch of one GEMM entry point.  Writes into text (text_bytes including the terminator) the kernels the call
 * would launch on a whole MI355X, in launch order, as "kernel<variant> grid=..; ..", and touches no device -
 * it works without a GPU.  op: "nvfp4_scaled_mm" (workspace_bytes as given to nvf_nvfp4_scaled_mm_ws),
 * "nvfp4_scaled_mm_blockscale", "mxfp8_scaled_mm", "grouped_mm", "nvfp4_scaled_grouped_mm" (m = total rows).
 * Returns the status the real call would return from its argument checks. */
NVF_API int nvf_describe_dispatch(const char* op, int64_t m, int64_t n, int64_t k, int groups, int dtype,
                                  int64_t workspace_bytes, char* text, int64_t text_bytes);

#ifdef __cplusplus
}
#endif
#endif /* NVF_HIP_H_ */
