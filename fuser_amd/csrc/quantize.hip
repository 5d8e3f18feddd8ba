// NVFP4 / MXFP8 block quantizers for gfx950: one HBM pass, 16-byte loads, packed payload and block
// scales written in place (linear, 128x4 swizzled, or per-group padded 128x4).
//
// Semantics restated from runtime/block_quantization_kernels.cu:142-186 (MXFP8), :194-319 (NVFP4),
// :321-361 (scale-layout copy), :363-413 (grouped NVFP4) and the casts of runtime/casts.cu.
//
// Work decomposition: a wavefront owns one row segment of 1024 elements, 16 per lane (one NVFP4 block,
// half an MXFP8 block); a workgroup is 4 consecutive rows of one segment; details at each kernel.
#include "nvf_internal.h"

#include <cfloat>

namespace nvf {
namespace {

enum { LAYOUT_LINEAR = 0, LAYOUT_SWIZZLED = 1, LAYOUT_GROUPED = 2 };

// lane i <- lane i^1 / i^2 within a quad, lane i <- lane i+4 within a row of 16
__device__ __forceinline__ uint32_t dpp_xor1(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t dpp_xor2(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
}
__device__ __forceinline__ uint32_t dpp_shl4(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x104, 0xf, 0xf, true);  // row_shl:4
}

struct bf16_t { uint16_t v; };
struct f16_t { uint16_t v; };
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// last group g with offsets[g] <= row (what the reference's linear scan returns for sorted offsets)
__device__ __forceinline__ int find_group(const int32_t* __restrict__ offsets, int groups, int64_t row) {
  int lo = 0, hi = groups;  // invariant: answer in [lo, hi)
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (row < (int64_t)offsets[mid]) hi = mid; else lo = mid;
  }
  return lo;
}

// -------------------------------------------------------------------------------------------------
// NVFP4: one lane quantizes one 16-element block.
//   * A wavefront owns a row segment of 1024 elements; lane l loads elements [16l, 16l+16) with 16-byte
//     loads (two for 16-bit inputs, four for fp32), so a wavefront reads 2 KiB contiguous and writes
//     512 contiguous payload bytes; no cross-lane reduction and no duplicated scale arithmetic.
//   * A workgroup is 4 consecutive rows of one segment and lives for one such step: many short
//     workgroups in row-major order keep the HBM stream close to linear (5.8 TB/s on 65536 x 7168 bf16,
//     against 5.0 TB/s for workgroups that walk 128-row bands).
//   * The scale bytes of 4 neighbouring lanes are merged into one dword with two DPP steps; the dwords
//     of the 32 rows that share a 128-byte line of the 128x4 layout come from different workgroups and
//     are merged by the caches before they reach HBM.
//   * amax/6 and 1/x use a 3-instruction division (reciprocal constant resp. v_rcp_f32, one fused
//     residual correction); for biased exponents in [2, 250] it returns exactly the IEEE quotient for
//     every fp32 input (nvf_selftest_fast_division compares every such pattern with true division on the
//     device), and for a zero operand both forms end in the same result (0 resp. FLT_MAX after the clamp);
//     anything else (denormal, huge, Inf, NaN) makes the wavefront redo the block scale with true divisions.
// -------------------------------------------------------------------------------------------------
// 16 consecutive elements: the raw 16-byte loads are issued first and decoded to fp32 later, so that
// address-independent work (group lookup, global scale) overlaps the memory latency. Inactive lanes load
// from a valid dummy address and decode to zeros; `nonfinite` flags Inf or NaN among the 16.
template <typename T>
struct Raw16 {
  u32x4 q[sizeof(T) * 2];
};
template <typename T>
__device__ __forceinline__ Raw16<T> issue16(const T* p) {
  Raw16<T> r;
#pragma unroll
  for (int q = 0; q < (int)sizeof(T) * 2; ++q) r.q[q] = *(reinterpret_cast<const u32x4*>(p) + q);
  return r;
}
__device__ __forceinline__ void decode16(const Raw16<bf16_t>& r, bool active, float x[16], bool& nonfinite) {
  const uint32_t mask = active ? 0xffffffffu : 0u;
  uint32_t f = 0;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t u = r.q[q][j] & mask;
      x[8 * q + 2 * j] = bits_to_f32(u << 16);
      x[8 * q + 2 * j + 1] = bits_to_f32(u & 0xffff0000u);
      f |= (u & 0x7fff7fffu) + 0x00800080u;  // bit 15 / 31 set <=> that half is Inf or NaN
    }
  }
  nonfinite = (f & 0x80008000u) != 0;
}
__device__ __forceinline__ void decode16(const Raw16<f16_t>& r, bool active, float x[16], bool& nonfinite) {
  const uint32_t mask = active ? 0xffffffffu : 0u;
  uint32_t f = 0;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t u = r.q[q][j] & mask;
      x[8 * q + 2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u & 0xffffu));
      x[8 * q + 2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u >> 16));
      f |= (u & 0x7fff7fffu) + 0x04000400u;
    }
  }
  nonfinite = (f & 0x80008000u) != 0;
}
__device__ __forceinline__ void decode16(const Raw16<float>& r, bool active, float x[16], bool& nonfinite) {
  const uint32_t mask = active ? 0xffffffffu : 0u;
  nonfinite = false;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x[4 * q + j] = bits_to_f32(r.q[q][j] & mask);
      nonfinite |= !(fabsf(x[4 * q + j]) < INFINITY);
    }
  }
}

constexpr int kSegCols = 1024;  // elements per wavefront row segment

// value -> nearest value of the 16-bit type T (round to nearest even), as fp32
template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<bf16_t>(float v) { return (float)(__bf16)v; }
template <>
__device__ __forceinline__ float round_to<f16_t>(float v) { return (float)(_Float16)v; }
template <>
__device__ __forceinline__ float round_to<float>(float v) { return v; }

// SILU_MUL: the quantizer's input is silu(in) * in_up, evaluated the way the eager chain
// `torch.nn.functional.silu(gate) * up` evaluates it on tensors of type T - silu as x / (1 + exp(-x)) in fp32,
// rounded to T, the product in fp32, rounded to T - so the fused kernel returns the bytes of the chain
// (benchmarks/python/layers_for_inference_benchmark.py:504 followed by the grouped quantizer) without the
// chain's write and re-read of the intermediate.
template <typename T, int LAYOUT, bool SILU_MUL = false>
__global__ __launch_bounds__(256) void nvfp4_quantize_kernel(const T* __restrict__ in, const T* __restrict__ in_up,
                                                             int64_t rows, int64_t cols,
                                                             const float* __restrict__ gs_ptr,
                                                             const int32_t* __restrict__ in_off,
                                                             const int32_t* __restrict__ out_off, int groups,
                                                             uint32_t segs, uint8_t* __restrict__ out_fp4,
                                                             uint8_t* __restrict__ out_sf) {
  // workgroup = 4 consecutive rows of one 1024-column segment; consecutive workgroups walk the segments
  // of the same 4 rows, so the chip streams the input almost linearly
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t band = blockIdx.x / segs;
  const uint32_t seg = blockIdx.x - band * segs;
  const int64_t row = (int64_t)band * 4 + wave;
  const int64_t col = (int64_t)seg * kSegCols + lane * 16;
  const bool col_ok = col < cols;
  const bool active = col_ok && row < rows;
  const int64_t sf_cols = cols >> 4;
  const int64_t padded = (sf_cols + 3) & ~(int64_t)3;
  const int64_t sf_col = col >> 4;  // scale column of this lane's block
  const bool word_scales = !(LAYOUT == LAYOUT_LINEAR && (sf_cols & 3) != 0);

  const Raw16<T> raw = issue16(active ? in + row * cols + col : in);
  Raw16<T> raw_up;
  if constexpr (SILU_MUL) raw_up = issue16(active ? in_up + row * cols + col : in_up);

  const bool use_gs = gs_ptr != nullptr;
  const float gs = use_gs ? *gs_ptr : 1.0f;
  const float decode = 1.0f / gs;  // :236

  int64_t sf_row_base = 0;  // byte offset of (row, scale column 0) in the scale buffer
  if constexpr (LAYOUT == LAYOUT_GROUPED) {
    if (row < rows) {
      // row is wavefront-uniform: the search runs on the scalar unit and its cache while the loads fly
      const int g = find_group(in_off, groups, row);
      sf_row_base = (int64_t)out_off[g] * padded + swizzle_128x4(row - in_off[g], 0, padded);
    }
  } else if constexpr (LAYOUT == LAYOUT_SWIZZLED) {
    sf_row_base = swizzle_128x4(row, 0, padded);  // rows past `rows` inside the last tile receive zeros
  } else {
    sf_row_base = row * sf_cols;
  }

  float x[16];
  bool nonfinite;
  decode16(raw, active, x, nonfinite);
  if constexpr (SILU_MUL) {
    float u[16];
    bool up_nonfinite;
    decode16(raw_up, active, u, up_nonfinite);
    nonfinite = false;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float act = round_to<T>(x[j] / (1.0f + expf(-x[j])));
      x[j] = round_to<T>(act * u[j]);
      nonfinite |= !(fabsf(x[j]) < INFINITY);
    }
  }
  const bool wave_nonfinite = __builtin_amdgcn_ballot_w64(nonfinite) != 0;

  // amax, NaN ignored (fmaxf), start -inf: block_quantization_kernels.cu:124-128
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < 16; ++j) m = fmaxf(m, fabsf(x[j]));
  float r;  // factor of the block's values ahead of the e2m1 cast
  const uint32_t q8 = nvfp4_block_scale(m, use_gs, gs, decode, active, r);

  uint32_t p0 = 0, p1 = 0;
  if (!wave_nonfinite) {
    p0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p0, x[0] * r, x[1] * r, 1.0f, 0);
    p0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p0, x[2] * r, x[3] * r, 1.0f, 1);
    p0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p0, x[4] * r, x[5] * r, 1.0f, 2);
    p0 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p0, x[6] * r, x[7] * r, 1.0f, 3);
    p1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p1, x[8] * r, x[9] * r, 1.0f, 0);
    p1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p1, x[10] * r, x[11] * r, 1.0f, 1);
    p1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p1, x[12] * r, x[13] * r, 1.0f, 2);
    p1 = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p1, x[14] * r, x[15] * r, 1.0f, 3);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      p0 |= f32x2_to_e2m1_byte(x[2 * j] * r, x[2 * j + 1] * r) << (8 * j);
      p1 |= f32x2_to_e2m1_byte(x[8 + 2 * j] * r, x[8 + 2 * j + 1] * r) << (8 * j);
    }
  }
  if (active) __builtin_nontemporal_store(u32x2{p0, p1}, reinterpret_cast<u32x2*>(out_fp4 + ((row * cols + col) >> 1)));

  if (!word_scales) {
    if (active) out_sf[sf_row_base + sf_col] = (uint8_t)q8;  // scale rows are not word aligned
    return;
  }
  // merge the scale bytes of 4 neighbouring blocks; the quad leader stores the dword
  uint32_t v = active ? (q8 << (8 * (lane & 3))) : 0u;
  v |= dpp_xor1(v);
  v |= dpp_xor2(v);
  if ((lane & 3) == 0 && col_ok) {
    if constexpr (LAYOUT == LAYOUT_SWIZZLED) {
      *reinterpret_cast<uint32_t*>(out_sf + sf_row_base + ((sf_col >> 2) << 9)) = v;
    } else if constexpr (LAYOUT == LAYOUT_GROUPED) {
      if (row < rows) *reinterpret_cast<uint32_t*>(out_sf + sf_row_base + ((sf_col >> 2) << 9)) = v;
    } else {
      if (row < rows) *reinterpret_cast<uint32_t*>(out_sf + sf_row_base + sf_col) = v;
    }
  }
}

template <typename T, int LAYOUT, bool SILU_MUL>
int launch_nvfp4_layout(const T* in, const T* in_up, int64_t rows, int64_t cols, const float* gs, const int32_t* in_off,
                        const int32_t* out_off, int groups, uint8_t* out_fp4, uint8_t* out_sf, hipStream_t stream) {
  const int64_t segs = ceil_div(cols, kSegCols);
  // rows the grid must cover: the swizzled layout also zero-fills the padding rows of the last tile
  const int64_t cover = LAYOUT == LAYOUT_SWIZZLED ? round_up(rows, 128) : rows;
  const int64_t wgs = ceil_div(cover, 4) * segs;
  if (wgs >= ((int64_t)1 << 31)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "tensor of %lld x %lld is too large for one launch",
                                             (long long)rows, (long long)cols);
  if (note_launch("nvfp4_quantize_kernel<layout=%d> grid=%lld", LAYOUT, (long long)wgs)) return NVF_OK;
  hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT, SILU_MUL>), dim3((unsigned)wgs), dim3(256), 0, stream, in, in_up, rows,
                     cols, gs, in_off, out_off, groups, (uint32_t)segs, out_fp4, out_sf);
  return check_launch("nvfp4_quantize_kernel");
}

template <typename T, bool SILU_MUL>
int launch_nvfp4_typed(const T* in, const T* in_up, int64_t rows, int64_t cols, const float* gs, int layout,
                       const int32_t* in_off, const int32_t* out_off, int groups, uint8_t* out_fp4, uint8_t* out_sf,
                       hipStream_t stream) {
  if (layout == LAYOUT_SWIZZLED)
    return launch_nvfp4_layout<T, LAYOUT_SWIZZLED, SILU_MUL>(in, in_up, rows, cols, gs, in_off, out_off, groups, out_fp4, out_sf,
                                                             stream);
  if (layout == LAYOUT_GROUPED)
    return launch_nvfp4_layout<T, LAYOUT_GROUPED, SILU_MUL>(in, in_up, rows, cols, gs, in_off, out_off, groups, out_fp4, out_sf,
                                                            stream);
  return launch_nvfp4_layout<T, LAYOUT_LINEAR, SILU_MUL>(in, in_up, rows, cols, gs, in_off, out_off, groups, out_fp4, out_sf,
                                                         stream);
}

// -------------------------------------------------------------------------------------------------
// Global (per-tensor) NVFP4 encode scale 448 * 6 / max|x| on the device, for the quantizer's global_scale
// argument; restates compute_nvfp4_global_scale of tests/python/direct/test_narrow_precision.py:138-156
// without its host round trip: 1.0 for an all-zero tensor, clamped to FLT_MAX, NaN if the tensor holds
// one (torch.max propagates it), the quotient evaluated in double and rounded once to fp32 as Python
// does.  |x| is compared through its fp32 bit pattern, whose unsigned order is the numeric order of
// non-negative floats with NaN on top; the maximum is order-independent, hence deterministic.
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t abs_bits(bf16_t v) { return (uint32_t)(v.v & 0x7fffu) << 16; }
__device__ __forceinline__ uint32_t abs_bits(f16_t v) {
  return f32_to_bits((float)__builtin_bit_cast(_Float16, (uint16_t)(v.v & 0x7fffu)));
}
__device__ __forceinline__ uint32_t abs_bits(float v) { return f32_to_bits(v) & 0x7fffffffu; }

__global__ void amax_init_kernel(uint32_t* cell) { *cell = 0u; }

template <typename T>
__global__ __launch_bounds__(256) void amax_kernel(const T* __restrict__ in, int64_t n, int64_t head, int64_t nvec,
                                                   uint32_t* __restrict__ cell) {
  constexpr int VE = 16 / (int)sizeof(T);  // elements per 16-byte load
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  uint32_t m = 0;
  const u32x4* vec = reinterpret_cast<const u32x4*>(in + head);
  auto fold = [&](const u32x4 q) {
    T e[VE];
    __builtin_memcpy(e, &q, 16);
#pragma unroll
    for (int j = 0; j < VE; ++j) m = max(m, abs_bits(e[j]));
  };
  int64_t i = tid;
  for (; i + 3 * stride < nvec; i += 4 * stride) {  // four loads in flight per thread
    const u32x4 q0 = __builtin_nontemporal_load(vec + i), q1 = __builtin_nontemporal_load(vec + i + stride);
    const u32x4 q2 = __builtin_nontemporal_load(vec + i + 2 * stride), q3 = __builtin_nontemporal_load(vec + i + 3 * stride);
    fold(q0);
    fold(q1);
    fold(q2);
    fold(q3);
  }
  for (; i < nvec; i += stride) fold(__builtin_nontemporal_load(vec + i));
  // elements before the first and after the last whole 16-byte vector
  const int64_t tail0 = head + nvec * VE;
  for (int64_t t = tid; t < head + (n - tail0); t += stride) m = max(m, abs_bits(in[t < head ? t : tail0 + (t - head)]));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, d, 64));
  if ((threadIdx.x & 63) == 0 && m != 0) atomicMax(cell, m);
}

__device__ __forceinline__ float amax_bits_to_global_scale(uint32_t amax_bits) {
  const float amax = bits_to_f32(amax_bits);
  if (amax != amax) return amax;
  if (amax == 0.0f) return 1.0f;
  const double q = 2688.0 / (double)amax;  // FLOAT8_E4M3_MAX * FLOAT4_E2M1_MAX
  return q > (double)FLT_MAX ? FLT_MAX : (float)q;
}

__global__ void amax_to_global_scale_kernel(uint32_t* cell) {
  *reinterpret_cast<float*>(cell) = amax_bits_to_global_scale(*cell);
}

// small tensors: one workgroup does the whole job in one launch
template <typename T>
__global__ __launch_bounds__(1024) void global_scale_small_kernel(const T* __restrict__ in, int64_t n, float* __restrict__ out) {
  __shared__ uint32_t wave_max[16];
  uint32_t m = 0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) m = max(m, abs_bits(in[i]));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, d, 64));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < 16; ++w) m = max(m, wave_max[w]);
    *out = amax_bits_to_global_scale(m);
  }
}

template <typename T>
int launch_global_scale_typed(const T* in, int64_t n, float* out, hipStream_t stream) {
  constexpr int VE = 16 / (int)sizeof(T);
  if (n <= 65536) {
    hipLaunchKernelGGL(global_scale_small_kernel<T>, dim3(1), dim3(1024), 0, stream, in, n, out);
    return check_launch("nvfp4_global_scale");
  }
  uint32_t* cell = reinterpret_cast<uint32_t*>(out);
  hipLaunchKernelGGL(amax_init_kernel, dim3(1), dim3(1), 0, stream, cell);
  if (n > 0) {
    const uintptr_t addr = reinterpret_cast<uintptr_t>(in);
    int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));  // elements up to 16-byte alignment
    if (head > n) head = n;
    const int64_t nvec = (n - head) / VE;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    const int64_t want = ceil_div(nvec > 0 ? nvec : 1, 256 * 4);  // at least 4 loads per thread
    const int64_t cap = (int64_t)cus * 8;
    hipLaunchKernelGGL(amax_kernel<T>, dim3((unsigned)(want < cap ? want : cap)), dim3(256), 0, stream, in, n, head, nvec, cell);
  }
  hipLaunchKernelGGL(amax_to_global_scale_kernel, dim3(1), dim3(1), 0, stream, cell);
  return check_launch("nvfp4_global_scale");
}

// -------------------------------------------------------------------------------------------------
// MXFP8: 32-element blocks, scale = ue8m0_rp(amax * (1/448)), payload = e4m3(x * 2^-(e-127)).
// A lane holds 16 elements (half a block, amax merged with its neighbour by one DPP step) and stores 16
// payload bytes; a wavefront owns a 1024-element row segment, a workgroup 4 consecutive rows of it, in
// the same row-major order of short workgroups as the NVFP4 kernel.
// -------------------------------------------------------------------------------------------------
template <typename T, bool SWIZZLE>
__global__ __launch_bounds__(256) void mxfp8_quantize_kernel(const T* __restrict__ in, int64_t rows, int64_t cols,
                                                             uint32_t segs, uint8_t* __restrict__ out_fp8,
                                                             uint8_t* __restrict__ out_sf) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const uint32_t band = blockIdx.x / segs;
  const uint32_t seg = blockIdx.x - band * segs;
  const int64_t row = (int64_t)band * 4 + wave;
  const int64_t col = (int64_t)seg * kSegCols + lane * 16;
  const bool col_ok = col < cols;  // cols % 32 == 0, so both lanes of a block agree
  const bool active = col_ok && row < rows;
  const int64_t sf_cols = cols >> 5;
  const int64_t padded = (sf_cols + 3) & ~(int64_t)3;
  const int64_t sf_col = col >> 5;
  const bool word_stores = SWIZZLE || (sf_cols & 3) == 0;

  const Raw16<T> raw = issue16(active ? in + row * cols + col : in);
  float x[16];
  bool nonfinite;
  decode16(raw, active, x, nonfinite);
  const bool wave_nonfinite = __builtin_amdgcn_ballot_w64(nonfinite) != 0;
  // amax, NaN ignored (fmaxf), start -inf: block_quantization_kernels.cu:124-128
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < 16; ++j) m = fmaxf(m, fabsf(x[j]));
  m = fmaxf(m, bits_to_f32(dpp_xor1(f32_to_bits(m))));
  const uint32_t e = f32_to_e8m0_rp(m * (1.0f / 448));                   // :168-169
  const float inv = (e == 0) ? 1.0f : bits_to_f32((254u - e) << 23);     // :134-140
  uint32_t w[4] = {0, 0, 0, 0};
  if (!wave_nonfinite) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      w[j] = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(x[4 * j] * inv, -448.0f, 448.0f),
                                             __builtin_amdgcn_fmed3f(x[4 * j + 1] * inv, -448.0f, 448.0f), w[j], false);
      w[j] = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(x[4 * j + 2] * inv, -448.0f, 448.0f),
                                             __builtin_amdgcn_fmed3f(x[4 * j + 3] * inv, -448.0f, 448.0f), w[j], true);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) w[j >> 2] |= f32_to_e4m3_satfinite(x[j] * inv) << (8 * (j & 3));
  }
  if (active)
    __builtin_nontemporal_store(u32x4{w[0], w[1], w[2], w[3]}, reinterpret_cast<u32x4*>(out_fp8 + row * cols + col));

  if (!word_stores) {
    if (active && !(lane & 1)) out_sf[row * sf_cols + sf_col] = (uint8_t)e;  // scale rows are not word aligned
    return;
  }
  // the scale bytes of 4 neighbouring blocks (8 lanes) merged into lane 0 of every 8
  uint32_t v = ((lane & 1) || !active) ? 0u : (e << (8 * ((lane >> 1) & 3)));
  v |= dpp_xor2(v);
  v |= dpp_shl4(v);
  if ((lane & 7) == 0 && col_ok) {
    if constexpr (SWIZZLE) {
      *reinterpret_cast<uint32_t*>(out_sf + swizzle_128x4(row, sf_col, padded)) = v;  // padding rows: zeros
    } else {
      if (row < rows) *reinterpret_cast<uint32_t*>(out_sf + row * sf_cols + sf_col) = v;
    }
  }
}

template <typename T>
int launch_mxfp8_typed(const T* in, int64_t rows, int64_t cols, int swizzle, uint8_t* out_fp8, uint8_t* out_sf,
                       hipStream_t stream) {
  const int64_t segs = ceil_div(cols, kSegCols);
  const int64_t cover = swizzle ? round_up(rows, 128) : rows;
  const int64_t wgs = ceil_div(cover, 4) * segs;
  if (wgs >= ((int64_t)1 << 31)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "tensor of %lld x %lld is too large for one launch",
                                             (long long)rows, (long long)cols);
  if (swizzle) {
    hipLaunchKernelGGL((mxfp8_quantize_kernel<T, true>), dim3((unsigned)wgs), dim3(256), 0, stream, in, rows, cols,
                       (uint32_t)segs, out_fp8, out_sf);
  } else {
    hipLaunchKernelGGL((mxfp8_quantize_kernel<T, false>), dim3((unsigned)wgs), dim3(256), 0, stream, in, rows, cols,
                       (uint32_t)segs, out_fp8, out_sf);
  }
  return check_launch("mxfp8_quantize_kernel");
}

// -------------------------------------------------------------------------------------------------
// Scale-layout copy and element-wise casts
// -------------------------------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void preprocess_sf_kernel(const E* __restrict__ in, int64_t rows, int64_t cols,
                                                            const int32_t* __restrict__ in_off,
                                                            const int32_t* __restrict__ out_off, int groups,
                                                            E* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= rows * cols) return;
  const int64_t r = idx / cols, c = idx % cols;
  const int64_t padded = (cols + 3) & ~(int64_t)3;
  const int g = find_group(in_off, groups, r);
  out[(int64_t)out_off[g] * padded + swizzle_128x4(r - in_off[g], c, padded)] = in[idx];
}

template <int KIND>
__global__ __launch_bounds__(256) void cast_kernel(const float* __restrict__ in, int64_t n, uint8_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float x = in[i];
  uint32_t r;
  if constexpr (KIND == 0) r = f32x2_to_e2m1_byte(x, 0.0f) & 0xfu;
  else if constexpr (KIND == 1) r = f32_to_e4m3_satfinite(x);
  else r = f32_to_e8m0_rp(x);
  out[i] = (uint8_t)r;
}

}  // namespace

int launch_nvfp4_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, const float* gs, int layout,
                          const int32_t* in_off, const int32_t* out_off, int groups, void* out_fp4, void* out_sf,
                          hipStream_t stream) {
  uint8_t* q = static_cast<uint8_t*>(out_fp4);
  uint8_t* s = static_cast<uint8_t*>(out_sf);
  switch (in_dtype) {
    case NVF_F32:
      return launch_nvfp4_typed<float, false>(static_cast<const float*>(in), nullptr, rows, cols, gs, layout, in_off, out_off,
                                              groups, q, s, stream);
    case NVF_BF16:
      return launch_nvfp4_typed<bf16_t, false>(static_cast<const bf16_t*>(in), nullptr, rows, cols, gs, layout, in_off, out_off,
                                               groups, q, s, stream);
    case NVF_F16:
      return launch_nvfp4_typed<f16_t, false>(static_cast<const f16_t*>(in), nullptr, rows, cols, gs, layout, in_off, out_off,
                                              groups, q, s, stream);
  }
  return fail(NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
}

int launch_nvfp4_silu_mul_quantize(const void* gate, const void* up, int in_dtype, int64_t rows, int64_t cols, const float* gs,
                                   int layout, const int32_t* in_off, const int32_t* out_off, int groups, void* out_fp4,
                                   void* out_sf, hipStream_t stream) {
  uint8_t* q = static_cast<uint8_t*>(out_fp4);
  uint8_t* s = static_cast<uint8_t*>(out_sf);
  switch (in_dtype) {
    case NVF_BF16:
      return launch_nvfp4_typed<bf16_t, true>(static_cast<const bf16_t*>(gate), static_cast<const bf16_t*>(up), rows, cols, gs,
                                              layout, in_off, out_off, groups, q, s, stream);
    case NVF_F16:
      return launch_nvfp4_typed<f16_t, true>(static_cast<const f16_t*>(gate), static_cast<const f16_t*>(up), rows, cols, gs,
                                             layout, in_off, out_off, groups, q, s, stream);
  }
  return fail(NVF_ERR_INVALID_ARGUMENT, "silu-mul quantize takes bf16 or f16 inputs, got dtype %d", in_dtype);
}

int launch_nvfp4_global_scale(const void* in, int in_dtype, int64_t n, float* out, hipStream_t stream) {
  switch (in_dtype) {
    case NVF_F32: return launch_global_scale_typed(static_cast<const float*>(in), n, out, stream);
    case NVF_BF16: return launch_global_scale_typed(static_cast<const bf16_t*>(in), n, out, stream);
    case NVF_F16: return launch_global_scale_typed(static_cast<const f16_t*>(in), n, out, stream);
  }
  return fail(NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
}

int launch_mxfp8_quantize(const void* in, int in_dtype, int64_t rows, int64_t cols, int swizzle, void* out_fp8,
                          void* out_sf, hipStream_t stream) {
  uint8_t* q = static_cast<uint8_t*>(out_fp8);
  uint8_t* s = static_cast<uint8_t*>(out_sf);
  switch (in_dtype) {
    case NVF_F32: return launch_mxfp8_typed(static_cast<const float*>(in), rows, cols, swizzle, q, s, stream);
    case NVF_BF16: return launch_mxfp8_typed(static_cast<const bf16_t*>(in), rows, cols, swizzle, q, s, stream);
    case NVF_F16: return launch_mxfp8_typed(static_cast<const f16_t*>(in), rows, cols, swizzle, q, s, stream);
  }
  return fail(NVF_ERR_INVALID_ARGUMENT, "unknown input dtype %d", in_dtype);
}

int launch_preprocess_sf(const void* in, int elem_size, int64_t rows, int64_t cols, const int32_t* in_off,
                         const int32_t* out_off, int groups, void* out, hipStream_t stream) {
  const int64_t n = rows * cols;
  if (n == 0) return NVF_OK;
  dim3 grid((unsigned)ceil_div(n, 256));
  switch (elem_size) {
    case 1:
      hipLaunchKernelGGL(preprocess_sf_kernel<uint8_t>, grid, dim3(256), 0, stream, static_cast<const uint8_t*>(in), rows,
                         cols, in_off, out_off, groups, static_cast<uint8_t*>(out));
      break;
    case 2:
      hipLaunchKernelGGL(preprocess_sf_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(in),
                         rows, cols, in_off, out_off, groups, static_cast<uint16_t*>(out));
      break;
    case 4:
      hipLaunchKernelGGL(preprocess_sf_kernel<uint32_t>, grid, dim3(256), 0, stream, static_cast<const uint32_t*>(in),
                         rows, cols, in_off, out_off, groups, static_cast<uint32_t*>(out));
      break;
    default:
      return fail(NVF_ERR_INVALID_ARGUMENT, "element size %d is not 1, 2 or 4", elem_size);
  }
  return check_launch("preprocess_sf_kernel");
}

namespace {
// Every fp32 pattern with biased exponent in [2, 250] (both signs are the same arithmetic; positive ones are
// what the quantizer meets): the 3-instruction forms against true division.  out[0] / out[2] count the
// mismatches of 1/x and x/6, out[1] / out[3] hold the smallest mismatching pattern (0xffffffff: none).
__global__ __launch_bounds__(256) void division_selftest_kernel(uint32_t* __restrict__ out) {
  uint32_t bad_rcp = 0, bad_div = 0, first_rcp = 0xffffffffu, first_div = 0xffffffffu;
  const uint32_t mant = blockIdx.x * 256u + threadIdx.x;  // 2^15 workgroups x 256 = every 23-bit mantissa
  for (uint32_t e = 2; e <= 250; ++e) {
    const uint32_t bits = (e << 23) | mant;
    const float v = bits_to_f32(bits);
    if (f32_to_bits(fast_rcp(v)) != f32_to_bits(1.0f / v)) { ++bad_rcp; first_rcp = min(first_rcp, bits); }
    if (f32_to_bits(fast_div6(v)) != f32_to_bits(v / 6.0f)) { ++bad_div; first_div = min(first_div, bits); }
  }
  if (bad_rcp) { atomicAdd(out + 0, bad_rcp); atomicMin(out + 1, first_rcp); }
  if (bad_div) { atomicAdd(out + 2, bad_div); atomicMin(out + 3, first_div); }
}
__global__ void division_selftest_init_kernel(uint32_t* out) {
  out[0] = 0; out[1] = 0xffffffffu; out[2] = 0; out[3] = 0xffffffffu;
}
}  // namespace

int launch_division_selftest(uint32_t* out4, hipStream_t stream) {
  hipLaunchKernelGGL(division_selftest_init_kernel, dim3(1), dim3(1), 0, stream, out4);
  hipLaunchKernelGGL(division_selftest_kernel, dim3(1u << 15), dim3(256), 0, stream, out4);
  return check_launch("division_selftest_kernel");
}

int launch_cast(int kind, const float* in, int64_t n, uint8_t* out, hipStream_t stream) {
  if (n == 0) return NVF_OK;
  dim3 grid((unsigned)ceil_div(n, 256));
  if (kind == 0) hipLaunchKernelGGL(cast_kernel<0>, grid, dim3(256), 0, stream, in, n, out);
  else if (kind == 1) hipLaunchKernelGGL(cast_kernel<1>, grid, dim3(256), 0, stream, in, n, out);
  else hipLaunchKernelGGL(cast_kernel<2>, grid, dim3(256), 0, stream, in, n, out);
  return check_launch("cast_kernel");
}

}  // namespace nvf
