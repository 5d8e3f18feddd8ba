// NVFP4 / MXFP8 block quantizers for gfx950: one HBM pass, 16-byte coalesced loads, amax reduced
// across lanes with DPP, packed payload and block scales written in place (linear, 128x4 swizzled,
// or per-group padded 128x4).
//
// Semantics restated from runtime/block_quantization_kernels.cu:142-186 (MXFP8), :194-319 (NVFP4),
// :321-361 (scale-layout copy), :363-413 (grouped NVFP4) and the casts of runtime/casts.cu.
//
// Work decomposition (all kernels): a wavefront owns one row segment of 512 consecutive elements,
// lane l holding elements [8l, 8l+8) -> a 1 KiB contiguous read and a 256 B (fp4) / 512 B (fp8)
// contiguous payload write per wavefront.  A 256-thread workgroup walks a band of 32*ROW_ITERS rows;
// with ROW_ITERS == 4 a lane visits rows r, r+32, r+64, r+96 so that the four scale words it
// gathers are the 16 contiguous bytes the 128x4 layout gives those rows.
#include "nvf_internal.h"

#include <cfloat>

namespace nvf {
namespace {

enum { LAYOUT_LINEAR = 0, LAYOUT_SWIZZLED = 1, LAYOUT_GROUPED = 2 };

constexpr int kSegCols = 512;  // elements per wavefront row segment

// lane i <- lane i^1 / i^2 within a quad, lane i <- lane i+4 / i+8 within a row of 16
__device__ __forceinline__ uint32_t dpp_xor1(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t dpp_xor2(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
}
__device__ __forceinline__ uint32_t dpp_shl4(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x104, 0xf, 0xf, true);  // row_shl:4
}
__device__ __forceinline__ uint32_t dpp_shl8(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x108, 0xf, 0xf, true);  // row_shl:8
}

// ---- loading 8 consecutive elements as fp32, with a cheap "contains Inf or NaN" flag ----
struct bf16_t { uint16_t v; };
struct f16_t { uint16_t v; };
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void load8(const bf16_t* p, float x[8], bool& nan) {
  const u32x4 u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  uint32_t f = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[2 * j] = bits_to_f32(u[j] << 16);
    x[2 * j + 1] = bits_to_f32(u[j] & 0xffff0000u);
    f |= ((u[j] & 0x7fff7fffu) + 0x00800080u);  // bit 15 / 31 set <=> that half is Inf or NaN
  }
  nan = (f & 0x80008000u) != 0;
}
__device__ __forceinline__ void load8(const f16_t* p, float x[8], bool& nan) {
  const u32x4 u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  uint32_t f = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[j] & 0xffffu));
    x[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[j] >> 16));
    f |= ((u[j] & 0x7fff7fffu) + 0x04000400u);
  }
  nan = (f & 0x80008000u) != 0;
}
__device__ __forceinline__ void load8(const float* p, float x[8], bool& nan) {
  const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p) + 1);
#pragma unroll
  for (int j = 0; j < 4; ++j) { x[j] = a[j]; x[4 + j] = b[j]; }
  nan = false;
#pragma unroll
  for (int j = 0; j < 8; ++j) nan |= !(fabsf(x[j]) < INFINITY);
}

// amax of 8 values, NaN ignored (fmaxf), start -inf: block_quantization_kernels.cu:124-128
__device__ __forceinline__ float amax8(const float x[8]) {
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(x[j]));
  return m;
}

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
// NVFP4
// -------------------------------------------------------------------------------------------------
template <typename T, int LAYOUT, int ROW_ITERS>
__global__ __launch_bounds__(256) void nvfp4_quantize_kernel(const T* __restrict__ in, int64_t rows, int64_t cols,
                                                             const float* __restrict__ gs_ptr,
                                                             const int32_t* __restrict__ in_off,
                                                             const int32_t* __restrict__ out_off, int groups,
                                                             uint8_t* __restrict__ out_fp4,
                                                             uint8_t* __restrict__ out_sf) {
  constexpr int kBandRows = 32 * ROW_ITERS;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row0 = (int64_t)blockIdx.y * kBandRows;
  const int64_t col = (int64_t)blockIdx.x * kSegCols + lane * 8;
  const bool col_ok = col < cols;
  const int64_t sf_cols = cols >> 4;
  const int64_t padded = (sf_cols + 3) & ~(int64_t)3;
  const int64_t sf_col = col >> 4;  // scale column of this lane's block

  const bool use_gs = gs_ptr != nullptr;
  const float gs = use_gs ? *gs_ptr : 1.0f;
  const float decode = 1.0f / gs;  // :236

  __shared__ int64_t row_sf_base[kBandRows];
  if constexpr (LAYOUT == LAYOUT_GROUPED) {
    if (threadIdx.x < kBandRows) {
      const int64_t r = row0 + threadIdx.x;
      int64_t base = 0;
      if (r < rows) {
        const int g = find_group(in_off, groups, r);
        base = (int64_t)out_off[g] * padded + swizzle_128x4(r - in_off[g], 0, padded);
      }
      row_sf_base[threadIdx.x] = base;
    }
    __syncthreads();
  }

#pragma unroll 1
  for (int t = 0; t < 8; ++t) {
    const int rb = t * 4 + wave;  // row inside a 32-row group
    uint32_t sfw[ROW_ITERS];
    float x[ROW_ITERS][8];
    bool nan = false;
#pragma unroll
    for (int i = 0; i < ROW_ITERS; ++i) {
      const int64_t row = row0 + rb + 32 * i;
      if (col_ok && row < rows) {
        bool n;
        load8(in + row * cols + col, x[i], n);
        nan |= n;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[i][j] = 0.0f;
      }
    }
    const bool wave_has_nan = __builtin_amdgcn_ballot_w64(nan) != 0;  // any non-finite input in the wavefront

#pragma unroll
    for (int i = 0; i < ROW_ITERS; ++i) {
      const int64_t row = row0 + rb + 32 * i;
      float m = amax8(x[i]);
      m = fmaxf(m, bits_to_f32(dpp_xor1(f32_to_bits(m))));  // the two lanes of a 16-element block
      float s = m / 6.0f;                                    // :224
      if (use_gs) s = s * gs;                                // :226
      s = fminf(s, FLT_MAX);                                 // :228
      const uint32_t q8 = f32_to_e4m3_satfinite(s);          // :230
      const float sf = e4m3_to_f32(q8);                      // :233
      const float r = use_gs ? fminf(1.0f / (sf * decode), FLT_MAX) : fminf(1.0f / sf, FLT_MAX);  // :237/:239

      uint32_t p = 0;
      if (!wave_has_nan) {
        p = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p, x[i][0] * r, x[i][1] * r, 1.0f, 0);
        p = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p, x[i][2] * r, x[i][3] * r, 1.0f, 1);
        p = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p, x[i][4] * r, x[i][5] * r, 1.0f, 2);
        p = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(p, x[i][6] * r, x[i][7] * r, 1.0f, 3);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) p |= f32x2_to_e2m1_byte(x[i][2 * j] * r, x[i][2 * j + 1] * r) << (8 * j);
      }
      const bool active = col_ok && row < rows;
      if (active) *reinterpret_cast<uint32_t*>(out_fp4 + ((row * cols + col) >> 1)) = p;

      if (LAYOUT == LAYOUT_LINEAR && (sf_cols & 3) != 0) {
        // scale rows are not word aligned: one byte per block, written by its even lane
        if (active && !(lane & 1)) out_sf[row * sf_cols + sf_col] = (uint8_t)q8;
        sfw[i] = 0;
      } else {
        // gather the 4 scale bytes of 64 consecutive elements into lane 0 of each 8-lane group
        uint32_t v = ((lane & 1) || !active) ? 0u : (q8 << (8 * ((lane >> 1) & 3)));
        v |= dpp_xor2(v);
        v |= dpp_shl4(v);
        sfw[i] = v;
      }
    }

    if ((lane & 7) == 0 && col_ok && !(LAYOUT == LAYOUT_LINEAR && (sf_cols & 3) != 0)) {
      if constexpr (LAYOUT == LAYOUT_SWIZZLED && ROW_ITERS == 4) {
        // rows rb, rb+32, rb+64, rb+96 of one 128-row tile: 16 contiguous bytes
        uint8_t* dst = out_sf + (int64_t)blockIdx.y * (padded << 7) + ((sf_col >> 2) << 9) + (rb << 4);
        *reinterpret_cast<uint4*>(dst) = make_uint4(sfw[0], sfw[1], sfw[2], sfw[3]);
      } else {
#pragma unroll
        for (int i = 0; i < ROW_ITERS; ++i) {
          const int64_t row = row0 + rb + 32 * i;
          if constexpr (LAYOUT == LAYOUT_SWIZZLED) {
            // rows past `rows` inside the last 128-row tile receive zeros
            *reinterpret_cast<uint32_t*>(out_sf + swizzle_128x4(row, sf_col, padded)) = sfw[i];
          } else if constexpr (LAYOUT == LAYOUT_GROUPED) {
            if (row < rows)
              *reinterpret_cast<uint32_t*>(out_sf + row_sf_base[rb + 32 * i] + ((sf_col >> 2) << 9)) = sfw[i];
          } else {
            if (row < rows) *reinterpret_cast<uint32_t*>(out_sf + row * sf_cols + sf_col) = sfw[i];
          }
        }
      }
    }
  }
}

template <typename T>
int launch_nvfp4_typed(const T* in, int64_t rows, int64_t cols, const float* gs, int layout, const int32_t* in_off,
                       const int32_t* out_off, int groups, uint8_t* out_fp4, uint8_t* out_sf, hipStream_t stream) {
  const unsigned gx = (unsigned)ceil_div(cols, kSegCols);
  // Large inputs: 128-row bands (16-byte scale stores).  Small inputs: 32-row bands so that more
  // compute units get work.
  const bool big = rows * cols >= ((int64_t)1 << 24);
  if (layout == LAYOUT_SWIZZLED) {
    if (big) {
      dim3 grid(gx, (unsigned)ceil_div(rows, 128));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_SWIZZLED, 4>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    } else {
      dim3 grid(gx, (unsigned)(round_up(rows, 128) / 32));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_SWIZZLED, 1>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    }
  } else if (layout == LAYOUT_GROUPED) {
    if (big) {
      dim3 grid(gx, (unsigned)ceil_div(rows, 128));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_GROUPED, 4>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    } else {
      dim3 grid(gx, (unsigned)ceil_div(rows, 32));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_GROUPED, 1>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    }
  } else {
    if (big) {
      dim3 grid(gx, (unsigned)ceil_div(rows, 128));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_LINEAR, 4>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    } else {
      dim3 grid(gx, (unsigned)ceil_div(rows, 32));
      hipLaunchKernelGGL((nvfp4_quantize_kernel<T, LAYOUT_LINEAR, 1>), grid, dim3(256), 0, stream, in, rows, cols, gs,
                         in_off, out_off, groups, out_fp4, out_sf);
    }
  }
  return check_launch("nvfp4_quantize_kernel");
}

// -------------------------------------------------------------------------------------------------
// MXFP8: 32-element blocks (4 lanes), scale = ue8m0_rp(amax * (1/448)), payload = e4m3(x * 2^-(e-127))
// -------------------------------------------------------------------------------------------------
template <typename T, bool SWIZZLE>
__global__ __launch_bounds__(256) void mxfp8_quantize_kernel(const T* __restrict__ in, int64_t rows, int64_t cols,
                                                             uint8_t* __restrict__ out_fp8,
                                                             uint8_t* __restrict__ out_sf) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t row0 = (int64_t)blockIdx.y * 32;
  const int64_t col = (int64_t)blockIdx.x * kSegCols + lane * 8;
  const bool col_ok = col < cols;
  const int64_t sf_cols = cols >> 5;
  const int64_t padded = (sf_cols + 3) & ~(int64_t)3;
  const int64_t sf_col = col >> 5;
  const bool word_stores = SWIZZLE || (sf_cols & 3) == 0;

#pragma unroll 1
  for (int t = 0; t < 8; ++t) {
    const int64_t row = row0 + t * 4 + wave;
    const bool active = col_ok && row < rows;
    float x[8];
    bool nan = false;
    if (active) {
      load8(in + row * cols + col, x, nan);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = 0.0f;
    }
    const bool wave_has_nan = __builtin_amdgcn_ballot_w64(nan) != 0;  // any non-finite input in the wavefront
    float m = amax8(x);
    m = fmaxf(m, bits_to_f32(dpp_xor1(f32_to_bits(m))));
    m = fmaxf(m, bits_to_f32(dpp_xor2(f32_to_bits(m))));
    const uint32_t e = f32_to_e8m0_rp(m * (1.0f / 448));                   // :168-169
    const float inv = (e == 0) ? 1.0f : bits_to_f32((254u - e) << 23);     // :134-140
    uint32_t lo = 0, hi = 0;
    if (!wave_has_nan) {
      float y[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = __builtin_amdgcn_fmed3f(x[j] * inv, -448.0f, 448.0f);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], lo, false);
      lo = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], lo, true);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], hi, false);
      hi = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], hi, true);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lo |= f32_to_e4m3_satfinite(x[j] * inv) << (8 * j);
        hi |= f32_to_e4m3_satfinite(x[4 + j] * inv) << (8 * j);
      }
    }
    if (active) *reinterpret_cast<uint2*>(out_fp8 + row * cols + col) = make_uint2(lo, hi);

    if (word_stores) {
      uint32_t v = ((lane & 3) || !active) ? 0u : (e << (8 * ((lane >> 2) & 3)));
      v |= dpp_shl4(v);
      v |= dpp_shl8(v);
      if ((lane & 15) == 0 && col_ok) {
        if constexpr (SWIZZLE) {
          *reinterpret_cast<uint32_t*>(out_sf + swizzle_128x4(row, sf_col, padded)) = v;
        } else {
          if (row < rows) *reinterpret_cast<uint32_t*>(out_sf + row * sf_cols + sf_col) = v;
        }
      }
    } else {
      if (active && !(lane & 3)) out_sf[row * sf_cols + sf_col] = (uint8_t)e;
    }
  }
}

template <typename T>
int launch_mxfp8_typed(const T* in, int64_t rows, int64_t cols, int swizzle, uint8_t* out_fp8, uint8_t* out_sf,
                       hipStream_t stream) {
  const unsigned gx = (unsigned)ceil_div(cols, kSegCols);
  if (swizzle) {
    dim3 grid(gx, (unsigned)(round_up(rows, 128) / 32));
    hipLaunchKernelGGL((mxfp8_quantize_kernel<T, true>), grid, dim3(256), 0, stream, in, rows, cols, out_fp8, out_sf);
  } else {
    dim3 grid(gx, (unsigned)ceil_div(rows, 32));
    hipLaunchKernelGGL((mxfp8_quantize_kernel<T, false>), grid, dim3(256), 0, stream, in, rows, cols, out_fp8, out_sf);
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
      return launch_nvfp4_typed(static_cast<const float*>(in), rows, cols, gs, layout, in_off, out_off, groups, q, s, stream);
    case NVF_BF16:
      return launch_nvfp4_typed(static_cast<const bf16_t*>(in), rows, cols, gs, layout, in_off, out_off, groups, q, s, stream);
    case NVF_F16:
      return launch_nvfp4_typed(static_cast<const f16_t*>(in), rows, cols, gs, layout, in_off, out_off, groups, q, s, stream);
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

int launch_cast(int kind, const float* in, int64_t n, uint8_t* out, hipStream_t stream) {
  if (n == 0) return NVF_OK;
  dim3 grid((unsigned)ceil_div(n, 256));
  if (kind == 0) hipLaunchKernelGGL(cast_kernel<0>, grid, dim3(256), 0, stream, in, n, out);
  else if (kind == 1) hipLaunchKernelGGL(cast_kernel<1>, grid, dim3(256), 0, stream, in, n, out);
  else hipLaunchKernelGGL(cast_kernel<2>, grid, dim3(256), 0, stream, in, n, out);
  return check_launch("cast_kernel");
}

}  // namespace nvf
