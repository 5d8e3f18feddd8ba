// mxfp8_scaled_mm for gfx950 (cutlass/mxfp8_scaled_mm.cu:290-319): C = alpha * A * B^T with e4m3
// operands and one e8m0 scale per 32 K-elements, on v_mfma_scale_f32_32x32x64_f8f6f4.
//
// Operand layout of the instruction (fp8 x fp8), measured on hardware:
//   lane l = i + 32*g (i = row of A / column of B, g in {0,1}) supplies 32 bytes:
//     bytes  0..15 = K [16g,      16g + 16)
//     bytes 16..31 = K [32 + 16g, 32 + 16g + 16)
//   and the scale byte of lane i + 32*j applies to row i, K-block j (K [32j, 32j+32)).
// The 128x4 scale layout stores, for 32 consecutive rows, 16 bytes per row position holding
// (rows r, r+32, r+64, r+96) x (4 consecutive K-blocks): one 16-byte load per lane fetches every
// scale a 128-row wave tile needs for a 128-deep K step.
#include "nvf_internal.h"

namespace nvf {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct Params {
  const uint8_t* a;
  const uint8_t* b;
  const uint8_t* sfa;
  const uint8_t* sfb;
  const float* alpha;
  void* out;
  int m, n, k;
};

__device__ __forceinline__ uint32_t pack2(float a, float b, bool out_bf16) {
  if (out_bf16) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, v);
  }
  f16x2 v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ int lds_pos(int row, int chunk) { return row * 8 + (chunk ^ (row & 7)); }

template <int BM, int BN, bool OUT_BF16>
__global__ __launch_bounds__(256) void mxfp8_gemm_kernel(const Params p) {
  constexpr int BK = 128;  // bytes == elements
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  extern __shared__ u32x4 lds[];
  u32x4* lds_a = lds;
  u32x4* lds_b = lds + BM * 8;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lg = lane >> 5;

  const int tiles_m = (p.m + BM - 1) / BM;
  const int mt = blockIdx.x % tiles_m, nt = blockIdx.x / tiles_m;
  const int m0 = mt * BM, n0 = nt * BN;
  const int sf_cols = p.k / 32;
  const int sf_padded = (sf_cols + 3) & ~3;
  const int nk = (p.k + BK - 1) / BK;

  const uint8_t* a_base = p.a + (int64_t)m0 * p.k;
  const uint8_t* b_base = p.b + (int64_t)n0 * p.k;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  constexpr int A_TOTAL = BM * 8, B_TOTAL = BN * 8;
  constexpr int A_CH = (A_TOTAL + 255) / 256, B_CH = (B_TOTAL + 255) / 256;
  u32x4 sa[A_CH], sb[B_CH];
  // scale words: [sub-tile] -> 4 e8m0 bytes (K-blocks of this 128-deep step) of row (sub-tile*32 + li)
  uint32_t sca[TM], scb[TN], sca_next[TM], scb_next[TN];

  auto issue_loads = [&](int ks) {
    const int kb0 = ks * BK;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, chunk = c & 7;
      const bool ok = (c < A_TOTAL) && (m0 + row < p.m) && (kb0 + chunk * 16 < p.k);
      sa[i] = u32x4{0, 0, 0, 0};
      if (ok) sa[i] = *reinterpret_cast<const u32x4*>(a_base + (int64_t)row * p.k + kb0 + chunk * 16);
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, chunk = c & 7;
      const bool ok = (c < B_TOTAL) && (n0 + row < p.n) && (kb0 + chunk * 16 < p.k);
      sb[i] = u32x4{0, 0, 0, 0};
      if (ok) sb[i] = *reinterpret_cast<const u32x4*>(b_base + (int64_t)row * p.k + kb0 + chunk * 16);
    }
    // Scales of rows past m / n and of K-blocks past k belong to zero payload; they are forced to
    // 2^0 (0x7F) so that padding bytes (possibly the NaN code 0xFF) never meet the zeros.
    const int valid_blocks = sf_cols - ks * 4;  // >= 1
    const uint32_t keep = valid_blocks >= 4 ? 0xffffffffu : ((1u << (8 * valid_blocks)) - 1u);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = m0 + wm * WTM + i * 32 + li;
      uint32_t w = 0;
      if (row < p.m) w = *reinterpret_cast<const uint32_t*>(p.sfa + swizzle_128x4(row, ks * 4, sf_padded)) & keep;
      else w = 0x7f7f7f7fu & keep;
      sca_next[i] = w | (0x7f7f7f7fu & ~keep);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = n0 + wn * WTN + j * 32 + li;
      uint32_t w = 0;
      if (row < p.n) w = *reinterpret_cast<const uint32_t*>(p.sfb + swizzle_128x4(row, ks * 4, sf_padded)) & keep;
      else w = 0x7f7f7f7fu & keep;
      scb_next[j] = w | (0x7f7f7f7fu & ~keep);
    }
  };

  issue_loads(0);
  for (int ks = 0; ks < nk; ++ks) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + 256 * i;
      if (c < A_TOTAL) lds_a[lds_pos(c >> 3, c & 7)] = sa[i];
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + 256 * i;
      if (c < B_TOTAL) lds_b[lds_pos(c >> 3, c & 7)] = sb[i];
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) sca[i] = sca_next[i];
#pragma unroll
    for (int j = 0; j < TN; ++j) scb[j] = scb_next[j];
    __syncthreads();
    if (ks + 1 < nk) issue_loads(ks + 1);

#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      i32x8 fa[TM], fb[TN];
      const int c_lo = sub * 4 + lg, c_hi = sub * 4 + 2 + lg;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm * WTM + i * 32 + li;
        const u32x4 lo = lds_a[lds_pos(row, c_lo)], hi = lds_a[lds_pos(row, c_hi)];
        fa[i] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn * WTN + j * 32 + li;
        const u32x4 lo = lds_b[lds_pos(row, c_lo)], hi = lds_b[lds_pos(row, c_hi)];
        fb[j] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
      // K-block of this lane inside the 128-deep step: 2*sub + lg
      const int sh = 8 * (2 * sub + lg);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int s_a = (int)((sca[i] >> sh) & 0xffu);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int s_b = (int)((scb[j] >> sh) & 0xffu);
          // B fragment first: the accumulator then holds 4 consecutive N-elements per register quad
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, s_b, 0, s_a);
        }
      }
    }
  }

  const float alpha = p.alpha[0];
  uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int mrow = m0 + wm * WTM + i * 32 + li;
    if (mrow >= p.m) continue;
    uint16_t* orow = out + (int64_t)mrow * p.n;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int ncol = n0 + wn * WTN + j * 32 + rq * 8 + lg * 4;
        if (ncol < p.n) {
          u32x2 v;
          v[0] = pack2(acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha, OUT_BF16);
          v[1] = pack2(acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha, OUT_BF16);
          *reinterpret_cast<u32x2*>(orow + ncol) = v;
        }
      }
    }
  }
}

template <int BM, int BN, bool OUT_BF16>
int launch_cfg(const Params& p, hipStream_t stream) {
  auto kern = mxfp8_gemm_kernel<BM, BN, OUT_BF16>;
  constexpr int lds_bytes = (BM + BN) * 128;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail(NVF_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    configured = true;
  }
  const int64_t tiles = ceil_div(p.m, BM) * ceil_div(p.n, BN);
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), lds_bytes, stream, p);
  return check_launch("mxfp8_gemm_kernel");
}

template <bool OUT_BF16>
int launch_sized(const Params& p, hipStream_t stream) {
  auto tiles = [&](int bm, int bn) { return ceil_div(p.m, bm) * ceil_div(p.n, bn); };
  if (tiles(256, 256) >= 256) return launch_cfg<256, 256, OUT_BF16>(p, stream);
  if (tiles(128, 128) >= 256) return launch_cfg<128, 128, OUT_BF16>(p, stream);
  return launch_cfg<64, 64, OUT_BF16>(p, stream);
}

}  // namespace

int launch_mxfp8_gemm(const void* a, const void* b, const void* sfa, const void* sfb, const float* alpha, void* out,
                      int64_t m, int64_t n, int64_t k, int out_dtype, hipStream_t stream) {
  if (m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "dimension exceeds int32");
  Params p{static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), static_cast<const uint8_t*>(sfa),
           static_cast<const uint8_t*>(sfb), alpha, out, (int)m, (int)n, (int)k};
  return out_dtype == NVF_BF16 ? launch_sized<true>(p, stream) : launch_sized<false>(p, stream);
}

}  // namespace nvf
