// GEMMs whose MFMA operands are 16-bit floats, for gfx950:
//   * nvfp4_scaled_mm          (cutlass/nvfp4_scaled_mm.cu:283-312)
//   * nvfp4_scaled_grouped_mm  (cutlass/nvfp4_scaled_group_mm.cu:714-788, pointer rule :83-155)
//   * grouped_mm               (cutlass/group_mm.cu:518-571, pointer rule :76-105)
//
// NVFP4 has one e4m3 scale per 16 elements, which the block-32 / e8m0 scaled MFMA of gfx950 cannot
// express.  An e2m1 value times an e4m3 scale has at most 6 significant bits and an exponent range
// of 2^-10 .. 2^11, so it is exactly representable in fp16: tiles are dequantised to fp16 while
// they are staged into LDS and fed to v_mfma_f32_32x32x16_f16 with fp32 accumulation.  Every
// product is exact; only the fp32 accumulation order differs from any other correct implementation.
//
// The tile kernels (one for 16-bit operands, one for NVFP4) are persistent: a workgroup walks (group,
// m-tile, n-tile) work items whose list is derived on the device from problem_sizes, so no host
// synchronisation is needed and empty groups cost nothing.  The dense op is the one-group case.
// Specialised kernels take the shapes they fit: 256x256 persistent NVFP4 and grouped 16-bit kernels,
// and a weight-streaming NVFP4 kernel for up to 128 activation rows.
//
// Output layout trick: the MFMA is issued with the B fragment as first operand, so that a lane's
// accumulator registers hold 4 consecutive N-elements of one output row and are stored as 8 bytes.
#include "nvf_internal.h"

#include <mutex>

namespace nvf {
namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMaxGroups = 1024;  // same bound as the reference's <<<1, num_experts>>> set-up kernel

struct Params {
  const uint8_t* a;
  const uint8_t* b;
  const uint8_t* sfa;
  const uint8_t* sfb;
  const float* alpha;
  void* out;
  const int32_t* problem_sizes;   // nullptr => dense
  const int32_t* expert_offsets;
  const int32_t* sf_offsets;
  int groups;
  int m, n, k;
  // split of K over workgroups (dense NVFP4 tile kernel only): work item w = tile w / splits, K spans
  // [ (w % splits) * spans_per_split, ... ); fp32 partial tiles go to partial[split][m][n]
  float* partial = nullptr;
  int splits = 1;
  int spans_per_split = 0;
  // NVFP4 tile kernel, grouped: 1 = rows [0, rows & ~255) of every group are computed by the 256x256 kernel,
  // take only the rows after them
  int skip_whole_256 = 0;
  // skinny kernel: first activation row this launch computes (its slabs of 16*TT rows follow in blockIdx.y order)
  int m_base = 0;
  // grouped skinny kernel: the group sizes it serves; the tile kernel skips groups of fewer than min_rows rows
  int rows_lo = 0, rows_hi = 0, min_rows = 0;
  int tail_done = 0;  // grouped NVFP4 dispatch: the ends of the large groups have been computed by an earlier launch
  // block-scaled result (nvfp4_scaled_mm_blockscale): out = packed e2m1 [m, n/2], out_sf = e4m3 scales in the 128x4
  // layout of [roundUp(m,128), roundUp(n/16,4)], gnorm = the result's global (encode) scale on the device
  uint8_t* out_sf = nullptr;
  const float* gnorm = nullptr;
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

// LDS tile: rows x 64 16-bit elements (128 bytes per row); 16-byte chunk c of row r sits at chunk
// position c ^ ((r >> 1) & 7): two rows fill the 64 banks once, so the MFMA fragment reads (16
// consecutive lanes = 16 consecutive rows, one chunk) are conflict-free.
__device__ __forceinline__ int lds_pos2(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }
__device__ __forceinline__ int lds_pos(int row, int chunk) { return lds_pos2(row, chunk); }

// Block-scaled epilogue (cutlass/nvfp4_scaled_mm_blockscale.cu:87-93: the product is quantized to NVFP4 again along
// N before it leaves the kernel).  One 32x32 accumulator tile: lane (li, lg) holds row li, columns 8q + 4lg + e in
// register 4q + e, so each of the row's two 16-column blocks is shared by the lanes (li, 0) and (li, 1): amax over
// the lane's 8 values, one exchange with lane ^ 32, then the block quantizer's arithmetic
// (runtime/block_quantization_kernels.cu:224-263) on alpha * acc.  For block b both lanes get the scale code q8[b];
// h[b] holds this lane's 4 of the block's 8 payload bytes: bits 0..15 = bytes 2lg, 2lg+1, bits 16..31 = bytes
// 4+2lg, 5+2lg.  Must be called by whole wavefronts.
__device__ __forceinline__ void quantize_acc_tile(const f32x16& acc, float alpha, float gs, float decode, bool active, uint32_t h[2],
                                                  uint32_t q8[2]) {
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    float x[8];
    float m = -INFINITY;
    bool nonfinite = false;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      x[e] = acc[8 * b + e] * alpha;
      m = fmaxf(m, fabsf(x[e]));  // NaN ignored, as the quantizer does
      nonfinite |= !(fabsf(x[e]) < INFINITY);
    }
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    m = fmaxf(m, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, m))));
    float r;
    q8[b] = nvfp4_block_scale(m, true, gs, decode, active, r);
    uint32_t w = 0;
    if (__builtin_amdgcn_ballot_w64(nonfinite) == 0) {
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[0] * r, x[1] * r, 1.0f, 0);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[2] * r, x[3] * r, 1.0f, 1);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[4] * r, x[5] * r, 1.0f, 2);
      w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[6] * r, x[7] * r, 1.0f, 3);
    } else {  // explicit NaN rule of the narrow cast
#pragma unroll
      for (int t = 0; t < 4; ++t) w |= f32x2_to_e2m1_byte(x[2 * t] * r, x[2 * t + 1] * r) << (8 * t);
    }
    h[b] = w;
  }
}

// fills n bytes with zero (the padding of the block-scaled result's scale buffer for ragged shapes)
__global__ __launch_bounds__(256) void zero_fill_kernel(uint32_t* __restrict__ dst, int64_t words) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < words) dst[i] = 0u;
}

template <int BM, int BN, bool BF16_MMA, bool OUT_BF16>
__global__ __launch_bounds__(256) void gemm16_kernel(const Params p) {
  constexpr int BK = 64;
  constexpr int WTM = BM / 2, WTN = BN / 2;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  extern __shared__ u32x4 lds[];  // two buffers of (A tile, B tile)
  constexpr int BUF_UNITS = (BM + BN) * 8;
  __shared__ int tile_prefix[kMaxGroups + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.n + BN - 1) / BN;
  const bool dense = p.problem_sizes == nullptr;

  // ---- work list: prefix sums of tiles per group ----
  if (dense) {
    if (tid == 0) {
      tile_prefix[0] = 0;
      tile_prefix[1] = ((p.m + BM - 1) / BM) * tiles_n;
    }
  } else {
    // serial scan by one wavefront in chunks of 64 groups
    if (wave == 0) {
      int running = 0;
      for (int base = 0; base < p.groups; base += 64) {
        const int g = base + lane;
        int cnt = 0;
        if (g < p.groups) {
          const int mg = p.problem_sizes[g * 3];
          cnt = mg > 0 ? ((mg + BM - 1) / BM) * tiles_n : 0;
        }
        int incl = cnt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int o = __shfl_up(incl, d, 64);
          if (lane >= d) incl += o;
        }
        if (g < p.groups) tile_prefix[g + 1] = running + incl;
        running += __shfl(incl, 63, 64);
      }
      if (lane == 0) tile_prefix[0] = 0;
    }
  }
  __syncthreads();
  const int total_tiles = tile_prefix[p.groups];

  const int kbytes = p.k * 2;  // bytes per operand row
  const int nk = (p.k + BK - 1) / BK;

  for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
    // ---- decode work item ----
    int g = 0;
    {
      int lo = 0, hi = p.groups;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile < tile_prefix[mid]) hi = mid; else lo = mid;
      }
      g = lo;
    }
    const int m_g = dense ? p.m : p.problem_sizes[g * 3];
    const int64_t row_off = dense ? 0 : p.expert_offsets[g];
    const int tiles_m = (m_g + BM - 1) / BM;
    const int local = tile - tile_prefix[g];
    const int mt = local % tiles_m, nt = local / tiles_m;
    const int m0 = mt * BM, n0 = nt * BN;

    const uint8_t* a_base = p.a + (row_off + m0) * (int64_t)kbytes;
    const uint8_t* b_base = p.b + ((int64_t)g * p.n + n0) * (int64_t)kbytes;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // ---- staging registers ----
    constexpr int A_TOTAL = BM * 8;  // 16-byte global chunks per tile
    constexpr int B_TOTAL = BN * 8;
    constexpr int A_CH = (A_TOTAL + 255) / 256;       // ... per thread
    constexpr int B_CH = (B_TOTAL + 255) / 256;
    u32x4 sa[A_CH], sb[B_CH];

    auto issue_loads = [&](int ks) {
      const int kbyte0 = ks * (BK * 2);
#pragma unroll
      for (int i = 0; i < A_CH; ++i) {
        const int c = tid + 256 * i;
        const int row = c >> 3, chunk = c & 7;
        const bool ok = (c < A_TOTAL) && (m0 + row < m_g) && (kbyte0 + chunk * 16 < kbytes);
        sa[i] = u32x4{0, 0, 0, 0};
        if (ok) sa[i] = *reinterpret_cast<const u32x4*>(a_base + (int64_t)row * kbytes + kbyte0 + chunk * 16);
      }
#pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        const int c = tid + 256 * i;
        const int row = c >> 3, chunk = c & 7;
        const bool ok = (c < B_TOTAL) && (n0 + row < p.n) && (kbyte0 + chunk * 16 < kbytes);
        sb[i] = u32x4{0, 0, 0, 0};
        if (ok) sb[i] = *reinterpret_cast<const u32x4*>(b_base + (int64_t)row * kbytes + kbyte0 + chunk * 16);
      }
    };

    auto store_lds = [&](int buf) {
      u32x4* lds_a = lds + buf * BUF_UNITS;
      u32x4* lds_b = lds_a + BM * 8;
#pragma unroll
      for (int i = 0; i < A_CH; ++i) {
        const int c = tid + 256 * i;
        if (c >= A_TOTAL) break;
        lds_a[lds_pos(c >> 3, c & 7)] = sa[i];
      }
#pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        const int c = tid + 256 * i;
        if (c >= B_TOTAL) break;
        lds_b[lds_pos(c >> 3, c & 7)] = sb[i];
      }
    };

    // K loop: the loads of step ks+1 are in flight under the MFMAs of step ks, then converted into the
    // other LDS buffer; one barrier per step
    issue_loads(0);
    store_lds(0);  // every wave is past the barrier that ended the previous tile's last step
    __syncthreads();
    for (int ks = 0; ks < nk; ++ks) {
      const u32x4* lds_a = lds + (ks & 1) * BUF_UNITS;
      const u32x4* lds_b = lds_a + BM * 8;
      if (ks + 1 < nk) issue_loads(ks + 1);

#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        u32x4 fa[TM], fb[TN];
        const int chunk = kk * 2 + (lane >> 5);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = lds_a[lds_pos(wm * WTM + i * 32 + (lane & 31), chunk)];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = lds_b[lds_pos(wn * WTN + j * 32 + (lane & 31), chunk)];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if constexpr (BF16_MMA) {
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[j]),
                                                                  __builtin_bit_cast(bf16x8, fa[i]), acc[i][j], 0, 0, 0);
            } else {
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fb[j]),
                                                                 __builtin_bit_cast(f16x8, fa[i]), acc[i][j], 0, 0, 0);
            }
          }
      }
      if (ks + 1 < nk) store_lds((ks + 1) & 1);
      __syncthreads();
    }

    // ---- epilogue: acc[i][j][r] = C[m = lane%32][n = (r/4)*8 + (lane/32)*4 + r%4] of its 32x32 tile ----
    uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mrow = m0 + wm * WTM + i * 32 + (lane & 31);
      if (mrow >= m_g) continue;
      uint16_t* orow = out + (row_off + mrow) * (int64_t)p.n;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int ncol = n0 + wn * WTN + j * 32 + rq * 8 + (lane >> 5) * 4;
          if (ncol < p.n) {
            u32x2 v;
            v[0] = pack2(acc[i][j][rq * 4 + 0], acc[i][j][rq * 4 + 1], OUT_BF16);
            v[1] = pack2(acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3], OUT_BF16);
            *reinterpret_cast<u32x2*>(orow + ncol) = v;
          }
        }
      }
    }
  }
}

// Grouped NVFP4: the rows of a group of m_g rows that the 256x256 kernel computes: its whole 256-row tiles, and a
// last tile of more than 128 rows (its missing rows read as zero through the buffer range and are not stored).
// The tile kernel takes the rows from there on; a value >= m_g means none are left.
__device__ __forceinline__ int rows_in_256_tiles(int m_g) {
  const int whole = m_g & ~255;
  return m_g - whole > 128 ? whole + 256 : whole;
}

// -------------------------------------------------------------------------------------------------
// NVFP4 tile kernel for every shape the specialised NVFP4 kernels below do not take (ragged sizes, groups,
// fp32 result).  Same persistent walk over (group, m-tile, n-tile) items, LDS layout and MFMA loop as the
// kernel above; what differs is how operands get from global memory into LDS:
//   * Loads cover a span of 128 elements of K (two 64-deep steps): thread unit c = row c/4, 16-byte piece
//     c%4, so four neighbouring lanes read 64 contiguous bytes of a row, and one dword load fetches the
//     scales of a row's four blocks (the two lanes that share a dword pick their half).  A load whose
//     lanes each touch a different cache line keeps the address unit busy for 64 cycles; with 32 bytes
//     per row and two-byte scale loads per step that, not the MFMAs, bounded this kernel.
//   * Of each 16-byte piece (two scale blocks) the first block is consumed by the even step of the span and
//     the second by the odd step: the same permutation of K for both operands, so the dot products are
//     unchanged and every lane converts in every step.
//   * The span after the current one is requested at the start of the even step and first needed when the
//     odd step converts its even half: a full step of MFMAs hides the latency.
// Requires K % 32 == 0 (a piece never straddles the end of a row).
// -------------------------------------------------------------------------------------------------
template <int BM, int BN, bool OUT_BF16, bool OUT_F32, bool SPLIT_K = false, bool OUT_FP4 = false>
__global__ __launch_bounds__(256) void nvfp4_tile_kernel(const Params p) {
  constexpr int WTM = BM / 2, WTN = BN / 2;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  extern __shared__ u32x4 lds[];  // two buffers of (A tile, B tile), 64 fp16 of K per row
  constexpr int BUF_UNITS = (BM + BN) * 8;
  __shared__ int tile_prefix[kMaxGroups + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.n + BN - 1) / BN;
  const bool dense = p.problem_sizes == nullptr;

  if (dense) {
    if (tid == 0) {
      tile_prefix[0] = 0;
      tile_prefix[1] = ((p.m + BM - 1) / BM) * tiles_n;
    }
  } else if (wave == 0) {  // serial scan in chunks of 64 groups
    int running = 0;
    for (int base = 0; base < p.groups; base += 64) {
      const int g = base + lane;
      int cnt = 0;
      if (g < p.groups) {
        const int mg = p.problem_sizes[g * 3];
        const int rest = mg < p.min_rows ? 0 : mg - (p.skip_whole_256 ? rows_in_256_tiles(mg) : 0);
        cnt = rest > 0 ? ((rest + BM - 1) / BM) * tiles_n : 0;
      }
      int incl = cnt;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (g < p.groups) tile_prefix[g + 1] = running + incl;
      running += __shfl(incl, 63, 64);
    }
    if (lane == 0) tile_prefix[0] = 0;
  }
  __syncthreads();
  const int splits = SPLIT_K ? p.splits : 1;
  const int total_tiles = tile_prefix[p.groups] * splits;

  const int kbytes = p.k >> 1;
  const int sf_cols = p.k >> 4;
  const int sf_padded = (sf_cols + 3) & ~3;
  const int nspans = (p.k + 127) >> 7;

  constexpr int A_CH = BM / 64, B_CH = BN / 64;  // 16-byte pieces per thread and span
  struct Raw { u32x4 a[A_CH], b[B_CH]; uint32_t sa[A_CH], sb[B_CH]; };
  const int urow = tid >> 2, upiece = tid & 3;  // unit i of a thread: row urow + 64 * i

  for (int item = blockIdx.x; item < total_tiles; item += gridDim.x) {
    const int tile = SPLIT_K ? item / splits : item;
    const int split = SPLIT_K ? item - tile * splits : 0;
    const int span0 = SPLIT_K ? split * p.spans_per_split : 0;                       // this item's K spans
    const int span1 = SPLIT_K ? min(span0 + p.spans_per_split, nspans) : nspans;     // (never empty)
    int g = 0;
    {
      int lo = 0, hi = p.groups;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile < tile_prefix[mid]) hi = mid; else lo = mid;
      }
      g = lo;
    }
    const int m_g = dense ? p.m : p.problem_sizes[g * 3];
    const int64_t row_off = dense ? 0 : p.expert_offsets[g];
    const int skipped = (!dense && p.skip_whole_256) ? rows_in_256_tiles(m_g) : 0;
    const int tiles_m = (m_g - skipped + BM - 1) / BM;
    const int local = tile - tile_prefix[g];
    const int mt = local % tiles_m, nt = local / tiles_m;
    const int m0 = skipped + mt * BM, n0 = nt * BN;

    const uint8_t* a_base = p.a + (row_off + m0) * (int64_t)kbytes;
    const uint8_t* b_base = p.b + ((int64_t)g * p.n + n0) * (int64_t)kbytes;
    const uint8_t* sfa_base = p.sfa + (dense ? 0 : (int64_t)p.sf_offsets[g]) * sf_cols;  // group slab, swizzled on its own
    const uint8_t* sfb_base = p.sfb + (int64_t)g * p.n * sf_cols;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto issue_span = [&](Raw& r, int sp) {
      const int kb = sp * 64 + upiece * 16;            // byte in the row
      const int sf_col = sp * 8 + (upiece >> 1) * 4;   // first of the 4 blocks the dword covers
      const bool k_ok = kb < kbytes;
#pragma unroll
      for (int i = 0; i < A_CH; ++i) {
        const int row = urow + 64 * i;
        const bool ok = k_ok && (m0 + row < m_g);
        r.a[i] = u32x4{0, 0, 0, 0};
        r.sa[i] = 0;
        if (ok) {
          r.a[i] = *reinterpret_cast<const u32x4*>(a_base + (int64_t)row * kbytes + kb);
          r.sa[i] = *reinterpret_cast<const uint32_t*>(sfa_base + swizzle_128x4(m0 + row, sf_col, sf_padded));
        }
      }
#pragma unroll
      for (int i = 0; i < B_CH; ++i) {
        const int row = urow + 64 * i;
        const bool ok = k_ok && (n0 + row < p.n);
        r.b[i] = u32x4{0, 0, 0, 0};
        r.sb[i] = 0;
        if (ok) {
          r.b[i] = *reinterpret_cast<const u32x4*>(b_base + (int64_t)row * kbytes + kb);
          r.sb[i] = *reinterpret_cast<const uint32_t*>(sfb_base + swizzle_128x4(n0 + row, sf_col, sf_padded));
        }
      }
    };

    // block `parity` of every piece -> fp16 -> LDS buffer buf (chunks 2*piece, 2*piece+1 of the row)
    auto convert_one = [&](u32x4 q, uint32_t s4, int parity, u32x4* dst_tile, int row) {
      const uint32_t s2 = s4 >> ((upiece & 1) * 16);  // this piece's two scale bytes
      const float f = parity ? __builtin_amdgcn_cvt_f32_fp8((int)s2, 1) : __builtin_amdgcn_cvt_f32_fp8((int)s2, 0);
      const f16x2 sv = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f, f));  // exact: e4m3 fits fp16
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        const uint32_t w = q[2 * parity + cc];
        const f16x2 h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 0) * sv;
        const f16x2 h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 1) * sv;
        const f16x2 h2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 2) * sv;
        const f16x2 h3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 1.0f, 3) * sv;
        dst_tile[lds_pos2(row, upiece * 2 + cc)] = u32x4{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                                                         __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3)};
      }
    };
    auto convert = [&](const Raw& r, int parity, int buf) {
      u32x4* lds_a = lds + buf * BUF_UNITS;
      u32x4* lds_b = lds_a + BM * 8;
#pragma unroll
      for (int i = 0; i < A_CH; ++i) convert_one(r.a[i], r.sa[i], parity, lds_a, urow + 64 * i);
#pragma unroll
      for (int i = 0; i < B_CH; ++i) convert_one(r.b[i], r.sb[i], parity, lds_b, urow + 64 * i);
    };
    auto mfma_step = [&](int buf) {
      const u32x4* lds_a = lds + buf * BUF_UNITS;
      const u32x4* lds_b = lds_a + BM * 8;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        u32x4 fa[TM], fb[TN];
        const int chunk = kk * 2 + (lane >> 5);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = lds_a[lds_pos2(wm * WTM + i * 32 + (lane & 31), chunk)];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = lds_b[lds_pos2(wn * WTN + j * 32 + (lane & 31), chunk)];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fb[j]), __builtin_bit_cast(f16x8, fa[i]),
                                                               acc[i][j], 0, 0, 0);
      }
    };

    Raw cur, nxt;
    issue_span(cur, span0);
    convert(cur, 0, 0);  // every wave is past the barrier that ended the previous tile's last step
    __syncthreads();
    // one span: `c` holds it (its even step is in buffer 0 already), `n` takes the span after it; with the larger
    // tiles the two register sets swap names from span to span, so no span is copied
    auto one_span = [&](Raw& c, Raw& n, int sp) {
      const bool more = sp + 1 < span1;
      if (more) issue_span(n, sp + 1);
      mfma_step(0);
      convert(c, 1, 1);
      __syncthreads();
      mfma_step(1);
      if (more) convert(n, 0, 0);
      __syncthreads();
    };
    if constexpr (BM >= 128 && !SPLIT_K) {
      int sp = span0;
      for (; sp + 1 < span1; sp += 2) {
        one_span(cur, nxt, sp);
        one_span(nxt, cur, sp + 1);
      }
      if (sp < span1) one_span(cur, nxt, sp);
    } else {  // (small tiles and short K ranges: measured slower with the doubled loop body)
      for (int sp = span0; sp < span1; ++sp) {
        one_span(cur, nxt, sp);
        cur = nxt;
      }
    }

    // ---- epilogue: acc[i][j][r] = C[m = lane%32][n = (r/4)*8 + (lane/32)*4 + r%4] of its 32x32 tile ----
    const float alpha = SPLIT_K ? 1.0f : (dense ? p.alpha[0] : p.alpha[g]);  // split: applied by the reduction
    if constexpr (OUT_FP4) {
      // block-scaled result: every 32x32 accumulator tile becomes 32 rows x 16 payload bytes and 32 x 2 scale bytes
      // (N % 32 == 0: a tile's columns exist or not as a whole)
      const float gs = p.gnorm[0], decode = 1.0f / gs;
      const int sf_out_padded = ((p.n >> 4) + 3) & ~3;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int mrow = m0 + wm * WTM + i * 32 + (lane & 31);
        const bool row_ok = mrow < m_g;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int ncol = n0 + wn * WTN + j * 32;
          if (ncol >= p.n) continue;  // wave-uniform
          uint32_t h[2], q8[2];
          quantize_acc_tile(acc[i][j], alpha, gs, decode, row_ok, h, q8);
          if (row_ok) {
            uint8_t* orow = static_cast<uint8_t*>(p.out) + (int64_t)mrow * (p.n >> 1) + (ncol >> 1) + 2 * (lane >> 5);
#pragma unroll
            for (int b = 0; b < 2; ++b) {
              *reinterpret_cast<uint16_t*>(orow + b * 8) = (uint16_t)(h[b] & 0xffffu);
              *reinterpret_cast<uint16_t*>(orow + b * 8 + 4) = (uint16_t)(h[b] >> 16);
            }
            if ((lane >> 5) == 0)
              *reinterpret_cast<uint16_t*>(p.out_sf + swizzle_128x4(mrow, ncol >> 4, sf_out_padded)) = (uint16_t)(q8[0] | (q8[1] << 8));
          }
        }
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mrow = m0 + wm * WTM + i * 32 + (lane & 31);
      if (mrow >= m_g) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int ncol = n0 + wn * WTN + j * 32 + rq * 8 + (lane >> 5) * 4;
          if (ncol >= p.n) continue;
          if constexpr (SPLIT_K) {
            float* frow = p.partial + ((int64_t)split * p.m + mrow) * (int64_t)p.n;
            *reinterpret_cast<f32x4*>(frow + ncol) =
                f32x4{acc[i][j][rq * 4 + 0], acc[i][j][rq * 4 + 1], acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3]};
          } else if constexpr (OUT_F32) {
            float* frow = static_cast<float*>(p.out) + (row_off + mrow) * (int64_t)p.n;
            *reinterpret_cast<f32x4*>(frow + ncol) = f32x4{acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha,
                                                           acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha};
          } else {
            uint16_t* orow = static_cast<uint16_t*>(p.out) + (row_off + mrow) * (int64_t)p.n;
            u32x2 v;
            v[0] = pack2(acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha, OUT_BF16);
            v[1] = pack2(acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(orow + ncol) = v;
          }
        }
      }
    }
  }
}

// out[m][n] = alpha * (partial[0][m][n] + partial[1][m][n] + ...), summed in that order
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits, int64_t mn,
                                                            const float* __restrict__ alpha_ptr, uint16_t* __restrict__ out) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= mn) return;  // mn % 4 == 0 (N % 32 == 0)
  f32x4 s = *reinterpret_cast<const f32x4*>(partial + i);
  for (int k = 1; k < splits; ++k) s += *reinterpret_cast<const f32x4*>(partial + (int64_t)k * mn + i);
  const float alpha = alpha_ptr[0];
  u32x2 v;
  v[0] = pack2(s[0] * alpha, s[1] * alpha, OUT_BF16);
  v[1] = pack2(s[2] * alpha, s[3] * alpha, OUT_BF16);
  *reinterpret_cast<u32x2*>(out + i) = v;
}

// -------------------------------------------------------------------------------------------------
// NVFP4 fast path: 256x256 (or 128x256) tile, N % 256 == 0, K % 128 == 0, K >= 256; dense with M % 256 (128) == 0,
// or the whole 256-row tiles of every group of the grouped op; 16-bit or fp32 result.
//   * 512 threads: 8 wavefronts as 2 (m) x 4 (n), each with a 128x64 (64x64) accumulator tile, two per SIMD.
//     A single wavefront issues at most one non-MFMA instruction per ~8 cycles, which is too little for
//     the conversion work next to 32-cycle MFMAs; with two wavefronts per SIMD one converts while the
//     other's MFMA runs.
//   * Persistent workgroups walk the tiles in an XCD-aware order; the operand stream (global -> registers
//     -> fp16 in LDS) runs continuously across tile borders, two 128-deep spans ahead of the MFMAs.
//   * Loads cover two 64-deep steps (a span of 128 elements of K) at a time so that four neighbouring
//     lanes read 64 contiguous bytes of a row: thread t loads 16 payload bytes (two scale blocks) and
//     their 2 scale bytes for rows t/4 and t/4+128 of both operand tiles.  Of each such piece the first
//     block belongs to the even step and the second to the odd step: inside a span the even step
//     consumes blocks 0,2,4,6 and the odd step blocks 1,3,5,7 (the same permutation of K for A and B, so
//     the dot products are unchanged), which keeps every lane busy in every step.
//   * Conversion to fp16: one v_cvt_scalef32_pk_f16_fp4 and one v_pk_mul_f16 per two elements; the scale
//     goes e4m3 -> fp32 -> packed fp16 pair in two instructions (every e4m3 value is an fp16 value).
//   * Every piece of non-MFMA work is cut into MFMA-slot sized parts (3 conversion instructions, one LDS
//     access, one global load) and pinned between two MFMAs, because the two wavefronts of a SIMD run
//     in phase and a long run of other instructions in both would idle the matrix pipe.
//   * One barrier per step, placed before the last quarter of its MFMAs: by then every wave has written
//     its share of the next step and holds this step's last fragments in registers.
// LDS: two buffers of an A tile and a B tile (stored A0, A1, B0, B1), each tile 256 rows x 128 bytes with 16-byte
// chunk c of row r at chunk position c ^ ((r >> 1) & 7): conflict-free for the fragment reads.
// -------------------------------------------------------------------------------------------------
// TM = 32-row accumulator tiles of a wavefront along M: 4 -> 256x256 workgroup tile, 2 -> 128x256 (dense shapes
// whose 256x256 tiles would leave compute units idle; 1.5 times the conversion work per MFMA).  The statement
// order for TM = 4 is the one the 8192^3 measurements were made with.
template <bool OUT_BF16, bool GROUPED, int TM = 4, bool OUT_F32 = false, bool PAIRS = false, bool OUT_FP4 = false>
__global__ __launch_bounds__(512) void nvfp4_gemm_256_kernel(const Params p) {
  static_assert(TM == 4 || TM == 2, "tile height");
  constexpr int BM = 64 * TM, BN = 256;
  constexpr int A_UNITS = BM * 8;            // 16-byte units of the A tile (fp16, 64 of K per row)
  constexpr int TILE_UNITS = 2048;           // ... of the B tile
  constexpr int BUF_UNITS = A_UNITS + TILE_UNITS;
  // LDS order: A tile of buffer 0, A tile of buffer 1, B tile of buffer 0, B tile of buffer 1.  The two buffers of an
  // operand are then less than 64 KiB apart, so that a lane's fragment address for (operand, sub-step) serves both
  // buffers and all row tiles through the 16-bit immediate offset of the LDS instructions.
  auto tile_units = [](int buf, int op) { return op ? 2 * A_UNITS + buf * TILE_UNITS : buf * A_UNITS; };
  constexpr int AR = TM / 2;                 // A rows a thread stages per span (rows srow + 128 i)
  constexpr int NMK = 2 * TM;                // MFMAs per 16-deep sub-step
  constexpr int NCU = 2 * AR + 4;            // conversion units per step: operand, row, half scale block
  constexpr int NFU = TM + 2;                // fragment reads per sub-step
  extern __shared__ u32x4 lds[];
  __shared__ int tile_prefix[GROUPED ? kMaxGroups + 1 : 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int li = lane & 31, lg = lane >> 5;
  const int srow = tid >> 2, spiece = tid & 3;  // staging: rows srow and srow+128, 16-byte piece of a 64-byte span

  // ---- persistent tile walk: workgroup ids are dealt round-robin to the 8 XCDs, XCD x owns the tile
  // range [x*chunk, (x+1)*chunk); with the 8 (m) x 4 (n) blocked numbering the 32 tiles an XCD works on
  // at a time share 8 A panels and 4 B panels in its L2.
  // GROUPED: the work list holds the 256-row tiles of every group that rows_in_256_tiles() names: the whole
  // ones and a last one of more than 128 rows, whose rows past the group read as zero and are not stored; what
  // is left at the end of a group goes to the tile kernel.  With 128-row tiles (TM == 2) the list is instead one
  // tile per weight panel for every group of rows_lo..rows_hi (<= 128) rows and, if min_rows is set, for the end
  // (what rows_in_256_tiles() leaves) of every group of at least min_rows rows.
  const int tiles_m = p.m / BM, tiles_n = p.n / BN;
  int total = tiles_m * tiles_n;
  if constexpr (GROUPED) {
    if (wave == 0) {  // prefix sums of tiles per group, 64 groups per round
      int running = 0;
      for (int base = 0; base < p.groups; base += 64) {
        const int g = base + lane;
        int cnt = 0;
        if (g < p.groups) {
          const int mg = p.problem_sizes[g * 3];
          if constexpr (TM == 4) cnt = (rows_in_256_tiles(mg) / BM) * tiles_n;
          else  // one 128-row tile per weight panel: a group of the class, or (min_rows set) the end of a larger group
            cnt = ((mg >= p.rows_lo && mg <= p.rows_hi) || (p.min_rows && mg >= p.min_rows && mg > rows_in_256_tiles(mg))) ? tiles_n : 0;
        }
        int incl = cnt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int o = __shfl_up(incl, d, 64);
          if (lane >= d) incl += o;
        }
        if (g < p.groups) tile_prefix[g + 1] = running + incl;
        running += __shfl(incl, 63, 64);
      }
      if (lane == 0) tile_prefix[0] = 0;
    }
    __syncthreads();
    total = __builtin_amdgcn_readfirstlane(tile_prefix[p.groups]);
  }
  const int chunk_tiles = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int range_end = min((xcd + 1) * chunk_tiles, total);
  const bool blocked = (tiles_m & 7) == 0 && (tiles_n & 3) == 0;
  // tile -> group, first row of the tile among all rows of A (m0), among the rows of the group (gm0), n0
  struct Where { int g; int64_t m0; int gm0, n0, valid; };  // valid: rows of the tile that exist (grouped: the last tile of a group)
  auto tile_where = [&](int t) {
    Where w;
    if constexpr (GROUPED) {
      int lo = 0, hi = p.groups;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (t < tile_prefix[mid]) hi = mid; else lo = mid;
      }
      w.g = __builtin_amdgcn_readfirstlane(lo);
      const int m_g = __builtin_amdgcn_readfirstlane(p.problem_sizes[w.g * 3]);
      const int64_t row_off = __builtin_amdgcn_readfirstlane(p.expert_offsets[w.g]);
      const int full_m = TM == 4 ? rows_in_256_tiles(m_g) / BM : 1;
      const int local = __builtin_amdgcn_readfirstlane(t - tile_prefix[w.g]);
      // bands of 4 m-tiles, n-major inside a band: 32 consecutive tiles share 4 A and 8 B panels
      const int band = local / (4 * tiles_n), in_band = local - band * 4 * tiles_n;
      const int band_h = min(4, full_m - 4 * band);
      const int nt = in_band / band_h, mt = 4 * band + (in_band - nt * band_h);
      w.gm0 = TM == 4 ? mt * BM : (m_g <= BM ? 0 : rows_in_256_tiles(m_g));
      w.m0 = row_off + w.gm0;
      w.n0 = nt * BN;
      w.valid = min(BM, m_g - w.gm0);
    } else {
      int mt, nt;
      if (blocked) {
        const int sb = t >> 5, q = t & 31;
        mt = (sb % (tiles_m >> 3)) * 8 + (q & 7);
        nt = (sb / (tiles_m >> 3)) * 4 + (q >> 3);
      } else {
        mt = t % tiles_m;
        nt = t / tiles_m;
      }
      w.g = 0;
      w.gm0 = mt * BM;
      w.m0 = w.gm0;
      w.n0 = nt * BN;
      w.valid = BM;
    }
    return w;
  };
  const int first_tile = xcd * chunk_tiles + slot;
  if (first_tile >= range_end) return;

  const int kbytes = p.k >> 1;
  const int nmac = p.k >> 7;       // 128-deep load spans per tile (>= 2)
  const int sf_padded = p.k >> 4;  // K % 128 == 0: no padding columns
  const int64_t row128 = (int64_t)128 * kbytes;       // payload distance of the thread's two rows
  const int64_t sfrow128 = (int64_t)128 * sf_padded;  // same for the scales (next 128-row tile)

  // ---- operand stream: the tile the stream is in (lp) and the tile it enters next (np), as wave-uniform
  // addresses of the tiles' first rows (scalar registers; they advance by scalar selects), and this thread's
  // fixed 32-bit offsets inside any tile: its row and 16-byte piece, and its scale word (blocks 2*spiece,
  // 2*spiece+1 of the span: 128x4 layout column tile spiece>>1, bytes 2*(spiece&1)..).  A tile's first row is
  // a multiple of 128, so the swizzled scale address splits into the tile's part and the thread's part.
  // a_bytes / a_bytes2: bytes of the existing A rows among the tile's rows 0..127 / 128..255 (buffer ranges)
  struct RowPtrs { const uint8_t *a, *b, *sa, *sb; int a_bytes, a_bytes2; };
  auto tile_ptrs = [&](int t) {
    const Where w = tile_where(t);
    RowPtrs r;
    r.a = p.a + w.m0 * kbytes;
    // the last tile of a group may have fewer rows than the tile: the rows past the group read as zero
    r.a_bytes = GROUPED ? min(w.valid, 128) * kbytes : 0x7fffffff;
    r.a_bytes2 = GROUPED ? max(w.valid - 128, 0) * kbytes : 0x7fffffff;
    r.b = p.b + ((int64_t)w.g * p.n + w.n0) * kbytes;
    // (a group's activation scales are a slab of their own, swizzled from its first row)
    const int64_t sa_slab = GROUPED ? (int64_t)__builtin_amdgcn_readfirstlane(p.sf_offsets[w.g]) * sf_padded : 0;
    r.sa = p.sfa + sa_slab + swizzle_128x4(w.gm0, 0, sf_padded);
    r.sb = p.sfb + (int64_t)w.g * p.n * sf_padded + swizzle_128x4(w.n0, 0, sf_padded);
    return r;
  };
  const uint32_t off_ab = (uint32_t)srow * (uint32_t)kbytes + (uint32_t)spiece * 16u;
  const uint32_t off_sf = (uint32_t)swizzle_128x4(srow, 0, sf_padded) + (uint32_t)(spiece >> 1) * 512u + (uint32_t)(spiece & 1) * 2u;
  RowPtrs lp = tile_ptrs(first_tile);
  RowPtrs np = lp;
  int l_mac = 0;
  struct Raw { u32x4 a[2], b[2]; uint32_t sa[2], sb[2]; };
  // load unit q (0..7) of the span the stream is at; advance_stream() after the eighth
  // Buffer loads: the tile's first row as the resource's base, the span and the second row as the scalar
  // offset, the thread's fixed offset as the vector offset, so that no address is worked out in vector registers.
  auto rsrc = [](const uint8_t* base, int bytes = 0x7fffffff) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(base), 0, bytes, 0x00020000);
  };
  auto issue_load_unit = [&](Raw& r, int q) {
    const int o = l_mac * 64, so = l_mac * 1024;
    if (q == 0) r.a[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.a, lp.a_bytes), off_ab, o, 0);
    // (rows 128.. of the tile through a resource of their own, so that the range check that zeroes the rows past a
    // group never depends on whether the hardware counts the scalar offset)
    if (q == 1 && AR == 2) r.a[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.a + row128, lp.a_bytes2), off_ab, o, 0);
    if (q == 2) r.b[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.b), off_ab, o, 0);
    if (q == 3) r.b[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.b), off_ab, o + (int)row128, 0);
    if (q == 4) r.sa[0] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sa), off_sf, so, 0);
    if (q == 5 && AR == 2) r.sa[1] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sa), off_sf, so + (int)sfrow128, 0);
    if (q == 6) r.sb[0] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sb), off_sf, so, 0);
    if (q == 7) r.sb[1] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sb), off_sf, so + (int)sfrow128, 0);
  };
  auto advance_stream = [&]() {
    const bool wrap = (l_mac + 1 == nmac);
    l_mac = wrap ? 0 : l_mac + 1;
    lp.a = wrap ? np.a : lp.a;
    lp.a_bytes = wrap ? np.a_bytes : lp.a_bytes;
    lp.a_bytes2 = wrap ? np.a_bytes2 : lp.a_bytes2;
    lp.b = wrap ? np.b : lp.b;
    lp.sa = wrap ? np.sa : lp.sa;
    lp.sb = wrap ? np.sb : lp.sb;
  };

  // ---- conversion for a step of parity P: unit u (0..7) = operand u>>2, row (u>>1)&1, half block u&1 (with 128
  // rows of A, its second row does not exist: conversion unit v of the NCU real ones is unit v + 2 from v = 2 on).
  // A unit is cut into three parts of about 3 VALU instructions each.
  auto scale_pair = [&](uint32_t s2, int b) {
    const float f = b ? __builtin_amdgcn_cvt_f32_fp8((int)s2, 1) : __builtin_amdgcn_cvt_f32_fp8((int)s2, 0);
    return __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f, f));  // exact: e4m3 fits fp16
  };
  uint32_t cq;  // payload dword of the unit in progress
  f16x2 ch[4];  // its four converted pairs
  f16x2 sv[2][2];
  auto convert_phase = [&](const Raw& r, int parity, int u, int phase, int wbuf) {
    const int op = u >> 2, i = (u >> 1) & 1, cc = u & 1;
    if (phase == 0) {
      if (cc == 0) sv[op][i] = scale_pair(op ? r.sb[i] : r.sa[i], parity);
      cq = op ? r.b[i][2 * parity + cc] : r.a[i][2 * parity + cc];
      ch[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(cq, 1.0f, 0);
      ch[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(cq, 1.0f, 1);
      ch[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(cq, 1.0f, 2);
    } else if (phase == 1) {
      ch[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(cq, 1.0f, 3);
      ch[0] = ch[0] * sv[op][i];
      ch[1] = ch[1] * sv[op][i];
    } else {
      ch[2] = ch[2] * sv[op][i];
      ch[3] = ch[3] * sv[op][i];
      lds[tile_units(wbuf, op) + lds_pos2(srow + 128 * i, spiece * 2 + cc)] =
          u32x4{__builtin_bit_cast(uint32_t, ch[0]), __builtin_bit_cast(uint32_t, ch[1]), __builtin_bit_cast(uint32_t, ch[2]),
                __builtin_bit_cast(uint32_t, ch[3])};
    }
  };

  // ---- MFMA fragments of one 16-deep sub-step, loaded in the order of their first use by the MFMA
  // sequence (a0 b0) (a0 b1) (a1 b0) ...: units 0..NFU-1 = a0, b0, b1, a1, a2, a3
  struct Frag { u32x4 a[4], b[2]; };
  auto load_frag_unit = [&](int buf, int kk, int q, Frag& f) {
    const int op = (q == 1 || q == 2) ? 1 : 0;
    const int t = op ? q - 1 : (q == 0 ? 0 : q - 2);
    const int row = (op ? wn * 64 : wm * (32 * TM)) + t * 32 + li;
    const u32x4 v = lds[tile_units(buf, op) + lds_pos2(row, kk * 2 + lg)];
    if (op) f.b[t] = v; else f.a[t] = v;
  };

  f32x16 acc[TM][2];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  };
  zero_acc();

  // Keeps the accumulator tiles "used" at this point of the program, so that the MFMAs producing them
  // cannot be moved past the statement that follows (they have no side effects of their own).
#define NVF_PIN_ACC()                                                                                        \
  do {                                                                                                       \
    asm volatile("" : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[1][0]), "+a"(acc[1][1]));                   \
    if constexpr (TM == 4) asm volatile("" : "+a"(acc[TM - 2][0]), "+a"(acc[TM - 2][1]), "+a"(acc[TM - 1][0]), "+a"(acc[TM - 1][1])); \
  } while (0)

  Raw cur, nxt;  // span whose odd step is converted next / span whose even step is converted next
  Frag fr[2];

  // The stream runs two spans ahead of the MFMAs; with two spans per tile it is a whole tile ahead.
  const int tiles_ahead = nmac == 2 ? 2 : 1;
  auto ptrs_or_current = [&](int t) { return t < range_end ? tile_ptrs(t) : lp; };

  // ---- prologue: spans 0 and 1 requested, even step of span 0 converted into buffer 0
  np = ptrs_or_current(first_tile + slots);
#pragma unroll
  for (int q = 0; q < 8; ++q) issue_load_unit(cur, q);
  advance_stream();
#pragma unroll
  for (int q = 0; q < 8; ++q) issue_load_unit(nxt, q);
  advance_stream();
  auto unit_of = [&](int v) { return (AR == 2 || v < 2) ? v : v + 2; };  // conversion unit v -> (operand, row, half) code
#pragma unroll
  for (int v = 0; v < NCU; ++v)
#pragma unroll
    for (int ph = 0; ph < 3; ++ph) convert_phase(cur, 0, unit_of(v), ph, 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int q = 0; q < NFU; ++q) load_frag_unit(0, 0, q, fr[0]);

  // The two in-flight spans (`cur`: its odd step is converted next, `nxt`: its even step) normally hand over by a
  // register copy at the end of every span.  With an even number of spans per tile (PAIRS) the loop body is
  // written for two spans with the names swapped in the second, which saves the 24 register-pair moves per span.
  auto span_no_copy = [&](Raw& odd_src, Raw& even_src) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        if (kk == 3) {
          NVF_PIN_ACC();
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NMK; ++q) {
          const int i = q >> 1, j = q & 1;
          const int slot_id = kk * NMK + q;
          if (q < NFU) load_frag_unit(kk < 3 ? h : (h ^ 1), (kk + 1) & 3, q, fr[(kk + 1) & 1]);
          if (kk < 3) {
#pragma unroll
            for (int part = slot_id * NCU / NMK; part < (slot_id + 1) * NCU / NMK; ++part)
              convert_phase(h ? even_src : odd_src, h ^ 1, unit_of(part / 3), part % 3, h ^ 1);
          }
          if (kk == 3 && h == 1) {  // odd_src is dead: it takes the span after even_src
#pragma unroll
            for (int l = q * 8 / NMK; l < (q + 1) * 8 / NMK; ++l) issue_load_unit(odd_src, l);
            if (q == NMK - 1) advance_stream();
          }
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fr[kk & 1].b[j]),
                                                             __builtin_bit_cast(f16x8, fr[kk & 1].a[i]), acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  for (int c_tile = first_tile; c_tile < range_end; c_tile += slots) {
    np = ptrs_or_current(c_tile + tiles_ahead * slots);
    if constexpr (PAIRS) {
      for (int c_mac = 0; c_mac < nmac; c_mac += 2) {
        span_no_copy(cur, nxt);
        span_no_copy(nxt, cur);
      }
    } else {
      for (int c_mac = 0; c_mac < nmac; ++c_mac) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {  // step g = 2*c_mac + h computes from LDS buffer h
          // h == 0: the odd step of the current span is converted into buffer 1
          // h == 1: the even step of the next span is converted into buffer 0; then that span becomes the
          //         current one and the span after it is requested
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) {
            if (kk == 3) {
              // every wave has written its share of step g+1 and read the last fragments of step g
              NVF_PIN_ACC();
              asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
              __builtin_amdgcn_s_barrier();
              asm volatile("" ::: "memory");
              if (h == 1) cur = nxt;
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < NMK; ++q) {
              const int i = q >> 1, j = q & 1;
              const int slot_id = kk * NMK + q;  // 3 * NMK slots for the 3 * NCU conversion parts of the step
              if (q < NFU) load_frag_unit(kk < 3 ? h : (h ^ 1), (kk + 1) & 3, q, fr[(kk + 1) & 1]);
              if (kk < 3) {
#pragma unroll
                for (int part = slot_id * NCU / NMK; part < (slot_id + 1) * NCU / NMK; ++part)
                  convert_phase(h ? nxt : cur, h ^ 1, unit_of(part / 3), part % 3, h ^ 1);
              }
              if (kk == 3 && h == 1) {
#pragma unroll
                for (int l = q * 8 / NMK; l < (q + 1) * 8 / NMK; ++l) issue_load_unit(nxt, l);
                if (q == NMK - 1) advance_stream();
              }
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fr[kk & 1].b[j]),
                                                                 __builtin_bit_cast(f16x8, fr[kk & 1].a[i]), acc[i][j], 0, 0, 0);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
      }
    }
    // ---- epilogue; the next tile's first step is already in LDS.
    // acc[i][j][r] = C[m = li][n = (r/4)*8 + lg*4 + r%4] of its 32x32 sub-tile.
    const Where cw = tile_where(c_tile);
    const float alpha = p.alpha[cw.g];
    if constexpr (OUT_FP4) {
      // Block-scaled result.  A wavefront's 32 x 64 block i is quantized tile by tile (quantize_acc_tile), its 32 rows
      // x 32 payload bytes are collected in a private piece of LDS (pitch 48 bytes) and leave as 16 bytes per lane,
      // two lanes to a row; the four scale codes of a row (its four 16-column blocks are one dword of the 128x4
      // layout) are kept per i and stored once at the end: 16 bytes per row for the 128 rows of a 256-row tile's
      // wavefront (they are one whole 128x4 scale tile), 8 bytes for the 64 rows of a 128-row tile's.
      const float gs = p.gnorm[0], decode = 1.0f / gs;
      int elane = lane;
      asm volatile("" : "+v"(elane));
      uint8_t* stage = reinterpret_cast<uint8_t*>(lds + 2 * BUF_UNITS) + wave * 2560;
      uint8_t* wr = stage + (elane & 31) * 48 + (elane >> 5) * 2;
      const uint8_t* rd = stage + (elane >> 1) * 48 + (elane & 1) * 16;
      const int64_t opitch = p.n >> 1;
      uint8_t* obase = static_cast<uint8_t*>(p.out) + (cw.m0 + wm * (32 * TM) + (elane >> 1)) * opitch + ((cw.n0 + wn * 64) >> 1) + (elane & 1) * 16;
      uint32_t sfw[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        sfw[i] = 0;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          uint32_t h[2], q8[2];
          quantize_acc_tile(acc[i][j], alpha, gs, decode, true, h, q8);
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            *reinterpret_cast<uint16_t*>(wr + j * 16 + b * 8) = (uint16_t)(h[b] & 0xffffu);
            *reinterpret_cast<uint16_t*>(wr + j * 16 + b * 8 + 4) = (uint16_t)(h[b] >> 16);
          }
          sfw[i] |= (q8[0] | (q8[1] << 8)) << (16 * j);
        }
        asm volatile("" ::: "memory");  // the read below sees the writes above: one wavefront's LDS accesses stay in order
        const u32x4 v = *reinterpret_cast<const u32x4*>(rd);
        *reinterpret_cast<u32x4*>(obase + (int64_t)(i * 32) * opitch) = v;
        asm volatile("" ::: "memory");
      }
      if (lg == 0) {
        const int sf_cols4 = p.n >> 6;  // 512-byte scale tiles per 128 rows (N % 256 == 0: no padding columns)
        uint8_t* sfp = p.out_sf + ((cw.m0 >> 7) * (int64_t)sf_cols4 + ((cw.n0 + wn * 64) >> 6)) * 512 + li * 16;
        if constexpr (TM == 4) *reinterpret_cast<u32x4*>(sfp + (int64_t)wm * sf_cols4 * 512) = u32x4{sfw[0], sfw[1], sfw[2], sfw[3]};
        else *reinterpret_cast<u32x2*>(sfp + wm * 8) = u32x2{sfw[0], sfw[1]};
      }
    } else if constexpr (OUT_F32) {
      // as below, with 32x16 blocks of fp32 (64-byte row segments)
      int elane = lane;
      asm volatile("" : "+v"(elane));
      uint8_t* stage = reinterpret_cast<uint8_t*>(lds + 2 * BUF_UNITS) + wave * 2560;
      uint8_t* wr = stage + (elane & 31) * 80 + (elane >> 5) * 16;
      const uint8_t* rd = stage + (elane >> 2) * 80 + (elane & 3) * 16;
      const uint32_t ooff = ((uint32_t)(elane >> 2) * (uint32_t)p.n + (uint32_t)(elane & 3) * 4u) * 4u;
      uint8_t* obase = reinterpret_cast<uint8_t*>(static_cast<float*>(p.out) + (cw.m0 + wm * (32 * TM)) * p.n + cw.n0 + wn * 64);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int jh = 0; jh < 4; ++jh) {  // 16 columns: block j = jh / 2, its rq pair jh % 2
          const int j = jh >> 1;
#pragma unroll
          for (int r2 = 0; r2 < 2; ++r2) {
            const int rq = (jh & 1) * 2 + r2;
            *reinterpret_cast<f32x4*>(wr + r2 * 32) = f32x4{acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha,
                                                            acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha};
          }
          asm volatile("" ::: "memory");  // one wavefront's LDS accesses stay in order
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(rd + t * 1280);
            *reinterpret_cast<f32x4*>(obase + ((int64_t)(i * 32 + 16 * t) * p.n + jh * 16) * 4 + ooff) = v;
          }
          asm volatile("" ::: "memory");
        }
      }
    } else {
      // A lane holds 8-byte pieces of 32 different rows; stored like that, a tile is 8192 sixteen-byte write
      // requests per compute unit, which cost the L2 more time than a K step of MFMAs.  Every 32x32 block of the
      // wavefront's tile is therefore turned round in a private 2.5 KiB of LDS (32 rows of 64 bytes at a pitch of
      // 80 bytes) and leaves in 16-byte pieces, 4 lanes to a row's 64 bytes.  This kernel has no register to
      // spare: one LDS address each for writing and reading (everything else is an immediate offset), one 32-bit
      // lane offset into the result next to a wave-uniform address; and the lane number passes through an empty
      // asm statement so that these are worked out here, after the K loop.
      int elane = lane;
      asm volatile("" : "+v"(elane));
      uint8_t* stage = reinterpret_cast<uint8_t*>(lds + 2 * BUF_UNITS) + wave * 2560;
      uint8_t* wr = stage + (elane & 31) * 80 + (elane >> 5) * 8;
      const uint8_t* rd = stage + (elane >> 2) * 80 + (elane & 3) * 16;
      const uint32_t ooff = ((uint32_t)(elane >> 2) * (uint32_t)p.n + (uint32_t)(elane & 3) * 8u) * 2u;
      uint8_t* obase = reinterpret_cast<uint8_t*>(static_cast<uint16_t*>(p.out) + (cw.m0 + wm * (32 * TM)) * p.n + cw.n0 + wn * 64);
      const int erow = elane >> 2;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            u32x2 v;
            v[0] = pack2(acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha, OUT_BF16);
            v[1] = pack2(acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(wr + rq * 16) = v;
          }
          asm volatile("" ::: "memory");  // the reads below see the writes above: one wavefront's LDS accesses stay in order
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int brow = i * 32 + 16 * t;  // first of the 16 rows of this piece, in the wavefront's tile
            const u32x4 v = *reinterpret_cast<const u32x4*>(rd + t * 1280);
            if (!GROUPED || wm * (32 * TM) + brow + erow < cw.valid)
              *reinterpret_cast<u32x4*>(obase + ((int64_t)brow * p.n + j * 32) * 2 + ooff) = v;
          }
          asm volatile("" ::: "memory");
        }
      }
    }
    zero_acc();
  }
#undef NVF_PIN_ACC
}

template <bool OUT_BF16, bool GROUPED, int TM, bool OUT_F32, bool PAIRS, bool OUT_FP4 = false>
int launch_nvfp4_fast_cfg(const Params& p, int cus, hipStream_t stream) {
  auto kern = nvfp4_gemm_256_kernel<OUT_BF16, GROUPED, TM, OUT_F32, PAIRS, OUT_FP4>;
  constexpr int lds_bytes = 2 * (64 * TM + 256) * 128 + 8 * 2560;  // 128 KiB / 96 KiB of tiles + the epilogue's 20 KiB
  // grouped: an upper bound (128-row tiles: one per weight panel and group of at least rows_lo rows)
  const int64_t tiles_m = (GROUPED && TM == 2) ? std::min<int64_t>(p.groups, p.m / std::max(p.rows_lo, 1)) : p.m / (64 * TM);
  const int64_t tiles = tiles_m * (p.n / 256);
  const unsigned grid = (unsigned)(tiles >= cus ? (cus & ~7) : ((tiles + 7) / 8) * 8);
  if (grid == 0) return NVF_OK;  // fewer rows in the whole call than the smallest group this launch serves: no work
  if (note_launch("nvfp4_gemm_256_kernel<grouped=%d,TM=%d,f32=%d,pairs=%d%s> grid=%u rows=%d..%d min_rows=%d", (int)GROUPED, TM, (int)OUT_F32,
                  (int)PAIRS, OUT_FP4 ? ",fp4_blockscale" : "", grid, p.rows_lo, p.rows_hi, p.min_rows))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, stream, p);
  return check_launch("nvfp4_gemm_256_kernel");
}

template <bool OUT_BF16, bool GROUPED, int TM = 4, bool OUT_F32 = false, bool OUT_FP4 = false>
int launch_nvfp4_fast(const Params& p, int cus, hipStream_t stream) {
  // an even number of 128-deep spans per tile: the variant whose two in-flight spans swap names instead of being copied
  if (((p.k >> 7) & 1) == 0) return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, true, OUT_FP4>(p, cus, stream);
  return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, false, OUT_FP4>(p, cus, stream);
}

// -------------------------------------------------------------------------------------------------
// NVFP4 skinny path: dense, up to 128 activation rows per launch (decode-sized activations; up to 256 rows in
// two launches), K % 128 == 0, N % (16*RT) == 0.  A launch streams the weight matrix exactly once, so the op
// is bound by HBM and by the conversion work, not by the MFMAs:
//   * A workgroup owns 16*RT weight rows for the whole of K and all M activation rows; its 8
//     wavefronts split K in interleaved 128-element chunks and their partial sums are added in a fixed
//     order through LDS (no atomics, no workspace, deterministic).
//   * In v_mfma_f32_16x16x32_f16 lane (i, g) supplies 8 elements of row i, and both operands use the same
//     (lane group, element) -> k assignment, so a lane holds the 16 payload bytes [32g, 32g+32) of its
//     row's chunk, converts them to fp16 in registers and feeds MFMA t = 0..3 with elements 8t..8t+7.
//     Weight rows are the first operand (output rows), activation rows the second, so a lane ends up
//     with 4 consecutive N-elements of one output row.
//   * A load in that lane order (lane = row % 16 + 16 * piece) touches 64 unrelated 16-byte pieces and
//     occupies the address unit for 64 cycles, which - not HBM, not latency - bounded an earlier version
//     that loaded straight into registers.  The tiles are therefore fetched with LDS-direct loads in
//     memory order (4 neighbouring lanes = 64 contiguous bytes of a row; scales as the 256 contiguous
//     bytes that hold a 16-row tile's scale words) into a private LDS ring of each wavefront and read
//     back in MFMA order; no barrier is involved because a wavefront only reads what it loaded itself.
//   LDS per slot: NT payload tiles of 16 rows x 64 B, piece p of row r at piece position p ^ ((r >> 2) & 3)
//   (conflict-free reads), then per operand one 1 KiB scale block per pair of tiles: [tile][col tile][row][16 B].
// -------------------------------------------------------------------------------------------------
// LDS-direct load.  lds_byte_addr and base are wave-uniform; lane L's 16 bytes land at lds_byte_addr + 16 * L.
// Issued from inline assembly: the compiler neither waits for it nor orders LDS reads against it, the
// kernels do that with explicit s_waitcnt vmcnt(n).
__device__ __forceinline__ void lds_dma16(uint32_t lds_byte_addr, const uint8_t* base, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_byte_addr), "v"(voff), "s"(base) : "memory", "m0");
}

// 32 packed e2m1 values and their two e4m3 block scales -> four MFMA operands of 8 fp16 values
__device__ __forceinline__ void dequant_frags(const u32x4 q, uint32_t s2, u32x4 out[4]) {
  const float f0 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 0), f1 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 1);
  const f16x2 sv[2] = {__builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f0, f0)),
                       __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f1, f1))};
#pragma unroll
  for (int w = 0; w < 4; ++w) {  // dword w = elements 8w..8w+7, scale block w/2
    const f16x2 h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[w], 1.0f, 0) * sv[w >> 1];
    const f16x2 h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[w], 1.0f, 1) * sv[w >> 1];
    const f16x2 h2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[w], 1.0f, 2) * sv[w >> 1];
    const f16x2 h3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[w], 1.0f, 3) * sv[w >> 1];
    out[w] = u32x4{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1), __builtin_bit_cast(uint32_t, h2),
                   __builtin_bit_cast(uint32_t, h3)};
  }
}

// GROUPED: one workgroup per (group, block of 16*RT weight rows); it serves groups of rows_lo .. rows_hi rows
// (at most 16*TT) and returns at once for the others, which other launches take.
// NSPLIT (grouped only, where the groups supply enough workgroups): the 8 wavefronts own 8 different blocks of
// 16*RT weight rows and each walks all of K on its own - a long pipeline per wavefront and no reduction -
// instead of sharing one block and splitting K.
template <int RT, int TT, bool OUT_BF16, int DEPTH, bool GROUPED = false, bool NSPLIT = false>
__global__ __launch_bounds__(512) void nvfp4_skinny_ring_kernel(const Params p) {
  static_assert(GROUPED || !NSPLIT, "the dense op has too few row blocks to give every wavefront its own");
  constexpr int W = 8;
  constexpr int NT = RT + TT;
  constexpr int B_SC = (RT + 1) / 2, A_SC = (TT + 1) / 2;     // scale blocks (1 KiB) per operand
  constexpr int SLOT_BYTES = (NT + B_SC + A_SC) * 1024;
  constexpr int NDMA = NT + B_SC + A_SC;                      // loads per chunk and wavefront
  // DEPTH 2: two chunks in flight per wavefront.  DEPTH 1 (many tiles per chunk): the next chunk is requested
  // as soon as the current one has been read out of LDS, and lands under its long conversion + MFMA phase.
  static_assert((DEPTH == 1 || DEPTH == 2) && W * DEPTH * SLOT_BYTES <= 160 * 1024 && DEPTH * NDMA <= 63, "ring does not fit");
  extern __shared__ f32x4 red[];  // ring during the K loop, then [W][tiles][64 lanes] partial sums
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int kbytes = p.k >> 1;
  int chunks = p.k >> 7;
  const int sf_padded = p.k >> 4;  // K % 128 == 0: no padding columns
  // dense with a workspace: blockIdx.z owns the chunks [c_lo, c_lo + chunks) of K and leaves an fp32 partial result
  int c_lo = 0;
  if (!GROUPED && p.partial != nullptr) {
    c_lo = (int)blockIdx.z * p.spans_per_split;
    chunks = min(chunks - c_lo, p.spans_per_split);
  }
  int n0, m_loc, grp = 0, asf_word0 = 0;  // asf_word0: which 32-row group of its 128-row scale tile the slab starts in
  int64_t a_row0 = p.m_base, asf_row0 = p.m_base, b_row0 = 0;  // first activation row, its scale row, first weight row
  if constexpr (GROUPED) {
    const int nblocks = p.n / (16 * RT * (NSPLIT ? W : 1));
    grp = blockIdx.x / nblocks;
    n0 = ((blockIdx.x - grp * nblocks) * (NSPLIT ? W : 1) + (NSPLIT ? wave : 0)) * (16 * RT);
    m_loc = __builtin_amdgcn_readfirstlane(p.problem_sizes[grp * 3]);
    if (m_loc < p.rows_lo || m_loc > p.rows_hi) return;
    a_row0 = __builtin_amdgcn_readfirstlane(p.expert_offsets[grp]);
    asf_row0 = __builtin_amdgcn_readfirstlane(p.sf_offsets[grp]);  // the group's own scale slab
    b_row0 = (int64_t)grp * p.n;
  } else {
    n0 = blockIdx.x * (16 * RT);
    // activation rows of this workgroup: [m_base, m_base + m_loc); blockIdx.y counts slabs of 16*TT rows
    // (TT = 2, 4 or 8 when there is more than one, so that a slab lies inside one 32-row scale group)
    const int m_base = p.m_base + (int)blockIdx.y * (16 * TT);
    a_row0 = m_base;
    asf_row0 = m_base & ~127;
    asf_word0 = (m_base & 127) >> 5;
    m_loc = min(p.m - m_base, 16 * TT);
  }
  const int tt_count = (m_loc + 15) >> 4;

  // ---- load side (memory order): lane L fetches row L/4, piece (L%4) ^ ((L/16)&3) of a payload tile
  const int lrow = lane >> 2, lpiece = (lane & 3) ^ ((lane >> 4) & 3);
  const uint8_t* b_base = p.b + (b_row0 + n0) * kbytes + c_lo * 64;
  const uint8_t* bsf_base = p.sfb + b_row0 * sf_padded + swizzle_128x4(n0 & ~127, 0, sf_padded) + (int64_t)c_lo * 1024;
  const uint8_t* a_base = p.a + a_row0 * kbytes + c_lo * 64;
  const uint8_t* asf_base = p.sfa + asf_row0 * sf_padded + (int64_t)c_lo * 1024;  // the 128-row scale tile of these rows (row0 % 128 == 0)
  uint32_t b_off[RT], a_off[TT], bsf_off[B_SC], asf_off[A_SC];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) b_off[rt] = (uint32_t)(rt * 16 + lrow) * (uint32_t)kbytes + lpiece * 16;
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) a_off[tt] = (uint32_t)min(tt * 16 + lrow, m_loc - 1) * (uint32_t)kbytes + lpiece * 16;
  // scale block j of an operand: lane L = tile 2j + (L>>5), col tile (L>>4)&1, row L&15: the 16 bytes that
  // hold the scale words of rows {row, row+32, row+64, row+96} (mod 128) for that col tile
#pragma unroll
  for (int j = 0; j < B_SC; ++j) {
    const int t = min(2 * j + (lane >> 5), RT - 1);
    const int row = (n0 & 127) + t * 16 + (lane & 15);
    bsf_off[j] = (uint32_t)((row & 31) * 16 + ((lane >> 4) & 1) * 512);
  }
#pragma unroll
  for (int j = 0; j < A_SC; ++j) {
    const int t = min(2 * j + (lane >> 5), TT - 1);
    const int row = t * 16 + (lane & 15);  // < 128: inside the first 128-row tile of the activations' scales
    asf_off[j] = (uint32_t)((row & 31) * 16 + ((lane >> 4) & 1) * 512);
  }
  const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)red);
  const uint32_t ring_base = lds_base + (uint32_t)wave * (DEPTH * SLOT_BYTES);
  auto issue_chunk = [&](int c_in, int slot) {  // c_in is wave-uniform
    if (c_in >= chunks) return;
    const uint32_t c = (uint32_t)c_in;
    const uint32_t sb = ring_base + (uint32_t)slot * SLOT_BYTES;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) lds_dma16(sb + rt * 1024, b_base, b_off[rt] + c * 64u);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      // with one slot every wait is for everything, so tiles without rows need not be fetched
      if (DEPTH == 2 || tt < tt_count) lds_dma16(sb + (RT + tt) * 1024, a_base, a_off[tt] + c * 64u);
    }
#pragma unroll
    for (int j = 0; j < B_SC; ++j) lds_dma16(sb + (NT + j) * 1024, bsf_base, bsf_off[j] + c * 1024u);
#pragma unroll
    for (int j = 0; j < A_SC; ++j) {
      if (DEPTH == 2 || 2 * j < tt_count) lds_dma16(sb + (NT + B_SC + j) * 1024, asf_base, asf_off[j] + c * 1024u);
    }
  };

  // ---- read side (MFMA order): lane (r, g) = row r, payload piece g, scale blocks 2g, 2g+1 of the chunk
  const int rd_payload = r * 64 + ((g ^ ((r >> 2) & 3)) * 16);
  int rd_bsc[RT], rd_asc[TT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int rowgroup = (((n0 & 127) + rt * 16) >> 5) & 3;  // which of the 4 words of the 16 bytes
    rd_bsc[rt] = (NT + (rt >> 1)) * 1024 + ((rt & 1) * 2 + (g >> 1)) * 256 + r * 16 + rowgroup * 4;
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
    rd_asc[tt] = (NT + B_SC + (tt >> 1)) * 1024 + ((tt & 1) * 2 + (g >> 1)) * 256 + r * 16 + (asf_word0 + ((tt * 16) >> 5)) * 4;
  const int sc_shift = (g & 1) * 16;

  const float alpha = p.alpha[grp];
  uint16_t* out = static_cast<uint16_t*>(p.out);
  // Accumulators acc[RT][TTC] of the TTC activation tiles this workgroup was compiled for (tt_count <= TTC of them
  // hold rows) -> result: stored directly (NSPLIT) or summed over the wavefronts through LDS.
  auto finish = [&](auto ttc_c, auto& acc) {
    constexpr int TTC = decltype(ttc_c)::value;
    if constexpr (NSPLIT) {
      // every wavefront holds finished sums: element e of lane l = weight row 4*(l/16) + e, activation row l%16
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) {
        const int tok = tt * 16 + r;
        if (tok < m_loc) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            u32x2 v;
            v[0] = pack2(acc[rt][tt][0] * alpha, acc[rt][tt][1] * alpha, OUT_BF16);
            v[1] = pack2(acc[rt][tt][2] * alpha, acc[rt][tt][3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(out + (a_row0 + tok) * p.n + n0 + rt * 16 + 4 * g) = v;
          }
        }
      }
      return;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-direct load may be pending when the ring is reused
    __syncthreads();

    // ---- sum the wavefronts' partial tiles in wave order and store: all tiles in one round if they fit the
    // ring's memory (RT * TT <= 8), else one round per weight-row tile
    constexpr int ROUNDS = RT * TT <= 8 ? 1 : RT;
    constexpr int RPR = RT / ROUNDS;  // weight-row tiles per round
    const int tiles = RPR * tt_count;   // tile index inside a round: rt * tt_count + tt
    const int units = tiles * 64;
#pragma unroll
    for (int round = 0; round < ROUNDS; ++round) {
      if (round > 0) __syncthreads();
#pragma unroll
      for (int r2 = 0; r2 < RPR; ++r2)
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt)
          if (tt < tt_count) red[(wave * tiles + r2 * tt_count + tt) * 64 + lane] = acc[round * RPR + r2][tt];
      __syncthreads();
      for (int u = tid; u < units; u += 512) {
        const int l = u & 63, tile = u >> 6;
        const int r2 = tile / tt_count, tt = tile - r2 * tt_count;
        f32x4 s = red[u];
#pragma unroll
        for (int w = 1; w < W; ++w) s += red[w * units + u];
        const int tok = tt * 16 + (l & 15);
        if (tok < m_loc) {
          const int64_t at = (a_row0 + tok) * p.n + n0 + (round * RPR + r2) * 16 + 4 * (l >> 4);
          if (!GROUPED && p.partial != nullptr) {  // this K range's sums as they are; the reduction applies alpha
            *reinterpret_cast<f32x4*>(p.partial + (int64_t)blockIdx.z * p.m * p.n + at) = s;
          } else {
            u32x2 v;
            v[0] = pack2(s[0] * alpha, s[1] * alpha, OUT_BF16);
            v[1] = pack2(s[2] * alpha, s[3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(out + at) = v;
          }
        }
      }
    }
  };

  constexpr int CSTEP = NSPLIT ? 1 : W;  // distance of a wavefront's consecutive chunks
  const int c_first = NSPLIT ? 0 : wave;
  // Many activation tiles (TT > 2): the chunk loop is compiled for the group's number of row tiles (no branches in
  // it, accumulators for just those tiles); for counts whose accumulators leave the registers for it, a chunk's
  // conversions are folded into its MFMA steps.
  constexpr bool kFineRing = TT > 2 && DEPTH == 1;
  if constexpr (kFineRing) {
    auto load_b_part = [&](uint32_t c) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) lds_dma16(ring_base + rt * 1024, b_base, b_off[rt] + c * 64u);
#pragma unroll
      for (int j = 0; j < B_SC; ++j) lds_dma16(ring_base + (NT + j) * 1024, bsf_base, bsf_off[j] + c * 1024u);
    };
    int fine_lrow = lrow;  // re-derived per use: eight row offsets kept in registers would not fit
    auto load_a_tile = [&](uint32_t c, int tt) {
      asm volatile("" : "+v"(fine_lrow));
      lds_dma16(ring_base + (RT + tt) * 1024, a_base, (uint32_t)min(tt * 16 + fine_lrow, m_loc - 1) * (uint32_t)kbytes + lpiece * 16 + c * 64u);
    };
    auto load_a_scales = [&](uint32_t c, int j) { lds_dma16(ring_base + (NT + B_SC + j) * 1024, asf_base, asf_off[j] + c * 1024u); };
    const char* sp = reinterpret_cast<const char*>(red) + wave * SLOT_BYTES;
    auto read_a_tile = [&](int tt, u32x4& aq, uint32_t& as) {
      aq = *reinterpret_cast<const u32x4*>(sp + (RT + tt) * 1024 + rd_payload);
      as = *reinterpret_cast<const uint32_t*>(sp + rd_asc[tt]) >> sc_shift;
    };
    // e4m3 scales of a lane's two blocks -> fp16 pairs; one dword (8 values of one block) -> one MFMA operand
    auto scale_pairs = [&](uint32_t s2, f16x2 sv[2]) {
      const float f0 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 0), f1 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 1);
      sv[0] = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f0, f0));
      sv[1] = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f1, f1));
    };
    auto dequant_dword = [&](uint32_t qw, f16x2 sv) {
      const f16x2 h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 0) * sv;
      const f16x2 h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 1) * sv;
      const f16x2 h2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 2) * sv;
      const f16x2 h3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 3) * sv;
      return u32x4{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1), __builtin_bit_cast(uint32_t, h2),
                   __builtin_bit_cast(uint32_t, h3)};
    };
    // One chunk with TTC activation tiles.  The whole slot is read out into registers at once and refilled with
    // the wavefront's next chunk, which then has a whole chunk's time to land.  The chunk is four 32-deep MFMA
    // steps of TTC groups of RT MFMAs; the operands of the next step - one dword of every weight and activation
    // tile - are converted between the groups of the current one, so that they issue while the matrix pipe works.
    auto chunk = [&](auto ttc_c, uint32_t c, auto& acc) {
      constexpr int TTC = decltype(ttc_c)::value;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      u32x4 q[RT], aq[TTC];
      uint32_t sc[RT], as[TTC];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) q[rt] = *reinterpret_cast<const u32x4*>(sp + rt * 1024 + rd_payload);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) read_a_tile(tt, aq[tt], as[tt]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: may be refilled
      if (c + CSTEP < (uint32_t)chunks) {
        load_b_part(c + CSTEP);
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) {
          load_a_tile(c + CSTEP, tt);
          if ((tt & 1) || tt + 1 == TTC) load_a_scales(c + CSTEP, tt >> 1);
        }
      }
      f16x2 sv[RT][2], asv[TTC][2];
      u32x4 fb[RT], fa[TTC], fbn[RT], fan[TTC];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        scale_pairs(sc[rt], sv[rt]);
        fb[rt] = dequant_dword(q[rt][0], sv[rt][0]);
      }
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) {
        scale_pairs(as[tt], asv[tt]);
        fa[tt] = dequant_dword(aq[tt][0], asv[tt][0]);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        auto part_work = [&](int part) {  // parts 0 .. RT-1: weight tiles, RT .. RT+TTC-1: activation tiles
          if (t == 3) return;
          if (part < RT) fbn[part] = dequant_dword(q[part][t + 1], sv[part][(t + 1) >> 1]);
          else fan[part - RT] = dequant_dword(aq[part - RT][t + 1], asv[part - RT][(t + 1) >> 1]);
        };
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) {
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            acc[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[rt]), __builtin_bit_cast(f16x8, fa[tt]),
                                                                 acc[rt][tt], 0, 0, 0);
#pragma unroll
          for (int part = tt * (RT + TTC) / TTC; part < (tt + 1) * (RT + TTC) / TTC; ++part) part_work(part);
        }
        if (t < 3) {
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) fb[rt] = fbn[rt];
#pragma unroll
          for (int tt = 0; tt < TTC; ++tt) fa[tt] = fan[tt];
        }
      }
    };
    // One whole-slot refill per chunk, as in the kernels with few activation tiles: for tile counts whose
    // accumulators leave no registers for the finer scheme.
    auto chunk_coarse = [&](auto ttc_c, uint32_t c, auto& acc) {
      constexpr int TTC = decltype(ttc_c)::value;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      u32x4 q[RT];
      uint32_t sc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) q[rt] = *reinterpret_cast<const u32x4*>(sp + rt * 1024 + rd_payload);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
      u32x4 fb[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) dequant_frags(q[rt], sc[rt], fb[rt]);
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) {
        __builtin_amdgcn_sched_barrier(0);
        u32x4 aq;
        uint32_t as;
        read_a_tile(tt, aq, as);
        if (tt + 1 == TTC) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the last read of the slot is complete
          if (c + CSTEP < (uint32_t)chunks) {
            load_b_part(c + CSTEP);
#pragma unroll
            for (int t2 = 0; t2 < TTC; ++t2) {
              load_a_tile(c + CSTEP, t2);
              if ((t2 & 1) || t2 + 1 == TTC) load_a_scales(c + CSTEP, t2 >> 1);
            }
          }
        }
        u32x4 fa[4];
        dequant_frags(aq, as, fa);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            acc[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[rt][t]),
                                                                 __builtin_bit_cast(f16x8, fa[t]), acc[rt][tt], 0, 0, 0);
      }
    };
    // s_waitcnt vmcnt(n) for a wave-uniform n (the operand is an immediate)
    auto wait_loads = [&](int n) {
      switch (n) {
#define NVF_VMCNT_CASE(n) case n: asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory"); break;
        NVF_VMCNT_CASE(1) NVF_VMCNT_CASE(2) NVF_VMCNT_CASE(3) NVF_VMCNT_CASE(4) NVF_VMCNT_CASE(5) NVF_VMCNT_CASE(6)
        NVF_VMCNT_CASE(7) NVF_VMCNT_CASE(8) NVF_VMCNT_CASE(9) NVF_VMCNT_CASE(10) NVF_VMCNT_CASE(11) NVF_VMCNT_CASE(12)
        NVF_VMCNT_CASE(13) NVF_VMCNT_CASE(14) NVF_VMCNT_CASE(15) NVF_VMCNT_CASE(16) NVF_VMCNT_CASE(17) NVF_VMCNT_CASE(18)
        NVF_VMCNT_CASE(19) NVF_VMCNT_CASE(20) NVF_VMCNT_CASE(21) NVF_VMCNT_CASE(22) NVF_VMCNT_CASE(23) NVF_VMCNT_CASE(24)
        NVF_VMCNT_CASE(25) NVF_VMCNT_CASE(26) NVF_VMCNT_CASE(27) NVF_VMCNT_CASE(28) NVF_VMCNT_CASE(29) NVF_VMCNT_CASE(30)
#undef NVF_VMCNT_CASE
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
    };
    // one dword of an MFMA operand: two of a raw dword's eight values (byte `sel`), times their block's scale
    auto dequant_pair = [&](uint32_t qw, int sel, f16x2 sv) {
      const f16x2 h = (sel == 0   ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 0)
                       : sel == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 1)
                       : sel == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 2)
                                  : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 3)) * sv;
      return __builtin_bit_cast(uint32_t, h);
    };
    // One chunk for tile counts whose accumulators leave no registers for the scheme above (RT * TTC > 20).  A
    // wavefront issues one conversion instruction per 8 cycles at best and an MFMA of this shape per 16, so a chunk
    // that converts a tile and then multiplies it takes the sum of both; here the two instructions that make one
    // dword of an activation operand follow every MFMA, so that they issue while the matrix pipe works: the 8 MFMAs
    // on the first half of a tile's K range (2 steps x RT weight tiles) carry the conversion of its second half, the 8
    // on the second half that of the next tile's first half.  Only the weight operands of the whole chunk are
    // converted up front.  A tile's raw bytes are read out of LDS one tile ahead and its slot is refilled with the
    // wavefront's next chunk at once, the weight part right at the start of the chunk: every load has most of a
    // chunk's time to land.  Loads complete in the order of issue, and that order is fixed - weight part, then per
    // tile its bytes and, after every second tile and the last, the scale block of the pair - so the waits are for
    // counts that follow from it.
    auto chunk_pipe = [&](auto ttc_c, uint32_t c, auto& acc) {
      constexpr int TTC = decltype(ttc_c)::value;
      constexpr int NS = (TTC + 1) / 2, NA = TTC + NS, LB = RT + B_SC;
      const bool has_next = c + CSTEP < (uint32_t)chunks;
      // loads of this chunk still pending once tile tt and the scale block of its pair have landed
      auto after_tile = [&](int tt) {
        const int last_of_pair = (tt | 1) < TTC ? (tt | 1) : TTC - 1;
        return NA - 1 - (last_of_pair + (last_of_pair >> 1) + 1);
      };
      wait_loads(NA);  // the weight part has landed
      u32x4 q[RT];
      uint32_t sc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) q[rt] = *reinterpret_cast<const u32x4*>(sp + rt * 1024 + rd_payload);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
      wait_loads(after_tile(0));
      u32x4 aq, aqn = {0, 0, 0, 0};
      uint32_t as, asn = 0;
      read_a_tile(0, aq, as);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: may be refilled
      if (has_next) {
        load_b_part(c + CSTEP);
        load_a_tile(c + CSTEP, 0);
        if (TTC == 1) load_a_scales(c + CSTEP, 0);
      }
      u32x4 fb[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        f16x2 sv[2];
        scale_pairs(sc[rt], sv);
#pragma unroll
        for (int t = 0; t < 4; ++t) fb[rt][t] = dequant_dword(q[rt][t], sv[t >> 1]);
      }
      f16x2 asv[2], asvn[2];
      scale_pairs(as, asv);
      u32x4 fa[2], fan[2];
      fa[0] = dequant_dword(aq[0], asv[0]);
      fa[1] = dequant_dword(aq[1], asv[0]);
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) {
        __builtin_amdgcn_sched_barrier(0);
        if (tt + 1 < TTC) {
          // pending behind tile tt+1: the rest of this chunk's tiles, the next chunk's weight part and its tiles 0..tt
          wait_loads(after_tile(tt + 1) + (has_next ? LB + (tt + 1) + ((tt + 1) >> 1) : 0));
          read_a_tile(tt + 1, aqn, asn);
        }
        // K steps 0 and 1 of tile tt; behind every MFMA one dword of the operands of its steps 2 and 3
#pragma unroll
        for (int m = 0; m < 8; ++m) {
          const int t = m >> 2, rt = m & 3;
#pragma unroll
          for (int r2 = rt; r2 < RT; r2 += 4)
            acc[r2][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[r2][t]), __builtin_bit_cast(f16x8, fa[t]),
                                                                 acc[r2][tt], 0, 0, 0);
          fan[m >> 2][m & 3] = dequant_pair(aq[2 + (m >> 2)], m & 3, asv[1]);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (tt + 1 < TTC) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // tile tt+1 is in registers: its slot may be refilled
          if (has_next) {
            load_a_tile(c + CSTEP, tt + 1);
            if (((tt + 1) & 1) || tt + 2 == TTC) load_a_scales(c + CSTEP, (tt + 1) >> 1);
          }
          scale_pairs(asn, asvn);
        }
        // K steps 2 and 3 of tile tt; behind every MFMA one dword of the next tile's operands of steps 0 and 1
#pragma unroll
        for (int m = 0; m < 8; ++m) {
          const int t = m >> 2, rt = m & 3;
#pragma unroll
          for (int r2 = rt; r2 < RT; r2 += 4)
            acc[r2][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[r2][2 + t]), __builtin_bit_cast(f16x8, fan[t]),
                                                                 acc[r2][tt], 0, 0, 0);
          if (tt + 1 < TTC) fa[m >> 2][m & 3] = dequant_pair(aqn[m >> 2], m & 3, asvn[0]);
          __builtin_amdgcn_sched_barrier(0);
        }
        aq = aqn;
        asv[1] = asvn[1];
      }
    };
    auto run = [&](auto ttc_c) {
      constexpr int TTC = decltype(ttc_c)::value;
      constexpr bool kFits = RT * TTC <= 20;  // accumulator registers that leave room for the finer scheme
      f32x4 acc[RT][TTC];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) acc[rt][tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      if (c_first < chunks) {
        load_b_part((uint32_t)c_first);
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) {
          load_a_tile((uint32_t)c_first, tt);
          if ((tt & 1) || tt + 1 == TTC) load_a_scales((uint32_t)c_first, tt >> 1);
        }
      }
      for (int c = c_first; c < chunks; c += CSTEP) {
        if constexpr (!kFits && RT == 4) chunk_pipe(ttc_c, (uint32_t)c, acc);
        else if constexpr (!kFits) chunk_coarse(ttc_c, (uint32_t)c, acc);
        else chunk(ttc_c, (uint32_t)c, acc);
      }
      finish(ttc_c, acc);
    };
    switch (tt_count) {
      case 1: run(std::integral_constant<int, 1>{}); break;
      case 2: run(std::integral_constant<int, 2>{}); break;
      case 3: run(std::integral_constant<int, 3>{}); break;
      case 4: run(std::integral_constant<int, (TT >= 4 ? 4 : 1)>{}); break;
      case 5: run(std::integral_constant<int, (TT >= 5 ? 5 : 1)>{}); break;
      case 6: run(std::integral_constant<int, (TT >= 6 ? 6 : 1)>{}); break;
      case 7: run(std::integral_constant<int, (TT >= 7 ? 7 : 1)>{}); break;
      case 8: run(std::integral_constant<int, (TT >= 8 ? 8 : 1)>{}); break;
      default: break;
    }
  } else {
    f32x4 acc[RT][TT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) acc[rt][tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue_chunk(c_first + d * CSTEP, d);
    int slot = 0;
    for (int c = c_first; c < chunks; c += CSTEP) {
      // the oldest chunk in flight has landed when only the loads of the next one (if there is one) are pending
      if (DEPTH == 2 && c + CSTEP < chunks)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const char* sp = reinterpret_cast<const char*>(red) + (wave * DEPTH + slot) * SLOT_BYTES;
      // the activation tiles are read out of LDS together with the weight tiles (few of them) or one at a time
      // right before their conversion (many: their registers would not fit)
      constexpr bool kLazyA = TT > 2;
      constexpr int NQ = kLazyA ? RT : NT;
      u32x4 q[NQ];
      uint32_t sc[NQ];
#pragma unroll
      for (int t = 0; t < NQ; ++t) q[t] = *reinterpret_cast<const u32x4*>(sp + t * 1024 + rd_payload);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
      if constexpr (!kLazyA) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) sc[RT + tt] = *reinterpret_cast<const uint32_t*>(sp + rd_asc[tt]) >> sc_shift;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: the slot may be refilled
        issue_chunk(c + DEPTH * CSTEP, slot);
      }
      u32x4 fb[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) dequant_frags(q[rt], sc[rt], fb[rt]);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        if (tt < tt_count) {
          u32x4 aq;
          uint32_t as;
          if constexpr (kLazyA) {
            aq = *reinterpret_cast<const u32x4*>(sp + (RT + tt) * 1024 + rd_payload);
            as = *reinterpret_cast<const uint32_t*>(sp + rd_asc[tt]) >> sc_shift;
            if (tt + 1 == tt_count) {
              asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the last read of the slot is complete
              issue_chunk(c + DEPTH * CSTEP, slot);
            }
          } else {
            aq = q[kLazyA ? 0 : RT + tt];
            as = sc[kLazyA ? 0 : RT + tt];
          }
          u32x4 fa[4];
          dequant_frags(aq, as, fa);
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
              acc[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[rt][t]),
                                                                   __builtin_bit_cast(f16x8, fa[t]), acc[rt][tt], 0, 0, 0);
        }
      }
      if constexpr (DEPTH == 2) slot ^= 1;
    }
    finish(std::integral_constant<int, TT>{}, acc);
  }
}

template <int RT, int TT, bool OUT_BF16>
int launch_nvfp4_skinny_ring_cfg(const Params& p, hipStream_t stream, int slabs = 1) {
  constexpr int SLOT_KIB = RT + TT + (RT + 1) / 2 + (TT + 1) / 2;
  // one slot per wavefront also where two would fit (M=16, N=14336, K=4096: 8.0 -> 7.5 us; K=14336: 9.6 -> 9.2 us)
  constexpr int DEPTH = 1;
  auto kern = nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH>;
  // the ring; the reduction reuses it and needs 8 KiB per partial tile of a round
  constexpr int red_kib = 8 * (RT * TT <= 8 ? RT * TT : TT);
  constexpr int ring_kib = 8 * DEPTH * SLOT_KIB;
  constexpr int lds_bytes = (ring_kib > red_kib ? ring_kib : red_kib) * 1024;
  static_assert(lds_bytes <= 160 * 1024, "LDS");
  const int splits = p.partial != nullptr ? p.splits : 1;
  if (splits > 1 ? note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d> grid=%ux%dx%d split_k + splitk_reduce_kernel", RT, TT,
                               (unsigned)(p.n / (16 * RT)), slabs, splits)
                 : note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d> grid=%ux%d", RT, TT, (unsigned)(p.n / (16 * RT)), slabs))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.n / (16 * RT)), (unsigned)slabs, (unsigned)splits), dim3(512), lds_bytes, stream, p);
  if (const int rc = check_launch("nvfp4_skinny_ring_kernel")) return rc;
  if (p.partial == nullptr) return NVF_OK;
  const int64_t mn = (int64_t)p.m * p.n;
  hipLaunchKernelGGL(splitk_reduce_kernel<OUT_BF16>, dim3((unsigned)ceil_div(mn / 4, 256)), dim3(256), 0, stream, p.partial, splits, mn, p.alpha,
                     static_cast<uint16_t*>(p.out));
  return check_launch("splitk_reduce_kernel");
}

template <int RT, int TT, bool OUT_BF16, bool NSPLIT>
int launch_nvfp4_skinny_grouped(const Params& p0, int rows_lo, int rows_hi, hipStream_t stream) {
  constexpr int SLOT_KIB = RT + TT + (RT + 1) / 2 + (TT + 1) / 2;
  // One slot per wavefront also where two would fit: measured faster for the groups of up to 32 rows (512 rows
  // over 256 experts, K=7168: 401 -> 375 us; K=2048: 432 -> 413 us).  Forcing the registers down to two
  // workgroups per compute unit on top of that costs more than it gains (450 us).
  constexpr int DEPTH = 1;
  auto kern = nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH, true, NSPLIT>;
  constexpr int red_kib = NSPLIT ? 0 : 8 * (RT * TT <= 8 ? RT * TT : TT);
  constexpr int ring_kib = 8 * DEPTH * SLOT_KIB;
  constexpr int lds_bytes = (ring_kib > red_kib ? ring_kib : red_kib) * 1024;
  static_assert(lds_bytes <= 160 * 1024, "LDS");
  Params p = p0;
  p.rows_lo = rows_lo;
  p.rows_hi = rows_hi;
  const int64_t wgs = (int64_t)p.groups * (p.n / (16 * RT * (NSPLIT ? 8 : 1)));
  if (wgs >= ((int64_t)1 << 31)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "too many (group, row block) pairs for one launch");
  if (note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d,grouped,nsplit=%d> grid=%lld rows=%d..%d", RT, TT, (int)NSPLIT, (long long)wgs, rows_lo,
                  rows_hi))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(512), lds_bytes, stream, p);
  return check_launch("nvfp4_skinny_ring_kernel (grouped)");
}

// -------------------------------------------------------------------------------------------------
// Grouped NVFP4, groups of up to 16 * TT rows against many weight rows (the mid-sized experts of a prefill): one
// work item per (group of the launch's row range, block of 8 * 16 * RT weight rows), found from the device-resident
// group sizes by a prefix scan, so that the items are dense in the workgroup index and every XCD gets the same
// number of them.  Each of the 8 wavefronts owns 16 * RT weight rows and walks all of K (no reduction), streaming
// its weights through private LDS slots like the streaming kernel above.  The group's activation rows are
// converted once per workgroup and chunk: wavefront w converts row tile w (16 rows, 128 deep) and leaves it in
// LDS as fp16 MFMA operands in lane order, where all 8 wavefronts read it (two buffers, one barrier per chunk).
// In the streaming kernel every wavefront converts every row tile it multiplies; here a wavefront converts one
// and multiplies all of them.
// A chunk is four 32-deep MFMA steps of TTC groups of RT MFMAs.  Everything else is dealt out between those
// groups, so that it issues while the matrix pipe works: the conversion of the weight operands of the next MFMA
// step, the conversion of this wavefront's activation tile of the next chunk, the read-out of the next chunk's
// weights and the loads that refill what has been read out.
// Loads complete in the order of issue, and that order is fixed - per chunk: activation tile of chunk c+2, weight
// part of chunk c+1+BSLOTS - so the waits are for counts that follow from it.  (Two chunks' weight parts issued
// together, for 128 contiguous bytes per row and visit, measured slower: what counts is how far ahead of its use
// a load is issued - with every compute unit busy a load takes two to three times as long as on an idle chip.)
// -------------------------------------------------------------------------------------------------
template <int RT, int TT, int BSLOTS, bool OUT_BF16>
__global__ __launch_bounds__(512) void nvfp4_group_panel_kernel(const Params p) {
  constexpr int W = 8;
  constexpr int B_SC = (RT + 1) / 2;
  constexpr int LB = RT + B_SC;              // loads of a chunk's weight part per wavefront
  constexpr int BSLOT = LB * 1024;           // weight tiles + their scale blocks
  constexpr int ASLOT = 2 * 1024;            // one activation tile + the scale block it belongs to
  constexpr int FP16_TILE = 4 * 1024;        // a converted tile: 4 MFMA steps x 64 lanes x 16 bytes
  extern __shared__ f32x4 panel_lds[];       // [W][BSLOTS][BSLOT] | [W][ASLOT] | [2][TT][FP16_TILE]
  __shared__ int item_prefix[kMaxGroups + 1];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int kbytes = p.k >> 1;
  const int chunks = p.k >> 7;
  const int sf_padded = p.k >> 4;  // K % 128 == 0: no padding columns
  const int nblocks = p.n / (16 * RT * W);

  // ---- which item: groups of the row range, in group order, nblocks items each
  if (wave == 0) {
    int running = 0;
    for (int base = 0; base < p.groups; base += 64) {
      const int gi = base + lane;
      int cnt = 0;
      if (gi < p.groups) {
        const int mg = p.problem_sizes[gi * 3];
        cnt = (mg >= p.rows_lo && mg <= p.rows_hi) ? 1 : 0;
      }
      int incl = cnt;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (gi < p.groups) item_prefix[gi + 1] = running + incl;
      running += __shfl(incl, 63, 64);
    }
    if (lane == 0) item_prefix[0] = 0;
  }
  __syncthreads();
  const int item_group = blockIdx.x / nblocks;  // the item's group is the item_group-th of the row range
  if (item_group >= item_prefix[p.groups]) return;
  int grp;
  {
    int lo = 0, hi = p.groups;  // the largest index with item_prefix[index] <= item_group
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (item_group < item_prefix[mid]) hi = mid; else lo = mid;
    }
    grp = __builtin_amdgcn_readfirstlane(lo);
  }
  const int n0 = ((blockIdx.x - item_group * nblocks) * W + wave) * (16 * RT);
  const int m_loc = __builtin_amdgcn_readfirstlane(p.problem_sizes[grp * 3]);
  const int64_t a_row0 = __builtin_amdgcn_readfirstlane(p.expert_offsets[grp]);
  const int64_t asf_row0 = __builtin_amdgcn_readfirstlane(p.sf_offsets[grp]);  // the group's own scale slab
  const int64_t b_row0 = (int64_t)grp * p.n;
  const int tt_count = (m_loc + 15) >> 4;
  const int my_tile = min(wave, tt_count - 1);  // wavefronts past the last tile fetch and convert it again (same code, same bytes)

  // ---- load side (memory order): lane L fetches row L/4, piece (L%4) ^ ((L/16)&3) of a payload tile
  const int lrow = lane >> 2, lpiece = (lane & 3) ^ ((lane >> 4) & 3);
  const uint8_t* b_base = p.b + (b_row0 + n0) * kbytes;
  const uint8_t* bsf_base = p.sfb + b_row0 * sf_padded + swizzle_128x4(n0 & ~127, 0, sf_padded);
  const uint8_t* a_base = p.a + a_row0 * kbytes;
  const uint8_t* asf_base = p.sfa + asf_row0 * sf_padded;
  uint32_t b_off[RT], bsf_off[B_SC];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) b_off[rt] = (uint32_t)(rt * 16 + lrow) * (uint32_t)kbytes + lpiece * 16;
  // scale block j of an operand: lane L = tile 2j + (L>>5), col tile (L>>4)&1, row L&15: the 16 bytes that
  // hold the scale words of rows {row, row+32, row+64, row+96} (mod 128) for that col tile
#pragma unroll
  for (int j = 0; j < B_SC; ++j) {
    const int t = min(2 * j + (lane >> 5), RT - 1);
    const int row = (n0 & 127) + t * 16 + (lane & 15);
    bsf_off[j] = (uint32_t)((row & 31) * 16 + ((lane >> 4) & 1) * 512);
  }
  const uint32_t a_off = (uint32_t)min(my_tile * 16 + lrow, m_loc - 1) * (uint32_t)kbytes + lpiece * 16;
  uint32_t asf_off;
  {
    const int t = min((my_tile & ~1) + (lane >> 5), 7);
    const int row = t * 16 + (lane & 15);
    asf_off = (uint32_t)((row & 31) * 16 + ((lane >> 4) & 1) * 512);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)panel_lds);
  const uint32_t bslot0 = lds0 + (uint32_t)wave * (BSLOTS * BSLOT), aslot = lds0 + W * BSLOTS * BSLOT + (uint32_t)wave * ASLOT;
  char* const lds_c = reinterpret_cast<char*>(panel_lds);
  const char* const bsp0 = lds_c + wave * (BSLOTS * BSLOT);
  const char* const asp = lds_c + W * BSLOTS * BSLOT + wave * ASLOT;
  char* const fp16 = lds_c + W * (BSLOTS * BSLOT + ASLOT);
  auto load_b = [&](uint32_t c) {  // chunk c lives in slot c % BSLOTS
    const uint32_t bslot = bslot0 + (c % BSLOTS) * BSLOT;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) lds_dma16(bslot + rt * 1024, b_base, b_off[rt] + c * 64u);
#pragma unroll
    for (int j = 0; j < B_SC; ++j) lds_dma16(bslot + (RT + j) * 1024, bsf_base, bsf_off[j] + c * 1024u);
  };
  auto load_a = [&](uint32_t c) {
    lds_dma16(aslot, a_base, a_off + c * 64u);
    lds_dma16(aslot + 1024, asf_base, asf_off + c * 1024u);
  };
  // s_waitcnt vmcnt(n) for a wave-uniform n (the operand is an immediate)
  auto wait_loads = [&](int n) {
    switch (n) {
#define NVF_VMCNT_CASE(n) case n: asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory"); break;
      NVF_VMCNT_CASE(1) NVF_VMCNT_CASE(2) NVF_VMCNT_CASE(3) NVF_VMCNT_CASE(4) NVF_VMCNT_CASE(5) NVF_VMCNT_CASE(6)
      NVF_VMCNT_CASE(7) NVF_VMCNT_CASE(8) NVF_VMCNT_CASE(9) NVF_VMCNT_CASE(10) NVF_VMCNT_CASE(11) NVF_VMCNT_CASE(12)
      NVF_VMCNT_CASE(13) NVF_VMCNT_CASE(14) NVF_VMCNT_CASE(15) NVF_VMCNT_CASE(16)
#undef NVF_VMCNT_CASE
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  };
  static_assert(2 * LB + 4 <= 16, "wait_loads covers up to 16 loads in flight");

  // ---- read side (MFMA order): lane (r, g) = row r, payload piece g, scale blocks 2g, 2g+1 of the chunk
  const int rd_payload = r * 64 + ((g ^ ((r >> 2) & 3)) * 16);
  int rd_bsc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int rowgroup = (((n0 & 127) + rt * 16) >> 5) & 3;  // which of the 4 words of the 16 bytes
    rd_bsc[rt] = (RT + (rt >> 1)) * 1024 + ((rt & 1) * 2 + (g >> 1)) * 256 + r * 16 + rowgroup * 4;
  }
  const int rd_asc = 1024 + ((my_tile & 1) * 2 + (g >> 1)) * 256 + r * 16 + ((my_tile * 16) >> 5) * 4;
  const int sc_shift = (g & 1) * 16;

  // e4m3 scales of a lane's two blocks -> fp16 pairs; one dword (8 values of one block) -> one MFMA operand
  auto scale_pairs = [&](uint32_t s2, f16x2 sv[2]) {
    const float f0 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 0), f1 = __builtin_amdgcn_cvt_f32_fp8((int)s2, 1);
    sv[0] = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f0, f0));
    sv[1] = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(f1, f1));
  };
  auto dequant_dword = [&](uint32_t qw, f16x2 sv) {
    const f16x2 h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 0) * sv;
    const f16x2 h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 1) * sv;
    const f16x2 h2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 2) * sv;
    const f16x2 h3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw, 1.0f, 3) * sv;
    return u32x4{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1), __builtin_bit_cast(uint32_t, h2),
                 __builtin_bit_cast(uint32_t, h3)};
  };
  auto read_b = [&](int c, u32x4 q[RT], uint32_t sc[RT]) {
    const char* const bsp = bsp0 + (c % BSLOTS) * BSLOT;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) q[rt] = *reinterpret_cast<const u32x4*>(bsp + rt * 1024 + rd_payload);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(bsp + rd_bsc[rt]) >> sc_shift;
  };

  const float alpha = p.alpha[grp];
  uint16_t* out = static_cast<uint16_t*>(p.out);

  auto run = [&](auto ttc_c) {
    constexpr int TTC = decltype(ttc_c)::value;
    f32x4 acc[RT][TTC];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) acc[rt][tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- before the loop: chunk 0's activation tile is converted, its weights are read out and their first
    // operands converted; then in flight, in this order (BSLOTS = 2: weight part 1 first): activation tile 1,
    // weight part 1 (BSLOTS = 2: weight part 2)
    u32x4 q[RT];            // packed weights of the current chunk
    f16x2 sv[RT][2];        // their scales
    u32x4 fb[RT];           // weight operands of the current MFMA step
    load_b(0);
    load_a(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    {
      const u32x4 aq = *reinterpret_cast<const u32x4*>(asp + rd_payload);
      const uint32_t as = *reinterpret_cast<const uint32_t*>(asp + rd_asc) >> sc_shift;
      uint32_t sc[RT];
      read_b(0, q, sc);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (BSLOTS == 2 && 1 < chunks) load_b(1);
      if (1 < chunks) load_a(1);
      if (BSLOTS < chunks) load_b(BSLOTS);
      f16x2 asv[2];
      scale_pairs(as, asv);
      char* dst = fp16 + my_tile * FP16_TILE + lane * 16;
#pragma unroll
      for (int t = 0; t < 4; ++t) *reinterpret_cast<u32x4*>(dst + t * 1024) = dequant_dword(aq[t], asv[t >> 1]);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        scale_pairs(sc[rt], sv[rt]);
        fb[rt] = dequant_dword(q[rt][0], sv[rt][0]);
      }
    }

    for (int c = 0; c < chunks; ++c) {
      const int buf = c & 1;
      const bool has1 = c + 1 < chunks, has2 = c + 2 < chunks;
      const bool has_b_next = c + BSLOTS < chunks;          // weight part issued during the previous chunk
      const bool has_b_new = c + 1 + BSLOTS < chunks;       // weight part issued during this chunk
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // this wavefront's tile of chunk c is in LDS
      // every wavefront has written its tile of this chunk and has finished reading the other buffer
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      const char* src = fp16 + buf * TT * FP16_TILE + lane * 16;
      char* dst = fp16 + ((buf ^ 1) * TT + my_tile) * FP16_TILE + lane * 16;
      // Activation operands come out of LDS kAhead groups before their use: a group is shorter than the latency of
      // the read.  Group number t * TTC + tt uses tile tt, MFMA step t.
      constexpr int kAhead = 3, kGroups = 4 * TTC;
      u32x4 ring[kAhead + 1];
      auto fetch = [&](int gi) {
        if (gi < kGroups) ring[gi % (kAhead + 1)] = *reinterpret_cast<const u32x4*>(src + (gi % TTC) * FP16_TILE + (gi / TTC) * 1024);
      };
#pragma unroll
      for (int gi = 0; gi < kAhead; ++gi) fetch(gi);
      // this wavefront's raw activation tile of chunk c+1: behind it in flight only the weight part issued during
      // the previous chunk
      u32x4 aq = {0, 0, 0, 0};
      uint32_t as = 0;
      f16x2 asv[2];
      if (has1) {
        wait_loads(has_b_next ? LB : 0);
        aq = *reinterpret_cast<const u32x4*>(asp + rd_payload);
        as = *reinterpret_cast<const uint32_t*>(asp + rd_asc) >> sc_shift;
      }
      u32x4 fbn[RT], qn[RT];
      uint32_t scn[RT];
      f16x2 svn[RT][2];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        qn[rt] = q[rt];
        scn[rt] = 0;
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        // The work between the groups of MFMA step t, one part per group (what is left over after the last group):
        //   parts 0 .. RT-1: weight operand of tile `part` for MFMA step t+1 (t = 3: for step 0 of the next chunk)
        //   part RT:         dword t of the activation tile of chunk c+1 -> fp16, into the other buffer
        //   part RT+1:       t = 0: scales of that tile; t = 1: refill of the raw activation slot (chunk c+2);
        //                    t = 2: read-out of the next chunk's weights; t = 3: refill of the slot read out
        auto part_work = [&](int part) {
          if (part < RT) {
            if (t < 3) fbn[part] = dequant_dword(q[part][t + 1], sv[part][(t + 1) >> 1]);
            else {
              scale_pairs(scn[part], svn[part]);
              fbn[part] = dequant_dword(qn[part][0], svn[part][0]);
            }
          } else if (part == RT) {
            if (t == 0) scale_pairs(as, asv);
            *reinterpret_cast<u32x4*>(dst + t * 1024) = dequant_dword(aq[t], asv[t >> 1]);
          } else if (part == RT + 1) {
            if (t == 1) {
              if (has2) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the raw tile has been read out
                load_a((uint32_t)c + 2);
              }
            } else if (t == 2) {
              if (has1) {
                // behind the weight part of chunk c+1: (BSLOTS = 2: activation tile c+1 - used up -, weight part
                // c+2,) activation tile c+2
                wait_loads((has2 ? 2 : 0) + (BSLOTS == 2 ? 2 + (has2 ? LB : 0) : 0));
                read_b(c + 1, qn, scn);
              }
            } else if (t == 3) {
              if (has_b_new) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: may be refilled
                load_b((uint32_t)c + 1 + BSLOTS);
              }
            }
          }
        };
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) {
          __builtin_amdgcn_sched_barrier(0);
          const int gi = t * TTC + tt;
          fetch(gi + kAhead);
          const u32x4 fa = ring[gi % (kAhead + 1)];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            acc[rt][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fb[rt]), __builtin_bit_cast(f16x8, fa),
                                                                 acc[rt][tt], 0, 0, 0);
          // the loads and the read-out first (part RT+1), then the conversions
          if (tt == 0) part_work(RT + 1);
          if (tt > 0 && tt - 1 <= RT) part_work(tt - 1);
          if (tt + 1 == TTC) {
#pragma unroll
            for (int part = TTC - 1; part <= RT; ++part) part_work(part);
          }
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) fb[rt] = fbn[rt];
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        q[rt] = qn[rt];
        sv[rt][0] = svn[rt][0];
        sv[rt][1] = svn[rt][1];
      }
    }

    // every wavefront holds finished sums: element e of lane l = weight row 4*(l/16) + e, activation row l%16
#pragma unroll
    for (int tt = 0; tt < TTC; ++tt) {
      const int tok = tt * 16 + r;
      if (tok < m_loc) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          u32x2 v;
          v[0] = pack2(acc[rt][tt][0] * alpha, acc[rt][tt][1] * alpha, OUT_BF16);
          v[1] = pack2(acc[rt][tt][2] * alpha, acc[rt][tt][3] * alpha, OUT_BF16);
          *reinterpret_cast<u32x2*>(out + (a_row0 + tok) * p.n + n0 + rt * 16 + 4 * g) = v;
        }
      }
    }
  };
  switch (tt_count) {  // (tt_count <= TT: the launcher's row range)
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, (TT >= 2 ? 2 : 1)>{}); break;
    case 3: run(std::integral_constant<int, (TT >= 3 ? 3 : 1)>{}); break;
    case 4: run(std::integral_constant<int, (TT >= 4 ? 4 : 1)>{}); break;
    case 5: run(std::integral_constant<int, (TT >= 5 ? 5 : 1)>{}); break;
    case 6: run(std::integral_constant<int, (TT >= 6 ? 6 : 1)>{}); break;
    case 7: run(std::integral_constant<int, (TT >= 7 ? 7 : 1)>{}); break;
    case 8: run(std::integral_constant<int, (TT >= 8 ? 8 : 1)>{}); break;
    default: break;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-direct load may outlive the workgroup
}

template <int RT, int TT, int BSLOTS, bool OUT_BF16>
int launch_nvfp4_group_panel(const Params& p0, int rows_lo, int rows_hi, hipStream_t stream) {
  auto kern = nvfp4_group_panel_kernel<RT, TT, BSLOTS, OUT_BF16>;
  constexpr int lds_bytes = 8 * (BSLOTS * (RT + (RT + 1) / 2) + 2) * 1024 + 2 * TT * 4096;
  static_assert(lds_bytes + (kMaxGroups + 1) * 4 <= 160 * 1024, "LDS");
  if (rows_hi > 16 * TT) return fail(NVF_ERR_LAUNCH, "group panel kernel: %d rows do not fit %d row tiles", rows_hi, TT);
  Params p = p0;
  p.rows_lo = rows_lo;
  p.rows_hi = rows_hi;
  // one workgroup per (group, block) of all groups: the group sizes live on the device and need not add up to the
  // rows of `a`, so no tighter bound is safe; workgroups past the last item return right after the prefix scan
  const int64_t wgs = (p.m < rows_lo ? 0 : (int64_t)p.groups) * (p.n / (128 * RT));
  if (wgs >= ((int64_t)1 << 31)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "too many (group, row block) pairs for one launch");
  if (note_launch("nvfp4_group_panel_kernel<RT=%d,TT=%d,slots=%d> grid=%lld rows=%d..%d", RT, TT, BSLOTS, (long long)wgs, rows_lo, rows_hi))
    return NVF_OK;
  if (wgs == 0) return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(512), lds_bytes, stream, p);
  return check_launch("nvfp4_group_panel_kernel");
}

template <int TT, bool OUT_BF16>
int launch_nvfp4_skinny_rt(const Params& p, int rt, hipStream_t stream, int slabs) {
  return rt == 4 ? launch_nvfp4_skinny_ring_cfg<4, TT, OUT_BF16>(p, stream, slabs)
       : rt == 2 ? launch_nvfp4_skinny_ring_cfg<2, TT, OUT_BF16>(p, stream, slabs)
                 : launch_nvfp4_skinny_ring_cfg<1, TT, OUT_BF16>(p, stream, slabs);
}

// Cost, in arbitrary units, of streaming the weights against M activation rows as slabs of `slab` rows with rt weight
// tiles (16 rows) per workgroup.  Every workgroup converts rt weight tiles and the tt row tiles of its slab per
// 128-deep chunk (a wavefront takes every eighth chunk), so few large workgroups convert least, while small ones (less
// LDS, fewer accumulators) share a compute unit and fill the chip at small N.  The constants are a fit to timings of
// the nine (slab, rt) forms over M = 48..256, N = 1024..14336, K = 2048..14336 (144 shapes: the form picked is within
// 8 % of the fastest for 134 of them, 1.8 % off on average; a fixed rule by N alone was 13 % off); for 1..32 rows
// (112 shapes) its pick of rt is 0.2 % off the fastest on average.
int64_t nvfp4_skinny_cost(int64_t m, int64_t n, int64_t k, int slab, int rt, int cus) {
  if (n % (16 * rt) != 0) return INT64_MAX;
  const int64_t slabs = m <= slab ? 1 : ceil_div(m, slab);
  const int tt = m <= slab ? (m <= 16 ? 1 : m <= 32 ? 2 : m <= 64 ? 4 : 8) : slab / 16;
  const int64_t wgs = slabs * (n / (16 * rt));
  const int lds_kib = 8 * (rt + tt + (rt + 1) / 2 + (tt + 1) / 2);
  int64_t per_cu = std::min(160 / lds_kib, 4);  // workgroups that share a compute unit
  if (rt * tt > 16) per_cu = 1;                 // (their accumulators take the registers)
  else if (rt * tt > 6) per_cu = std::min<int64_t>(per_cu, 2);
  if (per_cu < 1) per_cu = 1;
  const int64_t chunks = ceil_div(k >> 7, 8);
  const int64_t resident = std::min(per_cu, ceil_div(wgs, cus));
  const int64_t rounds = ceil_div(wgs, cus * per_cu);
  const int64_t per_chunk = (rt + tt) * 183 + rt * tt * 18 + 100;
  const int64_t wg_time = chunks * per_chunk * (100 + 73 * (resident - 1)) / 100 + rt * tt * 110 + 5070;
  return rounds * wg_time;
}

// best (slab height, weight tiles per workgroup) for more than 32 rows and its estimated cost
int64_t nvfp4_skinny_best(int64_t m, int64_t n, int64_t k, int cus, int* slab_out, int* rt_out) {
  int slab = 128, rt = 1;
  int64_t best = INT64_MAX;
  for (const int s : {128, 64, 32})
    for (const int r : {4, 2, 1}) {
      const int64_t c = nvfp4_skinny_cost(m, n, k, s, r, cus);
      if (c < best) best = c, slab = s, rt = r;
    }
  if (slab_out) *slab_out = slab;
  if (rt_out) *rt_out = rt;
  return best;
}

template <bool OUT_BF16>
int launch_nvfp4_skinny(const Params& p, int cus, hipStream_t stream) {
  // Up to 32 rows: one slab of 1 or 2 row tiles (16 x 6144 x 7168: 8.0 us with 1 weight tile per workgroup, 7.0 with 2).
  // More rows: slabs of 128, 64 or 32 rows side by side in one launch (blockIdx.y = slab; the last one may be ragged;
  // the slabs after the first find the weights in the last-level cache) with 1, 2 or 4 weight tiles per workgroup,
  // whichever the cost estimate above prefers (M=128, N=4096, K=4096: 10.8 us as two slabs of 64 rows x 1 weight tile,
  // 8.3 us x 2 tiles; M=256, N=4096, K=14336: 62 -> 34 us; M=256, N=6144, K=7168: 48 -> 29 us).
  int slab, rt;
  nvfp4_skinny_best(p.m, p.n, p.k, cus, &slab, &rt);
  if (p.m > slab) {
    const int slabs = (int)ceil_div(p.m, slab);
    return slab == 128 ? launch_nvfp4_skinny_rt<8, OUT_BF16>(p, rt, stream, slabs)
         : slab == 64  ? launch_nvfp4_skinny_rt<4, OUT_BF16>(p, rt, stream, slabs)
                       : launch_nvfp4_skinny_rt<2, OUT_BF16>(p, rt, stream, slabs);
  }
  return p.m <= 16 ? launch_nvfp4_skinny_rt<1, OUT_BF16>(p, rt, stream, 1)
       : p.m <= 32 ? launch_nvfp4_skinny_rt<2, OUT_BF16>(p, rt, stream, 1)
       : p.m <= 64 ? launch_nvfp4_skinny_rt<4, OUT_BF16>(p, rt, stream, 1)
                   : launch_nvfp4_skinny_rt<8, OUT_BF16>(p, rt, stream, 1);
}

// -------------------------------------------------------------------------------------------------
// grouped_mm fast path (16-bit operands): 256x256 tiles, N % 256 == 0, K % 64 == 0, K >= 128.
//   * Persistent workgroups walk the (group, m-tile, n-tile) list derived on the device from
//     problem_sizes; each XCD owns a contiguous part of the list, whose neighbouring tiles share the
//     group's weight panel in that XCD's L2.
//   * Tiles travel global -> LDS with 16-byte LDS-direct loads issued from inline assembly into a double
//     buffer (256 rows x 128 bytes per operand and 64-deep K step); the load stream runs two steps ahead
//     of the MFMAs and continues across tile and group borders.  Rows past the end of a group load the
//     group's last row again (never another group's memory past the tensor) and are not stored.
//   * MFMA fragments are double-buffered in registers: the LDS reads of the next half step are in flight
//     under the 32 MFMAs of the current one; one barrier per K step.
// LDS layout as in the NVFP4 fast path: chunk c of row r at chunk position c ^ ((r >> 1) & 7).
// -------------------------------------------------------------------------------------------------
template <bool BF16_MMA, bool OUT_BF16, bool STREAM_OUT>
__global__ __launch_bounds__(256, 1) void grouped16_gemm_256_kernel(const Params p) {
  constexpr int BM = 256, BN = 256;
  constexpr int kBand = 4;  // m-tiles that share a weight panel while it is in an XCD's L2 (8: measured no better)
  constexpr int TILE_UNITS = 2048;           // 16-byte units per operand tile (256 rows x 8 chunks)
  constexpr int BUF_UNITS = 2 * TILE_UNITS;  // A + B
  extern __shared__ u32x4 lds[];
  __shared__ int tile_prefix[kMaxGroups + 1];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lg = lane >> 5;
  const int tiles_n = p.n / BN;

  // ---- work list: prefix sums of 256-row tiles per group (one wavefront, 64 groups per round)
  if (wave == 0) {
    int running = 0;
    for (int base = 0; base < p.groups; base += 64) {
      const int g = base + lane;
      int cnt = 0;
      if (g < p.groups) {
        const int mg = p.problem_sizes[g * 3];
        cnt = mg > 0 ? (mg + BM - 1) / BM : 0;
      }
      int incl = cnt;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      if (g < p.groups) tile_prefix[g + 1] = running + incl;
      running += __shfl(incl, 63, 64);
    }
    if (lane == 0) tile_prefix[0] = 0;
  }
  __syncthreads();
  // Workgroup ids are dealt round-robin to the 8 XCDs.  The tiles of a group are walked in bands of up to 4 m-tiles,
  // n-major inside a band, so that 32 consecutive tiles share 4 A and 8 B panels in an XCD's L2 and a weight panel
  // comes in from memory once per band.  DEAL (n-tiles a multiple of
  // 8): XCD x takes the n-tiles x, x+8, ... of every band, i.e. its own list of (tiles / 8) tiles of the same make-up as
  // every other XCD's: each expert's weights stream in through all eight XCDs and all of them meet the cheap and
  // the expensive tiles (small groups are bound by streaming their weights once) at the same rate.  Otherwise XCD
  // x owns the contiguous eighth [x*chunk, (x+1)*chunk) of the one list.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const bool deal = (tiles_n & 7) == 0;
  const int per_m = deal ? tiles_n >> 3 : tiles_n;  // list entries per m-tile
  const int total = __builtin_amdgcn_readfirstlane(tile_prefix[p.groups]) * per_m;
  const int chunk_tiles = (total + 7) >> 3;
  const int range_end = deal ? total : min((xcd + 1) * chunk_tiles, total);
  const int first_tile = deal ? slot : xcd * chunk_tiles + slot;
  if (first_tile >= range_end) return;

  const int kb = p.k * 2;   // bytes per operand row
  const int nk = p.k >> 6;  // 64-deep steps

  struct Tile { const uint8_t *a, *b; int valid; int64_t out_row; int n0; };
  auto tile_info = [&](int t) {
    int lo = 0, hi = p.groups;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (t < tile_prefix[mid] * per_m) hi = mid; else lo = mid;
    }
    const int g = __builtin_amdgcn_readfirstlane(lo);
    // (loaded through the vector path, which is coherent with this kernel's own stores; made scalar here)
    const int m_g = __builtin_amdgcn_readfirstlane(p.problem_sizes[g * 3]);
    const int64_t row_off = __builtin_amdgcn_readfirstlane(p.expert_offsets[g]);
    const int tiles_m = (m_g + BM - 1) / BM;
    const int local = __builtin_amdgcn_readfirstlane(t - tile_prefix[g] * per_m);
    // bands of up to kBand m-tiles of near-equal height (9 m-tiles: 5 + 4), n-major inside a band
    const int nb = (tiles_m + kBand - 1) / kBand, base_h = tiles_m / nb, taller = tiles_m - base_h * nb;  // the first `taller` bands have base_h + 1
    const int mrow = local / per_m;  // m-tiles of the group that lie in earlier bands, plus a remainder
    const int split = taller * (base_h + 1);
    const int band = mrow < split ? mrow / (base_h + 1) : taller + (mrow - split) / base_h;
    const int band_h = band < taller ? base_h + 1 : base_h;
    const int band_m0 = band < taller ? band * (base_h + 1) : split + (band - taller) * base_h;
    const int in_band = local - band_m0 * per_m;
    const int ntl = in_band / band_h, mt = band_m0 + (in_band - ntl * band_h);
    const int nt = deal ? xcd + 8 * ntl : ntl;
    Tile r;
    r.a = p.a + (row_off + (int64_t)mt * BM) * kb;
    r.b = p.b + ((int64_t)g * p.n + (int64_t)nt * BN) * kb;
    r.valid = min(BM, m_g - mt * BM);
    r.out_row = row_off + (int64_t)mt * BM;
    r.n0 = nt * BN;
    return r;
  };

  // ---- LDS-direct load addressing.  Wave w issues 8 loads per operand per K step; load j covers LDS
  // units [(w*8+j)*64, +64) = rows (w*8+j)*8 .. +7; lane L lands at unit +L, i.e. row +(L>>3), chunk
  // position L&7, which must hold global chunk (L&7) ^ ((row>>1)&7) = (L&7) ^ ((L>>4) | ((j&1)<<2)).
  const uint32_t lrow = (uint32_t)(wave * 64 + (lane >> 3));  // row of this lane in load 0
  const uint32_t coff_even = (uint32_t)(((lane & 7) ^ (lane >> 4)) << 4);
  const uint32_t coff_odd = (uint32_t)(((lane & 7) ^ ((lane >> 4) | 4)) << 4);
  const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds);

  // ---- load stream: the tile the next loads are issued for (lp) and the one after it (np); it
  // advances without branches so that the hot loop stays one basic block
  Tile lp = tile_info(first_tile);
  Tile np = lp;
  int l_ks = 0, l_count = 0;
  // Unit q (0..15) of a step: operand q&1, rows (wave*8 + q/2)*8 .. +7
  auto issue_step_unit = [&](int q) {
    const int buf = l_count & 1;
    const int j = q >> 1;
    const uint32_t l = lds_base + (uint32_t)(buf * BUF_UNITS + (q & 1) * TILE_UNITS + wave * 512) * 16u + j * 1024u;
    const uint32_t row = lrow + 8u * j;
    const uint32_t coff = (j & 1) ? coff_odd : coff_even;
    if (q & 1) {
      lds_dma16(l, lp.b + ((int64_t)l_ks << 7), row * (uint32_t)kb + coff);
    } else {
      lds_dma16(l, lp.a + ((int64_t)l_ks << 7), min(row, (uint32_t)(lp.valid - 1)) * (uint32_t)kb + coff);
    }
  };
  auto issue_step_tail = [&]() {
    ++l_count;
    const bool wrap = (l_ks + 1 == nk);
    l_ks = wrap ? 0 : l_ks + 1;
    lp.a = wrap ? np.a : lp.a;
    lp.b = wrap ? np.b : lp.b;
    lp.valid = wrap ? np.valid : lp.valid;
  };
  // Fragment storage: [operand: 0 = A, 1 = B][sub-tile][MFMA of the half step].  Unit q (0..15) of a
  // half step is one ds_read_b128: operand q>>3, sub-tile (q>>1)&3, MFMA q&1.
  struct Frags { u32x4 h[2][4][2]; };
  auto load_unit = [&](int buf, int sub, int q, Frags& f) {
    const int op = q >> 3, t = (q >> 1) & 3, half = q & 1;
    const u32x4* base = lds + buf * BUF_UNITS + op * TILE_UNITS;
    const int row = (op ? wn : wm) * 128 + t * 32 + li;
    f.h[op][t][half] = base[lds_pos2(row, sub * 4 + lg + 2 * half)];
  };

  f32x16 acc[4][4];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  };
  zero_acc();
  auto mfma2 = [&](const Frags& f, int i, int j) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      if constexpr (BF16_MMA) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, f.h[1][j][kk]),
                                                            __builtin_bit_cast(bf16x8, f.h[0][i][kk]), acc[i][j], 0, 0, 0);
      } else {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, f.h[1][j][kk]),
                                                           __builtin_bit_cast(f16x8, f.h[0][i][kk]), acc[i][j], 0, 0, 0);
      }
    }
  };

  // Keeps the 16 accumulator tiles "used" at this point of the program, so that the MFMAs producing
  // them cannot be moved past the statement that follows (they have no side effects of their own).
#define NVF_PIN_ACC()                                                                                          \
  do {                                                                                                         \
    asm volatile("" : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]),     \
                 "+a"(acc[1][1]), "+a"(acc[1][2]), "+a"(acc[1][3]));                                           \
    asm volatile("" : "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]), "+a"(acc[3][0]),     \
                 "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));                                           \
  } while (0)

  Frags f0, f1;  // fragments of the first / second half (K 0..31 / 32..63) of a step

  // The stream runs two steps ahead of the MFMAs; with two steps per tile it is a whole tile ahead and
  // already leaves the first tile during this prologue.
  const int tiles_ahead = nk == 2 ? 2 : 1;
  np = (first_tile + slots < range_end) ? tile_info(first_tile + slots) : lp;
#pragma unroll
  for (int q = 0; q < 16; ++q) issue_step_unit(q);  // step 0
  issue_step_tail();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int q = 0; q < 16; ++q) issue_step_unit(q);  // step 1
  issue_step_tail();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int q = 0; q < 16; ++q) load_unit(0, 0, q, f0);

  int g = 0;
  Tile ct = tile_info(first_tile);
  for (int c_tile = first_tile; c_tile < range_end; c_tile += slots) {
    // prepare the tile the stream enters next (past the end of the list: any valid tile, loaded and ignored)
    const Tile nt_info = (c_tile + slots < range_end) ? tile_info(c_tile + slots) : ct;
    np = (c_tile + tiles_ahead * slots < range_end) ? tile_info(c_tile + tiles_ahead * slots) : ct;
    for (int c_ks = 0; c_ks < nk; ++c_ks, ++g) {
      const int buf = g & 1;
      // ---- first half: MFMAs on f0, interleaved with the LDS reads that fill f1
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        load_unit(buf, 1, q, f1);
        mfma2(f0, q >> 2, q & 3);
        __builtin_amdgcn_sched_barrier(0);
      }
      NVF_PIN_ACC();
      // Everything this wave loaded for step g+1 has landed and its reads of buf are complete; after
      // the barrier that holds for every wave, so buf^1 may be read and buf may be overwritten.
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      // ---- second half: MFMAs on f1, interleaved with the LDS reads of the next step's f0 (from buf^1;
      // after the last step they read stale data that is never used) and the loads of step g+2 into buf
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        load_unit(buf ^ 1, 0, q, f0);
        issue_step_unit(q);
        if (q == 15) issue_step_tail();
        mfma2(f1, q >> 2, q & 3);
        __builtin_amdgcn_sched_barrier(0);
      }
      NVF_PIN_ACC();
    }
    // ---- epilogue of this tile; the loads of the next tile's first two steps are already in flight.
    // acc[i][j][r] = C[m = li][n = (r/4)*8 + lg*4 + r%4] of its 32x32 sub-tile.
    // A lane holds 8-byte pieces of 32 different rows; stored like that, a tile is 8192 sixteen-byte write
    // requests per compute unit.  Every 32x64 block of the wavefront's tile is therefore turned round in a
    // private 4.5 KiB of LDS (32 rows of 128 bytes at a pitch of 144 bytes) and leaves in 16-byte pieces, 8 lanes
    // to a row's 128 bytes.  One LDS address each for writing and reading (the rest are immediate offsets) and
    // one 32-bit lane offset next to a wave-uniform result address keep the epilogue out of the spill area.
    int elane = lane;
    asm volatile("" : "+v"(elane));
    uint8_t* stage = reinterpret_cast<uint8_t*>(lds + 2 * BUF_UNITS) + wave * 4608;
    uint8_t* wr = stage + (elane & 31) * 144 + (elane >> 5) * 8;
    const uint8_t* rd = stage + (elane >> 3) * 144 + (elane & 7) * 16;
    const uint32_t ooff = ((uint32_t)(elane >> 3) * (uint32_t)p.n + (uint32_t)(elane & 7) * 8u) * 2u;
    uint8_t* obase = reinterpret_cast<uint8_t*>(static_cast<uint16_t*>(p.out) + (ct.out_row + wm * 128) * (int64_t)p.n + ct.n0 + wn * 128);
    const int erow = wm * 128 + (elane >> 3);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            const int j = jh * 2 + j2;
            u32x2 v;
            v[0] = pack2(acc[i][j][rq * 4 + 0], acc[i][j][rq * 4 + 1], OUT_BF16);
            v[1] = pack2(acc[i][j][rq * 4 + 2], acc[i][j][rq * 4 + 3], OUT_BF16);
            *reinterpret_cast<u32x2*>(wr + (j2 * 4 + rq) * 16) = v;
          }
        }
        asm volatile("" ::: "memory");  // the reads below see the writes above: one wavefront's LDS accesses stay in order
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int brow = i * 32 + 8 * t;  // first of the 8 rows of this piece, in the wavefront's tile
          const u32x4 v = *reinterpret_cast<const u32x4*>(rd + t * 1152);
          if (erow + brow < ct.valid) {
            u32x4* dst = reinterpret_cast<u32x4*>(obase + ((int64_t)brow * p.n + jh * 64) * 2 + ooff);
            if constexpr (STREAM_OUT) __builtin_nontemporal_store(v, dst);
            else *dst = v;
          }
        }
        asm volatile("" ::: "memory");
      }
    }
    zero_acc();
    ct = nt_info;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-direct load may outlive the workgroup
#undef NVF_PIN_ACC
}

template <bool BF16_MMA, bool OUT_BF16, bool STREAM_OUT>
int launch_grouped16_fast_cfg(const Params& p, int cus, hipStream_t stream) {
  auto kern = grouped16_gemm_256_kernel<BF16_MMA, OUT_BF16, STREAM_OUT>;
  constexpr int lds_bytes = 2 * 2 * 2048 * 16 + 4 * 4608;  // 128 KiB of tiles + the epilogue's 18 KiB
  if (note_launch("grouped16_gemm_256_kernel<stream_out=%d> grid=%d", (int)STREAM_OUT, cus & ~7)) return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(cus & ~7)), dim3(256), lds_bytes, stream, p);
  return check_launch("grouped16_gemm_256_kernel");
}

template <bool BF16_MMA, bool OUT_BF16>
int launch_grouped16_fast(const Params& p, int cus, hipStream_t stream) {
  // Operands and result together beyond what the 256 MB last-level cache holds: the result leaves with
  // non-temporal stores, which keeps it from pushing operand panels out (single 8192-row group, 8192^3: +2.6 %,
  // 16384 x 4096 x 4096: +7 %); smaller problems are better off with plain stores.
  const int64_t bytes = 2 * ((int64_t)p.m * p.k + (int64_t)p.groups * p.n * p.k + (int64_t)p.m * p.n);
  return bytes > ((int64_t)224 << 20) ? launch_grouped16_fast_cfg<BF16_MMA, OUT_BF16, true>(p, cus, stream)
                                       : launch_grouped16_fast_cfg<BF16_MMA, OUT_BF16, false>(p, cus, stream);
}

template <int BM, int BN, bool BF16_MMA, bool OUT_BF16>
int launch_cfg(const Params& p, int grid, hipStream_t stream) {
  auto kern = gemm16_kernel<BM, BN, BF16_MMA, OUT_BF16>;
  constexpr int lds_bytes = 2 * (BM + BN) * 128;
  if (note_launch("gemm16_kernel<%d,%d> grid=%d", BM, BN, grid)) return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, p);
  return check_launch("gemm16_kernel");
}

template <int BM, int BN, bool OUT_BF16, bool OUT_F32 = false, bool OUT_FP4 = false>
int launch_nvfp4_tile(const Params& p, int grid, hipStream_t stream) {
  auto kern = nvfp4_tile_kernel<BM, BN, OUT_BF16, OUT_F32, false, OUT_FP4>;
  constexpr int lds_bytes = 2 * (BM + BN) * 128;
  if (note_launch("nvfp4_tile_kernel<%d,%d,f32=%d%s> grid=%d skip_whole_256=%d min_rows=%d", BM, BN, (int)OUT_F32, OUT_FP4 ? ",fp4_blockscale" : "", grid,
                  p.skip_whole_256, p.min_rows))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, p);
  return check_launch("nvfp4_tile_kernel");
}

// Dense NVFP4 without a workspace: the weight-streaming kernel, the persistent kernel with 256x256 or 128x256 tiles,
// or the tile kernels?  Costs in units of one round of 256x256 tiles over the compute units = 100 (24 us per 1024 of
// K): a round of 128-row tiles costs 58 (half the flops at 86 % of the rate); the tile kernels run their 128x128 tiles
// two to a compute unit: 68 per such round, 45 for a last round of one tile per compute unit, and 22..47 when there
// is no more than that in all (all measured: M = 128..1024, N = 2048..14336, K = 4096 and 14336).
struct DensePlan {
  enum Kernel { kStream, kTiles256, kTiles128, kOther } kernel;
  int64_t ns;  // estimated duration (INT64_MAX: no estimate)
};
DensePlan nvfp4_dense_plan(int64_t m, int64_t n, int64_t k, int cus) {
  const bool stream_ok = (k & 127) == 0 && (n & 15) == 0 && k * 64 < (1ll << 31);  // 32-bit lane offsets
  const bool persistent_ok = (m & 127) == 0 && (n & 255) == 0 && (k & 127) == 0 && k >= 256;
  int64_t cost256 = INT64_MAX, cost128 = INT64_MAX, cost_tile = INT64_MAX;
  if (persistent_ok) {
    const int64_t t256 = (m & 255) == 0 ? (m / 256) * (n / 256) : 0, t128 = (m / 128) * (n / 256);
    cost256 = t256 ? 100 * ceil_div(t256, cus) : INT64_MAX;
    cost128 = 58 * ceil_div(t128, cus);
    const int64_t small = 2 * t128, full = small / (2 * cus), rest = small - full * 2 * cus;
    cost_tile = full * 68 + (rest == 0 ? 0 : rest > cus ? 68 : full ? 45 : 22 + 25 * rest / cus);
  }
  const int64_t cost_min = std::min(cost256, std::min(cost128, cost_tile));
  const int64_t rest_ns = persistent_ok ? 6000 + cost_min * 240 * k / 1024 : INT64_MAX;
  if (stream_ok) {
    // the streaming kernel's estimate is in ns within 0.8 (K = 2048) .. 1.1 (K = 14336)
    const int64_t stream_ns = nvfp4_skinny_best(m, n, k, cus, nullptr, nullptr) * (k < 3072 ? 82 : k < 6144 ? 96 : k < 10240 ? 103 : 110) / 100;
    bool stream;
    if (m <= 256) {
      stream = true;  // at most two passes over the weights (256 x 14336 x 4096: 38 instead of 58 us on tiles)
    } else if (persistent_ok && k >= 2048) {
      // by estimated duration (measured: 512 x 4096 x 14336 115 -> 57 us, 384 x 8192 x 7168 82 -> 57 us,
      // 640 x 14336 x 14336 381 -> 268 us; 1024 x 8192 x 4096 stays on 128x256 tiles: 64 against 76 us)
      stream = stream_ns <= rest_ns;
    } else {
      // Ragged shapes, which only the tile kernels take otherwise: with a deep K and a small N the streaming kernel
      // fills the chip where they cannot, while its workgroups (one per 128 rows x 16 columns at such N) cover the
      // compute units at most 3 times, 2 times for K < 4096 (measured: 300 x 3072 x 2048 in 18 instead of 16 us,
      // 1000 x 288 x 2560, 2100 x 96 x 4096).
      const int64_t rounds = ceil_div(ceil_div(m, 128) * (n / 16), cus);
      stream = k >= 2048 && rounds <= (k >= 4096 ? 3 : 2);
    }
    if (stream) return {DensePlan::kStream, stream_ns};
  }
  if (persistent_ok) {
    if (cost256 <= cost128 && cost256 <= cost_tile) return {DensePlan::kTiles256, rest_ns};
    if (cost128 <= cost_tile) return {DensePlan::kTiles128, rest_ns};
  }
  return {DensePlan::kOther, rest_ns};
}

// Dense shapes whose M is not a multiple of 128 and that only the tile kernels would take whole: the number of rows
// (the last multiple of 128) that go to a launch of their own, if that shape gets a better kernel; else 0.  If that
// kernel is the weight-streaming one, which takes any number of rows, the answer is m: no cut, all rows to it.
int64_t nvfp4_rows_before_remainder(int64_t m, int64_t n, int64_t k, int cus) {
  if (m <= 128 || (m & 127) == 0 || (k & 15) != 0) return 0;
  if (nvfp4_dense_plan(m, n, k, cus).kernel != DensePlan::kOther) return 0;
  // the cut is the last multiple of 128 or of 256 (which allows 256x256 tiles), whichever is estimated faster
  int64_t best = INT64_MAX, cut = 0;
  for (const int64_t c : {m & ~(int64_t)127, m & ~(int64_t)255}) {
    if (c < 128) continue;
    const DensePlan main = nvfp4_dense_plan(c, n, k, cus), rest = nvfp4_dense_plan(m - c, n, k, cus);
    if (main.kernel == DensePlan::kOther || rest.kernel != DensePlan::kStream || main.ns == INT64_MAX) continue;
    if (main.ns + rest.ns < best) best = main.ns + rest.ns, cut = main.kernel == DensePlan::kStream ? m : c;
  }
  return cut;
}

// Split of K for dense NVFP4 shapes with fewer 128x128 tiles than compute units and a deep K (decode and
// small prefill batches against a down projection): about two work items per compute unit, at least eight
// 128-deep spans each.  Every split writes and the reduction re-reads an fp32 copy of the output, so for
// K below 8192 the split costs more than it gains (measured) and 1 is returned.
int nvfp4_splits(int64_t m, int64_t n, int64_t k, int cus) {
  const int64_t tiles = ceil_div(m, 128) * ceil_div(n, 128), nspans = ceil_div(k, 128);
  if (m <= 64 || tiles >= cus || nspans < 64) return 1;
  // not where the weight-streaming kernel runs, which splits K over the wavefronts of a workgroup (256 x 2048 x 8192:
  // 14 us against 28 us for this split; 512 x 4096 x 14336: 56 against 78 us)
  if (nvfp4_dense_plan(m, n, k, cus).kernel == DensePlan::kStream) return 1;
  int64_t s = (2 * (int64_t)cus) / tiles;
  if (s > nspans / 8) s = nspans / 8;
  if (s > 32) s = 32;
  return s < 2 ? 1 : (int)s;
}

// Split of K over workgroups for the weight-streaming kernel with one slab of 65..96 activation rows: every
// workgroup converts all activation rows of its K range next to its weight rows, so 64 weight rows per workgroup
// (4 tiles against 8 activation tiles: 12 conversions for 32 MFMA tiles) halve the conversion work of 16 (1 against
// 8: 9 for 8), and where N / 64 workgroups leave compute units idle, K is split over as many workgroups as fit.
int nvfp4_skinny_splits(int64_t m, int64_t n, int64_t k, int cus) {
  // (measured against the forms without a split: 65 x 4096 x 14336 18.7 against 21.7 us, 96 x 8192 x 14336 30.9
  // against 33.2, 65 x 6144 x 8192 17.7 against 19.1; from 97 rows on, or with a weight matrix of less than 48 Mi
  // elements, the second launch costs more than the split gains: 128 x 8192 x 14336 38.1 against 35.3, 65 x 4096 x 8192
  // 16.3 against 13.9, 65 x 2048 x 14336 15.5 against 14.0)
  if (m <= 64 || m > 96 || (k & 127) != 0 || (n & 63) != 0 || k * 64 >= (1ll << 31) || n * k < (48ll << 20)) return 1;
  const int64_t wgs = n / 64, chunks = k >> 7;
  int64_t s = cus / wgs;
  if (s > chunks / 28) s = chunks / 28;
  if (s > 8) s = 8;
  if (wgs * s * 2 < cus) return 1;  // would leave most compute units idle: the tile kernel's split has more items
  return s < 2 ? 1 : (int)s;
}

template <bool OUT_BF16>
int launch_nvfp4_splitk(const Params& p0, int splits, float* workspace, hipStream_t stream) {
  Params p = p0;
  const int nspans = (p.k + 127) >> 7;
  p.spans_per_split = (nspans + splits - 1) / splits;
  p.splits = (nspans + p.spans_per_split - 1) / p.spans_per_split;  // no empty split
  p.partial = workspace;
  auto kern = nvfp4_tile_kernel<128, 128, OUT_BF16, false, true>;
  constexpr int lds_bytes = 2 * (128 + 128) * 128;
  const int64_t items = ceil_div(p.m, 128) * ceil_div(p.n, 128) * p.splits;
  if (note_launch("nvfp4_tile_kernel<128,128,split_k> grid=%lld splits=%d + splitk_reduce_kernel", (long long)items, p.splits)) return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)items), dim3(256), lds_bytes, stream, p);
  int rc = check_launch("nvfp4_tile_kernel (split K)");
  if (rc != NVF_OK) return rc;
  const int64_t mn = (int64_t)p.m * p.n;
  hipLaunchKernelGGL(splitk_reduce_kernel<OUT_BF16>, dim3((unsigned)ceil_div(mn / 4, 256)), dim3(256), 0, stream, workspace, p.splits,
                     mn, p.alpha, static_cast<uint16_t*>(p.out));
  return check_launch("splitk_reduce_kernel");
}

// tile kernel of the operand type: NVFP4 or 16-bit
template <int BM, int BN, bool NVFP4, bool BF16_MMA, bool OUT_BF16>
int launch_tile(const Params& p, int grid, hipStream_t stream) {
  if constexpr (NVFP4) return launch_nvfp4_tile<BM, BN, OUT_BF16>(p, grid, stream);
  else return launch_cfg<BM, BN, BF16_MMA, OUT_BF16>(p, grid, stream);
}

// Grouped NVFP4: rows in all from which a call counts as a prefill, whose large groups get launches of their own on the
// persistent kernel.  Below, those launches find a handful of tiles each and run one after the other at a tile's
// latency (256 experts, Zipf loads, K=7168: 2048 rows 732 -> 576 us, 4096 rows 769 -> 608 us without them; 8192 rows
// 807 with against 753 without, but evenly loaded experts 639 against 771).
constexpr int64_t kPrefillRows = 6144;

template <bool NVFP4, bool BF16_MMA, bool OUT_BF16>
int launch_sized(const Params& p, int64_t m_hint, int cus, void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  // Pick the largest tile that still yields about one work item per compute unit.
  auto tiles = [&](int bm, int bn) { return ceil_div(m_hint, bm) * ceil_div(p.n, bn); };
  const bool dense = p.problem_sizes == nullptr;
  if constexpr (NVFP4) {
    if (dense && workspace != nullptr) {
      const int skinny_splits = nvfp4_skinny_splits(p.m, p.n, p.k, cus);
      if (skinny_splits > 1 && workspace_bytes >= (int64_t)skinny_splits * p.m * p.n * 4) {
        Params q = p;
        const int chunks = p.k >> 7;
        q.partial = static_cast<float*>(workspace);
        q.spans_per_split = (chunks + skinny_splits - 1) / skinny_splits;
        q.splits = (chunks + q.spans_per_split - 1) / q.spans_per_split;  // no empty split
        return launch_nvfp4_skinny_ring_cfg<4, 8, OUT_BF16>(q, stream, 1);
      }
      const int splits = nvfp4_splits(p.m, p.n, p.k, cus);
      if (splits > 1 && workspace_bytes >= (int64_t)splits * p.m * p.n * 4)
        return launch_nvfp4_splitk<OUT_BF16>(p, splits, static_cast<float*>(workspace), stream);
    }
    if (dense) {
      const DensePlan plan = nvfp4_dense_plan(p.m, p.n, p.k, cus);
      if (plan.kernel == DensePlan::kStream) return launch_nvfp4_skinny<OUT_BF16>(p, cus, stream);
      if (plan.kernel == DensePlan::kTiles256) return launch_nvfp4_fast<OUT_BF16, false, 4>(p, cus, stream);
      if (plan.kernel == DensePlan::kTiles128) return launch_nvfp4_fast<OUT_BF16, false, 2>(p, cus, stream);
    }
  }
  if constexpr (!NVFP4) {
    // grouped_mm with groups of a few hundred rows on average: persistent LDS-direct kernel
    if (!dense && m_hint >= 256 * (int64_t)p.groups && tiles(256, 256) >= cus / 2 && (p.n & 255) == 0 && (p.k & 63) == 0 &&
        p.k >= 128 && (int64_t)p.k * 2 * 256 < (1ll << 31))
      return launch_grouped16_fast<BF16_MMA, OUT_BF16>(p, cus, stream);
  }
  if constexpr (NVFP4) {
    // Grouped NVFP4: groups of up to 128 rows (MoE decode, the small experts of a prefill) stream their expert's
    // weights once through the skinny kernel; the launches below then skip them.  The group sizes live on
    // the device, so every kernel is always launched; workgroups without work return at once.
    if (!dense && p.min_rows == 0 && (p.n & 63) == 0 && (p.k & 127) == 0 && (int64_t)p.k * 64 < (1ll << 31)) {
      // With a shallow K a split of K over the wavefronts leaves each only a chunk or two: they then own
      // different weight rows instead (K=2048, N=7168: 549 -> 464 us for 64 tokens x top-8; deeper K: slower).
      int rc, tail_done = 0;
      if (p.k < 4096 && (p.n & 255) == 0) rc = launch_nvfp4_skinny_grouped<2, 2, OUT_BF16, true>(p, 1, 32, stream);
      else rc = launch_nvfp4_skinny_grouped<4, 2, OUT_BF16, false>(p, 1, 32, stream);
      if (rc != NVF_OK) return rc;
      if ((p.k < 4096 || m_hint < kPrefillRows) && (p.n & 255) == 0 && p.k >= 256) {
        // shallow K: one 128x256 tile of the persistent kernel per weight panel converts a group's rows once per 256
        // weight rows; the streaming kernel whose wavefronts own rows converts them once per wavefront.  Few rows
        // in all (a decode step): such groups are rare and the persistent kernel costs least when it finds none.
        Params mid = p;
        mid.rows_lo = 33;
        mid.rows_hi = 128;
        if (m_hint >= kPrefillRows) mid.min_rows = 129;  // the 256x256 kernel follows: take the ends of its groups along
        tail_done = mid.min_rows != 0;
        if (m_hint >= kPrefillRows && (p.n & 511) == 0 && p.k >= 1024) {
          // a prefill: the groups of up to 80 rows on the panel kernel, which multiplies row tiles of 16 (config 5,
          // K=2048: 5376 tiles of 128x256 in 680 us -> 325 us + 1792 tiles in 227 us)
          rc = launch_nvfp4_group_panel<4, 5, 2, OUT_BF16>(p, 33, 80, stream);
          if (rc != NVF_OK) return rc;
          mid.rows_lo = 81;
        }
        rc = launch_nvfp4_fast<OUT_BF16, true, 2>(mid, cus, stream);
      } else if (p.k < 4096 && (p.n & 255) == 0) {
        rc = launch_nvfp4_skinny_grouped<2, 8, OUT_BF16, true>(p, 33, 128, stream);
      } else if ((p.n & 511) == 0) {
        rc = launch_nvfp4_group_panel<4, 5, 2, OUT_BF16>(p, 33, 80, stream);
        if (rc == NVF_OK) {
          // groups of 81..128 rows and the ends of the groups that the 256x256 kernel takes: 128x256 tiles of the
          // persistent kernel, at 1.2 times the rate of the 128x128 tile kernel
          Params ends = p;
          ends.rows_lo = 81;
          ends.rows_hi = 128;
          ends.min_rows = 129;
          tail_done = 1;
          rc = launch_nvfp4_fast<OUT_BF16, true, 2>(ends, cus, stream);
        }
      } else {
        rc = launch_nvfp4_skinny_grouped<4, 8, OUT_BF16, false>(p, 33, 128, stream);
      }
      if (rc != NVF_OK) return rc;
      Params rest = p;
      rest.min_rows = 129;
      rest.tail_done = tail_done;
      return launch_sized<NVFP4, BF16_MMA, OUT_BF16>(rest, m_hint, cus, workspace, workspace_bytes, stream);
    }
    // Grouped NVFP4 with room for whole 256-row tiles: those go to the 256x256 kernel (about 1.4 times as
    // fast per flop), the ends of the groups to the 128x128 tile kernel.  The group sizes live on the
    // device, so both kernels are always launched; one that finds no work returns at once.
    if (!dense && (p.n & 255) == 0 && (p.k & 127) == 0 && p.k >= 256 && m_hint >= kPrefillRows) {
      const int rc = launch_nvfp4_fast<OUT_BF16, true>(p, cus, stream);
      if (rc != NVF_OK || p.tail_done) return rc;
      Params rest = p;
      rest.skip_whole_256 = 1;
      const int64_t upper = 2 * (int64_t)p.groups * ceil_div(p.n, 128), cap = 2 * (int64_t)cus;
      return launch_nvfp4_tile<128, 128, OUT_BF16>(rest, (int)(upper < cap ? upper : cap), stream);
    }
  }
  // grouped: the tile height follows the average group (a 256-row tile on a 77-row group is mostly padding)
  if (dense ? tiles(256, 256) >= cus : m_hint >= 512 * (int64_t)p.groups) {
    const int64_t upper = dense ? tiles(256, 256) : (ceil_div(p.m, 256) + p.groups) * ceil_div(p.n, 256);
    return launch_tile<256, 256, NVFP4, BF16_MMA, OUT_BF16>(p, (int)(upper < cus ? upper : cus), stream);
  }
  if (tiles(128, 128) >= cus || !dense) {
    const int64_t upper = dense ? tiles(128, 128) : (ceil_div(p.m, 128) + p.groups) * ceil_div(p.n, 128);
    const int64_t cap = 2 * (int64_t)cus;
    return launch_tile<128, 128, NVFP4, BF16_MMA, OUT_BF16>(p, (int)(upper < cap ? upper : cap), stream);
  }
  const int64_t upper = tiles(64, 64);
  const int64_t cap = 4 * (int64_t)cus;
  return launch_tile<64, 64, NVFP4, BF16_MMA, OUT_BF16>(p, (int)(upper < cap ? upper : cap), stream);
}

// Dense NVFP4 whose result leaves the kernel re-quantized to NVFP4 (FP4: nvfp4_scaled_mm_blockscale) or as the fp32
// product itself (that op's optional dump of what it quantized).  Both take the same kernel for a shape, so that
// the dump holds exactly the accumulators the quantized result was made from.
template <bool FP4>
int launch_nvfp4_wide(const Params& p, int cus, hipStream_t stream) {
  auto tiles = [&](int bm, int bn) { return ceil_div(p.m, bm) * ceil_div(p.n, bn); };
  if (FP4 && ((p.m & 127) != 0 || ((p.n >> 4) & 3) != 0)) {
    // ragged: the padding rows / columns of the scale buffer's last 128x4 tiles are written as zero first
    const int64_t words = round_up(p.m, 128) * round_up(p.n >> 4, 4) / 4;
    if (!note_launch("zero_fill_kernel grid=%lld", (long long)ceil_div(words, 256))) {
      hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)ceil_div(words, 256)), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(p.out_sf), words);
      if (const int rc = check_launch("zero_fill_kernel")) return rc;
    }
  }
  if ((p.n & 255) == 0 && (p.k & 127) == 0 && p.k >= 256) {
    // as for the 16-bit results: persistent 256x256 or 128x256 tiles where they fill the compute units
    const int64_t t256 = (p.m & 255) == 0 ? tiles(256, 256) : 0, t128 = (p.m & 127) == 0 ? tiles(128, 256) : 0;
    const int64_t cost256 = t256 ? 100 * ceil_div(t256, cus) : INT64_MAX;
    const int64_t cost128 = t128 ? 58 * ceil_div(t128, cus) : INT64_MAX;
    const int64_t cost_tile = 144 * tiles(128, 256) / (2 * cus);
    if (t256 && cost256 <= cost128 && cost256 <= cost_tile) return launch_nvfp4_fast<false, false, 4, !FP4, FP4>(p, cus, stream);
    if (t128 && cost128 <= cost_tile) return launch_nvfp4_fast<false, false, 2, !FP4, FP4>(p, cus, stream);
  }
  if (tiles(256, 256) >= cus) return launch_nvfp4_tile<256, 256, false, !FP4, FP4>(p, cus, stream);
  if (tiles(128, 128) >= cus) {
    const int64_t t = tiles(128, 128);
    return launch_nvfp4_tile<128, 128, false, !FP4, FP4>(p, (int)(t < 2 * cus ? t : 2 * cus), stream);
  }
  const int64_t t = tiles(64, 64);
  return launch_nvfp4_tile<64, 64, false, !FP4, FP4>(p, (int)(t < 4 * cus ? t : 4 * cus), stream);
}

}  // namespace

int launch_gemm16(int op, const Gemm16Args& a, hipStream_t stream) {
  if (a.groups > kMaxGroups) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "at most %d groups are supported, got %d", kMaxGroups, a.groups);
  if (a.m > INT32_MAX || a.n > INT32_MAX || a.k > INT32_MAX) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "dimension exceeds int32");
  // (the kernels address a tile's 256 rows with 32-bit byte offsets)
  if (a.k >= (1 << 22)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "K = %lld: at most 4194303 is supported", (long long)a.k);
  Params p;
  p.a = static_cast<const uint8_t*>(a.a);
  p.b = static_cast<const uint8_t*>(a.b);
  p.sfa = static_cast<const uint8_t*>(a.sfa);
  p.sfb = static_cast<const uint8_t*>(a.sfb);
  p.alpha = a.alpha;
  p.out = a.out;
  p.problem_sizes = a.problem_sizes;
  p.expert_offsets = a.expert_offsets;
  p.sf_offsets = a.sf_offsets;
  p.groups = op == 0 ? 1 : a.groups;
  p.m = (int)a.m;
  p.n = (int)a.n;
  p.k = (int)a.k;
  const int cus = cu_count();
  const bool bf16 = a.dtype == NVF_BF16;
  if (op == 0 && a.dtype == NVF_F32) return launch_nvfp4_wide<false>(p, cus, stream);
  if (op == 0 && a.dtype == kDtypeFp4BlockScaled) {
    p.out_sf = static_cast<uint8_t*>(a.out_sf);
    p.gnorm = a.gnorm;
    return launch_nvfp4_wide<true>(p, cus, stream);
  }
  if (op == 0 || op == 1) {
    auto launch = [&](const Params& q, void* workspace, int64_t workspace_bytes) {
      return bf16 ? launch_sized<true, false, true>(q, q.m, cus, workspace, workspace_bytes, stream)
                  : launch_sized<true, false, false>(q, q.m, cus, workspace, workspace_bytes, stream);
    };
    // Dense with M not a multiple of 128 (a prefill of any token count), which leaves the whole call to the tile
    // kernels: the rows up to the last multiple of 128 go to whatever kernel that shape gets, the remaining rows
    // (at most 127, a whole number of 128-row scale tiles further on) to the weight-streaming kernel in a launch of
    // their own (4000 x 4096 x 4096: 145 -> 116 us; 8100 x 8192 x 8192: 1002 -> 850 us).
    const int64_t main_rows = op == 0 ? nvfp4_rows_before_remainder(p.m, p.n, p.k, cus) : 0;
    if (main_rows == p.m) return bf16 ? launch_nvfp4_skinny<true>(p, cus, stream) : launch_nvfp4_skinny<false>(p, cus, stream);
    if (main_rows) {
      Params main = p, rest = p;
      main.m = (int)main_rows;
      rest.m = p.m - main.m;
      const int64_t sf_padded = ((int64_t)(p.k >> 4) + 3) & ~(int64_t)3;
      rest.a = p.a + (int64_t)main.m * (p.k >> 1);
      rest.sfa = p.sfa + (int64_t)main.m * sf_padded;
      rest.out = static_cast<uint8_t*>(p.out) + (int64_t)main.m * p.n * 2;
      if (const int rc = launch(main, a.workspace, a.workspace_bytes)) return rc;
      return launch(rest, nullptr, 0);
    }
    return launch(p, a.workspace, a.workspace_bytes);
  }
  return bf16 ? launch_sized<false, true, true>(p, a.m, cus, nullptr, 0, stream)
              : launch_sized<false, false, false>(p, a.m, cus, nullptr, 0, stream);
}

// -------------------------------------------------------------------------------------------------
// Scratch memory that needs no allocation: the fp32 partial tiles of the split of K, for callers that cannot
// allocate (code under HIP graph capture, tight serving loops).  One array per device, held until the process
// ends; it keeps the contents of the last call, and the split-K kernels need no clearing because every partial
// tile the reduction reads has been written by the launch before it.  Calls that overlap on one device race.
// -------------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of this device's copy of the array.  The array's name is only a host-side stand-in; the address
// comes from hipGetSymbolAddress, asked once per device with that device current.
int static_scratch(void** ptr) {
  static std::mutex mu;
  static void* addr[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(NVF_ERR_NO_DEVICE, "hipGetDevice failed");
  if (dev < 0 || dev >= 64) return fail(NVF_ERR_NO_DEVICE, "device id %d is out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (addr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) return fail(NVF_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    addr[dev] = p;
  }
  *ptr = addr[dev];
  return NVF_OK;
}

int64_t nvfp4_gemm_workspace_bytes(int64_t m, int64_t n, int64_t k) {
  if (m <= 0 || n <= 0 || k <= 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX) return 0;
  if (const int64_t main_rows = nvfp4_rows_before_remainder(m, n, k, cu_count())) {
    if (main_rows == m) return 0;  // all rows to the weight-streaming kernel
    m = main_rows;                 // the launch that may split K
  }
  const int skinny_splits = nvfp4_skinny_splits(m, n, k, cu_count());
  const int splits = skinny_splits > 1 ? skinny_splits : nvfp4_splits(m, n, k, cu_count());
  return splits > 1 ? (int64_t)splits * m * n * 4 : 0;
}

}  // namespace nvf
