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
  // grouped skinny kernel: 0 = one block of workgroups per group (those of other sizes return at once); otherwise the
  // launch has class_slots blocks and block i looks for the i-th group of rows_lo..rows_hi rows
  int class_slots = 0;
  int tail_done = 0;  // grouped NVFP4 dispatch: the ends of the large groups have been computed by an earlier launch
  // block-scaled result (nvfp4_scaled_mm_blockscale): out = packed e2m1 [m, n/2], out_sf = e4m3 scales in the 128x4
  // layout of [roundUp(m,128), roundUp(n/16,4)], gnorm = the result's global (encode) scale on the device
  uint8_t* out_sf = nullptr;
  const float* gnorm = nullptr;
  // dense weight-streaming kernel: 0 = 16-bit result, 1 = the block-scaled result above, 2 = the fp32 product itself
  int stream_result = 0;
  // ... with stream_result 1: the kernel also zeroes the padding rows and columns of the scale buffer's last 128x4 tiles
  int stream_zero_pad = 0;
  // dense NVFP4 with a 16-bit result: elements between rows of the result; 0: n (a launch that computes some of the
  // columns sets it)
  int ldc = 0;
  __host__ __device__ int out_pitch() const { return ldc ? ldc : n; }
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

// The kernels, one file each (this translation unit includes them: they share the helpers above and the launchers below)
#include "gemm16_tile_kernels.inl"
#include "nvfp4_persistent_kernel.inl"
#include "nvfp4_streaming_kernel.inl"
#include "nvfp4_group_panel_kernel.inl"
#include "grouped16_kernel.inl"

// -------------------------------------------------------------------------------------------------
// Launchers of the tile kernels and the dispatch
// -------------------------------------------------------------------------------------------------
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
// the streaming kernel's cost estimate is in ns within 0.8 (K = 2048) .. 1.1 (K = 14336)
// (the form with 4 wavefronts: its discount in the cost holds among the streaming forms; against the tiles it made 26 of
// 91 changed picks slower, at K = 2048 and 7168, and 43 faster, so there only 4 % of it stay, for 3072 <= K < 6144:
// 1536 x 11008 x 4096 162 -> 139 us, 160 x 29568 x 4096 58 -> 46)
int64_t nvfp4_stream_ns(int64_t m, int64_t n, int64_t k, int cus) {
  int slab, rt;
  int64_t cost = nvfp4_skinny_best(m, n, k, cus, &slab, &rt);
  if (slab == 128 && rt == 4 && m > 64 && (k & 127) == 0 && ceil_div(m, 128) * (n / 64) > cus)
    cost = cost * (k >= 3072 && k < 6144 ? 96 : 100) / nvfp4_four_wavefront_percent(k);
  return cost * (k < 3072 ? 82 : k < 6144 ? 96 : k < 10240 ? 103 : 110) / 100;
}
struct DensePlan {
  enum Kernel { kStream, kTiles256, kTiles128, kOther } kernel;
  int64_t ns;  // estimated duration (INT64_MAX: no estimate)
};
DensePlan nvfp4_dense_plan(int64_t m, int64_t n, int64_t k, int cus) {
  const bool stream_ok = (k & 31) == 0 && (n & 15) == 0 && k * 64 < (1ll << 31);  // 32-bit lane offsets (a short last chunk is fine)
  // (a short last span is fine; so is, with whole spans, a last row tile with fewer rows, which counts as a whole one:
  // 384 x 28672 x 4096 as 224 tiles of 256 rows in one round instead of 336 of 128 rows in two)
  const bool persistent_shape = (n & 255) == 0 && (k & 31) == 0 && k >= 256;
  const bool ok256 = persistent_shape && ((m & 255) == 0 || ((k & 127) == 0 && m > 128));
  const bool persistent_ok = persistent_shape && ((m & 127) == 0 || ((k & 127) == 0 && m > 128));
  int64_t cost256 = INT64_MAX, cost128 = INT64_MAX, cost_tile = INT64_MAX;
  if (persistent_ok) {
    const int64_t t256 = ok256 ? ceil_div(m, 256) * (n / 256) : 0, t128 = ceil_div(m, 128) * (n / 256);
    cost256 = t256 ? 100 * ceil_div(t256, cus) : INT64_MAX;
    cost128 = 58 * ceil_div(t128, cus);
    const int64_t small = 2 * t128, full = small / (2 * cus), rest = small - full * 2 * cus;
    cost_tile = full * 68 + (rest == 0 ? 0 : rest > cus ? 68 : full ? 45 : 22 + 25 * rest / cus);
  }
  const int64_t cost_min = std::min(cost256, std::min(cost128, cost_tile));
  const int64_t rest_ns = persistent_ok ? 6000 + cost_min * 240 * ((k + 127) & ~127ll) / 1024 : INT64_MAX;
  if (stream_ok) {
    const int64_t stream_ns = nvfp4_stream_ns(m, n, k, cus);
    bool stream;
    if (m <= 128 || (m <= 256 && !(persistent_ok && k >= 2048))) {
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

// What a dense call does about an N that is no multiple of 256 (29568, 1408): 0 nothing; 1 the whole call goes to the
// weight-streaming kernel (which takes any N % 16 == 0); 2 the columns up to the last multiple of 256 go to whatever
// kernel that shape gets and the remaining columns (weight rows) to a launch of their own that writes into the same rows
// of the result.  A cut competes with the kernel the whole shape gets: the tile kernels (no estimate) lose to any cut;
// the weight-streaming kernel loses to one whose main part runs on the persistent kernel and is estimated 5 % faster.
// (ns: the estimated duration of what is returned, where there is one)
int nvfp4_n_cut(int64_t m, int64_t n, int64_t k, int cus, int64_t* ns = nullptr) {
  if (ns) *ns = INT64_MAX;
  if ((n & 255) == 0 || n <= 256 || m <= 128 || (k & 31) != 0 || k < 256) return 0;
  const DensePlan whole = nvfp4_dense_plan(m, n, k, cus);
  const DensePlan main_plan = nvfp4_dense_plan(m, n & ~255, k, cus), rest_plan = nvfp4_dense_plan(m, n & 255, k, cus);
  const bool whole_other = whole.kernel == DensePlan::kOther;
  if (main_plan.kernel == DensePlan::kOther) return 0;
  const bool have_cut_ns = rest_plan.kernel == DensePlan::kStream && main_plan.ns != INT64_MAX;
  const int64_t cut_ns = have_cut_ns ? main_plan.ns + rest_plan.ns : INT64_MAX;
  if (whole_other) {
    if (main_plan.kernel != DensePlan::kStream) {
      if (ns) *ns = cut_ns;
      return 2;
    }
    // all columns to the streaming kernel, or - a few columns past a whole number of rounds of its workgroups cost a
    // round - those in a launch of their own (512 x 4224 x 8224: 264 workgroups at once, or 256 and then 8)
    const int64_t stream_ns = (k & 31) == 0 && (n & 15) == 0 ? nvfp4_stream_ns(m, n, k, cus) : INT64_MAX;
    const bool cut = have_cut_ns && cut_ns < stream_ns - stream_ns / 20;
    if (ns) *ns = cut ? cut_ns : stream_ns;
    return cut ? 2 : 1;
  }
  if (whole.kernel == DensePlan::kStream && main_plan.kernel != DensePlan::kStream && have_cut_ns && cut_ns < whole.ns - whole.ns / 20) {
    if (ns) *ns = cut_ns;
    return 2;
  }
  return 0;
}

// Dense shapes whose M is not a multiple of 128 and that only the tile kernels would take whole: the number of rows
// (the last multiple of 128) that go to a launch of their own, if that shape gets a better kernel; else 0.  If that
// kernel is the weight-streaming one, which takes any number of rows, the answer is m: no cut, all rows to it.
int64_t nvfp4_rows_before_remainder(int64_t m, int64_t n, int64_t k, int cus) {
  if (m <= 128 || (m & 127) == 0 || (k & 15) != 0) return 0;
  // Against the kernel the whole shape gets: the tile kernels (no estimate) lose to any cut; the weight-streaming kernel
  // loses to a cut whose first part runs on the persistent kernel and is estimated 5 % faster or more (192 rows against
  // 28672 weight rows: 128 of them on 128x256 tiles).
  const DensePlan whole = nvfp4_dense_plan(m, n, k, cus);
  const bool whole_other = whole.kernel == DensePlan::kOther;
  if (!whole_other && whole.kernel != DensePlan::kStream) return 0;
  // the cut is the last multiple of 128 or of 256 (which allows 256x256 tiles), whichever is estimated faster
  int64_t best = whole_other ? INT64_MAX : whole.ns - whole.ns / 20, cut = 0;
  for (const int64_t c : {m & ~(int64_t)127, m & ~(int64_t)255}) {
    if (c < 128) continue;
    const DensePlan main = nvfp4_dense_plan(c, n, k, cus), rest = nvfp4_dense_plan(m - c, n, k, cus);
    if (main.kernel == DensePlan::kOther || rest.kernel != DensePlan::kStream || main.ns == INT64_MAX) continue;
    if (!whole_other && main.kernel == DensePlan::kStream) continue;  // (the whole shape is on that kernel already)
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
  if (s < 2) return 1;
  // N no multiple of 256: the split has to be estimated faster (25 us + 2 us per span of an item, two items to a compute
  // unit) than what the call does otherwise - all columns, or those up to the last multiple of 256, on another kernel
  // (384 x 4224 x 8224 50 us against 42 us streamed, 384 x 6176 x 14368 100 against 122 us)
  int64_t other_ns;
  if (nvfp4_n_cut(m, n, k, cus, &other_ns) != 0 && other_ns < 25000 + 2000 * ceil_div(nspans, s) * ceil_div(tiles * s, 2 * (int64_t)cus)) return 1;
  return (int)s;
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
  // grouped NVFP4: does the call count as a prefill (see kPrefillRows)?  Also with fewer rows where the large groups'
  // launches find (nearly) a round of 256x256 tiles - with 128 rows per group on average, or two rounds whatever the groups
  // (8 experts, 1536 rows, N=14336, K=4096: 320 -> 223 us; 16 experts, 3072 rows: 540 -> 394; 128 experts, 5632 rows,
  // N=7168, K=2048: 460 -> 336; at 96 rows per group and one round the other launches stay faster: 125 against 167 us)
  const int64_t tiles256 = (m_hint / 256) * (p.n / 256);
  const bool is_prefill = m_hint >= kPrefillRows || (8 * tiles256 >= 7 * (int64_t)cus && m_hint >= 128 * (int64_t)p.groups) || tiles256 >= 2 * (int64_t)cus;
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
    // grouped_mm with groups of 128 rows or more on average and tiles for half the compute units: persistent LDS-direct
    // kernel (at 128..255 rows per group the 128x128 tile kernel used to run: 8 experts, 1536 rows, N=14336, K=4096 373 ->
    // 272 us; 64 experts, 8192 rows, N=7168, K=2048 571 -> 449 us; below 128 rows per group it stays faster)
    if (!dense && m_hint >= 128 * (int64_t)p.groups && tiles(256, 256) >= cus / 2 && (p.n & 255) == 0 && (p.k & 63) == 0 &&
        p.k >= 128 && (int64_t)p.k * 2 * 256 < (1ll << 31))
      return launch_grouped16_fast<BF16_MMA, OUT_BF16>(p, cus, stream);
  }
  if constexpr (NVFP4) {
    // Grouped NVFP4: groups of up to 128 rows (MoE decode, the small experts of a prefill) stream their expert's
    // weights once through the skinny kernel; the launches below then skip them.  The group sizes live on
    // the device, so every kernel is always launched; workgroups without work return at once.
    if (!dense && p.min_rows == 0 && (p.n & 63) == 0 && (p.k & 127) != 0 && (p.k & 31) == 0 && (int64_t)p.k * 64 < (1ll << 31)) {
      // K % 128 = 32, 64 or 96: the groups of up to 128 rows on the streaming kernel's variant with a short last chunk
      // (the form that splits K over the wavefronts), larger groups on the tile kernels
      int rc = launch_nvfp4_skinny_grouped<4, 2, OUT_BF16, false>(p, 1, 32, stream);
      if (rc == NVF_OK) rc = launch_nvfp4_skinny_grouped<4, 8, OUT_BF16, false>(p, 33, 128, stream);
      if (rc != NVF_OK) return rc;
      Params rest = p;
      rest.min_rows = 129;
      return launch_sized<NVFP4, BF16_MMA, OUT_BF16>(rest, m_hint, cus, workspace, workspace_bytes, stream);
    }
    if (!dense && p.min_rows == 0 && (p.n & 63) == 0 && (p.k & 127) == 0 && (int64_t)p.k * 64 < (1ll << 31)) {
      // With a shallow K a split of K over the wavefronts leaves each only a chunk or two: they then own
      // different weight rows instead (K=2048, N=7168: 549 -> 464 us for 64 tokens x top-8; deeper K: slower),
      // 64 each where N allows (a group's rows converted once per 4 weight tiles: 512 rows over 256 experts 409 -> 388 us).
      int rc, tail_done = 0;
      if (p.k < 4096 && (p.n & 511) == 0) rc = launch_nvfp4_skinny_grouped<4, 2, OUT_BF16, true>(p, 1, 32, stream);
      else if (p.k < 4096 && (p.n & 255) == 0) rc = launch_nvfp4_skinny_grouped<2, 2, OUT_BF16, true>(p, 1, 32, stream);
      else rc = launch_nvfp4_skinny_grouped<4, 2, OUT_BF16, false>(p, 1, 32, stream);
      if (rc != NVF_OK) return rc;
      // Below the prefill size the groups of 33..128 rows are few: they stream their weights like the smaller ones,
      // found by rank among the groups of their size (a launch with few workgroups when there are few rows in all).  A
      // 128x256 tile of the persistent kernel walks all of K on one compute unit: with 64 or 256 experts, 512..5600
      // rows and K = 4096..14336 the call is 5-40 % slower that way wherever such groups exist and 0-3 % faster where
      // none does; with K < 4096 the tiles win from about 2048 rows on.
      if (m_hint <= 1024 || (p.k >= 4096 && !is_prefill)) {
        rc = launch_nvfp4_skinny_grouped<4, 8, OUT_BF16, false>(p, 33, 128, stream);
      } else if ((p.k < 4096 || !is_prefill) && (p.n & 255) == 0 && p.k >= 256) {
        // shallow K: one 128x256 tile of the persistent kernel per weight panel converts a group's rows once per 256
        // weight rows; the streaming kernel whose wavefronts own rows converts them once per wavefront.
        Params mid = p;
        mid.rows_lo = 33;
        mid.rows_hi = 128;
        if (is_prefill) mid.min_rows = 129;  // the 256x256 kernel follows: take the ends of its groups along
        tail_done = mid.min_rows != 0;
        if (is_prefill && (p.n & 511) == 0 && p.k >= 1024) {
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
    if (!dense && (p.n & 255) == 0 && (p.k & 31) == 0 && p.k >= 256 && is_prefill) {
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
int launch_nvfp4_wide_part(const Params& p, int cus, hipStream_t stream);

template <bool FP4>
int launch_nvfp4_wide(const Params& p, int cus, hipStream_t stream) {
  // A call that one launch of the weight-streaming kernel or of the persistent kernel (whose last row tile may hold
  // fewer rows) takes whole leaves that padding zero itself: no launch for it.
  const DensePlan::Kernel like16 = (p.k & 127) == 0 ? nvfp4_dense_plan(p.m, p.n, p.k, cus).kernel : DensePlan::kOther;
  const bool one_launch = like16 == DensePlan::kStream || like16 == DensePlan::kTiles256 || like16 == DensePlan::kTiles128;
  const bool cut_m = !one_launch && (p.n & 255) == 0 && (p.k & 127) == 0 && p.k >= 256 && p.m > 256 && (p.m & 127) != 0 &&
                     ceil_div(p.m / 128 * 128, 128) * (p.n / 256) >= cus / 2;
  const bool streams_whole = like16 == DensePlan::kStream;
  if (FP4 && !one_launch && ((p.m & 127) != 0 || ((p.n >> 4) & 3) != 0)) {
    // ragged: the padding rows / columns of the scale buffer's last 128x4 tiles are written as zero first
    const int64_t words = round_up(p.m, 128) * round_up(p.n >> 4, 4) / 4;
    if (!note_launch("zero_fill_kernel grid=%lld", (long long)ceil_div(words, 256))) {
      hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)ceil_div(words, 256)), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(p.out_sf), words);
      if (const int rc = check_launch("zero_fill_kernel")) return rc;
    }
  }
  if (cut_m) {
    // M not a multiple of 128 and enough rows for the persistent kernel: the rows up to the last multiple of 128 go
    // there, the rest to the tile kernels (their part of the result and of its scale tiles starts a whole number of
    // 128-row tiles further on)
    Params main = p, rest = p;
    main.m = p.m & ~127;
    rest.m = p.m - main.m;
    rest.a = p.a + (int64_t)main.m * (p.k >> 1);
    rest.sfa = p.sfa + (int64_t)main.m * round_up(p.k >> 4, 4);
    rest.out = static_cast<uint8_t*>(p.out) + (FP4 ? (int64_t)main.m * (p.n >> 1) : (int64_t)main.m * p.n * 4);
    if (FP4) rest.out_sf = p.out_sf + (int64_t)main.m * round_up(p.n >> 4, 4);
    if (const int rc = launch_nvfp4_wide_part<FP4>(main, cus, stream)) return rc;
    return launch_nvfp4_wide_part<FP4>(rest, cus, stream);
  }
  if (FP4 && streams_whole) {
    Params q = p;
    q.stream_zero_pad = 1;
    return launch_nvfp4_wide_part<FP4>(q, cus, stream);
  }
  return launch_nvfp4_wide_part<FP4>(p, cus, stream);
}

template <bool FP4>
int launch_nvfp4_wide_part(const Params& p, int cus, hipStream_t stream) {
  auto tiles = [&](int bm, int bn) { return ceil_div(p.m, bm) * ceil_div(p.n, bn); };
  // Decode-sized and other shapes that the 16-bit op streams: the same kernel, whose last stage then quantizes the
  // summed product (or stores it as it is) instead of rounding it to 16 bits (16 x 4096 x 4096: 28 -> 6 us, 128 x 4096 x
  // 14336: 85 -> 24 us on the tile kernels before).
  if ((p.k & 127) == 0 && nvfp4_dense_plan(p.m, p.n, p.k, cus).kernel == DensePlan::kStream) {
    Params q = p;
    q.stream_result = FP4 ? 1 : 2;
    return launch_nvfp4_skinny<true>(q, cus, stream);
  }
  if ((p.n & 255) == 0 && (p.k & 127) == 0 && p.k >= 256) {
    // as for the 16-bit results: persistent 256x256 or 128x256 tiles where they fill the compute units
    const DensePlan::Kernel like16 = nvfp4_dense_plan(p.m, p.n, p.k, cus).kernel;
    if (like16 == DensePlan::kTiles256) return launch_nvfp4_fast<false, false, 4, !FP4, FP4>(p, cus, stream);
    if (like16 == DensePlan::kTiles128) return launch_nvfp4_fast<false, false, 2, !FP4, FP4>(p, cus, stream);
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
  p.ldc = (int)a.ldc;
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
    // Dense with N not a multiple of 256 (29568, 1408) and enough rows for the persistent kernel: the columns up to the
    // last multiple of 256 go to whatever kernel that shape gets, the remaining columns (weight rows) to a launch of
    // their own that writes into the same rows of the result.
    const bool split_wins = op == 0 && a.workspace != nullptr && nvfp4_splits(p.m, p.n, p.k, cus) > 1 &&
                            a.workspace_bytes >= (int64_t)nvfp4_splits(p.m, p.n, p.k, cus) * p.m * p.n * 4;
    if (const int n_cut = op == 0 && !split_wins ? nvfp4_n_cut(p.m, p.n, p.k, cus) : 0) {
      if (n_cut == 1) return bf16 ? launch_nvfp4_skinny<true>(p, cus, stream) : launch_nvfp4_skinny<false>(p, cus, stream);
      {
        Gemm16Args main = a, rest = a;
        main.n = p.n & ~255;
        rest.n = p.n - main.n;
        main.ldc = rest.ldc = a.ldc ? a.ldc : a.n;
        main.workspace = rest.workspace = nullptr;  // (a split of K keeps partial results at the pitch of its own N)
        main.workspace_bytes = rest.workspace_bytes = 0;
        const int64_t sf_padded = ((int64_t)(p.k >> 4) + 3) & ~(int64_t)3;
        rest.b = static_cast<const uint8_t*>(a.b) + main.n * (p.k >> 1);
        rest.sfb = static_cast<const uint8_t*>(a.sfb) + main.n * sf_padded;
        rest.out = static_cast<uint8_t*>(a.out) + main.n * 2;
        if (const int rc = launch_gemm16(op, main, stream)) return rc;
        return launch_gemm16(op, rest, stream);
      }
    }
    const int64_t main_rows = op == 0 ? nvfp4_rows_before_remainder(p.m, p.n, p.k, cus) : 0;
    if (main_rows == p.m) return bf16 ? launch_nvfp4_skinny<true>(p, cus, stream) : launch_nvfp4_skinny<false>(p, cus, stream);
    if (main_rows) {
      Params main = p, rest = p;
      main.m = (int)main_rows;
      rest.m = p.m - main.m;
      const int64_t sf_padded = ((int64_t)(p.k >> 4) + 3) & ~(int64_t)3;
      rest.a = p.a + (int64_t)main.m * (p.k >> 1);
      rest.sfa = p.sfa + (int64_t)main.m * sf_padded;
      rest.out = static_cast<uint8_t*>(p.out) + (int64_t)main.m * p.out_pitch() * 2;
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
