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
  int m_base = 0;  // skinny kernel: first activation row this launch computes, a multiple of the slab height (32, 64 or 128)
  int ldc = 0;     // elements between rows of the result; 0: n (a launch that computes some of the columns sets it)
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

// LDS tile: rows of 128 bytes; 16-byte chunk c of row r sits at chunk position c ^ ((r >> 1) & 7): two rows fill
// the 64 banks once, so the fragment reads (16 consecutive lanes = 16 consecutive rows, one chunk) are conflict-free
__device__ __forceinline__ int lds_pos(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }

template <int BM, int BN, bool OUT_BF16>
__global__ __launch_bounds__(256) void mxfp8_gemm_kernel(const Params p) {
  constexpr int BK = 128;  // bytes == elements
  constexpr int WTM = BM / 2, WTN = BN / 2;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  extern __shared__ u32x4 lds[];  // two buffers of (A tile, B tile)
  constexpr int BUF_UNITS = (BM + BN) * 8;

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

  auto store_lds = [&](int buf) {
    u32x4* lds_a = lds + buf * BUF_UNITS;
    u32x4* lds_b = lds_a + BM * 8;
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
  };

  // K loop: the loads of step ks+1 are in flight under the MFMAs of step ks, then stored into the other
  // LDS buffer; one barrier per step
  issue_loads(0);
  store_lds(0);
  __syncthreads();
  for (int ks = 0; ks < nk; ++ks) {
    const u32x4* lds_a = lds + (ks & 1) * BUF_UNITS;
    const u32x4* lds_b = lds_a + BM * 8;
#pragma unroll
    for (int i = 0; i < TM; ++i) sca[i] = sca_next[i];
#pragma unroll
    for (int j = 0; j < TN; ++j) scb[j] = scb_next[j];
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
    if (ks + 1 < nk) store_lds((ks + 1) & 1);
    __syncthreads();
  }

  const float alpha = p.alpha[0];
  uint16_t* out = static_cast<uint16_t*>(p.out);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int mrow = m0 + wm * WTM + i * 32 + li;
    if (mrow >= p.m) continue;
    uint16_t* orow = out + (int64_t)mrow * p.out_pitch();
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


// -------------------------------------------------------------------------------------------------
// Fast path: 256x256 or 128x256 tile, M % 256 (128) == N % 256 == K % 128 == 0.
//   * Tiles travel global -> LDS with 16-byte LDS-direct loads (no staging registers) into a double
//     buffer.  They are issued from inline assembly so that the compiler does not serialise them
//     against the LDS reads of the other buffer; completion is enforced by the explicit
//     s_waitcnt vmcnt(0) in front of the one barrier per 128-deep K step.
//   * MFMA fragments are double-buffered in registers: the LDS reads of the next half step are in
//     flight under the 16 MFMAs of the current one.
//   * A load issued in the middle of step ks is consumed after the barrier in the middle of step
//     ks+1, i.e. it has 32 MFMAs (~2000 cycles) to land.
// LDS layout per operand tile: 256 rows x 128 bytes; 16-byte chunk c of row r at chunk position
// c ^ ((r >> 1) & 7): conflict-free for the fragment reads (16 consecutive lanes = 16 consecutive
// rows, one chunk) on the 64-bank LDS.
// -------------------------------------------------------------------------------------------------
__device__ __forceinline__ int lds_pos2(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }

__device__ __forceinline__ void lds_dma16(uint32_t lds_byte_addr, const uint8_t* base, uint32_t voff) {
  // lds_byte_addr and base are wave-uniform; lane L's 16 bytes land at lds_byte_addr + 16 * L
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_byte_addr), "v"(voff), "s"(base) : "memory", "m0");
}

// TM = 32-row accumulator tiles of a wavefront along M: 4 -> 256x256 workgroup tile, 2 -> 128x256 (for shapes
// whose 256x256 tiles would leave compute units idle).  The statement order for TM = 4 is the one the 8192^3
// measurements were made with.
// RAGGED_K: K is a multiple of 32 but not of 128.  The last K step of a tile then holds K % 128 elements per row: the
// lanes whose 16 bytes lie past the end of the row write zeros to their LDS unit instead of loading (the bytes there
// belong to the next row), and the scale bytes of the blocks past K - padding columns of the scale layout, whose content
// is not defined - are replaced by 2^0, so that the step adds exact zeros.
template <int TM, bool OUT_BF16, bool STREAM_OUT, bool RAGGED_K = false, bool RAGGED_M = false>
__global__ __launch_bounds__(256, 1) void mxfp8_gemm_256_kernel(const Params p) {
  constexpr int BM = 64 * TM, BN = 256;
  constexpr int A_UNITS = BM * 8;             // 16-byte units of the A tile (BM rows x 8 chunks)
  constexpr int TILE_UNITS = 2048;            // ... of the B tile
  constexpr int BUF_UNITS = A_UNITS + TILE_UNITS;
  constexpr int NM = 4 * TM;                  // MFMAs per half step
  constexpr int NF = 2 * TM + 8;              // fragment reads (ds_read_b128) per half step
  constexpr int ND = 2 * TM + 8;              // LDS-direct loads per wavefront and K step
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lg = lane >> 5;

  // ---- persistent tile walk.  Workgroup ids are dealt round-robin to the 8 XCDs, so XCD x owns the
  // contiguous tile range [x*chunk, (x+1)*chunk) and its workgroups take consecutive tiles of it in
  // each round: with the 8 (m) x 4 (n) blocked tile numbering below, the 32 tiles an XCD works on at
  // any time share 8 A panels and 4 B panels in that XCD's L2.
  // RAGGED_M: the last row tile holds fewer than BM rows (a kernel of its own: clamping the row of every activation
  // load costs the others time).  Its missing rows load the last row again and are not stored; the scale layout is
  // padded to 128 rows, so only a 256-row tile can ask for a scale tile that does not exist (it takes the last one).
  const int tiles_m = RAGGED_M ? (p.m + BM - 1) / BM : p.m / BM, tiles_n = p.n / BN;
  const int total = tiles_m * tiles_n;
  const int chunk_tiles = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int range_end = min((xcd + 1) * chunk_tiles, total);
  // (n-tiles past the last multiple of 4: blocks of 8 (m) x 1..3 (n) after all the others; 8192 x 29440 x 8192, 115
  // n-tiles: 2.33 -> 2.7 PFLOP/s against the plain m-major order)
  const bool blocked = (tiles_m & 7) == 0 && tiles_n >= 4;
  const int bulk_tiles = tiles_m * (tiles_n & ~3);
  auto tile_coords = [&](int t, int& m0, int& n0) {
    int mt, nt;
    if (blocked && t < bulk_tiles) {
      const int sb = t >> 5, w = t & 31;
      mt = (sb % (tiles_m >> 3)) * 8 + (w & 7);
      nt = (sb / (tiles_m >> 3)) * 4 + (w >> 3);
    } else if (blocked) {
      const int u = t - bulk_tiles, bs = 8 * (tiles_n & 3), sb = u / bs, w = u - sb * bs;
      mt = sb * 8 + (w & 7);
      nt = (tiles_n & ~3) + (w >> 3);
    } else {
      mt = t % tiles_m;
      nt = t / tiles_m;
    }
    m0 = mt * BM;
    n0 = nt * BN;
  };
  const int first_tile = xcd * chunk_tiles + slot;
  if (first_tile >= range_end) return;

  const int nk = (p.k + 127) >> 7;
  const int sf_tiles_k = ((p.k >> 5) + 3) >> 2;  // 512-byte scale tiles per 128-row tile
  const int k_tail = p.k & 127;                  // elements of the last step (RAGGED_K: 32, 64 or 96)

  // ---- LDS-direct load addressing.  Wave w issues 8 loads per operand per K step; load j covers LDS
  // units [(w*8+j)*64, +64) = rows (w*8+j)*8 .. +7; lane L lands at unit +L, i.e. row +(L>>3), chunk
  // position L&7, which must hold global chunk (L&7) ^ ((row>>1)&7) = (L&7) ^ ((L>>4) | ((j&1)<<2)).
  const uint32_t row_off = (uint32_t)(lane >> 3) * (uint32_t)p.k;
  const uint32_t voff_even = row_off + (uint32_t)(((lane & 7) ^ (lane >> 4)) << 4);
  const uint32_t voff_odd = row_off + (uint32_t)(((lane & 7) ^ ((lane >> 4) | 4)) << 4);
  const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds);
  const uint32_t step8 = 8u * (uint32_t)p.k;  // 8 rows
  // RAGGED_K: does this lane's chunk of an even / odd load unit exist in the last step?
  const bool tail_even = (((lane & 7) ^ (lane >> 4)) << 4) < k_tail;
  const bool tail_odd = (((lane & 7) ^ ((lane >> 4) | 4)) << 4) < k_tail;

  // ---- load stream state: the (tile, K step) the next loads are issued for
  // ---- load stream: the loads of step g+2 are issued while step g is computed, so the stream runs
  // ahead of the compute loop and crosses into the next tile two steps early.  All of its state is
  // wave-uniform and it advances without branches (the next tile's base pointers are prepared at the
  // top of the tile loop), so that the hot loop stays one basic block.
  struct TilePtrs { const uint8_t *a, *b, *sa, *sb; int valid; };
  auto tile_ptrs = [&](int t) {
    int m0, n0;
    tile_coords(t, m0, n0);
    TilePtrs r;
    // (RAGGED_M: the tile's first row; the wavefront's share is part of the lane's clamped row)
    r.a = p.a + ((int64_t)m0 + (RAGGED_M ? 0 : wave * (BM / 4))) * p.k;
    r.b = p.b + ((int64_t)n0 + wave * 64) * p.k;
    r.valid = p.m - m0;  // rows of the tile that exist (RAGGED_M: possibly fewer than BM)
    // one 16-byte scale load per lane per K step: rows {li, li+32, li+64, li+96} of the wave's 128-row
    // scale tile x 4 K-blocks
    int sa_tile = (m0 >> 7) + (TM == 4 ? wm : 0);
    if (RAGGED_M) sa_tile = min(sa_tile, ((p.m + 127) >> 7) - 1);
    r.sa = p.sfa + ((int64_t)sa_tile * sf_tiles_k) * 512;
    r.sb = p.sfb + ((int64_t)((n0 >> 7) + wn) * sf_tiles_k) * 512;
    return r;
  };
  TilePtrs lp = tile_ptrs(first_tile);  // tile the stream is in
  TilePtrs np = lp;                     // tile it enters next
  int l_ks = 0, l_count = 0;            // K step inside lp; steps issued so far
  const uint32_t sc_lane_off = (uint32_t)li * 16u;
  u32x4 sc_la, sc_lb;  // scales in flight (for step l_count - 1)
  // Unit q (0..ND-1) of a step's tile loads: 8 rows of one operand.  A and B alternate while A has rows left
  // (operand q&1, rows (q/2)*8 .. +7 of the wavefront's share), then the rest of B.  Past the end of the
  // stream the last tile is loaded again (into a buffer nobody reads any more).
  auto issue_step_unit = [&](int q) {
    const int buf = l_count & 1;
    const int op = q < 4 * TM ? (q & 1) : 1;
    const int j = q < 4 * TM ? (q >> 1) : q - 2 * TM;
    const uint32_t l = lds_base + (uint32_t)(buf * BUF_UNITS + (op ? A_UNITS + wave * 512 : wave * (BM * 2))) * 16u + j * 1024u;
    const uint8_t* gp = (op ? lp.b : lp.a) + ((int64_t)l_ks << 7);
    uint32_t voff = ((j & 1) ? voff_odd : voff_even) + (uint32_t)j * step8;
    if (RAGGED_M && op == 0) {
      const uint32_t row = min((uint32_t)(wave * (BM / 4) + j * 8) + (uint32_t)(lane >> 3), (uint32_t)(lp.valid - 1));
      voff = row * (uint32_t)p.k + (((j & 1) ? voff_odd : voff_even) - row_off);
    }
    if (RAGGED_K && l_ks == nk - 1) {
      if ((j & 1) ? tail_odd : tail_even) lds_dma16(l, gp, voff);
      else *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(lds) + (l - lds_base) + lane * 16) = u32x4{0, 0, 0, 0};
      return;
    }
    lds_dma16(l, gp, voff);
  };
  // After the 16 units: the step's scale loads, then advance the stream (selects only).
  auto issue_step_tail = [&]() {
    sc_la = *reinterpret_cast<const u32x4*>(lp.sa + (int64_t)l_ks * 512 + sc_lane_off);
    sc_lb = *reinterpret_cast<const u32x4*>(lp.sb + (int64_t)l_ks * 512 + sc_lane_off);
    ++l_count;
    const bool wrap = (l_ks + 1 == nk);
    l_ks = wrap ? 0 : l_ks + 1;
    lp.a = wrap ? np.a : lp.a;
    lp.b = wrap ? np.b : lp.b;
    lp.sa = wrap ? np.sa : lp.sa;
    lp.sb = wrap ? np.sb : lp.sb;
    if (RAGGED_M) lp.valid = wrap ? np.valid : lp.valid;
  };
  // Fragment storage: [operand: 0 = A, 1 = B][sub-tile][half].  Unit q (0..NF-1) of a half step is one
  // ds_read_b128: the 2*TM units of A (sub-tile q/2, half q&1), then the 8 units of B.
  struct Frags { u32x4 h[2][4][2]; };
  auto load_unit = [&](int buf, int sub, int q, Frags& f) {
    const int op = q >= 2 * TM ? 1 : 0;
    const int u = op ? q - 2 * TM : q;
    const int t = u >> 1, half = u & 1;
    const u32x4* base = lds + buf * BUF_UNITS + op * A_UNITS;
    const int row = (op ? wn * 128 : wm * (32 * TM)) + t * 32 + li;
    f.h[op][t][half] = base[lds_pos2(row, sub * 4 + lg + 2 * half)];
  };
  auto frag = [&](const Frags& f, int op, int t) {
    const u32x4 lo = f.h[op][t][0], hi = f.h[op][t][1];
    return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };

  f32x16 acc[TM][4];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  };
  zero_acc();

  // Keeps the 16 accumulator tiles "used" at this point of the program, so that the MFMAs producing
  // them cannot be moved past the statement that follows (they have no side effects of their own).
#define NVF_PIN_ACC()                                                                                          \
  do {                                                                                                         \
    asm volatile("" : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]),     \
                 "+a"(acc[1][1]), "+a"(acc[1][2]), "+a"(acc[1][3]));                                           \
    if constexpr (TM == 4)                                                                                     \
      asm volatile("" : "+a"(acc[TM - 2][0]), "+a"(acc[TM - 2][1]), "+a"(acc[TM - 2][2]), "+a"(acc[TM - 2][3]), \
                   "+a"(acc[TM - 1][0]), "+a"(acc[TM - 1][1]), "+a"(acc[TM - 1][2]), "+a"(acc[TM - 1][3]));     \
  } while (0)

  const float alpha = p.alpha[0];
  const int sh = lg * 8;  // lane group 1 supplies K-blocks 1 and 3 of a step

  Frags f0, f1;      // fragments of the first / second half (K 0..63 / 64..127) of a step
  u32x4 wa, wb;      // scales of the step being computed, shifted for this lane group
  u32x4 na, nb;      // scales of the next step

  // The stream runs two steps ahead of the MFMAs; with two steps per tile it is a whole tile ahead and
  // already leaves the first tile during this prologue.
  const int tiles_ahead = nk == 2 ? 2 : 1;
  np = (first_tile + slots < range_end) ? tile_ptrs(first_tile + slots) : lp;
#pragma unroll
  for (int q = 0; q < ND; ++q) issue_step_unit(q);  // step 0
  issue_step_tail();
  na = sc_la; nb = sc_lb;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // scale word of accumulator row tile i: rows {li + 32 c} of a 128-row scale tile are component c of the load;
  // with 64 rows per wavefront (TM == 2) the wavefront's half of the tile is components 2 wm, 2 wm + 1
  // (tail: the scales are those of a tile's last step, RAGGED_K only)
  auto take_scales = [&](bool tail = false) {
    if (RAGGED_K && tail) {
      const uint32_t keep = (1u << (k_tail >> 2)) - 1u, fill = 0x7f7f7f7fu & ~keep;  // k_tail / 32 bytes stay
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        na[c] = (na[c] & keep) | fill;
        nb[c] = (nb[c] & keep) | fill;
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) wa[i] = (TM == 4 ? na[i] : (wm ? na[2 + (i & 1)] : na[i & 1])) >> sh;
#pragma unroll
    for (int j = 0; j < 4; ++j) wb[j] = nb[j] >> sh;
  };
  take_scales();
#pragma unroll
  for (int q = 0; q < ND; ++q) issue_step_unit(q);  // step 1
  issue_step_tail();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
#pragma unroll
  for (int q = 0; q < NF; ++q) load_unit(0, 0, q, f0);

  int g = 0;
  for (int c_tile = first_tile; c_tile < range_end; c_tile += slots) {
    // the stream is inside this tile by now; prepare the tile it will enter two steps before the end
    np = (c_tile + tiles_ahead * slots < range_end) ? tile_ptrs(c_tile + tiles_ahead * slots) : lp;
    for (int c_ks = 0; c_ks < nk; ++c_ks, ++g) {
      const int buf = g & 1;
      // ---- first half: MFMAs on f0, interleaved one-to-one with the LDS reads that fill f1
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < NM; ++q) {
        const int i = q >> 2, j = q & 3;
#pragma unroll
        for (int u = q * NF / NM; u < (q + 1) * NF / NM; ++u) load_unit(buf, 1, u, f1);
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(frag(f0, 1, j), frag(f0, 0, i), acc[i][j], 0, 0, 0, (int)wb[j], 0, (int)wa[i]);
        __builtin_amdgcn_sched_barrier(0);
      }
      NVF_PIN_ACC();
      // Everything this wave loaded for step g+1 has landed and its reads of buf are complete; after
      // the barrier that holds for every wave, so buf^1 may be read and buf may be overwritten.
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      // The scale words of step g+1 are consumed here and nowhere earlier: their load is covered by the
      // wait above, and any wait placed before it would also stall on the tile loads just issued.
      asm volatile("" : "+v"(sc_la), "+v"(sc_lb) : : "memory");
      na = sc_la; nb = sc_lb;
      // ---- second half: MFMAs on f1, interleaved with the LDS reads of the next step's f0 (from buf^1;
      // after the last step they read stale data that is never used) and the loads of step g+2 into buf
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < NM; ++q) {
        const int i = q >> 2, j = q & 3;
#pragma unroll
        for (int u = q * NF / NM; u < (q + 1) * NF / NM; ++u) load_unit(buf ^ 1, 0, u, f0);
#pragma unroll
        for (int u = q * ND / NM; u < (q + 1) * ND / NM; ++u) issue_step_unit(u);
        if (q == NM - 1) issue_step_tail();  // scalar bookkeeping in the shadow of the MFMAs already queued
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(frag(f1, 1, j), frag(f1, 0, i), acc[i][j], 0, 0, 2, (int)wb[j], 2, (int)wa[i]);
        __builtin_amdgcn_sched_barrier(0);
      }
      NVF_PIN_ACC();
      take_scales(c_ks + 2 == nk);  // the scales of the next step
    }
    // ---- epilogue of this tile; the loads of the next tile's first two steps are already in flight.
    // acc[i][j][r] = C[m = li][n = (r/4)*8 + lg*4 + r%4] of its 32x32 sub-tile.
    // A lane holds 8-byte pieces of 32 different rows; stored like that, a tile is 8192 sixteen-byte write
    // requests per compute unit and the L2 takes longer over them than over a whole K step of MFMAs.  Every
    // 32x64 block of the wavefront's tile is therefore turned round in a private 4.5 KiB of LDS (32 rows of 128
    // bytes at a pitch of 144 bytes) and leaves in 16-byte pieces, 8 lanes to a row's 128 bytes.  One LDS address
    // each for writing and reading (the rest are immediate offsets) and one 32-bit lane offset next to a
    // wave-uniform result address; the lane number passes through an empty asm statement so that they are worked
    // out here, after the K loop.
    int m0, n0;
    tile_coords(c_tile, m0, n0);
    int elane = lane;
    asm volatile("" : "+v"(elane));
    uint8_t* stage = reinterpret_cast<uint8_t*>(lds + 2 * BUF_UNITS) + wave * 4608;
    uint8_t* wr = stage + (elane & 31) * 144 + (elane >> 5) * 8;
    const uint8_t* rd = stage + (elane >> 3) * 144 + (elane & 7) * 16;
    const int ldc = p.out_pitch();
    const uint32_t ooff = ((uint32_t)(elane >> 3) * (uint32_t)ldc + (uint32_t)(elane & 7) * 8u) * 2u;
    uint8_t* obase = reinterpret_cast<uint8_t*>(static_cast<uint16_t*>(p.out) + (int64_t)(m0 + wm * (32 * TM)) * ldc + n0 + wn * 128);
    const int rows_left = p.m - m0 - wm * (32 * TM) - (elane >> 3);  // RAGGED_M: rows from this lane's first one to the end
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            const int j = jh * 2 + j2;
            u32x2 v;
            v[0] = pack2(acc[i][j][rq * 4 + 0] * alpha, acc[i][j][rq * 4 + 1] * alpha, OUT_BF16);
            v[1] = pack2(acc[i][j][rq * 4 + 2] * alpha, acc[i][j][rq * 4 + 3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(wr + (j2 * 4 + rq) * 16) = v;
          }
        }
        asm volatile("" ::: "memory");  // the reads below see the writes above: one wavefront's LDS accesses stay in order
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(rd + t * 1152);
          u32x4* dst = reinterpret_cast<u32x4*>(obase + ((int64_t)(i * 32 + 8 * t) * ldc + jh * 64) * 2 + ooff);
          if (RAGGED_M && i * 32 + 8 * t >= rows_left) continue;
          if constexpr (STREAM_OUT) __builtin_nontemporal_store(v, dst);
          else *dst = v;
        }
        asm volatile("" ::: "memory");
      }
    }
    zero_acc();
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-direct load may outlive the workgroup
#undef NVF_PIN_ACC
}

template <int TM, bool OUT_BF16, bool STREAM_OUT, bool RAGGED_K, bool RAGGED_M = false>
int launch_fast_cfg(const Params& p, hipStream_t stream) {
  auto kern = mxfp8_gemm_256_kernel<TM, OUT_BF16, STREAM_OUT, RAGGED_K, RAGGED_M>;
  constexpr int lds_bytes = 2 * (64 * TM + 256) * 128 + 4 * 4608;  // 128 KiB / 96 KiB of tiles + the epilogue's 18 KiB
  const int64_t tiles = ceil_div(p.m, 64 * TM) * (p.n / 256);
  if (!RAGGED_M && p.m % (64 * TM) != 0) return fail(NVF_ERR_LAUNCH, "mxfp8_gemm_256_kernel: M = %d is no multiple of %d", p.m, 64 * TM);
  const int cus = cu_count() & ~7;  // workgroup ids are dealt round-robin to the 8 XCDs
  const unsigned grid = (unsigned)(tiles >= cus ? cus : ((tiles + 7) / 8) * 8);
  if (note_launch("mxfp8_gemm_256_kernel<TM=%d,stream_out=%d%s%s> grid=%u", TM, (int)STREAM_OUT, RAGGED_K ? ",ragged_k" : "",
                  RAGGED_M ? ",ragged_m" : "", grid))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device (and per instantiation of this launcher)
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, stream, p);
  return check_launch("mxfp8_gemm_256_kernel");
}

template <int TM, bool OUT_BF16>
int launch_fast(const Params& p, hipStream_t stream) {
  // Operands and result together beyond what the 256 MB last-level cache holds: the result would push the
  // operand panels out of it (and out of the L2s) on its way to memory, so it leaves with non-temporal stores
  // (8192^3: +5 %, 16384 x 16384 x 2048: +17 %; smaller problems lose 1-5 % that way).
  const bool stream_out = ((int64_t)p.m + p.n) * p.k + 2 * (int64_t)p.m * p.n > (int64_t)224 << 20;
  if (p.m % (64 * TM) != 0 && (p.k & 127) != 0)
    return stream_out ? launch_fast_cfg<TM, OUT_BF16, true, true, true>(p, stream) : launch_fast_cfg<TM, OUT_BF16, false, true, true>(p, stream);
  if (p.m % (64 * TM) != 0) return stream_out ? launch_fast_cfg<TM, OUT_BF16, true, false, true>(p, stream) : launch_fast_cfg<TM, OUT_BF16, false, false, true>(p, stream);
  if ((p.k & 127) != 0) return stream_out ? launch_fast_cfg<TM, OUT_BF16, true, true>(p, stream) : launch_fast_cfg<TM, OUT_BF16, false, true>(p, stream);
  return stream_out ? launch_fast_cfg<TM, OUT_BF16, true, false>(p, stream) : launch_fast_cfg<TM, OUT_BF16, false, false>(p, stream);
}

// -------------------------------------------------------------------------------------------------
// Skinny path: slabs of up to 128 activation rows (decode-sized activations; more rows as several slabs, the
// whole ones side by side in one launch, blockIdx.y = slab), K % 32 == 0, N % (16*RT) == 0.  A slab streams
// the weight matrix exactly once, so the op is bound by HBM (by the last-level cache for the slabs after the
// first):
//   * A workgroup owns 16*RT weight rows for the whole of K and all M activation rows; its W = 8 wavefronts
//     (4 in the form of which two workgroups share a compute unit) split K in interleaved 128-element chunks and their partial sums are added in a fixed order through
//     LDS (no atomics, no workspace, deterministic).
//   * v_mfma_scale_f32_16x16x128_f8f6f4, measured operand layout: lane (i, g) = i + 16 g supplies row i,
//     bytes 0..15 = K [16g, 16g+16) and bytes 16..31 = K [64+16g, 64+16g+16); the scale byte of lane
//     (i, j) applies to row i, K-block j.  Weight rows are the first operand, so a lane ends up with 4
//     consecutive N-elements of one output row.
//   * A load in that lane order would touch 64 unrelated 16-byte pieces per instruction, which the address
//     unit handles one by one.  Every wavefront therefore fetches its tiles with LDS-direct loads in memory
//     order (8 neighbouring lanes = the 128 contiguous bytes of a row's chunk; the scales as the 256
//     contiguous bytes that hold a 16-row tile's scale words) into a private ring of DEPTH slots in LDS and
//     reads them back in MFMA lane order; no barrier in the K loop, a wavefront reads only what it loaded.
//   LDS per slot: NT tiles of 16 rows x 128 B (piece p of row r at position p ^ ((r >> 1) & 7): conflict-free
//   reads), then 256 B of scale words per tile.
// -------------------------------------------------------------------------------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));

// (W = 4, 4 x 4 tiles: 168 VGPRs + 64 AGPRs as compiled, so two workgroups fit a compute unit.  Asking for 2 wavefronts per
// SIMD in the launch bounds moves the accumulators into the VGPRs: 96 x 16384 x 4096 19.1 -> 21.8 us, 512 x 4096 x 7168 28.2 ->
// 26.1, others equal; not done.)
template <int RT, int TT, bool OUT_BF16, int DEPTH, bool RAGGED_K = false, int W = 8>
__global__ __launch_bounds__(W * 64) void mxfp8_skinny_kernel(const Params p) {
  constexpr int NT = RT + TT;
  // activation rows r and r + 32 share their 16-byte scale group, so 32 groups serve any number of tiles
  constexpr int A_SC_BYTES = (TT < 2 ? TT : 2) * 256;
  constexpr int SLOT_BYTES = NT * 2048 + RT * 256 + A_SC_BYTES;
  constexpr int NDMA = 2 * NT + 2;  // loads per chunk and wavefront
  static_assert(DEPTH >= 1 && DEPTH <= 3 && W * DEPTH * SLOT_BYTES <= 160 * 1024 && DEPTH * NDMA <= 63 && RT <= 4 && TT <= 8,
                "ring does not fit");
  extern __shared__ u32x4 lds[];  // ring during the K loop, then [W][tiles][64 lanes] partial sums
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * RT);
  // activation rows of this workgroup: [m_base, m_base + m_loc); blockIdx.y counts slabs of 16*TT rows
  const int m_base = p.m_base + (int)blockIdx.y * (16 * TT);
  const int m_loc = min(p.m - m_base, 16 * TT);
  const int tt_count = (m_loc + 15) >> 4;
  // K % 128 = 32, 64 or 96: the last chunk is short.  Lanes whose 16 bytes lie past the end of the row write zeros to
  // their LDS unit instead of loading, and the scale bytes of the blocks past K (padding columns of the scale layout,
  // content not defined) are replaced by 2^0, so that the chunk adds exact zeros for them.
  const int chunks = (p.k + 127) >> 7;
  const int k_tail = p.k & 127;
  const int tail_chunk = RAGGED_K ? chunks - 1 : -1;  // (a kernel of its own: K % 128 != 0)
  const int sf_padded = ((p.k >> 5) + 3) & ~3;  // scale columns with the layout's padding

  // ---- load side (memory order).  Payload: tile t, load j (rows 8j..8j+7): lane L = row 8j + L/8, piece
  // (L & 7) ^ ((4j + L/16) & 7).  Scales: lane L = tile L/16, row L%16: the 16 bytes that hold the scale
  // words of rows {row, row+32, row+64, row+96} (mod 128) for the chunk's 4 K-blocks.
  const uint8_t* b_base = p.b + (int64_t)n0 * p.k;
  const uint8_t* bsf_base = p.sfb + (int64_t)(n0 >> 7) * ((int64_t)sf_padded << 7);
  uint32_t b_off[RT][2], a_off[TT][2];
  bool in_tail[2];  // does the lane's piece of load j exist in a short last chunk?
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = 8 * j + (lane >> 3);
    const uint32_t piece = (uint32_t)((lane & 7) ^ ((4 * j + (lane >> 4)) & 7)) * 16u;
    in_tail[j] = (int)piece < k_tail;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) b_off[rt][j] = (uint32_t)(rt * 16 + row) * (uint32_t)p.k + piece;
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) a_off[tt][j] = (uint32_t)min(tt * 16 + row, m_loc - 1) * (uint32_t)p.k + piece;
  }
  const int st = lane >> 4;  // tile whose scales this lane fetches
  const uint32_t bsf_off = (uint32_t)((((n0 & 127) + min(st, RT - 1) * 16 + r) & 31) * 16);
  const uint8_t* a_base = p.a + (int64_t)m_base * p.k;
  const uint8_t* asf_base = p.sfa + (int64_t)(m_base >> 7) * ((int64_t)sf_padded << 7);
  const uint32_t asf_off = (uint32_t)((lane & 31) * 16);  // scale group of rows {lane, lane + 32, ...} of the 128-row tile
  const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds);
  const uint32_t ring_base = lds_base + (uint32_t)wave * (DEPTH * SLOT_BYTES);
  auto issue_chunk = [&](int c_in, int slot) {  // c_in is wave-uniform
    if (c_in >= chunks) return;
    const uint32_t c = (uint32_t)c_in;
    const uint32_t sb = ring_base + (uint32_t)slot * SLOT_BYTES;
    if (RAGGED_K && c_in == tail_chunk) {
      char* const zp = reinterpret_cast<char*>(lds) + (sb - lds_base) + lane * 16;
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (in_tail[j]) lds_dma16(sb + t * 2048 + j * 1024, t < RT ? b_base : a_base, (t < RT ? b_off[t][j] : a_off[t - RT][j]) + c * 128u);
          else *reinterpret_cast<u32x4*>(zp + t * 2048 + j * 1024) = u32x4{0, 0, 0, 0};
        }
    } else {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int j = 0; j < 2; ++j) lds_dma16(sb + rt * 2048 + j * 1024, b_base, b_off[rt][j] + c * 128u);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int j = 0; j < 2; ++j) lds_dma16(sb + (RT + tt) * 2048 + j * 1024, a_base, a_off[tt][j] + c * 128u);
    }
    // one load each for the scales of all weight tiles / all activation tiles (lanes of tiles that do not
    // exist stay off: a disabled lane writes nothing)
    if (lane < 16 * RT) lds_dma16(sb + NT * 2048, bsf_base, bsf_off + c * 512u);
    if (lane < A_SC_BYTES / 16) lds_dma16(sb + NT * 2048 + RT * 256, asf_base, asf_off + c * 512u);
  };

  // ---- read side (MFMA order)
  const int rd_lo = r * 128 + ((g ^ ((r >> 1) & 7)) * 16);
  const int rd_hi = r * 128 + (((g + 4) ^ ((r >> 1) & 7)) * 16);
  int rd_bsc[RT], rd_asc[TT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) rd_bsc[rt] = NT * 2048 + rt * 256 + r * 16 + ((((n0 & 127) + rt * 16) >> 5) & 3) * 4;
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
    rd_asc[tt] = NT * 2048 + RT * 256 + ((tt & 1) * 16 + r) * 16 + ((((m_base & 127) + tt * 16) >> 5) & 3) * 4;
  const int sc_shift = g * 8;

  f32x4 acc[RT][TT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) acc[rt][tt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue_chunk(wave + d * W, d);
  int slot = 0;
  for (int c = wave; c < chunks; c += W) {
    // the oldest chunk in flight has landed when only the loads of the younger ones are pending
    const int younger = min(DEPTH - 1, (chunks - 1 - c) / W);
    if (younger >= 2)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH >= 3 ? 2 * NDMA : 0) : "memory");
    else if (younger == 1)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH >= 2 ? NDMA : 0) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const char* sp = reinterpret_cast<const char*>(lds) + (wave * DEPTH + slot) * SLOT_BYTES;
    u32x4 lo[NT], hi[NT];
    uint32_t sc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      lo[t] = *reinterpret_cast<const u32x4*>(sp + t * 2048 + rd_lo);
      hi[t] = *reinterpret_cast<const u32x4*>(sp + t * 2048 + rd_hi);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) sc[RT + tt] = *reinterpret_cast<const uint32_t*>(sp + rd_asc[tt]) >> sc_shift;
    if (RAGGED_K && c == tail_chunk && g * 32 >= k_tail) {  // this lane's K-block lies past K
#pragma unroll
      for (int t = 0; t < NT; ++t) sc[t] = 0x7f;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: the slot may be refilled
    issue_chunk(c + DEPTH * W, slot);
    slot = (slot + 1 == DEPTH) ? 0 : slot + 1;
    auto frag = [&](int t) {
      return i32x8{(int)lo[t][0], (int)lo[t][1], (int)lo[t][2], (int)lo[t][3], (int)hi[t][0], (int)hi[t][1], (int)hi[t][2], (int)hi[t][3]};
    };
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
      if (tt < tt_count) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][tt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(frag(rt), frag(RT + tt), acc[rt][tt], 0, 0, 0, (int)sc[rt], 0,
                                                                         (int)sc[RT + tt]);
      }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no LDS-direct load may be pending when the ring is reused
  __syncthreads();

  // ---- sum the wavefronts' partial tiles in wave order and store (RT * TT <= 16 tiles of 1 KiB per wave)
  f32x4* red = reinterpret_cast<f32x4*>(lds);
  const float alpha = p.alpha[0];
  uint16_t* out = static_cast<uint16_t*>(p.out);
  const int tiles = RT * tt_count;  // tile index: rt * tt_count + tt
  const int units = tiles * 64;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
      if (tt < tt_count) red[(wave * tiles + rt * tt_count + tt) * 64 + lane] = acc[rt][tt];
  __syncthreads();
  for (int u = tid; u < units; u += W * 64) {
    const int l = u & 63, tile = u >> 6;
    const int rt = tile / tt_count, tt = tile - rt * tt_count;
    f32x4 s = red[u];
#pragma unroll
    for (int w = 1; w < W; ++w) s += red[w * units + u];
    // element e of lane l: weight row 4*(l/16) + e (output column), activation row l%16 (output row)
    const int tok = tt * 16 + (l & 15);
    if (tok < m_loc) {
      u32x2 v;
      v[0] = pack2(s[0] * alpha, s[1] * alpha, OUT_BF16);
      v[1] = pack2(s[2] * alpha, s[3] * alpha, OUT_BF16);
      *reinterpret_cast<u32x2*>(out + (int64_t)(m_base + tok) * p.out_pitch() + n0 + rt * 16 + 4 * (l >> 4)) = v;
    }
  }
}

template <int RT, int TT, bool OUT_BF16, int W = 8>
int launch_skinny_cfg(const Params& p, hipStream_t stream, int slabs = 1) {
  constexpr int SLOT = (RT + TT) * 2048 + RT * 256 + (TT < 2 ? TT : 2) * 256;
  constexpr int DEPTH = W != 8 ? 1 : 8 * 3 * SLOT <= 160 * 1024 ? 3 : (8 * 2 * SLOT <= 160 * 1024 ? 2 : 1);
  // (4 wavefronts: K % 128 == 0 only, and a ring of one slot, so that two workgroups share a compute unit's LDS)
  if (W != 8 && (p.k & 127) != 0) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "mxfp8_skinny_kernel: 4 wavefronts need K % 128 == 0");
  auto kern = W == 8 && (p.k & 127) != 0 ? mxfp8_skinny_kernel<RT, TT, OUT_BF16, DEPTH, W == 8, W> : mxfp8_skinny_kernel<RT, TT, OUT_BF16, DEPTH, false, W>;
  constexpr int ring = W * DEPTH * SLOT, red = W * RT * TT * 1024;
  constexpr int lds_bytes = ring > red ? ring : red;
  static_assert(lds_bytes <= 160 * 1024, "LDS");
  if (note_launch("mxfp8_skinny_kernel<RT=%d,TT=%d%s> grid=%ux%d m_base=%d", RT, TT, W == 4 ? ",W=4" : "", (unsigned)(p.n / (16 * RT)), slabs, p.m_base)) return NVF_OK;
  static std::atomic<uint64_t> configured[2] = {{0}, {0}};  // per kernel, one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured[(p.k & 127) != 0])) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.n / (16 * RT)), (unsigned)slabs), dim3(W * 64), lds_bytes, stream, p);
  return check_launch("mxfp8_skinny_kernel");
}

template <int TT, bool OUT_BF16>
int launch_skinny_rt(const Params& p, int rt, hipStream_t stream, int slabs) {
  if constexpr (TT == 8) return launch_skinny_cfg<1, 8, OUT_BF16>(p, stream, slabs);
  else
    return rt == 4 ? launch_skinny_cfg<4, TT, OUT_BF16>(p, stream, slabs)
         : rt == 2 ? launch_skinny_cfg<2, TT, OUT_BF16>(p, stream, slabs)
                   : launch_skinny_cfg<1, TT, OUT_BF16>(p, stream, slabs);
}

// Estimated duration of the skinny kernel for (slab height, weight tiles per workgroup), in units of about 1 ns: the
// workgroups (one per slab and 16*rt weight rows; one per compute unit at a time, the ring fills its LDS) run in
// rounds over the compute units; a wavefront visits ceil(chunks / 8) chunks, each costing the LDS-direct loads of
// its rt + tt tiles and rt * tt MFMAs, then comes the reduction of rt * tt partial tiles.  A last round that is only
// partly filled costs 70 % of a full one plus its share of the rest; the weight stream bounds the whole from below.
// Constants fitted to a sweep of the seven forms over 140 shapes (M 48..256, N 1024..14336, K 2048..14336): the form
// picked is within 7 % of the best everywhere.
// (duration: the estimate is compared with another kernel's; then a round of workgroups streams the weight rows it
// covers, not all of them - with 28672 weight rows a slab takes two rounds, which made the other floor twice the
// measured time; the choice of the form keeps the floor it was fitted with)
// (w = 4: the form with 4 wavefronts and a ring of one slot, 64-row slabs x 4 weight tiles.  Two of its workgroups share
// a compute unit, so up to twice as many as there are compute units run in one round where the form with 8 wavefronts
// takes two; a wavefront then visits twice the chunks, each 27 % dearer.  Only for that case, and K % 128 == 0.
// Measured, 8 -> 4 wavefronts: 128 x 14336 x 4096 (448 workgroups) 25.4 -> 19.9 us, 64 x 28672 x 4096 26.0 -> 24.1,
// 256 x 7168 x 2048 12.7 -> 10.5, 192 x 7168 x 2048 (336) 11.9 -> 9.8; but with one round either way 256 x 4096 x 4096
// 10.6 -> 12.8 us, 256 x 4096 x 14336 24.9 -> 30.4.  Over the 234 of 2448 shapes (M 33..2048, N 1024..32896, K 512..14336)
// whose launch the form changes, the time falls by 16 % in the geometric mean, by 28-32 % at K <= 1024, where it also
// takes over from the persistent kernel: 160 x 8192 x 1024 10.8 -> 6.5 us.)
int64_t mxfp8_skinny_cost(int64_t m, int64_t n, int64_t k, int slab, int rt, int64_t cus, bool duration = false, int w = 8) {
  if ((slab == 128 && rt != 1) || n % (16 * rt) != 0) return INT64_MAX;
  if (w == 4) {
    const int64_t wgs4 = ceil_div(m, 64) * (n / 64);
    if (slab != 64 || rt != 4 || (n & 63) != 0 || (k & 127) != 0 || m <= 32 || wgs4 <= cus || wgs4 > 2 * cus) return INT64_MAX;
    // (a deep K makes the second, partly filled round of the other form cheap against its first: 96 x 12288 x 14336,
    // 384 workgroups, 51 -> 55 us; and many slabs of few columns gain nothing from K = 7168 on: 1024 x 2048 x 7168 28 -> 30 us)
    if ((k > 8192 && 4 * wgs4 < 7 * cus) || (k > 4096 && m > 8 * 64)) return INT64_MAX;
    const int64_t per_chunk4 = ((4 + 4) * 145 + 4 * 4 * 10 + 100) * 127 / 100;
    return std::max(2 * ceil_div(k >> 7, 8) * per_chunk4 + 4 * 4 * 193 + 2493, n * k / 5400);
  }
  const int64_t slabs = m <= slab ? 1 : ceil_div(m, slab);
  const int tt = m <= slab ? (m <= 16 ? 1 : m <= 32 ? 2 : m <= 64 ? 4 : 8) : slab / 16;
  if (tt == 8 && rt != 1) return INT64_MAX;
  const int64_t wgs = slabs * (n / (16 * rt));
  const int64_t chunks = ceil_div((k + 127) >> 7, 8);
  const int64_t per_chunk = (rt + tt) * 145 + rt * tt * 10 + 100;
  const int64_t wg_time = chunks * per_chunk + rt * tt * 193 + 2493;
  const int64_t full = wgs / cus, rest = wgs - full * cus;
  // every round of workgroups streams the weights again, out of the last-level cache at best: 5.6 TB/s
  // (256 x 14336 x 14336 as 4 slabs in 3.5 rounds: 123 us for 4 x 205 MB)
  const int64_t stream = ceil_div(wgs, cus) * (duration ? std::min<int64_t>(n, cus * 16 * rt) : n) * k / 5400;
  return std::max((full * 100 + (rest ? 70 + 30 * rest / cus : 0)) * wg_time / 100, stream);
}

// best form of the skinny kernel for more than 32 rows: estimated duration, slab height and weight tiles per workgroup
int64_t mxfp8_skinny_best(int64_t m, int64_t n, int64_t k, int64_t cus, int* slab_out, int* rt_out, int* w_out) {
  int slab = 128, rt = 1, w = 8;
  int64_t best = INT64_MAX;
  for (const int s : {32, 64, 128})  // (equal estimates: the lower slab, measured 2-9 % faster)
    for (const int r : {1, 2, 4}) {
      const int64_t c = mxfp8_skinny_cost(m, n, k, s, r, cus);
      if (c < best) best = c, slab = s, rt = r;
    }
  if (const int64_t c = mxfp8_skinny_cost(m, n, k, 64, 4, cus, false, 4); c < best) best = c, slab = 64, rt = 4, w = 4;
  if (slab_out) *slab_out = slab;
  if (rt_out) *rt_out = rt;
  if (w_out) *w_out = w;
  return best;
}
// estimated duration of the form that mxfp8_skinny_best picks, in ns
int64_t mxfp8_skinny_ns(int64_t m, int64_t n, int64_t k, int64_t cus) {
  int slab, rt, w;
  if (mxfp8_skinny_best(m, n, k, cus, &slab, &rt, &w) == INT64_MAX) return INT64_MAX;
  return mxfp8_skinny_cost(m, n, k, slab, rt, cus, true, w) * 963 / 1000;
}

template <bool OUT_BF16>
int launch_skinny(const Params& p, hipStream_t stream) {
  // Up to 32 rows: one slab of 1 or 2 activation tiles (16 x 6144 x 4096: 8.0 us with 1 weight tile per workgroup in 1.5
  // rounds, 6.2 us with 2); more rows: slabs of 128, 64 or 32 rows side by side in one launch (blockIdx.y = slab; the last one may be ragged;
  // the slabs after the first find the weights in the last-level cache) with 1, 2 or 4 weight tiles per workgroup
  // (1 with 128-row slabs, whose 8 activation tiles fill the ring), whichever the estimate above prefers
  // (128 x 4096 x 4096: 10.5 us as one slab of 128 rows, 7.6 us as 4 slabs of 32 rows x 4 weight tiles;
  // 256 x 4096 x 14336: 49.9 -> 26.1 us; 128 x 8192 x 7168: 28.0 -> 16.6 us).
  int slab, rt, w;
  mxfp8_skinny_best(p.m, p.n, p.k, cu_count(), &slab, &rt, &w);
  // Decode sizes against weight rows a multiple of 8 KiB apart: 2 weight tiles per workgroup stream them slower than
  // 1 or 4 do (measured, 8 rows: 8192 x 8192 15.8 us with 2, 14.3 with 1, 12.6 with 4; 7168 x 8192 13.6 / 12.5 / 11.4;
  // other K: as estimated), so 4 where that still leaves 80 workgroups
  if (p.m <= 32 && rt == 2 && (p.k & 8191) == 0 && (p.n & 63) == 0 && p.n / 64 >= 80) rt = 4;
  const int slabs = p.m <= slab ? 1 : (int)ceil_div(p.m, slab);
  const int rows = p.m <= slab ? p.m : slab;
  if (w == 4) return launch_skinny_cfg<4, 4, OUT_BF16, 4>(p, stream, slabs);
  return rows <= 16 ? launch_skinny_rt<1, OUT_BF16>(p, rt, stream, slabs)
       : rows <= 32 ? launch_skinny_rt<2, OUT_BF16>(p, rt, stream, slabs)
       : rows <= 64 ? launch_skinny_rt<4, OUT_BF16>(p, rt, stream, slabs)
                    : launch_skinny_rt<8, OUT_BF16>(p, rt, stream, slabs);
}

template <int BM, int BN, bool OUT_BF16>
int launch_cfg(const Params& p, hipStream_t stream) {
  auto kern = mxfp8_gemm_kernel<BM, BN, OUT_BF16>;
  constexpr int lds_bytes = 2 * (BM + BN) * 128;
  const int64_t tiles = ceil_div(p.m, BM) * ceil_div(p.n, BN);
  if (note_launch("mxfp8_gemm_kernel<%d,%d> grid=%lld", BM, BN, (long long)tiles)) return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(256), lds_bytes, stream, p);
  return check_launch("mxfp8_gemm_kernel");
}

// Which kernel a shape gets.  Persistent LDS-direct kernel with 256x256 or 128x256 tiles: a 128-row tile costs about
// 0.61 of a 256-row tile (half the flops at 82 % of the rate, measured), and the time goes with the rounds of tiles
// over the compute units; below 48 tiles the tile kernels do as well.
enum class Plan { kStream, kTiles256, kTiles128, kOther };
// (ns: the estimated duration, where there is an estimate)
Plan mxfp8_plan(int64_t m, int64_t n, int64_t k, int64_t cus, int64_t* ns = nullptr) {
  if (ns) *ns = INT64_MAX;
  const bool skinny_ok = (k & 31) == 0 && (n & 15) == 0 && k * 64 < (1ll << 31);  // 32-bit lane offsets (a short last chunk is fine)
  // (the persistent kernel takes any K % 32 == 0: its last step may be short)
  // (a last row tile with fewer rows: the variant that clamps the rows of its activation loads; the tile counts as a
  // whole one.  640 x 14336 x 4096: 280 tiles of 128 rows in 2 rounds 60 us, 168 of 256 rows 43 us)
  const bool fast_shape = (k & 31) == 0 && k >= 256 && (n & 255) == 0 && k * 256 < (1ll << 31);
  const bool ok256 = fast_shape && ((m & 255) == 0 || m > 128);
  const bool ok128 = fast_shape && ((m & 127) == 0 || m > 64);
  const int64_t t256 = ok256 ? ceil_div(m, 256) * (n / 256) : 0, t128 = ok128 ? ceil_div(m, 128) * (n / 256) : 0;
  const int64_t cost256 = t256 >= 128 ? 100 * ceil_div(t256, cus) : INT64_MAX;
  const int64_t cost128 = t128 >= 48 ? 61 * ceil_div(t128, cus) : INT64_MAX;
  const bool fast = cost256 != INT64_MAX || cost128 != INT64_MAX;
  const int64_t fast_ns = fast ? 5000 + std::min(cost256, cost128) * 113 * ((k + 127) & ~127ll) / 1024 : INT64_MAX;
  if (skinny_ok) {
    const int64_t skinny_ns = mxfp8_skinny_ns(m, n, k, cus);
    if (ns) *ns = skinny_ns;
    if (m <= 32) return Plan::kStream;
    if (fast) {
      // Skinny or persistent kernel by estimated duration: a round of 128x256 tiles takes 6.9 us per 1024 of K plus
      // about 5 us (so cost 100 = 11.3 us per 1024 of K), the skinny kernel what its estimate says (its unit is
      // 0.96 ns).  Measured: 256 x 14336 x 4096 31 (persistent) against 47 us, 512 x 4096 x 7168 51 against 30 us
      // (skinny), 1024 x 2048 x 14336 97 against 48 us, 1024 x 4096 x 4096 31 against 34 us.
      // (129..256 rows are three or four slabs of 64, which the estimate puts 15-22 % low against a wide N: 160 and 192 x
      // 14336 x 4096 run 37 and 40 us streamed, estimated 31, and 31 us on 112 tiles of 128 rows; 256 x 11008 x 4096
      // 38 against 31 us)
      const int64_t margin = m > 128 && m <= 256 ? skinny_ns / 5 : 0;
      if (skinny_ns + margin <= fast_ns) return Plan::kStream;
    } else {
      // No persistent kernel for the shape (ragged M or N, or too few tiles): up to 256 rows, i.e. four passes over
      // the weights, the skinny kernel beats the tile kernels (128 x 4096 x 14336: 20 instead of 117 us); with more
      // rows, a deep K and a small N it fills the chip where they cannot, while its 128-row x 16-column workgroups
      // cover the compute units at most 3 times (measured, K >= 2048).
      const int64_t skinny_rounds = ceil_div(ceil_div(m, 128) * (n / 16), cus);
      if (m <= 256 || (skinny_rounds <= 3 && k >= 2048)) return Plan::kStream;
    }
  }
  if (ns) *ns = fast_ns;
  if (fast) return cost256 <= cost128 ? Plan::kTiles256 : Plan::kTiles128;
  return Plan::kOther;
}

template <bool OUT_BF16>
int launch_sized(const Params& p, hipStream_t stream) {
  auto tiles = [&](int bm, int bn) { return ceil_div(p.m, bm) * ceil_div(p.n, bn); };
  const int64_t cus = cu_count();
  int64_t whole_ns;
  const Plan whole = mxfp8_plan(p.m, p.n, p.k, cus, &whole_ns);
  // A cut along N or M competes with the kernel the whole shape gets: the tile kernels (no estimate) lose to any cut
  // that works; the weight-streaming kernel loses to a cut whose main part runs on the persistent kernel and is
  // estimated 5 % faster or more (384 x 29568 x 8192: 291 us on tiles, 256 x 29568 x 8192: 169 us streamed).
  const bool whole_other = whole == Plan::kOther;
  const int64_t bar = whole_other ? INT64_MAX : whole == Plan::kStream ? whole_ns - whole_ns / 20 : 0;
  auto is_tiles = [](Plan q) { return q == Plan::kTiles256 || q == Plan::kTiles128; };
  // N not a multiple of 256 (29568, 1408): the columns up to the last multiple of 256 go to whatever kernel that shape
  // gets, the remaining columns (weight rows) to a launch of their own that writes into the same rows of the result
  // (8192 x 29568 x 8192: 4.1 -> 1.3 ms).
  if ((p.n & 255) != 0 && p.n > 256 && (p.n & 15) == 0 && p.m > 64 && (p.k & 31) == 0 && p.k >= 256) {
    int64_t main_ns, rest_ns;
    const Plan main_plan = mxfp8_plan(p.m, p.n & ~255, p.k, cus, &main_ns), rest_plan = mxfp8_plan(p.m, p.n & 255, p.k, cus, &rest_ns);
    if (whole_other && main_plan == Plan::kStream) return launch_skinny<OUT_BF16>(p, stream);  // (takes any N % 16 == 0)
    if (main_plan != Plan::kOther && (whole_other || (is_tiles(main_plan) && rest_plan == Plan::kStream && main_ns != INT64_MAX &&
                                                       rest_ns != INT64_MAX && main_ns + rest_ns < bar))) {
      Params main = p, rest = p;
      main.n = p.n & ~255;
      rest.n = p.n - main.n;
      main.ldc = rest.ldc = p.out_pitch();
      const int64_t sf_padded = ((int64_t)(p.k >> 5) + 3) & ~(int64_t)3;
      rest.b = p.b + (int64_t)main.n * p.k;
      rest.sfb = p.sfb + (int64_t)main.n * sf_padded;
      rest.out = static_cast<uint8_t*>(p.out) + (int64_t)main.n * 2;
      if (const int rc = launch_sized<OUT_BF16>(main, stream)) return rc;
      return launch_sized<OUT_BF16>(rest, stream);
    }
  }
  // M not a multiple of 128 (a prefill of any token count): the rows up to the last multiple of 128 go to whatever kernel
  // that shape gets, the remaining rows (at most 127, a whole number of 128-row scale tiles further on) to the skinny
  // kernel in a launch of their own (4000 x 4096 x 4096: 197 -> 77 us; 8100 x 8192 x 8192: 1475 -> 390 us).
  // The cut is the last multiple of 128 or of 256 (which allows 256x256 tiles), whichever is estimated faster
  // (8100 x 8192 x 8192: 546 us cut at 8064, 128x256 tiles; 390 us cut at 7936).
  if (p.m > 128 && (p.m & 127) != 0 && (p.k & 31) == 0 && (whole_other || whole == Plan::kStream)) {
    int64_t best = bar;
    int cut = 0;
    for (const int c : {p.m & ~127, p.m & ~255}) {
      int64_t ns_main, ns_rest;
      if (c < 128) continue;
      const Plan main_plan = mxfp8_plan(c, p.n, p.k, cus, &ns_main);
      if (main_plan == Plan::kOther || mxfp8_plan(p.m - c, p.n, p.k, cus, &ns_rest) != Plan::kStream) continue;
      if (!whole_other && main_plan == Plan::kStream) continue;  // (the whole shape is on that kernel already)
      if (ns_main == INT64_MAX || ns_rest == INT64_MAX) continue;
      if (ns_main + ns_rest < best) best = ns_main + ns_rest, cut = main_plan == Plan::kStream ? p.m : c;
    }
    if (cut == p.m) return launch_skinny<OUT_BF16>(p, stream);  // (the skinny kernel takes any number of rows)
    if (cut) {
      Params main = p, rest = p;
      main.m = cut;
      rest.m = p.m - cut;
      const int64_t sf_padded = ((int64_t)(p.k >> 5) + 3) & ~(int64_t)3;
      rest.a = p.a + (int64_t)cut * p.k;
      rest.sfa = p.sfa + (int64_t)cut * sf_padded;
      rest.out = static_cast<uint8_t*>(p.out) + (int64_t)cut * p.out_pitch() * 2;
      if (const int rc = launch_sized<OUT_BF16>(main, stream)) return rc;
      return launch_sized<OUT_BF16>(rest, stream);
    }
  }
  switch (whole) {
    case Plan::kStream: return launch_skinny<OUT_BF16>(p, stream);
    case Plan::kTiles256: return launch_fast<4, OUT_BF16>(p, stream);
    case Plan::kTiles128: return launch_fast<2, OUT_BF16>(p, stream);
    case Plan::kOther: break;
  }
  if (tiles(256, 256) >= cus) return launch_cfg<256, 256, OUT_BF16>(p, stream);
  if (tiles(128, 128) >= cus) return launch_cfg<128, 128, OUT_BF16>(p, stream);
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
