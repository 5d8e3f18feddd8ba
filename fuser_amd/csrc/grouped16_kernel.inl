// Persistent 256x256 kernel for grouped_mm (16-bit operands) of gemm16.hip (included there, inside namespace nvf).
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
