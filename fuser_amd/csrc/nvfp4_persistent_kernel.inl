// Persistent 256x256 / 128x256 NVFP4 kernel of gemm16.hip (included there, inside namespace nvf).
// -------------------------------------------------------------------------------------------------
// NVFP4 fast path: 256x256 (or 128x256) tile, N % 256 == 0, K % 128 == 0 (dense with a 16-bit result: K % 32 == 0),
// K >= 256; dense with M % 256 (128) == 0,
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
// RAGGED_K (16-bit result; grouped: the 256x256 tiles): K % 128 = 32, 64 or 96.  A tile's last span is short: the threads whose 32 elements lie
// past K fetch their row's first piece instead of the next row's bytes, and their scale load runs past the range of its
// buffer resource on purpose, which makes it return zero - and a zero scale makes a block count as zero.
// RAGGED_M (dense): the last row tile holds fewer than BM rows.  As for the last tile of a group, the
// buffer range of the activations ends with the last row, so the rows past it read as zero, and they are not stored;
// the scale tile of a 256-row tile's second half may not exist and then reads as zero the same way.
template <bool OUT_BF16, bool GROUPED, int TM = 4, bool OUT_F32 = false, bool PAIRS = false, bool OUT_FP4 = false, bool RAGGED_K = false,
          bool RAGGED_M = false>
__global__ __launch_bounds__(512) void nvfp4_gemm_256_kernel(const Params p) {
  static_assert(TM == 4 || TM == 2, "tile height");
  static_assert(!RAGGED_M || !GROUPED, "a short last row tile: dense calls (the groups' tiles are always of that kind)");
  constexpr bool PARTIAL = GROUPED || RAGGED_M;  // tiles may hold fewer rows than BM
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
  const int tiles_m = (RAGGED_M ? p.m + BM - 1 : p.m) / BM, tiles_n = p.n / BN;
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
  // (n-tiles past the last multiple of 4: blocks of 8 (m) x 1..3 (n) after all the others)
  const bool blocked = (tiles_m & 7) == 0 && tiles_n >= 4;
  const int bulk_tiles = tiles_m * (tiles_n & ~3);
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
      if (blocked && t < bulk_tiles) {
        const int sb = t >> 5, q = t & 31;
        mt = (sb % (tiles_m >> 3)) * 8 + (q & 7);
        nt = (sb / (tiles_m >> 3)) * 4 + (q >> 3);
      } else if (blocked) {
        const int u = t - bulk_tiles, bs = 8 * (tiles_n & 3), sb = u / bs, q = u - sb * bs;
        mt = sb * 8 + (q & 7);
        nt = (tiles_n & ~3) + (q >> 3);
      } else {
        mt = t % tiles_m;
        nt = t / tiles_m;
      }
      w.g = 0;
      w.gm0 = mt * BM;
      w.m0 = w.gm0;
      w.n0 = nt * BN;
      w.valid = RAGGED_M ? min(BM, p.m - w.gm0) : BM;
    }
    return w;
  };
  const int first_tile = xcd * chunk_tiles + slot;
  if (first_tile >= range_end) return;

  const int kbytes = p.k >> 1;
  const int nmac = (p.k + 127) >> 7;            // 128-deep load spans per tile (>= 2)
  const int sf_padded = ((p.k >> 4) + 3) & ~3;  // scale columns with the layout's padding
  const int64_t row128 = (int64_t)128 * kbytes;       // payload distance of the thread's two rows
  const int64_t sfrow128 = (int64_t)128 * sf_padded;  // same for the scales (next 128-row tile)

  // ---- operand stream: the tile the stream is in (lp) and the tile it enters next (np), as wave-uniform
  // addresses of the tiles' first rows (scalar registers; they advance by scalar selects), and this thread's
  // fixed 32-bit offsets inside any tile: its row and 16-byte piece, and its scale word (blocks 2*spiece,
  // 2*spiece+1 of the span: 128x4 layout column tile spiece>>1, bytes 2*(spiece&1)..).  A tile's first row is
  // a multiple of 128, so the swizzled scale address splits into the tile's part and the thread's part.
  // a_bytes / a_bytes2: bytes of the existing A rows among the tile's rows 0..127 / 128..255 (buffer ranges)
  struct RowPtrs { const uint8_t *a, *b, *sa, *sb; int a_bytes, a_bytes2, sa_bytes2; };
  auto tile_ptrs = [&](int t) {
    const Where w = tile_where(t);
    RowPtrs r;
    r.a = p.a + w.m0 * kbytes;
    // the last tile of a group may have fewer rows than the tile: the rows past the group read as zero
    r.a_bytes = PARTIAL ? min(w.valid, 128) * kbytes : 0x7fffffff;
    r.a_bytes2 = PARTIAL ? max(w.valid - 128, 0) * kbytes : 0x7fffffff;
    r.sa_bytes2 = RAGGED_M && w.valid <= 128 ? 0 : 0x7fffffff;  // (no rows 128.. : their scale tile may not exist)
    r.b = p.b + ((int64_t)w.g * p.n + w.n0) * kbytes;
    // (a group's activation scales are a slab of their own, swizzled from its first row)
    const int64_t sa_slab = GROUPED ? (int64_t)__builtin_amdgcn_readfirstlane(p.sf_offsets[w.g]) * sf_padded : 0;
    r.sa = p.sfa + sa_slab + swizzle_128x4(w.gm0, 0, sf_padded);
    r.sb = p.sfb + (int64_t)w.g * p.n * sf_padded + swizzle_128x4(w.n0, 0, sf_padded);
    return r;
  };
  const uint32_t off_ab_full = (uint32_t)srow * (uint32_t)kbytes + (uint32_t)spiece * 16u;
  const uint32_t off_sf_full = (uint32_t)swizzle_128x4(srow, 0, sf_padded) + (uint32_t)(spiece >> 1) * 512u + (uint32_t)(spiece & 1) * 2u;
  // RAGGED_K: the offsets for a tile's last span
  const bool in_tail = spiece * 32 < (p.k & 127);
  const uint32_t off_ab_tail = in_tail ? off_ab_full : off_ab_full - (uint32_t)spiece * 16u;
  const uint32_t off_sf_tail = in_tail ? off_sf_full : 0x7fffffffu;
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
    const bool tail = RAGGED_K && l_mac == nmac - 1;  // wave-uniform
    const uint32_t off_ab = tail ? off_ab_tail : off_ab_full, off_sf = tail ? off_sf_tail : off_sf_full;
    if (q == 0) r.a[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.a, lp.a_bytes), off_ab, o, 0);
    // (rows 128.. of the tile through a resource of their own, so that the range check that zeroes the rows past a
    // group never depends on whether the hardware counts the scalar offset)
    if (q == 1 && AR == 2) r.a[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.a + row128, lp.a_bytes2), off_ab, o, 0);
    if (q == 2) r.b[0] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.b), off_ab, o, 0);
    if (q == 3) r.b[1] = __builtin_amdgcn_raw_buffer_load_b128(rsrc(lp.b), off_ab, o + (int)row128, 0);
    if (q == 4) r.sa[0] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sa), off_sf, so, 0);
    if (q == 5 && AR == 2) {
      if constexpr (RAGGED_M) r.sa[1] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sa + sfrow128, lp.sa_bytes2), off_sf, so, 0);
      else r.sa[1] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sa), off_sf, so + (int)sfrow128, 0);
    }
    if (q == 6) r.sb[0] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sb), off_sf, so, 0);
    if (q == 7) r.sb[1] = __builtin_amdgcn_raw_buffer_load_b16(rsrc(lp.sb), off_sf, so + (int)sfrow128, 0);
  };
  auto advance_stream = [&]() {
    const bool wrap = (l_mac + 1 == nmac);
    l_mac = wrap ? 0 : l_mac + 1;
    lp.a = wrap ? np.a : lp.a;
    lp.a_bytes = wrap ? np.a_bytes : lp.a_bytes;
    lp.a_bytes2 = wrap ? np.a_bytes2 : lp.a_bytes2;
    if (RAGGED_M) lp.sa_bytes2 = wrap ? np.sa_bytes2 : lp.sa_bytes2;
    lp.b = wrap ? np.b : lp.b;
    lp.sa = wrap ? np.sa : lp.sa;
    lp.sb = wrap ? np.sb : lp.sb;
  };

  // ---- the thread's LDS byte addresses: per operand, one for each half scale block it stages and one for each of the
  // four 16-deep sub-steps it reads fragments of (the swizzle makes those differ by an exclusive or, not by a sum).
  // They pass through empty asm statements, so that the compiler keeps exactly these twelve registers and reaches
  // buffer, row tile and second staging row through the instructions' immediate offsets.
  uint8_t* const lds_b = reinterpret_cast<uint8_t*>(lds);
  uint32_t stage_at[2][2], frag_at[2][4];
#pragma unroll
  for (int op = 0; op < 2; ++op) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      stage_at[op][cc] = (uint32_t)(tile_units(0, op) + lds_pos2(srow, spiece * 2 + cc)) * 16u;
      asm volatile("" : "+v"(stage_at[op][cc]));
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      frag_at[op][kk] = (uint32_t)(tile_units(0, op) + lds_pos2((op ? wn * 64 : wm * (32 * TM)) + li, kk * 2 + lg)) * 16u;
      asm volatile("" : "+v"(frag_at[op][kk]));
    }
  }

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
      *reinterpret_cast<u32x4*>(lds_b + stage_at[op][cc] + (wbuf * (op ? TILE_UNITS : A_UNITS) + i * 1024) * 16) =
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
    const u32x4 v = *reinterpret_cast<const u32x4*>(lds_b + frag_at[op][kk] + (buf * (op ? TILE_UNITS : A_UNITS) + t * 256) * 16);
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
        if (!RAGGED_M || wm * (32 * TM) + i * 32 + (elane >> 1) < cw.valid) *reinterpret_cast<u32x4*>(obase + (int64_t)(i * 32) * opitch) = v;
        asm volatile("" ::: "memory");
      }
      // (RAGGED_M: the rows past M read as zero, so their scale codes are zero - exactly what the padding rows of the
      // last 128-row scale tile must hold; a 256-row tile with at most 128 rows has no second scale tile to write)
      if (lg == 0 && (!RAGGED_M || TM == 2 || wm * 128 < cw.valid)) {
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
            if (!RAGGED_M || wm * (32 * TM) + i * 32 + 16 * t + (elane >> 2) < cw.valid)
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
      const int ldc = p.out_pitch();
      const uint32_t ooff = ((uint32_t)(elane >> 2) * (uint32_t)ldc + (uint32_t)(elane & 3) * 8u) * 2u;
      uint8_t* obase = reinterpret_cast<uint8_t*>(static_cast<uint16_t*>(p.out) + (cw.m0 + wm * (32 * TM)) * ldc + cw.n0 + wn * 64);
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
            if (!PARTIAL || wm * (32 * TM) + brow + erow < cw.valid)
              *reinterpret_cast<u32x4*>(obase + ((int64_t)brow * ldc + j * 32) * 2 + ooff) = v;
          }
          asm volatile("" ::: "memory");
        }
      }
    }
    zero_acc();
  }
#undef NVF_PIN_ACC
}

template <bool OUT_BF16, bool GROUPED, int TM, bool OUT_F32, bool PAIRS, bool OUT_FP4 = false, bool RAGGED_K = false, bool RAGGED_M = false>
int launch_nvfp4_fast_cfg(const Params& p, int cus, hipStream_t stream) {
  auto kern = nvfp4_gemm_256_kernel<OUT_BF16, GROUPED, TM, OUT_F32, PAIRS, OUT_FP4, RAGGED_K, RAGGED_M>;
  if (!GROUPED && !RAGGED_M && p.m % (64 * TM) != 0) return fail(NVF_ERR_LAUNCH, "nvfp4_gemm_256_kernel: M = %d is no multiple of %d", p.m, 64 * TM);
  constexpr int lds_bytes = 2 * (64 * TM + 256) * 128 + 8 * 2560;  // 128 KiB / 96 KiB of tiles + the epilogue's 20 KiB
  // grouped: an upper bound (128-row tiles: one per weight panel and group of at least rows_lo rows)
  const int64_t tiles_m = (GROUPED && TM == 2) ? std::min<int64_t>(p.groups, p.m / std::max(p.rows_lo, 1)) : (p.m + (RAGGED_M ? 64 * TM - 1 : 0)) / (64 * TM);
  const int64_t tiles = tiles_m * (p.n / 256);
  const unsigned grid = (unsigned)(tiles >= cus ? (cus & ~7) : ((tiles + 7) / 8) * 8);
  if (grid == 0) return NVF_OK;  // fewer rows in the whole call than the smallest group this launch serves: no work
  if (note_launch("nvfp4_gemm_256_kernel<grouped=%d,TM=%d,f32=%d,pairs=%d%s%s%s> grid=%u rows=%d..%d min_rows=%d", (int)GROUPED, TM, (int)OUT_F32,
                  (int)PAIRS, OUT_FP4 ? ",fp4_blockscale" : "", RAGGED_M ? ",ragged_m" : "", RAGGED_K ? ",ragged_k" : "", grid, p.rows_lo, p.rows_hi,
                  p.min_rows))
    return NVF_OK;
  static std::atomic<uint64_t> configured{0};  // one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured)) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds_bytes, stream, p);
  return check_launch("nvfp4_gemm_256_kernel");
}

template <bool OUT_BF16, bool GROUPED, int TM = 4, bool OUT_F32 = false, bool OUT_FP4 = false>
int launch_nvfp4_fast(const Params& p, int cus, hipStream_t stream) {
  // an even number of 128-deep spans per tile: the variant whose two in-flight spans swap names instead of being copied
  if constexpr ((!GROUPED || TM == 4) && !OUT_F32 && !OUT_FP4) {
    if ((p.k & 127) != 0) {  // a short last span: an even number of spans counts it
      if ((((p.k + 127) >> 7) & 1) == 0) return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, true, OUT_FP4, true>(p, cus, stream);
      return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, false, OUT_FP4, true>(p, cus, stream);
    }
  }
  if constexpr (!GROUPED) {
    if (p.m % (64 * TM) != 0) {  // a last row tile with fewer rows
      if (((p.k >> 7) & 1) == 0) return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, true, OUT_FP4, false, true>(p, cus, stream);
      return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, false, OUT_FP4, false, true>(p, cus, stream);
    }
  }
  if (((p.k >> 7) & 1) == 0) return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, true, OUT_FP4>(p, cus, stream);
  return launch_nvfp4_fast_cfg<OUT_BF16, GROUPED, TM, OUT_F32, false, OUT_FP4>(p, cus, stream);
}
