// Grouped NVFP4 kernel for groups of 33..80 rows of gemm16.hip (included there, inside namespace nvf).
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
    for (int rt = 0; rt < RT; ++rt) lds_dma16(bslot + rt * 1024, b_base + c * 64u, b_off[rt]);
#pragma unroll
    for (int j = 0; j < B_SC; ++j) lds_dma16(bslot + (RT + j) * 1024, bsf_base + c * 1024u, bsf_off[j]);
  };
  // (the chunk moves the wave-uniform base address, not the lanes' offsets: scalar additions)
  auto load_a = [&](uint32_t c) {
    lds_dma16(aslot, a_base + c * 64u, a_off);
    lds_dma16(aslot + 1024, asf_base + c * 1024u, asf_off);
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
    // packed weights of a chunk and their scales: two sets that take turns as "current" and "next", so that no
    // register moves from one to the other at the end of a chunk
    struct Weights { u32x4 q[RT]; f16x2 sv[RT][2]; };
    Weights w0, w1;
    u32x4 (&q)[RT] = w0.q;
    f16x2 (&sv)[RT][2] = w0.sv;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      w1.q[rt] = u32x4{0, 0, 0, 0};
      w1.sv[rt][0] = w1.sv[rt][1] = f16x2{0, 0};
    }
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

    // raw activation tile and weight scales of the next chunk: read out only while there is a next chunk, and what
    // the last chunk converts from the stale values goes to a buffer nobody reads
    u32x4 aq = {0, 0, 0, 0};
    uint32_t as = 0;
    uint32_t scn[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) scn[rt] = 0;
    auto chunk = [&](int c, Weights& cur, Weights& nxt) {
      u32x4 (&q)[RT] = cur.q;
      f16x2 (&sv)[RT][2] = cur.sv;
      u32x4 (&qn)[RT] = nxt.q;
      f16x2 (&svn)[RT][2] = nxt.sv;
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
      f16x2 asv[2];
      if (has1) {
        wait_loads(has_b_next ? LB : 0);
        aq = *reinterpret_cast<const u32x4*>(asp + rd_payload);
        as = *reinterpret_cast<const uint32_t*>(asp + rd_asc) >> sc_shift;
      }
      u32x4 fbn[RT];
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
    };
    int c = 0;
    for (; c + 1 < chunks; c += 2) {
      chunk(c, w0, w1);
      chunk(c + 1, w1, w0);
    }
    if (c < chunks) chunk(c, w0, w1);

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
