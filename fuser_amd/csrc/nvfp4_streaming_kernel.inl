// Weight-streaming NVFP4 kernel of gemm16.hip (included there, inside namespace nvf): the kernel, its launchers and the
// cost estimate that picks slab height and weight tiles per workgroup.
// -------------------------------------------------------------------------------------------------
// NVFP4 skinny path: dense, up to 128 activation rows per launch (decode-sized activations; up to 256 rows in
// two launches), K % 32 == 0, N % (16*RT) == 0.  A launch streams the weight matrix exactly once, so the op
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
// RAGGED_K: K % 128 != 0 (a kernel of its own: the tests for the short chunk cost the others 4-8 %).
// W: wavefronts per workgroup, 8 or (dense, 4 x 8 tiles) 4; two wavefronts per SIMD in both cases, i.e. at most 256
// registers, so that two workgroups of 4 fit a compute unit.
template <int RT, int TT, bool OUT_BF16, int DEPTH, bool GROUPED = false, bool NSPLIT = false, bool RAGGED_K = false, int W = 8>
__global__ __launch_bounds__(W * 64, 2) void nvfp4_skinny_ring_kernel(const Params p) {
  static_assert(GROUPED || !NSPLIT, "the dense op has too few row blocks to give every wavefront its own");
  constexpr int NT = RT + TT;
  // Scale blocks (1 KiB) per operand and chunk: one.  A block holds, for a pair of 16-row tiles, the 16-byte pieces of
  // the 128x4 layout with the scale words of rows {row, row+32, row+64, row+96}: the pairs of an operand (rows 32 apart)
  // find their words in the same pieces, so the block of the first pair serves them all.
  constexpr int B_SC = 1, A_SC = 1;
  // (two places for the activations' block where a chunk's tiles are read one by one while the next chunk's loads are
  // already under way: the chunks of a wavefront alternate between them)
  constexpr int A_SC_PLACES = TT > 2 ? 2 : 1;
  constexpr int SLOT_BYTES = (NT + B_SC + A_SC_PLACES) * 1024;
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
  // K % 128 = 32, 64 or 96: the last chunk is short.  A zero scale makes an NVFP4 block count as zero whatever its
  // payload, so it is enough that the lanes whose 32 elements lie past K (a) fetch bytes that exist - their own row's
  // first piece and the chunk's first scale column tile instead of the next row's bytes and a column tile that the
  // layout may not have - and (b) use zero for the scales of their two blocks, whatever the layout's padding holds.
  int chunks = (p.k + 127) >> 7;
  const int k_tail = p.k & 127;
  const int sf_padded = ((p.k >> 4) + 3) & ~3;  // scale columns with the layout's padding
  // dense with a workspace: blockIdx.z owns the chunks [c_lo, c_lo + chunks) of K and leaves an fp32 partial result
  int c_lo = 0;
  if (!GROUPED && p.partial != nullptr) {
    c_lo = (int)blockIdx.z * p.spans_per_split;
    chunks = min(chunks - c_lo, p.spans_per_split);
  }
  const int tail_chunk = ((p.k + 127) >> 7) - 1 - c_lo;  // the short chunk, counted like this workgroup's chunks
  auto is_tail = [&](int c) { return RAGGED_K && c == tail_chunk; };
  // (worked out where they are used, from a lane number the compiler cannot trace: no registers held for them)
  auto tail_subs = [&](uint32_t& ld_sub, uint32_t& sc_sub) {
    int tl = threadIdx.x & 63;
    asm volatile("" : "+v"(tl));
    const int piece = (tl & 3) ^ ((tl >> 4) & 3);
    ld_sub = piece * 32 < k_tail ? 0u : (uint32_t)piece * 16u;  // back to the row's first piece
    sc_sub = ((tl >> 4) & 1) * 64 < k_tail ? 0u : 512u;         // back to the chunk's first column tile
  };
  auto tail_keep = [&]() {  // read side: all ones if the lane's blocks 2g, 2g+1 of the chunk exist
    int tl = threadIdx.x & 63;
    asm volatile("" : "+v"(tl));
    return (tl >> 4) * 32 < k_tail ? 0xffffffffu : 0u;
  };
  int n0, m_loc, grp = 0, asf_word0 = 0;  // asf_word0: which 32-row group of its 128-row scale tile the slab starts in
  int64_t a_row0 = p.m_base, asf_row0 = p.m_base, b_row0 = 0;  // first activation row, its scale row, first weight row
  if constexpr (GROUPED) {
    const int nblocks = p.n / (16 * RT * (NSPLIT ? W : 1));
    const int block = blockIdx.x / nblocks;
    grp = block;
    if (p.class_slots != 0) {
      // the block-th group of the size class, in group order: every wavefront counts the groups, 256 at a time (four
      // loads in flight: a workgroup that finds no group of its own is gone after one round trip to the L2)
      grp = -1;
      int before = 0;
      for (int base = 0; base < p.groups && grp < 0; base += 256) {
        int mg[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int gi = base + u * 64 + lane;
          mg[u] = gi < p.groups ? p.problem_sizes[gi * 3] : 0;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          uint64_t in_class = __builtin_amdgcn_ballot_w64(mg[u] >= p.rows_lo && mg[u] <= p.rows_hi);
          const int count = __builtin_popcountll(in_class);
          if (grp < 0 && block < before + count) {
            for (int skip = block - before; skip > 0; --skip) in_class &= in_class - 1;
            grp = base + u * 64 + __builtin_ctzll(in_class);
          }
          before += count;
        }
      }
      if (grp < 0) return;
    }
    n0 = ((blockIdx.x - block * nblocks) * (NSPLIT ? W : 1) + (NSPLIT ? wave : 0)) * (16 * RT);
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
    if (is_tail(c_in)) {
      uint32_t ld_sub, sc_sub;
      tail_subs(ld_sub, sc_sub);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) lds_dma16(sb + rt * 1024, b_base, b_off[rt] - ld_sub + c * 64u);
#pragma unroll
      for (int tt = 0; tt < TT; ++tt)
        if (DEPTH == 2 || tt < tt_count) lds_dma16(sb + (RT + tt) * 1024, a_base, a_off[tt] - ld_sub + c * 64u);
#pragma unroll
      for (int j = 0; j < B_SC; ++j) lds_dma16(sb + (NT + j) * 1024, bsf_base, bsf_off[j] - sc_sub + c * 1024u);
#pragma unroll
      for (int j = 0; j < A_SC; ++j)
        if (DEPTH == 2 || 2 * j < tt_count) lds_dma16(sb + (NT + B_SC + j) * 1024, asf_base, asf_off[j] - sc_sub + c * 1024u);
      return;
    }
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
    rd_bsc[rt] = NT * 1024 + ((rt & 1) * 2 + (g >> 1)) * 256 + r * 16 + rowgroup * 4;
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
    rd_asc[tt] = (NT + B_SC) * 1024 + ((tt & 1) * 2 + (g >> 1)) * 256 + r * 16 + (asf_word0 + ((tt * 16) >> 5)) * 4;
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
            *reinterpret_cast<u32x2*>(out + (a_row0 + tok) * p.out_pitch() + n0 + rt * 16 + 4 * g) = v;
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
      for (int u = tid; u < units; u += W * 64) {
        const int l = u & 63, tile = u >> 6;
        const int r2 = tile / tt_count, tt = tile - r2 * tt_count;
        f32x4 s = red[u];
#pragma unroll
        for (int w = 1; w < W; ++w) s += red[w * units + u];
        const int tok = tt * 16 + (l & 15);
        if (!GROUPED && p.stream_result == 1) {
          // Block-scaled result: the quantizer's arithmetic (runtime/block_quantization_kernels.cu:224-263) on alpha *
          // sum.  The 16 columns of a row's block are this lane's four and those of the lanes 16, 32 and 48 further on.
          const float gs = p.gnorm[0], decode = 1.0f / gs;
          const float x0 = s[0] * alpha, x1 = s[1] * alpha, x2 = s[2] * alpha, x3 = s[3] * alpha;
          float amax = fmaxf(fmaxf(fmaxf(fmaxf(-INFINITY, fabsf(x0)), fabsf(x1)), fabsf(x2)), fabsf(x3));  // NaN ignored
          const bool nonfinite = !(fabsf(x0) < INFINITY) || !(fabsf(x1) < INFINITY) || !(fabsf(x2) < INFINITY) || !(fabsf(x3) < INFINITY);
          amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
          amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
          float rr;
          const uint32_t q8 = nvfp4_block_scale(amax, true, gs, decode, tok < m_loc, rr);
          uint32_t w = 0;
          if (__builtin_amdgcn_ballot_w64(nonfinite) == 0) {
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x0 * rr, x1 * rr, 1.0f, 0);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x2 * rr, x3 * rr, 1.0f, 1);
          } else {  // explicit NaN rule of the narrow cast
            w = f32x2_to_e2m1_byte(x0 * rr, x1 * rr) | (f32x2_to_e2m1_byte(x2 * rr, x3 * rr) << 8);
          }
          if (tok < m_loc) {
            const int col4 = n0 + (round * RPR + r2) * 16 + 4 * (l >> 4);
            *reinterpret_cast<uint16_t*>(static_cast<uint8_t*>(p.out) + (a_row0 + tok) * (int64_t)(p.n >> 1) + (col4 >> 1)) = (uint16_t)w;
            if ((l >> 4) == 0) p.out_sf[swizzle_128x4(a_row0 + tok, col4 >> 4, (((int64_t)p.n >> 4) + 3) & ~(int64_t)3)] = (uint8_t)q8;
          }
        }
        if (tok < m_loc) {
          const int col = n0 + (round * RPR + r2) * 16 + 4 * (l >> 4);
          const int64_t at = (a_row0 + tok) * p.out_pitch() + col;
          if (!GROUPED && p.partial != nullptr) {  // this K range's sums as they are; the reduction applies alpha
            *reinterpret_cast<f32x4*>(p.partial + ((int64_t)blockIdx.z * p.m + a_row0 + tok) * p.n + col) = s;
          } else if (!GROUPED && p.stream_result == 2) {  // the fp32 product
            *reinterpret_cast<f32x4*>(static_cast<float*>(p.out) + (a_row0 + tok) * (int64_t)p.n + col) =
                f32x4{s[0] * alpha, s[1] * alpha, s[2] * alpha, s[3] * alpha};
          } else if (!GROUPED && p.stream_result == 1) {
            // (block-scaled result: stored below, outside the test for the row - its shuffles need the whole wavefront)
          } else {
            u32x2 v;
            v[0] = pack2(s[0] * alpha, s[1] * alpha, OUT_BF16);
            v[1] = pack2(s[2] * alpha, s[3] * alpha, OUT_BF16);
            *reinterpret_cast<u32x2*>(out + at) = v;
          }
        }
      }
    }
    if (!GROUPED && p.stream_result == 1 && p.stream_zero_pad != 0 && blockIdx.y == gridDim.y - 1) {
      // block-scaled result: the padding of the scale buffer's last 128x4 tiles is zero - the rows past M (this
      // workgroup's scale columns; the last slab's workgroups) and the columns past N / 16 (the last workgroup)
      const int64_t sf_cols = (int64_t)p.n >> 4, padded = (sf_cols + 3) & ~(int64_t)3;
      const int m_pad = (p.m + 127) & ~127;
      for (int i = tid; i < (m_pad - p.m) * RT; i += W * 64)
        p.out_sf[swizzle_128x4(p.m + i / RT, (n0 >> 4) + i % RT, padded)] = 0;
      if (blockIdx.x == gridDim.x - 1 && padded != sf_cols) {
        const int pc = (int)(padded - sf_cols);
        for (int i = tid; i < m_pad * pc; i += W * 64) p.out_sf[swizzle_128x4(i / pc, sf_cols + i % pc, padded)] = 0;
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
      if (is_tail((int)c)) {
        uint32_t ld_sub, sc_sub;
        tail_subs(ld_sub, sc_sub);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) lds_dma16(ring_base + rt * 1024, b_base, b_off[rt] - ld_sub + c * 64u);
#pragma unroll
        for (int j = 0; j < B_SC; ++j) lds_dma16(ring_base + (NT + j) * 1024, bsf_base, bsf_off[j] - sc_sub + c * 1024u);
        return;
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) lds_dma16(ring_base + rt * 1024, b_base, b_off[rt] + c * 64u);
#pragma unroll
      for (int j = 0; j < B_SC; ++j) lds_dma16(ring_base + (NT + j) * 1024, bsf_base, bsf_off[j] + c * 1024u);
    };
    int fine_lrow = lrow;  // re-derived per use: eight row offsets kept in registers would not fit
    auto load_a_tile = [&](uint32_t c, int tt) {
      asm volatile("" : "+v"(fine_lrow));
      uint32_t ld_sub = 0, sc_sub;
      if (is_tail((int)c)) tail_subs(ld_sub, sc_sub);
      lds_dma16(ring_base + (RT + tt) * 1024, a_base,
                (uint32_t)min(tt * 16 + fine_lrow, m_loc - 1) * (uint32_t)kbytes + lpiece * 16 - ld_sub + c * 64u);
    };
    auto load_a_scales = [&](uint32_t c, uint32_t place = 0) {
      uint32_t ld_sub, sc_sub = 0;
      if (is_tail((int)c)) tail_subs(ld_sub, sc_sub);
      lds_dma16(ring_base + (NT + B_SC) * 1024 + place * 1024u, asf_base, asf_off[0] - sc_sub + c * 1024u);
    };
    const char* sp = reinterpret_cast<const char*>(red) + wave * SLOT_BYTES;
    auto read_a_tile = [&](uint32_t c, int tt, u32x4& aq, uint32_t& as, uint32_t place = 0) {
      aq = *reinterpret_cast<const u32x4*>(sp + (RT + tt) * 1024 + rd_payload);
      as = *reinterpret_cast<const uint32_t*>(sp + rd_asc[tt] + place * 1024u) >> sc_shift;
      if (is_tail((int)c)) as &= tail_keep();
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
      for (int tt = 0; tt < TTC; ++tt) read_a_tile(c, tt, aq[tt], as[tt]);
      if (is_tail((int)c)) {
        const uint32_t keep = tail_keep();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) sc[rt] &= keep;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: may be refilled
      if (c + CSTEP < (uint32_t)chunks) {
        load_b_part(c + CSTEP);
#pragma unroll
        for (int tt = 0; tt < TTC; ++tt) {
          load_a_tile(c + CSTEP, tt);
          if (tt == (TTC > 1 ? 1 : 0)) load_a_scales(c + CSTEP);
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
      if (is_tail((int)c)) {
        const uint32_t keep = tail_keep();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) sc[rt] &= keep;
      }
      u32x4 fb[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) dequant_frags(q[rt], sc[rt], fb[rt]);
#pragma unroll
      for (int tt = 0; tt < TTC; ++tt) {
        __builtin_amdgcn_sched_barrier(0);
        u32x4 aq;
        uint32_t as;
        read_a_tile(c, tt, aq, as);
        if (tt + 1 == TTC) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the last read of the slot is complete
          if (c + CSTEP < (uint32_t)chunks) {
            load_b_part(c + CSTEP);
#pragma unroll
            for (int t2 = 0; t2 < TTC; ++t2) {
              load_a_tile(c + CSTEP, t2);
              if (t2 == (TTC > 1 ? 1 : 0)) load_a_scales(c + CSTEP);
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
      constexpr int NA = TTC + A_SC, LB = RT + B_SC;
      const bool has_next = c + CSTEP < (uint32_t)chunks;
      // this chunk's block of activation scales: tiles 2.. read their words from it after the next chunk's block has
      // been requested, which therefore goes to the other place
      const uint32_t place = ((c - (uint32_t)c_first) / CSTEP) & 1u;
      // loads of this chunk still pending once tile tt and the scale block of its pair have landed
      auto after_tile = [&](int tt) {  // (the scale block follows tile 1, or tile 0 if that is the only one)
        return NA - (tt <= 1 ? (TTC > 1 ? 3 : 2) : tt + 2);
      };
      wait_loads(NA);  // the weight part has landed
      u32x4 q[RT];
      uint32_t sc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) q[rt] = *reinterpret_cast<const u32x4*>(sp + rt * 1024 + rd_payload);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) sc[rt] = *reinterpret_cast<const uint32_t*>(sp + rd_bsc[rt]) >> sc_shift;
      if (is_tail((int)c)) {
        const uint32_t keep = tail_keep();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) sc[rt] &= keep;
      }
      wait_loads(after_tile(0));
      u32x4 aq, aqn = {0, 0, 0, 0};
      uint32_t as, asn = 0;
      read_a_tile(c, 0, aq, as, place);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read out: may be refilled
      if (has_next) {
        load_b_part(c + CSTEP);
        load_a_tile(c + CSTEP, 0);
        if (TTC == 1) load_a_scales(c + CSTEP, place ^ 1u);
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
          wait_loads(after_tile(tt + 1) + (has_next ? LB + (tt + 1) + (tt >= 1 ? 1 : 0) : 0));
          read_a_tile(c, tt + 1, aqn, asn, place);
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
            if (tt == 0) load_a_scales(c + CSTEP, place ^ 1u);
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
          if (tt == (TTC > 1 ? 1 : 0)) load_a_scales((uint32_t)c_first);
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
      }
      if (is_tail(c)) {
        const uint32_t keep = tail_keep();
#pragma unroll
        for (int t = 0; t < NQ; ++t) sc[t] &= keep;
      }
      if constexpr (!kLazyA) {
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
            if (is_tail(c)) as &= tail_keep();
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

template <int RT, int TT, bool OUT_BF16, int W = 8>
int launch_nvfp4_skinny_ring_cfg(const Params& p, hipStream_t stream, int slabs = 1) {
  constexpr int SLOT_KIB = RT + TT + (RT + 1) / 2 + (TT + 1) / 2;
  // one slot per wavefront also where two would fit (M=16, N=14336, K=4096: 8.0 -> 7.5 us; K=14336: 9.6 -> 9.2 us)
  constexpr int DEPTH = 1;
  // More workgroups than compute units (slabs of 128 rows x blocks of 64 weight rows): 4 wavefronts each, so that two
  // share a compute unit (72 KiB of LDS each, 2 wavefronts per SIMD either way) and one streams while the other reduces,
  // stores and starts.  Measured, 8 -> 4 wavefronts: 192 x 14336 x 4096 (448 workgroups) 33.6 -> 28.0 us, 256 x 14336 x 4096
  // 40.2 -> 36.5, 128 x 28672 x 4096 38.8 -> 35.1, 384 x 16384 x 4096 (768) 58.8 -> 53.1, 512 x 8192 x 8192 66.1 -> 63.6;
  // but up to one workgroup per compute unit 128 x 14336 x 4096 22.1 -> 27.3.
  if constexpr (W == 8 && RT == 4 && TT == 8) {
    if ((p.k & 127) == 0 && p.partial == nullptr && (int64_t)(p.n / 64) * slabs > cu_count())
      return launch_nvfp4_skinny_ring_cfg<RT, TT, OUT_BF16, 4>(p, stream, slabs);
  }
  auto kern = W == 8 && (p.k & 127) != 0 ? nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH, false, false, W == 8, W>
                                         : nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH, false, false, false, W>;
  // the ring; the reduction reuses it and needs 1 KiB per wavefront and partial tile of a round
  constexpr int red_kib = W * (RT * TT <= 8 ? RT * TT : TT);
  constexpr int ring_kib = W * DEPTH * SLOT_KIB;
  constexpr int lds_bytes = (ring_kib > red_kib ? ring_kib : red_kib) * 1024;
  static_assert(lds_bytes <= 160 * 1024, "LDS");
  const int splits = p.partial != nullptr ? p.splits : 1;
  if (splits > 1 ? note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d> grid=%ux%dx%d split_k + splitk_reduce_kernel", RT, TT,
                               (unsigned)(p.n / (16 * RT)), slabs, splits)
                 : note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d%s> grid=%ux%d", RT, TT, W == 4 ? ",W=4" : "", (unsigned)(p.n / (16 * RT)), slabs))
    return NVF_OK;
  static std::atomic<uint64_t> configured[2] = {{0}, {0}};  // per kernel, one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured[(p.k & 127) != 0])) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.n / (16 * RT)), (unsigned)slabs, (unsigned)splits), dim3(W * 64), lds_bytes, stream, p);
  if (const int rc = check_launch("nvfp4_skinny_ring_kernel")) return rc;
  if (p.partial == nullptr) return NVF_OK;
  const int64_t mn = (int64_t)p.m * p.n;
  hipLaunchKernelGGL(splitk_reduce_kernel<OUT_BF16>, dim3((unsigned)ceil_div(mn / 4, 256)), dim3(256), 0, stream, p.partial, splits, mn, p.alpha,
                     static_cast<uint16_t*>(p.out));
  return check_launch("splitk_reduce_kernel");
}

template <int RT, int TT, bool OUT_BF16, bool NSPLIT, int W = 8>
int launch_nvfp4_skinny_grouped(const Params& p0, int rows_lo, int rows_hi, hipStream_t stream) {
  constexpr int SLOT_KIB = RT + TT + (RT + 1) / 2 + (TT + 1) / 2;
  // One slot per wavefront also where two would fit: measured faster for the groups of up to 32 rows (512 rows
  // over 256 experts, K=7168: 401 -> 375 us; K=2048: 432 -> 413 us).  Forcing the registers down to two
  // workgroups per compute unit on top of that costs more than it gains (450 us).
  constexpr int DEPTH = 1;
  auto kern = W == 8 && (p0.k & 127) != 0 ? nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH, true, NSPLIT, W == 8, W>
                                          : nvfp4_skinny_ring_kernel<RT, TT, OUT_BF16, DEPTH, true, NSPLIT, false, W>;
  constexpr int red_kib = NSPLIT ? 0 : W * (RT * TT <= 8 ? RT * TT : TT);
  constexpr int ring_kib = W * DEPTH * SLOT_KIB;
  constexpr int lds_bytes = (ring_kib > red_kib ? ring_kib : red_kib) * 1024;
  static_assert(lds_bytes <= 160 * 1024, "LDS");
  Params p = p0;
  p.rows_lo = rows_lo;
  p.rows_hi = rows_hi;
  // Groups of rows_lo rows or more: at most m / rows_lo of them exist (the groups are disjoint row ranges of the
  // activations), so the launch has that many blocks of workgroups and each looks its group up.  One block per group
  // costs a decode step with 256 experts 20-30 us of workgroups that return at once.
  if (rows_lo > 1) p.class_slots = (int)std::min<int64_t>(p.groups, p.m / rows_lo);
  if (rows_lo > 1 && p.class_slots == 0) return NVF_OK;  // fewer rows in all than one such group has
  const int64_t wgs = (int64_t)(p.class_slots ? p.class_slots : p.groups) * (p.n / (16 * RT * (NSPLIT ? 8 : 1)));
  // (groups of 33-128 rows, more workgroups than compute units: 4 wavefronts each and two to a compute unit, as in the
  // dense launch; 8 experts x 64 rows, N=14336, K=4096: 111 -> 86 us, 32 x 40 rows, N=7168: 180 -> 142, 64 x 64 rows,
  // N=2048, K=7168: 187 -> 164)
  if constexpr (W == 8 && RT == 4 && TT == 8 && !NSPLIT) {
    if ((p.k & 127) == 0 && wgs > cu_count()) return launch_nvfp4_skinny_grouped<RT, TT, OUT_BF16, NSPLIT, 4>(p0, rows_lo, rows_hi, stream);
  }
  if (wgs >= ((int64_t)1 << 31)) return fail(NVF_ERR_UNSUPPORTED_SHAPE, "too many (group, row block) pairs for one launch");
  if (note_launch("nvfp4_skinny_ring_kernel<RT=%d,TT=%d,grouped,nsplit=%d%s> grid=%lld rows=%d..%d", RT, TT, (int)NSPLIT, W == 4 ? ",W=4" : "", (long long)wgs,
                  rows_lo, rows_hi))
    return NVF_OK;
  static std::atomic<uint64_t> configured[2] = {{0}, {0}};  // per kernel, one bit per device
  if (const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, configured[(p.k & 127) != 0])) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(W * 64), lds_bytes, stream, p);
  return check_launch("nvfp4_skinny_ring_kernel (grouped)");
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
inline int nvfp4_four_wavefront_percent(int64_t k) { return k < 768 ? 73 : k < 1536 ? 78 : k < 3072 ? 85 : k < 6144 ? 89 : k < 10240 ? 92 : 95; }
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
  const int64_t chunks = ceil_div((k + 127) >> 7, 8);
  const int64_t resident = std::min(per_cu, ceil_div(wgs, cus));
  const int64_t rounds = ceil_div(wgs, cus * per_cu);
  const int64_t per_chunk = (rt + tt) * 183 + rt * tt * 18 + 100;
  const int64_t wg_time = chunks * per_chunk * (100 + 73 * (resident - 1)) / 100 + rt * tt * 110 + 5070;
  // (4 x 8 tiles with more workgroups than compute units run as workgroups of 4 wavefronts, two to a compute unit:
  // measured 27 % (K = 512) .. 5 % (K = 14336) faster than the rounds of one workgroup per compute unit)
  if (rt == 4 && tt == 8 && (k & 127) == 0 && wgs > cus) {
    // (two workgroups share a compute unit and a short one makes room early: the workgroups of a last slab with fewer
    // row tiles count by their share of a full one's time - 320 x 11008 x 2048: 2.6 slabs x 172 in 2 rounds, not 3)
    int64_t rounds4 = rounds;
    const int tt_last = m > slab ? (int)ceil_div(m % slab, 16) : 0;
    if (tt_last != 0) {
      const int64_t wg_last = chunks * ((rt + tt_last) * 183 + rt * tt_last * 18 + 100) + rt * tt_last * 110 + 5070;
      rounds4 = ceil_div((slabs - 1) * (n / 64) * wg_time + (n / 64) * wg_last, wg_time * cus);
    }
    return rounds4 * wg_time * nvfp4_four_wavefront_percent(k) / 100;
  }
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
