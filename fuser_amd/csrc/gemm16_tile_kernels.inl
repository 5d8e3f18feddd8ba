// Tile kernels of gemm16.hip (included there, inside namespace nvf): 16-bit operands (grouped_mm and its dense form),
// NVFP4 operands for any shape (fp32 / block-scaled result, split of K), and the reduction of a split.
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
            uint16_t* orow = static_cast<uint16_t*>(p.out) + (row_off + mrow) * (int64_t)p.out_pitch();
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
