/*
 * CPU restatement of the reference's quantized-GEMM hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file; it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have an independent statement of the reference semantics to
 * compare the HIP kernels against.
 *
 * Every function cites the reference source it restates (paths relative to the
 * reference checkout).  Scalar, single-threaded, written for clarity.
 *
 * Parity status
 *   pinned   : e2m1 / e4m3 / e8m0 codecs (all finite inputs), 128x4 swizzle,
 *              NVFP4 and MXFP8 block quantizers, grouped scale placement,
 *              dequantisation.  Each is checked in tests/ against closed forms,
 *              library casts, brute force and the fixtures under tests/golden/.
 *   unpinned : the result of the narrow casts for NaN inputs (and for negative
 *              or NaN inputs of the unsigned e8m0 cast).  The reference defines
 *              them only through PTX `cvt.*.satfinite`, no reference test
 *              exercises them, and no NVIDIA hardware is available.  The values
 *              chosen here follow the PTX ISA text: e4m3 NaN -> 0x7F,
 *              e2m1 NaN -> +6 (0x7), ue8m0 NaN -> 0xFF.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

enum { ORC_F32 = 0, ORC_BF16 = 1, ORC_F16 = 2 };

/* ------------------------------------------------------------------ bits */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* runtime/casts.cu: __bfloat2float -- a bf16 is the top half of an fp32. */
ORC_API float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* runtime/casts.cu: __half2float -- IEEE binary16 -> binary32, exact. */
ORC_API float orc_f16_to_f32(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31;
  int e = (h >> 10) & 31;
  uint32_t m = h & 1023;
  if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
  if (e == 0) {
    float v = ldexpf((float)m, -24);
    return (h >> 15) ? -v : v;
  }
  return u2f(s | ((uint32_t)(e - 15 + 127) << 23) | (m << 13));
}

static float load_as_f32(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case ORC_F32: return ((const float*)p)[i];
    case ORC_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[i]);
    default: return orc_f16_to_f32(((const uint16_t*)p)[i]);
  }
}

/* -------------------------------------------------------------- e2m1 (fp4)
 * runtime/casts.cu:1074-1111  `cvt.rn.satfinite.e2m1x2.f32`
 * Round to nearest, ties to even code, on the grid {0,.5,1,1.5,2,3,4,6};
 * magnitudes above 6 (and infinities) saturate to 6.  Code = sign<<3 | index.
 * Written as a nearest-grid-point search so that it shares no structure with
 * threshold-compare or hardware implementations. */
static const float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

ORC_API uint8_t orc_f32_to_e2m1(float x) {
  if (x != x) return 0x7; /* unpinned: PTX satfinite maps NaN to +MAX_NORM */
  uint8_t sign = (uint8_t)((f2u(x) >> 31) << 3);
  double a = fabs((double)x);
  int best = 0;
  double best_d = a; /* distance to 0 */
  for (int i = 1; i < 8; ++i) {
    double d = fabs(a - (double)kE2M1[i]);
    if (d < best_d || (d == best_d && (i & 1) == 0)) { /* tie -> even code */
      best = i;
      best_d = d;
    }
  }
  if (a > 6.0) best = 7;
  return sign | (uint8_t)best;
}

/* tests/python/direct_utils/narrow_precision.py:53-73 -- 16-entry decode LUT */
ORC_API float orc_e2m1_to_f32(uint8_t code) {
  float v = kE2M1[code & 7];
  return (code & 8) ? -v : v;
}

/* -------------------------------------------------------------- e4m3fn
 * runtime/casts.cu:755-776 `cvt.rn.f16x2.e4m3x2` then half->float: exact decode.
 * 1-4-3, bias 7, no infinities, S.1111.111 = NaN, subnormals m*2^-9. */
ORC_API float orc_e4m3_to_f32(uint8_t v) {
  int e = (v >> 3) & 15, m = v & 7;
  float r;
  if (e == 15 && m == 7) r = NAN;
  else if (e == 0) r = ldexpf((float)m, -9);
  else r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return (v & 0x80) ? -r : r;
}

/* runtime/casts.cu:698-712 `cvt.rn.satfinite.e4m3x2.f32`
 * Round to nearest even onto the e4m3 grid, saturating to +-448. */
ORC_API uint8_t orc_f32_to_e4m3(float x) {
  if (x != x) return 0x7f; /* unpinned */
  uint8_t sign = (uint8_t)((f2u(x) >> 31) << 7);
  double a = fabs((double)x);
  if (a >= 448.0) return sign | 0x7e;
  /* spacing: 2^-9 below 2^-6, else 2^(floor(log2 a) - 3) */
  int ex;
  (void)frexp(a, &ex); /* a = f * 2^ex, f in [0.5,1) -> floor(log2 a) = ex-1 */
  int e = (a == 0.0) ? -6 : ex - 1;
  if (e < -6) e = -6;
  double ulp = ldexp(1.0, e - 3);
  double q = nearbyint(a / ulp); /* default rounding mode = ties to even; a/ulp is exact */
  double r = q * ulp;
  if (r >= 448.0) return sign | 0x7e; /* cannot happen for a < 448, kept for clarity */
  /* encode r */
  if (r < ldexp(1.0, -6)) return sign | (uint8_t)q; /* subnormal: q in 0..7 (q == 8 is 2^-6) */
  (void)frexp(r, &ex);
  int re = ex - 1;
  int m = (int)(r / ldexp(1.0, re - 3)) - 8;
  return sign | (uint8_t)(((re + 7) << 3) | m);
}

/* -------------------------------------------------------------- ue8m0
 * runtime/casts.cu:913-927 `cvt.rp.satfinite.ue8m0x2.f32`
 * Unsigned power of two 2^(e-127); round toward +infinity, so the result is
 * the smallest representable power of two >= x; 0xFF is NaN; saturate at 0xFE. */
ORC_API uint8_t orc_f32_to_e8m0_rp(float x) {
  if (x != x) return 0xff; /* unpinned */
  if (x <= 0.0f) return 0; /* unpinned for negative inputs; exact for +-0 */
  if (isinf(x)) return 0xfe;
  int ex;
  double f = frexp((double)x, &ex); /* x = f * 2^ex, f in [0.5, 1) */
  int p = (f == 0.5) ? ex - 1 : ex;  /* ceil(log2 x) */
  int e = p + 127;
  if (e < 0) e = 0;
  if (e > 254) e = 254;
  return (uint8_t)e;
}

ORC_API float orc_e8m0_to_f32(uint8_t e) {
  if (e == 0xff) return NAN;
  return ldexpf(1.0f, (int)e - 127);
}

/* ------------------------------------------------------- 128x4 swizzle
 * runtime/block_quantization_kernels.cu:15-57 outputOffsetAfterSwizzlePadding<32,4,4>
 * (same layout as :291-316, tests/python/direct_utils/narrow_precision.py:27-43
 * and csrc/ir/utils.cpp:1729-1751).  Byte offset of scale (row, col) inside a
 * [roundUp(R,128), padded_cols] buffer, padded_cols a multiple of 4. */
ORC_API int64_t orc_swizzle_128x4_offset(int64_t row, int64_t col, int64_t padded_cols) {
  int64_t row_tile = row / 128;
  int64_t row_in_tile = row % 128;
  int64_t row_inner = row_in_tile / 32; /* 0..3 */
  int64_t row_outer = row_in_tile % 32; /* 0..31 */
  int64_t col_tile = col / 4;
  int64_t col_in = col % 4;
  return row_tile * padded_cols * 128 + col_tile * 512 + row_outer * 16 + row_inner * 4 + col_in;
}

/* expert lookup of runtime/block_quantization_kernels.cu:338-344 / :387-393 */
static int find_group(int64_t row, const int32_t* input_offsets, int groups) {
  int g = groups - 1;
  for (int i = 1; i < groups; ++i) {
    if (row < input_offsets[i]) {
      g = i - 1;
      break;
    }
  }
  return g;
}

/* -------------------------------------------------- NVFP4 block quantizer
 * runtime/block_quantization_kernels.cu:194-263 block_quantize_to_nvfp4_util
 * One block = 16 contiguous innermost elements, fp32 arithmetic in this order. */
static uint8_t quantize_block16(const float* x, const float* global_scale, uint8_t* payload8) {
  float amax = -INFINITY;
  for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(x[i])); /* :124-128, fmax ignores NaN */
  const float float_max = 3.40282346638528859811704183484516925440e+38f;
  volatile float s = amax / 6.0f; /* :224 */
  if (global_scale) s = s * global_scale[0]; /* :226 */
  s = fminf(s, float_max); /* :228 */
  uint8_t q8 = orc_f32_to_e4m3(s); /* :230 */
  volatile float sf = orc_e4m3_to_f32(q8); /* :233 */
  volatile float r;
  if (global_scale) {
    volatile float decode = 1.0f / global_scale[0]; /* :236 */
    volatile float t = sf * decode;
    r = fminf(1.0f / t, float_max); /* :237 */
  } else {
    r = fminf(1.0f / sf, float_max); /* :239 */
  }
  for (int j = 0; j < 8; ++j) {
    volatile float y0 = x[2 * j] * r; /* :249 */
    volatile float y1 = x[2 * j + 1] * r;
    /* runtime/casts.cu:1081-1088: even element -> low nibble */
    payload8[j] = (uint8_t)(orc_f32_to_e2m1(y0) | (orc_f32_to_e2m1(y1) << 4));
  }
  return q8;
}

/* runtime/block_quantization_kernels.cu:265-319 block_quantize_to_nvfp4
 * in: [rows, cols] row-major, cols % 16 == 0.
 * out_fp4: [rows, cols/2] bytes.  out_sf: linear [rows, cols/16] when swizzle == 0,
 * else the 128x4 layout inside [roundUp(rows,128), roundUp(cols/16,4)] (padding untouched). */
ORC_API void orc_block_quantize_nvfp4(const void* in, int dtype, int64_t rows, int64_t cols,
                                      const float* global_scale, int swizzle, uint8_t* out_fp4,
                                      uint8_t* out_sf) {
  int64_t sf_cols = cols / 16;
  int64_t padded = (sf_cols + 3) / 4 * 4;
  float x[16];
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t b = 0; b < sf_cols; ++b) {
      for (int i = 0; i < 16; ++i) x[i] = load_as_f32(in, dtype, r * cols + b * 16 + i);
      uint8_t q8 = quantize_block16(x, global_scale, out_fp4 + (r * cols + b * 16) / 2);
      int64_t off = swizzle ? orc_swizzle_128x4_offset(r, b, padded) : r * sf_cols + b;
      out_sf[off] = q8;
    }
  }
}

/* runtime/block_quantization_kernels.cu:363-413 grouped_block_quantize_to_nvfp4
 * Scales of group g go to rows [output_offsets[g], ...) of a
 * [sum roundUp(m_g,128), roundUp(cols/16,4)] buffer, each group swizzled on its own. */
ORC_API void orc_grouped_block_quantize_nvfp4(const void* in, int dtype, int64_t rows, int64_t cols,
                                              const int32_t* input_offsets, const int32_t* output_offsets,
                                              int groups, const float* global_scale, uint8_t* out_fp4,
                                              uint8_t* out_sf) {
  int64_t sf_cols = cols / 16;
  int64_t padded = (sf_cols + 3) / 4 * 4;
  float x[16];
  for (int64_t r = 0; r < rows; ++r) {
    int g = find_group(r, input_offsets, groups);
    int64_t rr = r - input_offsets[g];
    for (int64_t b = 0; b < sf_cols; ++b) {
      for (int i = 0; i < 16; ++i) x[i] = load_as_f32(in, dtype, r * cols + b * 16 + i);
      uint8_t q8 = quantize_block16(x, global_scale, out_fp4 + (r * cols + b * 16) / 2);
      out_sf[(int64_t)output_offsets[g] * padded + orc_swizzle_128x4_offset(rr, b, padded)] = q8;
    }
  }
}

/* runtime/block_quantization_kernels.cu:321-361 preprocessGroupedMatmulInputSf
 * Pure layout: linear [rows, cols] elements of elem_size bytes -> per-group padded swizzled buffer. */
ORC_API void orc_preprocess_grouped_sf(const void* in, int elem_size, int64_t rows, int64_t cols,
                                       const int32_t* input_offsets, const int32_t* output_offsets,
                                       int groups, void* out) {
  int64_t padded = (cols + 3) / 4 * 4;
  for (int64_t r = 0; r < rows; ++r) {
    int g = find_group(r, input_offsets, groups);
    int64_t rr = r - input_offsets[g];
    for (int64_t c = 0; c < cols; ++c) {
      int64_t off = (int64_t)output_offsets[g] * padded + orc_swizzle_128x4_offset(rr, c, padded);
      memcpy((char*)out + off * elem_size, (const char*)in + (r * cols + c) * elem_size, elem_size);
    }
  }
}

/* -------------------------------------------------- MXFP8 block quantizer
 * runtime/block_quantization_kernels.cu:142-186 block_quantize_to_mxfp8, exp2f_rcp :131-140
 * One block = 32 contiguous elements; scale = ue8m0_rp(amax * (1/448)) stored linearly. */
ORC_API void orc_block_quantize_mxfp8(const void* in, int dtype, int64_t rows, int64_t cols, uint8_t* out_fp8,
                                      uint8_t* out_sf) {
  const float max_norm_rcp = 1.0f / 448;
  int64_t n = rows * cols;
  for (int64_t b = 0; b < n / 32; ++b) {
    float x[32];
    float amax = -INFINITY;
    for (int i = 0; i < 32; ++i) {
      x[i] = load_as_f32(in, dtype, b * 32 + i);
      amax = fmaxf(amax, fabsf(x[i]));
    }
    volatile float t = amax * max_norm_rcp;
    uint8_t e = orc_f32_to_e8m0_rp(t);
    out_sf[b] = e;
    float inv = (e == 0) ? 1.0f : u2f((uint32_t)(254 - (int)e) << 23);
    for (int i = 0; i < 32; ++i) {
      volatile float y = x[i] * inv;
      out_fp8[b * 32 + i] = orc_f32_to_e4m3(y);
    }
  }
}

/* -------------------------------------------------- dequantisation
 * tests/python/direct_utils/narrow_precision.py:16-21,46-106 dequantize_to_dtype:
 * value = e2m1 * e4m3 block scale (un-swizzled) * decode_scale, in fp32. */
ORC_API void orc_dequantize_nvfp4(const uint8_t* fp4, const uint8_t* sf_swizzled, int64_t rows, int64_t cols,
                                  float decode_scale, float* out) {
  int64_t padded = (cols / 16 + 3) / 4 * 4;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint8_t byte = fp4[(r * cols + c) / 2];
      uint8_t code = (c & 1) ? (byte >> 4) : (byte & 15);
      float sf = orc_e4m3_to_f32(sf_swizzled[orc_swizzle_128x4_offset(r, c / 16, padded)]);
      out[r * cols + c] = orc_e2m1_to_f32(code) * sf * decode_scale;
    }
}

/* tests/python/direct/test_cutlass_mxfp8_gemm.py:23-34 dequantize_mxfp8 */
ORC_API void orc_dequantize_mxfp8(const uint8_t* fp8, const uint8_t* sf_swizzled, int64_t rows, int64_t cols,
                                  float* out) {
  int64_t padded = (cols / 32 + 3) / 4 * 4;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      float sf = orc_e8m0_to_f32(sf_swizzled[orc_swizzle_128x4_offset(r, c / 32, padded)]);
      out[r * cols + c] = orc_e4m3_to_f32(fp8[r * cols + c]) * sf;
    }
}

/* bulk helpers so that tests can sweep whole input spaces without Python loops */
ORC_API void orc_f32_to_e2m1_n(const float* x, int64_t n, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_e2m1(x[i]);
}
ORC_API void orc_f32_to_e4m3_n(const float* x, int64_t n, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_e4m3(x[i]);
}
ORC_API void orc_f32_to_e8m0_rp_n(const float* x, int64_t n, uint8_t* out) {
  for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_e8m0_rp(x[i]);
}
