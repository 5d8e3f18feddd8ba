/* Exhaustive check of the quantizer's "amax / 6" shortcut (fuser_amd/csrc/quantize.hip, fast_div6): a
 * multiplication by RN(1/6) followed by one fused residual correction,
 *     q0 = m * r6;  q = fma(fma(-6, q0, m), r6, q0),
 * must equal the correctly rounded quotient m / 6.0f of runtime/block_quantization_kernels.cu:224 for every
 * fp32 m with biased exponent in [lo, hi] (argv).  fmaf is the IEEE fused multiply-add on both CPU and GPU, so
 * the CPU proves the GPU's arithmetic.  Prints "mismatches <n> first <hex>" and exits 0 iff n == 0. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

int main(int argc, char** argv) {
  const uint32_t lo = argc > 1 ? (uint32_t)atoi(argv[1]) : 2, hi = argc > 2 ? (uint32_t)atoi(argv[2]) : 250;
  const float r6 = 0x1.555556p-3f;
  uint64_t bad = 0;
  uint32_t first = 0xffffffffu;
  for (uint32_t e = lo; e <= hi; ++e)
    for (uint32_t mant = 0; mant < (1u << 23); ++mant) {
      const uint32_t bits = (e << 23) | mant;
      const float m = u2f(bits);
      const float q0 = m * r6;
      const float q = fmaf(fmaf(-6.0f, q0, m), r6, q0);
      if (f2u(q) != f2u(m / 6.0f)) {
        ++bad;
        if (bits < first) first = bits;
      }
    }
  printf("mismatches %llu first %08x\n", (unsigned long long)bad, first);
  return bad != 0;
}
