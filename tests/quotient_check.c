/* CPU check of the four-instruction quotient that the quantize kernels use
 * for scales of ordinary magnitude (quotient<true> in
 * onnx-mlir_amd/csrc/om_kernels.h): with r = RN(1 / s),
 *     q0 = RN(x * r), clamped to +-1024;  e = fma(-q0, s, x);  q = fma(e, r, q0)
 * must equal the IEEE quotient x / s bit for bit wherever the 8-bit result
 * can depend on it (|x / s| from 2^-3 to 2^10, s from 2^-96 to 2^96), and must
 * lead to the same 8-bit value everywhere else.  Prints the number of
 * differences found; test infrastructure only.
 *
 *   usage: quotient_check <random pairs per thread> <scales for the boundary sweep>
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline uint64_t rng(uint64_t *s) { *s ^= *s << 13; *s ^= *s >> 7; *s ^= *s << 17; return *s; }

static inline float fast_quotient(float x, float s, float r) {
  volatile float p = x * r; /* volatile: one rounding, no contraction */
  float q0 = fminf(fmaxf(p, -1024.0f), 1024.0f);
  float e = fmaf(-q0, s, x);
  return fmaf(e, r, q0);
}
/* the 8-bit value both quotients lead to (u8, zero point zp) */
static inline int quantized(float q, float zp) {
  float c = fminf(fmaxf(rintf(q) + zp, 0.0f), 255.0f);
  return (int)c;
}

int main(int argc, char **argv) {
  long long per_thread = argc > 1 ? atoll(argv[1]) : 20000000LL;
  long long scales = argc > 2 ? atoll(argv[2]) : 20000;
  long long bad_bits = 0, bad_q = 0, n = 0;
#pragma omp parallel reduction(+ : bad_bits, bad_q, n)
  {
    int t = 0;
#ifdef _OPENMP
    t = omp_get_thread_num();
#endif
    uint64_t st = 0x9E3779B97F4A7C15ull * (uint64_t)(t + 1);
    /* 1. random significands; quotient magnitudes 2^-3 .. 2^10, scales 2^-96 .. 2^96 */
    for (long long i = 0; i < per_thread; ++i) {
      uint64_t a = rng(&st), b = rng(&st);
      int es = (int)(a % 193) - 96, eq = (int)((a >> 8) % 13) - 3;
      uint32_t ms = (uint32_t)(a >> 20) & 0x7FFFFF, mx = (uint32_t)(b >> 20) & 0x7FFFFF;
      if ((b & 15) == 0) ms = 0x7FFFFF - (uint32_t)(b >> 50 & 3); /* significands of all ones */
      if ((b & 15) == 1) ms = (uint32_t)(b >> 50 & 3);
      if (es == 96) ms = 0;
      float s = u2f(((uint32_t)(es + 127) << 23) | ms);
      float x = u2f(((uint32_t)(es + eq + 127) << 23) | mx | ((uint32_t)(b >> 4 & 1) << 31));
      volatile float r = 1.0f / s;
      float q = x / s, f = fast_quotient(x, s, r);
      if (fabsf(q) <= 1024.0f && f2u(q) != f2u(f)) ++bad_bits;
      if (quantized(q, 77.0f) != quantized(f, 77.0f)) ++bad_q;
      ++n;
    }
    /* 2. any x at all (tiny, huge, infinite, NaN): the 8-bit result must agree */
    for (long long i = 0; i < per_thread / 4; ++i) {
      uint64_t a = rng(&st), b = rng(&st);
      int es = (int)(a % 193) - 96;
      float s = u2f(((uint32_t)(es + 127) << 23) | ((uint32_t)(a >> 20) & 0x7FFFFF));
      if (es == 96) s = 0x1p96f;
      float x = u2f((uint32_t)b);
      volatile float r = 1.0f / s;
      float zp = (float)(a >> 50 & 255);
      if (quantized(x / s, zp) != quantized(fast_quotient(x, s, r), zp)) ++bad_q;
      ++n;
    }
    /* 3. quotients within three ulps of k + 1/2 and of k, |k| <= 600 */
#pragma omp for schedule(static)
    for (long long i = 0; i < scales; ++i) {
      uint64_t a = rng(&st);
      a ^= (uint64_t)i * 0xD1B54A32D192ED03ull;
      int es = (int)(a % 193) - 96;
      uint32_t ms = (uint32_t)(a >> 20) & 0x7FFFFF;
      if ((a & 7) == 0) ms = 0x7FFFFF - (uint32_t)(a >> 50 & 7);
      if (es == 96) ms = 0;
      float s = u2f(((uint32_t)(es + 127) << 23) | ms);
      volatile float r = 1.0f / s;
      for (int k = -1200; k <= 1200; ++k) {
        float h = 0.5f * (float)k;
        uint32_t u = f2u((float)((double)h * (double)s));
        for (int d = -3; d <= 3; ++d) {
          float x = u2f(u + (uint32_t)d);
          float q = x / s, f = fast_quotient(x, s, r);
          if (k != 0 && f2u(q) != f2u(f)) ++bad_bits; /* k = 0: below 2^-3, only the 8-bit result counts */
          if (quantized(q, 131.0f) != quantized(f, 131.0f)) ++bad_q;
          ++n;
        }
      }
    }
  }
  printf("%lld pairs: %lld quotients differ, %lld 8-bit results differ\n", n, bad_bits, bad_q);
  return (bad_bits || bad_q) ? 1 : 0;
}
