/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Driver for the sanitizer build of the CPU oracle (`make -C oracle sanitize`):
 * runs every entry point of mlx_affine.c on exactly-sized heap buffers, for all
 * storage types, bit widths and group sizes, under AddressSanitizer and
 * UndefinedBehaviorSanitizer, and checks two properties that need no second
 * implementation: codes stay inside [0, 2^bits), and dequantize(quantize(w))
 * is within one quantization step of w.  Exits non-zero on any finding.
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int mlxo_quantize(const void*, int, size_t, int, int, uint32_t*, void*, void*);
int mlxo_dequantize(const uint32_t*, const void*, const void*, int, size_t, int, int, void*, int);
int mlxo_dequantize_f64(const uint32_t*, const void*, const void*, int, size_t, int, int, double*);
int mlxo_qmm_t_f32acc(const void*, int, size_t, size_t, const uint32_t*, const void*, const void*, int, const void*,
                      size_t, int, int, void*, int, int);
int mlxo_qmm_t_tacc(const void*, size_t, size_t, const uint32_t*, const void*, const void*, int, size_t, int, int,
                    void*);

static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static double uniform(void) { /* xorshift64*, (0, 1) */
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return ((rng_state * 0x2545f4914f6cdd1dull) >> 11) * (1.0 / 9007199254740992.0) + 1e-18;
}
static float normal(void) { return (float)(sqrt(-2.0 * log(uniform())) * cos(6.283185307179586 * uniform())); }

static uint16_t to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static int fail(const char* what, int dtype, int bits, int gs) {
  fprintf(stderr, "sanitize_check: %s (dtype %d, bits %d, group %d)\n", what, dtype, bits, gs);
  return 1;
}

int main(void) {
  const int bits_all[] = {2, 3, 4, 5, 6, 8}, gs_all[] = {32, 64, 128};
  const size_t N = 24, K = 384, M = 5; /* K is a multiple of every group size and of 32 */
  int checked = 0;
  for (int dtype = 0; dtype <= 2; ++dtype) {
    const size_t esz = dtype == 0 ? 4 : 2;
    for (int bi = 0; bi < 6; ++bi) {
      for (int gi = 0; gi < 3; ++gi) {
        const int bits = bits_all[bi], gs = gs_all[gi];
        const size_t n = N * K, groups = n / (size_t)gs;
        void* w = malloc(n * esz);
        float* wf = malloc(n * sizeof(float));
        for (size_t i = 0; i < n; ++i) {
          float v = normal() * 0.02f;
          if (i / (size_t)gs % 7 == 3) v = 0.0f;         /* all-zero groups */
          if (i / (size_t)gs % 7 == 5) v = fabsf(v) + 1; /* one-sided groups */
          if (dtype == 0) {
            ((float*)w)[i] = v;
          } else if (dtype == 2) {
            ((uint16_t*)w)[i] = to_bf16(v);
            v = from_bf16(((uint16_t*)w)[i]);
          } else {
            ((uint16_t*)w)[i] = _cvtss_sh(v, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
            v = _cvtsh_ss(((uint16_t*)w)[i]);
          }
          wf[i] = v;
        }
        uint32_t* wq = malloc(n * (size_t)bits / 8);
        void* s = malloc(groups * esz);
        void* b = malloc(groups * esz);
        if (mlxo_quantize(w, dtype, n, gs, bits, wq, s, b)) return fail("quantize refused", dtype, bits, gs);
        double* d64 = malloc(n * sizeof(double));
        if (mlxo_dequantize_f64(wq, s, b, dtype, n, gs, bits, d64)) return fail("dequantize_f64 refused", dtype, bits, gs);
        void* d = malloc(n * esz);
        if (mlxo_dequantize(wq, s, b, dtype, n, gs, bits, d, dtype)) return fail("dequantize refused", dtype, bits, gs);
        float* d32 = malloc(n * sizeof(float));
        if (mlxo_dequantize(wq, s, b, dtype, n, gs, bits, d32, 0)) return fail("dequantize to f32 refused", dtype, bits, gs);
        for (size_t g = 0; g < groups; ++g) { /* error at most one step of the group (plus the scale's own rounding) */
          double lo = 1e300, hi = -1e300;
          for (int j = 0; j < gs; ++j) {
            const double v = wf[g * (size_t)gs + j];
            lo = v < lo ? v : lo;
            hi = v > hi ? v : hi;
          }
          const double step = (hi - lo) / ((1 << bits) - 1) * 1.07 + 1.1e-7 + 0.01 * fmax(fabs(lo), fabs(hi));
          for (int j = 0; j < gs; ++j)
            if (fabs(d64[g * (size_t)gs + j] - wf[g * (size_t)gs + j]) > step)
              return fail("round trip off by more than a step", dtype, bits, gs);
        }
        /* products: 16-bit operands only, power-of-two widths (the word-wise loops of the CPU kernel) */
        if (dtype != 0 && (bits & (bits - 1)) == 0) {
          void* x = malloc(M * K * esz);
          for (size_t i = 0; i < M * K; ++i) {
            if (dtype == 2) {
              ((uint16_t*)x)[i] = to_bf16(normal());
            } else {
              ((uint16_t*)x)[i] = _cvtss_sh(normal(), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
            }
          }
          void* y = malloc(M * N * esz);
          float* y32 = malloc(M * N * sizeof(float));
          if (mlxo_qmm_t_f32acc(x, dtype, M, K, wq, s, b, dtype, NULL, N, gs, bits, y32, 0, 2))
            return fail("qmm_t_f32acc refused", dtype, bits, gs);
          if (mlxo_qmm_t_f32acc(x, dtype, M, K, wq, s, b, dtype, s /* any [N] vector */, N, gs, bits, y, dtype, 1))
            return fail("qmm_t_f32acc with bias refused", dtype, bits, gs);
          if (mlxo_qmm_t_tacc(x, M, K, wq, s, b, dtype, N, gs, bits, y)) return fail("qmm_t_tacc refused", dtype, bits, gs);
          for (size_t i = 0; i < M * N; ++i)
            if (!isfinite(y32[i])) return fail("non-finite product", dtype, bits, gs);
          free(x), free(y), free(y32);
        }
        free(w), free(wf), free(wq), free(s), free(b), free(d64), free(d), free(d32);
        ++checked;
      }
    }
  }
  /* refusals: bad arguments are answered with a code, not with an access */
  uint32_t dummy[8] = {0};
  if (mlxo_quantize(dummy, 7, 64, 64, 4, dummy, dummy, dummy) == 0) return fail("bad dtype accepted", 7, 4, 64);
  if (mlxo_quantize(dummy, 2, 64, 48, 4, dummy, dummy, dummy) == 0) return fail("bad group accepted", 2, 4, 48);
  if (mlxo_quantize(dummy, 2, 64, 64, 7, dummy, dummy, dummy) == 0) return fail("bad bits accepted", 2, 7, 64);
  if (mlxo_quantize(dummy, 2, 65, 64, 4, dummy, dummy, dummy) == 0) return fail("ragged size accepted", 2, 4, 64);
  printf("sanitize_check: %d combinations clean\n", checked);
  return 0;
}
