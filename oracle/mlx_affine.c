/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement, in plain C, of MLX's group-wise affine quantization and
 * of its quantized matmul with transposed weights, as reached from mflux
 * through nn.quantize (src/mflux/models/common/weights/loading/
 * weight_applier.py:43,46,103) and through every QuantizedLinear call
 * (e.g. src/mflux/models/flux/model/flux_transformer/
 * single_transformer_block.py:53,57).
 *
 * The arithmetic itself lives in the third-party package `mlx`
 * (pyproject.toml:31-32,69-70 pin mlx 0.30.3 on linux / 0.31.0 on darwin),
 * whose sources are not part of the reference tree.  What is restated here
 * is MLX's published CPU algorithm (mlx/backend/cpu/quantized.cpp:
 * quantize<T,U>, _qmm_t<T,bits,group_size>; mlx/ops.cpp: dequantize,
 * quantized_matmul).  Each point where MLX's back ends are known to differ
 * is isolated in a named macro below so that it can be flipped in one place.
 *
 * PARITY STATUS: the reference holds no golden vector, known-answer test or
 * fixture for these functions and MLX cannot be run here, so
 *   - mlxo_quantize:     "parity unpinned" against MLX for the five numeric
 *                        choices named by the MLXO_* macros; pinned against
 *                        hand-computed known answers, algebraic invariants
 *                        and an independent numpy restatement.
 *   - mlxo_dequantize:   pinned (definition q*s+b; round trips).
 *   - mlxo_qmm_t_*:      pinned as a textbook product x @ dequantize(w)^T
 *                        (checked against float64 numpy.matmul); MLX's
 *                        back-end specific rounding is "parity unpinned".
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this file's library.
 */
#include <immintrin.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ---- numeric choices of MLX's CPU kernel, one name each ---------------- */
/* tie rule of the two roundings: CPU uses std::rint (half to even); the
 * Metal kernel uses round() (half away from zero).                         */
#define MLXO_ROUND(v) rintf(v)
/* lower clamp of the provisional scale                                     */
#define MLXO_EPS 1e-7f
/* codes divide by the float32 scale (true IEEE division, no reciprocal),
 * using scale and bias BEFORE they are cast to the storage type            */
#define MLXO_CODE(e, bias, scale) (((e) - (bias)) / (scale))
/* initial values of the running min / max                                  */
#define MLXO_MIN_INIT INFINITY
#define MLXO_MAX_INIT (-INFINITY)
/* element i of a packed word sits at bit offset i*bits (lowest first)      */
#define MLXO_SHIFT(i, bits) ((i) * (bits))

enum { MLXO_F32 = 0, MLXO_F16 = 1, MLXO_BF16 = 2 };

/* ---- storage-type conversions ------------------------------------------ */
static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* IEEE half <-> float through the F16C instructions (round to nearest even) */
static inline float f16_to_f32(uint16_t h) { return _cvtsh_ss(h); }

static inline uint16_t f32_to_f16(float f) {
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}

static inline float load_as_f32(const void* p, int dtype, size_t i) {
  switch (dtype) {
    case MLXO_F32: return ((const float*)p)[i];
    case MLXO_F16: return f16_to_f32(((const uint16_t*)p)[i]);
    default: return bf16_to_f32(((const uint16_t*)p)[i]);
  }
}

static inline void store_from_f32(void* p, int dtype, size_t i, float v) {
  switch (dtype) {
    case MLXO_F32: ((float*)p)[i] = v; break;
    case MLXO_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
    default: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
  }
}

static int check_args(int dtype, int group_size, int bits) {
  if (dtype < 0 || dtype > 2) return -1;
  if (group_size != 32 && group_size != 64 && group_size != 128) return -2;
  if (bits != 2 && bits != 3 && bits != 4 && bits != 5 && bits != 6 && bits != 8) return -3;
  return 0;
}

/*
 * quantize: follows mlx/backend/cpu/quantized.cpp quantize<T,U> (the CPU
 * evaluation of mx.quantize, mode "affine") statement by statement.
 * w: n_elem values of `dtype`, n_elem % group_size == 0, groups are runs of
 * group_size consecutive elements.  out: n_elem*bits/32 words.
 */
int mlxo_quantize(const void* w, int dtype, size_t n_elem, int group_size,
                  int bits, uint32_t* out, void* scales, void* biases) {
  int rc = check_args(dtype, group_size, bits);
  if (rc) return rc;
  if (n_elem % (size_t)group_size) return -4;
  const float n_bins = (float)((1 << bits) - 1);
  /* MLX packs el_per_pack codes into bytes_per_pack bytes, lowest code in the
   * lowest bits: 32/bits codes per 4 bytes for 2, 4, 8 bits; 8 codes per 3
   * bytes (3 bits), 8 per 5 (5 bits), 4 per 3 (6 bits).                      */
  const int pow2 = (bits & (bits - 1)) == 0;
  const int el_per_pack = pow2 ? 32 / bits : (bits == 6 ? 4 : 8);
  const int bytes_per_pack = pow2 ? 4 : (bits == 5 ? 5 : 3);
  const int packs_per_group = group_size / el_per_pack;
  const size_t n_groups = n_elem / (size_t)group_size;
  uint8_t* out_bytes = (uint8_t*)out;

  /* groups are independent; the thread split changes nothing in the results */
#pragma omp parallel for schedule(static) if (n_groups > 4096)
  for (size_t g = 0; g < n_groups; ++g) {
    const size_t w_idx = g * (size_t)group_size;
    float w_min = MLXO_MIN_INIT;
    float w_max = MLXO_MAX_INIT;
    for (int j = 0; j < group_size; ++j) {
      float e = load_as_f32(w, dtype, w_idx + j);
      w_max = (w_max < e) ? e : w_max; /* std::max(w_max, e) */
      w_min = (e < w_min) ? e : w_min; /* std::min(w_min, e) */
    }
    int mask = fabsf(w_min) > fabsf(w_max);
    float scale = (w_max - w_min) / n_bins;
    scale = (scale < MLXO_EPS) ? MLXO_EPS : scale; /* std::max(., eps) */
    scale = mask ? scale : -scale;
    float edge = mask ? w_min : w_max;
    float q0 = MLXO_ROUND(edge / scale);
    float bias = 0.0f;
    if (q0 != 0.0f) {
      scale = edge / q0;
      bias = edge;
    }
    uint8_t* o = out_bytes + g * (size_t)packs_per_group * bytes_per_pack;
    for (int j = 0; j < packs_per_group; ++j) {
      uint64_t pack = 0;
      for (int k = 0; k < el_per_pack; ++k) {
        float e = load_as_f32(w, dtype, w_idx + (size_t)j * el_per_pack + k);
        float q = MLXO_ROUND(MLXO_CODE(e, bias, scale));
        q = (q < 0.0f) ? 0.0f : q;     /* std::max(q, 0) */
        q = (n_bins < q) ? n_bins : q; /* std::min(q, n_bins) */
        pack |= (uint64_t)q << MLXO_SHIFT(k, bits);
      }
      for (int b = 0; b < bytes_per_pack; ++b) o[j * bytes_per_pack + b] = (uint8_t)(pack >> (8 * b));
    }
    store_from_f32(scales, dtype, g, scale);
    store_from_f32(biases, dtype, g, bias);
  }
  return 0;
}

/* code idx of a buffer: bits [idx*bits, (idx+1)*bits) of its little-endian
 * bit stream (which is what both packing schemes above produce)            */
static inline uint32_t code_at(const uint32_t* wq, size_t idx, int bits) {
  const uint8_t* bytes = (const uint8_t*)wq;
  const size_t bit = idx * (size_t)bits;
  uint32_t window = bytes[bit >> 3];
  if ((bit & 7) + (size_t)bits > 8) window |= (uint32_t)bytes[(bit >> 3) + 1] << 8;
  return (window >> (bit & 7)) & ((1u << bits) - 1u);
}

/*
 * dequantize: w[i] = code[i] * scale[i/gs] + bias[i/gs]  (mlx/ops.cpp
 * dequantize).  Product and sum are each rounded to the storage type, as
 * MLX's element-wise graph does for a bf16/f16 array; for MLXO_F32 output
 * from narrower scales pass out_dtype = MLXO_F32 and the value is the
 * float32 expression with two roundings.
 */
int mlxo_dequantize(const uint32_t* wq, const void* scales, const void* biases,
                    int dtype, size_t n_elem, int group_size, int bits,
                    void* out, int out_dtype) {
  int rc = check_args(dtype, group_size, bits);
  if (rc) return rc;
  if (out_dtype < 0 || out_dtype > 2) return -1;
  for (size_t i = 0; i < n_elem; ++i) {
    float s = load_as_f32(scales, dtype, i / group_size);
    float b = load_as_f32(biases, dtype, i / group_size);
    float q = (float)code_at(wq, i, bits);
    float v;
    if (out_dtype == MLXO_F32) {
      v = q * s;
      v = v + b;
    } else {
      uint32_t tmp[1];
      store_from_f32(tmp, out_dtype, 0, q * s);
      v = load_as_f32(tmp, out_dtype, 0) + b;
    }
    store_from_f32(out, out_dtype, i, v);
  }
  return 0;
}

/*
 * Exact dequantisation into float64: code*scale+bias has at most 8+8 (+1)
 * significant bits for bf16 and 8+11 (+1) for f16 scales, so the float64
 * expression is exact.  This is the operand of the matmul oracle.
 */
int mlxo_dequantize_f64(const uint32_t* wq, const void* scales,
                        const void* biases, int dtype, size_t n_elem,
                        int group_size, int bits, double* out) {
  int rc = check_args(dtype, group_size, bits);
  if (rc) return rc;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n_elem; ++i) {
    double s = (double)load_as_f32(scales, dtype, i / group_size);
    double b = (double)load_as_f32(biases, dtype, i / group_size);
    out[i] = (double)code_at(wq, i, bits) * s + b;
  }
  return 0;
}

/*
 * qmm_t, float32 accumulation: y[m,n] = sum_k x[m,k]*(s[n,g]*q[n,k]+b[n,g])
 * in the loop order of mlx/backend/cpu/quantized.cpp _qmm_t (m, n, group,
 * word, element) with the running sum held in float32, as MLX's
 * _qmm_t_simd path does.  Optional bias[n] is added after the sum has been
 * rounded to y's type, which is what QuantizedLinear.__call__ does with a
 * second element-wise op.  threads <= 0 means all cores; 1 reproduces MLX's
 * single-threaded evaluation.  Used as bench.py's CPU baseline.
 */
int mlxo_qmm_t_f32acc(const void* x, int x_dtype, size_t M, size_t K,
                      const uint32_t* wq, const void* scales,
                      const void* biases, int sb_dtype, const void* bias,
                      size_t N, int group_size, int bits, void* y, int y_dtype,
                      int threads) {
  int rc = check_args(sb_dtype, group_size, bits);
  if (rc) return rc;
  if (bits & (bits - 1)) return -3; /* word-wise loop: 2, 4, 8 bits only */
  if (K % (size_t)group_size) return -4;
  const int el_per_int = 32 / bits;
  const size_t words_per_row = K / el_per_int;
  const size_t groups_per_row = K / group_size;
  const uint32_t bitmask = (1u << bits) - 1u;
#if defined(_OPENMP)
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
#pragma omp parallel for schedule(static) num_threads(threads)
  for (size_t n = 0; n < N; ++n) {
    for (size_t m = 0; m < M; ++m) {
      float sum = 0.0f;
      const uint32_t* wrow = wq + n * words_per_row;
      size_t k = 0;
      for (size_t g = 0; g < groups_per_row; ++g) {
        float s = load_as_f32(scales, sb_dtype, n * groups_per_row + g);
        float b = load_as_f32(biases, sb_dtype, n * groups_per_row + g);
        for (int wi = 0; wi < group_size / el_per_int; ++wi) {
          uint32_t word = *wrow++;
          for (int p = 0; p < el_per_int; ++p, ++k) {
            float xv = load_as_f32(x, x_dtype, m * K + k);
            sum += xv * (s * (float)(word & bitmask) + b);
            word >>= bits;
          }
        }
      }
      if (bias) {
        uint32_t tmp[1];
        float r = sum;
        if (y_dtype != MLXO_F32) {
          store_from_f32(tmp, y_dtype, 0, sum);
          r = load_as_f32(tmp, y_dtype, 0);
        }
        sum = r + load_as_f32(bias, sb_dtype, n);
      }
      store_from_f32(y, y_dtype, m * N + n, sum);
    }
  }
  return 0;
}

/*
 * qmm_t with the running sum held in the storage type T (every partial
 * result rounded to bf16/f16), which is what MLX's generic _qmm_t<T> does
 * where its SIMD width for T is 1 (x86 Linux builds).  Kept to document how
 * far that evaluation strays from exact math; never used as a parity target.
 */
int mlxo_qmm_t_tacc(const void* x, size_t M, size_t K, const uint32_t* wq,
                    const void* scales, const void* biases, int dtype,
                    size_t N, int group_size, int bits, void* y) {
  int rc = check_args(dtype, group_size, bits);
  if (rc) return rc;
  if (bits & (bits - 1)) return -3; /* word-wise loop: 2, 4, 8 bits only */
  if (dtype == MLXO_F32) return -1;
  const int el_per_int = 32 / bits;
  const size_t words_per_row = K / el_per_int;
  const size_t groups_per_row = K / group_size;
  const uint32_t bitmask = (1u << bits) - 1u;
#define RT(v) (store_from_f32(t, dtype, 0, (v)), load_as_f32(t, dtype, 0))
#pragma omp parallel for schedule(static)
  for (size_t n = 0; n < N; ++n) {
    uint32_t t[1];
    for (size_t m = 0; m < M; ++m) {
      float sum = 0.0f;
      const uint32_t* wrow = wq + n * words_per_row;
      size_t k = 0;
      for (size_t g = 0; g < groups_per_row; ++g) {
        float s = load_as_f32(scales, dtype, n * groups_per_row + g);
        float b = load_as_f32(biases, dtype, n * groups_per_row + g);
        for (int wi = 0; wi < group_size / el_per_int; ++wi) {
          uint32_t word = *wrow++;
          for (int p = 0; p < el_per_int; ++p, ++k) {
            float xv = load_as_f32(x, dtype, m * K + k);
            float wv = RT(RT(s * (float)(word & bitmask)) + b);
            sum = RT(sum + RT(xv * wv));
            word >>= bits;
          }
        }
      }
      store_from_f32(y, dtype, m * N + n, sum);
    }
  }
#undef RT
  return 0;
}

int mlxo_num_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
