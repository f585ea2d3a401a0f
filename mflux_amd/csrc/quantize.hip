// Group-wise affine quantize / pack and its inverse for gfx950.
//
// quantize: bit-identical to MLX's CPU evaluation of mx.quantize(mode="affine")
// (reached from mflux through nn.quantize,
// src/mflux/models/common/weights/loading/weight_applier.py:43,46,103).
// Two kernels.  16-bit inputs (the weights of every model) use
// quantize_group_per_lane_kernel, described at its definition.  float32 inputs
// use quantize_kernel: every lane owns 8 consecutive elements, so a group of GS
// elements is GS/8 neighbouring lanes of one
// wavefront; group min/max are butterfly reductions over those lanes (DPP
// lane moves).  All float32 operations produce the same values, in the same
// order, as the scalar algorithm: correctly rounded division,
// round-half-even, no contraction.
//
// HBM-bound: 2 bytes read and bits/8 + 4/GS bytes written per element.
#include "common.h"

namespace mfq {
namespace {

constexpr int kUnroll = 4;
constexpr float kEps = 1e-7f;

template <typename T>
__device__ inline void load8(const typename T::storage* w, int64_t chunk, float (&v)[8]) {
  const uint4 raw = reinterpret_cast<const uint4*>(w)[chunk];
  v[0] = lo_f32<T>(raw.x); v[1] = hi_f32<T>(raw.x);
  v[2] = lo_f32<T>(raw.y); v[3] = hi_f32<T>(raw.y);
  v[4] = lo_f32<T>(raw.z); v[5] = hi_f32<T>(raw.z);
  v[6] = lo_f32<T>(raw.w); v[7] = hi_f32<T>(raw.w);
}

template <>
__device__ inline void load8<F32>(const float* w, int64_t chunk, float (&v)[8]) {
  const float4 a = reinterpret_cast<const float4*>(w)[2 * chunk];
  const float4 b = reinterpret_cast<const float4*>(w)[2 * chunk + 1];
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// ---- exact float32 division with a shared reciprocal ----------------------
// The compiler's correctly rounded a / d is: scale the operands into a safe
// range (v_div_scale), r = rcp(d) refined once, a quotient refined twice with
// fused multiply-adds, undo the scaling (v_div_fmas) and patch special values
// (v_div_fixup).  When d is a normal number away from the ends of the exponent
// range, the quotient is not going to be subnormal and a is not tiny, neither
// operand is scaled and nothing is patched: the result IS the chain of fused
// multiply-adds below.  A group of 64 elements divides by the same scale 64
// times, so the reciprocal is computed once and each element costs five
// operations instead of eleven.
struct Divisor {
  float d, r;
  __device__ inline explicit Divisor(float den) : d(den) {
    const float r0 = __builtin_amdgcn_rcpf(den);
    r = __builtin_fmaf(__builtin_fmaf(-den, r0, 1.0f), r0, r0);
  }
  __device__ inline float divide(float n) const {
    float q = n * r;
    q = __builtin_fmaf(__builtin_fmaf(-d, q, n), r, q);
    return __builtin_fmaf(__builtin_fmaf(-d, q, n), r, q);
  }
};

__device__ inline uint32_t exponent_field(float f) { return (__float_as_uint(f) >> 23) & 0xffu; }

// Lane exchange inside a row of 16 lanes without going through LDS.
template <int kCtrl>
__device__ inline float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;      // lane i <- lane 15-i of its row

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void quantize_kernel(const typename T::storage* __restrict__ w,
                                                       uint32_t* __restrict__ wq,
                                                       typename T::storage* __restrict__ scales,
                                                       typename T::storage* __restrict__ biases,
                                                       int64_t n_chunks) {
  constexpr int kLanesPerGroup = GS / 8;
  constexpr float n_bins = (float)((1 << BITS) - 1);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const Divisor by_bins(n_bins);

  // The trip count is the same for every lane of a wavefront, and a group is
  // either wholly inside n_chunks or wholly outside, so the cross-lane
  // exchanges below only ever pair lanes that hold real data.
  for (int64_t c0 = first; c0 - lane < n_chunks; c0 += stride * kUnroll) {
    float v[kUnroll][8];
    bool ok[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * stride;
      ok[u] = c < n_chunks;
      if (ok[u]) {
        load8<T>(w, c, v[u]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[u][i] = 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * stride;
      float w_min = fminf(fminf(v[u][0], v[u][1]), v[u][2]);
      float w_max = fmaxf(fmaxf(v[u][0], v[u][1]), v[u][2]);
      w_min = fminf(fminf(w_min, v[u][3]), v[u][4]);
      w_max = fmaxf(fmaxf(w_max, v[u][3]), v[u][4]);
      w_min = fminf(fminf(w_min, v[u][5]), fminf(v[u][6], v[u][7]));
      w_max = fmaxf(fmaxf(w_max, v[u][5]), fmaxf(v[u][6], v[u][7]));
      w_min = fminf(w_min, dpp<kDppXor1>(w_min));
      w_max = fmaxf(w_max, dpp<kDppXor1>(w_max));
      w_min = fminf(w_min, dpp<kDppXor2>(w_min));
      w_max = fmaxf(w_max, dpp<kDppXor2>(w_max));
      if constexpr (kLanesPerGroup >= 8) {
        w_min = fminf(w_min, dpp<kDppHalfMirror>(w_min));
        w_max = fmaxf(w_max, dpp<kDppHalfMirror>(w_max));
      }
      if constexpr (kLanesPerGroup >= 16) {
        w_min = fminf(w_min, dpp<kDppMirror>(w_min));
        w_max = fmaxf(w_max, dpp<kDppMirror>(w_max));
      }
      const bool mask = fabsf(w_min) > fabsf(w_max);
      const float range = w_max - w_min;
      const float edge = mask ? w_min : w_max;
      // Every division below has a divisor and a dividend well inside the
      // normal range, and a quotient that is neither huge nor able to round to
      // a nonzero code while being subnormal, exactly when the range and the
      // edge are: range in [2^-63, 2^63], edge likewise and within 2^40 of the
      // range.  (Two distinct floats differ by at least 2^-24 of the larger,
      // so real data never fails the last test.)
      const uint32_t er = exponent_field(range), ee = exponent_field(edge);
      const bool tame = (er - 64u) <= 126u && (ee - 64u) <= 126u && ee <= er + 40u;
      float scale, bias = 0.0f;
      uint32_t code[8];
      if (tame) {
        scale = by_bins.divide(range);
        scale = (scale < kEps) ? kEps : scale;
        scale = mask ? scale : -scale;
        const float q0 = rintf(Divisor(scale).divide(edge));
        if (q0 != 0.0f) {
          scale = Divisor(q0).divide(edge);
          bias = edge;
        }
        const Divisor by_scale(scale);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float q = rintf(by_scale.divide(v[u][i] - bias));
          q = (q < 0.0f) ? 0.0f : q;
          q = (n_bins < q) ? n_bins : q;
          code[i] = (uint32_t)q;
        }
      } else {
        scale = range / n_bins;
        scale = (scale < kEps) ? kEps : scale;
        scale = mask ? scale : -scale;
        const float q0 = rintf(edge / scale);
        if (q0 != 0.0f) {
          scale = edge / q0;
          bias = edge;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float q = rintf((v[u][i] - bias) / scale);
          q = (q < 0.0f) ? 0.0f : q;
          q = (n_bins < q) ? n_bins : q;
          code[i] = (uint32_t)q;
        }
      }
      if (ok[u]) {
        if constexpr (BITS == 4) {
          uint32_t word = 0;
#pragma unroll
          for (int i = 0; i < 8; ++i) word |= code[i] << (4 * i);
          wq[c] = word;
        } else {
          uint2 words;
          words.x = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
          words.y = code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24);
          reinterpret_cast<uint2*>(wq)[c] = words;
        }
        if ((lane & (kLanesPerGroup - 1)) == 0) {
          scales[c / kLanesPerGroup] = T::from_f32(scale);
          biases[c / kLanesPerGroup] = T::from_f32(bias);
        }
      }
    }
  }
}

// 16-bit inputs: one lane quantizes one whole group.
//
// A wavefront takes 64 consecutive groups (64 * GS elements, contiguous in
// memory) per iteration: GS/8 coalesced 128-bit loads per lane, a transpose
// through a wavefront-private LDS region so that lane l ends up holding group
// l, then min/max, scale, bias and codes entirely inside the lane.  The
// per-group work (three divisions, the reciprocal of the scale) is then done
// once per group instead of once per 8 elements, no cross-lane reduction is
// needed, and scales/biases leave as 128 contiguous bytes per wavefront.
// LDS slots are XOR-swizzled so that both the row-wise writes and the
// group-wise reads touch every bank once per 16 lanes.
template <int kChunks>
__device__ inline int stage_slot(int group, int chunk) {
  // 64 banks of 4 bytes: 16 consecutive lanes must cover one 256-byte window.
  // 8 or 16 pieces per group: two groups / one group per window, XOR with bits
  // 1..3 of the group; 4 pieces per group: four groups per window, bits 2..3.
  const int f = kChunks >= 8 ? ((group >> 1) & 7) : ((group >> 2) & (kChunks - 1));
  return group * kChunks + (chunk ^ f);
}

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void quantize_group_per_lane_kernel(const uint16_t* __restrict__ w,
                                                                      uint32_t* __restrict__ wq,
                                                                      uint16_t* __restrict__ scales,
                                                                      uint16_t* __restrict__ biases,
                                                                      int64_t n_groups) {
  constexpr int kChunks = GS / 8;                 // 16-byte pieces per group
  constexpr int kWords = GS * BITS / 32;          // packed words per group
  constexpr float n_bins = (float)((1 << BITS) - 1);
  __shared__ uint4 stage_all[4][kWave * kChunks];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  uint4* stage = stage_all[wave];
  const uint4* w16 = reinterpret_cast<const uint4*>(w);
  const int64_t n_chunks = n_groups * kChunks;
  const int64_t wave_stride = (int64_t)gridDim.x * 4 * kWave;  // groups between a wavefront's iterations
  const Divisor by_bins(n_bins);

  const int64_t g_first = ((int64_t)blockIdx.x * 4 + wave) * kWave;
  // The codes of the wavefront's 64 groups are 256 kWords contiguous bytes.  Stored from the lane that made them
  // (4 kWords bytes each), every store instruction would touch every cache line of that range; they go
  // through the wavefront's LDS region once more instead, so that a store instruction writes 1 KiB of
  // consecutive memory.  That pays from 64 bytes of codes per group on (kWords % 16 == 0: 4.6 us of 42 at 8
  // bits and groups of 64); below, the direct stores are as fast or faster.
  auto store_groups = [&](int64_t g0, const uint32_t (&words)[kWords], float scale, float bias) __attribute__((always_inline)) {
    const int64_t g = g0 + lane;
    if constexpr (kWords % 16 == 0) {
      uint4* mine = stage + lane * (kWords / 4);
#pragma unroll
      for (int k = 0; k < kWords / 4; ++k)
        mine[k] = make_uint4(words[4 * k], words[4 * k + 1], words[4 * k + 2], words[4 * k + 3]);
      uint4* out = reinterpret_cast<uint4*>(wq + g0 * kWords);
      const int64_t pieces = (n_groups - g0 < kWave ? n_groups - g0 : kWave) * (kWords / 4);
#pragma unroll
      for (int k = 0; k < kWords / 4; ++k) {
        const uint4 v = stage[k * kWave + lane];
        if (k * kWave + lane < pieces) out[k * kWave + lane] = v;
      }
    } else if (g < n_groups) {
      uint32_t* out = wq + g * kWords;  // 4 * kWords bytes per group: the widest store that stays aligned
      if constexpr (kWords % 4 == 0) {
#pragma unroll
        for (int k = 0; k < kWords / 4; ++k)
          reinterpret_cast<uint4*>(out)[k] = make_uint4(words[4 * k], words[4 * k + 1], words[4 * k + 2], words[4 * k + 3]);
      } else if constexpr (kWords % 2 == 0) {
#pragma unroll
        for (int k = 0; k < kWords / 2; ++k) reinterpret_cast<uint2*>(out)[k] = make_uint2(words[2 * k], words[2 * k + 1]);
      } else {
#pragma unroll
        for (int k = 0; k < kWords; ++k) out[k] = words[k];
      }
    }
    if (g < n_groups) {
      scales[g] = T::from_f32(scale);
      biases[g] = T::from_f32(bias);
    }
  };
  for (int64_t g0 = g_first; g0 < n_groups; g0 += wave_stride) {
    uint4 raw[kChunks];
    // pieces past the end re-read the last one (no branch around a load): their groups are never stored
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int64_t c = g0 * kChunks + j * kWave + lane;
      raw[j] = w16[c < n_chunks ? c : n_chunks - 1];
    }
#pragma unroll
    for (int j = 0; j < kChunks; ++j) {
      const int slot = j * kWave + lane;
      stage[stage_slot<kChunks>(slot / kChunks, slot % kChunks)] = raw[j];
    }
    // the region is private to the wavefront and LDS operations of one
    // wavefront complete in order, so no barrier is needed
#pragma unroll
    for (int i = 0; i < kChunks; ++i) raw[i] = stage[stage_slot<kChunks>(lane, i)];

    auto element = [&](int i, int e) -> float {
      const uint32_t pair = e < 2 ? raw[i].x : e < 4 ? raw[i].y : e < 6 ? raw[i].z : raw[i].w;
      return (e & 1) ? hi_f32<T>(pair) : lo_f32<T>(pair);
    };
    float w_min = element(0, 0), w_max = w_min;
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
#pragma unroll
      for (int e = (i == 0 ? 1 : 0); e < 8; ++e) {
        const float x = element(i, e);
        w_min = fminf(w_min, x);
        w_max = fmaxf(w_max, x);
      }
    }
    const bool mask = fabsf(w_min) > fabsf(w_max);
    const float range = w_max - w_min;
    const float edge = mask ? w_min : w_max;
    const uint32_t er = exponent_field(range), ee = exponent_field(edge);
    const bool tame = (er - 64u) <= 126u && (ee - 64u) <= 126u && ee <= er + 40u;  // see quantize_kernel
    float scale, bias = 0.0f;
    // The group's codes form one little-endian bit stream, code i at bit
    // i*BITS: for 4 and 8 bits that is "element i of a word at bit i*BITS", for
    // 3, 5 and 6 bits it is MLX's 3- and 5-byte packs laid end to end.  The
    // loops are fully unrolled, so every shift and index below is a constant.
    uint32_t words[kWords];
    uint64_t stream = 0;
    int stream_bits = 0, n_words = 0;
    // code[e]: integral values in [0, n_bins].  4 and 8 bits go to bytes with one instruction each (even and odd
    // codes of a 4-bit word in two registers, joined by one shift-or); the other widths through the bit stream.
    auto pack = [&](int i, const float (&code)[8]) __attribute__((always_inline)) {
      if constexpr (BITS == 8 || BITS == 4) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo = __builtin_amdgcn_cvt_pk_u8_f32(code[BITS == 8 ? e : 2 * e], e, lo);
          hi = __builtin_amdgcn_cvt_pk_u8_f32(code[BITS == 8 ? 4 + e : 2 * e + 1], e, hi);
        }
        if constexpr (BITS == 8) {
          words[2 * i] = lo;
          words[2 * i + 1] = hi;
        } else {
          words[i] = lo | (hi << 4);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          stream |= (uint64_t)(uint32_t)code[e] << stream_bits;
          stream_bits += BITS;
          if (stream_bits >= 32) {
            words[n_words++] = (uint32_t)stream;
            stream >>= 32;
            stream_bits -= 32;
          }
        }
      }
    };
    if (tame) {
      scale = by_bins.divide(range);
      scale = (scale < kEps) ? kEps : scale;
      scale = mask ? scale : -scale;
      const float q0 = rintf(Divisor(scale).divide(edge));
      if (q0 != 0.0f) {
        scale = Divisor(q0).divide(edge);
        bias = edge;
      }
      const Divisor by_scale(scale);
#pragma unroll
      for (int i = 0; i < kChunks; ++i) {
        float code[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float q = rintf(by_scale.divide(element(i, e) - bias));
          code[e] = __builtin_amdgcn_fmed3f(q, 0.0f, n_bins);
        }
        pack(i, code);
      }
    } else {
      scale = range / n_bins;
      scale = (scale < kEps) ? kEps : scale;
      scale = mask ? scale : -scale;
      const float q0 = rintf(edge / scale);
      if (q0 != 0.0f) {
        scale = edge / q0;
        bias = edge;
      }
#pragma unroll
      for (int i = 0; i < kChunks; ++i) {
        float code[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float q = rintf((element(i, e) - bias) / scale);
          q = (q < 0.0f) ? 0.0f : q;
          q = (n_bins < q) ? n_bins : q;
          code[e] = (float)(uint32_t)q;  // (a NaN becomes code 0 here)
        }
        pack(i, code);
      }
    }
    store_groups(g0, words, scale, bias);
  }
}

// float32 input at 3, 5 and 6 bits (a checkpoint kept in float32 and mflux's -q 3/5/6,
// src/mflux/cli/defaults/defaults.py:63): one lane per group, which it reads twice -- for its limits, then for
// its codes, the second time out of the caches -- so that no more than eight values live in registers at a
// time; the arithmetic is the scalar algorithm statement by statement (exact divisions), the codes leave as the
// group's little-endian bit stream, scales and biases as float32.  A pass over weights this wide is rare (the
// models' weights arrive in 16 bits), so nothing here is tuned: each lane's loads are its own 4 GS bytes.
template <int GS, int BITS>
__global__ __launch_bounds__(256) void quantize_f32_stream_kernel(const float* __restrict__ w,
                                                                  uint32_t* __restrict__ wq,
                                                                  float* __restrict__ scales,
                                                                  float* __restrict__ biases, int64_t n_groups) {
  constexpr int kWords = GS * BITS / 32;
  constexpr float n_bins = (float)((1 << BITS) - 1);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_groups; g += stride) {
    const float4* src = reinterpret_cast<const float4*>(w + g * GS);
    float w_min = src[0].x, w_max = w_min;
#pragma unroll 4
    for (int i = 0; i < GS / 4; ++i) {
      const float4 v = src[i];
      w_min = fminf(fminf(fminf(w_min, v.x), fminf(v.y, v.z)), v.w);
      w_max = fmaxf(fmaxf(fmaxf(w_max, v.x), fmaxf(v.y, v.z)), v.w);
    }
    const bool mask = fabsf(w_min) > fabsf(w_max);
    const float edge = mask ? w_min : w_max;
    float scale = (w_max - w_min) / n_bins, bias = 0.0f;
    scale = (scale < kEps) ? kEps : scale;
    scale = mask ? scale : -scale;
    const float q0 = rintf(edge / scale);
    if (q0 != 0.0f) {
      scale = edge / q0;
      bias = edge;
    }
    uint32_t* out = wq + g * kWords;
    uint64_t stream = 0;
    int stream_bits = 0, n_words = 0;
#pragma unroll
    for (int i = 0; i < GS / 4; ++i) {
      const float4 v = src[i];
      const float x[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float q = rintf((x[e] - bias) / scale);
        q = (q < 0.0f) ? 0.0f : q;
        q = (n_bins < q) ? n_bins : q;
        stream |= (uint64_t)(uint32_t)q << stream_bits;  // (a NaN becomes code 0 here)
        stream_bits += BITS;
        if (stream_bits >= 32) {
          out[n_words++] = (uint32_t)stream;
          stream >>= 32;
          stream_bits -= 32;
        }
      }
    }
    scales[g] = scale;
    biases[g] = bias;
  }
}

// code * scale + bias as mx.dequantize evaluates it: an element-wise multiply and
// an element-wise add on arrays of the output type, so the product is rounded
// to that type before the bias is added and the sum is rounded again by the
// store (float32 output: the two float32 operations, never fused).  The matmul
// kernels do not go through this; they round fma(code, scale, bias) once.
template <typename TO>
__device__ inline float dequant_value(float q, float s, float b) {
  float p = q * s;
  if constexpr (sizeof(typename TO::storage) == 2) p = TO::to_f32(TO::from_f32(p));
  return p + b;
}

template <typename TS, typename TO, int GS, int BITS>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t* __restrict__ wq,
                                                         const typename TS::storage* __restrict__ scales,
                                                         const typename TS::storage* __restrict__ biases,
                                                         typename TO::storage* __restrict__ out,
                                                         int64_t n_chunks) {
  constexpr int kLanesPerGroup = GS / 8;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < n_chunks; c += stride) {
    const float s = TS::to_f32(scales[c / kLanesPerGroup]);
    const float b = TS::to_f32(biases[c / kLanesPerGroup]);
    float q[8];
    if constexpr (BITS == 4) {
      const uint32_t word = wq[c];
#pragma unroll
      for (int i = 0; i < 8; ++i) q[i] = (float)((word >> (4 * i)) & 0xfu);
    } else {
      const uint2 words = reinterpret_cast<const uint2*>(wq)[c];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        q[i] = ubyte_f32(words.x, i);
        q[4 + i] = ubyte_f32(words.y, i);
      }
    }
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = dequant_value<TO>(q[i], s, b);
    if constexpr (sizeof(typename TO::storage) == 2) {
      uint4 o;
      o.x = TO::pack2(r[0], r[1]);
      o.y = TO::pack2(r[2], r[3]);
      o.z = TO::pack2(r[4], r[5]);
      o.w = TO::pack2(r[6], r[7]);
      reinterpret_cast<uint4*>(out)[c] = o;
    } else {
      reinterpret_cast<float4*>(out)[2 * c] = make_float4(r[0], r[1], r[2], r[3]);
      reinterpret_cast<float4*>(out)[2 * c + 1] = make_float4(r[4], r[5], r[6], r[7]);
    }
  }
}

// Row gather + dequantize: out[i, :] = dequantize(row idx[i] of the packed
// matrix), the body of a quantized embedding lookup
// (src/mflux/models/flux/model/flux_text_encoder/t5_encoder/t5_encoder.py:11
// becomes a QuantizedEmbedding under the default predicate).  One workgroup per
// looked-up row.  Indices are wrapped once if negative and clamped into
// [0, n_rows): a bad index reads a valid row instead of faulting.
template <typename TS, typename TO, int GS, int BITS>
__global__ __launch_bounds__(256) void dequantize_rows_kernel(const uint32_t* __restrict__ wq,
                                                              const typename TS::storage* __restrict__ scales,
                                                              const typename TS::storage* __restrict__ biases,
                                                              const int64_t* __restrict__ idx, int64_t n_rows,
                                                              int chunks_per_row,
                                                              typename TO::storage* __restrict__ out) {
  constexpr int kLanesPerGroup = GS / 8;
  int64_t row = idx[blockIdx.x];
  if (row < 0) row += n_rows;
  row = row < 0 ? 0 : (row >= n_rows ? n_rows - 1 : row);
  const int64_t src0 = row * chunks_per_row, dst0 = (int64_t)blockIdx.x * chunks_per_row;
  for (int c = threadIdx.x; c < chunks_per_row; c += blockDim.x) {
    const int64_t cs = src0 + c;
    const float s = TS::to_f32(scales[cs / kLanesPerGroup]);
    const float b = TS::to_f32(biases[cs / kLanesPerGroup]);
    float q[8];
    if constexpr (BITS == 4) {
      const uint32_t word = wq[cs];
#pragma unroll
      for (int i = 0; i < 8; ++i) q[i] = (float)((word >> (4 * i)) & 0xfu);
    } else {
      const uint2 words = reinterpret_cast<const uint2*>(wq)[cs];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        q[i] = ubyte_f32(words.x, i);
        q[4 + i] = ubyte_f32(words.y, i);
      }
    }
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = dequant_value<TO>(q[i], s, b);
    const int64_t cd = dst0 + c;
    if constexpr (sizeof(typename TO::storage) == 2) {
      uint4 o;
      o.x = TO::pack2(r[0], r[1]);
      o.y = TO::pack2(r[2], r[3]);
      o.z = TO::pack2(r[4], r[5]);
      o.w = TO::pack2(r[6], r[7]);
      reinterpret_cast<uint4*>(out)[cd] = o;
    } else {
      reinterpret_cast<float4*>(out)[2 * cd] = make_float4(r[0], r[1], r[2], r[3]);
      reinterpret_cast<float4*>(out)[2 * cd + 1] = make_float4(r[4], r[5], r[6], r[7]);
    }
  }
}

// 3-, 5- and 6-bit codes: a thread takes 32 consecutive elements, which are
// BITS whole words of the row's bit stream, and unpacks them with constant
// shifts.  idx == nullptr: plain dequantize over n_units units; otherwise unit
// u of looked-up row blockIdx.y comes from row idx[blockIdx.y] (see
// dequantize_rows_kernel).
template <typename TS, typename TO, int GS, int BITS>
__global__ __launch_bounds__(256) void dequantize_stream_kernel(const uint32_t* __restrict__ wq,
                                                                const typename TS::storage* __restrict__ scales,
                                                                const typename TS::storage* __restrict__ biases,
                                                                const int64_t* __restrict__ idx, int64_t n_rows,
                                                                int64_t units_per_row, int64_t n_units,
                                                                typename TO::storage* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < n_units; u += stride) {
    int64_t src = u, dst = u;
    if (idx) {
      int64_t row = idx[blockIdx.y];
      if (row < 0) row += n_rows;
      row = row < 0 ? 0 : (row >= n_rows ? n_rows - 1 : row);
      src = row * units_per_row + u;
      dst = (int64_t)blockIdx.y * units_per_row + u;
    }
    const float s = TS::to_f32(scales[src * 32 / GS]);
    const float b = TS::to_f32(biases[src * 32 / GS]);
    uint32_t w[BITS + 1];
#pragma unroll
    for (int i = 0; i < BITS; ++i) w[i] = wq[src * BITS + i];
    w[BITS] = 0;
    float r[32];
#pragma unroll
    for (int e = 0; e < 32; ++e) {
      const int bit = e * BITS, word = bit / 32, sh = bit % 32;
      uint32_t code = w[word] >> sh;
      if (sh + BITS > 32) code |= w[word + 1] << (32 - sh);
      r[e] = dequant_value<TO>((float)(code & ((1u << BITS) - 1u)), s, b);
    }
    if constexpr (sizeof(typename TO::storage) == 2) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        uint4 o;
        o.x = TO::pack2(r[8 * k], r[8 * k + 1]);
        o.y = TO::pack2(r[8 * k + 2], r[8 * k + 3]);
        o.z = TO::pack2(r[8 * k + 4], r[8 * k + 5]);
        o.w = TO::pack2(r[8 * k + 6], r[8 * k + 7]);
        reinterpret_cast<uint4*>(out)[4 * dst + k] = o;
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        reinterpret_cast<float4*>(out)[8 * dst + k] = make_float4(r[4 * k], r[4 * k + 1], r[4 * k + 2], r[4 * k + 3]);
    }
  }
}

int grid_for(int64_t n_chunks, int per_thread) {
  const int64_t blocks = (n_chunks + 256LL * per_thread - 1) / (256LL * per_thread);
  const int64_t cap = 256 * 8;  // 8 workgroups per CU keeps ~128 KiB of loads in flight per CU
  return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

template <typename T, int GS>
int quantize_bits(const void* w, int64_t n_chunks, int bits, uint32_t* wq, void* scales, void* biases,
                  hipStream_t stream) {
  using S = typename T::storage;
  if constexpr (sizeof(S) == 2) {
    const int64_t n_groups = n_chunks / (GS / 8);
    // A wavefront takes 64 groups per trip.  At most 256 * 4 workgroups of four wavefronts are resident at
    // once on 256 CUs; beyond that every wavefront makes the same number of trips (fewer wavefronts rather than
    // a last round that only some of them run).
    const int64_t wave_trips = (n_groups + kWave - 1) / kWave;
    const int64_t cap_waves = 256 * 4 * 4;
    const int64_t trips = (wave_trips + cap_waves - 1) / cap_waves;
    const int64_t waves = (wave_trips + trips - 1) / trips;
    const int grid = (int)((waves + 3) / 4);
    auto launch = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, stream, (const S*)w, wq, (S*)scales, (S*)biases, n_groups);
    };
    switch (bits) {
      case 3: launch(quantize_group_per_lane_kernel<T, GS, 3>); break;
      case 4: launch(quantize_group_per_lane_kernel<T, GS, 4>); break;
      case 5: launch(quantize_group_per_lane_kernel<T, GS, 5>); break;
      case 6: launch(quantize_group_per_lane_kernel<T, GS, 6>); break;
      default: launch(quantize_group_per_lane_kernel<T, GS, 8>); break;
    }
  } else {
    const int grid = grid_for(n_chunks, kUnroll);
    if (bits == 3 || bits == 5 || bits == 6) {
      const int64_t n_groups = n_chunks / (GS / 8);
      const int g = grid_for(n_groups, 1);
      auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(g), dim3(256), 0, stream, (const float*)w, wq, (float*)scales, (float*)biases,
                           n_groups);
      };
      if (bits == 3) launch(quantize_f32_stream_kernel<GS, 3>);
      if (bits == 5) launch(quantize_f32_stream_kernel<GS, 5>);
      if (bits == 6) launch(quantize_f32_stream_kernel<GS, 6>);
    } else if (bits == 4) {
      hipLaunchKernelGGL((quantize_kernel<T, GS, 4>), dim3(grid), dim3(256), 0, stream, (const S*)w, wq, (S*)scales,
                         (S*)biases, n_chunks);
    } else {
      hipLaunchKernelGGL((quantize_kernel<T, GS, 8>), dim3(grid), dim3(256), 0, stream, (const S*)w, wq, (S*)scales,
                         (S*)biases, n_chunks);
    }
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T>
int quantize_gs(const void* w, int64_t n_chunks, int gs, int bits, uint32_t* wq, void* scales, void* biases,
                hipStream_t stream) {
  switch (gs) {
    case 32: return quantize_bits<T, 32>(w, n_chunks, bits, wq, scales, biases, stream);
    case 64: return quantize_bits<T, 64>(w, n_chunks, bits, wq, scales, biases, stream);
    default: return quantize_bits<T, 128>(w, n_chunks, bits, wq, scales, biases, stream);
  }
}

template <typename TS, typename TO, int GS>
int dequantize_bits(const uint32_t* wq, const void* scales, const void* biases, int64_t n_chunks, int bits,
                    void* out, hipStream_t stream) {
  using SS = typename TS::storage;
  using SO = typename TO::storage;
  const int grid = grid_for(n_chunks, 1);
  if (bits == 3 || bits == 5 || bits == 6) {
    const int64_t n_units = n_chunks / 4;  // 32 elements each
    const int g = grid_for(n_units, 1);
    auto launch = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(g), dim3(256), 0, stream, wq, (const SS*)scales, (const SS*)biases,
                         (const int64_t*)nullptr, (int64_t)0, (int64_t)0, n_units, (SO*)out);
    };
    if (bits == 3) launch(dequantize_stream_kernel<TS, TO, GS, 3>);
    if (bits == 5) launch(dequantize_stream_kernel<TS, TO, GS, 5>);
    if (bits == 6) launch(dequantize_stream_kernel<TS, TO, GS, 6>);
  } else if (bits == 4) {
    hipLaunchKernelGGL((dequantize_kernel<TS, TO, GS, 4>), dim3(grid), dim3(256), 0, stream, wq, (const SS*)scales,
                       (const SS*)biases, (SO*)out, n_chunks);
  } else {
    hipLaunchKernelGGL((dequantize_kernel<TS, TO, GS, 8>), dim3(grid), dim3(256), 0, stream, wq, (const SS*)scales,
                       (const SS*)biases, (SO*)out, n_chunks);
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename TS, typename TO>
int dequantize_gs(const uint32_t* wq, const void* scales, const void* biases, int64_t n_chunks, int gs, int bits,
                  void* out, hipStream_t stream) {
  switch (gs) {
    case 32: return dequantize_bits<TS, TO, 32>(wq, scales, biases, n_chunks, bits, out, stream);
    case 64: return dequantize_bits<TS, TO, 64>(wq, scales, biases, n_chunks, bits, out, stream);
    default: return dequantize_bits<TS, TO, 128>(wq, scales, biases, n_chunks, bits, out, stream);
  }
}

template <typename TS, typename TO, int GS>
int dequantize_rows_bits(const uint32_t* wq, const void* scales, const void* biases, const int64_t* idx, int64_t n_idx,
                         int64_t n_rows, int chunks_per_row, int bits, void* out, hipStream_t stream) {
  using SS = typename TS::storage;
  using SO = typename TO::storage;
  if (bits == 3 || bits == 5 || bits == 6) {
    if (n_idx > 65535) return MFQ_EUNSUPPORTED;  // looked-up rows ride on gridDim.y
    const int64_t upr = chunks_per_row / 4;
    const dim3 g((unsigned)((upr + 255) / 256), (unsigned)n_idx);
    auto launch = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, g, dim3(256), 0, stream, wq, (const SS*)scales, (const SS*)biases, idx, n_rows, upr,
                         upr, (SO*)out);
    };
    if (bits == 3) launch(dequantize_stream_kernel<TS, TO, GS, 3>);
    if (bits == 5) launch(dequantize_stream_kernel<TS, TO, GS, 5>);
    if (bits == 6) launch(dequantize_stream_kernel<TS, TO, GS, 6>);
  } else if (bits == 4) {
    hipLaunchKernelGGL((dequantize_rows_kernel<TS, TO, GS, 4>), dim3((unsigned)n_idx), dim3(256), 0, stream, wq,
                       (const SS*)scales, (const SS*)biases, idx, n_rows, chunks_per_row, (SO*)out);
  } else {
    hipLaunchKernelGGL((dequantize_rows_kernel<TS, TO, GS, 8>), dim3((unsigned)n_idx), dim3(256), 0, stream, wq,
                       (const SS*)scales, (const SS*)biases, idx, n_rows, chunks_per_row, (SO*)out);
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename TS, typename TO>
int dequantize_rows_gs(const uint32_t* wq, const void* scales, const void* biases, const int64_t* idx, int64_t n_idx,
                       int64_t n_rows, int chunks_per_row, int gs, int bits, void* out, hipStream_t stream) {
  switch (gs) {
    case 32:
      return dequantize_rows_bits<TS, TO, 32>(wq, scales, biases, idx, n_idx, n_rows, chunks_per_row, bits, out, stream);
    case 64:
      return dequantize_rows_bits<TS, TO, 64>(wq, scales, biases, idx, n_idx, n_rows, chunks_per_row, bits, out, stream);
    default:
      return dequantize_rows_bits<TS, TO, 128>(wq, scales, biases, idx, n_idx, n_rows, chunks_per_row, bits, out,
                                               stream);
  }
}

}  // namespace

int launch_quantize(const void* w, int dtype, int64_t rows, int64_t K, int gs, int bits, uint32_t* wq, void* scales,
                    void* biases, hipStream_t stream) {
  const int64_t n_chunks = rows * K / 8;
  switch (dtype) {
    case MFQ_BF16: return quantize_gs<BF16>(w, n_chunks, gs, bits, wq, scales, biases, stream);
    case MFQ_F16: return quantize_gs<F16>(w, n_chunks, gs, bits, wq, scales, biases, stream);
    case MFQ_F32: return quantize_gs<F32>(w, n_chunks, gs, bits, wq, scales, biases, stream);
    default: return MFQ_EDTYPE;
  }
}

int launch_dequantize(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype, int64_t rows,
                      int64_t K, int gs, int bits, void* out, int out_dtype, hipStream_t stream) {
  const int64_t n_chunks = rows * K / 8;
  if (sb_dtype == MFQ_BF16 && out_dtype == MFQ_BF16)
    return dequantize_gs<BF16, BF16>(wq, scales, biases, n_chunks, gs, bits, out, stream);
  if (sb_dtype == MFQ_BF16 && out_dtype == MFQ_F32)
    return dequantize_gs<BF16, F32>(wq, scales, biases, n_chunks, gs, bits, out, stream);
  if (sb_dtype == MFQ_F16 && out_dtype == MFQ_F16)
    return dequantize_gs<F16, F16>(wq, scales, biases, n_chunks, gs, bits, out, stream);
  if (sb_dtype == MFQ_F16 && out_dtype == MFQ_F32)
    return dequantize_gs<F16, F32>(wq, scales, biases, n_chunks, gs, bits, out, stream);
  if (sb_dtype == MFQ_F32 && out_dtype == MFQ_F32)
    return dequantize_gs<F32, F32>(wq, scales, biases, n_chunks, gs, bits, out, stream);
  return MFQ_EUNSUPPORTED;
}

int launch_dequantize_rows(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype,
                           const int64_t* idx, int64_t n_idx, int64_t n_rows, int64_t K, int gs, int bits, void* out,
                           int out_dtype, hipStream_t stream) {
  const int cpr = (int)(K / 8);
  if (sb_dtype == MFQ_BF16 && out_dtype == MFQ_BF16)
    return dequantize_rows_gs<BF16, BF16>(wq, scales, biases, idx, n_idx, n_rows, cpr, gs, bits, out, stream);
  if (sb_dtype == MFQ_BF16 && out_dtype == MFQ_F32)
    return dequantize_rows_gs<BF16, F32>(wq, scales, biases, idx, n_idx, n_rows, cpr, gs, bits, out, stream);
  if (sb_dtype == MFQ_F16 && out_dtype == MFQ_F16)
    return dequantize_rows_gs<F16, F16>(wq, scales, biases, idx, n_idx, n_rows, cpr, gs, bits, out, stream);
  if (sb_dtype == MFQ_F16 && out_dtype == MFQ_F32)
    return dequantize_rows_gs<F16, F32>(wq, scales, biases, idx, n_idx, n_rows, cpr, gs, bits, out, stream);
  if (sb_dtype == MFQ_F32 && out_dtype == MFQ_F32)
    return dequantize_rows_gs<F32, F32>(wq, scales, biases, idx, n_idx, n_rows, cpr, gs, bits, out, stream);
  return MFQ_EUNSUPPORTED;
}

}  // namespace mfq
