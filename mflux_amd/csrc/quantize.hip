// Group-wise affine quantize / pack and its inverse for gfx950.
//
// quantize: bit-identical to MLX's CPU evaluation of mx.quantize(mode="affine")
// (reached from mflux through nn.quantize,
// src/mflux/models/common/weights/loading/weight_applier.py:43,46,103).
// Every lane owns 8 consecutive elements (one 128-bit load for 16-bit
// types), so a group of GS elements is GS/8 neighbouring lanes of one
// wavefront; group min/max are butterfly reductions over those lanes.  All
// float32 operations are the same IEEE operations, in the same order, as the
// scalar algorithm: true division, round-half-even, no contraction.
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
      float w_min = v[u][0], w_max = v[u][0];
#pragma unroll
      for (int i = 1; i < 8; ++i) {
        w_min = fminf(w_min, v[u][i]);
        w_max = fmaxf(w_max, v[u][i]);
      }
#pragma unroll
      for (int off = 1; off < kLanesPerGroup; off <<= 1) {
        w_min = fminf(w_min, __shfl_xor(w_min, off));
        w_max = fmaxf(w_max, __shfl_xor(w_max, off));
      }
      const bool mask = fabsf(w_min) > fabsf(w_max);
      float scale = (w_max - w_min) / n_bins;
      scale = (scale < kEps) ? kEps : scale;
      scale = mask ? scale : -scale;
      const float edge = mask ? w_min : w_max;
      const float q0 = rintf(edge / scale);
      float bias = 0.0f;
      if (q0 != 0.0f) {
        scale = edge / q0;
        bias = edge;
      }
      uint32_t code[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float q = rintf((v[u][i] - bias) / scale);
        q = (q < 0.0f) ? 0.0f : q;
        q = (n_bins < q) ? n_bins : q;
        code[i] = (uint32_t)q;
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
    for (int i = 0; i < 8; ++i) r[i] = __builtin_fmaf(q[i], s, b);
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

int grid_for(int64_t n_chunks, int per_thread) {
  const int64_t blocks = (n_chunks + 256LL * per_thread - 1) / (256LL * per_thread);
  const int64_t cap = 256 * 8;  // 8 workgroups per CU keeps ~128 KiB of loads in flight per CU
  return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

template <typename T, int GS>
int quantize_bits(const void* w, int64_t n_chunks, int bits, uint32_t* wq, void* scales, void* biases,
                  hipStream_t stream) {
  using S = typename T::storage;
  const int grid = grid_for(n_chunks, kUnroll);
  if (bits == 4) {
    hipLaunchKernelGGL((quantize_kernel<T, GS, 4>), dim3(grid), dim3(256), 0, stream, (const S*)w, wq, (S*)scales,
                       (S*)biases, n_chunks);
  } else {
    hipLaunchKernelGGL((quantize_kernel<T, GS, 8>), dim3(grid), dim3(256), 0, stream, (const S*)w, wq, (S*)scales,
                       (S*)biases, n_chunks);
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
  if (bits == 4) {
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

}  // namespace mfq
