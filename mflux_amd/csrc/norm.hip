// LayerNorm without learned parameters followed by the adaLN modulation, the
// step in front of every modulated linear of mflux's DiT blocks:
//   y = LayerNorm(x, eps) * (1 + scale) + shift
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:22,
// ada_layer_norm_zero_single.py:19, ada_layer_norm_continuous.py:21,
// joint_transformer_block.py:86-87: nn.LayerNorm(dims, eps=1e-6, affine=False)
// and three element-wise operations, four passes over [M, K] in the reference).
// One pass here, bound by HBM: one wavefront per row, the row held in
// registers (K up to 8192), mean and variance in float32 by wavefront-wide sums.
// Roundings as the reference's operations round on a 16-bit array: the
// normalised value, 1 + scale, their product, and the sum with the shift are
// each rounded to the type.
#include "common.h"

namespace mfq {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kMaxChunks = 16;  // 16-byte pieces per lane: rows of up to 64 * 16 * 8 = 8192 elements

template <int kCtrl>
__device__ inline float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false));
}
// sum over the 64 lanes, in every lane
__device__ inline float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror: the sum of the lane's row of 16
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
}

// kChunks: 16-byte pieces of the row a lane holds (the last ones may lie past the row's end)
template <typename T, int kChunks>
__global__ __launch_bounds__(256) void layer_norm_modulate_kernel(const uint16_t* __restrict__ x,
                                                                  const uint16_t* __restrict__ scale,
                                                                  const uint16_t* __restrict__ shift,
                                                                  uint16_t* __restrict__ y, int M, int K,
                                                                  int rows_per_vector, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = blockIdx.x * 4 + threadIdx.x / kWave;
  if (row >= M) return;
  const int pieces = K / 8;
  const uint16_t* xr = x + (int64_t)row * K;
  u32x4 v[kChunks];
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int p = c * kWave + lane;
    v[c] = p < pieces ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr) + p) : u32x4{0u, 0u, 0u, 0u};
  }
  // the modulation vectors of this row's batch entry: requested now, used after the statistics
  u32x4 sc[kChunks], sh[kChunks];
  if (scale) {
    const int64_t vec = (int64_t)(row / rows_per_vector) * K;
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
      const int p = min(c * kWave + lane, pieces - 1);
      sc[c] = reinterpret_cast<const u32x4*>(scale + vec)[p];
      sh[c] = reinterpret_cast<const u32x4*>(shift + vec)[p];
    }
  }
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < kChunks; ++c)
#pragma unroll
    for (int i = 0; i < 4; ++i) sum += lo_f32<T>(v[c][i]) + hi_f32<T>(v[c][i]);
  const float mean = wave_sum(sum) / (float)K;
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    if (c * kWave + lane >= pieces) continue;  // the zeros past the row's end are not elements of it
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = lo_f32<T>(v[c][i]) - mean, b = hi_f32<T>(v[c][i]) - mean;
      sq = __builtin_fmaf(a, a, sq);
      sq = __builtin_fmaf(b, b, sq);
    }
  }
  const float rstd = 1.0f / __builtin_sqrtf(wave_sum(sq) / (float)K + eps);
  uint16_t* yr = y + (int64_t)row * K;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int p = c * kWave + lane;
    if (p >= pieces) continue;
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float n0 = T::to_f32(T::from_f32((lo_f32<T>(v[c][i]) - mean) * rstd));
      float n1 = T::to_f32(T::from_f32((hi_f32<T>(v[c][i]) - mean) * rstd));
      if (scale) {
        const float f0 = T::to_f32(T::from_f32(1.0f + lo_f32<T>(sc[c][i])));
        const float f1 = T::to_f32(T::from_f32(1.0f + hi_f32<T>(sc[c][i])));
        n0 = T::to_f32(T::from_f32(n0 * f0)) + lo_f32<T>(sh[c][i]);
        n1 = T::to_f32(T::from_f32(n1 * f1)) + hi_f32<T>(sh[c][i]);
      }
      out[i] = T::pack2(n0, n1);
    }
    reinterpret_cast<u32x4*>(yr)[p] = out;
  }
}

template <typename T, int kChunks>
int launch_chunks(int n_chunks, const void* x, int64_t M, int64_t K, const void* scale, const void* shift,
                  int64_t rows_per_vector, float eps, void* y, hipStream_t stream) {
  if (n_chunks == kChunks) {
    hipLaunchKernelGGL((layer_norm_modulate_kernel<T, kChunks>), dim3((unsigned)((M + 3) / 4)), dim3(256), 0, stream,
                       (const uint16_t*)x, (const uint16_t*)scale, (const uint16_t*)shift, (uint16_t*)y, (int)M,
                       (int)K, (int)rows_per_vector, eps);
    return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
  }
  if constexpr (kChunks < kMaxChunks)
    return launch_chunks<T, kChunks * 2>(n_chunks, x, M, K, scale, shift, rows_per_vector, eps, y, stream);
  return MFQ_EUNSUPPORTED;
}

}  // namespace

int launch_layer_norm_modulate(const void* x, int dtype, int64_t M, int64_t K, const void* scale, const void* shift,
                               int64_t rows_per_vector, float eps, void* y, hipStream_t stream) {
  if (K % 8 || K > 64 * 8 * kMaxChunks) return MFQ_EUNSUPPORTED;
  int n = 1;  // pieces per lane, rounded up to a power of two (1, 2, 4, 8, 16)
  while (n * 64 * 8 < K) n *= 2;
  if (dtype == MFQ_BF16) return launch_chunks<BF16, 1>(n, x, M, K, scale, shift, rows_per_vector, eps, y, stream);
  if (dtype == MFQ_F16) return launch_chunks<F16, 1>(n, x, M, K, scale, shift, rows_per_vector, eps, y, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
