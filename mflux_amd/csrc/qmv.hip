// Small-M (M <= 16) quantized matvec for gfx950: y = x @ dequant(W)^T (+ bias).
//
// This is the adaLN modulation shape of every DiT block in mflux
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12,
// src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37):
// one or a few activation rows against a wide weight, so the kernel is bound
// by streaming the packed weight from HBM once.
//
// A workgroup of four wavefronts owns 16 output features.  Every lane streams
// 128-bit pieces of "its" weight row (row = lane % 16), dequantises them in
// registers with one float32 fma per code, and feeds them to the 16x16x32
// matrix core as the A operand; the B operand is the matching slice of x
// (column = lane % 16 = activation row, zero beyond M), so all M <= 16 rows
// come at the cost of one.  The order of k inside the product is permuted
// consistently for both operands, which a dot product does not notice.  The
// four wavefronts split K and combine their float32 partial sums through LDS.
#include "common.h"

namespace mfq {
namespace {

constexpr int kRowsPerBlock = 16;
constexpr int kWavesPerBlock = 4;
constexpr int kChunkUnroll = 4;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ inline typename T::vec8 as_vec8(uint4 v) {
  return __builtin_bit_cast(typename T::vec8, v);
}

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void qmv_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                  const uint16_t* __restrict__ scales,
                                                  const uint16_t* __restrict__ biases,
                                                  const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                  int y_is_f32, int M, int N, int K) {
  constexpr int kCodesPerLoad = 128 / BITS;          // codes in one 128-bit load
  constexpr int kStepsPerLoad = kCodesPerLoad / 8;   // matrix-core steps fed by one load
  constexpr int kChunk = 4 * kCodesPerLoad;          // k covered by one wavefront-wide load

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int r = lane & 15;   // weight row within the tile / activation row
  const int q = lane >> 4;   // quarter of the chunk this lane streams
  const int n0 = blockIdx.x * kRowsPerBlock;
  const int n = min(n0 + r, N - 1);  // rows past N are clamped for loads, never stored
  const int groups = K / GS;

  const u32x4* wrow = reinterpret_cast<const u32x4*>(wq + (int64_t)n * (K * BITS / 32));
  const uint16_t* srow = scales + (int64_t)n * groups;
  const uint16_t* brow = biases + (int64_t)n * groups;
  const bool x_lane = r < M;
  const uint16_t* xrow = x + (int64_t)(x_lane ? r : 0) * K;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const int n_chunks = (K + kChunk - 1) / kChunk;

  for (int c0 = wave; c0 < n_chunks; c0 += kWavesPerBlock * kChunkUnroll) {
    u32x4 wv[kChunkUnroll];
    float s[kChunkUnroll], b[kChunkUnroll];
    int k_lane[kChunkUnroll];
    bool ok[kChunkUnroll];
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const int c = c0 + u * kWavesPerBlock;
      k_lane[u] = c * kChunk + q * kCodesPerLoad;
      ok[u] = k_lane[u] < K;
      if (ok[u]) {
        wv[u] = __builtin_nontemporal_load(wrow + k_lane[u] / kCodesPerLoad);
        s[u] = T::to_f32(srow[k_lane[u] / GS]);
        b[u] = T::to_f32(brow[k_lane[u] / GS]);
      } else {
        wv[u] = u32x4{0, 0, 0, 0};
        s[u] = 0.f;
        b[u] = 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < kChunkUnroll; ++u) {
      const uint32_t words[4] = {wv[u][0], wv[u][1], wv[u][2], wv[u][3]};
#pragma unroll
      for (int j = 0; j < kStepsPerLoad; ++j) {
        uint4 xf = make_uint4(0, 0, 0, 0);
        if (x_lane && ok[u]) xf = *reinterpret_cast<const uint4*>(xrow + k_lane[u] + 8 * j);
        uint4 wf;
        if constexpr (BITS == 4) {
          wf = dequant8_w4<T>(words[j], s[u], b[u]);
        } else {
          wf = dequant8_w8<T>(words[2 * j], words[2 * j + 1], s[u], b[u]);
        }
        acc = mfma16(as_vec8<T>(wf), as_vec8<T>(xf), acc);
      }
    }
  }

  // acc[i] is the partial sum for feature n0 + 4*q + i and activation row r.
  __shared__ float red[kWavesPerBlock][kRowsPerBlock][kRowsPerBlock + 1];
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave][r][4 * q + i] = acc[i];
  __syncthreads();

  const int m = threadIdx.x >> 4;
  const int f = threadIdx.x & 15;
  if (m < M && n0 + f < N) {
    float sum = red[0][m][f] + red[1][m][f] + red[2][m][f] + red[3][m][f];
    const int64_t o = (int64_t)m * N + n0 + f;
    if (y_is_f32) {
      if (bias) sum += T::to_f32(bias[n0 + f]);
      reinterpret_cast<float*>(y)[o] = sum;
    } else {
      uint16_t h = T::from_f32(sum);
      if (bias) h = T::from_f32(T::to_f32(h) + T::to_f32(bias[n0 + f]));
      reinterpret_cast<uint16_t*>(y)[o] = h;
    }
  }
}

template <typename T, int GS>
int launch_bits(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int bits, void* y, int y_dtype, hipStream_t stream) {
  const dim3 grid((unsigned)((N + kRowsPerBlock - 1) / kRowsPerBlock));
  const int y_is_f32 = y_dtype == MFQ_F32;
  if (bits == 4) {
    hipLaunchKernelGGL((qmv_kernel<T, GS, 4>), grid, dim3(256), 0, stream, (const uint16_t*)x, wq,
                       (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y, y_is_f32, (int)M,
                       (int)N, (int)K);
  } else {
    hipLaunchKernelGGL((qmv_kernel<T, GS, 8>), grid, dim3(256), 0, stream, (const uint16_t*)x, wq,
                       (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y, y_is_f32, (int)M,
                       (int)N, (int)K);
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T>
int launch_gs(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
              const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  switch (gs) {
    case 32: return launch_bits<T, 32>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, stream);
    case 64: return launch_bits<T, 64>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, stream);
    default: return launch_bits<T, 128>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, stream);
  }
}

}  // namespace

int launch_qmv(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               hipStream_t stream) {
  if (M > kRowsPerBlock) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16) return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
