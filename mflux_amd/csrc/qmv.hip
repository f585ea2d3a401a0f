// Small-M (M <= 16) quantized matvec for gfx950: y = x @ dequant(W)^T (+ bias).
//
// This is the adaLN modulation shape of every DiT block in mflux
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12,
// src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37):
// one or a few activation rows against a wide weight, so the kernel is bound
// by streaming the packed weight from HBM once.
//
// A workgroup of four wavefronts owns 16 output features and walks K in
// phases.  Every lane streams 128-bit pieces of "its" weight row
// (row = lane % 16), dequantises them in registers with one float32 fma per
// code, and feeds them to the 16x16x32 matrix core as the A operand; the B
// operand is the matching slice of x (column = lane % 16 = activation row,
// zero beyond M), so all M <= 16 rows come at the cost of one.  The order of k
// inside the product is permuted consistently for both operands, which a dot
// product does not notice.  x is staged through LDS one phase ahead and the
// weight loads of phase p+1 are issued before the arithmetic of phase p, so a
// wavefront always has two phases of HBM reads in flight.  The four
// wavefronts split each phase and combine their float32 sums through LDS.
#include "common.h"

namespace mfq {
namespace {

constexpr int kRowsPerBlock = 16;
constexpr int kWavesPerBlock = 4;
constexpr int kUnroll = 4;  // 128-bit weight loads per lane and phase

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ inline typename T::vec8 as_vec8(u32x4 v) {
  return __builtin_bit_cast(typename T::vec8, v);
}

template <typename T, int GS, int BITS>
struct Phase {
  static constexpr int kCodesPerLoad = 128 / BITS;         // codes in one 128-bit load
  static constexpr int kStepsPerLoad = kCodesPerLoad / 8;  // matrix-core steps fed by one load
  static constexpr int kChunk = 4 * kCodesPerLoad;         // k covered by one wavefront-wide load
  static constexpr int kPhase = kWavesPerBlock * kUnroll * kChunk;  // k covered by one phase
  static constexpr int kRowBytes = kPhase * 2 + 16;        // x tile row in LDS, padded

  static constexpr int kGroups = kPhase / GS;              // groups per row and phase
  static constexpr int kXTileOffset = 2 * kRowsPerBlock * kGroups * 2;  // scales + biases tiles come first

  u32x4 wv[kUnroll];

  // k of the first code this lane holds in load u of phase p
  __device__ static inline int k_of(int p, int wave, int u, int q) {
    return p * kPhase + (wave * kUnroll + u) * kChunk + q * kCodesPerLoad;
  }

  __device__ inline void issue(const u32x4* wrow, int p, int wave, int q, int K) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int k = k_of(p, wave, u, q);
      if (k < K) {
        wv[u] = __builtin_nontemporal_load(wrow + k / kCodesPerLoad);
      } else {  // past the end of the row: any codes against zero x
        wv[u] = u32x4{0, 0, 0, 0};
      }
    }
  }
};

// Copies the scales and biases of 16 rows for phase p into LDS as
// [2][16][kGroups] 16-bit values (zero past the end of a row), one element per
// thread and pass, so that neighbouring threads read neighbouring addresses.
template <int kGroups>
__device__ inline void stage_sb(const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases, char* tile,
                                int p, int n0, int N, int groups) {
  uint16_t* out = reinterpret_cast<uint16_t*>(tile);
  for (int i = threadIdx.x; i < 2 * kRowsPerBlock * kGroups; i += blockDim.x) {
    const int which = i / (kRowsPerBlock * kGroups);
    const int rem = i - which * (kRowsPerBlock * kGroups);
    const int row = rem / kGroups;
    const int g = p * kGroups + (rem - row * kGroups);
    const int n = min(n0 + row, N - 1);
    uint16_t v = 0;
    if (g < groups) v = (which ? biases : scales)[(int64_t)n * groups + g];
    out[i] = v;
  }
}

// Copies x[0:M, p*kPhase : (p+1)*kPhase] (zero past K) into an LDS tile.
template <int kPhase, int kRowBytes>
__device__ inline void stage_x(const uint16_t* __restrict__ x, char* tile, int p, int M, int K) {
  constexpr int kPieces = kPhase / 8;  // 16-byte pieces per row
  for (int i = threadIdx.x; i < M * kPieces; i += blockDim.x) {
    const int m = i / kPieces;
    const int piece = i - m * kPieces;
    const int k = p * kPhase + piece * 8;
    u32x4 v = {0, 0, 0, 0};
    if (k < K) v = *reinterpret_cast<const u32x4*>(x + (int64_t)m * K + k);
    *reinterpret_cast<u32x4*>(tile + m * kRowBytes + piece * 16) = v;
  }
}

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void qmv_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                  const uint16_t* __restrict__ scales,
                                                  const uint16_t* __restrict__ biases,
                                                  const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                  int y_is_f32, int M, int N, int K) {
  using P = Phase<T, GS, BITS>;
  extern __shared__ __attribute__((aligned(16))) char lds[];  // two x tiles of M rows each
  __shared__ float red[kWavesPerBlock][kRowsPerBlock][kRowsPerBlock + 1];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int r = lane & 15;   // weight row within the tile / activation row
  const int q = lane >> 4;   // quarter of the chunk this lane streams
  const int n0 = blockIdx.x * kRowsPerBlock;
  const int n = min(n0 + r, N - 1);  // rows past N are clamped for loads, never stored
  const int groups = K / GS;
  const int tile_bytes = P::kXTileOffset + M * P::kRowBytes;  // scales, biases, then M rows of x

  const u32x4* wrow = reinterpret_cast<const u32x4*>(wq + (int64_t)n * (K * BITS / 32));
  const bool x_lane = r < M;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const int n_phases = (K + P::kPhase - 1) / P::kPhase;

  P cur, nxt;
  stage_sb<P::kGroups>(scales, biases, lds, 0, n0, N, groups);
  stage_x<P::kPhase, P::kRowBytes>(x, lds + P::kXTileOffset, 0, M, K);
  cur.issue(wrow, 0, wave, q, K);
  __syncthreads();

  // One phase: prefetch phase p+1 into `next`, then consume `now`.  Called with
  // the two register sets alternating so that no copy forces an early wait.
  auto phase = [&](int p, const P& now, P& next) {
    const char* tile = lds + (p & 1) * tile_bytes;
    if (p + 1 < n_phases) {
      // staging loads first, weights second: the LDS stores then wait for the staging loads only
      char* next_tile = lds + ((p + 1) & 1) * tile_bytes;
      stage_sb<P::kGroups>(scales, biases, next_tile, p + 1, n0, N, groups);
      stage_x<P::kPhase, P::kRowBytes>(x, next_tile + P::kXTileOffset, p + 1, M, K);
      next.issue(wrow, p + 1, wave, q, K);
    }
    const uint16_t* sb = reinterpret_cast<const uint16_t*>(tile);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int k_tile = (wave * kUnroll + u) * P::kChunk + q * P::kCodesPerLoad;  // k inside the phase
      const float sc = T::to_f32(sb[r * P::kGroups + k_tile / GS]);
      const float bi = T::to_f32(sb[(kRowsPerBlock + r) * P::kGroups + k_tile / GS]);
#pragma unroll
      for (int j = 0; j < P::kStepsPerLoad; ++j) {
        u32x4 xf = {0, 0, 0, 0};
        if (x_lane)
          xf = *reinterpret_cast<const u32x4*>(tile + P::kXTileOffset + r * P::kRowBytes + (k_tile + 8 * j) * 2);
        uint4 wf;
        if constexpr (BITS == 4) {
          wf = dequant8_w4<T>(now.wv[u][j], sc, bi);
        } else {
          wf = dequant8_w8<T>(now.wv[u][2 * j], now.wv[u][2 * j + 1], sc, bi);
        }
        acc = mfma16(__builtin_bit_cast(typename T::vec8, wf), as_vec8<T>(xf), acc);
      }
    }
    __syncthreads();
  };
  for (int p = 0; p < n_phases; p += 2) {
    phase(p, cur, nxt);
    if (p + 1 < n_phases) phase(p + 1, nxt, cur);
  }

  // acc[i] is the partial sum for feature n0 + 4*q + i and activation row r.
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

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  using P = Phase<T, GS, BITS>;
  auto kernel = qmv_kernel<T, GS, BITS>;
  const size_t lds_bytes = 2 * ((size_t)P::kXTileOffset + (size_t)M * P::kRowBytes);
  static bool configured = false;
  if (!configured) {
    // largest request: M = 16 rows of a 4-bit phase (2048 k), double buffered, about 140 KiB
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            2 * (P::kXTileOffset + 16 * P::kRowBytes)) != hipSuccess)
      return MFQ_ELAUNCH;
    configured = true;
  }
  const dim3 grid((unsigned)((N + kRowsPerBlock - 1) / kRowsPerBlock));
  hipLaunchKernelGGL(kernel, grid, dim3(256), lds_bytes, stream, (const uint16_t*)x, wq, (const uint16_t*)scales,
                     (const uint16_t*)biases, (const uint16_t*)bias, y, (int)(y_dtype == MFQ_F32), (int)M, (int)N,
                     (int)K);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int GS>
int launch_bits(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int bits, void* y, int y_dtype, hipStream_t stream) {
  if (bits == 4) return launch_one<T, GS, 4>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
  return launch_one<T, GS, 8>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
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
