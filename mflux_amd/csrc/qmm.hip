// Large-M W4/W8 x A16 quantized matmul for gfx950:
//   y[M, N] = x[M, K] @ dequant(wq[N, K])^T (+ bias)
// the body of every QuantizedLinear call of mflux's diffusion transformers
// (e.g. src/mflux/models/flux/model/flux_transformer/
// single_transformer_block.py:53,57 at M = 4608).
//
// One workgroup of four wavefronts computes a 256 x 256 tile of y, each
// wavefront a 128 x 128 quadrant held as 4 x 4 accumulators of the 32x32x16
// matrix-core instruction.  Per 64-wide k step:
//   - x rows go HBM -> registers -> LDS as they are (128-bit moves);
//   - packed weights go HBM -> registers with 128-bit loads (thread t owns
//     weight row t of the tile), are dequantised with one float32 fma per code
//     (single rounding to the 16-bit type) and written to LDS as a second
//     16-bit tile, so the dequantisation cost is paid once per workgroup and
//     reused by 256 rows of x;
//   - global loads for step i+1 are issued before the matrix work of step i
//     and two LDS buffers alternate, so there is one barrier per step.
// LDS rows are 128 bytes; the 16-byte column index is XORed with row%8 so both
// the row-wise writes and the 32-row fragment reads are bank-conflict free.
#include "common.h"

namespace mfq {
namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;           // one 16-bit tile: 32 KiB
constexpr int kLdsBytes = 4 * kTileBytes;         // x and w tiles, double buffered

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ inline int swz(int row, int chunk) { return row * (BK * 2) + ((chunk ^ (row & 7)) << 4); }

template <typename T>
__device__ inline typename T::vec8 lds_frag(const char* tile, int row, int chunk) {
  return *reinterpret_cast<const typename T::vec8*>(tile + swz(row, chunk));
}

template <typename T, int GS, int BITS>
struct Loader {
  static constexpr int kWLoads = BK * BITS / 128;  // 128-bit loads per weight row per step (2 or 4)
  static constexpr int kGroupsPerStep = (BK + GS - 1) / GS;

  u32x4 xa[8];
  u32x4 wv[kWLoads];
  float s[kGroupsPerStep], b[kGroupsPerStep];

  __device__ inline void issue(const uint16_t* x, const uint32_t* wq, const uint16_t* scales, const uint16_t* biases,
                               int m0, int n0, int M, int N, int K, int k0) {
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = min(m0 + (t >> 3) + 32 * i, M - 1);
      xa[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)row * K + k0 + 8 * (t & 7));
    }
    const int n = min(n0 + t, N - 1);
    const u32x4* wrow = reinterpret_cast<const u32x4*>(wq + (int64_t)n * (K * BITS / 32) + k0 * BITS / 32);
#pragma unroll
    for (int i = 0; i < kWLoads; ++i) wv[i] = wrow[i];
    const int64_t g0 = (int64_t)n * (K / GS) + k0 / GS;
#pragma unroll
    for (int g = 0; g < kGroupsPerStep; ++g) {
      s[g] = T::to_f32(scales[g0 + g]);
      b[g] = T::to_f32(biases[g0 + g]);
    }
  }

  __device__ inline void commit(char* xs, char* ws) const {
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (t >> 3) + 32 * i;
      *reinterpret_cast<u32x4*>(xs + swz(row, t & 7)) = xa[i];
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {  // chunk c = codes 8c .. 8c+7 of this thread's weight row
      const int g = (c * 8) / GS;  // 0 unless GS == 32
      uint4 d;
      if constexpr (BITS == 4) {
        d = dequant8_w4<T>(wv[c >> 2][c & 3], s[g], b[g]);
      } else {
        d = dequant8_w8<T>(wv[c >> 1][(c & 1) * 2], wv[c >> 1][(c & 1) * 2 + 1], s[g], b[g]);
      }
      *reinterpret_cast<uint4*>(ws + swz(t, c)) = d;
    }
  }
};

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void qmm_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of tiles so that neighbours in the run (same weight columns, adjacent
  // x rows) share that XCD's L2.
  const int n_tiles = tiles_m * tiles_n;
  int tile = blockIdx.x;
  {
    const int per_xcd = n_tiles / 8;
    if (tile < per_xcd * 8) tile = (tile & 7) * per_xcd + (tile >> 3);
  }
  const int tm = tile % tiles_m;
  const int tn = tile / tiles_m;
  const int m0 = tm * BM;
  const int n0 = tn * BN;

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int wm = (wave >> 1) * 128;
  const int wn = (wave & 1) * 128;
  const int r = lane & 31;
  const int h = lane >> 5;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  Loader<T, GS, BITS> ld;
  const int steps = K / BK;
  ld.issue(x, wq, scales, biases, m0, n0, M, N, K, 0);
  ld.commit(lds, lds + 2 * kTileBytes);
  __syncthreads();

  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    const char* xs = lds + cur * kTileBytes;
    const char* ws = lds + (2 + cur) * kTileBytes;
    const bool more = step + 1 < steps;
    if (more) ld.issue(x, wq, scales, biases, m0, n0, M, N, K, (step + 1) * BK);

#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      typename T::vec8 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = lds_frag<T>(xs, wm + 32 * i + r, 2 * kk + h);
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = lds_frag<T>(ws, wn + 32 * j + r, 2 * kk + h);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mfma32(af[i], bf[j], acc[i][j]);
    }

    if (more) ld.commit(lds + (cur ^ 1) * kTileBytes, lds + (2 + (cur ^ 1)) * kTileBytes);
    __syncthreads();
  }

  // Epilogue: register e of an accumulator is row 8*(e/4) + 4*h + e%4, column r.
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = n0 + wn + 32 * j + r;
    if (col >= N) continue;
    const float bv = bias ? T::to_f32(bias[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row >= M) continue;
        const int64_t o = (int64_t)row * N + col;
        const float v = acc[i][j][e];
        if (y_is_f32) {
          reinterpret_cast<float*>(y)[o] = bias ? v + bv : v;
        } else {
          uint16_t hv = T::from_f32(v);
          if (bias) hv = T::from_f32(T::to_f32(hv) + bv);
          reinterpret_cast<uint16_t*>(y)[o] = hv;
        }
      }
    }
  }
}

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmm_kernel<T, GS, BITS>;
  static bool configured = false;  // raising the dynamic LDS limit is a per-function, per-process setting
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
      return MFQ_ELAUNCH;
    configured = true;
  }
  const int tiles_m = (int)((M + BM - 1) / BM);
  const int tiles_n = (int)((N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes, stream,
                     (const uint16_t*)x, wq, (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, tiles_m, tiles_n);
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

int launch_qmm(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               hipStream_t stream) {
  if (dtype == MFQ_BF16) return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
