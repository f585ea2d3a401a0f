// Large-M W4/W8 x A16 quantized matmul for gfx950:
//   y[M, N] = x[M, K] @ dequant(wq[N, K])^T (+ bias)
// the body of every QuantizedLinear call of mflux's diffusion transformers
// (e.g. src/mflux/models/flux/model/flux_transformer/
// single_transformer_block.py:53,57 at M = 4608).
//
// One workgroup of four wavefronts computes a 256 x 256 tile of y; wavefront w
// owns all 256 rows of output columns [64w, 64w+64) as 8 x 2 accumulators of
// the 32x32x16 matrix-core instruction.
//   - x goes HBM -> registers -> LDS (128-bit moves, one 64-wide k step ahead,
//     two LDS buffers, one barrier per step).  LDS rows are 128 bytes and the
//     16-byte column index is XORed with row%8, so the row-wise writes and the
//     32-row fragment reads are both bank-conflict free.
//   - packed weights never touch LDS: a lane of the matrix core's B operand
//     holds 8 consecutive k of one output column, which is exactly one uint32
//     of 4-bit codes (two of 8-bit codes).  Each lane streams 128-bit pieces of
//     its own weight row straight from HBM/L2 into registers one step ahead and
//     dequantises a word with one float32 fma per code (single rounding to the
//     16-bit type) right before the matrix instruction that consumes it.  No
//     column is dequantised by more than one wavefront.
//   - the k order inside a step is permuted (lane half h covers k 32h..32h+31)
//     identically for both operands, which the dot product does not notice.
#include "common.h"

namespace mfq {
namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;   // one 16-bit x tile: 32 KiB
constexpr int kLdsBytes = 2 * kTileBytes; // double buffered

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ inline int swz(int row, int chunk) { return row * (BK * 2) + ((chunk ^ (row & 7)) << 4); }

// Per-lane stream of packed weights for the wavefront's two 32-column tiles.
template <typename T, int GS, int BITS>
struct WeightRegs {
  static constexpr int kLoads = BITS / 4;  // 128-bit loads per column tile and step (32 codes per lane)
  u32x4 w[2][kLoads];
  float s[2], b[2];

  __device__ inline void issue(const uint32_t* const (&wrow)[2], const uint16_t* const (&srow)[2],
                               const uint16_t* const (&brow)[2], int k0, int h) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const u32x4* p = reinterpret_cast<const u32x4*>(wrow[j] + (k0 + 32 * h) * BITS / 32);
#pragma unroll
      for (int l = 0; l < kLoads; ++l) w[j][l] = p[l];
      const int g = (k0 + 32 * h) / GS;
      s[j] = T::to_f32(srow[j][g]);
      b[j] = T::to_f32(brow[j][g]);
    }
  }

  // codes 8*sub .. 8*sub+7 of this lane's 32, as 8 dequantised 16-bit values
  __device__ inline typename T::vec8 frag(int j, int sub) const {
    uint4 d;
    if constexpr (BITS == 4) {
      d = dequant8_w4<T>(w[j][0][sub], s[j], b[j]);
    } else {
      d = dequant8_w8<T>(w[j][sub >> 1][(sub & 1) * 2], w[j][sub >> 1][(sub & 1) * 2 + 1], s[j], b[j]);
    }
    return __builtin_bit_cast(typename T::vec8, d);
  }
};

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void qmm_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;

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

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wn = wave * 64;
  const int r = lane & 31;
  const int h = lane >> 5;

  f32x16 acc[8][2];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // this lane's two weight rows (columns of y); rows past N are clamped for loads
  const uint32_t* wrow[2];
  const uint16_t* srow[2];
  const uint16_t* brow[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = min(n0 + wn + 32 * j + r, N - 1);
    wrow[j] = wq + (int64_t)n * (K * BITS / 32);
    srow[j] = scales + (int64_t)n * (K / GS);
    brow[j] = biases + (int64_t)n * (K / GS);
  }
  // this thread's share of the x tile: 8 rows, one 16-byte column
  int xoff[8];  // element offsets; M*K < 2^31 is checked by the launcher
#pragma unroll
  for (int i = 0; i < 8; ++i) xoff[i] = min(m0 + (t >> 3) + 32 * i, M - 1) * K + 8 * (t & 7);

  u32x4 xa[8];
  auto issue_x = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) xa[i] = *reinterpret_cast<const u32x4*>(x + xoff[i] + k0);
  };
  auto commit_x = [&](char* tile_x) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(tile_x + swz((t >> 3) + 32 * i, t & 7)) = xa[i];
  };

  const int steps = K / BK;
  WeightRegs<T, GS, BITS> wa, wb;

  // One k step: prefetch step+1 (x into registers, weights into `next`), run
  // the matrix work of `step` from LDS buffer step&1 and `now`, then publish
  // the prefetched x tile.
  auto do_step = [&](int step, const WeightRegs<T, GS, BITS>& now, WeightRegs<T, GS, BITS>& next) {
    const char* xs = lds + (step & 1) * kTileBytes;
    // branch-free prefetch: the last step re-reads its own operands, which nobody consumes
    const int k_next = min(step + 1, steps - 1) * BK;
    issue_x(k_next);
    next.issue(wrow, srow, brow, k_next, h);
    // Fragment pipeline over 8 slots (4 k sub-steps x 2 halves of the rows):
    // the LDS reads of slot q+1 are issued before the matrix work of slot q.
    vec8 af[2][4];
    auto read_slot = [&](int q, vec8 (&dst)[4]) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dst[i] = *reinterpret_cast<const vec8*>(xs + swz(32 * (4 * (q & 1) + i) + r, 4 * h + (q >> 1)));
    };
    read_slot(0, af[0]);
    vec8 b0, b1;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (q < 7) read_slot(q + 1, af[(q + 1) & 1]);
      if ((q & 1) == 0) {
        b0 = now.frag(0, q >> 1);
        b1 = now.frag(1, q >> 1);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[4 * (q & 1) + i][0] = mfma32(af[q & 1][i], b0, acc[4 * (q & 1) + i][0]);
        acc[4 * (q & 1) + i][1] = mfma32(af[q & 1][i], b1, acc[4 * (q & 1) + i][1]);
      }
    }
    commit_x(lds + ((step + 1) & 1) * kTileBytes);
    __syncthreads();
  };

  issue_x(0);
  wa.issue(wrow, srow, brow, 0, h);
  commit_x(lds);
  __syncthreads();
  int step = 0;
  for (; step + 1 < steps; step += 2) {  // straight-line body: two steps with the weight registers swapped
    do_step(step, wa, wb);
    do_step(step + 1, wb, wa);
  }
  if (step < steps) do_step(step, wa, wb);

  // Epilogue: register e of an accumulator is row 8*(e/4) + 4*h + e%4, column r.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = n0 + wn + 32 * j + r;
    if (col >= N) continue;
    const float bv = bias ? T::to_f32(bias[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
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
  if (M * K >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;  // 32-bit element offsets into x
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
