// Low-rank update of a finished product for gfx950: y[M, N] += t[M, R] @ bs[N, R]^T.
//
// This is the LoRA branch of a wrapped linear layer,
//   base(x) + scale * (x @ A) @ B
// (src/mflux/models/common/lora/layer/linear_lora_layer.py:50-53, and the sum
// over several adapters in fused_linear_lora_layer.py:13-20), with
// t = x @ [A_1 | A_2 | ...] and bs = [scale_1 * B_1^T | scale_2 * B_2^T | ...].
// The GEMM kernels accumulate the update with the product themselves; this
// kernel serves the products that come from elsewhere (one to sixteen
// activation rows, odd bit widths dequantised for a library GEMM).
//
// A workgroup of four wavefronts owns 64 rows x 128 columns of y; wavefront w
// takes columns [32w, 32w+32) as two 32x32x16 matrix-core accumulators.  R is
// small (a LoRA rank, or the sum of a few), so both operands are read straight
// from memory as matrix fragments: a lane's 8 consecutive k of one row of bs or
// t are one 16-byte load.  y is read, updated in float32 and rounded back.
#include "common.h"

namespace mfq {
namespace {

constexpr int kRows = 64;
constexpr int kCols = 128;

template <typename T>
__global__ __launch_bounds__(256) void low_rank_add_kernel(const uint16_t* __restrict__ t,
                                                           const uint16_t* __restrict__ bs, int R, int M, int N,
                                                           void* __restrict__ y, int y_is_f32, int vec_ok) {
  using vec8 = typename T::vec8;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int n0 = blockIdx.x * kCols + 32 * wave;
  const int m0 = blockIdx.y * kRows;

  // rows past M / N are clamped for loads and never stored
  const uint16_t* brow = bs + (int64_t)min(n0 + r, N - 1) * R + 8 * h;
  const uint16_t* trow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) trow[i] = t + (int64_t)min(m0 + 32 * i + r, M - 1) * R + 8 * h;

  f32x16 acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  for (int k = 0; k < R; k += 16) {
    const vec8 bf = *reinterpret_cast<const vec8*>(brow + k);
#pragma unroll
    for (int i = 0; i < 2; ++i) acc[i] = mfma32(bf, *reinterpret_cast<const vec8*>(trow[i] + k), acc[i]);
  }

  // register e of accumulator i: row m0 + 32 i + r, column n0 + 8 (e / 4) + 4 h + e % 4
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = m0 + 32 * i + r;
    if (row >= M) continue;
#pragma unroll
    for (int eb = 0; eb < 4; ++eb) {
      const int col = n0 + 8 * eb + 4 * h;
      if (col >= N) continue;
      const int64_t o = (int64_t)row * N + col;
      if (y_is_f32) {
        float* dst = reinterpret_cast<float*>(y) + o;
        if (vec_ok) {
          float4 v = *reinterpret_cast<const float4*>(dst);
          v.x += acc[i][4 * eb];
          v.y += acc[i][4 * eb + 1];
          v.z += acc[i][4 * eb + 2];
          v.w += acc[i][4 * eb + 3];
          *reinterpret_cast<float4*>(dst) = v;
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (col + c < N) dst[c] += acc[i][4 * eb + c];
        }
      } else {
        uint16_t* dst = reinterpret_cast<uint16_t*>(y) + o;
        if (vec_ok) {
          uint2 v = *reinterpret_cast<const uint2*>(dst);
          v.x = T::pack2(lo_f32<T>(v.x) + acc[i][4 * eb], hi_f32<T>(v.x) + acc[i][4 * eb + 1]);
          v.y = T::pack2(lo_f32<T>(v.y) + acc[i][4 * eb + 2], hi_f32<T>(v.y) + acc[i][4 * eb + 3]);
          *reinterpret_cast<uint2*>(dst) = v;
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (col + c < N) dst[c] = T::from_f32(T::to_f32(dst[c]) + acc[i][4 * eb + c]);
        }
      }
    }
  }
}

template <typename T>
int launch(LowRank lr, int64_t M, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  const dim3 grid((unsigned)((N + kCols - 1) / kCols), (unsigned)((M + kRows - 1) / kRows));
  // four consecutive outputs move as one piece when no piece can straddle a row or be misaligned
  const int vec_ok = (N & 3) == 0 && aligned16(y);
  hipLaunchKernelGGL((low_rank_add_kernel<T>), grid, dim3(256), 0, stream, (const uint16_t*)lr.t,
                     (const uint16_t*)lr.bs, lr.R, (int)M, (int)N, y, (int)(y_dtype == MFQ_F32), vec_ok);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

}  // namespace

int launch_low_rank_add(int dtype, LowRank low_rank, int64_t M, int64_t N, void* y, int y_dtype,
                        hipStream_t stream) {
  if (low_rank.R == 0) return MFQ_OK;
  if ((M + kRows - 1) / kRows > 65535) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16) return launch<BF16>(low_rank, M, N, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch<F16>(low_rank, M, N, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
