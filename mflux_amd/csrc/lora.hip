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

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// ---- the down-projection in front of it: t[M, R] = x[M, K] @ A[K, R].
//
// x is read once (2 M K bytes: the kernel is bound by that read, and the whole of it is only a few times what
// must be in flight to cover the memory latency), so the work is cut for memory parallelism, not for the matrix
// cores: a workgroup of 8 wavefronts owns 16 rows of x, the trips (four pairs of 32-k steps: 512 bytes of each row,
// 8 KiB of x) are dealt to its wavefronts in turn, so that the workgroup reads one 4 KiB window of every row at a
// time, and a wavefront requests a whole trip before it uses any of it and the next one while it computes.
//   - the vector memory path takes about as long per cache line touched as per 128 bytes moved, so every load
//     covers whole lines: x goes row-segment-wise (8 lanes = one 128-byte line of a row) through a private LDS
//     region of the wavefront (no barrier), XOR-swizzled so that the fragment reads are conflict free;
//   - A is packed once per adapter set, so it is handed over in the order the matrix instruction consumes
//     (af [R/16][K/32][64 lanes][8]: lane 16 q + c of step s holds A[32 s + 8 q .. + 7][16 f + c]) and a
//     wavefront's fragment is 1 KiB of contiguous memory; it is small and stays in L2;
//   - the partial tiles meet in LDS and are added in the order of the wavefronts; A is the matrix
//     instruction's A operand so that a lane ends up with four consecutive columns of one row of t.
// F fragments of 16 columns of t per workgroup (blockIdx.y takes the next 16 F).
constexpr int kDownWaves = 8;
constexpr int kDownPairs = 4;                          // pairs of steps per trip
constexpr int kDownStage = kDownPairs * 16 * 128;      // bytes of x a wavefront stages per trip

template <typename T, int F>
__global__ __launch_bounds__(kDownWaves* kWave, 2) void low_rank_down_kernel(const uint16_t* __restrict__ x,
                                                                             const uint16_t* __restrict__ af, int M,
                                                                             int K, int R, uint16_t* __restrict__ t) {
  using vec8 = typename T::vec8;
  __shared__ __attribute__((aligned(16))) char lds[kDownWaves * kDownStage];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int c16 = lane & 15, q = lane >> 4;
  const int m0 = blockIdx.x * 16;
  const int f0 = blockIdx.y * F;
  char* stage = lds + wave * kDownStage;

  const int steps = K / 32, pairs = (steps + 1) / 2;
  // trips are dealt round-robin: trip t of wavefront w is pairs (t * 8 + w) * 4 .. + 3, so that at any time the
  // workgroup reads one window of 4 KiB per row (16 pages in flight instead of 128)
  const int p_begin = wave * kDownPairs, p_end = pairs, p_stride = kDownWaves * kDownPairs;
  // staging: piece h (0, 1) of a pair is rows 8 h + lane / 8, 16-byte column lane % 8 of the pair's 128 bytes;
  // in LDS the column is XORed with row % 8.  A pair's second step may lie past K (K % 64 == 32): its columns
  // re-read the first step's and are not used.
  const int srow = lane >> 3, scol = lane & 7;
  const uint16_t* xsrc[2];
  int sput[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    xsrc[h] = x + (int64_t)min(m0 + 8 * h + srow, M - 1) * K;  // rows past M re-read the last one
    sput[h] = (8 * h + srow) * 128 + ((scol ^ srow) << 4);
  }
  int sget[2];  // step j of a pair: row c16, column 4 j + q
#pragma unroll
  for (int j = 0; j < 2; ++j) sget[j] = c16 * 128 + (((4 * j + q) ^ (c16 & 7)) << 4);
  const uint16_t* asrc = af + ((int64_t)f0 * steps * kWave + lane) * 8;

  f32x4 acc[F];
#pragma unroll
  for (int f = 0; f < F; ++f) acc[f] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto request = [&](u32x4 (&xr)[kDownPairs][2], int p0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kDownPairs; ++u) {
      const int p = min(p0 + u, p_end - 1);  // pairs past the end repeat the last one and are not used
      const int col = min(64 * p + 8 * scol, K - 8);
#pragma unroll
      for (int h = 0; h < 2; ++h) xr[u][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xsrc[h] + col));
    }
  };
  u32x4 xr[kDownPairs][2];
  if (p_begin < p_end) request(xr, p_begin);
  for (int p0 = p_begin; p0 < p_end; p0 += p_stride) {
#pragma unroll
    for (int u = 0; u < kDownPairs; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) *reinterpret_cast<u32x4*>(stage + u * 2048 + sput[h]) = xr[u][h];
    // the next trip's x is on its way while this one meets its fragments of A
    if (p0 + p_stride < p_end) request(xr, p0 + p_stride);
    // (the region is private to the wavefront, whose LDS operations complete in order: no barrier)
#pragma unroll
    for (int u = 0; u < kDownPairs; ++u) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int s = 2 * (p0 + u) + j;
        if (p0 + u < p_end && s < steps) {
          const vec8 xf = *reinterpret_cast<const vec8*>(stage + u * 2048 + sget[j]);
#pragma unroll
          for (int f = 0; f < F; ++f)
            acc[f] = mfma16(*reinterpret_cast<const vec8*>(asrc + ((int64_t)f * steps + s) * (kWave * 8)), xf, acc[f]);
        }
      }
    }
  }
  __syncthreads();  // every wavefront is done with its staging region: the partial tiles go over it
  f32x4* parts = reinterpret_cast<f32x4*>(lds);
#pragma unroll
  for (int f = 0; f < F; ++f) parts[(wave * F + f) * kWave + lane] = acc[f];
  __syncthreads();
  if (wave < F) {  // wavefront f finishes fragment f: row m0 + c16, columns 16 (f0 + f) + 4 q .. + 3
    f32x4 v = parts[wave * kWave + lane];
#pragma unroll
    for (int w = 1; w < kDownWaves; ++w) {
      const f32x4 p = parts[(w * F + wave) * kWave + lane];
      v[0] += p[0]; v[1] += p[1]; v[2] += p[2]; v[3] += p[3];
    }
    const int row = m0 + c16;
    if (row < M)
      *reinterpret_cast<uint2*>(t + (int64_t)row * R + 16 * (f0 + wave) + 4 * q) =
          make_uint2(T::pack2(v[0], v[1]), T::pack2(v[2], v[3]));
  }
}

template <typename T>
int launch_down(const void* x, int64_t M, int64_t K, const void* at, int64_t R, void* t, hipStream_t stream) {  // at: fragment order
  const int frags = R % 64 == 0 ? 4 : (R % 32 == 0 ? 2 : 1);
  const dim3 grid((unsigned)((M + 15) / 16), (unsigned)(R / (16 * frags)));
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kDownWaves * kWave), 0, stream, (const uint16_t*)x, (const uint16_t*)at,
                       (int)M, (int)K, (int)R, (uint16_t*)t);
  };
  if (frags == 4) go(low_rank_down_kernel<T, 4>);
  else if (frags == 2) go(low_rank_down_kernel<T, 2>);
  else go(low_rank_down_kernel<T, 1>);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

}  // namespace

int launch_low_rank_down(const void* x, int dtype, int64_t M, int64_t K, const void* at, int64_t R, void* t,
                         hipStream_t stream) {
  if (dtype == MFQ_BF16) return launch_down<BF16>(x, M, K, at, R, t, stream);
  if (dtype == MFQ_F16) return launch_down<F16>(x, M, K, at, R, t, stream);
  return MFQ_EDTYPE;
}

int launch_low_rank_add(int dtype, LowRank low_rank, int64_t M, int64_t N, void* y, int y_dtype,
                        hipStream_t stream) {
  if (low_rank.R == 0) return MFQ_OK;
  if ((M + kRows - 1) / kRows > 65535) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16) return launch<BF16>(low_rank, M, N, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch<F16>(low_rank, M, N, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
