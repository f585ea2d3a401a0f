// Quantized matvec for one to four activation rows on gfx950, eight weight rows
// at a time on the int8 matrix-core instruction:
//   y[0:M, n] = x[0:M] . dequant(W[n]) (+ bias),  M <= 4, 8-bit codes, groups of 64.
// The adaLN modulation call of every DiT block
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12,
// src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37).
//
// v_mfma_i32_16x16x64_i8 multiplies A [16 x 64] by B [64 x 16]; lane (j, q) =
// (lane % 16, lane / 16) supplies 16 bytes of A's row j and of B's column j, both
// at k 16 q .. 16 q + 15, and receives D[4 q .. 4 q + 3][j].  Here
//   - B's column j is weight row j / 2 of a block of eight rows, over the 64 k of
//     HALF j % 2 of a 128-byte step: the lane's 16 bytes are piece 4 (j % 2) + q of
//     the row's 128 bytes, so one load instruction fetches eight rows x 128
//     contiguous bytes (eight whole cache lines; 16 rows x 64 bytes, the
//     instruction's natural operand, is half lines and measurably slower);
//   - A's rows 0..7 are x over the first half of the step, rows 8..15 over the
//     second half: activation row m as 15-bit fixed point (xq = rint(x * 2^e)),
//     high bytes in row 2 m, low bytes in row 2 m + 1.  Of D, column j's rows
//     0..7 (j even) or 8..15 (j odd) are the products that belong together; the
//     others pair a half of the weights with the other half of x and are dropped.
//     Up to four activation rows cost what one does.
//   - a code enters as the signed byte code - 128 (one XOR per word); a half step
//     is one group of 64 codes, so per instruction and lane, with Sx the sum of xq
//     over the group's 64 k,
//         d = 256 D_high + D_low + 128 Sx        (int32, exactly sum(xq code))
//         acc += scale * d + bias * Sx           (float32)
//     about 17 vector instructions per KiB of weights and no conversion of a code
//     to floating point.
// One workgroup of eight wavefronts per compute unit takes a contiguous run of
// blocks; wavefront w owns eighth w of K (its part of the image of x stays in
// registers: no wavefront waits for another before the end), with the loads of
// three blocks in flight in three register sets, all unconditional so that every
// wait leaves exactly the younger loads in flight.  The eight partial sums of a
// block meet in LDS at the end of the run, where each thread adds up one output.
#include <type_traits>

#include "common.h"

namespace mfq {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kOctRows = 8;       // weight rows per block
constexpr int kOctWaves = 8;      // wavefronts per workgroup: eighths of K
constexpr int kOctSets = 3;       // blocks in flight per wavefront
constexpr int kOctMaxBlocks = 12;  // blocks per workgroup (their partial sums wait in LDS)
constexpr int kOctLongRun = 9;    // blocks per workgroup when a compute unit's share exceeds that

constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;      // lane i <- lane 15-i of its row

template <int kCtrl>
__device__ inline int oct_dpp(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xf, 0xf, false);
}
// sum over the lane's row of 16 lanes, in every lane of the row
__device__ inline int oct_row16_sum(int v) {
  v += oct_dpp<kDppXor1>(v);
  v += oct_dpp<kDppXor2>(v);
  v += oct_dpp<kDppHalfMirror>(v);
  v += oct_dpp<kDppMirror>(v);
  return v;
}
__device__ inline int oct_wave_max(int v) {
  v = max(v, oct_dpp<kDppXor1>(v));
  v = max(v, oct_dpp<kDppXor2>(v));
  v = max(v, oct_dpp<kDppHalfMirror>(v));
  v = max(v, oct_dpp<kDppMirror>(v));
  return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

template <int kSteps>
struct ScaleWindow {
  uint32_t d[kSteps];  // dword s: the scales (or biases) of the two halves of step s
};

// kSteps: 128-byte steps per wavefront and row (K = 1024 kSteps); kM: activation rows the image is built for
// (1, 2 or 4; M = 3 runs as 4 with its last row repeated)
template <typename T, int kSteps, int kM, bool kSilu>
__global__ __launch_bounds__(64 * kOctWaves) void qmv_oct_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int blocks_per_wg) {
  constexpr int K = 128 * kOctWaves * kSteps;
  constexpr int kSlice = 128 * kSteps;       // bytes (= codes) per row and wavefront
  constexpr int kGroups = K / 64;
  constexpr int kPitch = kSlice + 16;        // image rows in LDS
  constexpr int kImageRows = 2 * kM;
  constexpr int kImageBytes = ((kImageRows * kPitch + kM * 2 * kSteps * 4) + 255) & ~255;  // + the sums of xq
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int j = lane & 15, q = lane >> 4;
  const int n8 = j >> 1, h = j & 1;
  char* image = lds + wave * kImageBytes;
  float* sums = reinterpret_cast<float*>(image + kImageRows * kPitch);
  float2* partials = reinterpret_cast<float2*>(lds + kOctWaves * kImageBytes);  // [block][wavefront][lane]

  const int n_blocks_all = N / kOctRows;
  const int blk_first = blockIdx.x * blocks_per_wg;
  const int n_blocks = min(blocks_per_wg, n_blocks_all - blk_first);
  const int blk_last = blk_first + n_blocks - 1;

  // the output this thread will add up at the end (block, weight row, activation row), and its layer bias:
  // requested now, with everything else, so that nothing is fetched behind the last barrier
  constexpr int kOuts = (kOctMaxBlocks * kOctRows * 4 + 64 * kOctWaves - 1) / (64 * kOctWaves);
  uint16_t out_bias[kOuts];
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = (int)threadIdx.x + i * 64 * kOctWaves;
    const int64_t row = (int64_t)(blk_first + min(o / M / kOctRows, n_blocks - 1)) * kOctRows + (o / M) % kOctRows;
    out_bias[i] = (bias ? bias : scales)[row];
  }

  // ---- requests: x first (it is needed first, and loads return in order), the first block behind it ----
  constexpr int kChunks = (32 * kSteps + 63) / 64;  // chunks of 4 consecutive k per lane and activation row
  uint2 raw[kM][kChunks];
#pragma unroll
  for (int m = 0; m < kM; ++m)
#pragma unroll
    for (int t = 0; t < kChunks; ++t) {
      const int c = min(lane + 64 * t, 32 * kSteps - 1);
      raw[m][t] = *reinterpret_cast<const uint2*>(x + (size_t)min(m, M - 1) * K + wave * kSlice + 4 * c);
    }

  const char* wlane = reinterpret_cast<const char*>(wq) + (size_t)n8 * K + wave * kSlice + 16 * (4 * h + q);
  const char* slane = reinterpret_cast<const char*>(scales) + ((size_t)n8 * kGroups + wave * 2 * kSteps) * 2;
  const char* blane = reinterpret_cast<const char*>(biases) + ((size_t)n8 * kGroups + wave * 2 * kSteps) * 2;
  u32x4 wv[kOctSets][kSteps];
  ScaleWindow<kSteps> sw[kOctSets], bw[kOctSets];
  // every load is unconditional (a block past the run's end is its last block again)
  auto issue = [&](int set, int blk) __attribute__((always_inline)) {
    const size_t b = (size_t)min(blk, blk_last);
    sw[set] = *reinterpret_cast<const ScaleWindow<kSteps>*>(slane + b * (kOctRows * kGroups * 2));
    bw[set] = *reinterpret_cast<const ScaleWindow<kSteps>*>(blane + b * (kOctRows * kGroups * 2));
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
      // (streaming loads: left to the default cache policy the same call takes 1.2 us longer)
      wv[set][s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wlane + b * (kOctRows * K) + 128 * s));
  };
  // the first block now, the other two behind the image of x: with two wavefronts on a SIMD the older one's
  // requests are served first, and all three blocks at once would set the younger one back by their whole length
  issue(0, blk_first);

  // ---- the integer image of this wavefront's eighth of x ------------------------------------------------
  // One power of two per activation row and eighth of K: the eighths' sums are scaled back before they meet,
  // so the wavefronts need not agree on it and nobody waits for anybody here.
  float unscale_m[kM];
#pragma unroll
  for (int m = 0; m < kM; ++m) {
    int amax = 0;
#pragma unroll
    for (int t = 0; t < kChunks; ++t) {
      if constexpr (kSilu) {
        raw[m][t].x = silu_pair<T>(raw[m][t].x);
        raw[m][t].y = silu_pair<T>(raw[m][t].y);
      }
      amax = max(amax, max(mag_bits(raw[m][t].x), mag_bits(raw[m][t].y)));
    }
    amax = oct_wave_max(amax);
    const int e = scale_exponent<T>(amax);
    const float mult = pow2(e);
    // an infinity or NaN anywhere in a row of x: every output of that row is NaN (through this eighth's sums)
    unscale_m[m] = not_finite<T>(amax) ? __builtin_nanf("") : pow2(-e);
#pragma unroll
    for (int t = 0; t < kChunks; ++t) {
      const int c = lane + 64 * t;
      const bool in = c < 32 * kSteps;
      uint32_t hi, lo;
      split4<T>(raw[m][t].x, raw[m][t].y, mult, hi, lo);
      if (in) {
        *reinterpret_cast<uint32_t*>(image + (2 * m) * kPitch + 4 * c) = hi;
        *reinterpret_cast<uint32_t*>(image + (2 * m + 1) * kPitch + 4 * c) = lo;
      }
      // the sum of xq over a half step's 64 k: its 16 chunks are the 16 lanes of a row of lanes
      const int part = __builtin_amdgcn_sdot4((int)hi, 0x01010101, 0, false) * 256 +
                       __builtin_amdgcn_sdot4((int)lo, 0x01010101, 0, false);
      const int total = oct_row16_sum(in ? part : 0);
      if (j == 0 && in) sums[m * 2 * kSteps + (c >> 4)] = (float)total;
    }
  }
  // (LDS written and read by this wavefront only: program order holds)
  // this lane's A operands: image row j % 8 over half j / 8 of every step (image rows past 2 kM: any row, their
  // results are never read)
  i32x4 xa[kSteps];
  {
    const char* arow = image + (j & 7 & (kImageRows - 1)) * kPitch + 64 * (j >> 3) + 16 * q;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) xa[s] = *reinterpret_cast<const i32x4*>(arow + 128 * s);
  }
  // results: register r of lane (j, q) is A's row 4 q + r against column j.  Of use where q / 2 == j % 2:
  // activation rows 2 (q % 2) (registers 0, 1: high, low bytes) and 2 (q % 2) + 1 (registers 2, 3)
  constexpr bool kTwo = kM > 1;  // one activation row: registers 2 and 3 hold nothing of use
  const int m_a = (2 * (q & 1)) & (kM - 1), m_b = (2 * (q & 1) + 1) & (kM - 1);
  // the sums of xq over this lane's half steps: as float for the bias term, and 128 times them as integers
  // (a code enters the matrix instruction as code - 128; adding 128 sum(xq) to its result gives sum(xq code))
  float sx_a[kSteps], sx_b[kSteps];
  int sx128_a[kSteps], sx128_b[kSteps];
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    sx_a[s] = sums[m_a * 2 * kSteps + 2 * s + h];
    sx_b[s] = kTwo ? sums[m_b * 2 * kSteps + 2 * s + h] : 0.f;
    sx128_a[s] = 128 * (int)sx_a[s];
    sx128_b[s] = 128 * (int)sx_b[s];
  }
  float us_a = unscale_m[0], us_b = unscale_m[kM > 1 ? 1 : 0];
#pragma unroll
  for (int m = 2; m < kM; ++m) {
    us_a = m_a == m ? unscale_m[m] : us_a;
    us_b = m_b == m ? unscale_m[m] : us_b;
  }

#pragma unroll
  for (int t = 1; t < kOctSets; ++t) issue(t, blk_first + t);
  auto consume = [&](int set, int slot) __attribute__((always_inline)) {
    float acc_a = 0.f, acc_b = 0.f;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      i32x4 wb;
#pragma unroll
      for (int k = 0; k < 4; ++k) wb[k] = (int)(wv[set][s][k] ^ 0x80808080u);  // code - 128 as signed bytes
      const i32x4 zero = {0, 0, 0, 0};
      const i32x4 d = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[s], wb, zero, 0, 0, 0);
      const float sc = T::to_f32((uint16_t)(h ? sw[set].d[s] >> 16 : sw[set].d[s]));
      const float bi = T::to_f32((uint16_t)(h ? bw[set].d[s] >> 16 : bw[set].d[s]));
      // sum(xq code) over the half step's group, exact: high and low bytes of xq joined as integers
      const int da = d[0] * 256 + d[1] + sx128_a[s];
      acc_a = __builtin_fmaf(sc, (float)da, acc_a);
      acc_a = __builtin_fmaf(bi, sx_a[s], acc_a);
      if constexpr (kTwo) {
        const int db = d[2] * 256 + d[3] + sx128_b[s];
        acc_b = __builtin_fmaf(sc, (float)db, acc_b);
        acc_b = __builtin_fmaf(bi, sx_b[s], acc_b);
      }
    }
    partials[(slot * kOctWaves + wave) * 64 + lane] = make_float2(acc_a * us_a, acc_b * us_b);
  };

  // Three blocks per trip, one per register set, and between the arithmetic of two blocks the requests for the
  // block three further on; the last trip requests nothing (loads still in flight at the end would hold their
  // registers, and the adding-up below, until they land).  A block past the run's end is computed again
  // into a slot of its own that nobody reads.
  int b = 0;
  for (; b + kOctSets < n_blocks; b += kOctSets) {
#pragma unroll
    for (int t = 0; t < kOctSets; ++t) {
      __builtin_amdgcn_sched_barrier(0);
      consume(t, b + t);
      __builtin_amdgcn_sched_barrier(0);
      issue(t, blk_first + b + t + kOctSets);
    }
  }
#pragma unroll
  for (int t = 0; t < kOctSets; ++t) {
    __builtin_amdgcn_sched_barrier(0);
    consume(t, min(b + t, n_blocks));
  }
  __syncthreads();

  // ---- one output per thread: block, weight row, activation row; 8 eighths x 2 halves of partial sums --------
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = (int)threadIdx.x + i * 64 * kOctWaves;
    const int out_m = o % M, out_row8 = (o / M) % kOctRows, out_blk = o / M / kOctRows;
    if (out_blk >= n_blocks) break;
    const int64_t out_row = (int64_t)(blk_first + out_blk) * kOctRows + out_row8;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < kOctWaves; ++w)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int src = (2 * out_row8 + hh) + 16 * (2 * hh + (out_m >> 1));
        const float2 p = partials[(out_blk * kOctWaves + w) * 64 + src];
        v += (out_m & 1) ? p.y : p.x;
      }
    const float bias_v = T::to_f32(out_bias[i]);
    if (y_is_f32) {
      reinterpret_cast<float*>(y)[(int64_t)out_m * N + out_row] = bias ? v + bias_v : v;
    } else {
      const uint16_t h0 = T::from_f32(v);
      const uint16_t h1 = T::from_f32(T::to_f32(h0) + bias_v);  // second rounding, as a separate add would do
      reinterpret_cast<uint16_t*>(y)[(int64_t)out_m * N + out_row] = bias ? h1 : h0;
    }
  }
}

template <typename T, int kSteps, int kM, bool kSilu>
int launch_oct(const void* x, int64_t M, const uint32_t* wq, const void* scales, const void* biases, const void* bias,
               int64_t N, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmv_oct_kernel<T, kSteps, kM, kSilu>;
  constexpr int kImageBytes = ((2 * kM * (128 * kSteps + 16) + kM * 2 * kSteps * 4) + 255) & ~255;
  constexpr int kLdsMax = kOctWaves * kImageBytes + (kOctMaxBlocks + 1) * kOctWaves * 512;
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLdsMax)) return MFQ_ELAUNCH;
  // One workgroup per compute unit while that is at most kOctMaxBlocks blocks each; longer weights in runs of
  // kOctLongRun blocks to as many workgroups as that takes (several resident per unit: a run's last loads and
  // its adding-up overlap the next run's first requests).
  const int64_t blocks = N / kOctRows;
  const int64_t cus = compute_units();
  int64_t per_wg = (blocks + cus - 1) / cus;
  if (per_wg > kOctMaxBlocks) per_wg = kOctLongRun;
  const int64_t n_wg = (blocks + per_wg - 1) / per_wg;
  const int lds = kOctWaves * kImageBytes + ((int)per_wg + 1) * kOctWaves * 512;
  hipLaunchKernelGGL(kernel, dim3((unsigned)n_wg), dim3(64 * kOctWaves), lds, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)per_wg);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int kSteps, bool kSilu>
int launch_oct_rows(const void* x, int64_t M, const uint32_t* wq, const void* scales, const void* biases,
                    const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  if (M == 1) return launch_oct<T, kSteps, 1, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
  if (M == 2) return launch_oct<T, kSteps, 2, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
  return launch_oct<T, kSteps, 4, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
}

template <typename T, bool kSilu>
int launch_oct_steps(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                     const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  switch (K / (128 * kOctWaves)) {
    case 1: return launch_oct_rows<T, 1, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 2: return launch_oct_rows<T, 2, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 3: return launch_oct_rows<T, 3, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 4: return launch_oct_rows<T, 4, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    default: return MFQ_EUNSUPPORTED;
  }
}

}  // namespace

// Shapes this kernel takes: 8-bit codes in groups of 64, one to four activation rows, K of 1024, 2048, 3072
// or 4096 (an eighth of a row is whole 128-byte steps), whole eights of weight rows, x and the weights
// 16-byte aligned, scales and biases 4-byte aligned.
bool qmv_oct_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* x, const void* scales,
                    const void* biases) {
  if (!(bits == 8 && gs == 64 && M >= 1 && M <= 4 && K % (128 * kOctWaves) == 0 && K >= 128 * kOctWaves && K <= 4096 && N % kOctRows == 0))
    return false;
  return aligned16(x) && ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 3u) == 0;
}

int launch_qmv_oct(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   hipStream_t stream, bool silu) {
  if (!qmv_oct_covers(M, K, N, gs, bits, x, scales, biases)) return MFQ_EUNSUPPORTED;
  if (dtype != MFQ_BF16 && dtype != MFQ_F16) return MFQ_EDTYPE;
  const bool bf = dtype == MFQ_BF16;
  if (silu)
    return bf ? launch_oct_steps<BF16, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream)
              : launch_oct_steps<F16, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
  return bf ? launch_oct_steps<BF16, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream)
            : launch_oct_steps<F16, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
}

}  // namespace mfq
