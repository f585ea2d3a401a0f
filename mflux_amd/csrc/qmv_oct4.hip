// Quantized matvec for one to four activation rows and 4-bit codes on gfx950,
// eight weight rows at a time on the int8 matrix-core instruction: the scheme
// of qmv_oct.hip (which see) for packed nibbles,
//   y[0:M, n] = x[0:M] . dequant(W[n]) (+ bias),  M <= 4, groups of 64.
// The adaLN modulation call of every DiT block of a 4-bit model
// (src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37,
// src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12).
//
// A load instruction again fetches eight rows x 128 contiguous bytes, now 256
// codes of each row: four groups.  Lane (j, q) = (lane % 16, lane / 16) holds
// piece 4 (j % 2) + q of row j / 2, 32 codes; their even nibbles (w & 0x0f..) and
// odd nibbles ((w >> 4) & 0x0f..) are the B operands of two
// v_mfma_i32_16x16x64_i8 that add into the same sums.  Column j's four lanes
// cover TWO groups (pieces 2g, 2g + 1 are group g of the column's half row), so
// the A operand tells them apart: A's row 8 h + 4 g + 2 m + l is activation row
// m (two of them per pair of instructions), high (l = 0) or low byte of its
// 15-bit fixed point, over the k of half h -- and zero in the lanes of the
// other group.  Column j's useful sums are rows 8 (j % 2) .. + 7: lane
// (j, 2 (j % 2) + g) receives group g's for both activation rows, one scale and
// bias per lane and step as in the 8-bit kernel.  Nibbles are non-negative, so
// nothing is offset:
//     d = 256 D_high + D_low      (int32, exactly sum(xq code) over the group)
//     acc += scale * d + bias * sum(xq)
// Three and four activation rows take a second pair of instructions on the same
// B operands.  Work layout, register sets, the meeting of the wavefronts'
// partial sums at the end: qmv_oct.hip's, with K split over kWaves4 wavefronts.
#include <type_traits>

#include "common.h"

namespace mfq {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kRows4 = 8;        // weight rows per block
constexpr int kSets4 = 3;        // blocks in flight per wavefront
constexpr int kMaxBlocks4 = 12;  // blocks per workgroup (their partial sums wait in LDS)
constexpr int kLongRun4 = 9;     // blocks per workgroup when a compute unit's share exceeds that

constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;      // lane i <- lane 15-i of its row

template <int kCtrl>
__device__ inline int oct4_dpp(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xf, 0xf, false);
}
// sum over the lane's eight (lanes 8 i .. 8 i + 7), in every lane of it
__device__ inline int oct4_sum8(int v) {
  v += oct4_dpp<kDppXor1>(v);
  v += oct4_dpp<kDppXor2>(v);
  v += oct4_dpp<kDppHalfMirror>(v);
  return v;
}
__device__ inline int oct4_wave_max(int v) {
  v = max(v, oct4_dpp<kDppXor1>(v));
  v = max(v, oct4_dpp<kDppXor2>(v));
  v = max(v, oct4_dpp<kDppHalfMirror>(v));
  v = max(v, oct4_dpp<kDppMirror>(v));
  return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

template <int kSteps>
struct ScaleWindow4 {
  uint32_t d[2 * kSteps];  // dword 2 s + h: the scales (or biases) of the two groups of half h of step s
};

// kWaves: wavefronts per workgroup, each with kSteps 128-byte steps of every row (K = 256 kWaves kSteps codes);
// kM: activation rows the image is built for (1, 2 or 4; M = 3 runs as 4 with its last row repeated)
template <typename T, int kWaves, int kSteps, int kM, bool kSilu>
__global__ __launch_bounds__(64 * kWaves) void qmv_oct4_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int blocks_per_wg) {
  constexpr int K = 256 * kWaves * kSteps;
  constexpr int kRowBytes = K / 2;
  constexpr int kSlice = 128 * kSteps;       // bytes per row and wavefront: 2 kSlice codes
  constexpr int kGroups = K / 64;
  constexpr int kPasses = kM > 2 ? 2 : 1;    // pairs of activation rows
  constexpr int kImageRows = 2 * kM;         // (activation row, high / low byte)
  constexpr int kPitch = 2 * kSlice + 32;    // an image row: kSlice bytes of even k, kSlice of odd k
  constexpr int kImageBytes = ((kImageRows * kPitch + kM * 4 * kSteps * 4) + 255) & ~255;  // + the sums of xq
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int j = lane & 15, q = lane >> 4;
  const int n8 = j >> 1, h = j & 1;
  char* image = lds + wave * kImageBytes;
  float* sums = reinterpret_cast<float*>(image + kImageRows * kPitch);  // [activation row][group of the slice]
  float2* partials = reinterpret_cast<float2*>(lds + kWaves * kImageBytes);  // [block][wavefront][pass][lane]

  const int n_blocks_all = N / kRows4;
  const int blk_first = blockIdx.x * blocks_per_wg;
  const int n_blocks = min(blocks_per_wg, n_blocks_all - blk_first);
  const int blk_last = blk_first + n_blocks - 1;

  // the outputs this thread will add up at the end (block, weight row, activation row), and their layer bias:
  // requested now, with everything else, so that nothing is fetched behind the last barrier
  constexpr int kOuts = (kMaxBlocks4 * kRows4 * 4 + 64 * kWaves - 1) / (64 * kWaves);
  uint16_t out_bias[kOuts];
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = (int)threadIdx.x + i * 64 * kWaves;
    const int64_t row = (int64_t)(blk_first + min(o / M / kRows4, n_blocks - 1)) * kRows4 + (o / M) % kRows4;
    out_bias[i] = (bias ? bias : scales)[row];
  }

  // ---- requests: x first (it is needed first, and loads return in order), the first block behind it ----
  // chunk c = 8 consecutive k (16 bytes of x): one word of codes
  constexpr int kChunks = (32 * kSteps + 63) / 64;
  u32x4 raw[kM][kChunks];
#pragma unroll
  for (int m = 0; m < kM; ++m)
#pragma unroll
    for (int t = 0; t < kChunks; ++t) {
      const int c = min(lane + 64 * t, 32 * kSteps - 1);
      raw[m][t] = *reinterpret_cast<const u32x4*>(x + (size_t)min(m, M - 1) * K + wave * 2 * kSlice + 8 * c);
    }

  const char* wlane = reinterpret_cast<const char*>(wq) + (size_t)n8 * kRowBytes + wave * kSlice + 16 * (4 * h + q);
  const char* slane = reinterpret_cast<const char*>(scales) + ((size_t)n8 * kGroups + wave * 4 * kSteps) * 2;
  const char* blane = reinterpret_cast<const char*>(biases) + ((size_t)n8 * kGroups + wave * 4 * kSteps) * 2;
  u32x4 wv[kSets4][kSteps];
  ScaleWindow4<kSteps> sw[kSets4], bw[kSets4];
  // every load is unconditional (a block past the run's end is its last block again)
  auto issue = [&](int set, int blk) __attribute__((always_inline)) {
    const size_t b = (size_t)min(blk, blk_last);
    sw[set] = *reinterpret_cast<const ScaleWindow4<kSteps>*>(slane + b * (kRows4 * kGroups * 2));
    bw[set] = *reinterpret_cast<const ScaleWindow4<kSteps>*>(blane + b * (kRows4 * kGroups * 2));
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
      wv[set][s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wlane + b * (kRows4 * kRowBytes) + 128 * s));
  };
  issue(0, blk_first);

  // ---- the integer image of this wavefront's part of x: per activation row and byte (high, low) one LDS row,
  // even k in its first kSlice bytes, odd k behind them --------------------------------------------------
  float unscale_m[kM];
#pragma unroll
  for (int m = 0; m < kM; ++m) {
    int amax = 0;
#pragma unroll
    for (int t = 0; t < kChunks; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (kSilu) raw[m][t][i] = silu_pair<T>(raw[m][t][i]);
        amax = max(amax, mag_bits(raw[m][t][i]));
      }
    amax = oct4_wave_max(amax);
    const int e = scale_exponent<T>(amax);
    const float mult = pow2(e);
    // an infinity or NaN anywhere in a row of x: every output of that row is NaN (through this part's sums)
    unscale_m[m] = not_finite<T>(amax) ? __builtin_nanf("") : pow2(-e);
#pragma unroll
    for (int t = 0; t < kChunks; ++t) {
      const int c = lane + 64 * t;
      const bool in = c < 32 * kSteps;
      // raw[..][i] = (x[2 i], x[2 i + 1]): even k in the low halves
      const u32x4 r = raw[m][t];
      const uint32_t ev0 = (r[0] & 0xffffu) | (r[1] << 16), ev1 = (r[2] & 0xffffu) | (r[3] << 16);
      const uint32_t od0 = (r[0] >> 16) | (r[1] & 0xffff0000u), od1 = (r[2] >> 16) | (r[3] & 0xffff0000u);
      uint32_t hi_e, lo_e, hi_o, lo_o;
      split4<T>(ev0, ev1, mult, hi_e, lo_e);
      split4<T>(od0, od1, mult, hi_o, lo_o);
      if (in) {
        *reinterpret_cast<uint32_t*>(image + (2 * m) * kPitch + 4 * c) = hi_e;
        *reinterpret_cast<uint32_t*>(image + (2 * m) * kPitch + kSlice + 16 + 4 * c) = hi_o;
        *reinterpret_cast<uint32_t*>(image + (2 * m + 1) * kPitch + 4 * c) = lo_e;
        *reinterpret_cast<uint32_t*>(image + (2 * m + 1) * kPitch + kSlice + 16 + 4 * c) = lo_o;
      }
      // the sum of xq over a group's 64 k: its 8 chunks are 8 neighbouring lanes
      const int part = (__builtin_amdgcn_sdot4((int)hi_e, 0x01010101, 0, false) +
                        __builtin_amdgcn_sdot4((int)hi_o, 0x01010101, 0, false)) * 256 +
                       __builtin_amdgcn_sdot4((int)lo_e, 0x01010101, 0, false) +
                       __builtin_amdgcn_sdot4((int)lo_o, 0x01010101, 0, false);
      const int total = oct4_sum8(in ? part : 0);
      if ((lane & 7) == 0 && in) sums[m * 4 * kSteps + (c >> 3)] = (float)total;
    }
  }
  // (LDS written and read by this wavefront only: program order holds)
  // this lane's A operands, pass p: A's row j = 8 h' + 4 g + 2 (m % 2) + l -- activation row 2 p + (j / 2) % 2,
  // byte l = j % 2, over half h' = j / 8 of every step, zero unless this lane's k (pieces 2 g, 2 g + 1 of the
  // half: q / 2 == g) belong to group g = (j / 4) % 2
  i32x4 xa_e[kPasses][kSteps], xa_o[kPasses][kSteps];
  {
    const bool mine = (q >> 1) == ((j >> 2) & 1);
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int m = (2 * p + ((j >> 1) & 1)) & (kM - 1);
      const char* arow = image + (2 * m + (j & 1)) * kPitch + 64 * (j >> 3) + 16 * q;
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        const i32x4 zero = {0, 0, 0, 0};
        xa_e[p][s] = mine ? *reinterpret_cast<const i32x4*>(arow + 128 * s) : zero;
        xa_o[p][s] = mine ? *reinterpret_cast<const i32x4*>(arow + kSlice + 16 + 128 * s) : zero;
      }
    }
  }
  // results: register r of lane (j, q) is A's row 4 q + r against column j.  Of use where q / 2 == j % 2: group
  // g = q % 2 of the column's half, activation rows 2 p (registers 0, 1: high, low bytes) and 2 p + 1 (2, 3)
  constexpr bool kTwo = kM > 1;  // one activation row: registers 2 and 3 hold nothing of use
  const int g = q & 1;
  float sx_a[kPasses][kSteps], sx_b[kPasses][kSteps], us_a[kPasses], us_b[kPasses];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int m_a = (2 * p) & (kM - 1), m_b = (2 * p + 1) & (kM - 1);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      sx_a[p][s] = sums[m_a * 4 * kSteps + 4 * s + 2 * h + g];
      sx_b[p][s] = kTwo ? sums[m_b * 4 * kSteps + 4 * s + 2 * h + g] : 0.f;
    }
    us_a[p] = unscale_m[m_a];
    us_b[p] = unscale_m[m_b];
  }

#pragma unroll
  for (int t = 1; t < kSets4; ++t) issue(t, blk_first + t);
  auto consume = [&](int set, int slot) __attribute__((always_inline)) {
    float acc_a[kPasses], acc_b[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) acc_a[p] = 0.f, acc_b[p] = 0.f;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      i32x4 ev, od;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        ev[k] = (int)(wv[set][s][k] & 0x0f0f0f0fu);
        od[k] = (int)((wv[set][s][k] >> 4) & 0x0f0f0f0fu);
      }
      // (selects between registers named at compile time: an index that depends on the lane would put the windows in memory)
      const uint32_t sd = h ? sw[set].d[2 * s + 1] : sw[set].d[2 * s];
      const uint32_t bd = h ? bw[set].d[2 * s + 1] : bw[set].d[2 * s];
      const float sc = T::to_f32((uint16_t)(g ? sd >> 16 : sd));
      const float bi = T::to_f32((uint16_t)(g ? bd >> 16 : bd));
#pragma unroll
      for (int p = 0; p < kPasses; ++p) {
        const i32x4 zero = {0, 0, 0, 0};
        i32x4 d = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa_e[p][s], ev, zero, 0, 0, 0);
        d = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa_o[p][s], od, d, 0, 0, 0);
        // sum(xq code) over the group, exact: high and low bytes of xq joined as integers
        acc_a[p] = __builtin_fmaf(sc, (float)(d[0] * 256 + d[1]), acc_a[p]);
        acc_a[p] = __builtin_fmaf(bi, sx_a[p][s], acc_a[p]);
        if constexpr (kTwo) {
          acc_b[p] = __builtin_fmaf(sc, (float)(d[2] * 256 + d[3]), acc_b[p]);
          acc_b[p] = __builtin_fmaf(bi, sx_b[p][s], acc_b[p]);
        }
      }
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      partials[((slot * kWaves + wave) * kPasses + p) * 64 + lane] = make_float2(acc_a[p] * us_a[p], acc_b[p] * us_b[p]);
  };

  // Three blocks per trip, one per register set, and between the arithmetic of two blocks the requests for the
  // block three further on; the last trip requests nothing.  A block past the run's end is computed again
  // into a slot of its own that nobody reads.
  int b = 0;
  for (; b + kSets4 < n_blocks; b += kSets4) {
#pragma unroll
    for (int t = 0; t < kSets4; ++t) {
      __builtin_amdgcn_sched_barrier(0);
      consume(t, b + t);
      __builtin_amdgcn_sched_barrier(0);
      issue(t, blk_first + b + t + kSets4);
    }
  }
#pragma unroll
  for (int t = 0; t < kSets4; ++t) {
    __builtin_amdgcn_sched_barrier(0);
    consume(t, min(b + t, n_blocks));
  }
  __syncthreads();

  // ---- one output per thread: block, weight row, activation row; per wavefront the two halves' two groups -----
#pragma unroll
  for (int i = 0; i < kOuts; ++i) {
    const int o = (int)threadIdx.x + i * 64 * kWaves;
    const int out_m = o % M, out_row8 = (o / M) % kRows4, out_blk = o / M / kRows4;
    if (out_blk >= n_blocks) break;
    const int64_t out_row = (int64_t)(blk_first + out_blk) * kRows4 + out_row8;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
#pragma unroll
      for (int hg = 0; hg < 4; ++hg) {  // half hg / 2, group hg % 2: lane (2 row + half, 2 half + group)
        const int src = (2 * out_row8 + (hg >> 1)) + 16 * hg;
        const float2 p = partials[((out_blk * kWaves + w) * kPasses + (out_m >> 1)) * 64 + src];
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

template <typename T, int kWaves, int kSteps, int kM, bool kSilu>
int launch_oct4(const void* x, int64_t M, const uint32_t* wq, const void* scales, const void* biases, const void* bias,
                int64_t N, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmv_oct4_kernel<T, kWaves, kSteps, kM, kSilu>;
  constexpr int kPasses = kM > 2 ? 2 : 1;
  constexpr int kImageBytes = ((2 * kM * (256 * kSteps + 32) + kM * 4 * kSteps * 4) + 255) & ~255;
  constexpr int kPerBlock = kWaves * kPasses * 512;
  constexpr int kLdsWanted = kWaves * kImageBytes + (kMaxBlocks4 + 1) * kPerBlock;
  constexpr int kLdsMax = kLdsWanted < 160 * 1024 ? kLdsWanted : 160 * 1024;
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLdsMax)) return MFQ_ELAUNCH;
  // one workgroup per compute unit while that is at most kMaxBlocks4 blocks each; longer weights in runs of
  // kLongRun4 blocks to as many workgroups as that takes
  const int64_t blocks = N / kRows4;
  const int64_t cus = compute_units();
  int64_t per_wg = (blocks + cus - 1) / cus;
  if (per_wg > kMaxBlocks4) per_wg = kLongRun4;
  while (kWaves * kImageBytes + ((int)per_wg + 1) * kPerBlock > kLdsMax) --per_wg;  // (many wavefronts, four rows)
  const int64_t n_wg = (blocks + per_wg - 1) / per_wg;
  const int lds = kWaves * kImageBytes + ((int)per_wg + 1) * kPerBlock;
  hipLaunchKernelGGL(kernel, dim3((unsigned)n_wg), dim3(64 * kWaves), lds, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)per_wg);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int kWaves, int kSteps, bool kSilu>
int launch_oct4_rows(const void* x, int64_t M, const uint32_t* wq, const void* scales, const void* biases,
                     const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  if (M == 1) return launch_oct4<T, kWaves, kSteps, 1, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
  if (M == 2) return launch_oct4<T, kWaves, kSteps, 2, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
  return launch_oct4<T, kWaves, kSteps, 4, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
}

template <typename T, bool kSilu>
int launch_oct4_k(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  // (K = 3072, twelve steps to a row: six wavefronts of two measured ahead of four of three and twelve of one)
  switch (K) {
    case 1024: return launch_oct4_rows<T, 4, 1, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 2048: return launch_oct4_rows<T, 8, 1, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 3072: return launch_oct4_rows<T, 6, 2, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    case 4096: return launch_oct4_rows<T, 8, 2, kSilu>(x, M, wq, scales, biases, bias, N, y, y_dtype, stream);
    default: return MFQ_EUNSUPPORTED;
  }
}

}  // namespace

// Shapes this kernel takes: 4-bit codes in groups of 64, one to four activation rows, K of 1024, 2048, 3072
// or 4096, whole eights of weight rows, x and the weights 16-byte aligned, scales and biases 4-byte aligned.
bool qmv_oct4_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* x, const void* scales,
                     const void* biases) {
  if (!(bits == 4 && gs == 64 && M >= 1 && M <= 4 && (K == 1024 || K == 2048 || K == 3072 || K == 4096) &&
        N % kRows4 == 0))
    return false;
  return aligned16(x) && ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 3u) == 0;
}

int launch_qmv_oct4(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                    hipStream_t stream, bool silu) {
  if (!qmv_oct4_covers(M, K, N, gs, bits, x, scales, biases)) return MFQ_EUNSUPPORTED;
  if (dtype != MFQ_BF16 && dtype != MFQ_F16) return MFQ_EDTYPE;
  const bool bf = dtype == MFQ_BF16;
  if (silu)
    return bf ? launch_oct4_k<BF16, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream)
              : launch_oct4_k<F16, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
  return bf ? launch_oct4_k<BF16, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream)
            : launch_oct4_k<F16, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, stream);
}

}  // namespace mfq
