// One activation row against a W4/W8 weight for gfx950, on the integer dot
// product of the vector pipeline:  y[N] = x[K] @ dequant(wq[N, K])^T (+ bias),
// the adaLN modulation call of every DiT block
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12,
// src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37).
//
// The kernel is bound by streaming the packed weight from HBM once, provided
// the arithmetic per code stays small.  Codes are unsigned integers, so the
// row of x is turned into integers as well, once per workgroup: with 2^e the
// power of two that brings the row's largest magnitude just below 2^14,
//   xq = rint(x * 2^e)   (|xq| <= 2^14; the rounding error, 2^-15 of the row's
//                         largest element, is far below one bfloat16 ulp of y)
//   xq = 256 * xh + xl,  xh and xl signed bytes,
// and four codes of a weight word meet four bytes of xh, then of xl, in one
// v_dot4 instruction each.  Per 16-byte piece of a weight row (one group or
// less) the integer sums give  D = sum(xq * code)  exactly, and with
// Sx = sum(xq) over the piece
//   sum(x * (scale * code + bias)) * 2^e = scale * D + bias * Sx,
// two float32 fma per piece.  An 8-bit code enters as the signed byte
// code - 128 (one XOR per word), which moves 128 * scale into the Sx term; a
// 4-bit word is split into its even and odd nibbles (three instructions).
// That is 3 (W8) or 7 (W4) vector instructions per 32-bit word of weights and
// no conversion of a code to floating point at all.
//
// Layout of the work as in the matrix-core kernel it replaces for these
// shapes: one wavefront per weight row at a time, lane l takes the 16-byte
// pieces 64 j + l of the row (every load instruction covers one contiguous
// KiB), the next row's loads are in flight while a row is consumed, a row's
// scales and biases come as one cooperative load, rows are dealt to the
// wavefronts in balanced contiguous runs.  The integer image of x is built by
// the workgroup's four wavefronts together, through LDS, and then held in
// registers.
#include <type_traits>

#include "common.h"

namespace mfq {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;      // lane i <- lane 15-i of its row

template <int kCtrl>
__device__ inline int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xf, 0xf, false);
}

// Sum / maximum over all 64 lanes, returned in every lane.
__device__ inline float wave_sum(float v) {
  v += __builtin_bit_cast(float, dpp_i32<kDppXor1>(__builtin_bit_cast(int, v)));
  v += __builtin_bit_cast(float, dpp_i32<kDppXor2>(__builtin_bit_cast(int, v)));
  v += __builtin_bit_cast(float, dpp_i32<kDppHalfMirror>(__builtin_bit_cast(int, v)));
  v += __builtin_bit_cast(float, dpp_i32<kDppMirror>(__builtin_bit_cast(int, v)));  // sum of the lane's row of 16
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
}
__device__ inline int wave_max(int v) {
  v = max(v, dpp_i32<kDppXor1>(v));
  v = max(v, dpp_i32<kDppXor2>(v));
  v = max(v, dpp_i32<kDppHalfMirror>(v));
  v = max(v, dpp_i32<kDppMirror>(v));
  return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

template <typename T, int BITS, int kLoads, bool kCoop>
struct DotRow {
  u32x4 w[kLoads];
  uint16_t s[kLoads], b[kLoads];  // per-lane loads (when `kCoop` is off)
  uint32_t sb;                    // cooperative load: lanes 0..31 hold scale pairs, 32..63 bias pairs

  // Every load is unconditional (addresses past the row's end are clamped into
  // it; what they bring meets zeros of x), so that the number of loads in
  // flight is known when the kernel waits for older ones.
  __device__ inline void issue(const char* wq, const uint16_t* scales, const uint16_t* biases,
                               int64_t row, int row_bytes, int groups, const int (&piece)[kLoads],
                               const int (&grp)[kLoads], int lane) {
    const char* wrow = wq + row * row_bytes;
    const uint16_t* srow = scales + row * groups;
    const uint16_t* brow = biases + row * groups;
    if constexpr (kCoop) {
      const int i = min(lane & 31, groups / 2 - 1);
      sb = reinterpret_cast<const uint32_t*>(lane < 32 ? srow : brow)[i];
    } else {
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        s[j] = srow[grp[j]];
        b[j] = brow[grp[j]];
      }
    }
#pragma unroll
    for (int j = 0; j < kLoads; ++j)
      w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + piece[j]));
  }
};

template <typename T, int BITS, int kLoads, bool kCoop, bool kSilu>
__global__ __launch_bounds__(256) void qmv_dot_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                      const uint16_t* __restrict__ scales,
                                                      const uint16_t* __restrict__ biases,
                                                      const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                      int y_is_f32, int N, int K, int gs_shift, int rows_per_wave,
                                                      int extra_rows) {
  using R = DotRow<T, BITS, kLoads, kCoop>;
  constexpr int kCodes = 128 / BITS;         // codes in one 16-byte piece
  constexpr int kXWords = BITS == 8 ? 8 : 16;  // 32-bit words of x image per piece
  extern __shared__ __attribute__((aligned(16))) uint32_t ximg[];  // [pieces][kXWords]
  __shared__ int wave_amax[4];
  const int lane = threadIdx.x & (kWave - 1);
  // uniform over the wavefront, and known to be: row addresses then live in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int row_bytes = K * BITS / 8;
  const int groups = K >> gs_shift;

  // ---- the integer image of x, built by the workgroup ---------------------------
  // chunk c = 4 consecutive k (W8) / 8 consecutive k (W4): the k of one weight word.
  // A thread converts chunks t, t + 256, ...: row_bytes / 1024 <= kLoads of them.
  constexpr int kChunkK = BITS == 8 ? 4 : 8;
  constexpr int kRawWords = kChunkK / 2;
  const int n_chunks = K / kChunkK;
  uint32_t raw[kLoads][kRawWords];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int c = min((int)threadIdx.x + 256 * i, n_chunks - 1);  // past the end: the last chunk again, not stored
    if constexpr (BITS == 8) {
      const uint2 v = *reinterpret_cast<const uint2*>(x + 4 * c);
      raw[i][0] = v.x;
      raw[i][1] = v.y;
    } else {
      const u32x4 v = *reinterpret_cast<const u32x4*>(x + 8 * c);
#pragma unroll
      for (int q = 0; q < 4; ++q) raw[i][q] = v[q];
    }
  }

  // this lane's pieces of a row, and the loads of the wavefront's first row: issued
  // behind the loads of x, they travel while x is converted (loads return in order)
  int piece[kLoads], grp[kLoads];
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const int p = j * kWave + lane;
    const bool in_row = p * 16 < row_bytes;
    piece[j] = in_row ? p * 16 : row_bytes - 16;  // past the end: the row's last piece again, against zeros of x
    grp[j] = in_row ? (p * kCodes) >> gs_shift : 0;
  }
  const int wave_id = blockIdx.x * 4 + wave;
  const int64_t row_begin = (int64_t)wave_id * rows_per_wave + min(wave_id, extra_rows);
  const int64_t row_end = row_begin + rows_per_wave + (wave_id < extra_rows ? 1 : 0);
  const char* wbytes = reinterpret_cast<const char*>(wq);
  // the layer's bias of the row whose result this lane will keep (lane i: the i-th row of the run), requested
  // ahead of the rows so that it has arrived with the first of them (loads return in order)
  const uint16_t lane_bias = (bias ? bias : scales)[min(row_begin + lane, (int64_t)N - 1)];
  R regs[2];
  // (a wavefront without rows, which a grid rounded up to whole workgroups can leave, re-reads the last row)
  regs[0].issue(wbytes, scales, biases, min(row_begin, (int64_t)N - 1), row_bytes, groups, piece, grp, lane);

  if constexpr (kSilu) {  // the activation in front of the linear, on the values as they arrive
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      if (wave * kWave + 256 * i >= n_chunks) continue;  // a wavefront whose chunks all lie past the end
#pragma unroll
      for (int q = 0; q < kRawWords; ++q) raw[i][q] = silu_pair<T>(raw[i][q]);
    }
  }
  int amax = 0;
#pragma unroll
  for (int i = 0; i < kLoads; ++i)
#pragma unroll
    for (int q = 0; q < kRawWords; ++q) amax = max(amax, mag_bits(raw[i][q]));
  amax = wave_max(amax);
  if (lane == 0) wave_amax[wave] = amax;
  __syncthreads();
  amax = max(max(wave_amax[0], wave_amax[1]), max(wave_amax[2], wave_amax[3]));
  const int e = scale_exponent<T>(amax);
  const float mult = pow2(e);
  // an infinity or NaN anywhere in x: every output is NaN
  const float unscale = not_finite<T>(amax) ? __builtin_nanf("") : pow2(-e);
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c >= n_chunks) continue;
    if constexpr (BITS == 8) {
      // piece c / 4, word c % 4: high bytes in words 0..3 of the piece, low bytes in 4..7
      uint32_t hi, lo;
      split4<T>(raw[i][0], raw[i][1], mult, hi, lo);
      ximg[(c >> 2) * 8 + (c & 3)] = hi;
      ximg[(c >> 2) * 8 + 4 + (c & 3)] = lo;
    } else {
      // a weight word holds codes k0..k0+7; its even nibbles are k0, k0+2, k0+4, k0+6.  Per word four
      // image words: high bytes of the even k, of the odd k, low bytes of the even k, of the odd k.
      // raw[i][q] = (x[2q], x[2q+1]): even k in the low halves
      const uint32_t ev0 = (raw[i][0] & 0xffffu) | (raw[i][1] << 16), ev1 = (raw[i][2] & 0xffffu) | (raw[i][3] << 16);
      const uint32_t od0 = (raw[i][0] >> 16) | (raw[i][1] & 0xffff0000u);
      const uint32_t od1 = (raw[i][2] >> 16) | (raw[i][3] & 0xffff0000u);
      uint32_t hi_e, lo_e, hi_o, lo_o;
      split4<T>(ev0, ev1, mult, hi_e, lo_e);
      split4<T>(od0, od1, mult, hi_o, lo_o);
      *reinterpret_cast<u32x4*>(ximg + c * 4) = u32x4{hi_e, hi_o, lo_e, lo_o};
    }
  }
  __syncthreads();

  // ---- the image of this lane's pieces, into registers -----------------------------
  uint32_t xw[kLoads][kXWords];
  float sx[kLoads];
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const int p = j * kWave + lane;
    const bool in_row = p * 16 < row_bytes;
    int sum_hi = 0, sum_lo = 0;
#pragma unroll
    for (int q = 0; q < kXWords / 4; ++q) {
      u32x4 v = {0, 0, 0, 0};
      if (in_row) v = *reinterpret_cast<const u32x4*>(ximg + p * kXWords + 4 * q);
#pragma unroll
      for (int i = 0; i < 4; ++i) xw[j][4 * q + i] = v[i];
    }
#pragma unroll
    for (int i = 0; i < kXWords; ++i) {
      const bool high = BITS == 8 ? i < 4 : (i & 3) < 2;
      if (high) {
        sum_hi = __builtin_amdgcn_sdot4((int)xw[j][i], 0x01010101, sum_hi, false);
      } else {
        sum_lo = __builtin_amdgcn_sdot4((int)xw[j][i], 0x01010101, sum_lo, false);
      }
    }
    sx[j] = (float)(sum_hi * 256 + sum_lo);
  }

  if (row_begin >= row_end) return;  // behind the last barrier

  float kept = 0.f;  // lane i: the sum of the i-th row of the run in hand
  auto consume = [&](const R& regs, int64_t row) __attribute__((always_inline)) {
    float tot = 0.f;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      float sc, bi;
      if constexpr (kCoop) {
        const int src = (grp[j] >> 1) * 4;  // byte address of the lane that holds the pair
        const uint32_t sp = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)regs.sb);
        const uint32_t bp = (uint32_t)__builtin_amdgcn_ds_bpermute(src + 128, (int)regs.sb);
        const int sh = (grp[j] & 1) * 16;
        sc = T::to_f32((uint16_t)(sp >> sh));
        bi = T::to_f32((uint16_t)(bp >> sh));
      } else {
        sc = T::to_f32(regs.s[j]);
        bi = T::to_f32(regs.b[j]);
      }
      int dh = 0, dl = 0;
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {
        const uint32_t w = regs.w[j][wd];
        if constexpr (BITS == 8) {
          const int c = (int)(w ^ 0x80808080u);  // code - 128 as signed bytes
          dh = __builtin_amdgcn_sdot4(c, (int)xw[j][wd], dh, false);
          dl = __builtin_amdgcn_sdot4(c, (int)xw[j][4 + wd], dl, false);
        } else {
          const int ev = (int)(w & 0x0f0f0f0fu), od = (int)((w >> 4) & 0x0f0f0f0fu);
          dh = __builtin_amdgcn_sdot4(ev, (int)xw[j][4 * wd], dh, false);
          dh = __builtin_amdgcn_sdot4(od, (int)xw[j][4 * wd + 1], dh, false);
          dl = __builtin_amdgcn_sdot4(ev, (int)xw[j][4 * wd + 2], dl, false);
          dl = __builtin_amdgcn_sdot4(od, (int)xw[j][4 * wd + 3], dl, false);
        }
      }
      const float d = (float)(dh * 256 + dl);
      // 8 bits: code = (code - 128) + 128, and the 128 joins the bias in front of Sx
      const float bo = BITS == 8 ? __builtin_fmaf(128.f, sc, bi) : bi;
      tot = __builtin_fmaf(sc, d, tot);
      tot = __builtin_fmaf(bo, sx[j], tot);
    }
    // every lane holds the row's result; lane (row - row_begin) % 64 keeps it until flush()
    // (selects, not branches: the loop body stays one block, which keeps the requests where they are put)
    // (scaling back, the layer's bias and the roundings wait for flush(), where every lane does its own row's)
    const float v = wave_sum(tot);
    kept = lane == (int)((row - row_begin) & 63) ? v : kept;
  };
  // Stores the results of rows [first, first + count), count <= 64, one per lane.
  // Results leave the wavefront once, at its end, and not row by row: a store
  // in flight between the loads would make every wait for a load a wait for
  // everything (loads and stores share one counter and may overtake each other).
  auto flush = [&](int64_t first, int count) {
    const float v = kept * unscale;
    const float bv = T::to_f32(lane_bias);
    if (lane < count) {
      if (y_is_f32) {
        reinterpret_cast<float*>(y)[first + lane] = bias ? v + bv : v;
      } else {
        const uint16_t h0 = T::from_f32(v);
        const uint16_t h1 = T::from_f32(T::to_f32(h0) + bv);  // second rounding, as a separate add on the 16-bit result
        reinterpret_cast<uint16_t*>(y)[first + lane] = bias ? h1 : h0;
      }
    }
  };

  // Two rows in flight per wavefront: row r + 1 is requested before row r is
  // consumed.  Inside the loop nothing is conditional: behind a branch the
  // compiler cannot know how many younger loads are in flight when it waits for
  // row r, and waits for all of them.  So the loop takes rows in pairs, an odd
  // run consumes its first row ahead of it (the loop then starts on the other
  // register set), and the request past the run's last row re-reads that row
  // (an L2 hit that is never consumed).
  const int64_t last = row_end - 1;
  auto pairs = [&](auto parity, int64_t first) __attribute__((always_inline)) {
    constexpr int kP = decltype(parity)::value;  // register set that holds row `first`
    for (int64_t row = first; row < row_end; row += 2) {
      // the requests stay between the arithmetic of two rows, in front of the waits for the older row
      __builtin_amdgcn_sched_barrier(0);
      regs[kP ^ 1].issue(wbytes, scales, biases, row + 1, row_bytes, groups, piece, grp, lane);
      __builtin_amdgcn_sched_barrier(0);
      consume(regs[kP], row);
      __builtin_amdgcn_sched_barrier(0);
      regs[kP].issue(wbytes, scales, biases, min(row + 2, last), row_bytes, groups, piece, grp, lane);
      __builtin_amdgcn_sched_barrier(0);
      consume(regs[kP ^ 1], row + 1);
    }
  };
  if ((row_end - row_begin) & 1) {
    regs[1].issue(wbytes, scales, biases, min(row_begin + 1, last), row_bytes, groups, piece, grp, lane);
    __builtin_amdgcn_sched_barrier(0);
    consume(regs[0], row_begin);
    pairs(std::integral_constant<int, 1>{}, row_begin + 1);
  } else {
    pairs(std::integral_constant<int, 0>{}, row_begin);
  }
  flush(row_begin, (int)(row_end - row_begin));  // at most 64 rows per wavefront (the launcher sees to it)
}

template <typename T, int BITS, int kLoads, bool kCoop, bool kSilu>
int launch_kernel(const void* x, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmv_dot_kernel<T, BITS, kLoads, kCoop, kSilu>;
  const size_t lds = (size_t)(K * BITS / 8 / 16) * (BITS == 8 ? 8 : 16) * 4;  // the x image: 2 bytes per element
  static PerDeviceInt cache;  // workgroups of this instantiation a compute unit holds
  const int resident = cache.get([&] {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, lds) != hipSuccess || n < 1) n = 1;
    return n > 4 ? 4 : n;
  });
  // Workgroups per compute unit: enough wavefronts for about 48 KiB of weight rows in flight (two
  // rows each), not more: every workgroup pays for its own image of x.  Measured at K = 3072: two
  // workgroups for 3 KiB rows (W8), four for 1.5 KiB rows (W4).  One fewer when that deals the rows
  // out evenly and the count in hand does not (18432 rows: 6 each on 3072 wavefronts, 4.5 on 4096).
  const int64_t row_bytes = K * BITS / 8;
  int per_cu = (int)((48 * 1024 / (2 * row_bytes) + 3) / 4);
  per_cu = per_cu < 2 ? 2 : per_cu > 4 ? 4 : per_cu;
  auto uneven = [&](int b) {
    const int64_t waves = (int64_t)compute_units() * b * 4;
    return N % waves != 0 && N > waves;
  };
  if (per_cu > 2 && uneven(per_cu) && !uneven(per_cu - 1)) --per_cu;
  if (per_cu > resident) per_cu = resident;
  int64_t blocks = (int64_t)compute_units() * per_cu;
  const int64_t max_blocks = (N + 3) / 4;  // at least one row per wavefront
  if (blocks > max_blocks) blocks = max_blocks;
  const int64_t min_blocks = (N + 255) / 256;  // at most 64 rows per wavefront: a lane keeps one result
  if (blocks < min_blocks) blocks = min_blocks;
  const int64_t n_waves = blocks * 4;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), lds, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)N, (int)K, gs_shift, (int)(N / n_waves), (int)(N % n_waves));
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int BITS, int kLoads, bool kSilu>
int launch_loads(int64_t n_loads, const void* x, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                 const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  if (n_loads == kLoads) {
    const int64_t groups = K >> gs_shift;
    const bool coop = groups <= 64 && groups % 2 == 0 &&
                      ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 3u) == 0;
    if (coop)
      return launch_kernel<T, BITS, kLoads, true, kSilu>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    return launch_kernel<T, BITS, kLoads, false, kSilu>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  }
  if constexpr (kLoads > 1)
    return launch_loads<T, BITS, kLoads - 1, kSilu>(n_loads, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype,
                                                    stream);
  return MFQ_EUNSUPPORTED;
}

// KiB-sized loads per row the kernel is instantiated for: the x image of a
// piece takes 8 (W8) or 16 (W4) registers
constexpr int kMaxLoadsW8 = 6;
constexpr int kMaxLoadsW4 = 3;

template <typename T, bool kSilu>
int launch_type(const void* x, int64_t K, const uint32_t* wq, const void* scales, const void* biases, const void* bias,
                int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  const int gs_shift = gs == 32 ? 5 : gs == 64 ? 6 : 7;
  const int64_t n = (K * bits / 8 + 1023) / 1024;
  if (bits == 8)
    return launch_loads<T, 8, kMaxLoadsW8, kSilu>(n, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  return launch_loads<T, 4, kMaxLoadsW4, kSilu>(n, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
}

}  // namespace

bool qmv_dot_covers(int64_t M, int64_t K, int bits) {
  const int64_t n = (K * bits / 8 + 1023) / 1024;
  return M == 1 && ((bits == 8 && n <= kMaxLoadsW8) || (bits == 4 && n <= kMaxLoadsW4));
}

int launch_qmv_dot(const void* x, int dtype, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                   const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream,
                   bool silu) {
  if (dtype != MFQ_BF16 && dtype != MFQ_F16) return MFQ_EDTYPE;
  const bool bf = dtype == MFQ_BF16;
  if (silu)
    return bf ? launch_type<BF16, true>(x, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream)
              : launch_type<F16, true>(x, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return bf ? launch_type<BF16, false>(x, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream)
            : launch_type<F16, false>(x, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
}

}  // namespace mfq
