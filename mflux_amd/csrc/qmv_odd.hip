// Quantized matvec for 3-, 5- and 6-bit weights and one activation row on
// gfx950: y[n] = x . dequant(W[n]) (+ bias).  These are the adaLN modulation
// linears (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12)
// of a model quantized with `-q 3`, `-q 5` or `-q 6`; without this kernel every
// such call would dequantise the whole weight first.
//
// MLX packs these widths as one little-endian bit stream per row (code i at bit
// i * bits).  One wavefront takes one weight row at a time; a lane takes units
// of 32 codes (32 * bits bits: 3, 5 or 6 whole 32-bit words, inside one group),
// unit 64 * j + lane in round j, so that a round of loads covers one contiguous
// run of the row.  A code is cut out of the stream with one shift or one
// alignbit (a compile-time position), two codes are merged into the exact
// 16-bit floats "offset + code" with one byte permute and one AND-OR
// (bfloat16 0x4300 | n = 128 + n, float16 0x6400 | n = 1024 + n), and the 4x4x4
// matrix-core instruction, whose block diagonal is a lane's own A.B, sums
// x * (offset + code) per lane and unit in float32;
//   scale * D + (bias - offset * scale) * sum(x)
// is the unit's contribution (no rounding of the weights).  The lane's slices
// of x stay in registers for the whole kernel; the next row's loads are in
// flight while the current one is consumed; the lanes' sums are added with DPP.
#include <type_traits>

#include "common.h"

namespace mfq {
namespace {

constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7-i of its half row
constexpr int kDppMirror = 0x140;      // lane i <- lane 15-i of its row

template <int kCtrl>
__device__ inline float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false));
}

// Sum over all 64 lanes, returned in every lane.
__device__ inline float wave_sum(float v) {
  v += dpp_f32<kDppXor1>(v);
  v += dpp_f32<kDppXor2>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppMirror>(v);  // every lane now holds the sum of its row of 16
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)) +
         __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
}

// The 32-bit window of a unit's words that starts at code i (the code is its low BITS bits).
template <int BITS, int kI>
__device__ inline uint32_t code_window(const uint32_t (&d)[BITS]) {
  constexpr int kPos = kI * BITS;
  constexpr int kWord = kPos >> 5, kShift = kPos & 31;
  if constexpr (kShift == 0) {
    return d[kWord];
  } else if constexpr (kShift + BITS <= 32) {
    return d[kWord] >> kShift;
  } else {
    return __builtin_amdgcn_alignbit(d[kWord + 1], d[kWord], kShift);
  }
}

// kUnits: units per lane and row, ceil(K / 32 / 64)
template <typename T, int BITS, int kUnits>
__global__ __launch_bounds__(256) void qmv_odd_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                      const uint16_t* __restrict__ scales,
                                                      const uint16_t* __restrict__ biases,
                                                      const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                      int y_is_f32, int N, int K, int gs_shift, int rows_per_wave,
                                                      int extra_rows) {
  using CF = CodeFloat<T>;
  constexpr float kOffset = CF::kOffset4;  // the magic for values below 128 / 1024
  const int lane = threadIdx.x & (kWave - 1);
  const int row_words = K * BITS / 32;
  const int groups = K >> gs_shift;

  // this lane's units: first word inside a row, group, the matching slices of
  // x (four values per matrix instruction, in code order) and their sums.  A
  // unit past the end of the row re-reads the row's first unit against x = 0.
  int word0[kUnits], grp[kUnits];
  uint2 xq[kUnits][8];
  float sx[kUnits];
#pragma unroll
  for (int j = 0; j < kUnits; ++j) {
    const int k0 = (j * kWave + lane) * 32;
    const bool in_row = k0 < K;
    word0[j] = in_row ? (j * kWave + lane) * BITS : 0;
    grp[j] = in_row ? (k0 >> gs_shift) : 0;
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      uint2 v = {0, 0};
      if (in_row) v = *reinterpret_cast<const uint2*>(x + k0 + 4 * t);
      xq[j][t] = v;
      sum += T::to_f32((uint16_t)v.x) + T::to_f32((uint16_t)(v.x >> 16)) + T::to_f32((uint16_t)v.y) +
             T::to_f32((uint16_t)(v.y >> 16));
    }
    sx[j] = sum;
  }

  // rows are dealt to wavefronts in contiguous, balanced runs (split computed on the host)
  // (the wavefront index read as a scalar: row addresses then live in scalar registers)
  const int wave_id = blockIdx.x * (blockDim.x / kWave) + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t row_begin = (int64_t)wave_id * rows_per_wave + min(wave_id, extra_rows);
  const int64_t row_end = row_begin + rows_per_wave + (wave_id < extra_rows ? 1 : 0);
  if (row_begin >= row_end) return;

  uint32_t pair_mask = (uint32_t)((1 << BITS) - 1) * 0x00010001u;
  uint32_t magic = CF::kNibble;
  asm volatile("" : "+s"(pair_mask), "+v"(magic));

  struct __attribute__((packed, aligned(4))) Unit {  // loaded as 128-, 96- and 64-bit pieces
    uint32_t d[BITS];
  };
  struct Row {
    uint32_t w[kUnits][BITS];
    uint16_t s[kUnits], b[kUnits];
    uint16_t bias;
  };
  auto issue = [&](Row& r, int64_t row) __attribute__((always_inline)) {
    const uint32_t* wrow = wq + row * row_words;
    const uint16_t* srow = scales + row * groups;
    const uint16_t* brow = biases + row * groups;
    // scales before codes: loads return in order, and a unit cannot be finished before its scale is there
#pragma unroll
    for (int j = 0; j < kUnits; ++j) {
      r.s[j] = srow[grp[j]];
      r.b[j] = brow[grp[j]];
    }
#pragma unroll
    for (int j = 0; j < kUnits; ++j) {
      const Unit u = *reinterpret_cast<const Unit*>(wrow + word0[j]);
#pragma unroll
      for (int e = 0; e < BITS; ++e) r.w[j][e] = u.d[e];
    }
    r.bias = (bias ? bias + row : srow)[0];  // without a bias: any readable address, the value is not used
  };

  uint32_t kept = 0;  // lane i: the finished output of the i-th row of the wavefront's run
  auto consume = [&](const Row& r, int64_t row) __attribute__((always_inline)) {
    f32x4 tot = {0.f, 0.f, 0.f, 0.f};  // register lane%4: this lane's sum of scale * D over its units
    float corr = 0.f;                  // this lane's sum of (bias - offset * scale) * sum(x)
#pragma unroll
    for (int j = 0; j < kUnits; ++j) {
      const float sc = T::to_f32(r.s[j]);
      const float bi = T::to_f32(r.b[j]);
      f32x4 d = {0.f, 0.f, 0.f, 0.f}, d2 = {0.f, 0.f, 0.f, 0.f};
      auto quad = [&](auto tc) __attribute__((always_inline)) {
        constexpr int t = decltype(tc)::value;  // codes 4t .. 4t+3
        // bytes: code a -> byte 0, code b -> byte 2, zero elsewhere; the mask drops the stream's next bits
        const uint32_t p0 = __builtin_amdgcn_perm(code_window<BITS, 4 * t + 1>(r.w[j]), code_window<BITS, 4 * t>(r.w[j]),
                                                  0x0c040c00u);
        const uint32_t p1 = __builtin_amdgcn_perm(code_window<BITS, 4 * t + 3>(r.w[j]),
                                                  code_window<BITS, 4 * t + 2>(r.w[j]), 0x0c040c00u);
        const uint2 a = make_uint2((p0 & pair_mask) | magic, (p1 & pair_mask) | magic);
        if (t & 1) {
          d2 = CF::mfma4(a, xq[j][t], d2);
        } else {
          d = CF::mfma4(a, xq[j][t], d);
        }
      };
      quad(std::integral_constant<int, 0>{});
      quad(std::integral_constant<int, 1>{});
      quad(std::integral_constant<int, 2>{});
      quad(std::integral_constant<int, 3>{});
      quad(std::integral_constant<int, 4>{});
      quad(std::integral_constant<int, 5>{});
      quad(std::integral_constant<int, 6>{});
      quad(std::integral_constant<int, 7>{});
      const float bo = __builtin_fmaf(-kOffset, sc, bi);
#pragma unroll
      for (int e = 0; e < 4; ++e) tot[e] = __builtin_fmaf(sc, d[e] + d2[e], tot[e]);
      corr = __builtin_fmaf(bo, sx[j], corr);
    }
    const int diag = lane & 3;
    float v = (diag == 0 ? tot[0] : diag == 1 ? tot[1] : diag == 2 ? tot[2] : tot[3]) + corr;
    v = wave_sum(v);  // in every lane; lane (row - row_begin) % 64 keeps the row's output until the run ends
    // (selects, not branches: the loop body stays one block, which keeps the requests where they are put)
    const float bv = T::to_f32(r.bias);
    const float v32 = bias ? v + bv : v;
    const uint16_t h0 = T::from_f32(v);
    const uint16_t h1 = T::from_f32(T::to_f32(h0) + bv);  // second rounding, as a separate add on the 16-bit result
    const uint32_t out = y_is_f32 ? __builtin_bit_cast(uint32_t, v32) : (uint32_t)(bias ? h1 : h0);
    kept = lane == (int)((row - row_begin) & 63) ? out : kept;
  };

  // Two rows in flight per wavefront: row r + 1 is requested before row r is
  // consumed.  Inside the loop nothing is conditional and nothing is stored:
  // behind a branch the compiler cannot know how many younger loads are in
  // flight when it waits for row r, and waits for all of them (a store between
  // the loads has the same effect).  So the loop takes rows in pairs, an odd run
  // consumes its first row ahead of it (the loop then starts on the other
  // register set), the request past the run's last row re-reads that row, and
  // the run's outputs (at most 64, the launcher sees to it) leave together.
  Row rr[2];
  issue(rr[0], row_begin);
  const int64_t last = row_end - 1;
  auto fence = [] () __attribute__((always_inline)) {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  auto pairs = [&](auto parity, int64_t first) __attribute__((always_inline)) {
    constexpr int kP = decltype(parity)::value;  // register set that holds row `first`
    for (int64_t row = first; row < row_end; row += 2) {
      // the requests stay between the arithmetic of two rows, in front of the waits for the older row
      // (the empty asm keeps the optimiser, the scheduling barrier the scheduler from moving them)
      fence();
      issue(rr[kP ^ 1], row + 1);
      fence();
      consume(rr[kP], row);
      fence();
      issue(rr[kP], min(row + 2, last));
      fence();
      consume(rr[kP ^ 1], row + 1);
    }
  };
  if ((row_end - row_begin) & 1) {
    issue(rr[1], min(row_begin + 1, last));
    fence();
    consume(rr[0], row_begin);
    pairs(std::integral_constant<int, 1>{}, row_begin + 1);
  } else {
    pairs(std::integral_constant<int, 0>{}, row_begin);
  }
  if (lane < (int)(row_end - row_begin)) {
    if (y_is_f32) {
      reinterpret_cast<uint32_t*>(y)[row_begin + lane] = kept;
    } else {
      reinterpret_cast<uint16_t*>(y)[row_begin + lane] = (uint16_t)kept;
    }
  }
}

template <typename T, int BITS, int kUnits>
int launch_kernel(const void* x, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmv_odd_kernel<T, BITS, kUnits>;
  static PerDeviceInt cache;
  const int blocks_per_cu = cache.get([&] {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess || n < 1) n = 1;
    return n > 4 ? 4 : n;
  });
  // as many workgroups as are resident at once, so that every wavefront gets one balanced run of rows
  int64_t blocks = (int64_t)compute_units() * blocks_per_cu;
  const int64_t max_blocks = (N + 3) / 4;
  if (blocks > max_blocks) blocks = max_blocks;
  const int64_t min_blocks = (N + 255) / 256;  // at most 64 rows per wavefront: a lane keeps one result
  if (blocks < min_blocks) blocks = min_blocks;
  const int64_t n_waves = blocks * 4;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)N, (int)K, gs_shift, (int)(N / n_waves), (int)(N % n_waves));
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int BITS>
int launch_units(int64_t units, const void* x, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                 const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  switch (units) {
    case 1: return launch_kernel<T, BITS, 1>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    case 2: return launch_kernel<T, BITS, 2>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    case 3: return launch_kernel<T, BITS, 3>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    case 4: return launch_kernel<T, BITS, 4>(x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    default: return MFQ_EUNSUPPORTED;
  }
}

template <typename T>
int launch_bits(int64_t units, int bits, const void* x, int64_t K, const uint32_t* wq, const void* scales,
                const void* biases, const void* bias, int64_t N, int gs_shift, void* y, int y_dtype,
                hipStream_t stream) {
  switch (bits) {
    case 3: return launch_units<T, 3>(units, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    case 5: return launch_units<T, 5>(units, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    case 6: return launch_units<T, 6>(units, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
    default: return MFQ_EUNSUPPORTED;
  }
}

}  // namespace

// One activation row against 3-, 5- or 6-bit weights with rows of at most 8192
// codes; anything else is MFQ_EUNSUPPORTED (the caller dequantises and uses a
// plain GEMM).
int launch_qmv_odd(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   hipStream_t stream) {
  if (M != 1 || K % 32 || K > 8192) return MFQ_EUNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(x) & 7u) != 0) return MFQ_EUNSUPPORTED;
  const int gs_shift = gs == 32 ? 5 : gs == 64 ? 6 : 7;
  const int64_t units = (K / 32 + kWave - 1) / kWave;
  if (dtype == MFQ_BF16)
    return launch_bits<BF16>(units, bits, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  if (dtype == MFQ_F16)
    return launch_bits<F16>(units, bits, x, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
