// Small-M (M <= 16) quantized matvec for gfx950: y = x @ dequant(W)^T (+ bias).
//
// This is the adaLN modulation shape of every DiT block in mflux
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12,
// src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37):
// one or a few activation rows against a wide weight, so the kernel is bound
// by streaming the packed weight from HBM once.
//
// Two kernels here.  One activation row against rows of up to 6 KiB (W8) or
// 3 KiB (W4) of codes, which is every such call mflux makes, runs the integer
// dot-product kernel of qmv_dot.hip; two to four activation rows the kernel of
// qmv_quad.hip.
//
// qmv_rows_kernel (M <= 4, rows of at most 6 KiB of codes): one wavefront per
// weight row at a time.  The lanes read the row as consecutive 16-byte pieces
// (lane l takes piece 64*j + l of the row in load j), i.e. every load
// instruction covers one contiguous KiB, which is the access pattern that
// reaches HBM speed; loads of the next row are in flight while the current one
// is consumed.  A lane owns the 8-element slices of x that match its pieces,
// held in registers for the whole kernel, and a piece lies inside one group.
// The codes are never converted: one AND-OR per pair of codes turns them into
// exact 16-bit floats "offset + code" (bfloat16 0x4300 | n = 128 + n for a
// 4-bit value, 0x4500 | n = 2048 + 16 n for the high half of an 8-bit code;
// float16 0x6400 | n = 1024 + n), and the 4x4x4 matrix-core instruction, whose
// 16 independent blocks multiply a lane's four A values with the same lane's
// four B values on the block diagonal, accumulates sum(x * (offset + code))
// per lane and piece in float32.  With the lane's sum of x over the piece, Sx,
//   sum(x * (scale * code + bias)) = scale * D + (bias - offset * scale) * Sx,
// two float32 fma per piece.  Against dequantising first, this leaves the
// weights unrounded (closer to exact arithmetic) and takes a quarter of the
// vector instructions.  The lanes' sums are added across the wavefront when
// the row ends.
//
// qmv_kernel (everything else up to M = 16): a workgroup of four wavefronts
// owns 16 output features and walks K in phases.  Every lane streams 128-bit
// pieces of "its" weight row (row = lane % 16), dequantises them in registers,
// and feeds them to the matrix core as the A operand; the B operand is the
// matching slice of x (column = lane % 16 = activation row, zero beyond M), so
// all M <= 16 rows come at the cost of one.  x is staged through LDS one phase
// ahead and the weight loads of phase p+1 are issued before the arithmetic of
// phase p.  The four wavefronts split each phase and combine their float32
// sums through LDS.
//
// In both kernels the order of k inside a product is permuted consistently for
// both operands, which a dot product does not notice.
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

// ---------------------------------------------------------------------------
// one wavefront per weight row
// ---------------------------------------------------------------------------
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

template <typename T, int BITS, int kM, int kMaxLoads, bool kCoop>
struct RowRegs {
  u32x4 w[kMaxLoads];
  uint16_t s[kMaxLoads], b[kMaxLoads];  // per-lane loads (when `coop` is off)
  uint32_t sb;                          // cooperative load: lanes 0..31 hold scale pairs, 32..63 bias pairs
  uint16_t bias;

  // piece[j]: byte offset of this lane's piece of load j inside a row, or -1
  // past the end of the row; grp[j]: its group index
  __device__ inline void issue(const char* wq, const uint16_t* scales, const uint16_t* biases, const uint16_t* bias_v,
                               int64_t row, int row_bytes, int groups, const int (&piece)[kMaxLoads],
                               const int (&grp)[kMaxLoads], int lane) {
    const char* wrow = wq + row * row_bytes;
    const uint16_t* srow = scales + row * groups;
    const uint16_t* brow = biases + row * groups;
    if constexpr (kCoop) {
      // one load instruction for the whole row's scales and biases (at most 64
      // groups, an even number): lane i < 32 takes scales 2i, 2i+1, lane 32+i
      // the biases; consume() hands them to the lanes that need them
      const int i = lane & 31;
      const uint32_t* src = reinterpret_cast<const uint32_t*>(lane < 32 ? srow : brow);
      sb = 2 * i < groups ? src[i] : 0u;
    } else {
#pragma unroll
      for (int j = 0; j < kMaxLoads; ++j) {
        s[j] = srow[grp[j]];
        b[j] = brow[grp[j]];
      }
    }
    // codes after the scales: loads return in order, and the first piece cannot
    // be dequantised before its scale is there
#pragma unroll
    for (int j = 0; j < kMaxLoads; ++j) {
      if (piece[j] >= 0) {
        w[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + piece[j]));
      } else {
        w[j] = u32x4{0, 0, 0, 0};
      }
    }
    bias = bias_v ? bias_v[row] : (uint16_t)0;
  }
};

// The 4x4x4 instruction: lane l belongs to block l/4 and holds row l%4 of the
// block's A (4 k values) and column l%4 of its B; result register i of the lane
// is element (i, l%4) of the block's product, so register l%4 is the dot
// product of the lane's own A and B values.
template <typename T, int BITS, int kM, int kMaxLoads, bool kCoop>
__global__ __launch_bounds__(256) void qmv_rows_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                       const uint16_t* __restrict__ scales,
                                                       const uint16_t* __restrict__ biases,
                                                       const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                       int y_is_f32, int M, int N, int K, int gs_shift, int rows_per_wave,
                                                       int extra_rows) {
  using R = RowRegs<T, BITS, kM, kMaxLoads, kCoop>;
  using CF = CodeFloat<T>;
  constexpr int kCodes = 128 / BITS;     // codes in one 16-byte piece
  constexpr int kPerWord = 32 / BITS;    // codes in one 32-bit word
  constexpr int kXOps = kCodes / 4;      // B operands (4 values of x each) per piece
  constexpr float kOffset = BITS == 4 ? CF::kOffset4 : CF::kOffset8;
  const int lane = threadIdx.x & (kWave - 1);
  const int row_bytes = K * BITS / 8;
  const int groups = K >> gs_shift;  // the launcher picked kMaxLoads = ceil(row_bytes / 1024)

  // this lane's pieces: position in the row, group, its slices of x in the
  // order the code pairs come out of a word, and the sum of each slice
  int piece[kMaxLoads], grp[kMaxLoads];
  uint2 xq[kM][kMaxLoads][kXOps];
  float sx[kM][kMaxLoads];
#pragma unroll
  for (int j = 0; j < kMaxLoads; ++j) {
    const int off = (j * kWave + lane) * 16;
    const bool in_row = off < row_bytes;
    const int k0 = (j * kWave + lane) * kCodes;
    piece[j] = in_row ? off : -1;
    grp[j] = in_row ? (k0 >> gs_shift) : 0;
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      float sum = 0.f;
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {  // the piece's four words
        if constexpr (BITS == 4) {
          // word = codes c0..c7; pairs (c0,c4) (c1,c5) | (c2,c6) (c3,c7)
          u32x4 v = {0, 0, 0, 0};
          if (in_row && m < M) v = *reinterpret_cast<const u32x4*>(x + (int64_t)m * K + k0 + 8 * wd);
          xq[m][j][2 * wd] = make_uint2((v[0] & 0xffffu) | (v[2] << 16), (v[0] >> 16) | (v[2] & 0xffff0000u));
          xq[m][j][2 * wd + 1] = make_uint2((v[1] & 0xffffu) | (v[3] << 16), (v[1] >> 16) | (v[3] & 0xffff0000u));
#pragma unroll
          for (int e = 0; e < 4; ++e) sum += T::to_f32((uint16_t)v[e]) + T::to_f32((uint16_t)(v[e] >> 16));
        } else {
          // word = codes c0..c3; pairs (c0,c2) (c1,c3)
          uint2 v = {0, 0};
          if (in_row && m < M) v = *reinterpret_cast<const uint2*>(x + (int64_t)m * K + k0 + 4 * wd);
          xq[m][j][wd] = make_uint2((v.x & 0xffffu) | (v.y << 16), (v.x >> 16) | (v.y & 0xffff0000u));
          sum += T::to_f32((uint16_t)v.x) + T::to_f32((uint16_t)(v.x >> 16)) + T::to_f32((uint16_t)v.y) +
                 T::to_f32((uint16_t)(v.y >> 16));
        }
      }
      sx[m][j] = sum;
    }
  }
  static_assert(kPerWord * 4 == kCodes, "a piece is four words");

  // rows are dealt to wavefronts in contiguous, balanced runs: rows_per_wave
  // each, one more for the first extra_rows wavefronts (the split is computed
  // on the host: an integer division here would delay the first loads)
  const int wave_id = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const int64_t row_begin = (int64_t)wave_id * rows_per_wave + min(wave_id, extra_rows);
  const int64_t row_end = row_begin + rows_per_wave + (wave_id < extra_rows ? 1 : 0);
  if (row_begin >= row_end) return;
  const char* wbytes = reinterpret_cast<const char*>(wq);

  // (word & mask) | magic is one instruction when the mask sits in a scalar and
  // the magic in a vector register; as literals they would cost two.
  uint32_t pair_mask = (BITS == 8 && CF::kWholeByte) ? 0x00ff00ffu : 0x000f000fu;
  uint32_t magic = CF::kNibble, magic_high = CF::kHighMagic;
  asm volatile("" : "+s"(pair_mask), "+v"(magic), "+v"(magic_high));

  auto consume = [&](const R& regs, int64_t row) __attribute__((always_inline)) {
    f32x4 tot[kM];  // register lane%4: this lane's sum of scale * D over its pieces
    float corr[kM];  // this lane's sum of (bias - offset * scale) * Sx
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      tot[m] = f32x4{0.f, 0.f, 0.f, 0.f};
      corr[m] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < kMaxLoads; ++j) {
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
      // one accumulation chain per piece and activation row; consecutive pieces
      // are independent of each other
      f32x4 d[kM];
#pragma unroll
      for (int m = 0; m < kM; ++m) d[m] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {
        const uint32_t w = regs.w[j][wd];
        if constexpr (BITS == 4) {
          const uint2 a0 = make_uint2((w & pair_mask) | magic, ((w >> 4) & pair_mask) | magic);
          const uint2 a1 = make_uint2(((w >> 8) & pair_mask) | magic, ((w >> 12) & pair_mask) | magic);
#pragma unroll
          for (int m = 0; m < kM; ++m) {
            d[m] = CF::mfma4(a0, xq[m][j][2 * wd], d[m]);
            d[m] = CF::mfma4(a1, xq[m][j][2 * wd + 1], d[m]);
          }
        } else if constexpr (CF::kWholeByte) {
          const uint2 a = make_uint2((w & pair_mask) | magic, ((w >> 8) & pair_mask) | magic);
#pragma unroll
          for (int m = 0; m < kM; ++m) d[m] = CF::mfma4(a, xq[m][j][wd], d[m]);
        } else {
          const uint2 lo = make_uint2((w & pair_mask) | magic, ((w >> 8) & pair_mask) | magic);
          const uint2 hi = make_uint2(((w >> 4) & pair_mask) | magic_high, ((w >> 12) & pair_mask) | magic_high);
#pragma unroll
          for (int m = 0; m < kM; ++m) {
            d[m] = CF::mfma4(lo, xq[m][j][wd], d[m]);
            d[m] = CF::mfma4(hi, xq[m][j][wd], d[m]);
          }
        }
      }
      const float bo = __builtin_fmaf(-kOffset, sc, bi);
#pragma unroll
      for (int m = 0; m < kM; ++m) {
#pragma unroll
        for (int e = 0; e < 4; ++e) tot[m][e] = __builtin_fmaf(sc, d[m][e], tot[m][e]);
        corr[m] = __builtin_fmaf(bo, sx[m][j], corr[m]);
      }
    }
    const int diag = lane & 3;
#pragma unroll
    for (int m = 0; m < kM; ++m) {
      float v = (diag == 0 ? tot[m][0] : diag == 1 ? tot[m][1] : diag == 2 ? tot[m][2] : tot[m][3]) + corr[m];
      v = wave_sum(v);
      if (lane == 0 && m < M) {
        const int64_t o = (int64_t)m * N + row;
        if (y_is_f32) {
          if (bias) v += T::to_f32(regs.bias);
          reinterpret_cast<float*>(y)[o] = v;
        } else {
          uint16_t hv = T::from_f32(v);
          if (bias) hv = T::from_f32(T::to_f32(hv) + T::to_f32(regs.bias));
          reinterpret_cast<uint16_t*>(y)[o] = hv;
        }
      }
    }
  };

  // kDepth rows in flight per wavefront: row r + kDepth - 1 is requested before
  // row r is consumed
  constexpr int kDepth = 2;
  R regs[kDepth];
#pragma unroll
  for (int d = 0; d < kDepth - 1; ++d)
    if (row_begin + d < row_end)
      regs[d].issue(wbytes, scales, biases, bias, row_begin + d, row_bytes, groups, piece, grp, lane);
  for (int64_t row = row_begin; row < row_end; row += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int64_t r = row + d;
      if (r < row_end) {
        if (r + kDepth - 1 < row_end)
          regs[(d + kDepth - 1) % kDepth].issue(wbytes, scales, biases, bias, r + kDepth - 1, row_bytes, groups, piece,
                                                grp, lane);
        consume(regs[d], r);
      }
    }
  }
}

template <typename T, int BITS, int kM, int kMaxLoads, bool kCoop>
int launch_rows_kernel(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                       const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  // as many workgroups as are resident at once (the register count of the
  // instantiation decides), so that every wavefront gets one balanced run of rows
  auto kernel = qmv_rows_kernel<T, BITS, kM, kMaxLoads, kCoop>;
  static PerDeviceInt cache;
  const int blocks_per_cu = cache.get([&] {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess || n < 1) n = 1;
    return n > 4 ? 4 : n;
  });
  int64_t blocks = (int64_t)compute_units() * blocks_per_cu;
  const int64_t max_blocks = (N + 3) / 4;  // at least one row per wavefront
  if (blocks > max_blocks) blocks = max_blocks;
  const int64_t n_waves = blocks * 4;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, gs_shift, (int)(N / n_waves),
                     (int)(N % n_waves));
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int BITS, int kM, int kMaxLoads>
int launch_rows_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                    const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  // a row's scales and biases travel as one cooperative load when they fit it:
  // at most 64 groups, an even number of them, 4-byte aligned arrays
  const int64_t groups = K >> gs_shift;
  const bool coop = groups <= 64 && groups % 2 == 0 &&
                    ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 3u) == 0;
  if (coop)
    return launch_rows_kernel<T, BITS, kM, kMaxLoads, true>(x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype,
                                                            stream);
  return launch_rows_kernel<T, BITS, kM, kMaxLoads, false>(x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype,
                                                           stream);
}

// The kernel is instantiated for the exact number of KiB-sized loads per row:
// up to 6 for one activation row, up to 3 for two to four (their x slices
// take four times the registers).
constexpr int kMaxLoadsOneRow = 6;
constexpr int kMaxLoadsFourRows = 3;

template <typename T, int BITS, int kM, int kLoads>
int launch_rows_loads(int64_t n_loads, const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                      const void* biases, const void* bias, int64_t N, int gs_shift, void* y, int y_dtype,
                      hipStream_t stream) {
  if (n_loads == kLoads)
    return launch_rows_one<T, BITS, kM, kLoads>(x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  if constexpr (kLoads > 1)
    return launch_rows_loads<T, BITS, kM, kLoads - 1>(n_loads, x, M, K, wq, scales, biases, bias, N, gs_shift, y,
                                                      y_dtype, stream);
  return MFQ_EUNSUPPORTED;
}

inline int64_t loads_per_row(int64_t K, int bits) { return (K * bits / 8 + 1023) / 1024; }

// One activation row: always (when the row fits the instantiated load counts).
// Two to four rows: only for short rows; with their x slices in registers the
// four-row instantiation keeps too few wavefronts resident on long rows and
// the workgroup-per-16-features kernel is faster there.
inline bool rows_kernel_covers(int64_t M, int64_t K, int bits) {
  const int64_t n = loads_per_row(K, bits);
  return (M == 1 && n <= kMaxLoadsOneRow) || (M <= 4 && n <= 1);
}

template <typename T>
int launch_rows(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  const int gs_shift = gs == 32 ? 5 : gs == 64 ? 6 : 7;
  const int64_t n = loads_per_row(K, bits);
  if (bits == 4) {
    if (M == 1)
      return launch_rows_loads<T, 4, 1, kMaxLoadsOneRow>(n, x, M, K, wq, scales, biases, bias, N, gs_shift, y,
                                                         y_dtype, stream);
    return launch_rows_loads<T, 4, 4, kMaxLoadsFourRows>(n, x, M, K, wq, scales, biases, bias, N, gs_shift, y,
                                                         y_dtype, stream);
  }
  if (M == 1)
    return launch_rows_loads<T, 8, 1, kMaxLoadsOneRow>(n, x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype,
                                                       stream);
  return launch_rows_loads<T, 8, 4, kMaxLoadsFourRows>(n, x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype,
                                                       stream);
}

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  using P = Phase<T, GS, BITS>;
  auto kernel = qmv_kernel<T, GS, BITS>;
  const size_t lds_bytes = 2 * ((size_t)P::kXTileOffset + (size_t)M * P::kRowBytes);
  // largest request: M = 16 rows of a 4-bit phase (2048 k), double buffered, about 140 KiB
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), 2 * (P::kXTileOffset + 16 * P::kRowBytes)))
    return MFQ_ELAUNCH;
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
#ifndef MFQ_NO_OCT
  if (qmv_oct_covers(M, K, N, gs, bits, x, scales, biases))
    return launch_qmv_oct(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (qmv_oct4_covers(M, K, N, gs, bits, x, scales, biases))
    return launch_qmv_oct4(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
#endif
  if (qmv_dot_covers(M, K, bits))
    return launch_qmv_dot(x, dtype, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  // two to four activation rows: four weight rows at a time (for a single row
  // the one-row-per-wavefront kernel below is the faster of the two)
  if (M >= 2 && qmv_quad_covers(M, K, N, gs, bits, scales, biases, bias, y, y_dtype))
    return launch_qmv_quad(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (rows_kernel_covers(M, K, bits)) {
    if (dtype == MFQ_BF16)
      return launch_rows<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
    if (dtype == MFQ_F16) return launch_rows<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
    return MFQ_EDTYPE;
  }
  if (dtype == MFQ_BF16) return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
