// Quantized matmul with the weight NOT transposed, for gfx950:
//   y[M, K] = x[M, N] @ dequant(wq[N, K])
// MLX's quantized_matmul(..., transpose=False).  It is the gradient of a
// quantized linear with respect to its input, which is what training a LoRA on a
// quantized base needs for every wrapped layer
// (src/mflux/models/common/training/lora/target_injector.py:30-33 wraps
// nn.QuantizedLinear in a trainable LoRALinear).
//
// The sum runs over the weight's ROWS, while the packing and the groups run
// along its columns, so the weights cannot reach the matrix cores the way they
// lie in memory: an operand register of the matrix instruction holds 8
// consecutive elements of the summed dimension.  Same tiling as the
// 128-column-tile GEMM (qmm_mid.hip): a workgroup computes 128 or 256 rows x 128
// output columns, the summed dimension in steps of 64 weight rows, both
// operands as XOR-swizzled 16-bit LDS tiles, global loads two steps ahead in
// registers, one barrier per step.  The weight tile is built transposed: of a
// step's 64 rows x 128 columns, thread t (of 256) takes the 8 columns 8(t%16)..+7
// of the 4 rows 4(t/16)..+3 -- per row one or two 32-bit words holding those 8
// codes (for the 3-, 5- and 6-bit packs a row is a bit stream and the 8 codes
// start at a byte, not a word: two words and one funnel shift by an amount that
// is fixed per thread), and that row's scale and bias of the columns' group --
// dequantises the 32 values (float32 fma, one rounding) and writes them as eight
// 8-byte pieces, one per column, each holding its four consecutive rows.
// Rows past N in the last step enter LDS as zeros on both sides.
#include <type_traits>

#include "common.h"
#include "tile_epilogue.h"

namespace mfq {
namespace {

constexpr int TC = 128;  // output columns per tile
constexpr int TR = 64;   // weight rows (summed) per step
constexpr int kTileW = TC * TR * 2;
constexpr int tile_m(int waves_m) { return 64 * waves_m; }
constexpr int threads_of(int waves_m) { return 2 * waves_m * kWave; }
constexpr int tile_x_bytes(int waves_m) { return tile_m(waves_m) * TR * 2; }
constexpr int lds_bytes(int waves_m) { return 2 * (tile_x_bytes(waves_m) + kTileW); }

__device__ inline int swz(int row, int chunk) { return row * (TR * 2) + ((chunk ^ ((row >> 1) & 7)) << 4); }

template <typename T, int GS, int BITS, int kWavesM>
__global__ __launch_bounds__(threads_of(kWavesM), 2) void qmm_n_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, void* __restrict__ y, int y_is_f32, int M, int N, int K, int tiles_m,
    int tiles_c) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;
  constexpr int TM = tile_m(kWavesM);
  constexpr int kThreads = threads_of(kWavesM);
  constexpr int kTileX = tile_x_bytes(kWavesM);
  constexpr int kBuf = kTileX + kTileW;
  constexpr int kXPass = kThreads / 8;  // x rows copied per pass (four passes)
  constexpr bool kStream = BITS != 4 && BITS != 8;
  constexpr int kWords = BITS == 4 ? 1 : 2;  // 32-bit words a thread loads per weight row

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int steps = (N + TR - 1) / TR;

  // tile sequence: an XCD walks a contiguous run, tile row fastest
  int tile = blockIdx.x;
  {
    const int n_tiles = tiles_m * tiles_c;
    const int per_xcd = n_tiles / 8;
    if (tile < per_xcd * 8) tile = (tile & 7) * per_xcd + (tile >> 3);
  }
  const int m0 = (tile % tiles_m) * TM;
  const int c0 = (tile / tiles_m) * TC;

  // x: thread t copies the 8 elements 8(t%8).. of row t/8 (+ kXPass per pass) of the step
  uint32_t xoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) xoff[i] = (uint32_t)min(m0 + (t >> 3) + kXPass * i, M - 1) * (uint32_t)N * 2u;
  const int xchunk = t & 7;
  // weights: 256 threads build the tile; with 512 threads the upper half requests the same and drops it
  const bool deq = t < 256;  // uniform per wavefront
  const int td = t & 255;
  const int cb = td & 15, rq = td >> 4;              // column block (8 columns), row quad (4 rows) of the step
  const int col = min(c0 + 8 * cb, K - 8);            // first of this thread's columns (K % 32 == 0; a tile may overhang K)
  const uint32_t row_words = (uint32_t)(K * BITS / 32);
  const uint32_t cbit = (uint32_t)col * BITS;
  const uint32_t word_lo = cbit >> 5, word_hi = min(word_lo + 1, row_words - 1);
  const uint32_t sh = cbit & 31u;                     // where the 8 codes start inside word_lo (0 for 4 and 8 bits)
  const uint32_t group = (uint32_t)(col / GS);
  const uint32_t groups_per_row = (uint32_t)(K / GS);
  const char* xbytes = reinterpret_cast<const char*>(x);

  const int wr_x = swz(t >> 3, t & 7);
  // LDS weight tile: row = output column, 16-byte chunk rq/2, half rq%2
  int wr_w[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) wr_w[j] = swz(8 * cb + j, rq >> 1) + 8 * (rq & 1);
  int rd[4];
#pragma unroll
  for (int sub = 0; sub < 4; ++sub) rd[sub] = swz(r, 4 * h + sub);

  struct Stage {
    u32x4 x[4];
    uint32_t w[4][kWords];
    uint16_t s[4], b[4];
  };
  Stage st[2];

  // Unconditional loads with compile-time register sets; q: step (steps past the end repeat the last one)
  auto load_w = [&](Stage& g, int q) __attribute__((always_inline)) {
    const int r0 = min(q, steps - 1) * TR + 4 * rq;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t row = (uint32_t)min(r0 + i, N - 1);
      const uint32_t* wrow = wq + (size_t)row * row_words;
      g.w[i][0] = wrow[word_lo];
      if constexpr (kWords == 2) g.w[i][1] = wrow[word_hi];
      g.s[i] = scales[(size_t)row * groups_per_row + group];
      g.b[i] = biases[(size_t)row * groups_per_row + group];
    }
  };
  auto load_x_piece = [&](Stage& g, int q, int i) __attribute__((always_inline)) {
    const int r0 = min(q, steps - 1) * TR + 8 * xchunk;
    g.x[i] = *reinterpret_cast<const u32x4*>(xbytes + xoff[i] + (size_t)min(r0, N - 8) * 2);
  };
  auto load = [&](Stage& g, int q) __attribute__((always_inline)) {
    load_w(g, q);
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x_piece(g, q, i);
  };

  // Quarter c of publishing a step: one 128-bit piece of x, and columns 2c, 2c+1 of the thread's weights
  // q: the step being published; what lies past N becomes zeros (N % 8 == 0: a piece of x and a
  // quad of weight rows are inside or outside as a whole)
  auto publish_part = [&](const Stage& g, int q, int c, int buf) __attribute__((always_inline)) {
    char* xd = lds + buf * kBuf;
    char* wd = xd + kTileX;
    const bool xpast = q * TR + 8 * xchunk >= N, wpast = q * TR + 4 * rq >= N;
    u32x4 xv = g.x[c];
    if (xpast) xv = u32x4{0u, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(xd + wr_x + kXPass * TR * 2 * c) = xv;
    if (deq) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int j = 2 * c + jj;  // column of the thread's eight
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t code;
          if constexpr (BITS == 4) {
            code = (g.w[i][0] >> (4 * j)) & 0xfu;
          } else if constexpr (BITS == 8) {
            code = (g.w[i][j >> 2] >> (8 * (j & 3))) & 0xffu;
          } else {
            // the 8 codes as a bit stream that starts at bit 0 of (lo, hi)
            const uint32_t lo = __builtin_amdgcn_alignbit(g.w[i][1], g.w[i][0], sh);
            const uint32_t hi = g.w[i][1] >> sh;
            const uint32_t pair[2] = {lo, hi};
            code = stream_code<BITS>(pair, j);
          }
          v[i] = __builtin_fmaf((float)code, T::to_f32(g.s[i]), T::to_f32(g.b[i]));
        }
        uint2 pk = make_uint2(T::pack2(v[0], v[1]), T::pack2(v[2], v[3]));
        if (wpast) pk = make_uint2(0u, 0u);
        *reinterpret_cast<uint2*>(wd + wr_w[j]) = pk;
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // step p on buffer p%2: the matrix work, with the quarters of publishing step p+1 to the other
  // buffer between its four sub-steps and each quarter's registers refilled for step p+3
  auto step = [&](auto parity, int p) __attribute__((always_inline)) {
    constexpr int buf = decltype(parity)::value;
    const char* xs = lds + buf * kBuf + 4096 * (2 * wm);
    const char* ws = lds + buf * kBuf + kTileX + 4096 * (2 * wn);
    vec8 af[2][2], bf[2][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) af[0][j] = *reinterpret_cast<const vec8*>(ws + rd[0] + 4096 * j);
#pragma unroll
    for (int i = 0; i < 2; ++i) bf[0][i] = *reinterpret_cast<const vec8*>(xs + rd[0] + 4096 * i);
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      if (sub < 3) {
#pragma unroll
        for (int j = 0; j < 2; ++j) af[(sub + 1) & 1][j] = *reinterpret_cast<const vec8*>(ws + rd[sub + 1] + 4096 * j);
#pragma unroll
        for (int i = 0; i < 2; ++i) bf[(sub + 1) & 1][i] = *reinterpret_cast<const vec8*>(xs + rd[sub + 1] + 4096 * i);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(af[sub & 1][j], bf[sub & 1][i], acc[i][j]);
      publish_part(st[buf ^ 1], p + 1, sub, buf ^ 1);
      load_x_piece(st[buf ^ 1], p + 3, sub);
      if (sub == 3) load_w(st[buf ^ 1], p + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };

  // prologue: steps 0, 1, 2 in flight, step 0 published
  load(st[0], 0);
  load(st[1], 1);
#pragma unroll
  for (int c = 0; c < 4; ++c) publish_part(st[0], 0, c, 0);
  load(st[0], 2);
  __syncthreads();
  int p = 0;
  for (; p + 2 <= steps; p += 2) {
    step(std::integral_constant<int, 0>{}, p);
    step(std::integral_constant<int, 1>{}, p + 1);
  }
  if (p < steps) step(std::integral_constant<int, 0>{}, p);

  store_block_64x64<T>(acc, lds, wave, lane, m0 + 64 * wm, c0 + 64 * wn, M, K, nullptr, static_cast<char*>(y), y_is_f32);
}

template <typename T, int GS, int BITS, int kWavesM>
int launch_kernel(const void* x, int64_t M, int64_t N, const uint32_t* wq, const void* scales, const void* biases,
                  int64_t K, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmm_n_kernel<T, GS, BITS, kWavesM>;
  constexpr int kLds = lds_bytes(kWavesM);
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLds)) return MFQ_ELAUNCH;
  const int tiles_m = (int)((M + tile_m(kWavesM) - 1) / tile_m(kWavesM));
  const int tiles_c = (int)((K + TC - 1) / TC);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_c)), dim3(threads_of(kWavesM)), kLds, stream,
                     (const uint16_t*)x, wq, (const uint16_t*)scales, (const uint16_t*)biases, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, tiles_m, tiles_c);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int GS, int BITS>
int launch_tile(const void* x, int64_t M, int64_t N, const uint32_t* wq, const void* scales, const void* biases,
                int64_t K, void* y, int y_dtype, hipStream_t stream) {
  if (M <= 128) return launch_kernel<T, GS, BITS, 2>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
  return launch_kernel<T, GS, BITS, 4>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
}

template <typename T, int GS>
int launch_bits(const void* x, int64_t M, int64_t N, const uint32_t* wq, const void* scales, const void* biases,
                int64_t K, int bits, void* y, int y_dtype, hipStream_t stream) {
  switch (bits) {
    case 3: return launch_tile<T, GS, 3>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
    case 4: return launch_tile<T, GS, 4>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
    case 5: return launch_tile<T, GS, 5>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
    case 6: return launch_tile<T, GS, 6>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
    default: return launch_tile<T, GS, 8>(x, M, N, wq, scales, biases, K, y, y_dtype, stream);
  }
}

template <typename T>
int launch_gs(const void* x, int64_t M, int64_t N, const uint32_t* wq, const void* scales, const void* biases,
              int64_t K, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  switch (gs) {
    case 32: return launch_bits<T, 32>(x, M, N, wq, scales, biases, K, bits, y, y_dtype, stream);
    case 64: return launch_bits<T, 64>(x, M, N, wq, scales, biases, K, bits, y, y_dtype, stream);
    default: return launch_bits<T, 128>(x, M, N, wq, scales, biases, K, bits, y, y_dtype, stream);
  }
}

}  // namespace

int launch_qmm_n(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                 const void* biases, int64_t K, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  if (N % 8) return MFQ_EUNSUPPORTED;  // x rows are read in 16-byte pieces and masked by the piece
  // 32-bit byte offsets into x; 32-bit tile counts
  if (M * N >= (int64_t)1 << 31 || ((M + 63) / 64) * ((K + TC - 1) / TC) >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16) return launch_gs<BF16>(x, M, N, wq, scales, biases, K, gs, bits, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch_gs<F16>(x, M, N, wq, scales, biases, K, gs, bits, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
