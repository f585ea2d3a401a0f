// Large-M quantized GEMM in two kernels (from 2048 activation rows on, where the copy starts to pay):
//   1. dequant_frag_kernel expands the packed weights ONCE per call into 16-bit values
//      (w_hat = round(fma(code, scale, bias)), the same single rounding as the fused
//      kernels) and writes them in the order the matrix instructions consume them:
//      blocks of 16 output rows x 64 k, 2 KiB each, laid out [half][lane][8 values], so
//      that one 16-byte load per lane of a wavefront is a matrix fragment and one
//      load instruction covers 1 KiB of contiguous memory;
//   2. frag_gemm_kernel multiplies x with that scratch copy: 256x256x64 tiles, four
//      wavefronts (one per SIMD, 256 rows x 64 columns each), v_mfma_f32_16x16x32
//      with the weights as the A operand straight from global memory into registers
//      and x from global memory straight into LDS (three tiles, no registers in
//      between), persistent workgroups that prefetch across tile boundaries and
//      store a tile's sums behind the first matrix instructions of their next tile;
//      the tail of the tile sequence cut along K into float32 planes as in qmm.hip, a
//      LoRA update as extra k behind the loop, the epilogues of epilogue.h in the
//      store; 192-column tiles where those fit one round of workgroups.
// Both kernels are also entry points of their own (launch_qmm_frag_copy,
// launch_qmm_frag_gemm) for weights whose copy the caller keeps.
// The fused kernel (qmm.hip) dequantises a weight once per 256 rows of x, M / 256
// times per call, in the shadow of its matrix instructions; here that vector work is
// gone from the matrix loop, which is what lets it use the 16-cycle instruction shape
// (half the issue slots per matrix instruction).  The price is the scratch copy
// (round_up(N, 16) * K * 2 bytes of workspace, HBM-bound to write) and a weight
// operand four (W4) or two (W8) times larger for the GEMM to read.
//
// mx.quantized_matmul(x, w, scales, biases, transpose=True) of
// src/mflux/models/common/weights/loading/weight_applier.py:43-103's quantized
// linears, as qmm.hip.
#include <type_traits>

#include "common.h"
#include "epilogue.h"

namespace mfq {
namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;          // one 16-bit x tile: 32 KiB
constexpr int kStageStride = 144;                // bytes per staged output row: 64 16-bit columns + 16 bytes of padding
constexpr int kStageRows = 64;                   // one wavefront stages 64 rows of its 64 columns at a time
constexpr int kStageBytes = kStageRows * kStageStride;
constexpr int kBiasBytes = 64 * 4;               // per wavefront: the bias of its 64 columns as float32
constexpr int kXBuffers = 3;                     // x tiles in LDS: in use, next, being filled
constexpr int kLdsBytes = kXBuffers * kTileBytes + 4 * kStageBytes + 4 * kBiasBytes;
constexpr int kBlockBytes = 16 * BK * 2;         // one block of the scratch copy: 16 rows x 64 k

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// see qmm.hip: 128-bit LDS accesses are conflict free with the 16-byte column XORed with bits 1..3 of the row
__device__ inline int swz(int row, int chunk) { return row * (BK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4); }

// see qmm.hip: XCD-contiguous runs of the tile sequence, bands of 4 tile rows, row index fastest
__host__ __device__ inline void tile_origin(int tile, int tiles_m, int tiles_n, int& m0, int& n0) {
  const int n_tiles = tiles_m * tiles_n;
  const int per_xcd = n_tiles / 8;
  if (tile < per_xcd * 8) tile = (tile & 7) * per_xcd + (tile >> 3);
  constexpr int kBandM = 4;
  const int band_tiles = kBandM * tiles_n;
  const int band = tile / band_tiles;
  const int rest = tiles_m - band * kBandM;
  const int band_rows = rest < kBandM ? rest : kBandM;
  const int in_band = tile - band * band_tiles;
  m0 = (band * kBandM + in_band % band_rows) * BM;
  n0 = (in_band / band_rows) * BN;
}

// ---------------------------------------------------------------------------------------------
// 1. the scratch copy.  A wavefront takes kPair neighbouring blocks of 16 rows x 64 k per trip (K / 64 is a
// multiple of kPair); lane (q, c16) = (lane / 16, lane % 16) works on row c16.  Loads are 16 bytes per lane
// with the four lanes of a row side by side (64 contiguous bytes per row and load: 8-byte loads fetched every
// 64-byte piece twice and cost a quarter more time), one scale and one bias per load (its 16 or 32 k lie in
// one group); every store instruction writes whole 256-byte runs of the copy, [block][half][lane].
template <typename T, int GS, int BITS, int kPair>
__global__ __launch_bounds__(256) void dequant_frag_kernel(const uint32_t* __restrict__ wq,
                                                           const uint16_t* __restrict__ scales,
                                                           const uint16_t* __restrict__ biases,
                                                           char* __restrict__ out, int N, int K, int n_blocks) {
  const int lane = threadIdx.x & (kWave - 1);
  const int c16 = lane & 15, q = lane >> 4;
  const int ks_per_row = K / BK;
  const int waves = gridDim.x * 4;
  for (int blk = (blockIdx.x * 4 + threadIdx.x / kWave) * kPair; blk < n_blocks; blk += waves * kPair) {
    const int nb = blk / ks_per_row, ks = blk - nb * ks_per_row;
    const int row = min(nb * 16 + c16, N - 1);  // rows past N repeat the last one; the GEMM never stores their columns
    if constexpr (BITS == 4) {
      // 16 bytes = 32 codes per load: the lane reads 16-byte piece q + 4 i of its row's kPair * 32 bytes (the
      // four lanes of a row cover 64 contiguous bytes per load), which holds k 32 (c & 1) .. + 32 of block
      // c / 2, i.e. the 16-k groups 2 (c & 1) and 2 (c & 1) + 1 of that block, and writes those four pieces
      constexpr int kLoads = kPair / 2;
      u32x4 w[kLoads];
      float s[kLoads], b[kLoads];
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        const int k0 = ks * BK + 32 * (q + 4 * i);
        w[i] = *reinterpret_cast<const u32x4*>(wq + ((int64_t)row * K + k0) / 8);
        const int64_t g = (int64_t)row * (K / GS) + k0 / GS;
        s[i] = T::to_f32(scales[g]), b[i] = T::to_f32(biases[g]);
      }
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        const int c = q + 4 * i;
        char* dst = out + (int64_t)(blk + (c >> 1)) * kBlockBytes + ((2 * (c & 1)) * 16 + c16) * 16;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const uint32_t word = w[i][2 * sub + half];
            u32x4 o;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
              const float c0 = (float)((word >> (8 * p)) & 0xfu), c1 = (float)((word >> (8 * p + 4)) & 0xfu);
              o[p] = T::pack2(__builtin_fmaf(c0, s[i], b[i]), __builtin_fmaf(c1, s[i], b[i]));
            }
            // plain stores: the GEMM behind reads the copy back through the memory-side cache
            *reinterpret_cast<u32x4*>(dst + 1024 * half + 256 * sub) = o;
          }
        }
      }
    } else {
      u32x4 w[kPair];
      float s[kPair], b[kPair];
#pragma unroll
      for (int u = 0; u < kPair; ++u) {
        const int k0 = (ks + u) * BK + 16 * q;
        w[u] = *reinterpret_cast<const u32x4*>(wq + ((int64_t)row * K + k0) / 4);
        const int64_t g = (int64_t)row * (K / GS) + k0 / GS;
        s[u] = T::to_f32(scales[g]), b[u] = T::to_f32(biases[g]);
      }
#pragma unroll
      for (int u = 0; u < kPair; ++u) {
        char* dst = out + (int64_t)(blk + u) * kBlockBytes + lane * 16;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          u32x4 o;
#pragma unroll
          for (int p = 0; p < 4; ++p) {  // values 2 p, 2 p + 1 of the half
            const uint32_t word = w[u][2 * half + (p >> 1)] >> (16 * (p & 1));
            const float c0 = (float)(word & 0xffu), c1 = (float)((word >> 8) & 0xffu);
            o[p] = T::pack2(__builtin_fmaf(c0, s[u], b[u]), __builtin_fmaf(c1, s[u], b[u]));
          }
          *reinterpret_cast<u32x4*>(dst + 1024 * half) = o;
        }
      }
    }
  }
}

// The same copy from MLX's 3-, 5- and 6-bit packs, where a row is one little-endian bit stream and 32 codes
// fill BITS whole words: a wavefront takes two neighbouring blocks per trip (K / 64 is even), lane (u, c16) =
// (lane / 16, lane % 16) the 32 codes of unit u of the pair's 128 k in row c16 -- BITS words, one scale and one
// bias (a unit lies in one group) -- and writes their four fragments of 8 values; the 16 lanes of a unit write
// 256 contiguous bytes per store.
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void dequant_frag_stream_kernel(const uint32_t* __restrict__ wq,
                                                                  const uint16_t* __restrict__ scales,
                                                                  const uint16_t* __restrict__ biases,
                                                                  char* __restrict__ out, int N, int K, int n_blocks) {
  const int lane = threadIdx.x & (kWave - 1);
  const int c16 = lane & 15, u = lane >> 4;
  const int ks_per_row = K / BK;
  const int waves = gridDim.x * 4;
  for (int blk = (blockIdx.x * 4 + threadIdx.x / kWave) * 2; blk < n_blocks; blk += waves * 2) {
    const int nb = blk / ks_per_row, ks = blk - nb * ks_per_row;
    const int row = min(nb * 16 + c16, N - 1);  // rows past N repeat the last one; the GEMM never stores their columns
    const int unit = 2 * ks + u;                // of the row's K / 32
    const uint32_t* src = wq + (int64_t)row * (K / 32 * BITS) + unit * BITS;
    uint32_t w[BITS];
#pragma unroll
    for (int i = 0; i < BITS; ++i) w[i] = src[i];
    const int64_t g = (int64_t)row * (K / GS) + (unit * 32) / GS;
    const float sc = T::to_f32(scales[g]), bi = T::to_f32(biases[g]);
    char* dst = out + (int64_t)(blk + (u >> 1)) * kBlockBytes + c16 * 16;
#pragma unroll
    for (int f = 0; f < 4; ++f) {  // codes 8 f .. 8 f + 7 of the unit: k 32 (u % 2) + 8 f of its block
      const int kk = 32 * (u & 1) + 8 * f;
      const uint4 v = dequant8_stream<T, BITS>(w, f, sc, bi);
      *reinterpret_cast<uint4*>(dst + 1024 * ((kk >> 3) & 1) + 256 * (kk >> 4)) = v;
    }
  }
}

// The copy for the product with the weight NOT transposed (y[M, K] = x[M, N] @ dequantize(W[N, K]), the input
// gradient of a quantized linear): the GEMM's output columns are then W's columns and its sum runs over W's
// rows, so the copy holds W^T in fragment order -- blocks of 16 columns k x 64 rows n, a fragment the 8
// consecutive n of one k.  A workgroup takes 64 rows x 256 columns: thread (rg, cg) = (t / 32, t % 32) loads the
// 8 columns 8 cg .. of the 8 rows 8 rg .. (one word per row at 4 bits, two at 8: the 32 threads of a row
// group read 128 or 256 contiguous bytes of each row), dequantises the 64 values and writes, per column, one
// whole fragment into an LDS image of the 16 blocks; the image then leaves as 16-byte pieces in memory order.
template <typename T, int GS, int BITS>
__global__ __launch_bounds__(256) void dequant_frag_t_kernel(const uint32_t* __restrict__ wq,
                                                             const uint16_t* __restrict__ scales,
                                                             const uint16_t* __restrict__ biases,
                                                             char* __restrict__ out, int N, int K, int tiles_k) {
  __shared__ __attribute__((aligned(16))) char img[16 * kBlockBytes];
  const int t = threadIdx.x;
  const int rg = t >> 5, cg = t & 31;
  const int st = blockIdx.x / tiles_k, tk = blockIdx.x - st * tiles_k;  // step of 64 rows, tile of 256 columns
  const int steps = N / BK;
  const int k0 = min(tk * 256 + 8 * cg, K - 8);  // columns past K (the last tile): the last eight again
  constexpr int kWords = BITS / 4;               // words of 8 codes
  uint32_t w[8][kWords];
  float sc[8], bi[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t n = (int64_t)st * BK + 8 * rg + i;
#pragma unroll
    for (int c = 0; c < kWords; ++c) w[i][c] = wq[(n * K + k0) * BITS / 32 + c];
    sc[i] = T::to_f32(scales[n * (K / GS) + k0 / GS]);
    bi[i] = T::to_f32(biases[n * (K / GS) + k0 / GS]);
  }
  // block cg / 2 of the tile, fragment (half, q, c16) = (rg % 2, rg / 2, 8 (cg % 2) + c)
  char* dst = img + (cg >> 1) * kBlockBytes + 1024 * (rg & 1) + ((rg >> 1) * 16 + 8 * (cg & 1)) * 16;
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t code = BITS == 4 ? (w[i][0] >> (4 * c)) & 0xfu : (w[i][c >> 2] >> (8 * (c & 3))) & 0xffu;
      v[i] = __builtin_fmaf((float)code, sc[i], bi[i]);
    }
    *reinterpret_cast<u32x4*>(dst + 16 * c) =
        u32x4{T::pack2(v[0], v[1]), T::pack2(v[2], v[3]), T::pack2(v[4], v[5]), T::pack2(v[6], v[7])};
  }
  __syncthreads();
  // block b of the tile is block (16 tk + b) * steps + st of the copy; blocks past the copy's last are dropped
  const int n_kb = (K + 15) / 16;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const int piece = p * 256 + t;  // 16-byte piece of the image
    const int b = piece >> 7;
    if (16 * tk + b < n_kb)
      *reinterpret_cast<u32x4*>(out + ((int64_t)(16 * tk + b) * steps + st) * kBlockBytes + 16 * (piece & 127)) =
          *reinterpret_cast<const u32x4*>(img + 16 * piece);
  }
}

// ---------------------------------------------------------------------------------------------
// 2. the GEMM.
//
// The matrix instruction with its sum accumulated in place, as assembly: the compiler is free to give an
// intrinsic's four result registers another place than its addend's, and with every one of the 256
// accumulation registers holding part of the tile it then rotates accumulators through the vector registers
// around every instruction.  Stated with the result tied to the addend, the instruction is opaque to the
// compiler's hazard recognizer, so the kernel keeps zeroing and the epilogue's reads in other basic blocks
// than the matrix instructions, separated from them by settle() below, and reads an accumulator between
// matrix instructions only where the last one on that register is some sixty instructions behind (acc_read);
// the build checks the generated code for both (_build.py).
__device__ __forceinline__ void mma16(bf16x8 a, bf16x8 b, f32x4& c) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mma16(f16x8 a, f16x8 b, f32x4& c) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// The first matrix instruction of a tile: the product alone, whatever the registers held.  Stated as an
// update all the same, so that the tile's sums stay in the registers the previous tile's were in.
__device__ __forceinline__ void mma16_first(bf16x8 a, bf16x8 b, f32x4& c) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mma16_first(f16x8 a, f16x8 b, f32x4& c) {
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "+a"(c) : "v"(a), "v"(b));
}
// An accumulator as four floats in vector registers, read HERE: the empty statement gives the accumulator a
// new name at this point, so that the reads cannot be hoisted to where all of them would be live at once.
__device__ __forceinline__ void acc_read(f32x4& c, float (&v)[4]) {
  asm volatile("" : "+a"(c));
  v[0] = c[0], v[1] = c[1], v[2] = c[2], v[3] = c[3];
}

// kCut: the instantiation that can cut the tail of the tile sequence along K (apart, so that the code of the
// shapes that run whole tiles only is what it is without it: the plane store costs the epilogue registers)
// kLowRank: lr_rank more k behind the item's own (a LoRA update, see qmm.hip), read straight from memory
// kJ: column tiles of 16 per wavefront, i.e. tiles of 256 rows x 64 kJ columns: 4, or 3 (192 columns) for
//     shapes whose 192-column tiles fit one round of workgroups (a quarter less work per workgroup than the
//     256-column tiles of the same round); without epilogue or K cut
// kDeferBias: the instantiation for calls with an output bias, whose deferred tile stores (do_step) add it
//     (apart, because the add in the slots of the other costs the calls without a bias a fifth of that pass)
template <typename T, bool kEpi, bool kCut, bool kLowRank, int kJ = 4, bool kDeferBias = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void frag_gemm_kernel(
    const uint16_t* __restrict__ x, const char* __restrict__ wfrag, const uint16_t* __restrict__ bias,
    void* __restrict__ y, int M, int N, int K, int tiles_m, int tiles_n, int n_whole, int tail_splits,
    float* __restrict__ planes, const uint16_t* __restrict__ lr_t, const uint16_t* __restrict__ lr_bs, int lr_rank,
    Epilogue epi) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;
  static_assert(kJ == 4 || (kJ == 3 && !kEpi && !kCut), "192-column tiles: plain whole tiles only");
  static_assert(!kDeferBias || (!kEpi && kJ == 4), "deferred stores with a bias: plain 256-column tiles");
  constexpr int kBN = 64 * kJ;  // columns of a tile
  const int n_tiles = tiles_m * tiles_n;
  const int n_items = n_whole + (n_tiles - n_whole) * tail_splits;
  const int steps_total = K / BK;  // even, at least 4 (the launcher has checked)

  // A work item is (tile, k range): the first n_whole tiles of the sequence run whole; each later one is cut
  // into tail_splits equal ranges of an even number of steps, every range into a float32 plane of its own
  // (qmm.hip's K cut: tail_reduce_kernel adds the planes up, rounds, applies bias and epilogue).
  struct Item {
    int m0, n0;
    int first_step, n_steps;
    int plane;  // -1: the tile is whole and goes to y
  };
  auto item_of = [&](int seq) {
    Item it;
    int tile = seq;
    it.first_step = 0;
    it.n_steps = steps_total;
    it.plane = -1;
    if (kCut && seq >= n_whole) {
      const int e = seq - n_whole;
      const int tail_tile = e / tail_splits;
      tile = n_whole + tail_tile;
      it.n_steps = steps_total / tail_splits;
      it.first_step = (e - tail_tile * tail_splits) * it.n_steps;
      it.plane = e;
    }
    tile_origin(tile, tiles_m, tiles_n, it.m0, it.n0);
    it.n0 = it.n0 / BN * kBN;
    return it;
  };
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wn = wave * (16 * kJ);
  const int c16 = lane & 15;
  const int q = lane >> 4;

  // Per-lane byte offsets of the tile the PREFETCH cursor is in: the blocks of the wavefront's four column tiles
  // (16 columns each; blocks past N repeat the last one) and the lane's eight x pieces (rows past M clamped).
  uint32_t woff[kJ], xoff[8];
  auto set_prefetch_tile = [&](int m0, int n0) {
#pragma unroll
    for (int j = 0; j < kJ; ++j) {
      const uint32_t nb = (uint32_t)min((n0 + wn) / 16 + j, (N - 1) / 16);
      woff[j] = nb * (uint32_t)steps_total * (uint32_t)kBlockBytes + (uint32_t)lane * 16u;
    }
    // lane l of a direct load lands in LDS at 16 l past the load's base: row l / 8 of the wavefront's eight,
    // 16-byte slot l % 8, which in the swizzled tile holds the row's piece (l % 8) ^ ((row / 2) % 8)
    const uint32_t piece = (uint32_t)((t & 7) ^ (((t >> 3) >> 1) & 7));  // 32 i rows further on: the same
#pragma unroll
    for (int i = 0; i < 8; ++i)
      xoff[i] = ((uint32_t)min(m0 + (t >> 3) + 32 * i, M - 1) * (uint32_t)K + 8u * piece) * 2u;
  };
  const char* xbytes = reinterpret_cast<const char*>(x);
  // 16 bytes per lane from global memory straight into LDS, 1 KiB per instruction (eight rows of the tile):
  // no registers, no LDS write instructions.  The compiler does not see these loads; it counts only the
  // weight loads, so its own waits can only be stricter than it thinks, and the waits for the tiles
  // themselves are stated below by count.
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  auto dma16 = [&](const char* sbase, uint32_t voff, uint32_t lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr)
                 : "memory", "m0");
  };
  int x_cur = 0, x_next = kTileBytes, x_fill = 2 * kTileBytes;  // LDS offsets of the three x tiles
  // x fragment of a pass: row c16 of a 16-row block (2048 bytes apart), 16-byte piece 2 q + pass, which holds
  // k 16 q + 8 pass + [0, 8) of the step: the k a lane's weight fragment of that pass holds
  int rd_slot[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) rd_slot[half] = swz(c16, 2 * q + half);

  vec8 wa[2 * kJ], wb[2 * kJ];  // weight fragments of the even / odd steps: [2 j + pass], column tile j
  char* out_base = static_cast<char*>(y);
  int out_stride = N;
  const uint16_t* out_bias = bias;
  f32x4 acc[16][kJ];  // [r][j][e]: row 16 r + c16, column 16 j + 4 q + e of the wavefront's 256 x 16 kJ block
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < kJ; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

  auto load_w = [&](vec8 (&set)[2 * kJ], int half, int step) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < kJ; ++j)
      set[2 * j + half] = *reinterpret_cast<const vec8*>(wfrag + (size_t)step * kBlockBytes + woff[j] + 1024 * half);
  };

  char* drain_out = nullptr;  // the previous tile's place in y while the accumulators still hold it
  bool pending = false;       // they do
  int m1 = 0, n1 = 0;  // the tile the prefetch cursor moves to in the middle of a tile's last-but-one step
  // Step p = two passes of 64 matrix instructions (16 row blocks x 4 column tiles).  Behind them: every
  // fourth slot the LDS read of the x fragment three row blocks ahead; in the first pass the request for
  // the second-pass fragments of step p+1 into `other` (step p-1 has finished with them), in the second
  // pass the request for the first-pass fragments of step p+2 into `now` and the eight direct loads of
  // the x tile of step p+2 into the LDS tile that step p-1 read -- one load every eighth (weights) or
  // seventh (x) slot rather than in a burst, which measured 1 % faster.  s_h1 / s_h0: the steps (counted inside
  // the cursor's tile) those requests are for; `sw`: the cursor enters the next tile between the passes.
  //
  // kDrain 3: the first step of an item; its first pass writes the bare products (no addend, so nothing is
  // zeroed between items).
  // kDrain 1: the same, and the accumulators may still hold the PREVIOUS tile (drain_out: its
  // place in y), and this is the first step of the next one.  Its first pass then empties them as it goes: the
  // matrix instructions of row block r write the bare product (no addend, so nothing is zeroed either) while
  // the slots behind them round row block r+1 to 16 bits and write it into the wavefront's staging region,
  // 32 rows (two row blocks) to a half; a filled half is read back as whole 128-byte row segments during the
  // next row block and stored during the one after, while the other half fills.  Every read of an accumulator
  // is at least 60 matrix instructions behind the one that wrote it.  The pass is issue-bound (about twice
  // its usual time) instead of the 6 us a tile's stores cost with the matrix pipeline idle.
  auto do_step = [&](auto drain_mode, bool sw, vec8 (&now)[2 * kJ], vec8 (&other)[2 * kJ], int s_h1, int s_h0)
      __attribute__((always_inline)) {
    constexpr int kDrain = decltype(drain_mode)::value;
    constexpr int kHalfBytes = kStageBytes / 2;
    static_assert(32 * kStageStride <= kHalfBytes, "32 staged rows to a half");
    char* st_w = nullptr;
    const char* st_r = nullptr;
    uint32_t out_off = 0;
    uint32_t rd_off[kJ], gl_off[kJ];  // 192-column tiles: the lane's piece of each read-back and store of a half
    u32x4 rb[kJ];
    float bv[kJ][4];  // kDeferBias: the bias of the lane's four columns of each column tile
    auto drain_part = [&](int r, int j) __attribute__((always_inline)) {
      uint32_t pk[2];
      float v[4];
      acc_read(acc[r][j], v);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        pk[c] = T::pack2(v[2 * c], v[2 * c + 1]);
        if constexpr (kDeferBias)  // second rounding, as a separate add on the 16-bit result would do
          pk[c] = T::pack2(lo_f32<T>(pk[c]) + bv[j][2 * c], hi_f32<T>(pk[c]) + bv[j][2 * c + 1]);
      }
      *reinterpret_cast<uint2*>(st_w + ((r >> 1) & 1) * kHalfBytes + 16 * (r & 1) * kStageStride + 32 * j) =
          make_uint2(pk[0], pk[1]);
    };
    // a half holds 32 rows of 2 kJ 16-byte pieces; read-back k of kJ takes pieces 64 k + lane in row-major
    // order: with 8 pieces to a row that is row 8 k + lane / 8, piece lane % 8
    auto drain_read = [&](int u, int k) __attribute__((always_inline)) {
      if constexpr (kJ == 4) {
        rb[k] = *reinterpret_cast<const u32x4*>(st_r + (u & 1) * kHalfBytes + 8 * k * kStageStride);
      } else {
        rb[k] = *reinterpret_cast<const u32x4*>(st_r + (u & 1) * kHalfBytes + rd_off[k]);
      }
    };
    auto drain_store = [&](int u, int k) __attribute__((always_inline)) {
      char* rows = drain_out + (size_t)(32 * u + (kJ == 4 ? 8 * k : 0)) * ((size_t)N * 2);
      if (pending) *reinterpret_cast<u32x4*>(rows + (kJ == 4 ? out_off : gl_off[k])) = rb[k];
    };
    if constexpr (kDrain == 1) {
      int lane_e = lane;  // opaque copy: keeps this per-tile address arithmetic out of the k loop's registers
      asm volatile("" : "+v"(lane_e));
      char* stage = lds + kXBuffers * kTileBytes + wave * kStageBytes;
      st_w = stage + (lane_e & 15) * kStageStride + 8 * (lane_e >> 4);
      if constexpr (kJ == 4) {
        st_r = stage + (lane_e >> 3) * kStageStride + 16 * (lane_e & 7);
        out_off = ((uint32_t)(lane_e >> 3) * (uint32_t)N + (uint32_t)wn + 8u * (uint32_t)(lane_e & 7)) * 2u;
      } else {
        st_r = stage;
#pragma unroll
        for (int k = 0; k < kJ; ++k) {
          const uint32_t idx = 64u * k + (uint32_t)lane_e, row = idx / (2 * kJ), piece = idx - row * (2 * kJ);
          rd_off[k] = row * kStageStride + 16u * piece;
          gl_off[k] = (row * (uint32_t)N + (uint32_t)wn + 8u * piece) * 2u;
        }
      }
      if constexpr (kDeferBias) {  // written by the tile that left its sums behind (below)
        const float* bias_f =
            reinterpret_cast<const float*>(lds + kXBuffers * kTileBytes + 4 * kStageBytes + wave * kBiasBytes);
#pragma unroll
        for (int j = 0; j < kJ; ++j) {
          const float4 b4 = *reinterpret_cast<const float4*>(bias_f + 16 * j + 4 * (lane_e >> 4));
          bv[j][0] = b4.x, bv[j][1] = b4.y, bv[j][2] = b4.z, bv[j][3] = b4.w;
        }
      }
      // The first reads of the old tile's sums: this block is entered over the loop's back edge, where no count of
      // instructions along the listing says how far behind the last matrix instructions are, so the distance is
      // stated here (32 wait states, more than any matrix instruction needs to retire), on the two row blocks
      // that are read before the first-pass matrix instructions of this step have put sixty of them in between.
      if constexpr (kJ == 4) {
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]),
                       "+a"(acc[1][1]), "+a"(acc[1][2]), "+a"(acc[1][3]));
      } else {
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[1][0]), "+a"(acc[1][1]),
                       "+a"(acc[1][2]));
      }
#pragma unroll
      for (int j = 0; j < kJ; ++j) drain_part(0, j);
      __builtin_amdgcn_sched_barrier(0);
    }
    const char* xs = lds + x_cur;
    const uint32_t fill = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)x_fill + (uint32_t)wave * 1024u);
    vec8 xf[4];
    auto read_frag = [&](int g) {  // g = 16 * pass + row block
      xf[g & 3] = *reinterpret_cast<const vec8*>(xs + rd_slot[g >> 4] + 2048 * (g & 15));
    };
    read_frag(0);
    read_frag(1);
    read_frag(2);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (half == 1) {
        if (sw) set_prefetch_tile(m1, n1);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r)
#pragma unroll
        for (int j = 0; j < kJ; ++j) {
          const int m = kJ * r + j;
          const int g = 16 * half + r;
          if (kDrain != 0 && half == 0) {
            mma16_first(now[2 * j + half], xf[g & 3], acc[r][j]);
            if constexpr (kDrain == 1) {
              if (r + 1 < 16) drain_part(r + 1, j);
              if (r & 1) drain_read(r >> 1, j);
              if (r >= 2 && !(r & 1)) drain_store((r - 2) >> 1, j);
            }
          } else {
            mma16(now[2 * j + half], xf[g & 3], acc[r][j]);
            if (kDrain == 1 && r == 0) drain_store(7, j);
          }
          if (j == 0 && g + 3 < 32) read_frag(g + 3);
          if ((m & 7) == 2 && (m >> 3) < kJ) {
            const int j1 = m >> 3;
            if (half == 0) {
              other[2 * j1 + 1] = *reinterpret_cast<const vec8*>(wfrag + (size_t)s_h1 * kBlockBytes + woff[j1] + 1024);
            } else {
              now[2 * j1] = *reinterpret_cast<const vec8*>(wfrag + (size_t)s_h0 * kBlockBytes + woff[j1]);
            }
          }
          constexpr int kDmaFirst = kJ == 4 ? 6 : 4, kDmaEvery = kJ == 4 ? 7 : 5;  // 8 loads over the pass's 16 kJ slots
          if (half == 1 && m >= kDmaFirst && (m - kDmaFirst) % kDmaEvery == 0 && m < kDmaFirst + 8 * kDmaEvery) {
            const int i = (m - kDmaFirst) / kDmaEvery;
            dma16(xbytes + (size_t)s_h0 * (BK * 2), xoff[i], fill + 4096u * i);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
    }
    // The x tile of the next step, requested during the previous step, must have landed in every wavefront's
    // part before anyone reads it: younger than those requests are the 2 kJ weight loads and the 8 direct loads
    // of this step (stores of a tile's epilogue in between only make the count stricter).
    if constexpr (kJ == 4) {
      asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(14)" ::: "memory");
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    const int done = x_cur;
    x_cur = x_next;
    x_next = x_fill;
    x_fill = done;
  };

  // Fills the pipeline for the tile the cursor is in: x(0) and x(1) into LDS, the
  // fragments of step 0 and the first-pass fragments of step 1.
  auto prime = [&](int s0) {  // s0: the item's first step
    const uint32_t w1k = lds_base + (uint32_t)wave * 1024u;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      dma16(xbytes + (size_t)s0 * (BK * 2), xoff[i], __builtin_amdgcn_readfirstlane(w1k + (uint32_t)x_cur) + 4096u * i);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      dma16(xbytes + (size_t)(s0 + 1) * (BK * 2), xoff[i],
            __builtin_amdgcn_readfirstlane(w1k + (uint32_t)x_next) + 4096u * i);
    load_w(wa, 0, s0);
    load_w(wa, 1, s0);
    load_w(wb, 0, s0 + 1);
    // both x tiles have landed (the fragments too); as an instruction the compiler sees, so that its own wait
    // counting enters the loop knowing that nothing is outstanding
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), the other counters at their maxima
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // 16-bit output with N a multiple of 8: each wavefront transposes its 256 x 64 block through its
  // private LDS region, 64 rows at a time (rows 144 bytes apart), so that every global store writes
  // complete 128-byte row segments; the read-back applies the epilogues of epilogue.h.
  auto store_tile_staged = [&](auto with_bias, int m0, int n0) {
    constexpr bool kBias = decltype(with_bias)::value;
    int lane_e = lane;  // opaque copy: keeps this per-tile address arithmetic out of the k loop's registers
    asm volatile("" : "+v"(lane_e));
    const int c16 = lane_e & 15;
    const int q = lane_e >> 4;
    const int lane = lane_e;
    char* stage = lds + kXBuffers * kTileBytes + wave * kStageBytes;
    uint16_t* yout = reinterpret_cast<uint16_t*>(out_base);
    const float* bias_f = reinterpret_cast<const float*>(lds + kXBuffers * kTileBytes + 4 * kStageBytes + wave * kBiasBytes);
    if constexpr (kBias) {
      *reinterpret_cast<float*>(lds + kXBuffers * kTileBytes + 4 * kStageBytes + wave * kBiasBytes + lane * 4) =
          T::to_f32(out_bias[min(n0 + wn + lane, N - 1)]);
    }
#pragma unroll
    for (int pass = 0; pass < 256 / kStageRows; ++pass) {
#pragma unroll
      for (int j = 0; j < kJ; ++j) {
        const int cl = 16 * j + 4 * q;  // column inside the wavefront's 16 kJ
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if constexpr (kBias) {
          const float4 b4 = *reinterpret_cast<const float4*>(bias_f + cl);
          bv[0] = b4.x, bv[1] = b4.y, bv[2] = b4.z, bv[3] = b4.w;
        }
#pragma unroll
        for (int r8 = 0; r8 < kStageRows / 16; ++r8) {
          const int r = kStageRows / 16 * pass + r8;
          uint32_t pk[2];
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            pk[c] = T::pack2(acc[r][j][2 * c], acc[r][j][2 * c + 1]);
            if constexpr (kBias)  // second rounding, as a separate add on the 16-bit result would do
              pk[c] = T::pack2(lo_f32<T>(pk[c]) + bv[2 * c], hi_f32<T>(pk[c]) + bv[2 * c + 1]);
          }
          *reinterpret_cast<uint2*>(stage + (16 * r8 + c16) * kStageStride + cl * 2) = make_uint2(pk[0], pk[1]);
          if (r8 & 1) __builtin_amdgcn_sched_barrier(0);
        }
      }
      const int cg = n0 + wn + 8 * (lane & 7);
      if constexpr (kEpi) {
        if (epi.kind == kEpiSwiglu) {
          const int cq = lane & 3;
          const int co = (wn >> 1) + 8 * cq;
#pragma unroll
          for (int k = 0; k < kStageRows / 16; ++k) {
            const int rl = 16 * k + (lane >> 2);
            const u32x4 g = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * cq);
            const u32x4 u = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 64 + 16 * cq);
            u32x4 v;
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = epi_swiglu_pair<T>(g[c], u[c]);
            const int row = m0 + kStageRows * pass + rl;
            if (row < M && n0 + wn + 8 * cq < N)
              *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + co) = v;
          }
          continue;
        }
        if (epi.kind == kEpiGateResidual) {
          u32x4 gate8 = {0u, 0u, 0u, 0u};
          if (cg < N) gate8 = *reinterpret_cast<const u32x4*>(epi.gate + cg);
          const uint16_t* res = epi.residual + (int64_t)m0 * N + cg;
#pragma unroll
          for (int k4 = 0; k4 < kStageRows / 32; ++k4) {
            u32x4 rv[4];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
              const int rl = 8 * (4 * k4 + kk) + (lane >> 3);
              const int row = min(m0 + kStageRows * pass + rl, M - 1);
              rv[kk] = cg < N ? *reinterpret_cast<const u32x4*>(res + (int64_t)(row - m0) * N) : gate8;
            }
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
              const int rl = 8 * (4 * k4 + kk) + (lane >> 3);
              u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * (lane & 7));
#pragma unroll
              for (int c = 0; c < 4; ++c) v[c] = epi_gate_residual_pair<T>(v[c], gate8[c], rv[kk][c]);
              const int row = m0 + kStageRows * pass + rl;
              if (row < M && cg < N) *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + (cg - n0)) = v;
            }
          }
          continue;
        }
      }
      if constexpr (kJ != 4) {  // 6 pieces to a staged row: read-back k takes pieces 64 k + lane in row-major order
#pragma unroll
        for (int k = 0; k < kStageRows * 2 * kJ / 64; ++k) {
          const int idx = 64 * k + lane, rl = idx / (2 * kJ), piece = idx - rl * (2 * kJ);
          const u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * piece);
          const int row = m0 + kStageRows * pass + rl, col = n0 + wn + 8 * piece;
          if (row < M && col < N) *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + (col - n0)) = v;
          if (k & 1) __builtin_amdgcn_sched_barrier(0);
        }
        continue;
      }
#pragma unroll
      for (int k = 0; k < kStageRows / 8; ++k) {
        const int rl = 8 * k + (lane >> 3);
        u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * (lane & 7));
        if constexpr (kEpi) {
          if (epi.kind == kEpiGelu && cg >= epi.act_from) {
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = epi_gelu_pair<T>(v[c]);
          }
        }
        const int row = m0 + kStageRows * pass + rl;
        if (row < M && cg < N) *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + (cg - n0)) = v;
        if (k & 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // The low-rank update: lr_rank more k, whose x side is lr_t [M, lr_rank] and whose weight side is
  // lr_bs [N, lr_rank], both 16-bit and unquantised.  They are few, so they bypass the pipeline: a lane's
  // 8 consecutive k of a row are one 16-byte load straight into a matrix fragment (k 32 c + 8 q + 0..7 of
  // chunk c of 32 on both sides; past the rank, zeros).
  auto low_rank_steps = [&](int m0, int n0) {
    int lane_e = lane;  // opaque copy: keeps this per-tile address arithmetic out of the k loop's registers
    asm volatile("" : "+v"(lane_e));
    const int c16 = lane_e & 15;
    const int q = lane_e >> 4;
    const char* tb = reinterpret_cast<const char*>(lr_t) + 16 * q;
    const char* bb = reinterpret_cast<const char*>(lr_bs) + 16 * q;
    const uint32_t pitch = (uint32_t)lr_rank * 2u;  // bytes per row of either matrix
    uint32_t boff[kJ];
#pragma unroll
    for (int j = 0; j < kJ; ++j) boff[j] = (uint32_t)min(n0 + wn + 16 * j + c16, N - 1) * pitch;
    const uint32_t toff = (uint32_t)min(m0 + c16, M - 1) * pitch;
    const uint32_t t_last = (uint32_t)(M - 1) * pitch;  // rows 16 r + c16 of the tile: 16 * pitch apart until the clamp
    const vec8 zero = __builtin_bit_cast(vec8, make_uint4(0u, 0u, 0u, 0u));
#pragma unroll 1
    for (uint32_t kb = 0; kb < pitch; kb += 64) {
      const bool in_rank = kb + 16u * (uint32_t)q < pitch;  // a rank of 16 (mod 32) fills half of the last chunk
      vec8 wf[kJ];
#pragma unroll
      for (int j = 0; j < kJ; ++j) wf[j] = in_rank ? *reinterpret_cast<const vec8*>(bb + boff[j] + kb) : zero;
#pragma unroll
      for (int quarter = 0; quarter < 4; ++quarter) {
        vec8 tf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          tf[i] = in_rank ? *reinterpret_cast<const vec8*>(
                                tb + min(toff + (uint32_t)(4 * quarter + i) * 16u * pitch, t_last) + kb)
                          : zero;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < kJ; ++j) mma16(wf[j], tf[i], acc[4 * quarter + i][j]);
      }
    }
  };

  // Every accumulator in its accumulation register, and more wait states than any matrix instruction needs
  // between the instructions in front and behind.
  auto settle = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; r += 4) {
      if constexpr (kJ == 4) {
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[r][0]), "+a"(acc[r][1]), "+a"(acc[r][2]), "+a"(acc[r][3]), "+a"(acc[r + 1][0]),
                       "+a"(acc[r + 1][1]), "+a"(acc[r + 1][2]), "+a"(acc[r + 1][3]), "+a"(acc[r + 2][0]),
                       "+a"(acc[r + 2][1]), "+a"(acc[r + 2][2]), "+a"(acc[r + 2][3]), "+a"(acc[r + 3][0]),
                       "+a"(acc[r + 3][1]), "+a"(acc[r + 3][2]), "+a"(acc[r + 3][3]));
      } else {
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[r][0]), "+a"(acc[r][1]), "+a"(acc[r][2]), "+a"(acc[r + 1][0]), "+a"(acc[r + 1][1]),
                       "+a"(acc[r + 1][2]), "+a"(acc[r + 2][0]), "+a"(acc[r + 2][1]), "+a"(acc[r + 2][2]),
                       "+a"(acc[r + 3][0]), "+a"(acc[r + 3][1]), "+a"(acc[r + 3][2]));
      }
    }
  };

  // Behind an epilogue: new values for the accumulators (the next item's first step overwrites them anyway), so
  // that the compiler has nothing of the old ones to keep alive across the stores.
  auto forget = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r)
#pragma unroll
      for (int j = 0; j < kJ; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[r][j][e] = 0.f;
  };

  // A k range's sums as float32 into its dense 256 x 256 plane: the same transpose through the wavefront's
  // LDS region, 32 rows at a time (a staged row is 64 floats plus 16 bytes), so that every global store
  // writes complete 256-byte row segments.
  auto store_plane = [&](float* plane) {
    constexpr int kStride = 64 * 4 + 16;
    static_assert(32 * kStride <= kStageBytes, "the float32 staging fits the wavefront's region");
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int c16 = lane_e & 15;
    const int q = lane_e >> 4;
    const int lane = lane_e;
    char* stage = lds + kXBuffers * kTileBytes + wave * kStageBytes;
    if constexpr (kJ == 4) {
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r2 = 0; r2 < 2; ++r2) {
          const int r = 2 * pass + r2;
          *reinterpret_cast<float4*>(stage + (16 * r2 + c16) * kStride + (16 * j + 4 * q) * 4) =
              make_float4(acc[r][j][0], acc[r][j][1], acc[r][j][2], acc[r][j][3]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int rl = 4 * k + (lane >> 4);
        const float4 v = *reinterpret_cast<const float4*>(stage + rl * kStride + 16 * (lane & 15));
        *reinterpret_cast<float4*>(plane + (32 * pass + rl) * BN + wn + 4 * (lane & 15)) = v;
        if (k & 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
    }
  };

  // The items of this workgroup in sequence: first its whole tiles, then (kCut) its k ranges of tail tiles.
  // The two kinds run through two instantiations of the same loop, each with one kind of store behind it: with
  // both stores behind one loop the compiler reads the accumulators ahead of the branch and spills them.
  bool primed = false;
  auto run = [&](auto to_planes, int seq, int end) __attribute__((always_inline)) {
    constexpr bool kPlanes = decltype(to_planes)::value;
    for (; seq < end; seq += gridDim.x) {
      const Item item = item_of(seq);
      const int m0 = item.m0, n0 = item.n0;
      const int steps = item.n_steps, s0 = item.first_step;
      if constexpr (!kPlanes) {
        out_base = static_cast<char*>(y) + ((size_t)m0 * N + n0) * 2;
        out_stride = N;
        if constexpr (kEpi) {
          if (epi.kind == kEpiSwiglu) {
            out_base = static_cast<char*>(y) + ((size_t)m0 * (N / 2) + n0 / 2) * 2;
            out_stride = N / 2;
          }
        }
      }
      if (!primed) {
        set_prefetch_tile(m0, n0);
        prime(s0);
      }
      const bool has_next = seq + (int)gridDim.x < n_items;
      Item next = item;
      if (has_next) next = item_of(seq + gridDim.x);
      m1 = next.m0, n1 = next.n0;
      // without a next item: the last pair again (loaded, not used)
      const int s_next = has_next ? next.first_step : s0 + steps - 2;
      // The first step of an item starts the sums (and stores the previous tile if that is still in the
      // accumulators); ONE body for every later pair of steps, the item's last included: the accumulators pass
      // through a single copy of those matrix instructions, so the compiler has no place to move them between
      // register files.
      if (!pending) settle();
      {
        const bool last = steps == 2;
        const int s_even = last ? s_next : s0 + 2;
        do_step(std::integral_constant<int, (kPlanes || kEpi) ? 3 : 1>{}, last, wa, wb, s0 + 1, s_even);
        do_step(std::integral_constant<int, 0>{}, false, wb, wa, s_even, last ? s_next + 1 : s0 + 3);
      }
      for (int p = 2; p < steps; p += 2) {
        const bool last = p == steps - 2;
        const int s_even = last ? s_next : s0 + p + 2;
        do_step(std::integral_constant<int, 0>{}, last, wa, wb, s0 + p + 1, s_even);
        do_step(std::integral_constant<int, 0>{}, false, wb, wa, s_even, last ? s_next + 1 : s0 + p + 3);
      }
      if constexpr (kLowRank) {
        if (s0 == 0) low_rank_steps(m0, n0);  // once per tile: by the item that has its first k range
      }
      primed = has_next;
      if constexpr (!kPlanes && !kEpi) {
        // A tile with all of its rows and columns inside y, followed by another whole tile, leaves its sums in
        // the accumulators: the next tile's first step stores them (a bias: in the kDeferBias instantiation).
        if (seq + (int)gridDim.x < end && m0 + BM <= M && n0 + kBN <= N && (kDeferBias || !out_bias)) {
          if constexpr (kDeferBias)
            *reinterpret_cast<float*>(lds + kXBuffers * kTileBytes + 4 * kStageBytes + wave * kBiasBytes + lane * 4) =
                T::to_f32(out_bias[n0 + wn + lane]);
          drain_out = out_base;
          pending = true;
          continue;
        }
      }
      pending = false;
      settle();
      if constexpr (kPlanes) {
        store_plane(planes + (size_t)item.plane * (BM * BN));
      } else if (out_bias) {
        store_tile_staged(std::true_type{}, m0, n0);
      } else {
        store_tile_staged(std::false_type{}, m0, n0);
      }
      forget();
    }
    return seq;
  };
  const int seq_tail = run(std::false_type{}, (int)blockIdx.x, kCut ? n_whole : n_items);
  if constexpr (kCut) run(std::true_type{}, seq_tail, n_items);
}

template <typename T, int GS>
int launch_dequant_bits(const uint32_t* wq, const void* scales, const void* biases, int bits, void* out, int64_t N,
                        int64_t K, hipStream_t stream) {
  const int64_t n_blocks = ((N + 15) / 16) * (K / BK);
  // blocks per wavefront and trip: 4 if that divides the row's count (8 measured slower), else 2
  const int pair = (K / BK) % 4 == 0 ? 4 : 2;
  const int64_t wanted = (n_blocks / pair + 3) / 4;
  const int cap = compute_units() * 16;
  const dim3 grid((unsigned)(wanted < cap ? wanted : cap));
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, wq, (const uint16_t*)scales, (const uint16_t*)biases,
                       (char*)out, (int)N, (int)K, (int)n_blocks);
  };
  if (bits == 3 || bits == 5 || bits == 6) {
    const int64_t want = (n_blocks / 2 + 3) / 4;
    const dim3 stream_grid((unsigned)(want < cap ? want : cap));
    auto go = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, stream_grid, dim3(256), 0, stream, wq, (const uint16_t*)scales,
                         (const uint16_t*)biases, (char*)out, (int)N, (int)K, (int)n_blocks);
    };
    if (bits == 3) go(dequant_frag_stream_kernel<T, GS, 3>);
    if (bits == 5) go(dequant_frag_stream_kernel<T, GS, 5>);
    if (bits == 6) go(dequant_frag_stream_kernel<T, GS, 6>);
  } else if (bits == 4) {
    if (pair == 4) launch(dequant_frag_kernel<T, GS, 4, 4>); else launch(dequant_frag_kernel<T, GS, 4, 2>);
  } else {
    if (pair == 4) launch(dequant_frag_kernel<T, GS, 8, 4>); else launch(dequant_frag_kernel<T, GS, 8, 2>);
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T>
int launch_dequant(const uint32_t* wq, const void* scales, const void* biases, int gs, int bits, void* out, int64_t N,
                   int64_t K, hipStream_t stream) {
  if (gs == 32) return launch_dequant_bits<T, 32>(wq, scales, biases, bits, out, N, K, stream);
  if (gs == 64) return launch_dequant_bits<T, 64>(wq, scales, biases, bits, out, N, K, stream);
  return launch_dequant_bits<T, 128>(wq, scales, biases, bits, out, N, K, stream);
}

template <typename T, bool kEpi, bool kCut, bool kLowRank, int kJ = 4, bool kDeferBias = false>
int launch_gemm(const void* x, int64_t M, int64_t K, const void* wfrag, const void* bias, int64_t N, void* y,
                int n_whole, int splits, float* planes, hipStream_t stream, LowRank lr, Epilogue epi) {
  auto kernel = frag_gemm_kernel<T, kEpi, kCut, kLowRank, kJ, kDeferBias>;
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLdsBytes)) return MFQ_ELAUNCH;
  const int tiles_m = (int)((M + BM - 1) / BM);
  const int tiles_n = (int)((N + 64 * kJ - 1) / (64 * kJ));
  const int n_tail = tiles_m * tiles_n - n_whole;
  const int n_items = n_whole + n_tail * splits;
  const int grid = n_items < compute_units() ? n_items : compute_units();  // one persistent workgroup per CU
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), kLdsBytes, stream, (const uint16_t*)x,
                     (const char*)wfrag, (const uint16_t*)bias, y, (int)M, (int)N, (int)K, tiles_m, tiles_n, n_whole,
                     splits, planes, (const uint16_t*)lr.t, (const uint16_t*)lr.bs, lr.R, epi);
  if (hipGetLastError() != hipSuccess) return MFQ_ELAUNCH;
  if (splits > 1)
    return launch_tail_reduce(T::code, planes, n_whole, splits, tiles_m, tiles_n, bias, M, N, y, T::code, stream, epi);
  return MFQ_OK;
}

template <typename T>
int launch_gemm_typed(const void* x, int64_t M, int64_t K, const void* copy, const void* bias, int64_t N, void* y,
                      float* planes, int n_whole, int splits, hipStream_t stream, LowRank lr, Epilogue epi) {
  auto go = [&](auto e, auto c, auto l) {
    return launch_gemm<T, decltype(e)::value, decltype(c)::value, decltype(l)::value>(
        x, M, K, copy, bias, N, y, n_whole, splits, planes, stream, lr, epi);
  };
  const std::true_type yes{};
  const std::false_type no{};
  // 192-column tiles where they fit one round of workgroups (the 256-column tiles of the same shape then do
  // too, with a third more work on each of fewer workgroups), unless the plan cuts that round along K
  const int64_t tiles_192 = ((M + BM - 1) / BM) * ((N + 191) / 192);
  if (epi.kind == kEpiNone && splits == 1 && tiles_192 <= compute_units()) {
    if (lr.R)
      return launch_gemm<T, false, false, true, 3>(x, M, K, copy, bias, N, y, (int)tiles_192, 1, planes, stream, lr, epi);
    return launch_gemm<T, false, false, false, 3>(x, M, K, copy, bias, N, y, (int)tiles_192, 1, planes, stream, lr, epi);
  }
  if (lr.R) return splits > 1 ? go(no, yes, yes) : go(no, no, yes);  // (no entry point combines update and epilogue)
  if (epi.kind != kEpiNone) return splits > 1 ? go(yes, yes, no) : go(yes, no, no);
  // with a bias and more than one whole tile to a workgroup: the instantiation whose deferred stores add it (the
  // one with the K cut's second loop for uncut calls too: without that loop behind it the compiler spills 292
  // registers on this variant)
  if (bias && n_whole > compute_units())
    return launch_gemm<T, false, true, false, 4, true>(x, M, K, copy, bias, N, y, n_whole, splits, planes, stream, lr,
                                                       epi);
  return splits > 1 ? go(no, yes, no) : go(no, no, no);
}

}  // namespace

bool qmm_frag_shape_ok(int64_t M, int64_t N, int64_t K, int bits) {
  // whole pairs of k steps and at least two of them; whole 16-byte pieces of y; 32-bit byte offsets into x
  // and into the scratch copy
  return (bits == 3 || bits == 4 || bits == 5 || bits == 6 || bits == 8) && K % (2 * BK) == 0 && K >= 4 * BK &&
         N % 8 == 0 && M * K < ((int64_t)1 << 31) &&
         ((N + 15) / 16) * 16 * K < ((int64_t)1 << 31);
}

// the copy, rounded up to whole 256 bytes so that what lies behind it is aligned
size_t qmm_frag_copy_bytes(int64_t N, int64_t K) { return ((size_t)(((N + 15) / 16) * 16 * K * 2) + 255) & ~(size_t)255; }

int launch_qmm_frag_copy(int dtype, const uint32_t* wq, const void* scales, const void* biases, int64_t N, int64_t K,
                         int gs, int bits, void* copy, hipStream_t stream) {
  if (!qmm_frag_shape_ok(1, N, K, bits)) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16) return launch_dequant<BF16>(wq, scales, biases, gs, bits, copy, N, K, stream);
  if (dtype == MFQ_F16) return launch_dequant<F16>(wq, scales, biases, gs, bits, copy, N, K, stream);
  return MFQ_EDTYPE;
}

int launch_qmm_frag_gemm(const void* x, int dtype, int64_t M, int64_t K, const void* copy, const void* bias, int64_t N,
                         void* y, float* planes, int n_whole, int splits, hipStream_t stream, LowRank lr,
                         Epilogue epi) {
  if (!qmm_frag_shape_ok(M, N, K, 4)) return MFQ_EUNSUPPORTED;
  if (lr.R && (epi.kind != kEpiNone || lr.R % 16)) return MFQ_EUNSUPPORTED;
  // 32-bit byte offsets into the update's operands
  if ((M + BM) * lr.R >= (int64_t)1 << 31 || (N + BN) * lr.R >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  if (splits > 1 && ((K / BK) % splits || (K / BK / splits) % 2)) return MFQ_EUNSUPPORTED;  // ranges of whole pairs of steps
  if (dtype == MFQ_BF16)
    return launch_gemm_typed<BF16>(x, M, K, copy, bias, N, y, planes, n_whole, splits, stream, lr, epi);
  if (dtype == MFQ_F16)
    return launch_gemm_typed<F16>(x, M, K, copy, bias, N, y, planes, n_whole, splits, stream, lr, epi);
  return MFQ_EDTYPE;
}

namespace {
template <typename T, int GS>
int launch_dequant_t_bits(const uint32_t* wq, const void* scales, const void* biases, int bits, void* out, int64_t N,
                          int64_t K, hipStream_t stream) {
  const int tiles_k = (int)((K + 255) / 256);
  const dim3 grid((unsigned)((N / BK) * tiles_k));
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, wq, (const uint16_t*)scales, (const uint16_t*)biases,
                       (char*)out, (int)N, (int)K, tiles_k);
  };
  if (bits == 4) go(dequant_frag_t_kernel<T, GS, 4>); else go(dequant_frag_t_kernel<T, GS, 8>);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}
template <typename T>
int launch_dequant_t(const uint32_t* wq, const void* scales, const void* biases, int gs, int bits, void* out, int64_t N,
                     int64_t K, hipStream_t stream) {
  if (gs == 32) return launch_dequant_t_bits<T, 32>(wq, scales, biases, bits, out, N, K, stream);
  if (gs == 64) return launch_dequant_t_bits<T, 64>(wq, scales, biases, bits, out, N, K, stream);
  return launch_dequant_t_bits<T, 128>(wq, scales, biases, bits, out, N, K, stream);
}
}  // namespace

// The two-kernel path for the weight NOT transposed: y[M, K] = x[M, N] @ dequantize(wq[N, K]).  The GEMM sees
// K output columns and sums over N.  4 and 8 bits, 16-bit y of x's type, whole pairs of 64-row steps.
bool qmm_frag_n_shape_ok(int64_t M, int64_t N, int64_t K, int bits) {
  return (bits == 4 || bits == 8) && K % 8 == 0 && N * K < ((int64_t)1 << 31) && qmm_frag_shape_ok(M, K, N, bits);
}

int launch_qmm_frag_n(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                      const void* biases, int64_t K, int gs, int bits, void* y, void* workspace, float* planes,
                      int n_whole, int splits, hipStream_t stream) {
  if (!qmm_frag_n_shape_ok(M, N, K, bits)) return MFQ_EUNSUPPORTED;
  int rc = MFQ_EDTYPE;
  if (dtype == MFQ_BF16) rc = launch_dequant_t<BF16>(wq, scales, biases, gs, bits, workspace, N, K, stream);
  if (dtype == MFQ_F16) rc = launch_dequant_t<F16>(wq, scales, biases, gs, bits, workspace, N, K, stream);
  if (rc) return rc;
  return launch_qmm_frag_gemm(x, dtype, M, N, workspace, nullptr, K, y, planes, n_whole, splits, stream, LowRank(),
                              Epilogue());
}

int launch_qmm_frag(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, void* workspace,
                    int n_whole, int splits, hipStream_t stream, LowRank lr, Epilogue epi) {
  if (!qmm_frag_shape_ok(M, N, K, bits)) return MFQ_EUNSUPPORTED;
  if (int rc = launch_qmm_frag_copy(dtype, wq, scales, biases, N, K, gs, bits, workspace, stream)) return rc;
  // the planes of a K cut lie behind the copy
  float* planes = reinterpret_cast<float*>(static_cast<char*>(workspace) + qmm_frag_copy_bytes(N, K));
  return launch_qmm_frag_gemm(x, dtype, M, K, workspace, bias, N, y, planes, n_whole, splits, stream, lr, epi);
}

}  // namespace mfq
