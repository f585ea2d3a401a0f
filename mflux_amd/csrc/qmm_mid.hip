// Medium-M W4/W8 x A16 quantized matmul for gfx950 (a few hundred activation
// rows: the text stream of mflux's joint transformer blocks, e.g.
// src/mflux/models/flux/model/flux_transformer/joint_transformer_block.py, and
// the T5 / Qwen text encoders at M = 256..1024):
//   y[M, N] = x[M, K] @ dequant(wq[N, K])^T (+ bias)
//
// With so few rows the 256 x 256 tiles of the large-M kernel are too few to
// fill the chip, and cutting K to make more of them costs a float32 plane of
// the output per cut.  Here a workgroup of four wavefronts computes a
// 128 x 128 tile, two workgroups share a compute unit (two wavefronts per SIMD
// hide each other's waits, so the code is left to the compiler's scheduler),
// and K is cut only when even these tiles are too few.
//   - both operands go through LDS as 16-bit tiles of 128 rows x 64 k, rows of
//     128 bytes with the 16-byte column index XORed with (row/2)%8: x is copied
//     (128-bit moves), the weights are dequantised on the way in, every code
//     exactly once per workgroup (thread t: feature t/2, half t%2 of the 64 k;
//     one float32 fma per code, single rounding to the 16-bit type);
//   - global loads run two k steps ahead in registers, the LDS tiles are
//     double buffered, one barrier per step;
//   - wavefront (wm, wn) owns rows [64wm, 64wm+64) x columns [64wn, 64wn+64) as
//     2 x 2 accumulators of the 32x32x16 matrix-core instruction, weights as
//     the A operand (so a lane ends up with four consecutive output columns).
#include <type_traits>
#include <utility>

#include "common.h"
#include "tile_epilogue.h"

namespace mfq {
namespace {

constexpr int TN = 128;
constexpr int TK = 64;
constexpr int kTileW = TN * TK * 2;  // the 16-bit weight tile: 16 KiB
// kWavesM wavefronts along M (2 or 4), two along N
constexpr int tile_m(int waves_m) { return 64 * waves_m; }
constexpr int threads_of(int waves_m) { return 2 * waves_m * kWave; }
constexpr int tile_x_bytes(int waves_m) { return tile_m(waves_m) * TK * 2; }
constexpr int lds_bytes(int waves_m) { return 2 * (tile_x_bytes(waves_m) + kTileW); }  // both tiles, double buffered

// 64 LDS banks of 4 bytes: a 128-bit access is conflict free when 16
// consecutive lanes cover one 256-byte window (two rows).
__device__ inline int swz(int row, int chunk) { return row * (TK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, kN - 1>)
template <typename F, int... kIs>
__device__ inline void for_each_index_impl(F&& f, std::integer_sequence<int, kIs...>) {
  (f(std::integral_constant<int, kIs>{}), ...);
}
template <int kN, typename F>
__device__ inline void for_each_index(F&& f) {
  for_each_index_impl(f, std::make_integer_sequence<int, kN>{});
}

// kFast: scales and biases are read as 8-byte pieces (four consecutive groups
// of a weight row) once per period of 4*GS/64 k steps; otherwise as one 2-byte
// value per step, and K may then end in half a step (K % 64 == 32, group size
// 32): what lies past K enters LDS as zeros on both sides.
//
// BITS 3, 5 and 6 (mflux's -q 3/5/6, src/mflux/cli/defaults/defaults.py:63): a
// row's codes are one little-endian bit stream, 32 codes in BITS whole words.
// 256 threads take one such unit each (feature t/2, half t%2 of the step) and
// cut the codes out at compile-time positions; with 512 threads the upper half
// only copies x.  For these widths the kernel serves every M above one row.
template <typename T, int GS, int BITS, bool kFast, int kWavesM>
__global__ __launch_bounds__(threads_of(kWavesM), 2) void qmm_mid_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int K, int tiles_m, int tiles_n, int steps, const uint16_t* __restrict__ lr_t,
    const uint16_t* __restrict__ lr_bs, int lr_rank, Epilogue epi) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;
  constexpr int TM = tile_m(kWavesM);
  constexpr int kThreads = threads_of(kWavesM);
  constexpr int kTileX = tile_x_bytes(kWavesM);
  constexpr int kBuf = kTileX + kTileW;       // one buffer: the x tile, then the weight tile
  constexpr bool kStream = BITS != 4 && BITS != 8;           // codes cut out of a bit stream
  constexpr int kDeqThreads = kStream ? 256 : kThreads;      // threads that dequantise
  constexpr int kCodes = TN * TK / kDeqThreads;  // weights such a thread dequantises per step: 32 or 16
  constexpr int kParts = TK / kCodes;         // threads per feature
  constexpr int kChunks = kCodes / 8;         // 8-code (16-byte) pieces it writes
  constexpr int kWords = kCodes * BITS / 32;  // 32-bit words of codes it loads
  constexpr int kPer = 4 * GS / TK;           // k steps covered by one 8-byte scale piece
  constexpr int kXPass = kThreads / 8;        // x rows copied per pass (four passes)

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wm = wave >> 1, wn = wave & 1;  // wm < kWavesM
  const int r = lane & 31;
  const int h = lane >> 5;

  // Work item = (k range, tile).  Workgroups are dealt round-robin to the 8
  // XCDs; item b is mapped so that an XCD walks a contiguous run of the tile
  // sequence (tile row fastest), sharing x tiles and weight tiles in its L2.
  const int n_tiles = tiles_m * tiles_n;
  const int split = blockIdx.x / n_tiles;
  int tile = blockIdx.x - split * n_tiles;
  {
    const int per_xcd = n_tiles / 8;
    if (tile < per_xcd * 8) tile = (tile & 7) * per_xcd + (tile >> 3);
  }
  const int m0 = (tile % tiles_m) * TM;
  const int n0 = (tile / tiles_m) * TN;
  const int kb = split * steps * TK;  // first k of the item
  char* y_item = static_cast<char*>(y) + (size_t)split * M * N * 4;  // split > 0 only with float32 planes

  // global offsets (bytes; they fit 32 bits, checked by the launcher)
  uint32_t xoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    xoff[i] = ((uint32_t)min(m0 + (t >> 3) + kXPass * i, M - 1) * (uint32_t)K + 8u * (t & 7)) * 2u;
  const bool deq = t < kDeqThreads;             // uniform per wavefront
  const int td = t % kDeqThreads;               // the other threads request what thread td does and drop it
  const int f = td / kParts, part = td % kParts;  // this thread's feature of the tile and part of the k step
  const int hh = part * kCodes / 32;            // which half of the step (the group, for groups of 32)
  const uint32_t wrow = (uint32_t)min(n0 + f, N - 1);
  constexpr int kPieceBytes = kCodes * BITS / 8;  // this thread's codes of one step
  const uint32_t woff = wrow * (uint32_t)(K * BITS / 8) + (uint32_t)(part * kPieceBytes);
  const uint32_t soff = wrow * (uint32_t)(K / GS) * 2u;
  const char* xbytes = reinterpret_cast<const char*>(x);
  const char* wbytes = reinterpret_cast<const char*>(wq);
  const char* sbytes = reinterpret_cast<const char*>(scales);
  const char* bbytes = reinterpret_cast<const char*>(biases);

  // LDS slots
  const int wr_x = swz(t >> 3, t & 7);
  int wr_w[kChunks];
#pragma unroll
  for (int c = 0; c < kChunks; ++c) wr_w[c] = swz(f, part * kChunks + c);
  int rd[4];
#pragma unroll
  for (int sub = 0; sub < 4; ++sub) rd[sub] = swz(r, 4 * h + sub);

  struct Stage {
    u32x4 x[4];
    uint32_t w[kWords];
    uint16_t s, b;  // !kFast
  };
  struct Period {  // kFast: scales and biases of four consecutive groups of the thread's weight row
    uint2 s, b;
  };
  Stage st[2];
  Period per[2];  // periods with an even / odd index

  // Everything below is unconditional and its register sets are chosen at
  // compile time, so that every wait for a load can leave exactly the younger
  // loads in flight.  q: k step inside the item (steps past the end repeat the
  // last one and are never consumed).
  // sel: -1, or the Period set to refill with the period that step q starts.
  auto load_rest = [&](auto sel, Stage& g, int q) __attribute__((always_inline)) {  // everything but x
    constexpr int kSel = decltype(sel)::value;
    const int k0 = kb + min(q, steps - 1) * TK;
    if constexpr (kFast) {
      if constexpr (kSel >= 0) {
        const int g0 = (k0 / GS) & ~3;
        per[kSel].s = *reinterpret_cast<const uint2*>(sbytes + soff + (size_t)g0 * 2);
        per[kSel].b = *reinterpret_cast<const uint2*>(bbytes + soff + (size_t)g0 * 2);
      }
    } else {
      const int g0 = min(k0 / GS + (GS == 32 ? hh : 0), K / GS - 1);
      g.s = *reinterpret_cast<const uint16_t*>(sbytes + soff + (size_t)g0 * 2);
      g.b = *reinterpret_cast<const uint16_t*>(bbytes + soff + (size_t)g0 * 2);
    }
    // a part past K (!kFast, K % 64 == 32) re-reads the row's last piece and is published as zeros
    int wcol = k0 * BITS / 8;
    if constexpr (!kFast) {
      wcol = min(wcol, K * BITS / 8 - (part + 1) * kPieceBytes);
    }
    const char* wsrc = wbytes + woff + wcol;
    if constexpr (kStream) {
#pragma unroll
      for (int l = 0; l < kWords; ++l) g.w[l] = *reinterpret_cast<const uint32_t*>(wsrc + 4 * l);
    } else if constexpr (kWords == 2) {
      const uint2 v = *reinterpret_cast<const uint2*>(wsrc);
      g.w[0] = v.x;
      g.w[1] = v.y;
    } else {
#pragma unroll
      for (int l = 0; l < kWords / 4; ++l) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(wsrc + 16 * l);
#pragma unroll
        for (int e = 0; e < 4; ++e) g.w[4 * l + e] = v[e];
      }
    }
  };
  auto load_x_piece = [&](Stage& g, int q, int i) __attribute__((always_inline)) {
    const int k0 = kb + min(q, steps - 1) * TK;
    int xcol = k0 * 2;
    if constexpr (!kFast) {  // a piece past K re-reads the row's last one and is published as zeros
      xcol = min(xcol, K * 2 - 16 * ((t & 7) + 1));
    }
    g.x[i] = *reinterpret_cast<const u32x4*>(xbytes + xoff[i] + xcol);
  };
  auto load = [&](auto sel, Stage& g, int q) __attribute__((always_inline)) {
    load_rest(sel, g, q);
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x_piece(g, q, i);
  };
  // the Period set step e of the unrolled sequence refills, if it starts a period
  auto sel_of = [](auto e) {
    constexpr int kE = decltype(e)::value % (2 * kPer);
    return std::integral_constant<int, (kFast && kE % kPer == 0) ? kE / kPer : -1>{};
  };

  // Scale and bias of this thread's 32 codes in step e of the unrolled sequence.
  auto scale_of = [&](auto e, const Stage& g, float& sc, float& bi) __attribute__((always_inline)) {
    if constexpr (kFast) {
      constexpr int kE = decltype(e)::value % (2 * kPer);
      constexpr int kIn = kE % kPer;
      const int idx = GS >= TK ? kIn * TK / GS : 2 * kIn + hh;  // group inside the period
      const Period& pr = per[kE / kPer];
      sc = T::to_f32((uint16_t)((((uint64_t)pr.s.y << 32) | pr.s.x) >> (16 * idx)));
      bi = T::to_f32((uint16_t)((((uint64_t)pr.b.y << 32) | pr.b.x) >> (16 * idx)));
    } else {
      sc = T::to_f32(g.s);
      bi = T::to_f32(g.b);
    }
  };
  // Quarter c of publishing a step's registers to buffer `buf`: one 128-bit
  // piece of x and (in every quarter, or every other one) eight dequantised
  // weights.
  // q: the step being published (its half past K, if any, becomes zeros).
  auto publish_part = [&](const Stage& g, int q, int c, float sc, float bi, int buf) __attribute__((always_inline)) {
    char* xd = lds + buf * kBuf;
    char* wd = xd + kTileX;
    const int k0 = kb + q * TK;
    u32x4 xv = g.x[c];
    if constexpr (!kFast) {
      if (k0 + 8 * (t & 7) >= K) xv = u32x4{0u, 0u, 0u, 0u};
    }
    *reinterpret_cast<u32x4*>(xd + wr_x + kXPass * TK * 2 * c) = xv;
    constexpr int kEvery = 4 / kChunks;
    if (c % kEvery == 0 && deq) {
      const int cw = c / kEvery;
      uint4 v;
      if constexpr (kStream) {
        v = dequant8_stream<T, BITS>(g.w, cw, sc, bi);
      } else if constexpr (BITS == 4) {
        v = dequant8_w4<T>(g.w[cw], sc, bi);
      } else {
        v = dequant8_w8<T>(g.w[2 * cw], g.w[2 * cw + 1], sc, bi);
      }
      if constexpr (!kFast) {
        if (k0 + part * kCodes >= K) v = make_uint4(0u, 0u, 0u, 0u);
      }
      *reinterpret_cast<uint4*>(wd + wr_w[cw]) = v;
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Step e of the unrolled sequence, k step p of the item: the matrix work on
  // buffer e%2, with quarter `sub` of publishing step p+1 to the other buffer
  // in the shadow of the matrix instructions of sub-step `sub` (a scheduling
  // barrier between sub-steps keeps the interleaving) and each quarter's
  // registers refilled for step p+3 as soon as they have been published.
  auto step = [&](auto e, int p) __attribute__((always_inline)) {
    constexpr int kE = decltype(e)::value;
    constexpr int buf = kE & 1;
    const Stage& next = st[buf ^ 1];
    const char* xs = lds + buf * kBuf + 4096 * (2 * wm);
    const char* ws = lds + buf * kBuf + kTileX + 4096 * (2 * wn);
    float sc, bi;
    scale_of(std::integral_constant<int, kE + 1>{}, next, sc, bi);
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
      publish_part(next, p + 1, sub, sc, bi, buf ^ 1);
      // the registers just published are refilled for step p+3 right away
      load_x_piece(st[buf ^ 1], p + 3, sub);
      if (sub == 3) load_rest(sel_of(std::integral_constant<int, kE + 3>{}), st[buf ^ 1], p + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };

  // prologue: steps 0, 1, 2 in flight, step 0 published
  {
    const std::integral_constant<int, 0> e0{};
    load(sel_of(e0), st[0], 0);
    load(sel_of(std::integral_constant<int, 1>{}), st[1], 1);
    float sc, bi;
    scale_of(e0, st[0], sc, bi);
#pragma unroll
    for (int c = 0; c < 4; ++c) publish_part(st[0], 0, c, sc, bi, 0);
    load(sel_of(std::integral_constant<int, 2>{}), st[0], 2);
    __syncthreads();
  }
  // The sequence is unrolled over two scale periods (kFast) or two steps.
  constexpr int kSeq = kFast ? 2 * kPer : 2;
  int p = 0;
  for (; p + kSeq <= steps; p += kSeq) for_each_index<kSeq>([&](auto e) __attribute__((always_inline)) { step(e, p + decltype(e)::value); });
  if constexpr (kFast) {
    // whole periods: what remains is one period
    if (p < steps) for_each_index<kPer>([&](auto e) __attribute__((always_inline)) { step(e, p + decltype(e)::value); });
  } else {
    if (p < steps) step(std::integral_constant<int, 0>{}, p);
  }

  // ---- low-rank update (lr_rank > 0): lr_rank more k after the item's own,
  // x side lr_t [M, lr_rank], weight side lr_bs [N, lr_rank], 16-bit and
  // unquantised.  They are few, so they come straight from memory as matrix
  // fragments (a lane's 8 consecutive k of a row are one 16-byte load); of the
  // k ranges of a tile the first one adds them.
  if (lr_rank > 0 && split == 0) {
    const uint16_t* trow[2];
    const uint16_t* brow[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      trow[i] = lr_t + (int64_t)min(m0 + 64 * wm + 32 * i + r, M - 1) * lr_rank + 8 * h;
      brow[i] = lr_bs + (int64_t)min(n0 + 64 * wn + 32 * i + r, N - 1) * lr_rank + 8 * h;
    }
#pragma unroll 1
    for (int k = 0; k < lr_rank; k += 16) {
      vec8 wf[2], xf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        wf[i] = *reinterpret_cast<const vec8*>(brow[i] + k);
        xf[i] = *reinterpret_cast<const vec8*>(trow[i] + k);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma32(wf[j], xf[i], acc[i][j]);
    }
  }

  // ---- epilogue: every LDS tile is free now (the loop ended with a barrier)
  store_block_64x64<T>(acc, lds, wave, lane, m0 + 64 * wm, n0 + 64 * wn, M, N, bias, y_item, y_is_f32, epi);
}

struct MidPlan {
  int splits;
  int steps;  // k steps per range
};

inline int period_of(int gs) { return 4 * gs / TK; }

// Up to 128 activation rows: 128-row tiles, two workgroups of four wavefronts
// per compute unit.  More: 256-row tiles (every dequantised weight then serves
// twice the matrix work), one workgroup of eight wavefronts per compute unit.
inline int waves_m_of(int64_t M) { return M <= 128 ? 2 : 4; }

// K is cut into equal ranges of whole scale periods (at least 8 k steps each)
// while the work items are fewer than the compute units and the cut keeps them
// within what runs at once.
inline MidPlan plan_mid(int64_t M, int64_t N, int64_t K, int period, int cus) {
  const int steps = (int)((K + TK - 1) / TK);  // K % 64 == 32: the last step is half empty
  const int waves_m = waves_m_of(M);
  const int tm = tile_m(waves_m);
  const int64_t tiles = ((M + tm - 1) / tm) * ((N + TN - 1) / TN);
  const int64_t slots = waves_m == 2 ? 2 * (int64_t)cus : cus;
  MidPlan plan{1, steps};
  if (K % TK || steps % period != 0) return plan;
  for (int s = 2; s <= steps / 8 && tiles * plan.splits < cus && tiles * s <= slots; ++s)
    if (steps % s == 0 && (steps / s) % period == 0) plan = MidPlan{s, steps / s};
  return plan;
}

template <typename T, int GS, int BITS, bool kFast, int kWavesM>
int launch_kernel(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, void* y, int y_dtype, MidPlan plan, hipStream_t stream, LowRank lr,
                  Epilogue epi) {
  auto kernel = qmm_mid_kernel<T, GS, BITS, kFast, kWavesM>;
  constexpr int kLds = lds_bytes(kWavesM);
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLds)) return MFQ_ELAUNCH;
  const int tiles_m = (int)((M + tile_m(kWavesM) - 1) / tile_m(kWavesM));
  const int tiles_n = (int)((N + TN - 1) / TN);
  const int64_t n_items = (int64_t)tiles_m * tiles_n * plan.splits;
  hipLaunchKernelGGL(kernel, dim3((unsigned)n_items), dim3(threads_of(kWavesM)), kLds, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, tiles_m, tiles_n, plan.steps,
                     (const uint16_t*)lr.t, (const uint16_t*)lr.bs, lr.R, epi);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int GS, int BITS, bool kFast>
int launch_tile(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, void* y, int y_dtype, MidPlan plan, hipStream_t stream, LowRank lr,
                Epilogue epi) {
  if (waves_m_of(M) == 2)
    return launch_kernel<T, GS, BITS, kFast, 2>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, plan, stream, lr, epi);
  return launch_kernel<T, GS, BITS, kFast, 4>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, plan, stream, lr, epi);
}

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, void* workspace, size_t workspace_bytes,
               hipStream_t stream, LowRank lr, Epilogue epi) {
  const int64_t steps = (K + TK - 1) / TK;
  constexpr int kPer = 4 * GS / TK;
  const bool aligned8 = ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 7u) == 0;
  if (!(K % TK == 0 && steps % kPer == 0 && aligned8))
    return launch_tile<T, GS, BITS, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, MidPlan{1, (int)steps},
                                           stream, lr, epi);
  const MidPlan plan = plan_mid(M, N, K, kPer, compute_units());
  const size_t need = (size_t)plan.splits * M * N * sizeof(float);
  if (plan.splits == 1 || !workspace || workspace_bytes < need || !aligned16(workspace))
    return launch_tile<T, GS, BITS, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, MidPlan{1, (int)steps},
                                          stream, lr, epi);
  // K cut into ranges: float32 planes, and the second kernel applies bias and epilogue
  if (int rc = launch_tile<T, GS, BITS, true>(x, M, K, wq, scales, biases, nullptr, N, workspace, MFQ_F32, plan,
                                              stream, lr, Epilogue()))
    return rc;
  return launch_splitk_reduce(T::code, workspace, plan.splits, M, N, bias, y, y_dtype, stream, epi);
}

// This file is compiled twice: as it is for 4 and 8 bits, and through
// qmm_mid_stream.hip (which defines MFQ_MID_STREAM and includes it) for the 3-,
// 5- and 6-bit packs, so that the two sets of instantiations build in parallel.
template <typename T, int GS>
int launch_bits(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int bits, void* y, int y_dtype, void* ws, size_t ws_bytes,
                hipStream_t stream, LowRank lr, Epilogue epi) {
#ifdef MFQ_MID_STREAM
  if (bits == 3)
    return launch_one<T, GS, 3>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
  if (bits == 5)
    return launch_one<T, GS, 5>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
  return launch_one<T, GS, 6>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
#else
  if (bits == 4)
    return launch_one<T, GS, 4>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
  return launch_one<T, GS, 8>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
#endif
}

template <typename T>
int launch_gs(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
              const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, void* ws, size_t ws_bytes,
              hipStream_t stream, LowRank lr, Epilogue epi) {
  switch (gs) {
    case 32:
      return launch_bits<T, 32>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, ws, ws_bytes, stream, lr, epi);
    case 64:
      return launch_bits<T, 64>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, ws, ws_bytes, stream, lr, epi);
    default:
      return launch_bits<T, 128>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, ws, ws_bytes, stream, lr, epi);
  }
}

}  // namespace

#ifdef MFQ_MID_STREAM
int launch_qmm_mid_stream(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                          const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                          void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank,
                          Epilogue epi) {
#else
size_t qmm_mid_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs) {
  const MidPlan plan = plan_mid(M, N, K, period_of(gs), compute_units());
  return plan.splits > 1 ? (size_t)plan.splits * M * N * sizeof(float) : 0;
}

int launch_qmm_mid(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank, Epilogue epi) {
  if (bits != 4 && bits != 8)
    return launch_qmm_mid_stream(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace,
                                 workspace_bytes, stream, low_rank, epi);
#endif
  // an epilogue lives in the 16-bit staged store (and in the second kernel of a K split)
  if (epi.kind != kEpiNone && (y_dtype == MFQ_F32 || N % 8)) return MFQ_EUNSUPPORTED;
  // 32-bit byte offsets into x, the packed weight and the scales
  if (M * K >= (int64_t)1 << 31 || N * K >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  if (dtype == MFQ_BF16)
    return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                           stream, low_rank, epi);
  if (dtype == MFQ_F16)
    return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                          stream, low_rank, epi);
  return MFQ_EDTYPE;
}

}  // namespace mfq
