// Large-M W4/W8 x A16 quantized matmul for gfx950:
//   y[M, N] = x[M, K] @ dequant(wq[N, K])^T (+ bias)
// the body of every QuantizedLinear call of mflux's diffusion transformers
// (e.g. src/mflux/models/flux/model/flux_transformer/
// single_transformer_block.py:53,57 at M = 4608).
//
// One workgroup of four wavefronts computes a 256 x 256 tile of y; wavefront w
// owns all 256 rows of output columns [64w, 64w+64) as 8 x 2 accumulators of
// the 32x32x16 matrix-core instruction.
//   - x goes HBM -> registers -> LDS (128-bit moves, one 64-wide k step ahead,
//     two LDS buffers, one barrier per step).  LDS rows are 128 bytes and the
//     16-byte column index is XORed with (row/2)%8, so the row-wise writes and
//     the 32-row fragment reads are both bank-conflict free.
//   - packed weights never touch LDS: a lane of the matrix core's B operand
//     holds 8 consecutive k of one output column, which is exactly one uint32
//     of 4-bit codes (two of 8-bit codes).  Each lane streams 128-bit pieces of
//     its own weight row straight from HBM/L2 into registers one step ahead and
//     dequantises a word with one float32 fma per code (single rounding to the
//     16-bit type) right before the matrix instruction that consumes it.  No
//     column is dequantised by more than one wavefront.
//   - scales and biases are read as 8-byte pieces (four consecutive groups of
//     one weight row) once per "period" of 4*GS/64 k steps and unpacked step by
//     step.  Reading the 2-byte values one step at a time refetches the same
//     cache line from L2 for every step of every row, which saturates the L2
//     and costs a third of the kernel's time.
//   - the k order inside a step is permuted (lane half h covers k 32h..32h+31)
//     identically for both operands, which the dot product does not notice.
#include <type_traits>

#include "common.h"
#include "epilogue.h"

namespace mfq {
namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;   // one 16-bit x tile: 32 KiB
constexpr int kStageStride = 144;         // bytes per staged output row: 64 16-bit columns + 16 bytes of padding
constexpr int kStageBytes = 128 * kStageStride;  // one wavefront stages 128 rows of its 64 columns at a time
constexpr int kBiasBytes = 64 * 4;  // per wavefront: the bias of its 64 columns as float32
constexpr int kLdsBytes = 2 * kTileBytes + 4 * kStageBytes + 4 * kBiasBytes;  // x tiles (double-buffered) + output staging + bias
constexpr int kWriteSub = 2;  // sub-step whose fillers publish the next x tile to LDS

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// LDS has 64 banks of 4 bytes: a 128-bit access is conflict free when every 16
// consecutive lanes cover one 256-byte window, i.e. two 128-byte rows.  XORing
// the 16-byte column index with bits 1..3 of the row makes that true both for
// the row-wise writes (8 lanes per row) and for the fragment reads (16 rows,
// one column).
__device__ inline int swz(int row, int chunk) { return row * (BK * 2) + ((chunk ^ ((row >> 1) & 7)) << 4); }

// Per-lane stream of packed weights for the wavefront's two 32-column tiles.
template <typename T, int GS, int BITS>
struct WeightRegs {
  static constexpr int kLoads = BITS / 4;  // 128-bit loads per column tile and step (32 codes per lane)
  u32x4 w[2][kLoads];
  float s[2], b[2];

  // woff/soff: this lane's byte offsets of its two weight rows / scale rows;
  // k0 is uniform, so every address is a uniform base plus a 32-bit lane offset.
  __device__ inline void issue_codes(const uint32_t* wq, const uint32_t (&woff)[2], int k0) {
    const char* wbase = reinterpret_cast<const char*>(wq) + (size_t)k0 * BITS / 8;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int l = 0; l < kLoads; ++l) w[j][l] = *reinterpret_cast<const u32x4*>(wbase + woff[j] + 16 * l);
  }

  // codes plus this step's scale and bias, one 2-byte load each (the path for
  // shapes the period-wise scale loads do not cover)
  __device__ inline void issue(const uint32_t* wq, const uint16_t* scales, const uint16_t* biases,
                               const uint32_t (&woff)[2], const uint32_t (&soff)[2], int k0) {
    issue_codes(wq, woff, k0);
    const char* sbase = reinterpret_cast<const char*>(scales) + (size_t)(k0 / GS) * 2;
    const char* bbase = reinterpret_cast<const char*>(biases) + (size_t)(k0 / GS) * 2;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      s[j] = T::to_f32(*reinterpret_cast<const uint16_t*>(sbase + soff[j]));
      b[j] = T::to_f32(*reinterpret_cast<const uint16_t*>(bbase + soff[j]));
    }
  }

  // code i (0..7) of sub-step `sub` of column tile j, as float
  __device__ inline float code(int j, int sub, int i, uint32_t even, uint32_t odd) const {
    if constexpr (BITS == 4) {
      return ubyte_f32((i & 1) ? odd : even, i >> 1);
    } else {
      return ubyte_f32(w[j][sub >> 1][(sub & 1) * 2 + (i >> 2)], i & 3);
    }
  }
  __device__ inline float deq(int j, int sub, int i, uint32_t even, uint32_t odd) const {
    return __builtin_fmaf(code(j, sub, i, even, odd), s[j], b[j]);
  }
};

// Scales and biases of four consecutive groups of the lane's two weight rows:
// one period of kPeriod = 4*GS/BK k steps.
template <typename T, int GS>
struct ScaleRegs {
  static constexpr int kPeriod = 4 * GS / BK;  // k steps covered by one load
  uint2 s[2], b[2];

  // g0: first group of the period (a multiple of 4); soff: byte offsets of the
  // lane's two scale rows
  __device__ inline void issue(const uint16_t* scales, const uint16_t* biases, const uint32_t (&soff)[2], int g0) {
    const char* sbase = reinterpret_cast<const char*>(scales) + (size_t)g0 * 2;
    const char* bbase = reinterpret_cast<const char*>(biases) + (size_t)g0 * 2;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      s[j] = *reinterpret_cast<const uint2*>(sbase + soff[j]);
      b[j] = *reinterpret_cast<const uint2*>(bbase + soff[j]);
    }
  }

  // Scale and bias of step e (0 <= e < kPeriod) of the period for lane half h.
  template <typename WR>
  __device__ inline void extract(WR& dst, int e, int h) const {
    const int idx = GS >= BK ? e * BK / GS : 2 * e + h;  // group inside the period
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint64_t sv = ((uint64_t)s[j].y << 32) | s[j].x;
      const uint64_t bv = ((uint64_t)b[j].y << 32) | b[j].x;
      dst.s[j] = T::to_f32((uint16_t)(sv >> (16 * idx)));
      dst.b[j] = T::to_f32((uint16_t)(bv >> (16 * idx)));
    }
  }
};

// Position `tile` of the tile sequence -> origin of the tile.  Workgroups are
// dealt round-robin to the 8 XCDs, so with a grid that is a multiple of 8 a
// workgroup stays on XCD b%8 and that XCD's workgroups walk a contiguous run of
// the sequence together.  Inside the run the tiles are ordered in bands of
// kBandM tile-rows, row index fastest, so the ~32 tiles in flight on one XCD
// share kBandM x-tiles and 8 weight-tiles per k step in that XCD's L2.
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

// kEpi: the tile's 16-bit results pass through `epi` (epilogue.h) on their way from the staging
// region to y; instantiated apart so that the plain kernel's code is what it was.
template <typename T, int GS, int BITS, bool kFast, bool kLowRank, bool kEpi>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void qmm_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int K, int tiles_m, int tiles_n, int n_whole, int tail_splits, float* __restrict__ planes,
    const uint16_t* __restrict__ lr_t, const uint16_t* __restrict__ lr_bs, int lr_rank, Epilogue epi) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;
  using WR = WeightRegs<T, GS, BITS>;
  using SR = ScaleRegs<T, GS>;

  const int n_tiles = tiles_m * tiles_n;
  // work items: the first n_whole tiles of the sequence whole, every later tile as tail_splits k ranges
  const int n_items = n_whole + (n_tiles - n_whole) * tail_splits;
  const int steps_total = K / BK;
  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wn = wave * 64;
  const int r = lane & 31;
  const int h = lane >> 5;

  // Persistent workgroups: workgroup b takes items b, b + grid, b + 2*grid, ...
  // The launcher makes the whole tiles a whole number of rounds; what is left
  // of the tile sequence (fewer tiles than compute units) can be cut along K
  // so that the last round is short instead of mostly idle: k range s of tail
  // tile t accumulates into float32 plane t * tail_splits + s (256 x 256,
  // dense) of `planes`, and a second kernel adds the planes into y.
  struct Item {
    int m0, n0;
    int first_step, n_steps;  // its k range, in steps
    int plane;                // -1: the whole tile, written to y; else the index of its float32 plane
  };
  auto item_of = [&](int seq) {
    Item it;
    int tile = seq;
    it.first_step = 0;
    it.n_steps = steps_total;
    it.plane = -1;
    if (seq >= n_whole) {
      const int e = seq - n_whole;
      const int tail_tile = e / tail_splits;
      tile = n_whole + tail_tile;
      it.n_steps = steps_total / tail_splits;
      it.first_step = (e - tail_tile * tail_splits) * it.n_steps;
      it.plane = e;
    }
    tile_origin(tile, tiles_m, tiles_n, it.m0, it.n0);
    return it;
  };
  int steps = steps_total;  // k steps of the item in hand

  // Per-lane byte offsets of the tile the PREFETCH cursor is in (it runs two k
  // steps ahead of the matrix work and enters the next tile two steps early;
  // the scale cursor runs one period further ahead still).  Rows past M / N are
  // clamped for loads.  Lane half h starts 32 codes into a step; with GS == 32
  // that is also one group further (the period-wise loads start at the row's
  // first group instead and pick the half when unpacking).  Offsets fit 32
  // bits (checked by the launcher).
  uint32_t woff[2], soff[2], xoff[8];
  auto set_scale_tile = [&](int n0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t n = (uint32_t)min(n0 + wn + 32 * j + r, N - 1);
      soff[j] = (n * (uint32_t)(K / GS) + (kFast ? 0u : (uint32_t)((32 * h) / GS))) * 2u;
    }
  };
  auto set_prefetch_tile = [&](int m0, int n0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t n = (uint32_t)min(n0 + wn + 32 * j + r, N - 1);
      woff[j] = n * (uint32_t)(K * BITS / 8) + (uint32_t)(32 * h * BITS / 8);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      xoff[i] = ((uint32_t)min(m0 + (t >> 3) + 32 * i, M - 1) * (uint32_t)K + 8u * (t & 7)) * 2u;
  };
  const char* xbytes = reinterpret_cast<const char*>(x);
  // LDS addresses: the write slot of this thread (row t/8 of each 32-row block)
  // and, per k sub-step, the read slot of this lane (row r of each 32-row block)
  const int wr_slot = swz(t >> 3, t & 7);
  int rd_slot[4];
#pragma unroll
  for (int sub = 0; sub < 4; ++sub) rd_slot[sub] = swz(r, 4 * h + sub);

  // x tile registers: set p receives the tile of a step with parity p, two
  // steps before it is used, and is published to LDS buffer p one step before.
  u32x4 xa[2][8];
  // where the item in hand writes its results: the address of element (m0, n0),
  // the row pitch in elements, the element type and the bias to add (planes:
  // float32, 256 apart, no bias)
  char* out_base = static_cast<char*>(y);
  int out_stride = N;
  bool out_f32 = y_is_f32;
  const uint16_t* out_bias = bias;
  WR wa, wb;            // packed weights of the current even / odd step
  SR sr;                // scales and biases of the period the prefetch cursor is in (kFast only)
  uint32_t bf[2][4];    // dequantised fragments of the next sub-step to run
  f32x16 acc[8][2];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Dequantisation of one 8-code fragment, cut into 7 chunks of at most four
  // VALU instructions so that a chunk fits in the shadow of one matrix
  // instruction.  tmp/even/odd carry state between the chunks of a fragment.
  struct Dq {
    float tmp[8];
    uint32_t even, odd;
  };
  // The empty asm statements pin each chunk where it is written: without them
  // the optimiser is free to sink the arithmetic to its first use (for the
  // last sub-step that is the next iteration) and to undo the byte-wise
  // extraction of the 4-bit codes.
  auto dq_chunk = [&](const WR& w, int j, int sub, int c, Dq& d, uint32_t (&out)[4]) __attribute__((always_inline)) {
    switch (c) {
      case 0:
        if constexpr (BITS == 4) {
          d.even = w.w[j][0][sub] & 0x0f0f0f0fu;
          d.odd = (w.w[j][0][sub] >> 4) & 0x0f0f0f0fu;
          asm volatile("" : "+v"(d.even), "+v"(d.odd));
        }
        break;
      case 1:
        d.tmp[0] = w.deq(j, sub, 0, d.even, d.odd);
        d.tmp[1] = w.deq(j, sub, 1, d.even, d.odd);
        asm volatile("" : "+v"(d.tmp[0]), "+v"(d.tmp[1]));
        break;
      case 2:
        out[0] = T::pack2(d.tmp[0], d.tmp[1]);
        d.tmp[2] = w.deq(j, sub, 2, d.even, d.odd);
        asm volatile("" : "+v"(out[0]), "+v"(d.tmp[2]));
        break;
      case 3:
        d.tmp[3] = w.deq(j, sub, 3, d.even, d.odd);
        out[1] = T::pack2(d.tmp[2], d.tmp[3]);
        asm volatile("" : "+v"(out[1]));
        break;
      case 4:
        d.tmp[4] = w.deq(j, sub, 4, d.even, d.odd);
        d.tmp[5] = w.deq(j, sub, 5, d.even, d.odd);
        asm volatile("" : "+v"(d.tmp[4]), "+v"(d.tmp[5]));
        break;
      case 5:
        out[2] = T::pack2(d.tmp[4], d.tmp[5]);
        d.tmp[6] = w.deq(j, sub, 6, d.even, d.odd);
        asm volatile("" : "+v"(out[2]), "+v"(d.tmp[6]));
        break;
      case 6:
        d.tmp[7] = w.deq(j, sub, 7, d.even, d.odd);
        out[3] = T::pack2(d.tmp[6], d.tmp[7]);
        asm volatile("" : "+v"(out[3]));
        break;
      default:
        break;
    }
  };
  auto as_frag = [](const uint32_t (&v)[4]) {
    return __builtin_bit_cast(vec8, make_uint4(v[0], v[1], v[2], v[3]));
  };

  // One k step, written as 64 groups of (one matrix instruction + its fillers)
  // in the order they are to issue; a scheduling barrier after every group
  // keeps that order.  `now` / `next` are the weight registers of this step and
  // the following one; k_pref is the k offset, inside the prefetch cursor's
  // tile, of the step two ahead.  Fillers, per 16-instruction sub-step: the
  // chunks of the two fragments the NEXT sub-step needs, one LDS read of the
  // next slot's x fragments after every other matrix instruction, and
  //   sub-step 0: global loads of the x tile two steps ahead (one per group),
  //   sub-step 2: the LDS writes that publish the x tile of the following step
  //               (early, so that they have landed when the step's closing
  //               barrier is reached),
  //   sub-step 3: global loads of the weights two steps ahead into `now`
  //               (consumed during sub-step 2).
  //   kFast: `now` also receives, at that point, the scale and bias of the step
  //               two ahead (step e_pref of the period held in `sr`); when that
  //               was the period's last step (`reload`), `sr` is refilled from
  //               group g_pref on, to be unpacked one step later.
  auto do_step = [&](auto parity, auto reload, WR& now, const WR& next, int k_pref, int e_pref, int g_pref)
      __attribute__((always_inline)) {
    constexpr int kP = decltype(parity)::value;  // parity of the step: LDS buffer and x register set
    constexpr bool kReload = decltype(reload)::value;
    const char* xs = lds + kP * kTileBytes;
    char* xd = lds + (kP ^ 1) * kTileBytes;
    vec8 af[2][4];
    auto read_frag = [&](int q, int i) {
      af[q & 1][i] = *reinterpret_cast<const vec8*>(xs + rd_slot[q >> 1] + 4096 * (4 * (q & 1) + i));
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) read_frag(0, i);
    uint32_t nb[2][4];
    Dq dq;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      const vec8 b0 = as_frag(bf[0]);
      const vec8 b1 = as_frag(bf[1]);
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const int q = 2 * sub + (m >> 3);
        const int i = (m & 7) >> 1;
        const int ai = 4 * (q & 1) + i;
        if (m & 1) {
          acc[ai][1] = mfma32(b1, af[q & 1][i], acc[ai][1]);
        } else {
          acc[ai][0] = mfma32(b0, af[q & 1][i], acc[ai][0]);
        }
        // fillers
        if (sub < 3) {
          dq_chunk(now, m >> 3, sub + 1, m & 7, dq, nb[m >> 3]);
        } else {
          dq_chunk(next, m >> 3, 0, m & 7, dq, nb[m >> 3]);
        }
        if ((m & 1) && q < 7) read_frag(q + 1, i);
        if (sub == 0 && m < 8) xa[kP][m] = *reinterpret_cast<const u32x4*>(xbytes + (size_t)k_pref * 2 + xoff[m]);
        if (sub == 3 && m == 0) {
          if constexpr (kFast) {
            now.issue_codes(wq, woff, k_pref);
            sr.extract(now, e_pref, h);
            if constexpr (kReload) sr.issue(scales, biases, soff, g_pref);
          } else {
            now.issue(wq, scales, biases, woff, soff, k_pref);
          }
        }
        if (sub == kWriteSub && (m & 1) == 0) *reinterpret_cast<u32x4*>(xd + wr_slot + 4096 * (m >> 1)) = xa[kP ^ 1][m >> 1];
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) bf[j][e] = nb[j][e];
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  const std::integral_constant<int, 0> even_step{};
  const std::integral_constant<int, 1> odd_step{};
  const std::false_type keep{};
  const std::true_type refill{};

  // Fills the pipeline for the tile the prefetch offsets point at: x(0) into
  // LDS buffer 0, x(1) into register set 1, weights of steps 0 and 1, and the
  // fragments of sub-step 0.
  auto prime = [&](int kb) {  // kb: first k of the item
    const int k1 = kb + min(1, steps - 1) * BK;
#pragma unroll
    for (int i = 0; i < 8; ++i) xa[1][i] = *reinterpret_cast<const u32x4*>(xbytes + (size_t)kb * 2 + xoff[i]);
    if constexpr (kFast) {
      sr.issue(scales, biases, soff, kb / GS);
      wa.issue_codes(wq, woff, kb);
      wb.issue_codes(wq, woff, k1);
      sr.extract(wa, 0, h);
      sr.extract(wb, 1, h);
      if constexpr (SR::kPeriod == 2) sr.issue(scales, biases, soff, kb / GS + 4);  // steps >= 4 here
    } else {
      wa.issue(wq, scales, biases, woff, soff, kb);
      wb.issue(wq, scales, biases, woff, soff, k1);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(lds + wr_slot + 4096 * i) = xa[1][i];
#pragma unroll
    for (int i = 0; i < 8; ++i) xa[1][i] = *reinterpret_cast<const u32x4*>(xbytes + (size_t)k1 * 2 + xoff[i]);
    Dq d;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int c = 0; c < 7; ++c) dq_chunk(wa, j, 0, c, d, bf[j]);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // The low-rank update (kLowRank): lr_rank more k after the item's own, whose
  // x side is lr_t [M, lr_rank] and whose weight side is lr_bs [N, lr_rank],
  // both 16-bit and unquantised.  They are few, so they bypass the pipeline: a
  // lane's 8 consecutive k of a row are one 16-byte load straight into a matrix
  // fragment (k 16 c + 8 h + 0..7 for chunk c of 16, the same for both sides).
  auto low_rank_steps = [&](int m0, int n0) {
    int lane_e = lane;  // opaque copy, see store_tile_staged
    asm volatile("" : "+v"(lane_e));
    const int r = lane_e & 31;
    const int h = lane_e >> 5;
    const char* tb = reinterpret_cast<const char*>(lr_t) + 16 * h;
    const char* bb = reinterpret_cast<const char*>(lr_bs) + 16 * h;
    const uint32_t pitch = (uint32_t)lr_rank * 2u;  // bytes per row of either matrix
    uint32_t boff[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) boff[j] = (uint32_t)min(n0 + wn + 32 * j + r, N - 1) * pitch;
    const uint32_t toff = (uint32_t)min(m0 + r, M - 1) * pitch;
    // rows 32 ai + r of the tile: 32 * pitch apart until the clamp at M - 1
    const uint32_t t_last = (uint32_t)(M - 1) * pitch;
#pragma unroll 1
    for (uint32_t kb = 0; kb < pitch; kb += 32) {
      vec8 wf[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) wf[j] = *reinterpret_cast<const vec8*>(bb + boff[j] + kb);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        vec8 xf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          xf[i] = *reinterpret_cast<const vec8*>(tb + min(toff + (uint32_t)(4 * half + i) * 32u * pitch, t_last) + kb);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[4 * half + i][j] = mfma32(wf[j], xf[i], acc[4 * half + i][j]);
      }
    }
  };

  // Writes the finished tile.  The weights were the matrix instruction's A
  // operand, so accumulator [ai][j] holds, in register e, output row
  // m0 + 32*ai + r and column n0 + wn + 32*j + 8*(e/4) + 4*h + e%4: four
  // consecutive columns per register quad, stored as one 8-byte (16-bit y) or
  // 16-byte (float32 y) piece.  Nothing waits for the stores; they drain while
  // the next tile is computed.
  auto store_tile_direct = [&](int m0, int n0) {
    int lane_e = lane;  // opaque copy, see store_tile_staged
    asm volatile("" : "+v"(lane_e));
    const int r = lane_e & 31;
    const int h = lane_e >> 5;
    const bool n_vec_ok = (N & 3) == 0 && (out_stride & 3) == 0;  // keeps every piece aligned and inside the row
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        const int col = n0 + wn + 32 * j + 8 * eb + 4 * h;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (out_bias) {
#pragma unroll
          for (int c = 0; c < 4; ++c) bv[c] = T::to_f32(out_bias[min(col + c, N - 1)]);
        }
#pragma unroll
        for (int ai = 0; ai < 8; ++ai) {
          const int row = m0 + 32 * ai + r;
          if (row >= M || col >= N) continue;
          float v[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] = acc[ai][j][4 * eb + c];
          const int64_t o = (int64_t)(row - m0) * out_stride + (col - n0);
          if (out_f32) {
            float* dst = reinterpret_cast<float*>(out_base) + o;
            if (out_bias) {
#pragma unroll
              for (int c = 0; c < 4; ++c) v[c] += bv[c];
            }
            if (n_vec_ok) {
              *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
              for (int c = 0; c < 4; ++c)
                if (col + c < N) dst[c] = v[c];
            }
          } else {
            uint16_t hv[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              hv[c] = T::from_f32(v[c]);
              if (out_bias) hv[c] = T::from_f32(T::to_f32(hv[c]) + bv[c]);
            }
            uint16_t* dst = reinterpret_cast<uint16_t*>(out_base) + o;
            if (n_vec_ok) {
              uint2 pk;
              pk.x = (uint32_t)hv[0] | ((uint32_t)hv[1] << 16);
              pk.y = (uint32_t)hv[2] | ((uint32_t)hv[3] << 16);
              *reinterpret_cast<uint2*>(dst) = pk;
            } else {
#pragma unroll
              for (int c = 0; c < 4; ++c)
                if (col + c < N) dst[c] = hv[c];
            }
          }
        }
      }
    }
  };

  // 16-bit output with N a multiple of 8: each wavefront transposes its
  // 256 x 64 block through a private LDS region, 128 rows at a time, so that
  // every global store instruction writes eight complete 128-byte row
  // segments (16 bytes per lane).  Rows of the staging region are 144 bytes
  // apart, which spreads both the 8-byte writes (32 rows at once) and the
  // 16-byte reads (8 rows at once) over all banks.  The region is private to
  // the wavefront, so no workgroup barrier is needed.
  auto store_tile_staged = [&](auto with_bias, int m0, int n0) {
    constexpr bool kBias = decltype(with_bias)::value;
    // An opaque copy of the lane id: everything below is derived from it, so
    // none of this per-tile address arithmetic can be hoisted out of the tile
    // loop and kept live (spilled) across the k loop.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int r = lane_e & 31;
    const int h = lane_e >> 5;
    const int lane = lane_e;
    char* stage = lds + 2 * kTileBytes + wave * kStageBytes;
    uint16_t* yout = reinterpret_cast<uint16_t*>(out_base);
    // the bias of the wavefront's 64 columns: one load (lane l takes column l), parked in LDS as
    // float32 and read back four columns at a time; fetched value by value where it is used, every
    // fetch would be waited for on its own, 32 times per tile
    const float* bias_f = reinterpret_cast<const float*>(lds + 2 * kTileBytes + 4 * kStageBytes + wave * kBiasBytes);
    if constexpr (kBias) {
      *reinterpret_cast<float*>(lds + 2 * kTileBytes + 4 * kStageBytes + wave * kBiasBytes + lane * 4) =
          T::to_f32(out_bias[min(n0 + wn + lane, N - 1)]);
    }
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) {
          const int cl = 32 * j + 8 * eb + 4 * h;  // column inside the wavefront's 64
          float bv[4] = {0.f, 0.f, 0.f, 0.f};
          if constexpr (kBias) {
            const float4 b4 = *reinterpret_cast<const float4*>(bias_f + cl);
            bv[0] = b4.x, bv[1] = b4.y, bv[2] = b4.z, bv[3] = b4.w;
          }
#pragma unroll
          for (int a4 = 0; a4 < 4; ++a4) {
            const int ai = 4 * pass + a4;
            uint32_t pk[2];
#pragma unroll
            for (int c = 0; c < 2; ++c) {
              pk[c] = T::pack2(acc[ai][j][4 * eb + 2 * c], acc[ai][j][4 * eb + 2 * c + 1]);
              if constexpr (kBias)  // second rounding, as a separate add on the 16-bit result would do
                pk[c] = T::pack2(lo_f32<T>(pk[c]) + bv[2 * c], hi_f32<T>(pk[c]) + bv[2 * c + 1]);
            }
            *reinterpret_cast<uint2*>(stage + (32 * a4 + r) * kStageStride + cl * 2) = make_uint2(pk[0], pk[1]);
          }
          // keep the compiler from converting the whole tile before the first write
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // read back row-wise: lane l takes 16 bytes (8 columns) of row 8*k + l/8
      const int cg = n0 + wn + 8 * (lane & 7);
      if constexpr (kEpi) {
        if (epi.kind == kEpiSwiglu) {
          // the wavefront's 64 columns are 32 of the gate projection, then their 32 of the up projection:
          // lane l takes 8 gate columns and the 8 up columns 32 further of row 16*k + l/4 and writes
          // 8 of the tile's 128 output columns (yout / out_stride address the [M, N/2] result)
          const int cq = lane & 3;
          const int co = (wn >> 1) + 8 * cq;  // output column inside the tile
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const int rl = 16 * k + (lane >> 2);
            const u32x4 g = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * cq);
            const u32x4 u = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 64 + 16 * cq);
            u32x4 v;
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = epi_swiglu_pair<T>(g[c], u[c]);
            const int row = m0 + 128 * pass + rl;
            if (row < M && n0 + wn + 8 * cq < N)
              *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + co) = v;
          }
          continue;
        }
        if (epi.kind == kEpiGateResidual) {
          u32x4 gate8 = {0u, 0u, 0u, 0u};
          if (cg < N) gate8 = *reinterpret_cast<const u32x4*>(epi.gate + cg);
          const uint16_t* res = epi.residual + (int64_t)m0 * N + cg;  // row m0 of this lane's columns
#pragma unroll
          for (int k4 = 0; k4 < 4; ++k4) {
            u32x4 rv[4];
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {  // four rows' residuals requested before the first is needed
              const int rl = 8 * (4 * k4 + kk) + (lane >> 3);
              const int row = min(m0 + 128 * pass + rl, M - 1);
              rv[kk] = cg < N ? *reinterpret_cast<const u32x4*>(res + (int64_t)(row - m0) * N) : gate8;
            }
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
              const int rl = 8 * (4 * k4 + kk) + (lane >> 3);
              u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * (lane & 7));
#pragma unroll
              for (int c = 0; c < 4; ++c) v[c] = epi_gate_residual_pair<T>(v[c], gate8[c], rv[kk][c]);
              const int row = m0 + 128 * pass + rl;
              if (row < M && cg < N) *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + (cg - n0)) = v;
            }
          }
          continue;
        }
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int rl = 8 * k + (lane >> 3);
        u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStageStride + 16 * (lane & 7));
        if constexpr (kEpi) {
          if (epi.kind == kEpiGelu && cg >= epi.act_from) {
#pragma unroll
            for (int c = 0; c < 4; ++c) v[c] = epi_gelu_pair<T>(v[c]);
          }
        }
        const int row = m0 + 128 * pass + rl;
        if (row < M && cg < N) *reinterpret_cast<u32x4*>(yout + (int64_t)(row - m0) * out_stride + (cg - n0)) = v;
        if (k & 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // float32 output with N a multiple of 4 (the planes of a K split, float32 y):
  // the same transpose, 64 rows at a time; a staged row is 64 floats plus 16
  // bytes of padding, which again spreads the 16-byte writes (32 rows at once)
  // and reads (4 rows at once) over all banks.  Every global store instruction
  // writes four complete 256-byte row segments.
  auto store_tile_staged_f32 = [&](int m0, int n0) {
    constexpr int kStride = 64 * 4 + 16;
    static_assert(64 * kStride <= kStageBytes, "float32 staging must fit the region of the 16-bit one");
    int lane_e = lane;  // opaque copy, see store_tile_staged
    asm volatile("" : "+v"(lane_e));
    const int r = lane_e & 31;
    const int h = lane_e >> 5;
    const int lane = lane_e;
    char* stage = lds + 2 * kTileBytes + wave * kStageBytes;
    float* yout = reinterpret_cast<float*>(out_base);
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) {
          const int cl = 32 * j + 8 * eb + 4 * h;  // column inside the wavefront's 64
          float bv[4] = {0.f, 0.f, 0.f, 0.f};
          if (out_bias) {
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[c] = T::to_f32(out_bias[min(n0 + wn + cl + c, N - 1)]);
          }
#pragma unroll
          for (int a2 = 0; a2 < 2; ++a2) {
            const int ai = 2 * pass + a2;
            *reinterpret_cast<float4*>(stage + (32 * a2 + r) * kStride + cl * 4) =
                make_float4(acc[ai][j][4 * eb] + bv[0], acc[ai][j][4 * eb + 1] + bv[1], acc[ai][j][4 * eb + 2] + bv[2],
                            acc[ai][j][4 * eb + 3] + bv[3]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // read back row-wise: lane l takes 16 bytes (4 columns) of row 4*k + l/16
      const int cg = n0 + wn + 4 * (lane & 15);
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const int rl = 4 * k + (lane >> 4);
        const float4 v = *reinterpret_cast<const float4*>(stage + rl * kStride + 16 * (lane & 15));
        const int row = m0 + 64 * pass + rl;
        if (row < M && cg < N) *reinterpret_cast<float4*>(yout + (int64_t)(row - m0) * out_stride + (cg - n0)) = v;
        if (k & 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  auto store_tile = [&](int m0, int n0) {
    if (!out_f32 && (out_stride & 7) == 0 && (N & 7) == 0) {
      if (out_bias) {
        store_tile_staged(std::true_type{}, m0, n0);
      } else {
        store_tile_staged(std::false_type{}, m0, n0);
      }
    } else if (out_f32 && (out_stride & 3) == 0 && (N & 3) == 0) {
      store_tile_staged_f32(m0, n0);
    } else {
      store_tile_direct(m0, n0);
    }
  };

  bool primed = false;
  for (int seq = blockIdx.x; seq < n_items; seq += gridDim.x) {
    const Item item = item_of(seq);
    const int m0 = item.m0, n0 = item.n0;
    steps = item.n_steps;
    const int kb = item.first_step * BK;          // first k of this item
    constexpr int kGroupsPerStep2 = 2 * BK / GS;  // groups per step, times two (GS == 128: one)
    const int gb = item.first_step * kGroupsPerStep2 / 2;  // its first group
    if (item.plane < 0) {
      out_base = static_cast<char*>(y) + ((size_t)m0 * N + n0) * (y_is_f32 ? 4 : 2);
      out_stride = N;
      if constexpr (kEpi) {
        if (epi.kind == kEpiSwiglu) {  // y is [M, N/2], 16-bit
          out_base = static_cast<char*>(y) + ((size_t)m0 * (N / 2) + n0 / 2) * 2;
          out_stride = N / 2;
        }
      }
      out_f32 = y_is_f32;
      out_bias = bias;
    } else {
      out_base = reinterpret_cast<char*>(planes + (size_t)item.plane * (BM * BN));
      out_stride = BN;
      out_f32 = true;
      out_bias = nullptr;
    }
    if (!primed) {
      set_scale_tile(n0);
      set_prefetch_tile(m0, n0);
      prime(kb);
    }
    if constexpr (kFast) {
      // Pairs of steps (p, p+1), laid out period by period so that what each
      // step unpacks is known at compile time.  The odd step of a pair unpacks
      // the scales of step p+3; when that is the last step of a period it also
      // refills `sr` with the period of step p+4.  The last period of the tile
      // is peeled: the scale cursor enters the next tile (if this workgroup has
      // one) before the pair that refills for it, the code / x cursor before
      // the last pair.  Without a next tile those prefetches re-read pieces of
      // this tile and are never consumed.
      constexpr int kPer = SR::kPeriod;
      auto pair = [&](auto pos, int k_a, int g) __attribute__((always_inline)) {
        // pos: position of the pair's even step inside its period
        constexpr int kPos = decltype(pos)::value;
        constexpr int e_a = (kPos + 2) % kPer, e_b = (kPos + 3) % kPer;
        do_step(even_step, keep, wa, wb, k_a, e_a, 0);
        if constexpr (e_b == kPer - 1) {
          do_step(odd_step, refill, wb, wa, k_a + BK, e_b, g);
        } else {
          do_step(odd_step, keep, wb, wa, k_a + BK, e_b, 0);
        }
      };
      // every pair of a period except its last two
      auto period_head = [&](int p) __attribute__((always_inline)) {
        if constexpr (kPer == 8) {
          pair(std::integral_constant<int, 0>{}, kb + (p + 2) * BK, 0);
          pair(std::integral_constant<int, 2>{}, kb + (p + 4) * BK, 0);
        }
      };
      const bool has_next = seq + (int)gridDim.x < n_items;
      for (int p = 0; p < steps - (kPer >= 4 ? kPer : 4); p += kPer) {
        period_head(p);
        if constexpr (kPer >= 4) {
          pair(std::integral_constant<int, kPer - 4>{}, kb + (p + kPer - 2) * BK, gb + (p + kPer) * kGroupsPerStep2 / 2);
          pair(std::integral_constant<int, kPer - 2>{}, kb + (p + kPer) * BK, 0);
        } else {
          pair(std::integral_constant<int, 0>{}, kb + (p + 2) * BK, gb + (p + 4) * kGroupsPerStep2 / 2);
        }
      }
      {
        const int p = steps - kPer;  // first step of the last period
        Item next = item;
        if (has_next) next = item_of(seq + gridDim.x);
        const int m1 = next.m0, n1 = next.n0;
        const int kb1 = next.first_step * BK, gb1 = next.first_step * kGroupsPerStep2 / 2;  // the next item's first k, group
        const int g_last = gb + p * kGroupsPerStep2 / 2;  // this item's last period, for prefetches nobody consumes
        const int k_last = kb + (steps - 2) * BK;
        if constexpr (kPer >= 4) {
          period_head(p);
          if (has_next) set_scale_tile(n1);
          pair(std::integral_constant<int, kPer - 4>{}, k_last, has_next ? gb1 : g_last);
          if (has_next) set_prefetch_tile(m1, n1);
          pair(std::integral_constant<int, kPer - 2>{}, has_next ? kb1 : k_last, 0);
        } else {
          // the main loop stopped one period early: steps - 4 and steps - 2 remain
          if (has_next) set_scale_tile(n1);
          pair(std::integral_constant<int, 0>{}, k_last, has_next ? gb1 : g_last);
          if (has_next) set_prefetch_tile(m1, n1);
          pair(std::integral_constant<int, 0>{}, has_next ? kb1 : k_last, has_next ? gb1 + 4 : g_last);
        }
      }
      primed = has_next;
    } else {
      int step = 0;
      for (; step + 1 < steps; step += 2) {  // never cut along K: kb == 0
        do_step(even_step, keep, wa, wb, min(step + 2, steps - 1) * BK, 0, 0);
        do_step(odd_step, keep, wb, wa, min(step + 3, steps - 1) * BK, 0, 0);
      }
      if (step < steps) do_step(even_step, keep, wa, wb, (steps - 1) * BK, 0, 0);
    }
    if constexpr (kLowRank) {
      if (item.first_step == 0) low_rank_steps(m0, n0);  // once per tile: by the item that has its first k range
    }
    store_tile(m0, n0);
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  }
}

// ---- the last round of tiles cut along K ---------------------------------------
// The tiles that fill whole rounds of the compute units run whole.  The tail of
// the sequence -- fewer tiles than compute units, which would keep most of the
// chip idle for a full tile time -- is cut into `splits` equal k ranges of whole
// scale periods when a caller-provided workspace is there: every range goes to
// its own dense 256 x 256 float32 plane and tail_reduce_kernel adds the planes
// up, rounds and applies the bias.
struct TailPlan {
  int n_whole;  // tiles of the sequence that run whole
  int splits;   // k ranges per tail tile; 1: nothing is cut
};

// period: k steps per scale period of the group size.  The cut must pay for
// its planes: a range saves steps - steps/splits k steps of about 1.6 us each
// on the critical path, a plane costs about 0.13 us of memory traffic (256 KiB
// written and read back) plus the second launch.
inline TailPlan plan_tail(int64_t M, int64_t N, int64_t K, int period, int cus) {
  const int steps = (int)(K / BK);
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int64_t tail = tiles % cus;
  TailPlan plan{(int)tiles, 1};
  if (tail == 0 || steps % period != 0 || steps < 8) return plan;
  int best = 1;
  for (int s = 2; s <= steps / 4 && tail * s <= cus; ++s)
    if (steps % s == 0 && (steps / s) % period == 0) best = s;
  if (best == 1) return plan;
  const double saved_us = 1.6 * (steps - steps / best);
  const double cost_us = 0.13 * (double)tail * best + 6.0;
  if (saved_us > 1.25 * cost_us) plan = TailPlan{(int)(tiles - tail), best};
  return plan;
}

inline int period_of(int gs) { return 4 * gs / BK; }

// y = sum of `splits` dense float32 planes of M x N (+ bias), through the epilogue: the second kernel of
// the 128-column-tile GEMM's K split.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ planes, int splits,
                                                            int64_t plane_elems, const uint16_t* __restrict__ bias,
                                                            int N, void* __restrict__ y, int y_is_f32, Epilogue epi) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // the value of the linear layer in column c: rounded, then the bias added and rounded again, as the fused
  // epilogue does (float32 y: one float32 sum)
  auto linear = [&](float v, int c) {
    const float bv = bias ? T::to_f32(bias[c]) : 0.f;
    if (y_is_f32) return v + bv;
    const float h = round_to<T>(v);
    return bias ? round_to<T>(h + bv) : h;
  };
  auto sum4 = [&](int64_t q) {
    float4 sum = reinterpret_cast<const float4*>(planes)[q];
    for (int sp = 1; sp < splits; ++sp) {
      const float4 v = reinterpret_cast<const float4*>(planes + sp * plane_elems)[q];
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    return sum;
  };
  // four consecutive outputs per thread when rows are a multiple of four long
  // (a quad then never straddles two rows), one otherwise
  if ((N & 3) == 0) {
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < plane_elems / 4; q += stride) {
      const int col = (int)((q * 4) % N);
      if (epi.kind == kEpiSwiglu && (col & 32)) continue;  // the up projection's columns are read by the gate's threads
      const float4 sum = sum4(q);
      float v[4] = {linear(sum.x, col), linear(sum.y, col + 1), linear(sum.z, col + 2), linear(sum.w, col + 3)};
      if (epi.kind == kEpiSwiglu) {  // N % 64 == 0; y is [M, N/2]
        const float4 ups = sum4(q + 8);
        const float u[4] = {linear(ups.x, col + 32), linear(ups.y, col + 33), linear(ups.z, col + 34), linear(ups.w, col + 35)};
        const int64_t row = (q * 4) / N;
        uint2 pk;
        pk.x = T::pack2(epi_swiglu<T>(v[0], u[0]), epi_swiglu<T>(v[1], u[1]));
        pk.y = T::pack2(epi_swiglu<T>(v[2], u[2]), epi_swiglu<T>(v[3], u[3]));
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(y) + row * (N / 2) + (col >> 6) * 32 + (col & 31)) = pk;
        continue;
      }
      if (epi.kind == kEpiGelu && col >= epi.act_from) {
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = epi_gelu<T>(v[c]);
      }
      if (epi.kind == kEpiGateResidual) {
        const uint2 g = *reinterpret_cast<const uint2*>(epi.gate + col);
        const uint2 r = reinterpret_cast<const uint2*>(epi.residual)[q];
        v[0] = epi_gate_residual<T>(v[0], lo_f32<T>(g.x), lo_f32<T>(r.x));
        v[1] = epi_gate_residual<T>(v[1], hi_f32<T>(g.x), hi_f32<T>(r.x));
        v[2] = epi_gate_residual<T>(v[2], lo_f32<T>(g.y), lo_f32<T>(r.y));
        v[3] = epi_gate_residual<T>(v[3], hi_f32<T>(g.y), hi_f32<T>(r.y));
      }
      if (y_is_f32) {
        reinterpret_cast<float4*>(y)[q] = make_float4(v[0], v[1], v[2], v[3]);
      } else {
        reinterpret_cast<uint2*>(y)[q] = make_uint2(T::pack2(v[0], v[1]), T::pack2(v[2], v[3]));
      }
    }
  } else {  // no epilogue on this path (the launcher refuses it)
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < plane_elems; i += stride) {
      float sum = planes[i];
      for (int sp = 1; sp < splits; ++sp) sum += planes[sp * plane_elems + i];
      const float v = linear(sum, (int)(i % N));
      if (y_is_f32) {
        reinterpret_cast<float*>(y)[i] = v;
      } else {
        reinterpret_cast<uint16_t*>(y)[i] = T::from_f32(v);
      }
    }
  }
}

// y tile = sum of the `splits` planes of each tail tile (+ bias), through the epilogue.  One thread per
// four consecutive columns of a tile row.
template <typename T>
__global__ __launch_bounds__(256) void tail_reduce_kernel(const float* __restrict__ planes, int n_whole, int splits,
                                                          int tiles_m, int tiles_n, const uint16_t* __restrict__ bias,
                                                          int M, int N, void* __restrict__ y, int y_is_f32,
                                                          Epilogue epi) {
  const int tail_tile = blockIdx.x / (BM * BN / 4 / 256);
  const int q = (blockIdx.x % (BM * BN / 4 / 256)) * 256 + threadIdx.x;  // quad inside the tile
  const int r = q / (BN / 4), c = (q % (BN / 4)) * 4;
  int m0, n0;
  tile_origin(n_whole + tail_tile, tiles_m, tiles_n, m0, n0);
  const int row = m0 + r, col = n0 + c;
  if (row >= M || col >= N) return;
  if (epi.kind == kEpiSwiglu && (c & 32)) return;  // the up projection's columns are read by the gate's threads
  const float* src = planes + (size_t)tail_tile * splits * (BM * BN) + r * BN + c;
  auto sum_at = [&](const float* p) {
    float4 sum = *reinterpret_cast<const float4*>(p);
    for (int sp = 1; sp < splits; ++sp) {
      const float4 v = *reinterpret_cast<const float4*>(p + (size_t)sp * (BM * BN));
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    return sum;
  };
  // the value of the linear layer in column cc: rounded, then the bias added and rounded again, as the fused
  // epilogue does (float32 y: one float32 sum)
  auto linear = [&](float v, int cc) {
    const float bv = bias ? T::to_f32(bias[cc]) : 0.f;
    if (y_is_f32) return v + bv;
    const float h = round_to<T>(v);
    return bias ? round_to<T>(h + bv) : h;
  };
  const float4 sum = sum_at(src);
  const float v[4] = {sum.x, sum.y, sum.z, sum.w};
  if (epi.kind == kEpiSwiglu) {
    const float4 ups = sum_at(src + 32);
    const float u[4] = {ups.x, ups.y, ups.z, ups.w};
    uint16_t* dst = reinterpret_cast<uint16_t*>(y) + (int64_t)row * (N / 2) + (col >> 6) * 32 + (col & 31);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[e] = T::from_f32(epi_swiglu<T>(linear(v[e], col + e), linear(u[e], col + 32 + e)));
    return;
  }
  const int64_t o = (int64_t)row * N + col;
  auto finish = [&](int e) {
    float out = linear(v[e], col + e);
    if (epi.kind == kEpiGelu && col + e >= epi.act_from) out = epi_gelu<T>(out);
    if (epi.kind == kEpiGateResidual)
      out = epi_gate_residual<T>(out, T::to_f32(epi.gate[col + e]), T::to_f32(epi.residual[o + e]));
    return out;
  };
  if ((N & 3) == 0) {  // the quad lies inside the row and is aligned: one store
    const float out[4] = {finish(0), finish(1), finish(2), finish(3)};
    if (y_is_f32) {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(y) + o) = make_float4(out[0], out[1], out[2], out[3]);
    } else {
      *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(y) + o) =
          make_uint2(T::pack2(out[0], out[1]), T::pack2(out[2], out[3]));
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (col + e >= N) break;
    const float out = finish(e);
    if (y_is_f32) {
      reinterpret_cast<float*>(y)[o + e] = out;
    } else {
      reinterpret_cast<uint16_t*>(y)[o + e] = T::from_f32(out);
    }
  }
}

template <typename T, int GS, int BITS, bool kFast, bool kLowRank = false, bool kEpi = false>
int launch_kernel(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, void* y, int y_dtype, TailPlan plan, void* planes, hipStream_t stream,
                  LowRank lr = LowRank(), Epilogue epi = Epilogue()) {
  auto kernel = qmm_kernel<T, GS, BITS, kFast, kLowRank, kEpi>;
  static PerDeviceInt configured;
  if (!raise_lds_limit(configured, reinterpret_cast<const void*>(kernel), kLdsBytes)) return MFQ_ELAUNCH;
  const int tiles_m = (int)((M + BM - 1) / BM);
  const int tiles_n = (int)((N + BN - 1) / BN);
  const int n_tail = tiles_m * tiles_n - plan.n_whole;
  const int n_items = plan.n_whole + n_tail * plan.splits;
  const int grid = n_items < compute_units() ? n_items : compute_units();  // one persistent workgroup per CU
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), kLdsBytes, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, tiles_m, tiles_n, plan.n_whole, plan.splits,
                     (float*)planes, (const uint16_t*)lr.t, (const uint16_t*)lr.bs, lr.R, epi);
  if (hipGetLastError() != hipSuccess) return MFQ_ELAUNCH;
  if (plan.splits > 1) {
    const unsigned blocks = (unsigned)n_tail * (BM * BN / 4 / 256);
    hipLaunchKernelGGL((tail_reduce_kernel<T>), dim3(blocks), dim3(256), 0, stream, (const float*)planes, plan.n_whole,
                       plan.splits, tiles_m, tiles_n, (const uint16_t*)bias, (int)M, (int)N, y,
                       (int)(y_dtype == MFQ_F32), epi);
    if (hipGetLastError() != hipSuccess) return MFQ_ELAUNCH;
  }
  return MFQ_OK;
}

inline size_t tail_plane_bytes(int64_t M, int64_t N, TailPlan plan) {
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  return plan.splits > 1 ? (size_t)(tiles - plan.n_whole) * plan.splits * BM * BN * sizeof(float) : 0;
}

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, void* workspace, size_t workspace_bytes,
               hipStream_t stream, LowRank lr, Epilogue epi) {
  // 32-bit byte offsets into x, the packed weight and the scales
  if (M * K >= (int64_t)1 << 31 || N * K >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  if ((M + BM) * lr.R >= (int64_t)1 << 31 || (N + BN) * lr.R >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const TailPlan whole{(int)tiles, 1};
  // period-wise scale loads: whole periods, at least two pairs of steps, and
  // 8-byte aligned scale rows
  const int64_t steps = K / BK;
  constexpr int kPer = ScaleRegs<T, GS>::kPeriod;
  const bool aligned8 = ((reinterpret_cast<uintptr_t>(scales) | reinterpret_cast<uintptr_t>(biases)) & 7u) == 0;
  const bool fast = steps % kPer == 0 && steps >= 4 && aligned8;
  TailPlan plan = fast ? plan_tail(M, N, K, kPer, compute_units()) : whole;
  if (plan.splits > 1 && (!workspace || workspace_bytes < tail_plane_bytes(M, N, plan) || !aligned16(workspace)))
    plan = whole;
#ifdef MFQ_QMM_EPI
  // the epilogues live in the staged 16-bit store of the period-wise kernel (the launcher has checked y and N)
  if (!fast || lr.R) return MFQ_EUNSUPPORTED;
  return launch_kernel<T, GS, BITS, true, false, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, plan,
                                                       workspace, stream, lr, epi);
#else
  if (!fast) {
    // the rare shapes without period-wise scale loads: the update comes from its own kernel
    const int rc =
        launch_kernel<T, GS, BITS, false>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, whole, nullptr, stream);
    return rc ? rc : launch_low_rank_add(T::code, lr, M, N, y, y_dtype, stream);
  }
  if (lr.R)
    return launch_kernel<T, GS, BITS, true, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, plan, workspace,
                                                  stream, lr);
  return launch_kernel<T, GS, BITS, true>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, plan, workspace, stream);
#endif
}

template <typename T, int GS>
int launch_bits(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int bits, void* y, int y_dtype, void* ws, size_t ws_bytes,
                hipStream_t stream, LowRank lr, Epilogue epi) {
  if (bits == 4)
    return launch_one<T, GS, 4>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
  return launch_one<T, GS, 8>(x, M, K, wq, scales, biases, bias, N, y, y_dtype, ws, ws_bytes, stream, lr, epi);
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
      return launch_bits<T, 128>(x, M, K, wq, scales, biases, bias, N, bits, y, y_dtype, ws, ws_bytes, stream, lr,
                                 epi);
  }
}

int launch_types(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                 const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                 void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank, Epilogue epi) {
  if (dtype == MFQ_BF16)
    return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                           stream, low_rank, epi);
  if (dtype == MFQ_F16)
    return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                          stream, low_rank, epi);
  return MFQ_EDTYPE;
}

}  // namespace

// This file is compiled twice: as it is, and through qmm_epi.hip (which defines
// MFQ_QMM_EPI and includes it) for the instantiations whose tiles pass through an
// epilogue, so that the two sets build in parallel.
#ifdef MFQ_QMM_EPI
int launch_qmm_epilogue(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                        const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                        void* workspace, size_t workspace_bytes, hipStream_t stream, Epilogue epi) {
  if (y_dtype == MFQ_F32 || N % 8) return MFQ_EUNSUPPORTED;  // the epilogues live in the 16-bit staged store
  return launch_types(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                      stream, LowRank(), epi);
}
#else
// Shapes whose 256 x 256 tiles would leave more than half of the compute units
// idle go to the 128-column-tile kernel, except many rows against a long K,
// where cutting K between 256 x 256 tiles measures about a tenth faster.
bool use_mid_kernel(int64_t M, int64_t N, int64_t K) {
  const bool few_tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN) * 2 <= compute_units();
  return few_tiles && !(M > 512 && K >= 8192);
}

#ifndef MFQ_ODD_FRAG_ROWS
#define MFQ_ODD_FRAG_ROWS 1024
#endif
constexpr int64_t kOddBitsFragRows = MFQ_ODD_FRAG_ROWS;

// The two-kernel path (qmm_frag.hip: a 16-bit scratch copy of the weights in fragment order, then a lean
// GEMM) takes the shapes it wins on: at least eight rows of tiles to spread the copy over.  It cuts K for
// the tail of the tile sequence by the same plan as the fused kernel.
bool prefer_frag_path(int64_t M, int64_t N, int64_t K, int gs, int bits) {
  // (3, 5 and 6 bits: the alternative is the 128-column-tile kernel with its codes cut out of a bit stream,
  // which the copy overtakes much earlier)
  const int64_t least_rows = (bits == 4 || bits == 8) ? 2048 : kOddBitsFragRows;
  return M >= least_rows && qmm_frag_shape_ok(M, N, K, bits) && !use_mid_kernel(M, N, K);
}

size_t qmm_min_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs) {
  if (K % BK) return 0;
  if (use_mid_kernel(M, N, K)) return qmm_mid_workspace_bytes(M, N, K, gs);
  return tail_plane_bytes(M, N, plan_tail(M, N, K, period_of(gs), compute_units()));
}

size_t qmm_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs, int bits) {
  const size_t planes = qmm_min_workspace_bytes(M, N, K, gs);
  return prefer_frag_path(M, N, K, gs, bits) ? qmm_frag_copy_bytes(N, K) + planes : planes;
}

int launch_tail_reduce(int dtype, const float* planes, int n_whole, int splits, int tiles_m, int tiles_n,
                       const void* bias, int64_t M, int64_t N, void* y, int y_dtype, hipStream_t stream, Epilogue epi) {
  const unsigned blocks = (unsigned)(tiles_m * tiles_n - n_whole) * (BM * BN / 4 / 256);
  if (dtype == MFQ_BF16) {
    hipLaunchKernelGGL((tail_reduce_kernel<BF16>), dim3(blocks), dim3(256), 0, stream, planes, n_whole, splits, tiles_m,
                       tiles_n, (const uint16_t*)bias, (int)M, (int)N, y, (int)(y_dtype == MFQ_F32), epi);
  } else if (dtype == MFQ_F16) {
    hipLaunchKernelGGL((tail_reduce_kernel<F16>), dim3(blocks), dim3(256), 0, stream, planes, n_whole, splits, tiles_m,
                       tiles_n, (const uint16_t*)bias, (int)M, (int)N, y, (int)(y_dtype == MFQ_F32), epi);
  } else {
    return MFQ_EDTYPE;
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

int launch_splitk_reduce(int dtype, const void* planes, int splits, int64_t M, int64_t N, const void* bias, void* y,
                         int y_dtype, hipStream_t stream, Epilogue epi) {
  const int64_t plane = M * N;
  const int64_t threads = (N & 3) == 0 ? plane / 4 : plane;
  const int64_t blocks = (threads + 255) / 256;
  const int cap = compute_units() * 8;
  const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
  if (dtype == MFQ_BF16) {
    hipLaunchKernelGGL((splitk_reduce_kernel<BF16>), grid, dim3(256), 0, stream, (const float*)planes, splits, plane,
                       (const uint16_t*)bias, (int)N, y, (int)(y_dtype == MFQ_F32), epi);
  } else if (dtype == MFQ_F16) {
    hipLaunchKernelGGL((splitk_reduce_kernel<F16>), grid, dim3(256), 0, stream, (const float*)planes, splits, plane,
                       (const uint16_t*)bias, (int)N, y, (int)(y_dtype == MFQ_F32), epi);
  } else {
    return MFQ_EDTYPE;
  }
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

// The K cut of the two-kernel path's GEMM when the copy is already there: ranges of whole pairs of k steps.
size_t qmm_prepared_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (K % (2 * BK)) return 0;
  return tail_plane_bytes(M, N, plan_tail(M, N, K, 2, compute_units()));
}

int launch_qmm_prepared(const void* x, int dtype, int64_t M, int64_t K, const void* copy, const void* bias, int64_t N,
                        void* y, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (!qmm_frag_shape_ok(M, N, K, 4)) return MFQ_EUNSUPPORTED;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  TailPlan plan = plan_tail(M, N, K, 2, compute_units());
  if (plan.splits > 1 && (!workspace || !aligned16(workspace) || workspace_bytes < tail_plane_bytes(M, N, plan)))
    plan = TailPlan{(int)tiles, 1};
  return launch_qmm_frag_gemm(x, dtype, M, K, copy, bias, N, y, static_cast<float*>(workspace), plan.n_whole,
                              plan.splits, stream, LowRank(), Epilogue());
}

// The untransposed product on the two-kernel path: from 1024 rows of x on (the kernel it replaces there,
// qmm_n.hip, runs at half the rate), where the transposed copy exists and the GEMM's tiles fill the chip.
static bool prefer_frag_n(int64_t M, int64_t N, int64_t K, int bits) {
  return M >= 1024 && qmm_frag_n_shape_ok(M, N, K, bits) && !use_mid_kernel(M, K, N);
}

size_t qmm_n_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs, int bits) {
  if (!prefer_frag_n(M, N, K, bits)) return 0;
  return qmm_frag_copy_bytes(K, N) + tail_plane_bytes(M, K, plan_tail(M, K, N, 2, compute_units()));
}

int launch_qmm_n_ws(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                    const void* biases, int64_t K, int gs, int bits, void* y, int y_dtype, void* workspace,
                    size_t workspace_bytes, hipStream_t stream) {
  if (y_dtype == dtype && workspace && aligned16(workspace) && prefer_frag_n(M, N, K, bits) &&
      workspace_bytes >= qmm_frag_copy_bytes(K, N)) {
    const int64_t tiles = ((M + BM - 1) / BM) * ((K + BN - 1) / BN);
    TailPlan plan = plan_tail(M, K, N, 2, compute_units());
    if (plan.splits > 1 && workspace_bytes < qmm_frag_copy_bytes(K, N) + tail_plane_bytes(M, K, plan))
      plan = TailPlan{(int)tiles, 1};
    float* planes = reinterpret_cast<float*>(static_cast<char*>(workspace) + qmm_frag_copy_bytes(K, N));
    return launch_qmm_frag_n(x, dtype, M, N, wq, scales, biases, K, gs, bits, y, workspace, planes, plan.n_whole,
                             plan.splits, stream);
  }
  return launch_qmm_n(x, dtype, M, N, wq, scales, biases, K, gs, bits, y, y_dtype, stream);
}

int launch_qmm(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank, Epilogue epi) {
  if (use_mid_kernel(M, N, K))
    return launch_qmm_mid(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace,
                          workspace_bytes, stream, low_rank, epi);
  // the two-kernel path where it wins and the caller has brought room for the scratch copy (and, behind it, for
  // the planes of the K cut: without those the tiles run whole)
  if (y_dtype == dtype && workspace && aligned16(workspace) && !(low_rank.R && epi.kind != kEpiNone) &&
      workspace_bytes >= qmm_frag_copy_bytes(N, K) && prefer_frag_path(M, N, K, gs, bits)) {
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    TailPlan plan = plan_tail(M, N, K, period_of(gs), compute_units());
    if (plan.splits > 1 && workspace_bytes < qmm_frag_copy_bytes(N, K) + tail_plane_bytes(M, N, plan))
      plan = TailPlan{(int)tiles, 1};
    return launch_qmm_frag(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, workspace, plan.n_whole,
                           plan.splits, stream, low_rank, epi);
  }
  if (epi.kind != kEpiNone)
    return launch_qmm_epilogue(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace,
                               workspace_bytes, stream, epi);
  return launch_types(x, dtype, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, workspace, workspace_bytes,
                      stream, low_rank, epi);
}
#endif

}  // namespace mfq
