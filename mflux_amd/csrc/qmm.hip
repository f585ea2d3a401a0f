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
//     16-byte column index is XORed with row%8, so the row-wise writes and the
//     32-row fragment reads are both bank-conflict free.
//   - packed weights never touch LDS: a lane of the matrix core's B operand
//     holds 8 consecutive k of one output column, which is exactly one uint32
//     of 4-bit codes (two of 8-bit codes).  Each lane streams 128-bit pieces of
//     its own weight row straight from HBM/L2 into registers one step ahead and
//     dequantises a word with one float32 fma per code (single rounding to the
//     16-bit type) right before the matrix instruction that consumes it.  No
//     column is dequantised by more than one wavefront.
//   - the k order inside a step is permuted (lane half h covers k 32h..32h+31)
//     identically for both operands, which the dot product does not notice.
#include <type_traits>

#include "common.h"

namespace mfq {
namespace {

constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kTileBytes = BM * BK * 2;   // one 16-bit x tile: 32 KiB
constexpr int kLdsBytes = 2 * kTileBytes; // double buffered

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ inline int swz(int row, int chunk) { return row * (BK * 2) + ((chunk ^ (row & 7)) << 4); }

// Per-lane stream of packed weights for the wavefront's two 32-column tiles.
template <typename T, int GS, int BITS>
struct WeightRegs {
  static constexpr int kLoads = BITS / 4;  // 128-bit loads per column tile and step (32 codes per lane)
  u32x4 w[2][kLoads];
  float s[2], b[2];

  // woff/soff: this lane's byte offsets of its two weight rows / scale rows;
  // k0 is uniform, so every address is a uniform base plus a 32-bit lane offset.
  __device__ inline void issue(const uint32_t* wq, const uint16_t* scales, const uint16_t* biases,
                               const uint32_t (&woff)[2], const uint32_t (&soff)[2], int k0) {
    const char* wbase = reinterpret_cast<const char*>(wq) + (size_t)k0 * BITS / 8;
    const char* sbase = reinterpret_cast<const char*>(scales) + (size_t)(k0 / GS) * 2;
    const char* bbase = reinterpret_cast<const char*>(biases) + (size_t)(k0 / GS) * 2;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int l = 0; l < kLoads; ++l) w[j][l] = *reinterpret_cast<const u32x4*>(wbase + woff[j] + 16 * l);
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

template <typename T, int GS, int BITS>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void qmm_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ bias, void* __restrict__ y, int y_is_f32, int M,
    int N, int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  using vec8 = typename T::vec8;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of tiles so that neighbours in the run (same weight columns, adjacent
  // x rows) share that XCD's L2.
  const int n_tiles = tiles_m * tiles_n;
  int tile = blockIdx.x;
  {
    const int per_xcd = n_tiles / 8;
    if (tile < per_xcd * 8) tile = (tile & 7) * per_xcd + (tile >> 3);
  }
  // Within an XCD's run, walk the tiles in bands of kBandM tile-rows, row
  // index fastest: the ~32 workgroups resident on one XCD then cover about
  // kBandM x 8 tiles and share kBandM x-tiles and 8 weight-tiles per k step.
  constexpr int kBandM = 4;
  const int band_tiles = kBandM * tiles_n;
  const int band = tile / band_tiles;
  const int band_rows = min(tiles_m - band * kBandM, kBandM);
  const int in_band = tile - band * band_tiles;
  const int tm = band * kBandM + in_band % band_rows;
  const int tn = in_band / band_rows;
  const int m0 = tm * BM;
  const int n0 = tn * BN;

  const int t = threadIdx.x;
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;
  const int wn = wave * 64;
  const int r = lane & 31;
  const int h = lane >> 5;

  f32x16 acc[8][2];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // this lane's two weight rows (columns of y); rows past N are clamped for
  // loads.  Lane half h starts 32 codes into the step; with GS == 32 that is
  // also one group further.  Byte offsets fit 32 bits (checked by the launcher).
  uint32_t woff[2], soff[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t n = (uint32_t)min(n0 + wn + 32 * j + r, N - 1);
    woff[j] = n * (uint32_t)(K * BITS / 8) + (uint32_t)(32 * h * BITS / 8);
    soff[j] = (n * (uint32_t)(K / GS) + (uint32_t)((32 * h) / GS)) * 2u;
  }
  // this thread's share of the x tile: 8 rows, one 16-byte column
  uint32_t xoff[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) xoff[i] = ((uint32_t)min(m0 + (t >> 3) + 32 * i, M - 1) * (uint32_t)K + 8u * (t & 7)) * 2u;
  const char* xbytes = reinterpret_cast<const char*>(x);
  // LDS addresses: the write slot of this thread (row t/8 of each 32-row block)
  // and, per k sub-step, the read slot of this lane (row r of each 32-row block)
  const int wr_slot = swz(t >> 3, t & 7);
  int rd_slot[4];
#pragma unroll
  for (int sub = 0; sub < 4; ++sub) rd_slot[sub] = swz(r, 4 * h + sub);

  u32x4 xa[8];
  auto issue_x = [&](int k0) {
    const char* base = xbytes + (size_t)k0 * 2;
#pragma unroll
    for (int i = 0; i < 8; ++i) xa[i] = *reinterpret_cast<const u32x4*>(base + xoff[i]);
  };
  auto commit_x = [&](char* tile_x) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(tile_x + wr_slot + 4096 * i) = xa[i];
  };

  const int steps = K / BK;
  WeightRegs<T, GS, BITS> wa, wb;

  // Dequantisation of one 8-code fragment, cut into 7 chunks of at most four
  // VALU instructions so that a chunk fits in the shadow of one matrix
  // instruction.  tmp/even/odd carry state between the chunks of a fragment.
  struct Dq {
    float tmp[8];
    uint32_t even, odd;
  };
  auto dq_chunk = [&](const WeightRegs<T, GS, BITS>& w, int j, int sub, int c, Dq& d, uint32_t (&out)[4]) {
    switch (c) {
      case 0:
        if constexpr (BITS == 4) {
          d.even = w.w[j][0][sub] & 0x0f0f0f0fu;
          d.odd = (w.w[j][0][sub] >> 4) & 0x0f0f0f0fu;
        }
        break;
      case 1:
        d.tmp[0] = w.deq(j, sub, 0, d.even, d.odd);
        d.tmp[1] = w.deq(j, sub, 1, d.even, d.odd);
        break;
      case 2:
        out[0] = T::pack2(d.tmp[0], d.tmp[1]);
        d.tmp[2] = w.deq(j, sub, 2, d.even, d.odd);
        break;
      case 3:
        d.tmp[3] = w.deq(j, sub, 3, d.even, d.odd);
        out[1] = T::pack2(d.tmp[2], d.tmp[3]);
        break;
      case 4:
        d.tmp[4] = w.deq(j, sub, 4, d.even, d.odd);
        d.tmp[5] = w.deq(j, sub, 5, d.even, d.odd);
        break;
      case 5:
        out[2] = T::pack2(d.tmp[4], d.tmp[5]);
        d.tmp[6] = w.deq(j, sub, 6, d.even, d.odd);
        break;
      case 6:
        d.tmp[7] = w.deq(j, sub, 7, d.even, d.odd);
        out[3] = T::pack2(d.tmp[6], d.tmp[7]);
        break;
      default:
        break;
    }
  };
  auto full_frag = [&](const WeightRegs<T, GS, BITS>& w, int j, uint32_t (&out)[4]) {
    Dq d;
#pragma unroll
    for (int c = 0; c < 7; ++c) dq_chunk(w, j, 0, c, d, out);
  };
  auto as_frag = [](const uint32_t (&v)[4]) {
    return __builtin_bit_cast(vec8, make_uint4(v[0], v[1], v[2], v[3]));
  };

  // One k step, written as 64 groups of (one matrix instruction + its fillers)
  // in the order they are to issue; a scheduling barrier after every group
  // keeps that order.  Fillers, per 16-instruction sub-step: the chunks of the
  // two fragments the NEXT sub-step needs, one LDS read of the next slot's x
  // fragments after every other matrix instruction, and
  //   sub-step 0: the global loads of the next step's x tile (one per group),
  //   sub-step 3: global loads of the weights of step+2 into `now` (whose
  //               contents were consumed during sub-step 2), then the LDS
  //               writes that publish the prefetched x tile.
  // bf carries the fragments of sub-step 0 in and those of the next step out.
  auto do_step = [&](auto parity, int step, WeightRegs<T, GS, BITS>& now, const WeightRegs<T, GS, BITS>& next,
                     uint32_t (&bf)[2][4]) {
    constexpr int kParity = decltype(parity)::value;  // == step & 1, known at compile time
    const char* xs = lds + kParity * kTileBytes;
    char* xd = lds + (kParity ^ 1) * kTileBytes;
    // branch-free prefetch: past the end the last step's operands are re-read and never consumed
    const int k_x = min(step + 1, steps - 1) * BK;
    const int k_w = min(step + 2, steps - 1) * BK;
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
          acc[ai][1] = mfma32(af[q & 1][i], b1, acc[ai][1]);
        } else {
          acc[ai][0] = mfma32(af[q & 1][i], b0, acc[ai][0]);
        }
        // fillers
        if (sub < 3) {
          dq_chunk(now, m >> 3, sub + 1, m & 7, dq, nb[m >> 3]);
        } else {
          dq_chunk(next, m >> 3, 0, m & 7, dq, nb[m >> 3]);
        }
        if ((m & 1) && q < 7) read_frag(q + 1, i);
        if (sub == 0 && m < 8) xa[m] = *reinterpret_cast<const u32x4*>(xbytes + (size_t)k_x * 2 + xoff[m]);
        if (sub == 3 && m == 0) now.issue(wq, scales, biases, woff, soff, k_w);
        if (sub == 3 && m >= 8) *reinterpret_cast<u32x4*>(xd + wr_slot + 4096 * (m - 8)) = xa[m - 8];
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

  issue_x(0);
  wa.issue(wq, scales, biases, woff, soff, 0);
  wb.issue(wq, scales, biases, woff, soff, min(1, steps - 1) * BK);
  commit_x(lds);
  uint32_t bf[2][4];
  full_frag(wa, 0, bf[0]);
  full_frag(wa, 1, bf[1]);
  __syncthreads();
  __builtin_amdgcn_sched_barrier(0);
  int step = 0;
  for (; step + 1 < steps; step += 2) {  // straight-line body: two steps with the weight registers swapped
    do_step(std::integral_constant<int, 0>{}, step, wa, wb, bf);
    do_step(std::integral_constant<int, 1>{}, step + 1, wb, wa, bf);
  }
  if (step < steps) do_step(std::integral_constant<int, 0>{}, step, wa, wb, bf);

  // Epilogue: register e of an accumulator is row 8*(e/4) + 4*h + e%4, column r.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = n0 + wn + 32 * j + r;
    if (col >= N) continue;
    const float bv = bias ? T::to_f32(bias[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + 32 * i + 8 * (e >> 2) + 4 * h + (e & 3);
        if (row >= M) continue;
        const int64_t o = (int64_t)row * N + col;
        const float v = acc[i][j][e];
        if (y_is_f32) {
          reinterpret_cast<float*>(y)[o] = bias ? v + bv : v;
        } else {
          uint16_t hv = T::from_f32(v);
          if (bias) hv = T::from_f32(T::to_f32(hv) + bv);
          reinterpret_cast<uint16_t*>(y)[o] = hv;
        }
      }
    }
  }
}

template <typename T, int GS, int BITS>
int launch_one(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
               const void* bias, int64_t N, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmm_kernel<T, GS, BITS>;
  static bool configured = false;  // raising the dynamic LDS limit is a per-function, per-process setting
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLdsBytes) != hipSuccess)
      return MFQ_ELAUNCH;
    configured = true;
  }
  // 32-bit byte offsets into x, the packed weight and the scales
  if (M * K >= (int64_t)1 << 31 || N * K >= (int64_t)1 << 31) return MFQ_EUNSUPPORTED;
  const int tiles_m = (int)((M + BM - 1) / BM);
  const int tiles_n = (int)((N + BN - 1) / BN);
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes, stream,
                     (const uint16_t*)x, wq, (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, tiles_m, tiles_n);
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

int launch_qmm(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               hipStream_t stream) {
  if (dtype == MFQ_BF16) return launch_gs<BF16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  if (dtype == MFQ_F16) return launch_gs<F16>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return MFQ_EDTYPE;
}

}  // namespace mfq
