// Quantized matvec for one to four activation rows on gfx950, four weight rows
// at a time: y[0:M, n] = x[0:M] . dequant(W[n]) (+ bias), M <= 4.  The adaLN
// modulation shape of mflux's transformer blocks
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12).
//
// The 4x4x4 matrix-core instruction computes 16 independent 4x4 products: lane
// l belongs to block l/4 and holds row l%4 of the block's A (4 k values) and
// column l%4 of its B; register i of lane (b, j) receives element (i, j).  Here
// a wavefront works on four consecutive weight rows r0..r0+3: block b covers
// 16-byte piece 16*load + b of each row, lane (b, i) holds that piece of row
// r0+i as A and the matching slice of activation row i as B.  All 16 results of
// a block are useful: register i of lane (b, j) accumulates row r0+i against
// activation row j, so up to four activation rows cost what one does, and every
// load instruction reads 256 contiguous bytes of each of four adjacent rows.
//   - everything runs on integers, on the int8 form of the instruction: every
//     activation row becomes 15-bit fixed point, xq = rint(x * 2^e) with 2^e
//     the power of two that brings the row's largest magnitude just under 2^14
//     (rounding error 2^-15 of that magnitude per element), split into a signed
//     high and low byte; a word of 8-bit codes goes in as it is, as the signed
//     bytes code - 128 (one XOR), a word of 4-bit codes as its even and its odd
//     nibbles (three instructions), each against the high and the low bytes of
//     x.  Per 16-byte piece (a piece lies in one group) the int32 sums give
//     D = sum(xq * code) exactly, and scale * D + bias * sum(xq) is the piece's
//     contribution (the 128 of the 8-bit form joins the bias), scaled back by
//     2^-e of its activation row at the end.  No code is converted to floating
//     point and no weight is rounded.  (With 16-bit float operands a bfloat16
//     8-bit code had to enter as two nibbles: 7 vector and 2 matrix instructions
//     per word against 1 and 2 now; 3072 -> 18432 at M = 4: 16.6 -> 15.2 us.)
//     Scale and bias of row r0+i reach the other lanes of the block as DPP quad
//     broadcasts;
//   - the B operands (the bytes of xq in the order of the codes of a word,
//     high bytes and low bytes side by side) sit in LDS for the whole kernel,
//     one conflict-free 512-byte line per operand pair; the scales and biases of the next four rows are fetched with one
//     16-byte load per lane and staged through a wavefront-private LDS region;
//   - weight loads run kRing pieces ahead in a ring of registers, across row
//     quads; all of them are unconditional (past the end: the wavefront's last
//     quad again) so that waits can leave exactly the younger loads in flight;
//   - the 16 blocks' sums are added with two DPP row rotations and two
//     ds_bpermute exchanges per result register.
#include <type_traits>
#include <utility>

#include "common.h"

namespace mfq {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kDppRowRor4 = 0x124;
constexpr int kDppRowRor8 = 0x128;

template <int kCtrl>
__device__ inline float dpp_f32(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false));
}

template <typename F, int... kIs>
__device__ inline void for_each_index_impl(F&& f, std::integer_sequence<int, kIs...>) {
  (f(std::integral_constant<int, kIs>{}), ...);
}
template <int kN, typename F>
__device__ inline void for_each_index(F&& f) {
  for_each_index_impl(f, std::make_integer_sequence<int, kN>{});
}

constexpr int kScaleRegion = 1024;  // per wavefront and buffer: 512 bytes of scales, 512 of biases

// kLoads: 256-byte pieces per weight row (K * BITS / 8 / 256); kRing divides it.
template <typename T, int BITS, int kLoads, int kRing, bool kSilu>
__global__ __launch_bounds__(256, 4) void qmv_quad_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq,
                                                       const uint16_t* __restrict__ scales,
                                                       const uint16_t* __restrict__ biases,
                                                       const uint16_t* __restrict__ bias, void* __restrict__ y,
                                                       int y_is_f32, int M, int N, int K, int gs_shift,
                                                       int quads_per_wave) {
  constexpr int kCodes = 128 / BITS;  // codes in one 16-byte piece
  constexpr int kXOps = kCodes / 4;   // B operand pairs (high and low bytes of 4 values of x) per piece
  constexpr int kXBytes = kLoads * kXOps * 512;  // the B operands of one lane set
  static_assert(kLoads % kRing == 0, "ring slots must be known at compile time");
  extern __shared__ __attribute__((aligned(16))) char lds[];  // x operands, slice sums, 4 x 2 scale regions

  const int lane = threadIdx.x & (kWave - 1);
  // uniform over the wavefront, and known to be: quad addresses then live in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int blk = lane >> 2, li = lane & 3;
  const int row_bytes = kLoads * 256;
  const int groups = K >> gs_shift;

  // quads of rows are dealt to wavefronts in contiguous runs of equal length
  // (the host sizes the grid for that; only the last run can be short or empty)
  const int wave_id = blockIdx.x * (blockDim.x / kWave) + wave;
  const int q_begin = wave_id * quads_per_wave;
  const int q_end = min(q_begin + quads_per_wave, N / 4);
  const bool has_work = q_begin < q_end;

  char* sreg = lds + kXBytes + kLoads * 256 + wave * 2 * kScaleRegion;  // this wavefront's two scale regions
  const char* wbytes = reinterpret_cast<const char*>(wq);
  // this lane's byte offset inside a quad's weights: row li, piece blk
  const uint32_t lane_woff = (uint32_t)li * (uint32_t)row_bytes + (uint32_t)blk * 16u;
  // scale fetch: lanes 0..31 take 16 bytes of the quad's scales, lanes 32..63 of its biases
  const int quad_sb_bytes = 8 * groups;  // four rows of one array
  const char* sb_src = reinterpret_cast<const char*>(lane < 32 ? scales : biases);
  const int sb_off = (lane & 31) * 16;
  // lanes past the quad's block re-read its last 16 bytes (into a part of the region nobody reads): a
  // load behind a branch would make the number of loads in flight unknown to the waits that follow
  const int sb_off_load = min(sb_off, quad_sb_bytes - 16);
  // where this lane finds the scale of piece (j, blk) of row li inside a region
  const int piece_groups = (16 * kCodes) >> gs_shift;  // groups one load instruction spans
  const int sidx0 = (li * groups + ((blk * kCodes) >> gs_shift)) * 2;

  auto load_scales = [&](int q) __attribute__((always_inline)) {
    return *reinterpret_cast<const u32x4*>(sb_src + (size_t)q * quad_sb_bytes + sb_off_load);
  };
  auto store_scales = [&](u32x4 v, int buf) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4*>(sreg + buf * kScaleRegion + (lane >> 5) * 512 + sb_off) = v;
  };
  auto load_piece = [&](int q, int j) __attribute__((always_inline)) {
    return __builtin_nontemporal_load(
        reinterpret_cast<const u32x4*>(wbytes + (size_t)q * 4 * row_bytes + lane_woff + 256 * j));
  };

  // ---- x: the B operands and the slice sums of every lane position are
  // computed once per workgroup (the four wavefronts share the pieces out) and
  // kept in LDS.  All of this wavefront's loads of x are requested first and
  // in one go, the first weight pieces and the first quad's scales right
  // behind them: loads return in order, so x issued behind the weights, or
  // piece after piece, would wait for HBM once per piece before the first
  // quad can start.  Unconditional like every load here: a piece past the
  // row's end or an activation row past M re-reads a valid one and is dropped.
  constexpr int kMine = (kLoads + 3) / 4;  // pieces of x a wavefront stages
  constexpr int kRawWords = BITS == 4 ? 4 : 2;
  const int x_row = min(li, M - 1);
  uint32_t raw[kMine][4][kRawWords];
#pragma unroll
  for (int i = 0; i < kMine; ++i) {
    const int j = min(wave + 4 * i, kLoads - 1);
    const int k0 = (j * 16 + blk) * kCodes;
#pragma unroll
    for (int wd = 0; wd < 4; ++wd) {  // the piece's four words
      if constexpr (BITS == 4) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(x + (int64_t)x_row * K + k0 + 8 * wd);
#pragma unroll
        for (int e = 0; e < 4; ++e) raw[i][wd][e] = v[e];
      } else {
        const uint2 v = *reinterpret_cast<const uint2*>(x + (int64_t)x_row * K + k0 + 4 * wd);
        raw[i][wd][0] = v.x;
        raw[i][wd][1] = v.y;
      }
    }
  }
  u32x4 ring[kRing];
  const int q_first = has_work ? q_begin : 0;
#pragma unroll
  for (int j = 0; j < kRing; ++j) ring[j] = load_piece(q_first, j);
  const u32x4 sb_first = load_scales(q_first);

  if constexpr (kSilu) {  // the activation in front of the linear, on the values as they arrive
#pragma unroll
    for (int i = 0; i < kMine; ++i)
#pragma unroll
      for (int wd = 0; wd < 4; ++wd)
#pragma unroll
        for (int e = 0; e < kRawWords; ++e) raw[i][wd][e] = silu_pair<T>(raw[i][wd][e]);
  }

  // ---- the integer image of the activation rows: per row one power of two brings its largest
  // magnitude just under 2^14 (lanes with the same lane % 4 hold the same row)
  int amax = 0;
#pragma unroll
  for (int i = 0; i < kMine; ++i)
#pragma unroll
    for (int wd = 0; wd < 4; ++wd)
#pragma unroll
      for (int e = 0; e < kRawWords; ++e) amax = max(amax, mag_bits(raw[i][wd][e]));
  amax = max(amax, __builtin_amdgcn_update_dpp(0, amax, kDppRowRor4, 0xf, 0xf, false));
  amax = max(amax, __builtin_amdgcn_update_dpp(0, amax, kDppRowRor8, 0xf, 0xf, false));
  amax = max(amax, __builtin_amdgcn_ds_bpermute((lane ^ 16) * 4, amax));
  amax = max(amax, __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, amax));
  int* row_amax = reinterpret_cast<int*>(lds + kXBytes + kLoads * 256 + 4 * 2 * kScaleRegion);  // [4 wavefronts][4 rows]
  if (lane < 4) row_amax[wave * 4 + lane] = amax;
  __syncthreads();
  amax = max(max(row_amax[li], row_amax[4 + li]), max(row_amax[8 + li], row_amax[12 + li]));
  const int e2 = scale_exponent<T>(amax);
  const float mult = li < M ? pow2(e2) : 0.f;  // activation rows past M: zeros
  // an infinity or NaN anywhere in a row of x: every output of that row is NaN
  const float unscale = not_finite<T>(amax) ? __builtin_nanf("") : pow2(-e2);
#pragma unroll
  for (int i = 0; i < kMine; ++i) {
    const int j = wave + 4 * i;
    int sum_hi = 0, sum_lo = 0;
#pragma unroll
    for (int wd = 0; wd < 4; ++wd) {
      if constexpr (BITS == 4) {
        // a weight word holds codes c0..c7; its even nibbles, as bytes, are c0 c2 c4 c6, the odd ones c1 c3 c5 c7.
        // raw[..][q] = (x[2q], x[2q+1]): even k in the low halves
        const uint32_t ev0 = (raw[i][wd][0] & 0xffffu) | (raw[i][wd][1] << 16);
        const uint32_t ev1 = (raw[i][wd][2] & 0xffffu) | (raw[i][wd][3] << 16);
        const uint32_t od0 = (raw[i][wd][0] >> 16) | (raw[i][wd][1] & 0xffff0000u);
        const uint32_t od1 = (raw[i][wd][2] >> 16) | (raw[i][wd][3] & 0xffff0000u);
        uint32_t hi_e, lo_e, hi_o, lo_o;
        split4<T>(ev0, ev1, mult, hi_e, lo_e);
        split4<T>(od0, od1, mult, hi_o, lo_o);
        if (j < kLoads) {
          *reinterpret_cast<uint2*>(lds + ((j * kXOps + 2 * wd) * 64 + lane) * 8) = make_uint2(hi_e, lo_e);
          *reinterpret_cast<uint2*>(lds + ((j * kXOps + 2 * wd + 1) * 64 + lane) * 8) = make_uint2(hi_o, lo_o);
        }
        sum_hi = __builtin_amdgcn_sdot4((int)hi_e, 0x01010101, sum_hi, false);
        sum_hi = __builtin_amdgcn_sdot4((int)hi_o, 0x01010101, sum_hi, false);
        sum_lo = __builtin_amdgcn_sdot4((int)lo_e, 0x01010101, sum_lo, false);
        sum_lo = __builtin_amdgcn_sdot4((int)lo_o, 0x01010101, sum_lo, false);
      } else {
        // a weight word holds codes c0..c3 as its bytes
        uint32_t hi, lo;
        split4<T>(raw[i][wd][0], raw[i][wd][1], mult, hi, lo);
        if (j < kLoads) *reinterpret_cast<uint2*>(lds + ((j * kXOps + wd) * 64 + lane) * 8) = make_uint2(hi, lo);
        sum_hi = __builtin_amdgcn_sdot4((int)hi, 0x01010101, sum_hi, false);
        sum_lo = __builtin_amdgcn_sdot4((int)lo, 0x01010101, sum_lo, false);
      }
    }
    if (j < kLoads) *reinterpret_cast<float*>(lds + kXBytes + (j * 64 + lane) * 4) = (float)(sum_hi * 256 + sum_lo);
  }
  __syncthreads();
  float sx[kLoads];
#pragma unroll
  for (int j = 0; j < kLoads; ++j) sx[j] = *reinterpret_cast<const float*>(lds + kXBytes + (j * 64 + lane) * 4);
  const char* xops = lds + lane * 8;

  if (!has_work) return;
  store_scales(sb_first, q_begin & 1);

  for (int q = q_begin; q < q_end; ++q) {
    const int qn = min(q + 1, q_end - 1);  // past the end: this wavefront's last quad again, never consumed
    const u32x4 sb_next = load_scales(qn);
    // the quad's four bias values, requested now and unconditionally (without a bias: from the scales,
    // unused): fetched where they are needed, behind a branch, the wait for them would have to cover
    // every weight load in flight and drain the ring once per quad
    // The address is uniform and 8-byte aligned (the launcher checks), which makes this a scalar load
    // with a counter of its own.
    const uint2 bq2 = static_cast<const uint2*>(__builtin_assume_aligned(bias ? bias : scales, 8))[q];
    const uint16_t bq[4] = {(uint16_t)bq2.x, (uint16_t)(bq2.x >> 16), (uint16_t)bq2.y, (uint16_t)(bq2.y >> 16)};
    const char* sb = sreg + (q & 1) * kScaleRegion + sidx0;
    f32x4 tot = {0.f, 0.f, 0.f, 0.f};  // register i: row r0+i against this lane's activation row
    for_each_index<kLoads>([&](auto jc) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      constexpr int slot = j % kRing;
      const float sc = T::to_f32(*reinterpret_cast<const uint16_t*>(sb + j * piece_groups * 2));
      const float bi = T::to_f32(*reinterpret_cast<const uint16_t*>(sb + 512 + j * piece_groups * 2));
      // 8 bits: code = (code - 128) + 128, and the 128 joins the bias in front of the slice sum
      const float bo = BITS == 8 ? __builtin_fmaf(128.f, sc, bi) : bi;
      // exact integer sums of code * xq over the piece, against the high and the low bytes of xq:
      // two accumulation chains, so that a matrix instruction need not wait for the one before it
      i32x4 dh = {0, 0, 0, 0}, dl = {0, 0, 0, 0};
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {
        const uint32_t w = ring[slot][wd];
        if constexpr (BITS == 4) {
          const int ev = (int)(w & 0x0f0f0f0fu), od = (int)((w >> 4) & 0x0f0f0f0fu);
          const uint2 xe = *reinterpret_cast<const uint2*>(xops + (j * kXOps + 2 * wd) * 512);
          const uint2 xo = *reinterpret_cast<const uint2*>(xops + (j * kXOps + 2 * wd + 1) * 512);
          dh = __builtin_amdgcn_mfma_i32_4x4x4i8(ev, (int)xe.x, dh, 0, 0, 0);
          dl = __builtin_amdgcn_mfma_i32_4x4x4i8(ev, (int)xe.y, dl, 0, 0, 0);
          dh = __builtin_amdgcn_mfma_i32_4x4x4i8(od, (int)xo.x, dh, 0, 0, 0);
          dl = __builtin_amdgcn_mfma_i32_4x4x4i8(od, (int)xo.y, dl, 0, 0, 0);
        } else {
          const int c = (int)(w ^ 0x80808080u);  // code - 128 as signed bytes
          const uint2 xb = *reinterpret_cast<const uint2*>(xops + (j * kXOps + wd) * 512);
          dh = __builtin_amdgcn_mfma_i32_4x4x4i8(c, (int)xb.x, dh, 0, 0, 0);
          dl = __builtin_amdgcn_mfma_i32_4x4x4i8(c, (int)xb.y, dl, 0, 0, 0);
        }
      }
      float d[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) d[e] = (float)(dh[e] * 256 + dl[e]);
      // refill the slot: the piece kRing further on, in this quad or the next
      if constexpr (j + kRing < kLoads) {
        ring[slot] = load_piece(q, j + kRing);
      } else {
        ring[slot] = load_piece(qn, j + kRing - kLoads);
      }
      // keep the refills in place (left to itself the scheduler sinks the loads
      // behind several pieces of arithmetic and the ring runs dry), but let the
      // arithmetic of two pieces interleave
      if constexpr (j % 2 == 1 || j == kLoads - 1) __builtin_amdgcn_sched_barrier(0);
      // register i belongs to row r0+i, whose scale and bias lane i of the quad holds
      tot[0] = __builtin_fmaf(dpp_f32<0x00>(sc), d[0], tot[0]);
      tot[1] = __builtin_fmaf(dpp_f32<0x55>(sc), d[1], tot[1]);
      tot[2] = __builtin_fmaf(dpp_f32<0xAA>(sc), d[2], tot[2]);
      tot[3] = __builtin_fmaf(dpp_f32<0xFF>(sc), d[3], tot[3]);
      tot[0] = __builtin_fmaf(dpp_f32<0x00>(bo), sx[j], tot[0]);
      tot[1] = __builtin_fmaf(dpp_f32<0x55>(bo), sx[j], tot[1]);
      tot[2] = __builtin_fmaf(dpp_f32<0xAA>(bo), sx[j], tot[2]);
      tot[3] = __builtin_fmaf(dpp_f32<0xFF>(bo), sx[j], tot[3]);
    });
    // the other region was last read one quad ago
    store_scales(sb_next, (q + 1) & 1);

    // add up the 16 blocks: lanes with the same lane%4
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = tot[i];
      v += dpp_f32<kDppRowRor4>(v);
      v += dpp_f32<kDppRowRor8>(v);
      v += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 16) * 4, __builtin_bit_cast(int, v)));
      v += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) * 4, __builtin_bit_cast(int, v)));
      tot[i] = v * unscale;
    }
    if (lane < M) {  // lane m holds y[m, r0..r0+3]
      const int64_t r0 = (int64_t)q * 4;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bv[i] = T::to_f32(bq[i]);
      }
      const int64_t o = (int64_t)lane * N + r0;
      if (y_is_f32) {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(y) + o) =
            make_float4(tot[0] + bv[0], tot[1] + bv[1], tot[2] + bv[2], tot[3] + bv[3]);
      } else {
        uint32_t pk[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          pk[c] = T::pack2(tot[2 * c], tot[2 * c + 1]);
          if (bias)  // second rounding, as a separate add on the 16-bit result would do
            pk[c] = T::pack2(T::to_f32((uint16_t)pk[c]) + bv[2 * c], T::to_f32((uint16_t)(pk[c] >> 16)) + bv[2 * c + 1]);
        }
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(y) + o) = make_uint2(pk[0], pk[1]);
      }
    }
  }
}

template <typename T, int BITS, int kLoads, int kRing, bool kSilu>
int launch_kernel(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                  const void* bias, int64_t N, int gs_shift, void* y, int y_dtype, hipStream_t stream) {
  auto kernel = qmv_quad_kernel<T, BITS, kLoads, kRing, kSilu>;
  constexpr int kXOps = 128 / BITS / 4;
  constexpr int kLds = kLoads * kXOps * 512 + kLoads * 256 + 4 * 2 * kScaleRegion + 64;  // + the rows' largest magnitudes
  static PerDeviceInt cache;
  const int blocks_per_cu = cache.get([&] {
    if (kLds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds) !=
            hipSuccess)
      return -1;
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, kLds) != hipSuccess || n < 1) n = 1;
    // two workgroups per compute unit: every workgroup stages x for itself, and more of them measured
    // slower (3072 -> 18432 at M = 4: 17.8 us with two, 19.0 us with three or four)
    return n > 2 ? 2 : n;
  });
  if (blocks_per_cu < 1) return MFQ_ELAUNCH;
  // At most that many wavefronts, and every one of them the same number of
  // quads: with 4608 quads, 1536 wavefronts of three finish together, whereas
  // 2048 wavefronts would leave 512 of them a third quad.
  const int64_t quads = N / 4;
  const int64_t max_waves = (int64_t)compute_units() * blocks_per_cu * 4;
  const int64_t per_wave = (quads + max_waves - 1) / max_waves;
  const int64_t n_waves = (quads + per_wave - 1) / per_wave;
  const int64_t blocks = (n_waves + 3) / 4;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), kLds, stream, (const uint16_t*)x, wq,
                     (const uint16_t*)scales, (const uint16_t*)biases, (const uint16_t*)bias, y,
                     (int)(y_dtype == MFQ_F32), (int)M, (int)N, (int)K, gs_shift, (int)per_wave);
  return hipGetLastError() == hipSuccess ? MFQ_OK : MFQ_ELAUNCH;
}

template <typename T, int BITS, bool kSilu>
int launch_loads(int64_t loads, const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                 const void* biases, const void* bias, int64_t N, int gs_shift, void* y, int y_dtype,
                 hipStream_t stream) {
#define MFQ_QUAD_CASE(L, R)                                                                                      \
  case L:                                                                                                        \
    return launch_kernel<T, BITS, L, R, kSilu>(x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream)
  switch (loads) {
    MFQ_QUAD_CASE(1, 1);
    MFQ_QUAD_CASE(2, 2);
    MFQ_QUAD_CASE(3, 3);
    MFQ_QUAD_CASE(4, 4);
    MFQ_QUAD_CASE(6, 6);
    MFQ_QUAD_CASE(8, 4);
    MFQ_QUAD_CASE(12, 6);
    MFQ_QUAD_CASE(16, 4);
    default:
      return MFQ_EUNSUPPORTED;
  }
#undef MFQ_QUAD_CASE
}

}  // namespace

// Shapes this kernel takes: M <= 4; whole quads of rows; rows that are a
// supported number of 256-byte pieces; at most 64 groups per row, an even
// number (the staged scale block of a quad is 16-byte pieces of at most 512
// bytes); K <= 4096 (the x operands' LDS copy); pointers aligned for the
// 16-byte scale fetches and the 8- / 16-byte stores.
bool qmv_quad_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* scales, const void* biases,
                     const void* bias, const void* y, int y_dtype) {
  if (reinterpret_cast<uintptr_t>(bias) & 7u) return false;  // four bias values travel as one 8-byte load
  const int64_t row_bytes = K * bits / 8;
  const int64_t loads = row_bytes / 256;
  const int64_t groups = K / gs;
  const bool loads_ok = row_bytes % 256 == 0 && (loads == 1 || loads == 2 || loads == 3 || loads == 4 || loads == 6 ||
                                                 loads == 8 || loads == 12 || loads == 16);
  const uintptr_t y_mask = y_dtype == MFQ_F32 ? 15u : 7u;
  return M >= 1 && M <= 4 && N % 4 == 0 && loads_ok && groups <= 64 && groups % 2 == 0 && K <= 4096 &&
         aligned16(scales) && aligned16(biases) && (reinterpret_cast<uintptr_t>(y) & y_mask) == 0;
}

namespace {
template <typename T, bool kSilu>
int launch_type(const void* x, int64_t M, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream) {
  const int gs_shift = gs == 32 ? 5 : gs == 64 ? 6 : 7;
  const int64_t loads = K * bits / 8 / 256;
  if (bits == 4)
    return launch_loads<T, 4, kSilu>(loads, x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
  return launch_loads<T, 8, kSilu>(loads, x, M, K, wq, scales, biases, bias, N, gs_shift, y, y_dtype, stream);
}
}  // namespace

int launch_qmv_quad(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                    hipStream_t stream, bool silu) {
  if (dtype != MFQ_BF16 && dtype != MFQ_F16) return MFQ_EDTYPE;
  const bool bf = dtype == MFQ_BF16;
  if (silu)
    return bf ? launch_type<BF16, true>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream)
              : launch_type<F16, true>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
  return bf ? launch_type<BF16, false>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream)
            : launch_type<F16, false>(x, M, K, wq, scales, biases, bias, N, gs, bits, y, y_dtype, stream);
}

}  // namespace mfq
