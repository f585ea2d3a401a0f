// Epilogue shared by the 128-column-tile GEMM kernels (qmm_mid.hip, qmm_n.hip):
// a wavefront's 64 x 64 block of float32 sums -> y, rounded, with the bias.
#pragma once

#include "common.h"
#include "epilogue.h"

namespace mfq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// acc[i][j], register e: output row mw + 32i + r, column nw + 32j + 8(e/4) + 4h + e%4
// (r = lane % 32, h = lane / 32).  y_item: the output matrix (M x N, row-major,
// 16-bit T or float32).  `lds` must be free (the k loop ended with a barrier):
// each wavefront transposes its block through a private region of it so that a
// global store instruction writes whole row segments.  bias: [N] or nullptr,
// added after the product has been rounded to T (two roundings, as a separate
// add on the 16-bit result would do).  epi (epilogue.h): applied to the 16-bit
// results on their way from the staging region to y (16-bit y with N % 8 == 0
// only: the launchers refuse an epilogue otherwise); for kEpiSwiglu y is [M, N/2].
template <typename T>
__device__ inline void store_block_64x64(const f32x16 (&acc)[2][2], char* lds, int wave, int lane, int mw, int nw, int M,
                                         int N, const uint16_t* __restrict__ bias, char* y_item, int y_is_f32,
                                         const Epilogue epi = Epilogue()) {
  const int r = lane & 31;
  const int h = lane >> 5;
  if (!y_is_f32 && (N & 7) == 0) {
    constexpr int kStride = 144;  // 64 16-bit columns + 16 bytes of padding
    char* stage = lds + wave * (64 * kStride);
    uint16_t* yout = reinterpret_cast<uint16_t*>(y_item);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        const int cl = 32 * j + 8 * eb + 4 * h;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
#pragma unroll
          for (int c = 0; c < 4; ++c) bv[c] = T::to_f32(bias[min(nw + cl + c, N - 1)]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          uint32_t pk[2];
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            pk[c] = T::pack2(acc[i][j][4 * eb + 2 * c], acc[i][j][4 * eb + 2 * c + 1]);
            if (bias)  // second rounding, as a separate add on the 16-bit result would do
              pk[c] = T::pack2(lo_f32<T>(pk[c]) + bv[2 * c], hi_f32<T>(pk[c]) + bv[2 * c + 1]);
          }
          *reinterpret_cast<uint2*>(stage + (32 * i + r) * kStride + cl * 2) = make_uint2(pk[0], pk[1]);
        }
      }
    }
    const int cg = nw + 8 * (lane & 7);
    if (epi.kind == kEpiSwiglu) {
      // the block's 64 columns are 32 of the gate projection, then their 32 of the up projection: lane l
      // takes 8 gate columns and the 8 up columns 32 further of row 16*k + l/4
      const int cq = lane & 3;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int rl = 16 * k + (lane >> 2);
        const u32x4 g = *reinterpret_cast<const u32x4*>(stage + rl * kStride + 16 * cq);
        const u32x4 u = *reinterpret_cast<const u32x4*>(stage + rl * kStride + 64 + 16 * cq);
        u32x4 v;
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = epi_swiglu_pair<T>(g[c], u[c]);
        const int row = mw + rl;
        if (row < M && nw < N) *reinterpret_cast<u32x4*>(yout + (int64_t)row * (N / 2) + (nw >> 1) + 8 * cq) = v;
      }
      return;
    }
    u32x4 gate8 = {0u, 0u, 0u, 0u};
    if (epi.kind == kEpiGateResidual && cg < N) gate8 = *reinterpret_cast<const u32x4*>(epi.gate + cg);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int rl = 8 * k + (lane >> 3);
      u32x4 v = *reinterpret_cast<const u32x4*>(stage + rl * kStride + 16 * (lane & 7));
      const int row = mw + rl;
      if (row < M && cg < N) {
        if (epi.kind == kEpiGelu && cg >= epi.act_from) {
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] = epi_gelu_pair<T>(v[c]);
        } else if (epi.kind == kEpiGateResidual) {
          const u32x4 res = *reinterpret_cast<const u32x4*>(epi.residual + (int64_t)row * N + cg);
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] = epi_gate_residual_pair<T>(v[c], gate8[c], res[c]);
        }
        *reinterpret_cast<u32x4*>(yout + (int64_t)row * N + cg) = v;
      }
    }
  } else if (y_is_f32 && (N & 3) == 0) {
    constexpr int kStride = 64 * 4 + 16;
    char* stage = lds + wave * (32 * kStride);
    float* yout = reinterpret_cast<float*>(y_item);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int eb = 0; eb < 4; ++eb) {
          const int cl = 32 * j + 8 * eb + 4 * h;
          float bv[4] = {0.f, 0.f, 0.f, 0.f};
          if (bias) {
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[c] = T::to_f32(bias[min(nw + cl + c, N - 1)]);
          }
          *reinterpret_cast<float4*>(stage + r * kStride + cl * 4) =
              make_float4(acc[i][j][4 * eb] + bv[0], acc[i][j][4 * eb + 1] + bv[1], acc[i][j][4 * eb + 2] + bv[2],
                          acc[i][j][4 * eb + 3] + bv[3]);
        }
      }
      const int cg = nw + 4 * (lane & 15);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int rl = 4 * k + (lane >> 4);
        const float4 v = *reinterpret_cast<const float4*>(stage + rl * kStride + 16 * (lane & 15));
        const int row = mw + 32 * i + rl;
        if (row < M && cg < N) *reinterpret_cast<float4*>(yout + (int64_t)row * N + cg) = v;
      }
    }
  } else {
    // any N: element-wise guarded stores straight from the accumulators
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int eb = 0; eb < 4; ++eb) {
        const int col = nw + 32 * j + 8 * eb + 4 * h;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int row = mw + 32 * i + r;
          if (row >= M) continue;
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            if (col + c >= N) continue;
            const float bv = bias ? T::to_f32(bias[col + c]) : 0.f;
            const int64_t o = (int64_t)row * N + col + c;
            if (y_is_f32) {
              reinterpret_cast<float*>(y_item)[o] = acc[i][j][4 * eb + c] + bv;
            } else {
              uint16_t hv = T::from_f32(acc[i][j][4 * eb + c]);
              if (bias) hv = T::from_f32(T::to_f32(hv) + bv);
              reinterpret_cast<uint16_t*>(y_item)[o] = hv;
            }
          }
        }
      }
    }
  }
}

}  // namespace mfq
