// What mflux does to a quantized linear's output before it writes the next
// tensor, done where the GEMM kernels write y (one pass over [M, N] instead of
// two to five):
//   kEpiGelu          y = gelu_approx(linear(x)) for the columns from act_from on
//                     (src/mflux/models/flux/model/flux_transformer/
//                     single_transformer_block.py:53-54: nn.gelu_approx(proj_mlp(.));
//                     feed_forward.py:13-15 of the joint blocks);
//   kEpiGateResidual  y = residual + gate * linear(x), gate one value per output
//                     column (single_transformer_block.py:57 with :45;
//                     joint_transformer_block.py:84-90: hidden + gate * ff(.));
//   kEpiSwiglu        y[:, c] = silu(linear(x)[:, g(c)]) * linear(x)[:, u(c)] with
//                     the gate (w1) and up (w3) projections stacked in blocks of 32
//                     rows: g(c) = 64 (c / 32) + c % 32, u(c) = g(c) + 32
//                     (src/mflux/models/z_image/model/z_image_transformer/
//                     feed_forward.py:13: w2(silu(w1 x) * w3 x)); y is [M, N / 2].
// The linear's output (and its bias add) is rounded to the 16-bit type T as the
// reference's linear rounds it; behind that
//   gate/residual: the product gate * y is rounded, then the sum -- the two
//           element-wise operations of the reference, bit for bit;
//   swiglu: sigmoid, x * sigmoid (MLX's nn.silu is those two operations), then
//           the product with the up projection, each rounded;
//   gelu:   evaluated in float32 and rounded ONCE.  This is a deliberate
//           departure: MLX's nn.gelu_approx is a chain of some eight element-wise
//           operations whose 16-bit intermediates each round, which this does not
//           imitate (the chain's exact order inside MLX is not on record here, so
//           imitating it would pin nothing).  The result is the correctly rounded
//           value of the formula, a few units in the last place from what the
//           reference's chain gives.
#pragma once

#include "common.h"

namespace mfq {

// gelu_approx(v) = 0.5 v (1 + tanh(sqrt(2/pi) (v + 0.044715 v^3))) = v * sigmoid(2 sqrt(2/pi) (v + 0.044715 v^3)),
// in float32 with the hardware exponential and reciprocal (one ulp each, far inside the rounding to 16 bits).
__device__ inline float gelu_approx_f32(float v) {
  const float u = v * __builtin_fmaf(0.044715f * v, v, 1.0f);                      // v + 0.044715 v^3
  const float e = __builtin_amdgcn_exp2f(u * (-2.0f * 0.7978845608028654f * 1.4426950408889634f));  // exp(-2 sqrt(2/pi) u)
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

template <typename T>
__device__ inline float round_to(float v) { return T::to_f32(T::from_f32(v)); }

// one value each; `v`, `up`, `gate`, `res` are values of T held as float32; the result is rounded to T by the caller's store
template <typename T>
__device__ inline float epi_gelu(float v) { return gelu_approx_f32(v); }
template <typename T>
__device__ inline float epi_gate_residual(float v, float gate, float res) { return res + round_to<T>(gate * v); }
template <typename T>
__device__ inline float epi_swiglu(float v, float up) {
  const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896341f);
  const float sg = round_to<T>(__builtin_amdgcn_rcpf(1.f + e));
  return round_to<T>(v * sg) * up;
}

// the same on packed pairs of T
template <typename T>
__device__ inline uint32_t epi_gelu_pair(uint32_t pk) {
  return T::pack2(epi_gelu<T>(lo_f32<T>(pk)), epi_gelu<T>(hi_f32<T>(pk)));
}
template <typename T>
__device__ inline uint32_t epi_gate_residual_pair(uint32_t pk, uint32_t gate, uint32_t res) {
  return T::pack2(epi_gate_residual<T>(lo_f32<T>(pk), lo_f32<T>(gate), lo_f32<T>(res)),
                  epi_gate_residual<T>(hi_f32<T>(pk), hi_f32<T>(gate), hi_f32<T>(res)));
}
template <typename T>
__device__ inline uint32_t epi_swiglu_pair(uint32_t pk, uint32_t up) {
  return T::pack2(epi_swiglu<T>(lo_f32<T>(pk), lo_f32<T>(up)), epi_swiglu<T>(hi_f32<T>(pk), hi_f32<T>(up)));
}

}  // namespace mfq
