// Shared device/host helpers for the mfq kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/mfq.h"

namespace mfq {

constexpr int kWave = 64;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Storage element tags.  `bits16` types travel as raw uint16_t in packed
// registers; conversions are explicit so that rounding points are visible.
struct BF16 {
  using storage = uint16_t;
  using vec8 = bf16x8;
  static constexpr int code = MFQ_BF16;
  __device__ static inline float to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
  // round to nearest even; the compiler selects v_cvt_pk_bf16_f32 for pairs
  __device__ static inline uint16_t from_f32(float f) {
    __bf16 b = (__bf16)f;
    return __builtin_bit_cast(uint16_t, b);
  }
  __device__ static inline uint32_t pack2(float lo, float hi) {
    bf16x2 v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
  }
};

struct F16 {
  using storage = uint16_t;
  using vec8 = f16x8;
  static constexpr int code = MFQ_F16;
  __device__ static inline float to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
  __device__ static inline uint16_t from_f32(float f) {
    _Float16 b = (_Float16)f;
    return __builtin_bit_cast(uint16_t, b);
  }
  __device__ static inline uint32_t pack2(float lo, float hi) {
    f16x2 v;
    v[0] = (_Float16)lo;
    v[1] = (_Float16)hi;
    return __builtin_bit_cast(uint32_t, v);
  }
};

// Matrix-core wrappers.  16x16x32: lane l holds row/col l%16 and the 8
// consecutive k values starting at 8*(l/16); the result holds rows
// 4*(l/16)+i (i = 0..3) of column l%16.  32x32x16: lane l holds row/col l%32
// and k values 8*(l/32)..+7; result register i is row 8*(i/4)+4*(l/32)+i%4 of
// column l%32.
__device__ inline f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ inline f32x4 mfma16(f16x8 a, f16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ inline f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ inline f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

struct F32 {
  using storage = float;
  static constexpr int code = MFQ_F32;
  __device__ static inline float to_f32(float f) { return f; }
  __device__ static inline float from_f32(float f) { return f; }
};

// low / high half of a packed pair of 16-bit elements
template <typename T>
__device__ inline float lo_f32(uint32_t p) { return T::to_f32((uint16_t)(p & 0xffffu)); }
template <typename T>
__device__ inline float hi_f32(uint32_t p) { return T::to_f32((uint16_t)(p >> 16)); }

// byte j of a word as float (selects v_cvt_f32_ubyte{j})
__device__ inline float ubyte_f32(uint32_t w, int j) { return (float)((w >> (8 * j)) & 0xffu); }

// Dequantise 8 consecutive codes into 8 packed 16-bit elements:
// value = fma(code, scale, bias) in float32, rounded once to T.
template <typename T>
__device__ inline uint4 dequant8_w4(uint32_t word, float s, float b) {
  const uint32_t even = word & 0x0f0f0f0fu;         // codes 0,2,4,6 in bytes 0..3
  const uint32_t odd = (word >> 4) & 0x0f0f0f0fu;   // codes 1,3,5,7
  uint4 r;
  r.x = T::pack2(__builtin_fmaf(ubyte_f32(even, 0), s, b), __builtin_fmaf(ubyte_f32(odd, 0), s, b));
  r.y = T::pack2(__builtin_fmaf(ubyte_f32(even, 1), s, b), __builtin_fmaf(ubyte_f32(odd, 1), s, b));
  r.z = T::pack2(__builtin_fmaf(ubyte_f32(even, 2), s, b), __builtin_fmaf(ubyte_f32(odd, 2), s, b));
  r.w = T::pack2(__builtin_fmaf(ubyte_f32(even, 3), s, b), __builtin_fmaf(ubyte_f32(odd, 3), s, b));
  return r;
}

template <typename T>
__device__ inline uint4 dequant8_w8(uint32_t w0, uint32_t w1, float s, float b) {
  uint4 r;
  r.x = T::pack2(__builtin_fmaf(ubyte_f32(w0, 0), s, b), __builtin_fmaf(ubyte_f32(w0, 1), s, b));
  r.y = T::pack2(__builtin_fmaf(ubyte_f32(w0, 2), s, b), __builtin_fmaf(ubyte_f32(w0, 3), s, b));
  r.z = T::pack2(__builtin_fmaf(ubyte_f32(w1, 0), s, b), __builtin_fmaf(ubyte_f32(w1, 1), s, b));
  r.w = T::pack2(__builtin_fmaf(ubyte_f32(w1, 2), s, b), __builtin_fmaf(ubyte_f32(w1, 3), s, b));
  return r;
}

// Code i of a little-endian bit stream of BITS-bit codes held in words w[0..];
// i is a compile-time constant after unrolling, so this is one bit-field
// extract, or one funnel shift and a mask where the code straddles two words.
template <int BITS>
__device__ inline uint32_t stream_code(const uint32_t* w, int i) {
  const int bit = i * BITS, word = bit / 32, sh = bit % 32;
  uint32_t c = w[word] >> sh;
  if (sh + BITS > 32) c |= w[word + 1] << (32 - sh);
  return c & ((1u << BITS) - 1u);
}

// codes 8c .. 8c+7 of a 32-code unit (BITS words) of MLX's 3-, 5- and 6-bit packs
template <typename T, int BITS>
__device__ inline uint4 dequant8_stream(const uint32_t* w, int c, float s, float b) {
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf((float)stream_code<BITS>(w, 8 * c + i), s, b);
  uint4 r;
  r.x = T::pack2(v[0], v[1]);
  r.y = T::pack2(v[2], v[3]);
  r.z = T::pack2(v[4], v[5]);
  r.w = T::pack2(v[6], v[7]);
  return r;
}

// Exact 16-bit float images of codes, two per register.
template <typename T>
struct CodeFloat;
template <>
struct CodeFloat<BF16> {
  static constexpr uint32_t kNibble = 0x43004300u;      // 128 + n, n < 128
  static constexpr uint32_t kHighMagic = 0x45004500u;   // 2048 + 16 n
  static constexpr bool kWholeByte = false;             // 8 significant bits: an 8-bit code goes in as two nibbles
  static constexpr float kOffset4 = 128.f, kOffset8 = 2048.f + 128.f;
  __device__ static inline f32x4 mfma4(uint2 a, uint2 b, f32x4 c) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
};
template <>
struct CodeFloat<F16> {
  static constexpr uint32_t kNibble = 0x64006400u;  // 1024 + n, n < 1024
  static constexpr uint32_t kHighMagic = 0;         // unused: a whole byte fits
  static constexpr bool kWholeByte = true;
  static constexpr float kOffset4 = 1024.f, kOffset8 = 1024.f;
  __device__ static inline f32x4 mfma4(uint2 a, uint2 b, f32x4 c) {
    typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
};

// ---- a row of 16-bit floats as 15-bit fixed point (the integer matvec kernels) --------------
// xq = rint(x * 2^e) with 2^e the power of two that brings the row's largest magnitude just
// under 2^14, split into a signed high and a signed low byte: xq = 256 * xh + xl.
// Magnitude bits of a 16-bit float: their integer order is the order of the magnitudes.
__device__ inline int mag_bits(uint32_t pair) { return (int)max(pair & 0x7fffu, (pair >> 16) & 0x7fffu); }

// 2^e as float32 for the exponent field E of the row's largest magnitude
// (|x| < 2^(E - bias + 1)), so that |x| * 2^e < 2^14; e is kept within what a
// normal float32 and its reciprocal can hold.
template <typename T>
__device__ inline int scale_exponent(int amax_bits);
template <>
__device__ inline int scale_exponent<BF16>(int amax_bits) {
  const int e = 14 - ((amax_bits >> 7) - 127 + 1);
  return min(max(e, -126), 126);
}
template <>
__device__ inline int scale_exponent<F16>(int amax_bits) {
  return 14 - ((amax_bits >> 10) - 15 + 1);  // -2 .. 28
}
template <typename T>
__device__ inline bool not_finite(int amax_bits);
template <>
__device__ inline bool not_finite<BF16>(int amax_bits) { return (amax_bits >> 7) == 255; }
template <>
__device__ inline bool not_finite<F16>(int amax_bits) { return (amax_bits >> 10) == 31; }

__device__ inline float pow2(int e) { return __builtin_bit_cast(float, (uint32_t)(127 + e) << 23); }

// four values of x -> their integer images, high bytes and low bytes packed in k order.
// xq = 256 * h + l with l the low byte read as signed, so h is the high byte of xq + 128;
// |xq| <= 2^14 fits the 16-bit halves the bytes are picked from.
template <typename T>
__device__ inline void split4(uint32_t p0, uint32_t p1, float mult, uint32_t& hi, uint32_t& lo) {
  typedef short s16x2 __attribute__((ext_vector_type(2)));
  const int q0 = (int)__builtin_rintf(lo_f32<T>(p0) * mult), q1 = (int)__builtin_rintf(hi_f32<T>(p0) * mult);
  const int q2 = (int)__builtin_rintf(lo_f32<T>(p1) * mult), q3 = (int)__builtin_rintf(hi_f32<T>(p1) * mult);
  const s16x2 q01 = __builtin_amdgcn_cvt_pk_i16(q0, q1), q23 = __builtin_amdgcn_cvt_pk_i16(q2, q3);
  const s16x2 half = {128, 128};
  const s16x2 t01 = q01 + half, t23 = q23 + half;
  // byte selectors: 0..3 name the bytes of the second operand, 4..7 those of the first
  lo = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, q23), __builtin_bit_cast(uint32_t, q01), 0x06040200u);
  hi = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, t23), __builtin_bit_cast(uint32_t, t01), 0x07050301u);
}

// SiLU of a pair of 16-bit floats as MLX's nn.silu computes it on that type,
// x * sigmoid(x) with the sigmoid rounded to the type before the product
// (src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12 feeds
// nn.silu(text_embeddings) to the modulation linear).
template <typename T>
__device__ inline uint32_t silu_pair(uint32_t pair) {
  uint32_t out = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float v = h ? hi_f32<T>(pair) : lo_f32<T>(pair);
    // hardware exponential and reciprocal (one ulp each, far inside the rounding to 16 bits that follows);
    // a denormal exponential flushed to 0 leaves the sigmoid at 1, an overflowing one makes it 0
    const float e = __builtin_amdgcn_exp2f(v * -1.44269504088896341f);
    const float sg = T::to_f32(T::from_f32(__builtin_amdgcn_rcpf(1.f + e)));
    out |= (uint32_t)T::from_f32(v * sg) << (16 * h);
  }
  return out;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launch parameters that depend on the device (compute units, resident
// workgroups of a kernel, "the LDS limit of this kernel has been raised") are
// cached per device: a process may drive several GPUs, each from its own
// threads.  A slot holds 0 until a thread has computed its value; two threads
// that race compute the same value and store it twice.  Nothing is cached for a
// device index outside the table.
constexpr int kMaxDevices = 64;

inline int device_index() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
  return dev;
}

struct PerDeviceInt {
  std::atomic<int> slot[kMaxDevices];

  // compute() returns the value (> 0) or a value <= 0 for "failed", which is
  // handed back and not kept.
  template <typename F>
  int get(F compute) {
    const int dev = device_index();
    if (dev < 0) return compute();
    int v = slot[dev].load(std::memory_order_acquire);
    if (v == 0) {
      v = compute();
      if (v > 0) slot[dev].store(v, std::memory_order_release);
    }
    return v;
  }
};

// Compute units of the current device (256 on an MI355X).
inline int compute_units() {
  static PerDeviceInt cache;
  const int n = cache.get([] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
    return prop.multiProcessorCount;
  });
  return n > 0 ? n : 256;
}

// Raises a kernel's dynamic LDS limit once per device; `done` is the launcher's
// own static cache (one per kernel instantiation).
inline bool raise_lds_limit(PerDeviceInt& done, const void* kernel, int bytes) {
  return done.get([&] {
           return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess ? 1 : -1;
         }) > 0;
}

// A low-rank update added to a product, y += t @ bs^T: t [M, R] holds the
// activations already multiplied by the LoRA down-projections, bs [N, R] the
// scaled up-projections, both row-major in the activation's 16-bit type, R a
// multiple of 16 (zero-padded).  R == 0: no update.
struct LowRank {
  const void* t = nullptr;
  const void* bs = nullptr;
  int R = 0;
};

// What a GEMM does to its 16-bit results on their way to y (the arithmetic is in epilogue.h).
enum EpilogueKind { kEpiNone = 0, kEpiGelu = 1, kEpiGateResidual = 2, kEpiSwiglu = 3 };

struct Epilogue {
  int kind = kEpiNone;
  const uint16_t* gate = nullptr;      // [N], 16-bit T
  const uint16_t* residual = nullptr;  // [M, N], 16-bit T
  int act_from = 0;                    // kEpiGelu: first column the activation applies to (a multiple of 8)
};

// Entry points of the individual translation units (host side).
int launch_quantize(const void* w, int dtype, int64_t rows, int64_t K, int gs, int bits, uint32_t* wq,
                    void* scales, void* biases, hipStream_t stream);
int launch_dequantize(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype, int64_t rows,
                      int64_t K, int gs, int bits, void* out, int out_dtype, hipStream_t stream);
int launch_dequantize_rows(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype,
                           const int64_t* idx, int64_t n_idx, int64_t n_rows, int64_t K, int gs, int bits, void* out,
                           int out_dtype, hipStream_t stream);
int launch_qmv(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               hipStream_t stream);
// one activation row on the vector pipeline's integer dot product (qmv_dot_covers() says whether it takes a shape)
bool qmv_dot_covers(int64_t M, int64_t K, int bits);
// `silu`: the row that meets the weights is silu(x), each value rounded to `dtype`
int launch_qmv_dot(const void* x, int dtype, int64_t K, const uint32_t* wq, const void* scales, const void* biases,
                   const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype, hipStream_t stream,
                   bool silu = false);
// 3-, 5- and 6-bit weights, one activation row; MFQ_EUNSUPPORTED for shapes it does not take
int launch_qmv_odd(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   hipStream_t stream);
// four weight rows at a time, M <= 4 (qmv_quad_covers() says whether it takes a shape)
bool qmv_quad_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* scales, const void* biases,
                     const void* bias, const void* y, int y_dtype);
// `silu`: the rows that meet the weights are silu(x), each value rounded to `dtype`
int launch_qmv_quad(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                    hipStream_t stream, bool silu = false);
// one to four activation rows, 8-bit codes: eight weight rows at a time on the int8 16x16x64 matrix
// instruction, K split over the eight wavefronts of a workgroup (qmv_oct_covers() says whether it takes a shape)
bool qmv_oct_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* x, const void* scales,
                    const void* biases);
int launch_qmv_oct(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   hipStream_t stream, bool silu = false);
// the same for 4-bit codes (qmv_oct4.hip)
bool qmv_oct4_covers(int64_t M, int64_t K, int64_t N, int gs, int bits, const void* x, const void* scales,
                     const void* biases);
int launch_qmv_oct4(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                    hipStream_t stream, bool silu = false);
// workspace: optional float32 scratch for the K-split of shapes with few output
// tiles (qmm_workspace_bytes() says how much; without it K is not split)
// low_rank: accumulated with the product by both GEMM kernels (a second kernel
// adds it after the matvec kernels)
int launch_qmm(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
               const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
               void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank = LowRank(),
               Epilogue epi = Epilogue());
// the instantiations of the same kernel with an epilogue (16-bit y, N % 8 == 0, period-wise scale loads;
// MFQ_EUNSUPPORTED otherwise)
int launch_qmm_epilogue(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                        const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                        void* workspace, size_t workspace_bytes, hipStream_t stream, Epilogue epi);
// y[M, N] += t @ bs^T, rounded to y's type (dtype: the type of t, bs and a 16-bit y)
int launch_low_rank_add(int dtype, LowRank low_rank, int64_t M, int64_t N, void* y, int y_dtype, hipStream_t stream);
// t[M, R] = x[M, K] @ A[K, R], A in fragment order ([R/16][K/32][4][16][8]); 16-bit type `dtype`; R % 16 == 0, K % 32 == 0
int launch_low_rank_down(const void* x, int dtype, int64_t M, int64_t K, const void* at, int64_t R, void* t,
                         hipStream_t stream);
// what a caller should bring (the K split's planes, or the scratch copy of the two-kernel path where that is
// preferred) and what the call cannot do without (the planes only)
size_t qmm_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs, int bits);
size_t qmm_min_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs);
// the two-kernel path (qmm_frag.hip): dequantize once into a 16-bit copy in fragment order, then a GEMM on
// 16x16x32 matrix instructions; 4 and 8 bits, 16-bit y of x's type, a low-rank update or an epilogue as
// launch_qmm / launch_qmm_epilogue.
// workspace (16-byte aligned): qmm_frag_copy_bytes(N, K) for the copy and, behind it, the float32 planes of a
// K cut (n_whole whole tiles, the others in `splits` ranges of whole pairs of k steps; splits == 1: no cut)
bool qmm_frag_shape_ok(int64_t M, int64_t N, int64_t K, int bits);
bool prefer_frag_path(int64_t M, int64_t N, int64_t K, int gs, int bits);  // where the two-kernel path is the faster
size_t qmm_frag_copy_bytes(int64_t N, int64_t K);
int launch_qmm_frag(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                    const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, void* workspace,
                    int n_whole, int splits, hipStream_t stream, LowRank low_rank, Epilogue epi);
// the same path for the weight not transposed, y[M, K] = x[M, N] @ dequantize(wq[N, K]): the copy holds W^T
// (qmm_frag_copy_bytes(K, N) of workspace, the planes of a K cut wherever `planes` points)
bool qmm_frag_n_shape_ok(int64_t M, int64_t N, int64_t K, int bits);
int launch_qmm_frag_n(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                      const void* biases, int64_t K, int gs, int bits, void* y, void* workspace, float* planes,
                      int n_whole, int splits, hipStream_t stream);
// y[M, K] = x[M, N] @ dequantize(wq[N, K]) with an optional workspace: with qmm_n_workspace_bytes() of it the
// two-kernel path takes the shapes it is the faster on, without it (or elsewhere) launch_qmm_n runs
size_t qmm_n_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs, int bits);
int launch_qmm_n_ws(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                    const void* biases, int64_t K, int gs, int bits, void* y, int y_dtype, void* workspace,
                    size_t workspace_bytes, hipStream_t stream);
// its two halves apart: the copy alone (weights that do not change between calls need it once), and the GEMM on a
// copy made before, with the planes of a K cut wherever the caller has room for them
int launch_qmm_frag_copy(int dtype, const uint32_t* wq, const void* scales, const void* biases, int64_t N, int64_t K,
                         int gs, int bits, void* copy, hipStream_t stream);
int launch_qmm_frag_gemm(const void* x, int dtype, int64_t M, int64_t K, const void* copy, const void* bias, int64_t N,
                         void* y, float* planes, int n_whole, int splits, hipStream_t stream, LowRank low_rank,
                         Epilogue epi);
// the GEMM on a prepared copy with the K cut planned here: `workspace` takes the planes (without room: whole tiles)
size_t qmm_prepared_workspace_bytes(int64_t M, int64_t N, int64_t K);
int launch_qmm_prepared(const void* x, int dtype, int64_t M, int64_t K, const void* copy, const void* bias, int64_t N,
                        void* y, void* workspace, size_t workspace_bytes, hipStream_t stream);
// y tiles = sums of the planes of a K cut (+ bias, epilogue): the second kernel of qmm.hip's and qmm_frag.hip's cut
int launch_tail_reduce(int dtype, const float* planes, int n_whole, int splits, int tiles_m, int tiles_n,
                       const void* bias, int64_t M, int64_t N, void* y, int y_dtype, hipStream_t stream, Epilogue epi);
// the 128-column-tile kernel for a few hundred activation rows, and for any M when K % 64 == 32
int launch_qmm_mid(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                   const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                   void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank = LowRank(),
                   Epilogue epi = Epilogue());
size_t qmm_mid_workspace_bytes(int64_t M, int64_t N, int64_t K, int gs);
// the same kernel for 3, 5 and 6 bits (any M above one row; K % 32 == 0)
int launch_qmm_mid_stream(const void* x, int dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                          const void* biases, const void* bias, int64_t N, int gs, int bits, void* y, int y_dtype,
                          void* workspace, size_t workspace_bytes, hipStream_t stream, LowRank low_rank = LowRank(),
                          Epilogue epi = Epilogue());
// y[M, K] = x[M, N] @ dequantize(wq[N, K]): the weight not transposed (N % 8 == 0)
int launch_qmm_n(const void* x, int dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                 const void* biases, int64_t K, int gs, int bits, void* y, int y_dtype, hipStream_t stream);
// y = LayerNorm(x, eps) (* (1 + scale) + shift): rows of up to 8192 16-bit elements, K % 8 == 0; scale and shift
// [M / rows_per_vector, K] or both nullptr
int launch_layer_norm_modulate(const void* x, int dtype, int64_t M, int64_t K, const void* scale, const void* shift,
                               int64_t rows_per_vector, float eps, void* y, hipStream_t stream);
// y = sum of `splits` float32 planes of M x N (+ bias), rounded to y's type; dtype is the type of bias and 16-bit y
int launch_splitk_reduce(int dtype, const void* planes, int splits, int64_t M, int64_t N, const void* bias, void* y,
                         int y_dtype, hipStream_t stream, Epilogue epi = Epilogue());

}  // namespace mfq
