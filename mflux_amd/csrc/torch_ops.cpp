// torch.ops.mfq.*: the PyTorch-ROCm face of libmfq.  Each op checks its tensors,
// allocates the outputs from torch's caching allocator on the inputs' device,
// and calls the C ABI of include/mfq.h on torch's current HIP stream: no device
// synchronisation, no state of its own.  (PyTorch-ROCm presents its HIP devices
// under the "cuda" device type, hence the ...MasqueradingAsCUDA guard and the
// CUDA dispatch key.)  Only the HIP dispatch key is
// registered, so a CPU tensor is refused by the dispatcher (there is no CPU
// implementation to fall back to).  mflux_amd.core calls these ops; the error
// texts a user sees for bad arguments are produced there, in MLX's wording.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <tuple>

#include "../../include/mfq.h"

namespace {

using at::Tensor;

int dtype_code(at::ScalarType t, const char* what) {
  switch (t) {
    case at::kFloat: return MFQ_F32;
    case at::kHalf: return MFQ_F16;
    case at::kBFloat16: return MFQ_BF16;
    default: TORCH_CHECK(false, "mfq: ", what, " must be float32, float16 or bfloat16, got ", t);
  }
}

void check_status(const char* fn, int rc) {
  TORCH_CHECK(rc == MFQ_OK, fn, " failed: ", mfq_strerror(rc), " (status ", rc, ")");
}

void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

void check_packed(const Tensor& wq, const Tensor& scales, const Tensor& biases) {
  TORCH_CHECK(wq.scalar_type() == at::kUInt32, "mfq: the packed weight must be uint32, got ", wq.scalar_type());
  TORCH_CHECK(wq.dim() == 2 && scales.dim() == 2 && biases.dim() == 2, "mfq: packed weight, scales and biases are 2-D");
  TORCH_CHECK(scales.scalar_type() == biases.scalar_type() && scales.sizes() == biases.sizes(),
              "mfq: scales and biases must agree in dtype and shape");
  TORCH_CHECK(wq.is_contiguous() && scales.is_contiguous() && biases.is_contiguous(), "mfq: operands must be contiguous");
  TORCH_CHECK(scales.device() == wq.device() && biases.device() == wq.device(), "mfq: operands on different devices");
}

std::tuple<Tensor, Tensor, Tensor> quantize_affine(const Tensor& w, int64_t group_size, int64_t bits) {
  TORCH_CHECK(w.dim() == 2 && w.is_contiguous(), "mfq::quantize_affine: w must be a contiguous matrix");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(w.device());
  const int64_t rows = w.size(0), K = w.size(1);
  TORCH_CHECK(group_size > 0 && K % group_size == 0 && (K * bits) % 32 == 0, "mfq::quantize_affine: bad K");
  Tensor wq = at::empty({rows, K * bits / 32}, w.options().dtype(at::kUInt32));
  Tensor scales = at::empty({rows, K / group_size}, w.options());
  Tensor biases = at::empty_like(scales);
  if (rows == 0) return {wq, scales, biases};
  check_status("mfq_quantize_affine",
               mfq_quantize_affine(w.data_ptr(), dtype_code(w.scalar_type(), "w"), rows, K, (int)group_size, (int)bits,
                                   static_cast<uint32_t*>(wq.data_ptr()), scales.data_ptr(), biases.data_ptr(),
                                   stream_of(w)));
  return {wq, scales, biases};
}

Tensor dequantize_affine(const Tensor& wq, const Tensor& scales, const Tensor& biases, int64_t group_size, int64_t bits,
                         at::ScalarType out_dtype) {
  check_packed(wq, scales, biases);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(wq.device());
  const int64_t rows = wq.size(0), K = wq.size(1) * 32 / bits;
  Tensor out = at::empty({rows, K}, scales.options().dtype(out_dtype));
  if (rows == 0) return out;
  check_status("mfq_dequantize_affine",
               mfq_dequantize_affine(static_cast<const uint32_t*>(wq.data_ptr()), scales.data_ptr(), biases.data_ptr(),
                                     dtype_code(scales.scalar_type(), "scales"), rows, K, (int)group_size, (int)bits,
                                     out.data_ptr(), dtype_code(out_dtype, "the output"), stream_of(wq)));
  return out;
}

Tensor dequantize_rows(const Tensor& wq, const Tensor& scales, const Tensor& biases, const Tensor& indices,
                       int64_t group_size, int64_t bits, at::ScalarType out_dtype) {
  check_packed(wq, scales, biases);
  TORCH_CHECK(indices.scalar_type() == at::kLong && indices.dim() == 1 && indices.is_contiguous() &&
                  indices.device() == wq.device(),
              "mfq::dequantize_rows: indices must be a contiguous int64 vector on the table's device");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(wq.device());
  const int64_t K = wq.size(1) * 32 / bits;
  Tensor out = at::empty({indices.size(0), K}, scales.options().dtype(out_dtype));
  if (indices.size(0) == 0) return out;
  check_status("mfq_dequantize_rows",
               mfq_dequantize_rows(static_cast<const uint32_t*>(wq.data_ptr()), scales.data_ptr(), biases.data_ptr(),
                                   dtype_code(scales.scalar_type(), "scales"), indices.data_ptr<int64_t>(),
                                   indices.size(0), wq.size(0), K, (int)group_size, (int)bits, out.data_ptr(),
                                   dtype_code(out_dtype, "the output"), stream_of(wq)));
  return out;
}

struct Matmul {
  int64_t M, K, N;
  int sb;
  const void* bias;
};

// common checks of the products; x is [M, K] in the scales' dtype
Matmul check_matmul(const char* fn, const Tensor& x, const Tensor& wq, const Tensor& scales, const Tensor& biases,
                    const c10::optional<Tensor>& bias, int64_t bits) {
  check_packed(wq, scales, biases);
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && x.device() == wq.device(), fn, ": x must be a contiguous matrix on ",
              wq.device());
  TORCH_CHECK(x.scalar_type() == scales.scalar_type(), fn, ": x and scales must share a 16-bit dtype");
  Matmul m{x.size(0), wq.size(1) * 32 / bits, wq.size(0), dtype_code(scales.scalar_type(), "scales"), nullptr};
  TORCH_CHECK(x.size(1) == m.K, fn, ": x has ", x.size(1), " columns, the weight ", m.K);
  if (bias.has_value()) {
    TORCH_CHECK(bias->dim() == 1 && bias->size(0) == m.N && bias->scalar_type() == scales.scalar_type() &&
                    bias->is_contiguous() && bias->device() == wq.device(),
                fn, ": bias must be a contiguous [N] vector of the scales' dtype");
    m.bias = bias->data_ptr();
  }
  return m;
}

// y = x @ dequantize(wq)^T (+ t @ bs^T) (+ bias); the float32 planes of a K
// split come from torch's allocator on the current stream, so their reuse is
// ordered after this call.  `ok` is false (and y undefined) when the library
// has no kernel for the combination (MFQ_EUNSUPPORTED).
std::tuple<Tensor, bool> qmm_t(const Tensor& x, const Tensor& wq, const Tensor& scales, const Tensor& biases,
             const c10::optional<Tensor>& bias, int64_t group_size, int64_t bits, at::ScalarType out_dtype,
             const c10::optional<Tensor>& lr_t, const c10::optional<Tensor>& lr_bs) {
  const Matmul m = check_matmul("mfq::qmm_t", x, wq, scales, biases, bias, bits);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor y = at::empty({m.M, m.N}, x.options().dtype(out_dtype));
  if (m.M == 0) return {y, true};
  const void *t = nullptr, *bs = nullptr;
  int64_t rank = 0;
  if (lr_t.has_value() || lr_bs.has_value()) {
    TORCH_CHECK(lr_t.has_value() && lr_bs.has_value(), "mfq::qmm_t: the low-rank update needs both t and bs");
    rank = lr_bs->size(1);
    TORCH_CHECK(lr_t->dim() == 2 && lr_bs->dim() == 2 && lr_t->size(0) == m.M && lr_t->size(1) == rank &&
                    lr_bs->size(0) == m.N && lr_t->scalar_type() == x.scalar_type() &&
                    lr_bs->scalar_type() == x.scalar_type() && lr_t->is_contiguous() && lr_bs->is_contiguous(),
                "mfq::qmm_t: the low-rank update is t [M, R], bs [N, R], contiguous, in x's dtype");
    t = lr_t->data_ptr();
    bs = lr_bs->data_ptr();
  }
  const size_t ws_bytes = mfq_qmm_t_workspace_bytes(m.M, m.K, m.N, (int)group_size, (int)bits);
  Tensor ws;
  if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  const int rc = mfq_qmm_t_low_rank(x.data_ptr(), m.sb, m.M, m.K, static_cast<const uint32_t*>(wq.data_ptr()),
                                    scales.data_ptr(), biases.data_ptr(), m.sb, m.bias, m.N, (int)group_size, (int)bits,
                                    t, bs, rank, y.data_ptr(), dtype_code(out_dtype, "the output"),
                                    ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, stream_of(x));
  if (rc == MFQ_EUNSUPPORTED) return {y, false};
  check_status("mfq_qmm_t_low_rank", rc);
  return {y, true};
}

// qmm_t with an epilogue of include/mfq.h's mfq_qmm_t_epilogue (1: gelu_approx from column act_from on,
// 2: residual + gate * y, 3: SwiGLU of gate / up rows stacked in blocks of 32, y is [M, N/2]); `ok` is false
// (and y undefined) when no kernel fuses it for the shape
std::tuple<Tensor, bool> qmm_t_epilogue(const Tensor& x, const Tensor& wq, const Tensor& scales, const Tensor& biases,
                                        const c10::optional<Tensor>& bias, int64_t group_size, int64_t bits,
                                        int64_t epilogue, const c10::optional<Tensor>& gate,
                                        const c10::optional<Tensor>& residual, int64_t act_from) {
  const Matmul m = check_matmul("mfq::qmm_t_epilogue", x, wq, scales, biases, bias, bits);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  const void *gate_p = nullptr, *res_p = nullptr;
  if (epilogue == MFQ_EPILOGUE_GATE_RESIDUAL) {
    TORCH_CHECK(gate.has_value() && residual.has_value(), "mfq::qmm_t_epilogue: gate and residual are required");
    TORCH_CHECK(gate->dim() == 1 && gate->size(0) == m.N && gate->scalar_type() == x.scalar_type() &&
                    gate->is_contiguous() && gate->device() == x.device(),
                "mfq::qmm_t_epilogue: gate must be a contiguous [N] vector of x's dtype");
    TORCH_CHECK(residual->dim() == 2 && residual->size(0) == m.M && residual->size(1) == m.N &&
                    residual->scalar_type() == x.scalar_type() && residual->is_contiguous() &&
                    residual->device() == x.device(),
                "mfq::qmm_t_epilogue: residual must be a contiguous [M, N] matrix of x's dtype");
    gate_p = gate->data_ptr();
    res_p = residual->data_ptr();
  }
  const int64_t n_out = epilogue == MFQ_EPILOGUE_SWIGLU ? m.N / 2 : m.N;
  Tensor y = at::empty({m.M, n_out}, x.options());
  if (m.M == 0) return {y, true};
  const size_t ws_bytes = mfq_qmm_t_workspace_bytes(m.M, m.K, m.N, (int)group_size, (int)bits);
  Tensor ws;
  if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  const int rc = mfq_qmm_t_epilogue(x.data_ptr(), m.sb, m.M, m.K, static_cast<const uint32_t*>(wq.data_ptr()),
                                    scales.data_ptr(), biases.data_ptr(), m.sb, m.bias, m.N, (int)group_size,
                                    (int)bits, (int)epilogue, gate_p, res_p, act_from, y.data_ptr(), m.sb,
                                    ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, stream_of(x));
  if (rc == MFQ_EUNSUPPORTED) return {y, false};
  check_status("mfq_qmm_t_epilogue", rc);
  return {y, true};
}

// y[M, K] = x[M, N] @ dequantize(wq[N, K]); `ok` is false when N is not a multiple of 8
std::tuple<Tensor, bool> qmm_n(const Tensor& x, const Tensor& wq, const Tensor& scales, const Tensor& biases,
                               int64_t group_size, int64_t bits, at::ScalarType out_dtype) {
  check_packed(wq, scales, biases);
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && x.device() == wq.device() && x.size(1) == wq.size(0) &&
                  x.scalar_type() == scales.scalar_type(),
              "mfq::qmm_n: x must be a contiguous [M, N] matrix of the scales' dtype on the weight's device");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  const int64_t M = x.size(0), N = wq.size(0), K = wq.size(1) * 32 / bits;
  Tensor y = at::empty({M, K}, x.options().dtype(out_dtype));
  if (M == 0) return {y, true};
  const int sb = dtype_code(scales.scalar_type(), "scales");
  // the transposed 16-bit copy of the two-kernel path (and the planes of its K cut), where that is used
  const size_t ws_bytes = mfq_qmm_n_workspace_bytes(M, N, K, (int)group_size, (int)bits);
  Tensor ws;
  if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kByte));
  const int rc = mfq_qmm_n_ws(x.data_ptr(), sb, M, N, static_cast<const uint32_t*>(wq.data_ptr()), scales.data_ptr(),
                              biases.data_ptr(), sb, K, (int)group_size, (int)bits, y.data_ptr(),
                              dtype_code(out_dtype, "the output"), ws_bytes ? ws.data_ptr() : nullptr, ws_bytes,
                              stream_of(x));
  if (rc == MFQ_EUNSUPPORTED) return {y, false};
  check_status("mfq_qmm_n", rc);
  return {y, true};
}

// one to four rows of silu(x) against the weights in one kernel; `ok` is false
// (and y undefined) when no fused kernel takes the shape
std::tuple<Tensor, bool> qmv_silu(const Tensor& x, const Tensor& wq, const Tensor& scales, const Tensor& biases,
                                  const c10::optional<Tensor>& bias, int64_t group_size, int64_t bits) {
  const Matmul m = check_matmul("mfq::qmv_silu", x, wq, scales, biases, bias, bits);
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor y = at::empty({m.M, m.N}, x.options());
  const int rc = mfq_qmv_silu(x.data_ptr(), m.sb, m.M, m.K, static_cast<const uint32_t*>(wq.data_ptr()),
                              scales.data_ptr(), biases.data_ptr(), m.sb, m.bias, m.N, (int)group_size, (int)bits,
                              y.data_ptr(), m.sb, stream_of(x));
  if (rc == MFQ_EUNSUPPORTED) return {y, false};
  check_status("mfq_qmv_silu", rc);
  return {y, true};
}

// LayerNorm(x, eps) * (1 + scale) + shift over the rows of x [M, K]; scale and shift [B, K] with M % B == 0 (or
// neither); `ok` is false when the rows are too long for the kernel
std::tuple<Tensor, bool> layer_norm_modulate(const Tensor& x, const c10::optional<Tensor>& scale,
                                             const c10::optional<Tensor>& shift, double eps) {
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "mfq::layer_norm_modulate: x must be a contiguous matrix");
  TORCH_CHECK(scale.has_value() == shift.has_value(), "mfq::layer_norm_modulate: scale and shift come together");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  const int64_t M = x.size(0), K = x.size(1);
  int64_t rows_per_vector = M;
  const void *sc = nullptr, *sh = nullptr;
  if (scale.has_value()) {
    TORCH_CHECK(scale->dim() == 2 && scale->size(1) == K && scale->sizes() == shift->sizes() && scale->size(0) > 0 &&
                    M % scale->size(0) == 0 && scale->scalar_type() == x.scalar_type() &&
                    shift->scalar_type() == x.scalar_type() && scale->is_contiguous() && shift->is_contiguous() &&
                    scale->device() == x.device() && shift->device() == x.device(),
                "mfq::layer_norm_modulate: scale and shift must be contiguous [B, K] matrices of x's dtype, M % B == 0");
    rows_per_vector = M / scale->size(0);
    sc = scale->data_ptr();
    sh = shift->data_ptr();
  }
  Tensor y = at::empty_like(x);
  if (M == 0) return {y, true};
  const int rc = mfq_layer_norm_modulate(x.data_ptr(), dtype_code(x.scalar_type(), "x"), M, K, sc, sh, rows_per_vector,
                                         (float)eps, y.data_ptr(), stream_of(x));
  if (rc == MFQ_EUNSUPPORTED) return {y, false};
  check_status("mfq_layer_norm_modulate", rc);
  return {y, true};
}

// t = x @ A, A in the fragment order of mfq_low_rank_down ([R/16, K/32, 4, 16, 8])
Tensor low_rank_down(const Tensor& x, const Tensor& af) {
  TORCH_CHECK(x.dim() == 2 && af.dim() == 5 && x.is_contiguous() && af.is_contiguous() && af.size(2) == 4 &&
                  af.size(3) == 16 && af.size(4) == 8 && x.size(1) == 32 * af.size(1) &&
                  x.scalar_type() == af.scalar_type(),
              "mfq::low_rank_down: x [M, K], af [R/16, K/32, 4, 16, 8], contiguous, of one 16-bit type");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  const int64_t R = 16 * af.size(0);
  Tensor t = at::empty({x.size(0), R}, x.options());
  check_status("mfq_low_rank_down", mfq_low_rank_down(x.data_ptr(), af.data_ptr(), dtype_code(x.scalar_type(), "x"),
                                                      x.size(0), x.size(1), R, t.data_ptr(), stream_of(x)));
  return t;
}

// y += t @ bs^T in place
void low_rank_add_(Tensor& y, const Tensor& t, const Tensor& bs) {
  TORCH_CHECK(y.dim() == 2 && t.dim() == 2 && bs.dim() == 2 && y.is_contiguous() && t.is_contiguous() &&
                  bs.is_contiguous() && t.size(0) == y.size(0) && bs.size(0) == y.size(1) && t.size(1) == bs.size(1) &&
                  t.scalar_type() == bs.scalar_type(),
              "mfq::low_rank_add_: y [M, N], t [M, R], bs [N, R], contiguous");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  check_status("mfq_low_rank_add",
               mfq_low_rank_add(t.data_ptr(), bs.data_ptr(), dtype_code(t.scalar_type(), "t"), y.size(0), y.size(1),
                                t.size(1), y.data_ptr(), dtype_code(y.scalar_type(), "y"), stream_of(y)));
}

}  // namespace

TORCH_LIBRARY(mfq, m) {
  m.def("quantize_affine(Tensor w, int group_size, int bits) -> (Tensor, Tensor, Tensor)");
  m.def("dequantize_affine(Tensor wq, Tensor scales, Tensor biases, int group_size, int bits, ScalarType out_dtype) -> Tensor");
  m.def("dequantize_rows(Tensor wq, Tensor scales, Tensor biases, Tensor indices, int group_size, int bits, ScalarType out_dtype) -> Tensor");
  m.def("qmm_t(Tensor x, Tensor wq, Tensor scales, Tensor biases, Tensor? bias, int group_size, int bits, ScalarType out_dtype, Tensor? lr_t, Tensor? lr_bs) -> (Tensor, bool)");
  m.def("qmm_t_epilogue(Tensor x, Tensor wq, Tensor scales, Tensor biases, Tensor? bias, int group_size, int bits, int epilogue, Tensor? gate, Tensor? residual, int act_from) -> (Tensor, bool)");
  m.def("qmm_n(Tensor x, Tensor wq, Tensor scales, Tensor biases, int group_size, int bits, ScalarType out_dtype) -> (Tensor, bool)");
  m.def("qmv_silu(Tensor x, Tensor wq, Tensor scales, Tensor biases, Tensor? bias, int group_size, int bits) -> (Tensor, bool)");
  m.def("layer_norm_modulate(Tensor x, Tensor? scale, Tensor? shift, float eps) -> (Tensor, bool)");
  m.def("low_rank_add_(Tensor(a!) y, Tensor t, Tensor bs) -> ()");
  m.def("low_rank_down(Tensor x, Tensor af) -> Tensor");
}

TORCH_LIBRARY_IMPL(mfq, CUDA, m) {  // the HIP backend answers to torch's CUDA dispatch key
  m.impl("quantize_affine", quantize_affine);
  m.impl("dequantize_affine", dequantize_affine);
  m.impl("dequantize_rows", dequantize_rows);
  m.impl("qmm_t", qmm_t);
  m.impl("qmm_t_epilogue", qmm_t_epilogue);
  m.impl("qmm_n", qmm_n);
  m.impl("qmv_silu", qmv_silu);
  m.impl("layer_norm_modulate", layer_norm_modulate);
  m.impl("low_rank_add_", low_rank_add_);
  m.impl("low_rank_down", low_rank_down);
}
