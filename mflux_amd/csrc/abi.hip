// C ABI of libmfq.so: argument validation and dispatch.  No kernel is
// launched unless every check has passed, so a caller's mistake is an error
// code and never a device fault.
#include "common.h"

namespace {

int check_common(int gs, int bits) {
  if (gs != 32 && gs != 64 && gs != 128) return MFQ_EGROUP;
  if (bits != 3 && bits != 4 && bits != 5 && bits != 6 && bits != 8) return MFQ_EBITS;
  return MFQ_OK;
}

bool is16(int dtype) { return dtype == MFQ_BF16 || dtype == MFQ_F16; }
bool known(int dtype) { return dtype == MFQ_F32 || is16(dtype); }

// The float32 planes of mfq_qmm_t_static's K split.  Every device the library
// runs on holds its own copy of this array, at its own address, until the
// process ends; the name below is only the host's handle for it, the address
// on the current device comes from hipGetSymbolAddress (scratch_on_device).
constexpr size_t kScratchBytes = MFQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
std::atomic<void*> scratch_ptr[mfq::kMaxDevices];

// Address of `scratch` on the current device, looked up once per device.
int scratch_on_device(void** out) {
  const int dev = mfq::device_index();
  if (dev < 0) return MFQ_ELAUNCH;
  void* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MFQ_ELAUNCH;
    scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return MFQ_OK;
}

}  // namespace

extern "C" {

int mfq_version(void) { return 100; }

const char* mfq_strerror(int status) {
  switch (status) {
    case MFQ_OK: return "ok";
    case MFQ_EDTYPE: return "unsupported dtype";
    case MFQ_EGROUP: return "group_size must be 32, 64 or 128";
    case MFQ_EBITS: return "bits must be 3, 4, 5, 6 or 8";
    case MFQ_ESHAPE: return "bad shape: sizes must be positive and K a multiple of group_size";
    case MFQ_ENULL: return "null pointer";
    case MFQ_EALIGN: return "buffers must be 16-byte aligned";
    case MFQ_ELAUNCH: return "HIP launch failed";
    case MFQ_EUNSUPPORTED: return "no kernel for this combination";
    case MFQ_ESCRATCH: return "the shape needs more scratch than the library's built-in buffer holds";
    default: return "unknown status";
  }
}

int mfq_quantize_affine(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int bits, uint32_t* wq,
                        void* scales, void* biases, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!known(dtype)) return MFQ_EDTYPE;
  if (rows <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (!w || !wq || !scales || !biases) return MFQ_ENULL;
  if (!mfq::aligned16(w) || !mfq::aligned16(wq)) return MFQ_EALIGN;
  return mfq::launch_quantize(w, dtype, rows, K, group_size, bits, wq, scales, biases, (hipStream_t)stream);
}

int mfq_dequantize_affine(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype, int64_t rows,
                          int64_t K, int group_size, int bits, void* out, int out_dtype, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!known(sb_dtype) || !known(out_dtype)) return MFQ_EDTYPE;
  if (rows <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (!wq || !scales || !biases || !out) return MFQ_ENULL;
  if (!mfq::aligned16(wq) || !mfq::aligned16(out)) return MFQ_EALIGN;
  return mfq::launch_dequantize(wq, scales, biases, sb_dtype, rows, K, group_size, bits, out, out_dtype,
                                (hipStream_t)stream);
}

int mfq_dequantize_rows(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype, const int64_t* indices,
                        int64_t n_indices, int64_t n_rows, int64_t K, int group_size, int bits, void* out,
                        int out_dtype, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!known(sb_dtype) || !known(out_dtype)) return MFQ_EDTYPE;
  if (n_indices <= 0 || n_rows <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (n_indices > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!wq || !scales || !biases || !indices || !out) return MFQ_ENULL;
  if (!mfq::aligned16(wq) || !mfq::aligned16(out)) return MFQ_EALIGN;
  return mfq::launch_dequantize_rows(wq, scales, biases, sb_dtype, indices, n_indices, n_rows, K, group_size, bits,
                                     out, out_dtype, (hipStream_t)stream);
}

size_t mfq_qmm_t_workspace_bytes(int64_t M, int64_t K, int64_t N, int group_size, int bits) {
  if (check_common(group_size, bits) != MFQ_OK) return 0;
  if (N <= 0 || K <= 0 || K % group_size || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
  if (bits != 4 && bits != 8) {
    if (M <= 1) return 0;
    if (mfq::prefer_frag_path(M, N, K, group_size, bits)) return mfq::qmm_workspace_bytes(M, N, K, group_size, bits);
    return mfq::qmm_mid_workspace_bytes(M, N, K, group_size);
  }
  if (M <= 16) return 0;
  return mfq::qmm_workspace_bytes(M, N, K, group_size, bits);
}

int mfq_qmm_t(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
              const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits, void* y,
              int y_dtype, void* stream) {
  return mfq_qmm_t_ws(x, x_dtype, M, K, wq, scales, biases, sb_dtype, bias, N, group_size, bits, y, y_dtype, nullptr, 0,
                      stream);
}

int mfq_qmm_t_ws(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                 const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits, void* y,
                 int y_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  return mfq_qmm_t_low_rank(x, x_dtype, M, K, wq, scales, biases, sb_dtype, bias, N, group_size, bits, nullptr, nullptr,
                            0, y, y_dtype, workspace, workspace_bytes, stream);
}

int mfq_qmm_t_static(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                     const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits, void* y,
                     int y_dtype, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  size_t need = mfq_qmm_t_workspace_bytes(M, K, N, group_size, bits);
  // a scratch copy of the weights that does not fit is done without (the fused kernel); the planes of a K split are not
  if (need > kScratchBytes && (bits == 4 || bits == 8) && M > 16) need = mfq::qmm_min_workspace_bytes(M, N, K, group_size);
  if (need > kScratchBytes) return MFQ_ESCRATCH;
  void* ws = nullptr;
  if (need) {
    if (int rc = scratch_on_device(&ws)) return rc;
  }
  return mfq_qmm_t_low_rank(x, x_dtype, M, K, wq, scales, biases, sb_dtype, bias, N, group_size, bits, nullptr, nullptr,
                            0, y, y_dtype, ws, need, stream);
}

size_t mfq_qmm_t_prepared_bytes(int64_t N, int64_t K, int bits) {
  if (N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || !mfq::qmm_frag_shape_ok(1, N, K, bits)) return 0;
  return mfq::qmm_frag_copy_bytes(N, K);
}

int mfq_qmm_t_prepare(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype, int64_t N, int64_t K,
                      int group_size, int bits, void* prepared, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!is16(sb_dtype)) return MFQ_EDTYPE;
  if (N <= 0 || K <= 0 || K % group_size || N > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!wq || !scales || !biases || !prepared) return MFQ_ENULL;
  if (!mfq::aligned16(wq) || !mfq::aligned16(prepared)) return MFQ_EALIGN;
  return mfq::launch_qmm_frag_copy(sb_dtype, wq, scales, biases, N, K, group_size, bits, prepared, (hipStream_t)stream);
}

size_t mfq_qmm_t_prepared_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
  if (!mfq::qmm_frag_shape_ok(M, N, K, 4)) return 0;
  return mfq::qmm_prepared_workspace_bytes(M, N, K);
}

int mfq_qmm_t_prepared(const void* x, int dtype, int64_t M, int64_t K, const void* prepared, const void* bias, int64_t N,
                       void* y, void* workspace, size_t workspace_bytes, void* stream) {
  if (!is16(dtype)) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0) return MFQ_ESHAPE;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!x || !prepared || !y) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(prepared) || !mfq::aligned16(y)) return MFQ_EALIGN;
  return mfq::launch_qmm_prepared(x, dtype, M, K, prepared, bias, N, y, workspace, workspace_bytes, (hipStream_t)stream);
}

int mfq_qmm_t_low_rank(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                       const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits,
                       const void* t, const void* bs, int64_t rank, void* y, int y_dtype, void* workspace,
                       size_t workspace_bytes, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (rank < 0 || rank > 1024 || rank % 16) return MFQ_ESHAPE;
  if (rank && (!t || !bs)) return MFQ_ENULL;
  if (rank && (!mfq::aligned16(t) || !mfq::aligned16(bs))) return MFQ_EALIGN;
  mfq::LowRank low_rank;
  if (rank) {
    low_rank.t = t;
    low_rank.bs = bs;
    low_rank.R = (int)rank;
  }
  const bool odd_bits = bits != 4 && bits != 8;
  if (!is16(x_dtype) || x_dtype != sb_dtype) return MFQ_EDTYPE;
  if (y_dtype != sb_dtype && y_dtype != MFQ_F32) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!x || !wq || !scales || !biases || !y) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(wq)) return MFQ_EALIGN;
  if (M > 16 && !mfq::aligned16(y)) return MFQ_EALIGN;  // the GEMM writes y in 16-byte pieces
  if (odd_bits) {
    // 3, 5, 6 bits: the one-row kernel for the rows it takes, the 128-column-tile GEMM for everything else
    if (M == 1) {
      const int rc = mfq::launch_qmv_odd(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                         (hipStream_t)stream);
      if (rc != MFQ_EUNSUPPORTED)
        return rc ? rc : mfq::launch_low_rank_add(x_dtype, low_rank, M, N, y, y_dtype, (hipStream_t)stream);
    }
    if (!mfq::aligned16(y)) return MFQ_EALIGN;
    // many rows and room for the scratch copy: the two-kernel path of the 4- and 8-bit weights
    if (M > 16 && K % 64 == 0 && y_dtype == x_dtype && workspace && mfq::aligned16(workspace) &&
        mfq::qmm_frag_shape_ok(M, N, K, bits) && workspace_bytes >= mfq::qmm_frag_copy_bytes(N, K) &&
        mfq::prefer_frag_path(M, N, K, group_size, bits))
      return mfq::launch_qmm(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype, workspace,
                             workspace_bytes, (hipStream_t)stream, low_rank);
    return mfq::launch_qmm_mid_stream(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                      workspace, workspace_bytes, (hipStream_t)stream, low_rank);
  }
  if (M <= 16) {
    const int rc = mfq::launch_qmv(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                   (hipStream_t)stream);
    return rc ? rc : mfq::launch_low_rank_add(x_dtype, low_rank, M, N, y, y_dtype, (hipStream_t)stream);
  }
  if (K % 64)  // group size 32 with K an odd multiple of it: the 128-column-tile GEMM pads the last k step with zeros
    return mfq::launch_qmm_mid(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype, nullptr, 0,
                               (hipStream_t)stream, low_rank);
  return mfq::launch_qmm(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype, workspace,
                         workspace_bytes, (hipStream_t)stream, low_rank);
}

int mfq_qmm_t_epilogue(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                       const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits,
                       int epilogue, const void* gate, const void* residual, int64_t act_from, void* y, int y_dtype,
                       void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (epilogue != MFQ_EPILOGUE_GELU && epilogue != MFQ_EPILOGUE_GATE_RESIDUAL && epilogue != MFQ_EPILOGUE_SWIGLU)
    return MFQ_ESHAPE;
  if (!is16(x_dtype) || x_dtype != sb_dtype || y_dtype != sb_dtype) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!x || !wq || !scales || !biases || !y) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(wq) || !mfq::aligned16(y)) return MFQ_EALIGN;
  mfq::Epilogue epi;
  epi.kind = epilogue;
  if (epilogue == MFQ_EPILOGUE_GELU) {
    if (act_from < 0 || act_from > N || act_from % 8) return MFQ_ESHAPE;
    epi.act_from = (int)act_from;
  } else if (epilogue == MFQ_EPILOGUE_GATE_RESIDUAL) {
    if (!gate || !residual) return MFQ_ENULL;
    if (!mfq::aligned16(gate) || !mfq::aligned16(residual)) return MFQ_EALIGN;
    epi.gate = static_cast<const uint16_t*>(gate);
    epi.residual = static_cast<const uint16_t*>(residual);
  } else if (N % 64) {
    return MFQ_ESHAPE;  // gate and up projections alternate in blocks of 32 rows
  }
  // the matvec kernels (M <= 16) have no epilogue, nor have rows that are not whole 16-byte pieces
  if (M <= 16 || N % 8) return MFQ_EUNSUPPORTED;
  if (bits != 4 && bits != 8)
    return mfq::launch_qmm_mid_stream(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                      workspace, workspace_bytes, (hipStream_t)stream, mfq::LowRank(), epi);
  if (K % 64)
    return mfq::launch_qmm_mid(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype, nullptr, 0,
                               (hipStream_t)stream, mfq::LowRank(), epi);
  return mfq::launch_qmm(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype, workspace,
                         workspace_bytes, (hipStream_t)stream, mfq::LowRank(), epi);
}

int mfq_qmm_n(const void* x, int x_dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
              const void* biases, int sb_dtype, int64_t K, int group_size, int bits, void* y, int y_dtype, void* stream) {
  return mfq_qmm_n_ws(x, x_dtype, M, N, wq, scales, biases, sb_dtype, K, group_size, bits, y, y_dtype, nullptr, 0, stream);
}

size_t mfq_qmm_n_workspace_bytes(int64_t M, int64_t N, int64_t K, int group_size, int bits) {
  if (check_common(group_size, bits) != MFQ_OK) return 0;
  if (M <= 0 || N <= 0 || K <= 0 || K % group_size || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
  return mfq::qmm_n_workspace_bytes(M, N, K, group_size, bits);
}

int mfq_qmm_n_ws(const void* x, int x_dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                 const void* biases, int sb_dtype, int64_t K, int group_size, int bits, void* y, int y_dtype,
                 void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!is16(x_dtype) || x_dtype != sb_dtype) return MFQ_EDTYPE;
  if (y_dtype != sb_dtype && y_dtype != MFQ_F32) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || N * (K * bits / 32) >= (int64_t)1 << 31) return MFQ_ESHAPE;
  if (!x || !wq || !scales || !biases || !y) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(wq) || !mfq::aligned16(y)) return MFQ_EALIGN;
  return mfq::launch_qmm_n_ws(x, x_dtype, M, N, wq, scales, biases, K, group_size, bits, y, y_dtype, workspace,
                              workspace_bytes, (hipStream_t)stream);
}

int mfq_qmv_silu(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq, const void* scales,
                 const void* biases, int sb_dtype, const void* bias, int64_t N, int group_size, int bits, void* y,
                 int y_dtype, void* stream) {
  if (int rc = check_common(group_size, bits)) return rc;
  if (!is16(x_dtype) || x_dtype != sb_dtype) return MFQ_EDTYPE;
  if (y_dtype != sb_dtype && y_dtype != MFQ_F32) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || K <= 0 || K % group_size) return MFQ_ESHAPE;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!x || !wq || !scales || !biases || !y) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(wq)) return MFQ_EALIGN;
  if (bits != 4 && bits != 8) return MFQ_EUNSUPPORTED;
#ifndef MFQ_NO_OCT
  if (mfq::qmv_oct_covers(M, K, N, group_size, bits, x, scales, biases))
    return mfq::launch_qmv_oct(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                               (hipStream_t)stream, true);
  if (mfq::qmv_oct4_covers(M, K, N, group_size, bits, x, scales, biases))
    return mfq::launch_qmv_oct4(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                (hipStream_t)stream, true);
#endif
  if (mfq::qmv_dot_covers(M, K, bits))
    return mfq::launch_qmv_dot(x, x_dtype, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                               (hipStream_t)stream, true);
  if (M >= 2 && M <= 4 && mfq::qmv_quad_covers(M, K, N, group_size, bits, scales, biases, bias, y, y_dtype))
    return mfq::launch_qmv_quad(x, x_dtype, M, K, wq, scales, biases, bias, N, group_size, bits, y, y_dtype,
                                (hipStream_t)stream, true);
  return MFQ_EUNSUPPORTED;
}

int mfq_layer_norm_modulate(const void* x, int dtype, int64_t M, int64_t K, const void* scale, const void* shift,
                            int64_t rows_per_vector, float eps, void* y, void* stream) {
  if (!is16(dtype)) return MFQ_EDTYPE;
  if (M <= 0 || K <= 0 || M > INT32_MAX || K > INT32_MAX) return MFQ_ESHAPE;
  if (!x || !y || (scale == nullptr) != (shift == nullptr)) return MFQ_ENULL;
  if (scale && (rows_per_vector <= 0 || M % rows_per_vector)) return MFQ_ESHAPE;
  if (!(eps >= 0.f)) return MFQ_ESHAPE;
  if (!mfq::aligned16(x) || !mfq::aligned16(y) || !mfq::aligned16(scale) || !mfq::aligned16(shift)) return MFQ_EALIGN;
  return mfq::launch_layer_norm_modulate(x, dtype, M, K, scale, shift, scale ? rows_per_vector : M, eps, y,
                                         (hipStream_t)stream);
}

int mfq_low_rank_down(const void* x, const void* at, int dtype, int64_t M, int64_t K, int64_t rank, void* t,
                      void* stream) {
  if (!is16(dtype)) return MFQ_EDTYPE;
  if (M <= 0 || K <= 0 || M > INT32_MAX || K > INT32_MAX || K % 32) return MFQ_ESHAPE;
  if (rank <= 0 || rank > 1024 || rank % 16) return MFQ_ESHAPE;
  if (M * K >= (int64_t)1 << 40) return MFQ_ESHAPE;
  if (!x || !at || !t) return MFQ_ENULL;
  if (!mfq::aligned16(x) || !mfq::aligned16(at) || !mfq::aligned16(t)) return MFQ_EALIGN;
  return mfq::launch_low_rank_down(x, dtype, M, K, at, rank, t, (hipStream_t)stream);
}

int mfq_low_rank_add(const void* t, const void* bs, int dtype, int64_t M, int64_t N, int64_t rank, void* y, int y_dtype,
                     void* stream) {
  if (!is16(dtype)) return MFQ_EDTYPE;
  if (y_dtype != dtype && y_dtype != MFQ_F32) return MFQ_EDTYPE;
  if (M <= 0 || N <= 0 || M > INT32_MAX || N > INT32_MAX) return MFQ_ESHAPE;
  if (rank <= 0 || rank > 1024 || rank % 16) return MFQ_ESHAPE;
  if (!t || !bs || !y) return MFQ_ENULL;
  if (!mfq::aligned16(t) || !mfq::aligned16(bs)) return MFQ_EALIGN;
  mfq::LowRank low_rank;
  low_rank.t = t;
  low_rank.bs = bs;
  low_rank.R = (int)rank;
  return mfq::launch_low_rank_add(dtype, low_rank, M, N, y, y_dtype, (hipStream_t)stream);
}

}  // extern "C"
