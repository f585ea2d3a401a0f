// Driver of the host-sanitizer build of the C ABI's argument validation
// (python -m mflux_amd._build --sanitize-abi): abi.hip is compiled with
// AddressSanitizer and UndefinedBehaviorSanitizer on its host side, linked with
// the ordinary kernel objects, and every entry point is called with arguments it
// must refuse before anything is launched, so the run needs no GPU.  The
// pointers are real host allocations of 64 bytes: a validation path that read
// through one of them would be caught.  Exits non-zero on any unexpected status.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../include/mfq.h"

static int failures = 0;
static void expect(const char* what, int got, int want) {
  if (got != want) {
    std::fprintf(stderr, "abi_sanitize_check: %s returned %d (%s), expected %d\n", what, got, mfq_strerror(got), want);
    ++failures;
  }
}

int main() {
  void* raw = nullptr;
  if (posix_memalign(&raw, 16, 64)) return 2;
  char* p = static_cast<char*>(raw);
  uint32_t* u = static_cast<uint32_t*>(raw);
  for (int code = 1; code >= -12; --code)
    if (!mfq_strerror(code) || !std::strlen(mfq_strerror(code))) ++failures;
  if (mfq_version() <= 0) ++failures;

  expect("quantize: group", mfq_quantize_affine(p, MFQ_BF16, 4, 64, 48, 4, u, p, p, nullptr), MFQ_EGROUP);
  expect("quantize: bits", mfq_quantize_affine(p, MFQ_BF16, 4, 64, 64, 7, u, p, p, nullptr), MFQ_EBITS);
  expect("quantize: dtype", mfq_quantize_affine(p, 9, 4, 64, 64, 4, u, p, p, nullptr), MFQ_EDTYPE);
  expect("quantize: K", mfq_quantize_affine(p, MFQ_BF16, 4, 96, 64, 4, u, p, p, nullptr), MFQ_ESHAPE);
  expect("quantize: rows", mfq_quantize_affine(p, MFQ_BF16, 0, 64, 64, 4, u, p, p, nullptr), MFQ_ESHAPE);
  expect("quantize: null", mfq_quantize_affine(nullptr, MFQ_BF16, 4, 64, 64, 4, u, p, p, nullptr), MFQ_ENULL);
  expect("quantize: align", mfq_quantize_affine(p + 2, MFQ_BF16, 4, 64, 64, 4, u, p, p, nullptr), MFQ_EALIGN);

  expect("dequantize: bits", mfq_dequantize_affine(u, p, p, MFQ_BF16, 4, 64, 64, 2, p, MFQ_BF16, nullptr), MFQ_EBITS);
  expect("dequantize: null", mfq_dequantize_affine(u, p, nullptr, MFQ_BF16, 4, 64, 64, 4, p, MFQ_BF16, nullptr), MFQ_ENULL);
  expect("dequantize: dtype", mfq_dequantize_affine(u, p, p, 5, 4, 64, 64, 4, p, MFQ_BF16, nullptr), MFQ_EDTYPE);

  const int64_t* idx = reinterpret_cast<const int64_t*>(raw);
  expect("rows: null", mfq_dequantize_rows(u, p, p, MFQ_BF16, nullptr, 2, 10, 128, 64, 4, p, MFQ_BF16, nullptr), MFQ_ENULL);
  expect("rows: count", mfq_dequantize_rows(u, p, p, MFQ_BF16, idx, 0, 10, 128, 64, 4, p, MFQ_BF16, nullptr), MFQ_ESHAPE);
  expect("rows: K", mfq_dequantize_rows(u, p, p, MFQ_BF16, idx, 2, 10, 100, 64, 4, p, MFQ_BF16, nullptr), MFQ_ESHAPE);

  auto qmm = [&](const void* x, int xd, int64_t M, int64_t K, const uint32_t* wq, int sd, int64_t N, int gs, int bits,
                 void* y, int yd) { return mfq_qmm_t(x, xd, M, K, wq, p, p, sd, nullptr, N, gs, bits, y, yd, nullptr); };
  expect("qmm_t: f32 x", qmm(p, MFQ_F32, 4, 128, u, MFQ_BF16, 8, 64, 4, p, MFQ_BF16), MFQ_EDTYPE);
  expect("qmm_t: mixed", qmm(p, MFQ_BF16, 4, 128, u, MFQ_F16, 8, 64, 4, p, MFQ_BF16), MFQ_EDTYPE);
  expect("qmm_t: y type", qmm(p, MFQ_BF16, 4, 128, u, MFQ_BF16, 8, 64, 4, p, MFQ_F16), MFQ_EDTYPE);
  expect("qmm_t: K", qmm(p, MFQ_BF16, 4, 100, u, MFQ_BF16, 8, 64, 4, p, MFQ_BF16), MFQ_ESHAPE);
  expect("qmm_t: M", qmm(p, MFQ_BF16, 0, 128, u, MFQ_BF16, 8, 64, 4, p, MFQ_BF16), MFQ_ESHAPE);
  expect("qmm_t: N", qmm(p, MFQ_BF16, 4, 128, u, MFQ_BF16, (int64_t)1 << 40, 64, 4, p, MFQ_BF16), MFQ_ESHAPE);
  expect("qmm_t: null", qmm(p, MFQ_BF16, 4, 128, nullptr, MFQ_BF16, 8, 64, 4, p, MFQ_BF16), MFQ_ENULL);
  expect("qmm_t: align", qmm(p + 4, MFQ_BF16, 4, 128, u, MFQ_BF16, 8, 64, 4, p, MFQ_BF16), MFQ_EALIGN);
  expect("qmm_t: group", qmm(p, MFQ_BF16, 4, 128, u, MFQ_BF16, 8, 16, 4, p, MFQ_BF16), MFQ_EGROUP);
  expect("qmm_t: stream y", qmm(p, MFQ_BF16, 4, 128, u, MFQ_BF16, 8, 64, 5, p + 2, MFQ_BF16), MFQ_EALIGN);

  auto lr = [&](const void* t, const void* bs, int64_t rank) {
    return mfq_qmm_t_low_rank(p, MFQ_BF16, 4, 128, u, p, p, MFQ_BF16, nullptr, 8, 64, 4, t, bs, rank, p, MFQ_BF16,
                              nullptr, 0, nullptr);
  };
  expect("low_rank: rank 8", lr(p, p, 8), MFQ_ESHAPE);
  expect("low_rank: rank -16", lr(p, p, -16), MFQ_ESHAPE);
  expect("low_rank: rank 2048", lr(p, p, 2048), MFQ_ESHAPE);
  expect("low_rank: null", lr(nullptr, p, 16), MFQ_ENULL);
  expect("low_rank: align", lr(p, p + 2, 16), MFQ_EALIGN);

  expect("add: dtype", mfq_low_rank_add(p, p, MFQ_F32, 4, 8, 16, p, MFQ_F32, nullptr), MFQ_EDTYPE);
  expect("add: rank", mfq_low_rank_add(p, p, MFQ_BF16, 4, 8, 24, p, MFQ_BF16, nullptr), MFQ_ESHAPE);
  expect("add: null", mfq_low_rank_add(p, nullptr, MFQ_BF16, 4, 8, 16, p, MFQ_BF16, nullptr), MFQ_ENULL);

  auto qn = [&](int xd, int64_t N, int64_t K, int bits, void* y) {
    return mfq_qmm_n(p, xd, 4, N, u, p, p, MFQ_BF16, K, 64, bits, y, MFQ_BF16, nullptr);
  };
  expect("qmm_n: dtype", qn(MFQ_F32, 8, 128, 4, p), MFQ_EDTYPE);
  expect("qmm_n: K", qn(MFQ_BF16, 8, 100, 4, p), MFQ_ESHAPE);
  expect("qmm_n: bits", qn(MFQ_BF16, 8, 128, 7, p), MFQ_EBITS);
  expect("qmm_n: align", qn(MFQ_BF16, 8, 128, 4, p + 8), MFQ_EALIGN);
  expect("qmm_n: N % 8", qn(MFQ_BF16, 12, 128, 4, p), MFQ_EUNSUPPORTED);

  auto silu = [&](int xd, int64_t M, int64_t K, int64_t N, int bits) {
    return mfq_qmv_silu(p, xd, M, K, u, p, p, MFQ_BF16, nullptr, N, 64, bits, p, MFQ_BF16, nullptr);
  };
  expect("silu: dtype", silu(MFQ_F16, 1, 3072, 64, 8), MFQ_EDTYPE);
  expect("silu: bits", silu(MFQ_BF16, 1, 3072, 64, 5), MFQ_EUNSUPPORTED);
  expect("silu: long row", silu(MFQ_BF16, 1, 8192, 64, 8), MFQ_EUNSUPPORTED);
  expect("silu: rows", silu(MFQ_BF16, 5, 3072, 64, 8), MFQ_EUNSUPPORTED);
  expect("silu: M", silu(MFQ_BF16, 0, 3072, 64, 8), MFQ_ESHAPE);

  expect("static: group", mfq_qmm_t_static(p, MFQ_BF16, 4, 128, u, p, p, MFQ_BF16, nullptr, 8, 48, 4, p, MFQ_BF16, nullptr),
         MFQ_EGROUP);
  expect("static: K", mfq_qmm_t_static(p, MFQ_BF16, 40, 100, u, p, p, MFQ_BF16, nullptr, 8, 64, 4, p, MFQ_BF16, nullptr),
         MFQ_ESHAPE);
  if (mfq_qmm_t_workspace_bytes(0, 128, 8, 64, 4) != 0 || mfq_qmm_t_workspace_bytes(4, 100, 8, 64, 4) != 0) ++failures;

  expect("prepare: dtype", mfq_qmm_t_prepare(u, p, p, MFQ_F32, 64, 256, 64, 4, p, nullptr), MFQ_EDTYPE);
  expect("prepare: K", mfq_qmm_t_prepare(u, p, p, MFQ_BF16, 64, 250, 64, 4, p, nullptr), MFQ_ESHAPE);
  expect("prepare: null", mfq_qmm_t_prepare(u, p, nullptr, MFQ_BF16, 64, 256, 64, 4, p, nullptr), MFQ_ENULL);
  expect("prepare: K", mfq_qmm_t_prepare(u, p, p, MFQ_BF16, 64, 192, 64, 4, p, nullptr), MFQ_EUNSUPPORTED);
  expect("prepared: dtype", mfq_qmm_t_prepared(p, MFQ_F32, 4, 256, p, nullptr, 64, p, nullptr, 0, nullptr), MFQ_EDTYPE);
  expect("prepared: M", mfq_qmm_t_prepared(p, MFQ_BF16, 0, 256, p, nullptr, 64, p, nullptr, 0, nullptr), MFQ_ESHAPE);
  expect("prepared: null", mfq_qmm_t_prepared(p, MFQ_BF16, 4, 256, nullptr, nullptr, 64, p, nullptr, 0, nullptr), MFQ_ENULL);
  expect("prepared: K", mfq_qmm_t_prepared(p, MFQ_BF16, 4, 192, p, nullptr, 64, p, nullptr, 0, nullptr), MFQ_EUNSUPPORTED);
  if (mfq_qmm_t_prepared_bytes(64, 192, 4) != 0 || mfq_qmm_t_prepared_bytes(64, 256, 4) != 64 * 256 * 2) ++failures;
  if (mfq_qmm_t_prepared_workspace_bytes(0, 256, 64) != 0) ++failures;

  std::free(raw);
  if (failures) return 1;
  std::printf("abi_sanitize_check: every refusal clean\n");
  return 0;
}
