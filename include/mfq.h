/*
 * mfq -- group-wise affine quantization and quantized matmul for one
 * MI355X (gfx950).  C ABI of libmfq.so.
 *
 * This is the boundary a host runtime binds to replace the three MLX
 * operations mflux's quantized-linear path lands in.  mflux has no FFI of its
 * own for this path: it calls mlx.nn.quantize and then invokes the resulting
 * QuantizedLinear modules, so each entry point below cites the reference call
 * site(s) whose work it performs.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer on the current HIP device, row-major
 *     and densely packed; the caller owns all buffers;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     all calls are asynchronous on it and perform no allocation other than
 *     where stated;
 *   - dtype codes are MFQ_F32 / MFQ_F16 / MFQ_BF16;
 *   - the return value is MFQ_OK (0) or a negative MFQ_E* code; nothing is
 *     thrown across the boundary and nothing is launched when an error is
 *     returned.  mfq_strerror() names a code.
 *   - packed layout (identical to MLX's): a row's codes form one little-endian
 *     bit stream, element i in bits [i*bits, (i+1)*bits).  For 4 and 8 bits
 *     that is the field at bit offset (i % (32/bits)) * bits of the uint32
 *     word i / (32/bits); for 3, 5 and 6 bits it is MLX's 3- and 5-byte packs
 *     laid end to end.  scales and biases hold one value per `group_size`
 *     consecutive elements of a row.
 *   - bits: 3, 4, 5, 6, 8 everywhere.
 */
#ifndef MFQ_H
#define MFQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum mfq_dtype { MFQ_F32 = 0, MFQ_F16 = 1, MFQ_BF16 = 2 };

enum mfq_status {
  MFQ_OK = 0,
  MFQ_EDTYPE = -1,     /* unknown or unsupported dtype code                  */
  MFQ_EGROUP = -2,     /* group_size not in {32, 64, 128}                    */
  MFQ_EBITS = -3,      /* bits not in {3, 4, 5, 6, 8}                        */
  MFQ_ESHAPE = -4,     /* K not a multiple of group_size, or a size <= 0     */
  MFQ_ENULL = -5,      /* a required pointer is NULL                         */
  MFQ_EALIGN = -6,     /* a buffer is not 16-byte aligned                    */
  MFQ_ELAUNCH = -7,    /* the HIP runtime refused the launch                 */
  MFQ_EUNSUPPORTED = -8, /* valid request that this build has no kernel for  */
  MFQ_ESCRATCH = -9     /* mfq_qmm_t_static: the shape's K split needs more
                           than MFQ_STATIC_SCRATCH_BYTES                      */
};

/* Library version: major*10000 + minor*100 + patch. */
int mfq_version(void);

/* Static, never-NULL description of a status code. */
const char* mfq_strerror(int status);

/*
 * Quantize `rows` rows of K elements each.
 * Replaces mx.quantize(w, group_size, bits, mode="affine") as reached from
 * nn.quantize at src/mflux/models/common/weights/loading/
 * weight_applier.py:43,46,103 (Linear.to_quantized -> QuantizedLinear.
 * from_linear).  Results are bit-identical to oracle/mlx_affine.c, a
 * restatement of MLX's CPU algorithm (quantize<T,U>); parity with MLX itself
 * is unpinned: MLX cannot be run where this library is built and the
 * reference holds no vector for this function.
 *   w       [rows, K]              dtype
 *   wq      [rows, K*bits/32]      uint32
 *   scales  [rows, K/group_size]   dtype
 *   biases  [rows, K/group_size]   dtype
 */
int mfq_quantize_affine(const void* w, int dtype, int64_t rows, int64_t K,
                        int group_size, int bits, uint32_t* wq, void* scales,
                        void* biases, void* stream);

/*
 * Inverse mapping w = code*scale + bias, written in `out_dtype`.
 * Replaces mx.dequantize; mflux needs it where a LoRA is baked into a
 * quantized base (src/mflux/models/common/lora/mapping/lora_saver.py:59-82).
 * mx.dequantize is an element-wise multiply followed by an element-wise add
 * on arrays of the output type: the product code * scale is rounded to
 * out_dtype, then the sum with the bias is rounded to out_dtype (for float32
 * output from 16-bit scales both steps are exact up to the one final
 * rounding).  Bit-identical to mlxo_dequantize of oracle/mlx_affine.c; parity
 * with MLX itself is unpinned.
 */
int mfq_dequantize_affine(const uint32_t* wq, const void* scales,
                          const void* biases, int sb_dtype, int64_t rows,
                          int64_t K, int group_size, int bits, void* out,
                          int out_dtype, void* stream);

/*
 * out[i, :] = dequantize(row indices[i] of the packed matrix): the lookup of a
 * quantized embedding table.  Replaces
 *   mx.dequantize(weight[x], scales[x], biases[x], group_size, bits)
 * of MLX's QuantizedEmbedding.__call__, which is what nn.quantize with the
 * default predicate (src/mflux/models/common/weights/loading/
 * weight_applier.py:30-31) turns every nn.Embedding into, e.g.
 * src/mflux/models/flux/model/flux_text_encoder/t5_encoder/t5_encoder.py:11.
 *   wq      [n_rows, K*bits/32]    uint32
 *   scales, biases [n_rows, K/group_size]   sb_dtype
 *   indices [n_indices]            int64 (device); negative values count from
 *                                  the end; values outside the table are
 *                                  clamped to its first / last row
 *   out     [n_indices, K]         out_dtype (sb_dtype or MFQ_F32)
 */
int mfq_dequantize_rows(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype,
                        const int64_t* indices, int64_t n_indices, int64_t n_rows, int64_t K,
                        int group_size, int bits, void* out, int out_dtype, void* stream);

/*
 * y[m, n] = sum_k x[m, k] * (scales[n, k/gs] * code[n, k] + biases[n, k/gs])
 *           (+ bias[n], added after y has been rounded to y_dtype, which is
 *           what QuantizedLinear.__call__ does with its second op).
 * Replaces mx.quantized_matmul(x, w, scales, biases, transpose=True, ...) plus
 * the bias add of every quantized nn.Linear call, e.g.
 *   src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53,57
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12
 *   src/mflux/models/z_image/model/z_image_transformer/feed_forward.py:13
 *   src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37
 *   x       [M, K]                 x_dtype (MFQ_BF16 or MFQ_F16; must equal sb_dtype)
 *   wq      [N, K*bits/32]         uint32
 *   scales  [N, K/group_size]      sb_dtype
 *   biases  [N, K/group_size]      sb_dtype
 *   bias    [N] or NULL            sb_dtype
 *   y       [M, N]                 y_dtype (sb_dtype or MFQ_F32)
 * M <= 16 runs the HBM-bound dequant-GEMV kernel, larger M one of two MFMA
 * GEMM kernels (128-column tiles while 256 x 256 tiles would leave more than
 * half of the compute units idle, 256 x 256 tiles otherwise).  3, 5 and 6 bits:
 * one activation row of up to 8192 elements has its own kernel, everything
 * else runs on the 128-column-tile GEMM.  For M > 4 the
 * dequantised weights are rounded once to x_dtype and sums are float32.  For
 * M <= 4 (4 and 8 bits; shapes the integer kernels take) every row of x
 * becomes 15-bit fixed point (one power of two per row brings its largest
 * magnitude under 2^14: an error of 2^-15 of that magnitude per element, exact
 * for small integers and one-hot rows), the integer products with the raw
 * codes are exact, and scale and bias are applied to their sums in float32; an
 * infinity or NaN in a row of x makes every output of that row NaN.
 */
int mfq_qmm_t(const void* x, int x_dtype, int64_t M, int64_t K,
              const uint32_t* wq, const void* scales, const void* biases,
              int sb_dtype, const void* bias, int64_t N, int group_size,
              int bits, void* y, int y_dtype, void* stream);

/*
 * mfq_qmm_t_ws with what the reference does to the linear's output next, done
 * where the GEMM writes y (one pass over [M, N] instead of two to five
 * element-wise ones).  `epilogue` is one of
 *   MFQ_EPILOGUE_GELU           y = gelu_approx(linear(x)) for the columns from
 *       act_from (a multiple of 8) on, linear(x) before them: the
 *       nn.gelu_approx(self.proj_mlp(.)) of
 *       src/mflux/models/flux/model/flux_transformer/single_transformer_block.py:53-54
 *       (act_from > 0 when q, k, v and proj_mlp run as one stacked layer) and the
 *       activation between the joint blocks' feed-forward linears (feed_forward.py:13-15);
 *   MFQ_EPILOGUE_GATE_RESIDUAL  y = residual + gate * linear(x), gate [N] and
 *       residual [M, N] in y's type, 16-byte aligned: residual + gate *
 *       proj_out(.) of single_transformer_block.py:45,57 and hidden + gate *
 *       ff(.) / gate * attn_output of joint_transformer_block.py:84-90;
 *   MFQ_EPILOGUE_SWIGLU         y[M, N/2] = silu(g) * u, where the weight's rows
 *       are the gate projection (w1) and the up projection (w3) in alternating
 *       blocks of 32 rows (N % 64 == 0): nn.silu(self.w1(x)) * self.w3(x) of
 *       src/mflux/models/z_image/model/z_image_transformer/feed_forward.py:13.
 * x, scales, biases, bias and y share one 16-bit type.  The linear's output
 * (and its bias add) is rounded to that type as the reference's linear rounds
 * it; then gate * y and the sum with the residual, each rounded (the
 * reference's two operations, bit for bit); sigmoid, x * sigmoid and the
 * product with the up projection, each rounded (MLX's nn.silu is two
 * operations).  gelu_approx is evaluated in float32 and rounded ONCE, on
 * purpose: MLX's nn.gelu_approx is a chain of element-wise operations whose
 * 16-bit intermediates each round, which is not imitated -- the result is the
 * correctly rounded value of the formula, a few units in the last place from
 * the reference's (parity with MLX unpinned at that level).
 * MFQ_EUNSUPPORTED for M <= 16 (the matvec kernels have no epilogue), N % 8 != 0,
 * and, with 256 x 256 tiles, shapes without whole scale periods (K/64 not a
 * multiple of 4 * group_size / 64): run mfq_qmm_t and apply the operations.
 * Unused pointer arguments are ignored; workspace as for mfq_qmm_t_ws.
 */
enum mfq_epilogue { MFQ_EPILOGUE_GELU = 1, MFQ_EPILOGUE_GATE_RESIDUAL = 2, MFQ_EPILOGUE_SWIGLU = 3 };
int mfq_qmm_t_epilogue(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq,
                       const void* scales, const void* biases, int sb_dtype, const void* bias,
                       int64_t N, int group_size, int bits, int epilogue, const void* gate,
                       const void* residual, int64_t act_from, void* y, int y_dtype, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * y[m, k] = sum_n x[m, n] * (scales[n, k/gs] * code[n, k] + biases[n, k/gs]):
 * the product with the weight NOT transposed.  Replaces
 * mx.quantized_matmul(x, w, scales, biases, transpose=False, ...), which is the
 * gradient of a quantized linear with respect to its input: MLX's autograd
 * evaluates it for every QuantizedLinear that
 * src/mflux/models/common/training/lora/target_injector.py:30-33 wraps in a
 * trainable LoRALinear.
 *   x       [M, N]                 x_dtype (MFQ_BF16 or MFQ_F16; must equal sb_dtype)
 *   wq      [N, K*bits/32]         uint32
 *   scales, biases [N, K/group_size]   sb_dtype
 *   y       [M, K]                 y_dtype (sb_dtype or MFQ_F32)
 * Dequantised weights are rounded once to x_dtype, sums are float32.
 * MFQ_EUNSUPPORTED when N is not a multiple of 8 (pad x with zero columns and
 * the packed weight, scales and biases with as many rows).
 */
int mfq_qmm_n(const void* x, int x_dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
              const void* biases, int sb_dtype, int64_t K, int group_size, int bits, void* y,
              int y_dtype, void* stream);

/*
 * mfq_qmm_n with an optional workspace; the same reference call
 * (mx.quantized_matmul(..., transpose=False), the input gradient of the
 * quantized linears that target_injector.py:30-33 wraps).  With
 * mfq_qmm_n_workspace_bytes(M, N, K, group_size, bits) bytes of 16-byte aligned
 * device memory (0: the shape does not use any), calls with many rows of x, 4-
 * or 8-bit weights and a 16-bit y run as two kernels: a 16-bit copy of the
 * dequantised weight, transposed into the order the matrix instructions
 * consume, then the GEMM of mfq_qmm_t's large-M path on it (about twice the
 * rate of the one-kernel form).  The workspace may be reused by the next call
 * on the same stream.  With a smaller workspace, or none, the call is
 * mfq_qmm_n.
 */
size_t mfq_qmm_n_workspace_bytes(int64_t M, int64_t N, int64_t K, int group_size, int bits);
int mfq_qmm_n_ws(const void* x, int x_dtype, int64_t M, int64_t N, const uint32_t* wq, const void* scales,
                 const void* biases, int sb_dtype, int64_t K, int group_size, int bits, void* y, int y_dtype,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * mfq_qmm_t with an optional float32 workspace.  Has no counterpart in the
 * reference (MLX allocates inside its ops).  Shapes whose output tiles do not
 * fill the GPU's compute units -- the text-stream linears of the double
 * blocks, M = 256 or 512 tokens against N = 3072, e.g.
 * src/mflux/models/qwen/model/qwen_transformer/qwen_transformer_block.py:36-37
 * on the caption tokens, or the last, mostly empty round of tiles of the image
 * stream at M = 6889 -- leave part of the chip idle; with a workspace K is
 * cut into ranges that run on different compute units, each range accumulates
 * into its own float32 plane of the workspace, and a second kernel adds the
 * planes, rounds and applies the bias (same two roundings as the fused
 * epilogue).  Large calls -- 16-bit y, K a multiple of 128, at least 2048
 * activation rows at 4 or 8 bits and 1024 at 3, 5 or 6 (where it starts to
 * pay), e.g. the single-stream
 * linears of FLUX.1 at M = 4608 -- use the workspace first for a 16-bit copy of
 * the dequantised weights (round_up(N, 16) * K * 2 bytes rounded up to 256,
 * written once per call in the order the matrix instructions consume it) and
 * multiply with a kernel that has no dequantisation in its loop; the planes of
 * a K cut, if the shape has a short last round of tiles, lie behind the copy.
 * The copy's values are the ones the fused kernels use (one rounding of
 * fma(code, scale, bias)); the float32 sums run in another order.
 * mfq_qmm_t_workspace_bytes() returns the size this shape would use on the
 * current device (0: no use for one, pass NULL).  A NULL or smaller workspace
 * is not an error: without room for the copy the call runs as mfq_qmm_t does
 * (the fused kernel, K not split), with room for the copy only its tiles run
 * whole.  The workspace must be 16-byte aligned; its contents before and after
 * the call are undefined; calls sharing one workspace must be ordered on one
 * stream.
 */
size_t mfq_qmm_t_workspace_bytes(int64_t M, int64_t K, int64_t N, int group_size, int bits);
int mfq_qmm_t_ws(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq,
                 const void* scales, const void* biases, int sb_dtype, const void* bias, int64_t N,
                 int group_size, int bits, void* y, int y_dtype, void* workspace,
                 size_t workspace_bytes, void* stream);

/*
 * The two halves of a large mfq_qmm_t_ws call apart, for weights that do not
 * change between calls (inference).  Has no counterpart in the reference: MLX
 * dequantises inside every quantized_matmul.  mfq_qmm_t_prepare writes the
 * 16-bit copy of the dequantised weights that mfq_qmm_t_ws makes per call --
 * one rounding of fma(code, scale, bias) to sb_dtype, in the order the matrix
 * instructions consume it, mfq_qmm_t_prepared_bytes(N, K, bits) bytes (2 per
 * weight; 0: no such copy for this shape: K not a
 * multiple of 128 or below 256, N not a multiple of 8, or more than 2 GiB) --
 * into a buffer the caller keeps, and mfq_qmm_t_prepared multiplies x
 * [M, K] of the same 16-bit type with it into y [M, N] of that type (+ bias):
 * bit-identical to what mfq_qmm_t_ws gives on its two-kernel path, for any M,
 * at 2 bytes per weight of memory held instead of bits / 8 -- on FLUX.1's
 * single-block linears at M = 4608 the copy is 7 % of the call.
 * `workspace` (optional, 16-byte aligned, mfq_qmm_t_prepared_workspace_bytes)
 * takes the float32 planes of a K cut of a short last round of tiles; without
 * it the tiles run whole.  MFQ_EUNSUPPORTED for shapes without a copy.
 */
size_t mfq_qmm_t_prepared_bytes(int64_t N, int64_t K, int bits);
int mfq_qmm_t_prepare(const uint32_t* wq, const void* scales, const void* biases, int sb_dtype,
                      int64_t N, int64_t K, int group_size, int bits, void* prepared, void* stream);
size_t mfq_qmm_t_prepared_workspace_bytes(int64_t M, int64_t K, int64_t N);
int mfq_qmm_t_prepared(const void* x, int dtype, int64_t M, int64_t K, const void* prepared,
                       const void* bias, int64_t N, void* y, void* workspace, size_t workspace_bytes,
                       void* stream);

/*
 * mfq_qmm_t_ws for callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  Has no counterpart in
 * the reference.  The float32 planes of the K split live in a buffer of
 * MFQ_STATIC_SCRATCH_BYTES that is part of the library's device image (every
 * GPU the library runs on holds its own copy until the process ends), so the
 * call allocates nothing and takes no workspace: same arguments as mfq_qmm_t,
 * same kernels and bit-identical results as mfq_qmm_t_ws with a workspace of
 * mfq_qmm_t_workspace_bytes() -- except that a copy of the dequantised weights
 * that does not fit the buffer is done without (the fused kernel then runs:
 * same tolerance, other bits).  A shape whose split needs more than the
 * buffer holds is refused with MFQ_ESCRATCH and nothing is launched (on a
 * 256-CU device: the last, short round of 256 x 256 tiles cut into more than
 * 128 planes, e.g. M = 6889 against 3072 -> 3072; use mfq_qmm_t_ws or
 * mfq_qmm_t there).  All calls on one GPU share that GPU's buffer: calls that
 * overlap on one GPU (two streams, two threads) race; order them on one
 * stream.  The buffer's contents between calls are undefined; nothing in it
 * has to be zero.  The first call on a device looks the buffer's address up
 * and configures the kernels; make it outside a graph capture.
 */
#define MFQ_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int mfq_qmm_t_static(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq,
                     const void* scales, const void* biases, int sb_dtype, const void* bias,
                     int64_t N, int group_size, int bits, void* y, int y_dtype, void* stream);

/*
 * y[m, n] = sum_k silu(x)[m, k] * (scales[n, k/gs] * code[n, k] + biases[n, k/gs]) (+ bias[n]):
 * the adaLN modulation call linear(nn.silu(text_embeddings)) of every
 * transformer block as one kernel, for one to four rows of x (the batch)
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:12
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero_single.py:12
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_continuous.py:15
 * (the reference runs nn.silu as an elementwise kernel of its own in front
 * of the quantized matmul).  silu(x) = x * sigmoid(x) with the sigmoid and
 * the product each rounded to x_dtype, as the two operations of MLX's nn.silu
 * on a 16-bit array round; the rounded rows then go through exactly what
 * mfq_qmm_t does for M <= 4.  Arguments as for mfq_qmm_t.
 * MFQ_EUNSUPPORTED when no fused kernel takes the shape (bits other than 4
 * and 8; M = 1 with rows of more than 6 KiB of 8-bit or 3 KiB of 4-bit codes;
 * M = 2..4 outside what the eight-rows kernels (K = 1024, 2048, 3072 or 4096,
 * group size 64, N a multiple of 8) and the four-rows kernel (K <= 4096, N a
 * multiple of 4, rows of 1, 2, 3, 4, 6, 8, 12 or 16 times 256 bytes) take;
 * M > 4): apply the activation separately and call mfq_qmm_t.
 */
int mfq_qmv_silu(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq,
                 const void* scales, const void* biases, int sb_dtype, const void* bias, int64_t N,
                 int group_size, int bits, void* y, int y_dtype, void* stream);

/*
 * A quantized linear layer with LoRA adapters on it in one call:
 *   y = x @ dequantize(wq, scales, biases)^T + t @ bs^T (+ bias).
 * Replaces the body of LoRALinear.__call__
 * (src/mflux/models/common/lora/layer/linear_lora_layer.py:50-53:
 * base_out + scale * ((x @ lora_A) @ lora_B)) and of FusedLoRALinear.__call__
 * (src/mflux/models/common/lora/layer/fused_linear_lora_layer.py:13-20, the sum
 * over several adapters) around a QuantizedLinear base.  The caller passes
 *   t  [M, rank] = x @ [lora_A_1 | lora_A_2 | ...]      (a plain small GEMM)
 *   bs [N, rank] = [scale_1 * lora_B_1^T | scale_2 * lora_B_2^T | ...]
 * both row-major and 16-byte aligned, in x_dtype, with rank (the sum of the
 * adapters' ranks) zero-padded to a multiple of 16, at most 1024.  The GEMM
 * kernels (M > 16) treat them as `rank` more k after the layer's own, in the
 * same float32 accumulators, so the product is rounded once (the reference
 * rounds the base output, both LoRA products, the scaling and the sum
 * separately); behind the matvec kernels (M <= 16) a second kernel adds the
 * update to the rounded product (mfq_low_rank_add).  rank == 0 (t, bs
 * ignored) is mfq_qmm_t_ws; everything else is as documented there, odd bit
 * widths for M = 1 included.
 */
int mfq_qmm_t_low_rank(const void* x, int x_dtype, int64_t M, int64_t K, const uint32_t* wq,
                       const void* scales, const void* biases, int sb_dtype, const void* bias,
                       int64_t N, int group_size, int bits, const void* t, const void* bs,
                       int64_t rank, void* y, int y_dtype, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * y = LayerNorm(x, eps) * (1 + scale) + shift, row by row: the normalisation
 * without learned parameters and the adaLN modulation in front of every
 * modulated linear of the DiT blocks, four element-wise passes in the reference
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero.py:22
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_zero_single.py:19
 *   src/mflux/models/flux/model/flux_transformer/ada_layer_norm_continuous.py:21
 *   src/mflux/models/flux/model/flux_transformer/joint_transformer_block.py:86-87
 * (nn.LayerNorm(dims, eps=1e-6, affine=False), then * (1 + scale), + shift).
 *   x, y    [M, K]                      dtype (MFQ_BF16 or MFQ_F16), 16-byte aligned
 *   scale, shift  [M / rows_per_vector, K]  dtype, 16-byte aligned: one vector per
 *                 batch entry, shared by rows_per_vector consecutive rows; both
 *                 NULL for the plain LayerNorm (rows_per_vector is then ignored)
 * Mean and variance are float32 sums over the row; the normalised value,
 * 1 + scale, their product and the sum with the shift are each rounded to
 * dtype, as the reference's separate operations on a 16-bit array round
 * (the order of the float32 sums inside MLX's layer norm: parity unpinned).
 * MFQ_EUNSUPPORTED for K > 8192 or K % 8 != 0.
 */
int mfq_layer_norm_modulate(const void* x, int dtype, int64_t M, int64_t K, const void* scale,
                            const void* shift, int64_t rows_per_vector, float eps, void* y, void* stream);

/*
 * t[M, rank] = x[M, K] @ A[K, rank]: the down-projection of the adapters,
 * mx.matmul(x, lora_A) of src/mflux/models/common/lora/layer/linear_lora_layer.py:50-53
 * for all adapters of a layer at once, A = [lora_A_1 | lora_A_2 | ...] (zero
 * columns up to a multiple of 16).  A is packed once per adapter set, so it is
 * handed over in the order the matrix instruction consumes, af
 * [rank/16][K/32][4][16][8]: af[f][s][q][c][e] = A[32 s + 8 q + e][16 f + c].
 * x, af and t are of the 16-bit type dtype; the sums are float32, rounded
 * once.  rank % 16 == 0, rank <= 1024, K % 32 == 0.  t is the first operand of
 * mfq_qmm_t_low_rank and mfq_low_rank_add.
 */
int mfq_low_rank_down(const void* x, const void* af, int dtype, int64_t M, int64_t K, int64_t rank, void* t,
                      void* stream);

/*
 * y[M, N] += t[M, rank] @ bs[N, rank]^T in float32, rounded to y_dtype (dtype
 * or MFQ_F32): the same adapters (see mfq_qmm_t_low_rank for t and bs) behind
 * a product that did not come from mfq_qmm_t_low_rank, e.g. one of the matvec
 * kernels (M <= 16) or mfq_qmm_n.
 */
int mfq_low_rank_add(const void* t, const void* bs, int dtype, int64_t M, int64_t N, int64_t rank,
                     void* y, int y_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MFQ_H */
