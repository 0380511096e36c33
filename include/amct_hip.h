/*
 * amct_hip.h -- C ABI of libamct_hip.so: the quantize / deploy hot path of AMCT
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - tensors are dense and row-major; 16-byte aligned bases take the fast
 *     kernels, anything else a slower general kernel (same results);
 *   - the library never allocates, frees or synchronises: the caller owns all
 *     buffers (including workspaces) and supplies the stream; every call only
 *     enqueues work on `stream` and returns (amct_col_minmax_noalloc keeps its
 *     workspace in a fixed device array of the library instead);
 *   - return value: 0 on success, a negative AMCT_E_* code otherwise
 *     (amct_hip_strerror gives the text); no exception crosses the boundary;
 *     a call that fails enqueues nothing and leaves its outputs untouched;
 *   - an empty problem (rows, M or n equal to 0) succeeds without enqueuing
 *     anything, and its tensor pointers may then be null (an empty torch
 *     tensor has a null data pointer);
 *   - dtype arguments use AMCT_F32 / AMCT_F16 / AMCT_BF16, numbered like the
 *     reference's DATA_MAP (amct_pytorch/utils/data_utils.py:19-23).
 *
 * Paths below are relative to the reference repository root.
 */
#ifndef AMCT_HIP_H
#define AMCT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* amct_stream_t;            /* a hipStream_t */

enum { AMCT_F32 = 0, AMCT_F16 = 1, AMCT_BF16 = 2 };

enum {
    AMCT_OK = 0,
    AMCT_E_BADARG = -1,                 /* null pointer, negative size, unknown enum */
    AMCT_E_UNSUPPORTED = -2,            /* shape / combination the kernels do not cover */
    AMCT_E_ALIGN = -3,                  /* alignment or divisibility requirement violated */
    AMCT_E_HIP = -4,                    /* the HIP runtime reported a launch error */
    AMCT_E_TOO_LARGE = -5               /* the problem exceeds the fixed scratch buffer of an allocation-free entry point */
};

/* symmetric scope rule */
enum {
    AMCT_SCOPE_AMCT = 0,                /* 2^(b-1)-1, +1 where |min| > |max|; eps guard
                                           (amct_pytorch/quantize_op/utils.py:87-92,158-176,26-51) */
    AMCT_SCOPE_ABSMAX = 1               /* absmax / qmax, no guard
                                           (amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py:128-137) */
};

/* per-column pre/post scaling fused into the weight kernels */
enum {
    AMCT_COL_NONE = 0,
    AMCT_COL_MUL = 1,                   /* w * c[k], rounded to w's dtype (amct_pytorch/utils/quant_util.py:96-111) */
    AMCT_COL_DIV = 2,                   /* w / c[k], rounded to w's dtype (amct_pytorch/utils/quant_util.py:143-159) */
    AMCT_COL_MUL_THEN_DIV = 3           /* w * c[k] before, result / c[k] after: one AWQ grid point
                                           (amct_pytorch/algorithm/awq.py:30-49) */
};

/* which part of the quantiser amct_quant_with_params runs */
enum {
    AMCT_STAGE_FULL = 0,                /* quantise (+ dequantise) */
    AMCT_STAGE_SCALE = 1,               /* dq = w/s + z, no rounding: do_quant (amct_pytorch/algorithm/awq.py:129-149) */
    AMCT_STAGE_DEQUANT = 2,             /* dq = (w - z) * s: do_dequant (amct_pytorch/algorithm/awq.py:152-170) */
    AMCT_STAGE_COL = 3                  /* dq = w * c[k] or w / c[k] only (amct_pytorch/utils/quant_util.py:96-111,143-159) */
};

/* kind of integer code output */
enum { AMCT_CODES_NONE = 0, AMCT_CODES_I8 = 1, AMCT_CODES_I32 = 2 };

int amct_hip_version(void);
const char* amct_hip_strerror(int code);

/* Plain device-to-device streaming copy (nbytes % 16 == 0).  No counterpart in the reference: it is
 * the yardstick for the bandwidth figures and for scaling hardware traffic counters. */
int amct_copy_bytes(const void* src, void* dst, int64_t nbytes, amct_stream_t stream);

/* Register-only MFMA loop on every CU (8 waves per CU, no memory traffic), int8 32x32x32 or bf16 32x32x16, with
 * constant or pseudo-random operand values.  No counterpart in the reference: it is the yardstick for the GEMM
 * figures, the rate the matrix pipe sustains under the power limit for that kind of data.  sink: >= 2 KiB of
 * device memory (never written in practice); *ops receives the number of operations (2 per multiply-add) the
 * launch performs. */
int amct_mfma_yardstick(int bf16, int random_operands, int iters, void* sink, int64_t* ops, amct_stream_t stream);

/* ---- column statistics over tokens (calibration of the smoothing factor) -----------------
 * Replaces the reductions of amct_pytorch/quantize_op/smooth_quant_module.py: :79-80 batch amax / amin over
 * all tokens per input channel, :88-91 the running update data_max = batch_max > data_max ? batch_max :
 * data_max (and the mirror image for the minimum), :121 |W|.amax(dim=0).
 * x [rows, cols]; col_max, col_min fp32 [cols] (either may be null).  absolute != 0 reduces |x|.
 * accumulate = 0 overwrites the outputs with this batch's values; accumulate != 0 applies the running update
 * to the values already there (a NaN batch value leaves them unchanged, as torch.where does).
 * max / min propagate NaN like torch.amax / amin.  workspace: amct_col_minmax_workspace_bytes(rows, cols)
 * bytes of device memory, 4-byte aligned, contents irrelevant before and after the call. */
size_t amct_col_minmax_workspace_bytes(int64_t rows, int64_t cols);
int amct_col_minmax(const void* x, float* col_max, float* col_min, int64_t rows, int64_t cols, int absolute,
                    int accumulate, int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream);

/* amct_col_minmax without a workspace argument.  No counterpart in the reference: it is for callers that cannot
 * allocate device memory around the call (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  Same arguments, kernels and results as amct_col_minmax; the per-chunk partials go to a fixed array
 * inside the library's device image instead (64 chunks x 2 x AMCT_COL_MINMAX_NOALLOC_MAX_COLS floats = 4 MiB, held
 * by every GPU the library runs on until the process ends).  cols > AMCT_COL_MINMAX_NOALLOC_MAX_COLS returns
 * AMCT_E_TOO_LARGE and enqueues nothing.  The call allocates and frees nothing.  The FIRST call on a device asks the
 * runtime for the array's address on that device (hipGetDevice, hipGetSymbolAddress: the runtime may load the
 * library's code object then), so make one ordinary call per device before capturing the entry point in a graph.
 * All calls on one GPU share that array, whatever their stream: calls that overlap on one GPU (different streams or
 * threads) race; calls on one stream do not.  Nothing has to be cleared between calls (the first pass overwrites
 * every partial the second pass reads). */
#define AMCT_COL_MINMAX_NOALLOC_MAX_COLS 8192
int amct_col_minmax_noalloc(const void* x, float* col_max, float* col_min, int64_t rows, int64_t cols, int absolute,
                            int accumulate, int dtype, amct_stream_t stream);

/* ---- loss of one AWQ grid point ---------------------------------------------------------------------
 * Replaces the expression of amct_pytorch/algorithm/awq.py:96, `(ori_out - quant_out).float().pow(4).mean()`:
 * loss[0] (fp32, device) = mean over the n elements of (dtype(y - yhat))^4, the difference rounded to the
 * tensors' dtype as the reference's subtraction does, the fourth power and the sum in fp32.  One pass over
 * both tensors; the summation order is fixed by n (same result on every call and device) but is not torch's,
 * so the value agrees with the reference's to the rounding of an fp32 sum.  n = 0 gives NaN, as torch does.
 * y, yhat 16-byte aligned; workspace: amct_awq_loss_workspace_bytes() bytes of device memory, 4-byte aligned,
 * contents irrelevant before and after the call. */
size_t amct_awq_loss_workspace_bytes(void);
int amct_awq_loss(const void* y, const void* yhat, int64_t n, int dtype, float* loss, void* workspace,
                  size_t workspace_bytes, amct_stream_t stream);

/* ---- A1: min / max per row (group = 0) or per group of `group` columns ----------------
 * Replaces get_weight_min_max_by_granularity (amct_pytorch/quantize_op/utils.py:111-136)
 * and the per-token reductions of amct_pytorch/quantize_op/minmax_module.py:96-105.
 * w [rows, cols]; mn, mx fp32 [rows * ceil(cols/group)] ([rows] when group = 0).
 * A ragged last group is zero-padded and the zeros take part
 * (amct_pytorch/utils/quant_util.py:23-36).  NaN propagates as in torch.max. */
int amct_minmax(const void* w, float* mn, float* mx, int64_t rows, int64_t cols, int group,
                int dtype, amct_stream_t stream);

/* ---- A2: (max, min) -> (scale, offset) --------------------------------------------------
 * Replaces calculate_scale_offset (amct_pytorch/quantize_op/utils.py:75-108).
 * mx, mn: n values of `in_dtype`; scale fp32 [n]; offset int32 [n] (ignored / may be null
 * when symmetric).  bad_count (int32[1], may be null) is incremented once per entry whose
 * scale, 1/scale or offset is not finite (check_scale_offset, utils.py:54-72); the caller
 * zeroes it beforehand and decides whether to read it. */
int amct_scale_offset(const void* mx, const void* mn, float* scale, int32_t* offset, int32_t* bad_count,
                      int64_t n, int bits, int symmetric, int scope_rule, int in_dtype,
                      amct_stream_t stream);

/* ---- A3 / A4 / A5 / A6: quantise with given factors -------------------------------------
 * Replaces quant_dequant_weight (amct_pytorch/utils/quant_util.py:162-188), quant_weight +
 * convert_dtype (:56-93), NpuQuantizationLinear.quant_wts
 * (amct_pytorch/deploy_op/npu_quantization_linear.py:72-87) and, with
 * round_via_src_dtype = 1, AWQ's do_quant -> convert_precision -> do_dequant
 * (amct_pytorch/algorithm/awq.py:129-170, amct_pytorch/utils/data_utils.py:48-66).
 * w [rows, cols]; scale fp32 and offset int32 (null = symmetric) indexed
 *   group > 0 : [rows, ceil(cols/group)]   group = 0 : [rows]   group = -1 : [1]
 * dq (same dtype as w, may be null) = ((clamp(rne(w/s + z), qmin, qmax)) - z) * s
 * codes (may be null) = clamp(rne(w/s + z), qmin, qmax) as int8 or int32, [rows, cols].
 * stage = AMCT_STAGE_SCALE / AMCT_STAGE_DEQUANT / AMCT_STAGE_COL run only one part (dq required,
 * codes null). */
int amct_quant_with_params(const void* w, const float* scale, const int32_t* offset,
                           void* dq, void* codes, int codes_kind,
                           const void* col_scale, int col_mode,
                           int64_t rows, int64_t cols, int group, int qmin, int qmax,
                           int round_via_src_dtype, int stage, int dtype, amct_stream_t stream);

/* ---- K1: A1 + A2 + A3/A4 fused, one read of w --------------------------------------------
 * group >= 0 only (per-tensor factors are composed from amct_minmax / amct_scale_offset /
 * amct_quant_with_params).  scale fp32 / offset int32 (null when symmetric) are OUTPUTS with
 * the indexing above.  bad_count as in amct_scale_offset. */
int amct_fakequant_int(const void* w, void* dq, void* codes, int codes_kind,
                       float* scale, int32_t* offset, int32_t* bad_count,
                       const void* col_scale, int col_mode,
                       int64_t rows, int64_t cols, int group, int bits, int symmetric,
                       int scope_rule, int qmin, int qmax, int round_via_src_dtype,
                       int dtype, amct_stream_t stream);

/* ---- K2: int4 per-group quantise + pack ---------------------------------------------------
 * Replaces the weight preparation of NpuWeightQuantizedLinear.__init__
 * (amct_pytorch/deploy_op/weight_npu_quant_module.py:38-66): min/max per group, factors,
 * codes, packing, factor narrowing -- in one pass.
 * w [rows, cols], cols % group == 0, group % 32 == 0.
 * packed   uint8 [rows, cols/2]: code + 8 (unsigned 0..15), even column in the low nibble
 * scales16 [rows, cols/group] of scale_dtype (AMCT_F16 / AMCT_BF16), may be null
 * scales32 fp32 [rows, cols/group], may be null
 * zeros    uint8 [rows, cols/group]: offset + 8 (8 everywhere when symmetric), may be null */
int amct_quant_int4_group_pack(const void* w, uint8_t* packed, void* scales16, int scale_dtype,
                               float* scales32, uint8_t* zeros, int32_t* bad_count,
                               const void* col_scale, int col_mode,
                               int64_t rows, int64_t cols, int group, int symmetric,
                               int dtype, amct_stream_t stream);

/* ---- int4 interchange layouts ---------------------------------------------------------------
 * amct_pack_int4_words replaces torch_npu.npu_convert_weight_to_int4pack as called at
 * amct_pytorch/deploy_op/weight_npu_quant_module.py:54-57: int32 [k, n] holding one signed
 * int4 each -> int32 [k, n/8], column 8*i+j in bits 4j..4j+3 of word i.
 * amct_words_to_nibbles_nk converts that [k, n/8] form to the GEMM layout
 * uint8 [n, k/2] (code + 8, even k in the low nibble). */
int amct_pack_int4_words(const int32_t* codes, int32_t* words, int64_t k, int64_t n, amct_stream_t stream);
int amct_words_to_nibbles_nk(const int32_t* words, uint8_t* packed, int64_t k, int64_t n, amct_stream_t stream);
/* amct_pack_nibbles_nk: int8 codes [rows, cols] (signed int4 values, as convert_dtype of
 * amct_pytorch/utils/quant_util.py:56-73 yields them) -> uint8 [rows, cols/2] in the GEMM layout.
 * amct_nibbles_nk_to_codes_kn: the way back to the reference's operand, int32 [k, n] signed codes
 * (amct_pytorch/deploy_op/weight_npu_quant_module.py:52-53). */
int amct_pack_nibbles_nk(const int8_t* codes, uint8_t* packed, int64_t rows, int64_t cols, amct_stream_t stream);
int amct_nibbles_nk_to_codes_kn(const uint8_t* packed, int32_t* codes, int64_t k, int64_t n, amct_stream_t stream);

/* ---- K3: activation quantise ------------------------------------------------------------------
 * amct_act_quant_per_token_int8: dynamic symmetric int8 per row -- the per-token statistics of
 * amct_pytorch/quantize_op/minmax_module.py:96-110 + calculate_scale_offset evaluated on the live
 * batch, then convert_dtype.  mode 0: AMCT 127/128 scope rule with eps guard; mode 1: absmax/127,
 * scale 1 for an all-zero row, clamp [-128,127]
 * (amct_pytorch/experimental/quantization/DeepSeekV3.2/cores/quantization/node.py:39-43,181-204).
 * smooth (dtype of x, [K], may be null) multiplies x first, rounded to x's dtype
 * (amct_pytorch/deploy_op/npu_quantization_linear.py:96-97).
 * amct_quantize: the static operator torch_npu.npu_quantize as called at
 * npu_quantization_linear.py:98-99 (div_mode=False): q = sat_int8(rne(x * scales + zero_points)),
 * scales / zero_points of x's dtype; per_token = 0: n_scales in {1, K} broadcast along the last
 * dim; per_token = 1: one per row. */
int amct_act_quant_per_token_int8(const void* x, const void* smooth, int8_t* q, float* scale,
                                  int64_t M, int64_t K, int mode, int dtype, amct_stream_t stream);
int amct_quantize(const void* x, const void* smooth, const void* scales, const void* zero_points,
                  int8_t* q, int64_t M, int64_t K, int64_t n_scales, int per_token, int dtype,
                  amct_stream_t stream);

/* ---- K4: microscaling block-32 formats (no counterpart in the reference) ------------------------
 * fmt: 0 = FP8 E4M3 (elements uint8 [rows, cols]), 1 = FP4 E2M1 (uint8 [rows, cols/2], even
 * column in the low nibble).  e8m0 uint8 [rows, cols/32].  scale_mode 0 = floor, 1 = round-up.
 * cols % 32 == 0. */
int amct_mx_quant(const void* x, uint8_t* elems, uint8_t* e8m0, int64_t rows, int64_t cols,
                  int fmt, int scale_mode, int dtype, amct_stream_t stream);
int amct_mx_dequant(const uint8_t* elems, const uint8_t* e8m0, void* y, int64_t rows, int64_t cols,
                    int fmt, int dtype, amct_stream_t stream);

/* ---- K5: HiFloat8 (no counterpart in the reference) ------------------------------------------------ */
int amct_hif8_encode(const void* x, uint8_t* y, int64_t n, int dtype, int saturate, amct_stream_t stream);
int amct_hif8_decode(const uint8_t* x, void* y, int64_t n, int dtype, amct_stream_t stream);

/* ---- K6: W8A8 Linear ----------------------------------------------------------------------------------
 * Replaces torch_npu.npu_quant_matmul as called at
 * amct_pytorch/deploy_op/npu_quantization_linear.py:100-102.
 * xq int8 [M, K]; wq int8 [N, K] (K contiguous: the storage behind the reference's transposed
 * [K, N] view, :53-55); s_ch fp32 [N]; s_tok fp32 [M] or null; bias: null, int32 [N]
 * (bias_kind 1, joins the accumulator) or fp32 [N] (bias_kind 2, added after the rescale).
 * out [M, N] of out_dtype = fp32(acc + ibias) * s_ch[n] * s_tok[m] + fbias, rounded once.
 * acc_out (int32 [M, N], may be null) receives the raw accumulators. */
int amct_gemm_w8a8(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch,
                   const void* bias, int bias_kind, void* out, int32_t* acc_out,
                   int64_t M, int64_t N, int64_t K, int out_dtype, amct_stream_t stream);
/* The same with a workspace (may be null): amct_gemm_w8a8_workspace_bytes(M, N, K) bytes the caller lends, 16-byte
 * aligned, contents irrelevant before and after the call.  The query asks for memory when the tiles of the launch would
 * leave CUs idle and the rows are long (few output columns against the number of CUs, K >= 4096: the down projection of
 * an MLP at 3 .. a few hundred rows): K is then split over several blocks per tile, which leave int32 partial sums in the
 * workspace, and a second kernel adds them and applies the epilogue.  Integer sums are exact, so the result is that of
 * amct_gemm_w8a8 bit for bit; 0 bytes otherwise; a null or smaller workspace is never an error. */
size_t amct_gemm_w8a8_workspace_bytes(int64_t M, int64_t N, int64_t K);
int amct_gemm_w8a8_ws(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch,
                      const void* bias, int bias_kind, void* out, int32_t* acc_out,
                      int64_t M, int64_t N, int64_t K, int out_dtype, void* workspace, size_t workspace_bytes,
                      amct_stream_t stream);

/* The deploy module's forward in one call: the static quantisation of the activations followed by the W8A8 Linear
 * (amct_pytorch/deploy_op/npu_quantization_linear.py:96-102: x * scale_factor, torch_npu.npu_quantize,
 * torch_npu.npu_quant_matmul).  x [M, K] of x_dtype; smooth, act_scale, act_offset as for amct_quantize (n_scales,
 * per_token likewise); the other operands as for amct_gemm_w8a8.  The result is that of amct_quantize followed by
 * amct_gemm_w8a8 bit for bit.  For M <= 16, K of 1024 / 2048 / 4096, bf16 or fp16 x and one scale per tensor or per
 * row, the activations are quantised inside the weight-streaming kernel while it stages them (one launch, no int8
 * copy of x in memory); otherwise the two kernels run one after the other and the int8 activations go through the
 * workspace: amct_linear_w8a8_workspace_bytes(M, N, K) bytes, 16-byte aligned, contents irrelevant before and after
 * (AMCT_E_BADARG when such a call comes without it). */
size_t amct_linear_w8a8_workspace_bytes(int64_t M, int64_t N, int64_t K);
int amct_linear_w8a8(const void* x, int x_dtype, const void* smooth, const void* act_scale, const void* act_offset,
                     int64_t n_scales, int per_token, const int8_t* wq, const float* s_tok, const float* s_ch,
                     const void* bias, int bias_kind, void* out, int64_t M, int64_t N, int64_t K, int out_dtype,
                     void* workspace, size_t workspace_bytes, amct_stream_t stream);

/* ---- K7: W4A16 Linear -------------------------------------------------------------------------------------
 * Replaces torch_npu.npu_weight_quant_batchmatmul as called at
 * amct_pytorch/deploy_op/weight_npu_quant_module.py:116-117 (with the x * scale_factor of :113-114
 * fused in).  x [M, K] of dtype (AMCT_BF16 or AMCT_F16, the source dtypes of
 * amct_pytorch/utils/vars.py:43-47); smooth [K] of dtype or null; wq uint8 [N, K/2] as written by
 * amct_quant_int4_group_pack; scales [N, K/group] of scale_dtype; zeros uint8 [N, K/group];
 * bias fp32 [N] or null.  out [M, N] of dtype = x' @ dtype((u - zero) * scale)^T + bias, fp32 accumulate.
 * workspace (may be null): amct_gemm_w4a16_workspace_bytes(M, N, K, group, smooth != null) bytes the caller lends,
 * 16-byte aligned, contents irrelevant before and after the call.  For M > 16 with smooth the multiply is then done
 * once up front instead of inside every column tile (same results; the fast bf16 tile kernels need it, without it such
 * calls take slower kernels that smooth in place).  From M = 1025 on the query also asks for N * K * 2 bytes: the weight
 * is then dequantised once into the workspace and the product runs as a plain 16-bit GEMM, which beats dequantising inside
 * every row tile from there on (same arithmetic; a smaller workspace keeps the fused kernels).  For long rows on few
 * column blocks (the down projection of an MLP at up to a few hundred rows) the query also asks for S * M * N * 4 bytes:
 * K is then split over S blocks per tile, whose fp32 partial sums a second kernel adds in a fixed order; likewise for
 * M <= 16 (from 5 rows on, for K >= 12288, or when K / 256 is not a multiple of 4) when K is 2 ... 16 slices of 4096, 2048
 * or 1024 elements (the last one shorter for other multiples of 256, e.g. 11008), which the weight-streaming kernel then
 * walks one per block.  0 bytes are
 * asked for otherwise; a null or smaller workspace is never an error.
 * Arithmetic of the dequantisation (the operator's own lives inside the un-vendored torch_npu, so the library fixes
 * two readings and says which one a call takes):
 *   exact    the weight-streaming kernel for M <= 16 (bf16 or fp16, K of 1024 / 2048 / 4096 or slices of those,
 *            group = 128) keeps the weight as the exact integer and applies scale and zero per group in fp32: the
 *            dequantised weight is not rounded (the fp32 weight * scale of tests/amct_pytorch/mock_torch_npu.py:33-55).
 *            Within 1e-5 of the row's largest output (+ the rounding of the output) of the exact result.
 *   rounded  every other kernel feeds dtype((u - zero) * scale) to the matrix pipe, whose operands are 16 bits wide.
 *            Each weight then carries a relative error of up to u = 2^-8 (bf16; 2^-11 for fp16), so an output differs
 *            from the exact result by at most u * sum_k |x'_k * w_k|, and for errors of independent sign by about
 *            u / sqrt(3) * sqrt(sum_k (x'_k * w_k)^2).  On W[14336, 4096] with N(0, 1) activations that is up to
 *            2.5e-3 of the row's largest output for bf16 (3e-4 for fp16): bf16 calls of more than 16 rows are NOT
 *            within 1e-3 of the exact result at K = 4096, and a token's output differs by that much between a call
 *            of up to 16 rows and a larger one.
 * amct_gemm_w4a16_weight_rounded answers 0 (exact) or 1 (rounded) for a call of that shape, dtype and workspace size
 * with 16-byte aligned operands (unaligned operands always take a rounding kernel); a negative error code for
 * arguments amct_gemm_w4a16 rejects. */
int amct_gemm_w4a16_weight_rounded(int64_t M, int64_t N, int64_t K, int group, int dtype, size_t workspace_bytes);
size_t amct_gemm_w4a16_workspace_bytes(int64_t M, int64_t N, int64_t K, int group, int has_smooth);
int amct_gemm_w4a16(const void* x, const void* smooth, const uint8_t* wq, const void* scales,
                    int scale_dtype, const uint8_t* zeros, const float* bias, void* out,
                    int64_t M, int64_t N, int64_t K, int group, int dtype,
                    void* workspace, size_t workspace_bytes, amct_stream_t stream);

/* ---- W8A16 Linear (int8 weight-only) ---------------------------------------------------------------------
 * The same operator with the int8 weight the reference's module registers when wts_type is int8
 * (amct_pytorch/deploy_op/weight_npu_quant_module.py:51-53: quant_weight yields int8 codes, only int4 is packed).
 * x [M, K] of dtype (AMCT_BF16 or AMCT_F16); smooth [K] of dtype or null; wq int8 [N, K] signed codes, K contiguous
 * (the transpose of the [K, N] buffer of :53); scales [N, K/group] of scale_dtype (group = K: one per output
 * channel, the reference's antiquant_group_size = 0); offsets int8 [N, K/group] = the quantiser's offset_w, null
 * when symmetric (the module registers its negation as antiquant_offset, :62-64); bias fp32 [N] or null.
 * out [M, N] of dtype = x' @ dtype((q - offset) * scale)^T + bias, fp32 accumulate.
 * As for the int4 weight there are two readings of the dequantisation: the weight-streaming kernel for M <= 16 (K of
 * 1024 / 2048 / 4096, group a power of two from 128 to K; through amct_gemm_w8a16_ws and its workspace also rows of
 * 2 ... 16 such slices, the last one shorter if need be -- K = 8192, 11008, 14336, 28672, 5120 ... --, groups up to a
 * slice, whole slices or the whole row, where that beats the other kernels) keeps the weight as the exact integer and
 * applies scale and offset per group in fp32 (within 2e-5 of the row's largest output of the exact result); every other
 * kernel feeds dtype((q - offset) * scale) to the matrix pipe, with the error bound stated for amct_gemm_w4a16 (up to
 * 2.5e-3 of the row's largest output for bf16 at K = 4096).  amct_gemm_w8a16_weight_rounded answers 0 (exact) or
 * 1 (rounded) for a call of that shape, dtype and workspace size (0 for amct_gemm_w8a16, which has none) with 16-byte
 * aligned operands. */
int amct_gemm_w8a16_weight_rounded(int64_t M, int64_t N, int64_t K, int group, int dtype, size_t workspace_bytes);
int amct_gemm_w8a16(const void* x, const void* smooth, const int8_t* wq, const void* scales, int scale_dtype,
                    const int8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K,
                    int group, int dtype, amct_stream_t stream);
/* The same with a workspace (may be null): amct_gemm_w8a16_workspace_bytes(M, N, K, group, smooth != null) bytes the
 * caller lends, 16-byte aligned, contents irrelevant before and after the call.  From M = 256 on the weight is then
 * dequantised once into it (N * K * 2 bytes; the smoothed activations follow), and the product runs as a plain 16-bit
 * GEMM on the 256x256 tiles of the W8A8 kernel: the same arithmetic as the tile kernel without workspace (the
 * dequantised weight rounded to dtype, fp32 accumulation), about three times as fast.  For fewer rows (M > 16) with smooth
 * the query asks for M * K * 2 bytes: the multiply is then done once up front and the fast tile kernels apply (K a
 * multiple of 256, groups a multiple of 64; they take precedence up to 384 rows, and up to 512 rows unless a last round
 * of 128x128 blocks would run half empty; for long rows on few column blocks with K split over blocks, whose fp32 partial sums follow the
 * activations in the workspace: S * M * N * 4 bytes more).  0 bytes are asked for otherwise; a null or smaller workspace
 * is never an error. */
size_t amct_gemm_w8a16_workspace_bytes(int64_t M, int64_t N, int64_t K, int group, int has_smooth);
int amct_gemm_w8a16_ws(const void* x, const void* smooth, const int8_t* wq, const void* scales, int scale_dtype,
                       const int8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                       int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream);

/* ---- GPTQ inner block ------------------------------------------------------------------------
 * The column loop of amct_pytorch/quantize_op/gptq_module.py:128-151 for one block of count <= 128 columns,
 * all rows in one launch.  For i = 0 .. count-1, per row n:
 *   wq = ((clamp(rne(w[n][i] / s + z), qmin, qmax)) - z) * s;  err = (w[n][i] - wq) / hinv[i][i];
 *   w[n][j] -= err * hinv[i][j] for j = i .. count-1;  err_out[n][i] = err
 * with s = scale[n * scale_stride + gidx[i]], z = offset[same index] (offset null: symmetric).  scale_stride = 0
 * shares one row of factors among all rows (per-tensor); gidx[i] is the factor column of block column i
 * (perm[i1 + i] / group_size for per-group factors, 0 otherwise).  w points at the block's first column inside
 * the column-sorted fp32 weight (row stride ld_w), hinv at the block's diagonal element (row stride ld_h);
 * err_out [rows, count] (row stride ld_e) feeds the reference's trailing update
 * weight[:, i2:] -= err_block @ hinv[i1:i2, i2:], which stays a library GEMM. */
int amct_gptq_block(float* w, int64_t ld_w, float* err_out, int64_t ld_e, const float* hinv, int64_t ld_h,
                    const float* scale, const int32_t* offset, int64_t scale_stride, const int32_t* gidx,
                    int64_t rows, int count, int qmin, int qmax, amct_stream_t stream);

/* ---- GPTQ Hessian accumulation --------------------------------------------------------------
 * The update of amct_pytorch/quantize_op/gptq_module.py:176-181 for 16-bit calibration activations:
 *   hessian *= n / (n + b);  x = sqrt(2 / (n + b)) * x.float();  hessian += x.t() @ x      (x [tokens, cols])
 * as hessian <- beta * hessian + alpha * (x^T x) with beta = n / (n + b), alpha = 2 / (n + b): the products of two
 * 16-bit values are exact in fp32 and are summed in fp32 on the matrix pipe, alpha is applied to the sum (the reference
 * scales every element by sqrt(alpha) first: the results agree to fp32 rounding, not bit for bit).  hessian fp32
 * [cols, cols], symmetric: only its lower triangle is read, both triangles are written; beta == 0 reads nothing, so the
 * first call may pass uninitialised memory.  x of dtype AMCT_BF16 or AMCT_F16 (fp32 activations: AMCT_E_UNSUPPORTED,
 * the caller keeps its fp32 product).  workspace: amct_hessian_update_workspace_bytes(tokens, cols) bytes, 16-byte
 * aligned (x transposed and padded to whole tiles), contents irrelevant before and after the call. */
size_t amct_hessian_update_workspace_bytes(int64_t tokens, int64_t cols);
int amct_hessian_update(float* hessian, const void* x, int64_t tokens, int64_t cols, float beta, float alpha,
                        int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream);

/* ---- interchange formats of the checkpoint converter ---------------------------------------
 * (amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py)
 * amct_fp8_block_dequant: weight_dequant :48-92.  w E4M3FN codes [rows, cols], scale fp32
 *   [ceil(rows/block), ceil(cols/block)]; out[r][c] = out_dtype(fp32(w[r][c]) * scale[r/block][c/block]).
 * amct_pack_int4_pairs_n: pack_4bit :110-127.  x int8 [n, k] holding int4 values, n even;
 *   y int8 [n/2, k] = (x[2i+1][k] << 4) | (x[2i][k] & 15): two output channels per byte.
 * amct_scale_f32_to_u64: scale_fp32_to_u64 :95-107.  out[i] = the bits of s[i] in the low 32 bits, 0 above. */
int amct_fp8_block_dequant(const uint8_t* w, const float* scale, void* out, int64_t rows, int64_t cols,
                           int block, int out_dtype, amct_stream_t stream);
int amct_pack_int4_pairs_n(const int8_t* x, int8_t* y, int64_t n, int64_t k, amct_stream_t stream);
int amct_scale_f32_to_u64(const float* s, uint64_t* out, int64_t n, amct_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AMCT_HIP_H */
