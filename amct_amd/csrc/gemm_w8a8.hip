// K6: W8A8 Linear.  out[m,n] = cast(fp32(sum_k xq[m,k]*wq[n,k] + ibias[n]) * s_ch[n] * s_tok[m] + fbias[n])
// Reference call site: amct_pytorch/deploy_op/npu_quantization_linear.py:100-102.
#include "amct_common.h"

namespace amct {

struct W8A8Args {
    const int8_t* xq;
    const int8_t* wq;
    const float* s_tok;
    const float* s_ch;
    const void* bias;
    void* out;
    int32_t* acc_out;
    int64_t M, N, K;
    int bias_kind;
    int out_dtype;
};

AMCT_DEV void w8a8_epilogue(const W8A8Args& a, int64_t m, int64_t n, int32_t acc) {
    if (a.bias_kind == 1) acc += reinterpret_cast<const int32_t*>(a.bias)[n];
    if (a.acc_out) a.acc_out[m * a.N + n] = acc;
    float f = (float)acc;
    f = f * a.s_ch[n];
    if (a.s_tok) f = f * a.s_tok[m];
    if (a.bias_kind == 2) f = f + reinterpret_cast<const float*>(a.bias)[n];
    const int64_t o = m * a.N + n;
    if (a.out_dtype == AMCT_BF16) store_scalar<AMCT_BF16>(a.out, o, f);
    else if (a.out_dtype == AMCT_F16) store_scalar<AMCT_F16>(a.out, o, f);
    else store_scalar<AMCT_F32>(a.out, o, f);
}

// general kernel: any M, N, K; one output per thread.  Used for shapes the tiled kernel
// does not cover.
__global__ __launch_bounds__(kBlock) void w8a8_general(W8A8Args a) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= a.M * a.N) return;
    const int64_t m = idx / a.N, n = idx - m * a.N;
    const int8_t* xr = a.xq + m * a.K;
    const int8_t* wr = a.wq + n * a.K;
    int32_t acc = 0;
    for (int64_t k = 0; k < a.K; ++k) acc += (int32_t)xr[k] * (int32_t)wr[k];
    w8a8_epilogue(a, m, n, acc);
}

}  // namespace amct

using namespace amct;

extern "C" int amct_gemm_w8a8(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch,
                              const void* bias, int bias_kind, void* out, int32_t* acc_out, int64_t M, int64_t N,
                              int64_t K, int out_dtype, amct_stream_t stream) {
    if (!xq || !wq || !s_ch || !out || M < 0 || N <= 0 || K <= 0) return AMCT_E_BADARG;
    if (bias_kind < 0 || bias_kind > 2 || (bias_kind != 0 && !bias)) return AMCT_E_BADARG;
    if (out_dtype != AMCT_F32 && out_dtype != AMCT_F16 && out_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (M == 0) return AMCT_OK;
    W8A8Args a{xq, wq, s_tok, s_ch, bias_kind ? bias : nullptr, out, acc_out, M, N, K, bias_kind, out_dtype};
    hipStream_t st = (hipStream_t)stream;
    const int64_t nb = (M * N + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(w8a8_general, dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    return hip_status();
}
