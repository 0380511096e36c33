// K7: W4A16 Linear.  out[m,n] = bf16( sum_k x'[m,k] * wdq[n,k] + bias[n] ), fp32 accumulate,
//   x'  = bf16(x * smooth[k])                         (weight_npu_quant_module.py:113-114)
//   wdq = bf16((u[n,k] - zero[n,k/g]) * scale[n,k/g]) (the operator called at :116-117)
// wq holds u = code + 8 as nibbles, even k in the low nibble.
#include "amct_common.h"

namespace amct {

struct W4A16Args {
    const uint16_t* x;
    const uint16_t* smooth;
    const uint8_t* wq;
    const void* scales;
    const uint8_t* zeros;
    const float* bias;
    uint16_t* out;
    int64_t M, N, K;
    int group;
    int scale_dtype;
};

AMCT_DEV float load_scale(const W4A16Args& a, int64_t i) {
    const uint16_t h = reinterpret_cast<const uint16_t*>(a.scales)[i];
    return a.scale_dtype == AMCT_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}

// general kernel: one output per thread, sequential fp32 accumulation over k
__global__ __launch_bounds__(kBlock) void w4a16_general(W4A16Args a) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= a.M * a.N) return;
    const int64_t m = idx / a.N, n = idx - m * a.N;
    const int64_t G = a.K / a.group;
    float acc = 0.f;
    for (int64_t k = 0; k < a.K; ++k) {
        float xv = bf16_bits_to_f32(a.x[m * a.K + k]);
        if (a.smooth) xv = round_to<AMCT_BF16>(xv * bf16_bits_to_f32(a.smooth[k]));
        const uint32_t byte = a.wq[n * (a.K / 2) + k / 2];
        const float u = (float)((k & 1) ? (byte >> 4) : (byte & 0xFu));
        const int64_t gi = n * G + k / a.group;
        const float w = round_to<AMCT_BF16>((u - (float)a.zeros[gi]) * load_scale(a, gi));
        acc = acc + xv * w;
    }
    if (a.bias) acc = acc + a.bias[n];
    a.out[m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc);
}

}  // namespace amct

using namespace amct;

extern "C" int amct_gemm_w4a16(const void* x, const void* smooth, const uint8_t* wq, const void* scales,
                               int scale_dtype, const uint8_t* zeros, const float* bias, void* out, int64_t M,
                               int64_t N, int64_t K, int group, int dtype, amct_stream_t stream) {
    if (!x || !wq || !scales || !zeros || !out || M < 0 || N <= 0 || K <= 0 || group <= 0) return AMCT_E_BADARG;
    if (scale_dtype != AMCT_F16 && scale_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16) return AMCT_E_UNSUPPORTED;
    if (K % group != 0 || K % 2 != 0) return AMCT_E_ALIGN;
    if (M == 0) return AMCT_OK;
    W4A16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group, scale_dtype};
    hipStream_t st = (hipStream_t)stream;
    const int64_t nb = (M * N + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(w4a16_general, dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    return hip_status();
}
