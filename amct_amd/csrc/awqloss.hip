// Loss of one AWQ grid point: mean((y - yhat)^4) over all elements of two tensors of one dtype.
// Replaces the expression of amct_pytorch/algorithm/awq.py:96 `(ori_out - quant_out).float().pow(4).mean()`,
// which runs as four kernels and seven passes over the data, by one pass that reads both tensors once.
// The difference is rounded to the tensors' dtype before it is widened, as the reference's subtraction does;
// d^4 is (d*d)*(d*d) in fp32.  The sum is deterministic: a fixed number of blocks, each a fixed partition of the
// elements, per-block partials folded in a fixed order by one block (pass 2), which also divides by n.
// The order of summation differs from torch's, so results agree to fp32 rounding of the sum, not bit for bit.
#include "amct_common.h"

namespace amct {

constexpr int kLossBlocks = 1024;      // partials (fixed, so the summation order does not depend on the device)
constexpr int kLossUnroll = 4;         // 16-byte vectors of each tensor in flight per lane

template <int DT> AMCT_DEV float loss_elem(const void* p, int64_t i) {
    if constexpr (DT == AMCT_F32) return reinterpret_cast<const float*>(p)[i];
    else if constexpr (DT == AMCT_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
    else return f16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
}

template <int DT>
__global__ __launch_bounds__(kBlock) void awq_loss_partial_k(const void* y, const void* yhat, int64_t n, float* partial) {
    constexpr int VEC = Tr<DT>::VEC;
    __shared__ float red[kBlock / 64];
    const int tid = threadIdx.x;
    const int64_t nvec = n / VEC;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    float s[kLossUnroll];
#pragma unroll
    for (int u = 0; u < kLossUnroll; ++u) s[u] = 0.f;
    const char* py = reinterpret_cast<const char*>(y);
    const char* ph = reinterpret_cast<const char*>(yhat);
    // vector v of the tensors belongs to lane v % stride; a lane keeps kLossUnroll running sums (vector u of its
    // iteration goes to sum u), so the partition and the order are fixed by n alone
    for (int64_t v0 = (int64_t)blockIdx.x * kBlock + tid; v0 < nvec; v0 += stride * kLossUnroll) {
        uint4 ra[kLossUnroll], rb[kLossUnroll];
#pragma unroll
        for (int u = 0; u < kLossUnroll; ++u) {
            const int64_t v = v0 + u * stride;
            const int64_t vc = v < nvec ? v : nvec - 1;              // unconditional loads, clamped
            ra[u] = ldg16_nt(py + vc * 16);
            rb[u] = ldg16_nt(ph + vc * 16);
        }
#pragma unroll
        for (int u = 0; u < kLossUnroll; ++u) {
            if (v0 + u * stride < nvec) {
                float a[VEC], b[VEC];
                unpack16<DT>(ra[u], a);
                unpack16<DT>(rb[u], b);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float d = round_to<DT>(a[j] - b[j]);
                    const float d2 = d * d;
                    s[u] = s[u] + d2 * d2;
                }
            }
        }
    }
    // the n % VEC elements behind the last whole vector: lane 0 of block 0
    if (blockIdx.x == 0 && tid == 0) {
        for (int64_t i = nvec * VEC; i < n; ++i) {
            const float d = round_to<DT>(loss_elem<DT>(y, i) - loss_elem<DT>(yhat, i));
            const float d2 = d * d;
            s[0] = s[0] + d2 * d2;
        }
    }
    float t = (s[0] + s[1]) + (s[2] + s[3]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t = t + __shfl_xor(t, off, 64);
    if ((tid & 63) == 0) red[tid >> 6] = t;
    __syncthreads();
    if (tid == 0) {
        float b = red[0];
#pragma unroll
        for (int w = 1; w < kBlock / 64; ++w) b = b + red[w];
        partial[blockIdx.x] = b;
    }
}

// one block: lane l folds partials l, l + 256, ... in order, then the lanes meet; result / n
__global__ __launch_bounds__(kBlock) void awq_loss_final_k(const float* partial, int nparts, int64_t n, float* loss) {
    __shared__ float red[kBlock / 64];
    const int tid = threadIdx.x;
    float t = 0.f;
    for (int i = tid; i < nparts; i += kBlock) t = t + partial[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t = t + __shfl_xor(t, off, 64);
    if ((tid & 63) == 0) red[tid >> 6] = t;
    __syncthreads();
    if (tid == 0) {
        float b = red[0];
#pragma unroll
        for (int w = 1; w < kBlock / 64; ++w) b = b + red[w];
        loss[0] = b / (float)n;
    }
}

}  // namespace amct

using namespace amct;

extern "C" size_t amct_awq_loss_workspace_bytes(void) { return (size_t)kLossBlocks * sizeof(float); }

extern "C" int amct_awq_loss(const void* y, const void* yhat, int64_t n, int dtype, float* loss, void* workspace,
                             size_t workspace_bytes, amct_stream_t stream) {
    if (n < 0 || !loss) return AMCT_E_BADARG;
    if (dtype != AMCT_F32 && dtype != AMCT_F16 && dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (n != 0 && (!y || !yhat)) return AMCT_E_BADARG;
    if (!workspace || workspace_bytes < amct_awq_loss_workspace_bytes() || ((uintptr_t)workspace & 3)) return AMCT_E_BADARG;
    if (n != 0 && (!aligned16(y) || !aligned16(yhat))) return AMCT_E_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    float* partial = reinterpret_cast<float*>(workspace);
    // n == 0: the mean of nothing is 0 / 0 = NaN, as torch's; the partial pass then writes zeros
    const int vec = dtype == AMCT_F32 ? 4 : 8;
    int64_t blocks = (n / vec + (int64_t)kBlock * kLossUnroll - 1) / ((int64_t)kBlock * kLossUnroll);
    if (blocks < 1) blocks = 1;
    if (blocks > kLossBlocks) blocks = kLossBlocks;
    if (dtype == AMCT_F32) hipLaunchKernelGGL((awq_loss_partial_k<AMCT_F32>), dim3((unsigned)blocks), dim3(kBlock), 0, st, y, yhat, n, partial);
    else if (dtype == AMCT_F16) hipLaunchKernelGGL((awq_loss_partial_k<AMCT_F16>), dim3((unsigned)blocks), dim3(kBlock), 0, st, y, yhat, n, partial);
    else hipLaunchKernelGGL((awq_loss_partial_k<AMCT_BF16>), dim3((unsigned)blocks), dim3(kBlock), 0, st, y, yhat, n, partial);
    hipLaunchKernelGGL(awq_loss_final_k, dim3(1), dim3(kBlock), 0, st, partial, (int)blocks, n, loss);
    return hip_status();
}
