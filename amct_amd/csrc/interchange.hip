// Interchange formats of the checkpoint converter (amct_pytorch/experimental/quantization/DeepSeekV3.2/deploy.py):
//   fp8 (E4M3FN) weights with one fp32 scale per 128 x 128 block -> bf16 / fp16 / fp32     weight_dequant  :48-92
//   int4 codes in int8, two output channels per byte                                     pack_4bit       :110-127
//   fp32 scales widened to 64-bit words (scale bits in the low half)                     scale_fp32_to_u64 :95-107
// All three are streaming kernels: 16 bytes per lane and access, unconditional (clamped) loads.
#include "amct_common.h"

namespace amct {

typedef float v2f __attribute__((ext_vector_type(2)));

// E4M3FN code -> fp32 (0x7F / 0xFF are NaN, no infinities)
AMCT_DEV float e4m3fn_to_f32(uint32_t c) {
    const uint32_t a = c & 0x7Fu;
    float f;
    if (a == 0x7Fu) f = __uint_as_float(0x7FC00000u);
    else if (a >= 8u) f = __uint_as_float((a << 20) + (120u << 23));
    else f = (float)a * 0.001953125f;                          // subnormals: a * 2^-9
    return (c & 0x80u) ? -f : f;
}

// out = dtype(fp32(w) * scale[row / B][col / B]).  One lane = the codes of one 16-byte output vector (4 for fp32, 8 for
// the 16-bit types), so that every store instruction of a wave writes 1 KiB of consecutive bytes; 8 rows in flight per
// lane.  (With 16 codes and up to four strided 16-byte stores per lane the kernel wrote partial lines: 93 us for
// W[7168,4096] to fp32.)  Codes are decoded two per instruction by the hardware conversion (v_cvt_pk_f32_fp8, exact).
template <int ODT>
__global__ __launch_bounds__(kBlock) void fp8_block_dequant_k(const uint8_t* w, const float* scale, void* out, int64_t rows,
                                                              int64_t cols, int block, int64_t scale_cols) {
    constexpr int VEC = Tr<ODT>::VEC;
    constexpr int U = 8;
    const int64_t vpr = cols / VEC;
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;   // vector inside the row
    const int64_t vc = v < vpr ? v : vpr - 1;                       // clamped: loads are unconditional
    const int64_t sc_col = (vc * VEC) / block;
    for (int64_t r0 = (int64_t)blockIdx.y * U; r0 < rows; r0 += (int64_t)gridDim.y * U) {
        uint32_t raw[U][VEC / 4];
        float sc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t r = r0 + u < rows ? r0 + u : rows - 1;
            const uint32_t* src = reinterpret_cast<const uint32_t*>(w + r * cols + vc * VEC);
#pragma unroll
            for (int d = 0; d < VEC / 4; ++d) raw[u][d] = __builtin_nontemporal_load(src + d);
            sc[u] = scale[(r / block) * scale_cols + sc_col];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float x[VEC];
#pragma unroll
            for (int d = 0; d < VEC / 4; ++d) {
                const v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[u][d], false);
                const v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[u][d], true);
                x[4 * d] = lo.x * sc[u];
                x[4 * d + 1] = lo.y * sc[u];
                x[4 * d + 2] = hi.x * sc[u];
                x[4 * d + 3] = hi.y * sc[u];
            }
            if (v < vpr && r0 + u < rows)
                stg16_nt(reinterpret_cast<char*>(out) + ((r0 + u) * cols + v * VEC) * Tr<ODT>::BYTES, pack16<ODT>(x));
        }
    }
}

template <int ODT>
__global__ __launch_bounds__(kBlock) void fp8_block_dequant_general_k(const uint8_t* w, const float* scale, void* out,
                                                                      int64_t rows, int64_t cols, int block,
                                                                      int64_t scale_cols) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= rows * cols) return;
    const int64_t row = i / cols, col = i - row * cols;
    store_scalar<ODT>(out, i, e4m3fn_to_f32(w[i]) * scale[(row / block) * scale_cols + col / block]);
}

// y[n2][k] = (x[2 n2 + 1][k] << 4) | (x[2 n2][k] & 15)
__global__ __launch_bounds__(kBlock) void pack_pairs_n_k(const int8_t* x, int8_t* y, int64_t k_bytes, int64_t nvec,
                                                         int64_t vec_per_row) {
    const int64_t gv = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t g = gv < nvec ? gv : nvec - 1;
    const int64_t row2 = g / vec_per_row, kv = g - row2 * vec_per_row;
    const uint4 lo = ldg16_nt(x + (2 * row2) * k_bytes + kv * 16);
    const uint4 hi = ldg16_nt(x + (2 * row2 + 1) * k_bytes + kv * 16);
    uint4 o;
    o.x = (lo.x & 0x0F0F0F0Fu) | ((hi.x << 4) & 0xF0F0F0F0u);
    o.y = (lo.y & 0x0F0F0F0Fu) | ((hi.y << 4) & 0xF0F0F0F0u);
    o.z = (lo.z & 0x0F0F0F0Fu) | ((hi.z << 4) & 0xF0F0F0F0u);
    o.w = (lo.w & 0x0F0F0F0Fu) | ((hi.w << 4) & 0xF0F0F0F0u);
    if (gv < nvec) stg16_nt(y + row2 * k_bytes + kv * 16, o);
}

__global__ __launch_bounds__(kBlock) void pack_pairs_n_general_k(const int8_t* x, int8_t* y, int64_t n2, int64_t k) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n2 * k) return;
    const int64_t row2 = i / k, col = i - row2 * k;
    const uint32_t lo = (uint8_t)x[(2 * row2) * k + col], hi = (uint8_t)x[(2 * row2 + 1) * k + col];
    y[i] = (int8_t)((lo & 15u) | ((hi << 4) & 0xF0u));
}

__global__ __launch_bounds__(kBlock) void widen_scale_k(const uint32_t* s, uint2* out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = make_uint2(s[i], 0u);
}

}  // namespace amct

using namespace amct;

extern "C" int amct_fp8_block_dequant(const uint8_t* w, const float* scale, void* out, int64_t rows, int64_t cols,
                                      int block, int out_dtype, amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || block <= 0) return AMCT_E_BADARG;
    if (out_dtype != AMCT_F32 && out_dtype != AMCT_F16 && out_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (rows == 0) return AMCT_OK;
    if (!w || !scale || !out) return AMCT_E_BADARG;
    hipStream_t st = (hipStream_t)stream;
    const int64_t scale_cols = (cols + block - 1) / block;
    const bool vec_ok = cols % 8 == 0 && block % 8 == 0 && aligned16(w) && aligned16(out);
#define AMCT_FD(DT)                                                                                               \
    {                                                                                                             \
        if (vec_ok) {                                                                                             \
            const int64_t vpr = cols / Tr<DT>::VEC;                                                               \
            const int64_t nbx = (vpr + kBlock - 1) / kBlock;                                                      \
            int64_t nby = (rows + 7) / 8;                                                                         \
            if (nby > 65535) nby = 65535;                                                                         \
            if (nbx > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;                                                      \
            hipLaunchKernelGGL((fp8_block_dequant_k<DT>), dim3((unsigned)nbx, (unsigned)nby), dim3(kBlock), 0, st, w, scale, \
                               out, rows, cols, block, scale_cols);                                               \
        } else {                                                                                                  \
            const int64_t nb = (rows * cols + kBlock - 1) / kBlock;                                               \
            if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;                                                       \
            hipLaunchKernelGGL((fp8_block_dequant_general_k<DT>), dim3((unsigned)nb), dim3(kBlock), 0, st, w, scale, \
                               out, rows, cols, block, scale_cols);                                               \
        }                                                                                                         \
    }
    switch (out_dtype) {
        case AMCT_F32: AMCT_FD(AMCT_F32) break;
        case AMCT_F16: AMCT_FD(AMCT_F16) break;
        default: AMCT_FD(AMCT_BF16) break;
    }
#undef AMCT_FD
    return hip_status();
}

extern "C" int amct_pack_int4_pairs_n(const int8_t* x, int8_t* y, int64_t n, int64_t k, amct_stream_t stream) {
    if (n < 0 || k < 0) return AMCT_E_BADARG;
    if (n % 2 != 0) return AMCT_E_ALIGN;
    if (n * k == 0) return AMCT_OK;
    if (!x || !y) return AMCT_E_BADARG;
    hipStream_t st = (hipStream_t)stream;
    if (k % 16 == 0 && aligned16(x) && aligned16(y)) {
        const int64_t vec_per_row = k / 16, nvec = (n / 2) * vec_per_row;
        const int64_t nb = (nvec + kBlock - 1) / kBlock;
        if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
        hipLaunchKernelGGL(pack_pairs_n_k, dim3((unsigned)nb), dim3(kBlock), 0, st, x, y, k, nvec, vec_per_row);
    } else {
        const int64_t nb = ((n / 2) * k + kBlock - 1) / kBlock;
        if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
        hipLaunchKernelGGL(pack_pairs_n_general_k, dim3((unsigned)nb), dim3(kBlock), 0, st, x, y, n / 2, k);
    }
    return hip_status();
}

extern "C" int amct_scale_f32_to_u64(const float* s, uint64_t* out, int64_t n, amct_stream_t stream) {
    if (n < 0) return AMCT_E_BADARG;
    if (n == 0) return AMCT_OK;
    if (!s || !out) return AMCT_E_BADARG;
    const int64_t nb = (n + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(widen_scale_k, dim3((unsigned)nb), dim3(kBlock), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint32_t*>(s), reinterpret_cast<uint2*>(out), n);
    return hip_status();
}
