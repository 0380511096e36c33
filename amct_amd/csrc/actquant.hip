// K3: activation quantisation to int8.
//   dynamic per-token: row min/max -> symmetric scale -> codes, one read of x
//     (statistics as amct_pytorch/quantize_op/minmax_module.py:96-105, factors as
//      amct_pytorch/quantize_op/utils.py:75-108, codes as amct_pytorch/utils/quant_util.py:56-73)
//   static: q = sat(rne(x * scale + zero_point)), the operator called at
//     amct_pytorch/deploy_op/npu_quantization_linear.py:98-99.
#include <type_traits>

#include "amct_common.h"

namespace amct {

AMCT_DEV uint32_t pack4_i8(const float* q) {
    return ((uint32_t)(int)q[0] & 0xFFu) | (((uint32_t)(int)q[1] & 0xFFu) << 8) | (((uint32_t)(int)q[2] & 0xFFu) << 16) |
           (((uint32_t)(int)q[3] & 0xFFu) << 24);
}

// one block per row, each lane caches NV vectors (K <= 256 * NV * VEC)
template <int DT, int NV>
__global__ __launch_bounds__(kBlock) void act_quant_token(const void* x, const void* smooth, int8_t* q, float* scale,
                                                          int64_t K, int mode) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    __shared__ float sm[2][kBlock / kWave];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int S = (int)(K / VEC);
    const float inf = __builtin_huge_valf();
    float v[NV][VEC];
    uint4 raw[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int vi = (i * kBlock + tid < S) ? i * kBlock + tid : S - 1;       // clamped: unconditional load
        raw[i] = ldg16_nt(reinterpret_cast<const char*>(x) + (row * K + (int64_t)vi * VEC) * BYTES);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) unpack16<DT>(raw[i], v[i]);
    if (smooth) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int vi = (i * kBlock + tid < S) ? i * kBlock + tid : S - 1;
            float c[VEC];
            unpack16<DT>(ldg16(reinterpret_cast<const char*>(smooth) + (int64_t)vi * VEC * BYTES), c);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[i][j] = round_to<DT>(v[i][j] * c[j]);
        }
    }
    float mx = -inf, mn = inf;
#pragma unroll
    for (int i = 0; i < NV; ++i) {                       // clamped duplicates cannot change a min/max
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            mx = fmax_nan(mx, v[i][j]);
            mn = fmin_nan(mn, v[i][j]);
        }
    }
    team_minmax<kWave>(mn, mx);
    if ((tid & (kWave - 1)) == 0) {
        sm[0][tid / kWave] = mn;
        sm[1][tid / kWave] = mx;
    }
    __syncthreads();
#pragma unroll
    for (int wv = 0; wv < kBlock / kWave; ++wv) {
        mn = fmin_nan(mn, sm[0][wv]);
        mx = fmax_nan(mx, sm[1][wv]);
    }
    float s;
    if (mode == 0) {
        s = make_factors<AMCT_F32>(mx, mn, 8, true, AMCT_SCOPE_AMCT).s;
    } else {
        // node.py:181-204: xmax = max(|min(amin,0)|, max(amax,0)); s = xmax / 127; s = 1 where xmax == 0
        const float hi = fmax_nan(mx, 0.f), lo = fmin_nan(mn, 0.f);
        const float amax = fmax_nan(__builtin_fabsf(lo), hi);
        s = amax / 127.0f;
        s = (amax == 0.f) ? 1.0f : s;
    }
    if (tid == 0) scale[row] = s;
    const Divisor dv = make_divisor(s);
    const uint32_t big = max(__float_as_uint(mx) & 0x7FFFFFFFu, __float_as_uint(mn) & 0x7FFFFFFFu);
    const bool fast = dv.fast && big < 0x5D800000u;      // uniform over the block
    auto emit = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int vi = i * kBlock + tid;
            float c[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) c[j] = quant_elem<DT, false, FAST>(v[i][j], dv, 0.f, false, -128.f, 127.f);
            if (vi < S) {
                uint32_t* p = reinterpret_cast<uint32_t*>(q + row * K + (int64_t)vi * VEC);
                if constexpr (VEC == 4) stg4_nt(p, pack4_i8(c));
                else stg8_nt(p, pack4_i8(c), pack4_i8(c + 4));
            }
        }
    };
    if (fast) emit(std::true_type{});
    else emit(std::false_type{});
}

// general: any K, scalar accesses, two passes over the row
template <int DT>
__global__ __launch_bounds__(kBlock) void act_quant_token_general(const void* x, const void* smooth, int8_t* q,
                                                                  float* scale, int64_t K, int mode) {
    __shared__ float sm[2][kBlock / kWave];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const float inf = __builtin_huge_valf();
    float mx = -inf, mn = inf;
    for (int64_t c = tid; c < K; c += kBlock) {
        float v = load_scalar<DT>(x, row * K + c);
        if (smooth) v = round_to<DT>(v * load_scalar<DT>(smooth, c));
        mx = fmax_nan(mx, v);
        mn = fmin_nan(mn, v);
    }
    team_minmax<kWave>(mn, mx);
    if ((tid & (kWave - 1)) == 0) {
        sm[0][tid / kWave] = mn;
        sm[1][tid / kWave] = mx;
    }
    __syncthreads();
#pragma unroll
    for (int wv = 0; wv < kBlock / kWave; ++wv) {
        mn = fmin_nan(mn, sm[0][wv]);
        mx = fmax_nan(mx, sm[1][wv]);
    }
    float s;
    if (mode == 0) {
        s = make_factors<AMCT_F32>(mx, mn, 8, true, AMCT_SCOPE_AMCT).s;
    } else {
        const float hi = fmax_nan(mx, 0.f), lo = fmin_nan(mn, 0.f);
        const float amax = fmax_nan(__builtin_fabsf(lo), hi);
        s = amax / 127.0f;
        s = (amax == 0.f) ? 1.0f : s;
    }
    if (tid == 0) scale[row] = s;
    for (int64_t c = tid; c < K; c += kBlock) {
        float v = load_scalar<DT>(x, row * K + c);
        if (smooth) v = round_to<DT>(v * load_scalar<DT>(smooth, c));
        q[row * K + c] = (int8_t)(int)quant_elem<DT, false>(v, s, 0.f, false, -128.f, 127.f);
    }
}

// static quantise, scalar indexing: the fallback for shapes and pointers the vector kernel below does not take
template <int DT>
__global__ __launch_bounds__(kBlock) void quantize_static(const void* x, const void* smooth, const void* scales,
                                                          const void* zps, int8_t* q, int64_t M, int64_t K,
                                                          int64_t n_scales, int per_token) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < M * K; e += stride) {
        const int64_t m = e / K, k = e - m * K;
        const int64_t si = per_token ? m : (n_scales == 1 ? 0 : k);
        float v = load_scalar<DT>(x, e);
        if (smooth) v = round_to<DT>(v * load_scalar<DT>(smooth, k));
        float t = v * load_scalar<DT>(scales, si);
        if (zps) t = t + load_scalar<DT>(zps, si);
        t = __builtin_amdgcn_fmed3f(__builtin_rintf(t), -128.f, 127.f);
        q[e] = (int8_t)(int)t;
    }
}

// static quantise, 16 bytes of x per thread and iteration (K a multiple of the vector length, aligned pointers):
// same arithmetic per element as the scalar kernel above
template <int DT>
__global__ __launch_bounds__(kBlock) void quantize_static_vec(const void* x, const void* smooth, const void* scales,
                                                              const void* zps, int8_t* q, int64_t nvec, uint32_t S,
                                                              int64_t n_scales, int per_token) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int U = 4;                                           // vectors in flight per thread
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const bool small = nvec <= 0xFFFFFFFFll;
    for (int64_t v0 = (int64_t)blockIdx.x * kBlock + threadIdx.x; v0 < nvec; v0 += stride * U) {
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t v = v0 + u * stride;
            raw[u] = ldg16_nt(reinterpret_cast<const char*>(x) + (v < nvec ? v : nvec - 1) * 16);   // clamped, unconditional
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t v = v0 + u * stride;
            if (v >= nvec) break;
            const int64_t m = small ? (int64_t)((uint32_t)v / S) : v / S;      // row of this vector
            const uint32_t kv = (uint32_t)(v - m * S);                          // vector inside the row
            float xv[VEC], sc[VEC], zp[VEC];
            unpack16<DT>(raw[u], xv);
            if (smooth) {
                float c[VEC];
                unpack16<DT>(ldg16(reinterpret_cast<const char*>(smooth) + (int64_t)kv * 16), c);
#pragma unroll
                for (int j = 0; j < VEC; ++j) xv[j] = round_to<DT>(xv[j] * c[j]);
            }
            if (per_token || n_scales == 1) {
                const int64_t si = per_token ? m : 0;
                const float s1 = load_scalar<DT>(scales, si), z1 = zps ? load_scalar<DT>(zps, si) : 0.f;
#pragma unroll
                for (int j = 0; j < VEC; ++j) { sc[j] = s1; zp[j] = z1; }
            } else {
                unpack16<DT>(ldg16(reinterpret_cast<const char*>(scales) + (int64_t)kv * 16), sc);
                if (zps) unpack16<DT>(ldg16(reinterpret_cast<const char*>(zps) + (int64_t)kv * 16), zp);
            }
            uint32_t out[VEC / 4];
#pragma unroll
            for (int wd = 0; wd < VEC / 4; ++wd) {
                out[wd] = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    float t = xv[4 * wd + b] * sc[4 * wd + b];
                    if (zps) t = t + zp[4 * wd + b];
                    t = __builtin_amdgcn_fmed3f(__builtin_rintf(t), -128.f, 127.f);
                    out[wd] |= ((uint32_t)(int)t & 0xFFu) << (8 * b);
                }
            }
            if constexpr (VEC == 8) stg8_nt(q + v * 8, out[0], out[1]);
            else *reinterpret_cast<uint32_t*>(q + v * 4) = out[0];
        }
    }
}

template <int DT>
static int run_token(const void* x, const void* smooth, int8_t* q, float* scale, int64_t M, int64_t K, int mode,
                     hipStream_t st) {
    constexpr int VEC = Tr<DT>::VEC;
    const bool vec_ok = K % VEC == 0 && aligned16(x) && (!smooth || aligned16(smooth)) &&
                        (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
    const int64_t S = K / VEC;
    const dim3 grid((unsigned)M), block(kBlock);
    if (vec_ok && S <= kBlock) hipLaunchKernelGGL((act_quant_token<DT, 1>), grid, block, 0, st, x, smooth, q, scale, K, mode);
    else if (vec_ok && S <= 2 * kBlock) hipLaunchKernelGGL((act_quant_token<DT, 2>), grid, block, 0, st, x, smooth, q, scale, K, mode);
    else if (vec_ok && S <= 4 * kBlock) hipLaunchKernelGGL((act_quant_token<DT, 4>), grid, block, 0, st, x, smooth, q, scale, K, mode);
    else if (vec_ok && S <= 8 * kBlock) hipLaunchKernelGGL((act_quant_token<DT, 8>), grid, block, 0, st, x, smooth, q, scale, K, mode);
    else if (vec_ok && S <= 16 * kBlock) hipLaunchKernelGGL((act_quant_token<DT, 16>), grid, block, 0, st, x, smooth, q, scale, K, mode);   // rows of up to 32768 16-bit elements
    else hipLaunchKernelGGL((act_quant_token_general<DT>), grid, block, 0, st, x, smooth, q, scale, K, mode);
    return hip_status();
}

}  // namespace amct

using namespace amct;

extern "C" int amct_act_quant_per_token_int8(const void* x, const void* smooth, int8_t* q, float* scale, int64_t M,
                                             int64_t K, int mode, int dtype, amct_stream_t stream) {
    if (M < 0 || K <= 0 || (mode != 0 && mode != 1)) return AMCT_E_BADARG;
    if (M == 0) return AMCT_OK;                                   // nothing is read: null pointers are fine
    if (!x || !q || !scale) return AMCT_E_BADARG;
    if (M > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case AMCT_F32: return run_token<AMCT_F32>(x, smooth, q, scale, M, K, mode, st);
        case AMCT_F16: return run_token<AMCT_F16>(x, smooth, q, scale, M, K, mode, st);
        case AMCT_BF16: return run_token<AMCT_BF16>(x, smooth, q, scale, M, K, mode, st);
        default: return AMCT_E_BADARG;
    }
}

extern "C" int amct_quantize(const void* x, const void* smooth, const void* scales, const void* zero_points, int8_t* q,
                             int64_t M, int64_t K, int64_t n_scales, int per_token, int dtype, amct_stream_t stream) {
    if (M < 0 || K <= 0) return AMCT_E_BADARG;
    if (per_token ? (n_scales != M) : (n_scales != 1 && n_scales != K)) return AMCT_E_BADARG;
    if (M == 0) return AMCT_OK;
    if (!x || !scales || !q) return AMCT_E_BADARG;
    hipStream_t st = (hipStream_t)stream;
    {
        const int vec = dtype == AMCT_F32 ? 4 : 8;
        const bool table = !per_token && n_scales != 1;            // one scale per column: read as vectors too
        if (K % vec == 0 && K / vec <= 0x7FFFFFFF && aligned16(x) && (!smooth || aligned16(smooth)) &&
            (!table || (aligned16(scales) && (!zero_points || aligned16(zero_points)))) &&
            (reinterpret_cast<uintptr_t>(q) & 7u) == 0) {
            const int64_t nvec = M * (K / vec);
            int64_t nbv = (nvec + kBlock * 4 - 1) / (kBlock * 4);
            if (nbv > 16384) nbv = 16384;
            const dim3 gridv((unsigned)nbv), blockv(kBlock);
            const uint32_t S = (uint32_t)(K / vec);
            switch (dtype) {
                case AMCT_F32: hipLaunchKernelGGL((quantize_static_vec<AMCT_F32>), gridv, blockv, 0, st, x, smooth, scales, zero_points, q, nvec, S, n_scales, per_token); return hip_status();
                case AMCT_F16: hipLaunchKernelGGL((quantize_static_vec<AMCT_F16>), gridv, blockv, 0, st, x, smooth, scales, zero_points, q, nvec, S, n_scales, per_token); return hip_status();
                case AMCT_BF16: hipLaunchKernelGGL((quantize_static_vec<AMCT_BF16>), gridv, blockv, 0, st, x, smooth, scales, zero_points, q, nvec, S, n_scales, per_token); return hip_status();
                default: return AMCT_E_BADARG;
            }
        }
    }
    int64_t nb = (M * K + kBlock - 1) / kBlock;
    if (nb > 65536) nb = 65536;
    const dim3 grid((unsigned)nb), block(kBlock);
    switch (dtype) {
        case AMCT_F32: hipLaunchKernelGGL((quantize_static<AMCT_F32>), grid, block, 0, st, x, smooth, scales, zero_points, q, M, K, n_scales, per_token); break;
        case AMCT_F16: hipLaunchKernelGGL((quantize_static<AMCT_F16>), grid, block, 0, st, x, smooth, scales, zero_points, q, M, K, n_scales, per_token); break;
        case AMCT_BF16: hipLaunchKernelGGL((quantize_static<AMCT_BF16>), grid, block, 0, st, x, smooth, scales, zero_points, q, M, K, n_scales, per_token); break;
        default: return AMCT_E_BADARG;
    }
    return hip_status();
}
