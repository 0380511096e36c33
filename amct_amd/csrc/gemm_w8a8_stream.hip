// K6 for M <= 16 (decode): the int8 weight is the only large traffic (59 MB for W[14336,4096]) and the memory system
// delivers it fastest when all of it is requested at once, in whole 128-byte lines.  Every wave of the launch is
// resident at the same time and issues ALL of its weight loads before anything else waits; the activations
// (at most 16 rows) are staged once per block in LDS by loads issued just before, and the MFMAs
// (v_mfma_i32_16x16x64_i8) follow the weights as they land.
// A block owns CG groups of 16 output columns; KS waves per column group split K.  A load instruction fetches 8
// weight rows x one 128-byte line: lane l reads row l % 8 (the second instruction of a pair rows 8 .. 15) and one
// 16-byte chunk of the line; the two registers of a pair then swap halves by DPP so that lanes 0 .. 15 of every lane
// group hold 16 different rows, as the MFMA wants: the first register feeds the MFMA over bytes 0 .. 63 of the line
// (chunk g in lane group g), the second the one over bytes 64 .. 127.
// Integer accumulation is exact, so the split of K changes nothing: the result is the accumulator of the tile
// kernels, and the epilogue is theirs, operation for operation:
//   out = cast(fp32(acc + ibias[n]) * s_ch[n] * s_tok[m] + fbias[n]).
#include "amct_common.h"

namespace amct {

typedef int q4i __attribute__((ext_vector_type(4)));

struct StreamArgs8 {
    const int8_t* xq;
    const int8_t* wq;
    const float* s_tok;
    const float* s_ch;
    const void* bias;
    void* out;
    int32_t* acc_out;
    int M, N, K;
    int bias_kind;
    uint32_t kv_magic;                               // floor(2^32 / (K / 16)) + 1: v / (K / 16) == mulhi(v, magic)
    // XDT != 0: the activations arrive as 16-bit floats and are quantised while they are staged,
    // q = sat_int8(rne(x' * act_scale + act_zp)) with x' = dt(x * smooth): the static quantisation of the deploy module
    // (amct_pytorch/deploy_op/npu_quantization_linear.py:98-99) in the arithmetic of amct_quantize, element for element.
    // kv_magic then divides by K / 8 (16-byte vectors of 8 elements).
    const void* x16;
    const void* smooth;                              // [K] or null
    const void* act_scale;                           // [1] or [M] (per_token)
    const void* act_zp;                              // the same shape, or null
    int per_token;
};

// XJ: 16-byte activation vectors a thread stages (clamped duplicates beyond the tensor)
template <int ODT, int KS, int CG, int NL, int XJ, int XDT = 0>
__global__ __launch_bounds__(KS * CG * 64) void w8a8_stream(StreamArgs8 a) {
    static_assert(NL % 2 == 0, "the weight loads come in pairs");
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int NT = KS * CG * 64;
    constexpr int COLS = CG * 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cg = wave / KS, ks = wave % KS;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * COLS;
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M;
    const uint32_t xstride = K + 16;                 // 16 bytes of padding: the 16 rows of a fragment read spread over the banks

    // ---- staging loads of the activations -----------------------------------------------------------------------
    constexpr uint32_t XE = XDT ? 8 : 16;            // elements of a 16-byte staging vector
    const uint32_t KV = K / XE, n_xv = M * KV;
    uint4 xv[XJ];
    uint32_t xoff[XJ];
    float qs[XDT ? XJ : 1], qz[XDT ? XJ : 1];
    uint4 cvec = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        const uint32_t vc = v < n_xv ? v : n_xv - 1;
        const uint32_t row = __umulhi(vc, a.kv_magic);            // vc / KV
        xoff[j] = row * xstride + (vc - row * KV) * XE;
        if constexpr (XDT != 0) {
            xv[j] = ldg16(reinterpret_cast<const char*>(a.x16) + (size_t)vc * 16);
            const int64_t si = a.per_token ? row : 0;
            qs[j] = load_scalar<XDT>(a.act_scale, si);
            qz[j] = a.act_zp ? load_scalar<XDT>(a.act_zp, si) : 0.f;
            // NT is a multiple of K / 8: every vector of a thread lies in the same columns
            if (j == 0 && a.smooth) cvec = ldg16(reinterpret_cast<const char*>(a.smooth) + (size_t)(vc - row * KV) * 16);
        } else {
            xv[j] = ldg16(a.xq + (size_t)vc * 16);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- the whole weight stream of this wave -------------------------------------------------------------------
    const uint32_t kw = K / KS;                      // bytes of K of this wave: NL / 2 lines of 128
    const int ncol = n0 + cg * 16 + r16;
    const uint32_t oct = lane >> 3;
    const uint32_t chunk = (oct & 1) ? 4 + (oct >> 1) : (oct >> 1);
    const int rlo = n0 + cg * 16 + (lane & 7), rhi = rlo + 8;
    const int8_t* wlo = a.wq + (size_t)(rlo < a.N ? rlo : a.N - 1) * K + ks * kw + chunk * 16;
    const int8_t* whi = a.wq + (size_t)(rhi < a.N ? rhi : a.N - 1) * K + ks * kw + chunk * 16;
    // Blocks of 16 waves have 128 registers per lane: eight 16-bit activation vectors in flight with their factors (56)
    // and all of the weights (64) do not fit beside each other, so such a launch requests the second half of its lines
    // when the activations have gone to LDS (the first half is still arriving then).
    constexpr int FIRST = (XDT != 0 && XJ >= 8 && KS * CG == 16) ? NL / 2 : NL;
    static_assert(FIRST % 2 == 0, "whole pairs");
    u4v wv[NL];
#pragma unroll
    for (int i = 0; i < FIRST; i += 2) {
        wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wlo + (i / 2) * 128));
        wv[i + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(whi + (i / 2) * 128));
    }
    __builtin_amdgcn_sched_barrier(0);
    // the factors of this lane's column and rows, needed last
    const int nc = ncol < a.N ? ncol : a.N - 1;
    const float sc = a.s_ch[nc];
    const int32_t ib = a.bias_kind == 1 ? reinterpret_cast<const int32_t*>(a.bias)[nc] : 0;
    const float fb = a.bias_kind == 2 ? reinterpret_cast<const float*>(a.bias)[nc] : 0.f;
    float tok[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = 4 * g + r;
        tok[r] = a.s_tok ? a.s_tok[m < (int)M ? m : (int)M - 1] : 1.0f;
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- stage the activations (waits are in issue order: the weights stay in flight) ---------------------------
    if constexpr (XDT != 0) {
        float c[8];
        if (a.smooth) unpack16<XDT>(cvec, c);
#pragma unroll
        for (int j = 0; j < XJ; ++j) {
            float f[8];
            unpack16<XDT>(xv[j], f);
            if (a.smooth) {
#pragma unroll
                for (int e = 0; e < 8; ++e) f[e] = round_to<XDT>(f[e] * c[e]);
            }
            uint32_t o[2] = {0u, 0u};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = f[e] * qs[j];
                if (a.act_zp) t = t + qz[j];
                t = __builtin_amdgcn_fmed3f(__builtin_rintf(t), -128.f, 127.f);
                o[e >> 2] |= ((uint32_t)(int)t & 0xFFu) << (8 * (e & 3));
            }
            if (tid + NT * j < n_xv) *reinterpret_cast<uint2*>(lds + xoff[j]) = make_uint2(o[0], o[1]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < XJ; ++j) {
            if (tid + NT * j < n_xv) *reinterpret_cast<uint4*>(lds + xoff[j]) = xv[j];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = FIRST; i < NL; i += 2) {
        wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wlo + (i / 2) * 128));
        wv[i + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(whi + (i / 2) * 128));
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // ---- follow the weights as they land ------------------------------------------------------------------------
    q4i acc = {0, 0, 0, 0};
    const uint8_t* xlane = lds + (r16 < (int)M ? r16 : (int)M - 1) * xstride + ks * kw + g * 16;
#pragma unroll
    for (int i = 0; i < NL; i += 2) {
        const q4i fa0 = *reinterpret_cast<const q4i*>(xlane + (i / 2) * 128);
        const q4i fa1 = *reinterpret_cast<const q4i*>(xlane + (i / 2) * 128 + 64);
        q4i b0, b1;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int lo = (int)wv[i][d], hi = (int)wv[i + 1][d];
            // row_ror:8 inside each row of 16 lanes; bank_mask picks the lanes that take the rotated value
            b0[d] = __builtin_amdgcn_update_dpp(lo, hi, 0x128, 0xF, 0xC, false);
            b1[d] = __builtin_amdgcn_update_dpp(hi, lo, 0x128, 0xF, 0x3, false);
        }
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa0, b0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa1, b1, acc, 0, 0, 0);
    }

    // ---- add the KS partial sums of a column group, epilogue ----------------------------------------------------
    if constexpr (KS > 1) {
        __syncthreads();                              // every wave is done reading activations: their rows are reused
        int* red = reinterpret_cast<int*>(lds);
        if (ks > 0) *reinterpret_cast<q4i*>(red + (((ks - 1) * CG + cg) * 64 + lane) * 4) = acc;
        __syncthreads();
        if (ks == 0) {
#pragma unroll
            for (int w = 0; w < KS - 1; ++w) {
                const q4i o = *reinterpret_cast<const q4i*>(red + ((w * CG + cg) * 64 + lane) * 4);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] += o[r];
            }
        }
    }
    if (ks == 0 && ncol < a.N) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = 4 * g + r;
            if (m >= (int)M) continue;
            const int32_t t = acc[r] + ib;
            const size_t o = (size_t)m * a.N + ncol;
            if (a.acc_out) a.acc_out[o] = t;
            float f = (float)t * sc;
            if (a.s_tok) f = f * tok[r];
            if (a.bias_kind == 2) f = f + fb;
            if constexpr (ODT == AMCT_F32) reinterpret_cast<float*>(a.out)[o] = f;
            else if constexpr (ODT == AMCT_BF16) reinterpret_cast<uint16_t*>(a.out)[o] = (uint16_t)f32_to_bf16_bits(f);
            else reinterpret_cast<uint16_t*>(a.out)[o] = (uint16_t)f32_to_f16_bits(f);
        }
    }
}

template <int ODT, int KS, int CG, int NL, int XDT = 0>
static int stream8_launch_x(const StreamArgs8& a, size_t lds_bytes, hipStream_t st) {
    constexpr int NT = KS * CG * 64;
    const int n_xv = a.M * (a.K / (XDT ? 8 : 16));
    const int xj = (n_xv + NT - 1) / NT;
    const dim3 grid((unsigned)((a.N + CG * 16 - 1) / (CG * 16)));
#define AMCT_STREAM8_GO(XJ)                                                                                         \
    {                                                                                                               \
        auto kern = &w8a8_stream<ODT, KS, CG, NL, XJ, XDT>;                                                         \
        if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) { \
            (void)hipGetLastError();                                                                                \
            return AMCT_E_HIP;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, st, a);                                                 \
        return hip_status();                                                                                        \
    }
    if constexpr (XDT == 0) {
        if (xj <= 1) AMCT_STREAM8_GO(1)
    }
    if (xj <= 2) AMCT_STREAM8_GO(2)
    if (xj <= 4) AMCT_STREAM8_GO(4)
    if (xj <= 8) AMCT_STREAM8_GO(8)
#undef AMCT_STREAM8_GO
    return AMCT_E_UNSUPPORTED;
}

template <int ODT, int XDT = 0>
static int stream8_shape(const StreamArgs8& a, int cg, int nl, size_t lds_bytes, hipStream_t st) {
#define AMCT_STREAM8_SHAPE(CG_, NL_) \
    if (cg == CG_ && nl == NL_) return stream8_launch_x<ODT, 4, CG_, NL_, XDT>(a, lds_bytes, st);
    AMCT_STREAM8_SHAPE(4, 16)
    AMCT_STREAM8_SHAPE(2, 16)
    AMCT_STREAM8_SHAPE(4, 8)
    AMCT_STREAM8_SHAPE(2, 8)
    AMCT_STREAM8_SHAPE(4, 4)
    AMCT_STREAM8_SHAPE(2, 4)
#undef AMCT_STREAM8_SHAPE
    return AMCT_E_UNSUPPORTED;
}

// Returns AMCT_E_UNSUPPORTED when the shape is not one this kernel takes (the caller then uses its other kernels).
int w8a8_stream_dispatch(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch, const void* bias,
                         int bias_kind, void* out, int32_t* acc_out, int64_t M, int64_t N, int64_t K, int out_dtype,
                         hipStream_t st) {
    // a wave streams K / 4 bytes of 16 weight rows as NL = K / 256 registers of 16 bytes, all in flight from the start
    if (M < 1 || M > 16 || (K != 1024 && K != 2048 && K != 4096) || N > (int64_t(1) << 30)) return AMCT_E_UNSUPPORTED;
    if (!aligned16(xq) || !aligned16(wq)) return AMCT_E_UNSUPPORTED;
    StreamArgs8 a{xq, wq, s_tok, s_ch, bias_kind ? bias : nullptr, out, acc_out, (int)M, (int)N, (int)K, bias_kind,
                  (uint32_t)(0x100000000ull / (uint64_t)(K / 16)) + 1u, nullptr, nullptr, nullptr, nullptr, 0};
    // Large activation blocks are staged by few, wide blocks (16 waves share one copy in LDS), small ones by blocks of
    // 8 waves.  Measured on W[14336,4096] (58.7 MB, us per call back to back): M = 1 10.8, M = 4 11.4, M = 16 12.4,
    // against 13.5 / 14.4 / 14.4 for the kernels this one replaced (blocks of 4 waves at M = 1: 11.3; blocks of 8 waves at
    // M = 16: 13.3); a plain read of 64 MiB takes 10.9.
    const size_t xbytes = (size_t)M * ((size_t)K + 16);
    const int cg = xbytes > 40 * 1024 ? 4 : 2;
    const int nl = (int)(K / 256);
    const size_t red = (size_t)3 * cg * 64 * 16;
    const size_t lds_bytes = xbytes > red ? xbytes : red;
    if (out_dtype == AMCT_BF16) return stream8_shape<AMCT_BF16>(a, cg, nl, lds_bytes, st);
    if (out_dtype == AMCT_F16) return stream8_shape<AMCT_F16>(a, cg, nl, lds_bytes, st);
    return stream8_shape<AMCT_F32>(a, cg, nl, lds_bytes, st);
}

// The same launch with the static quantisation of the activations done while they are staged (x of x_dtype bf16 or
// fp16; smooth, act_scale, act_zp of that type; per_token: one scale per row).  AMCT_E_UNSUPPORTED for other shapes.
int w8a8_stream_quant_dispatch(const void* x, int x_dtype, const void* smooth, const void* act_scale, const void* act_zp,
                               int per_token, const int8_t* wq, const float* s_tok, const float* s_ch, const void* bias,
                               int bias_kind, void* out, int64_t M, int64_t N, int64_t K, int out_dtype, hipStream_t st) {
    if (M < 1 || M > 16 || (K != 1024 && K != 2048 && K != 4096) || N > (int64_t(1) << 30)) return AMCT_E_UNSUPPORTED;
    if (x_dtype != AMCT_BF16 && x_dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    if (!aligned16(x) || !aligned16(wq) || (smooth && !aligned16(smooth))) return AMCT_E_UNSUPPORTED;
    StreamArgs8 a{nullptr, wq, s_tok, s_ch, bias_kind ? bias : nullptr, out, nullptr, (int)M, (int)N, (int)K, bias_kind,
                  (uint32_t)(0x100000000ull / (uint64_t)(K / 8)) + 1u, x, smooth, act_scale, act_zp, per_token};
    // the quantised image in LDS is what the int8 launch stages; block widths from the 16-bit source (twice the vectors)
    const size_t xbytes = (size_t)M * ((size_t)K + 16);
    const int cg = xbytes > 20 * 1024 ? 4 : 2;
    const int nl = (int)(K / 256);
    const size_t red = (size_t)3 * cg * 64 * 16;
    const size_t lds_bytes = xbytes > red ? xbytes : red;
#define AMCT_STREAM8_Q(ODT_)                                                                                  \
    return x_dtype == AMCT_BF16 ? stream8_shape<ODT_, AMCT_BF16>(a, cg, nl, lds_bytes, st)                    \
                                : stream8_shape<ODT_, AMCT_F16>(a, cg, nl, lds_bytes, st);
    if (out_dtype == AMCT_BF16) { AMCT_STREAM8_Q(AMCT_BF16) }
    if (out_dtype == AMCT_F16) { AMCT_STREAM8_Q(AMCT_F16) }
    AMCT_STREAM8_Q(AMCT_F32)
#undef AMCT_STREAM8_Q
}

}  // namespace amct
