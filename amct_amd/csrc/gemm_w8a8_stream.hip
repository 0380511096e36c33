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
};

// XJ: 16-byte activation vectors a thread stages (clamped duplicates beyond the tensor)
template <int ODT, int KS, int CG, int NL, int XJ>
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
    const uint32_t KV = K / 16, n_xv = M * KV;
    uint4 xv[XJ];
    uint32_t xoff[XJ];
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        const uint32_t vc = v < n_xv ? v : n_xv - 1;
        const uint32_t row = __umulhi(vc, a.kv_magic);            // vc / KV
        xoff[j] = row * xstride + (vc - row * KV) * 16;
        xv[j] = ldg16(a.xq + (size_t)vc * 16);
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
    u4v wv[NL];
#pragma unroll
    for (int i = 0; i < NL; i += 2) {
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
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        if (tid + NT * j < n_xv) *reinterpret_cast<uint4*>(lds + xoff[j]) = xv[j];
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

template <int ODT, int KS, int CG, int NL>
static int stream8_launch_x(const StreamArgs8& a, size_t lds_bytes, hipStream_t st) {
    constexpr int NT = KS * CG * 64;
    const int n_xv = a.M * (a.K / 16);
    const int xj = (n_xv + NT - 1) / NT;
    const dim3 grid((unsigned)((a.N + CG * 16 - 1) / (CG * 16)));
#define AMCT_STREAM8_GO(XJ)                                                                                         \
    {                                                                                                               \
        auto kern = &w8a8_stream<ODT, KS, CG, NL, XJ>;                                                              \
        if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) { \
            (void)hipGetLastError();                                                                                \
            return AMCT_E_HIP;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, st, a);                                                 \
        return hip_status();                                                                                        \
    }
    if (xj <= 1) AMCT_STREAM8_GO(1)
    if (xj <= 2) AMCT_STREAM8_GO(2)
    if (xj <= 4) AMCT_STREAM8_GO(4)
    if (xj <= 8) AMCT_STREAM8_GO(8)
#undef AMCT_STREAM8_GO
    return AMCT_E_UNSUPPORTED;
}

template <int ODT>
static int stream8_shape(const StreamArgs8& a, int cg, int nl, size_t lds_bytes, hipStream_t st) {
#define AMCT_STREAM8_SHAPE(CG_, NL_) \
    if (cg == CG_ && nl == NL_) return stream8_launch_x<ODT, 4, CG_, NL_>(a, lds_bytes, st);
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
                  (uint32_t)(0x100000000ull / (uint64_t)(K / 16)) + 1u};
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

}  // namespace amct
