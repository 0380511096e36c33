// Int8 weight-only Linear for M <= 16 (decode): the int8 weight is the only large traffic (59 MB for W[14336,4096])
// and is streamed the way the W8A8 and W4A16 kernels for a few rows stream theirs: every wave of the launch is resident
// at the same time and issues ALL its weight loads (whole 128-byte lines, 8 rows per instruction) before anything else
// waits; the activations are staged once per block through LDS with loads issued just before, smoothed on the way.
// A block owns CG groups of 16 output columns; 4 waves per column group split K.
// Arithmetic: x' = dt(x * smooth) as everywhere.  A weight enters the MFMA as the EXACT integer u = q + 128 in
// 0 .. 255 (one v_cvt_f32_ubyte per weight and one pack per pair; 255 needs 8 significant bits, which both 16-bit
// types have), every span of K that shares a scale is accumulated on its own (P = sum x' * u, fp32) and folded into
// the result as acc += s * P - s * (offset + 128) * X with X = the sum of the span's x' (one sum per 128 elements of
// K and row, computed once per block while staging).  That is sum x' * (q - offset) * s with the dequantised weight
// NOT rounded to 16 bits -- the fp32 `weight * scale` of the reference's CPU stand-in for this operator
// (tests/amct_pytorch/mock_torch_npu.py:33-55) -- whereas the tile kernels for larger M feed dt((q - offset) * s) to the
// matrix pipe; both are within the 1e-3 tolerance of the fp64 result.  Groups of 128, 256, ... up to the whole of K
// (per-channel and per-tensor factors) are spans of whole steps.
#include "amct_common.h"

namespace amct {

typedef float w8f4 __attribute__((ext_vector_type(4)));
typedef float w8f2 __attribute__((ext_vector_type(2)));
typedef __bf16 w8bf8 __attribute__((ext_vector_type(8)));
typedef __bf16 w8bf2 __attribute__((ext_vector_type(2)));
typedef _Float16 w8h8 __attribute__((ext_vector_type(8)));

template <int DT> struct W8Act;
template <> struct W8Act<AMCT_BF16> {
    static AMCT_DEV uint32_t pack2(float lo, float hi) {
        const w8f2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, w8bf2));      // round-half-even
    }
    static AMCT_DEV float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static AMCT_DEV float hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
    static AMCT_DEV w8f4 mfma(const uint4& a, const uint4& b, w8f4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w8bf8, a), __builtin_bit_cast(w8bf8, b), c, 0, 0, 0);
    }
    static AMCT_DEV uint32_t out_bits(float v) { return f32_to_bf16_bits(v); }
};
template <> struct W8Act<AMCT_F16> {
    static AMCT_DEV uint32_t pack2(float lo, float hi) { return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16); }
    static AMCT_DEV float lo(uint32_t w) { return f16_bits_to_f32(w & 0xFFFFu); }
    static AMCT_DEV float hi(uint32_t w) { return f16_bits_to_f32(w >> 16); }
    static AMCT_DEV w8f4 mfma(const uint4& a, const uint4& b, w8f4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(w8h8, a), __builtin_bit_cast(w8h8, b), c, 0, 0, 0);
    }
    static AMCT_DEV uint32_t out_bits(float v) { return f32_to_f16_bits(v); }
};

struct Stream16Args {
    const uint16_t* x;
    const uint16_t* smooth;
    const uint8_t* wq;                               // [N, K] int8 codes
    const uint16_t* scales;                          // [N, K / group]
    const uint8_t* offsets;                          // [N, K / group] int8, or null
    const float* bias;
    uint16_t* out;
    int M, N, K, G;                                  // G = K / group
    int per_group;                                   // steps of 128 of one group (group / 128)
    int span;                                        // steps of 128 that share a scale inside a wave's quarter of K
    int spans;                                       // such spans per wave
    int scale_f16;
    uint32_t kv_magic;                               // floor(2^32 / (K / 8)) + 1: v / (K / 8) == mulhi(v, magic)
};

// 8 bytes (two words) -> 8 values of dt, in byte order
template <int DT>
AMCT_DEV uint4 w8_expand(uint32_t w0, uint32_t w1) {
    // q + 128: the sign bit flipped
    w0 ^= 0x80808080u;
    w1 ^= 0x80808080u;
    // (float)((w >> 8 n) & 0xFF) is one v_cvt_f32_ubyteN
    return make_uint4(W8Act<DT>::pack2((float)(w0 & 0xFFu), (float)((w0 >> 8) & 0xFFu)),
                      W8Act<DT>::pack2((float)((w0 >> 16) & 0xFFu), (float)(w0 >> 24)),
                      W8Act<DT>::pack2((float)(w1 & 0xFFu), (float)((w1 >> 8) & 0xFFu)),
                      W8Act<DT>::pack2((float)((w1 >> 16) & 0xFFu), (float)(w1 >> 24)));
}

template <int DT>
AMCT_DEV float w8_sum8(const uint4& x) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w};
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) t = t + (W8Act<DT>::lo(xs[i]) + W8Act<DT>::hi(xs[i]));
    return t;
}
template <int DT>
AMCT_DEV uint4 w8_smooth8(const uint4& x, const uint4& c) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, cs[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = W8Act<DT>::pack2(W8Act<DT>::lo(xs[i]) * W8Act<DT>::lo(cs[i]), W8Act<DT>::hi(xs[i]) * W8Act<DT>::hi(cs[i]));
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// NLN: 128-byte lines (steps of 128 elements of K) of a wave; XJ: 16-byte activation vectors a thread stages; CVN:
// different smoothing vectors among them (vector j of a thread lies NT vectors behind vector j - 1, and a row has K / 8:
// when NT is a multiple of that, all of a thread's vectors sit in the same columns)
template <int DT, int CG, int NLN, int XJ, int CVN, bool SMOOTH>
__global__ __launch_bounds__(4 * CG * 64) void w8a16_stream(Stream16Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int KS = 4;
    constexpr int NT = KS * CG * 64;
    constexpr int COLS = CG * 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cg = wave / KS, ks = wave % KS;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * COLS;
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M, G = (uint32_t)a.G;
    const uint32_t xstride = K * 2 + 16;             // 16 bytes of padding: the 16 rows of a fragment read hit different banks
    const uint32_t xbytes = M * xstride;
    uint8_t* xs = lds;
    float* xsum = reinterpret_cast<float*>(lds + xbytes);   // [K / 128][16]: sum of x' per step and row

    // ---- staging loads (activations, smoothing factors) ------------------------------------------------------------
    const uint32_t KV = K / 8, n_xv = M * KV;
    uint4 xv[XJ], cv[CVN];
    uint32_t xrow[XJ], xkv[XJ];
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        const uint32_t vc = v < n_xv ? v : n_xv - 1;
        xrow[j] = __umulhi(vc, a.kv_magic);           // vc / KV
        xkv[j] = vc - xrow[j] * KV;
        xv[j] = ldg16(a.x + (size_t)xrow[j] * K + xkv[j] * 8);
        if constexpr (SMOOTH) {
            if (j < CVN) cv[j] = ldg16(a.smooth + xkv[j] * 8);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- the whole weight stream of this wave: NLN lines of 16 rows, two load instructions (rows 0 .. 7, 8 .. 15) each
    constexpr uint32_t kw = NLN * 128;               // elements (= bytes) of K of this wave
    const int ncol = n0 + cg * 16 + r16;
    const uint32_t oct = lane >> 3;
    const uint32_t chunk = (oct & 1) ? 4 + (oct >> 1) : (oct >> 1);
    const int rlo = n0 + cg * 16 + (lane & 7), rhi = rlo + 8;
    const uint8_t* wlo = a.wq + (size_t)(rlo < a.N ? rlo : a.N - 1) * K + ks * kw + chunk * 16;
    const uint8_t* whi = a.wq + (size_t)(rhi < a.N ? rhi : a.N - 1) * K + ks * kw + chunk * 16;
    // Blocks of 16 waves have 128 registers per lane: the activation vectors in flight (32) and all of the weights
    // (64) do not fit beside each other, so such a block requests the second half of its lines when the activations have
    // gone to LDS (the first half is still arriving then; narrower blocks request everything at once).
    constexpr int FIRST = CG == 4 ? (NLN + 1) / 2 : NLN;
    u4v wv[2 * NLN];
#pragma unroll
    for (int i = 0; i < FIRST; ++i) {
        wv[2 * i] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wlo + i * 128));
        wv[2 * i + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(whi + i * 128));
    }
    __builtin_amdgcn_sched_barrier(0);
    // the factors of this lane's column for the spans of this wave (at most NLN), needed when the first span ends
    const int nc = ncol < a.N ? ncol : a.N - 1;
    const uint32_t g_first = ((uint32_t)ks * NLN) / (uint32_t)a.per_group;     // the group of the wave's first span
    float fs[NLN], fc[NLN];
#pragma unroll
    for (int q = 0; q < NLN; ++q) {
        const uint32_t gi = q < a.spans ? g_first + q : g_first;
        const uint32_t gidx = gi < G ? gi : G - 1;
        const uint32_t sbits = a.scales[(size_t)nc * G + gidx];
        const int zq = a.offsets ? (int)reinterpret_cast<const int8_t*>(a.offsets)[(size_t)nc * G + gidx] : 0;
        fs[q] = a.scale_f16 ? f16_bits_to_f32(sbits) : bf16_bits_to_f32(sbits);
        fc[q] = -(fs[q] * (float)(zq + 128));                                  // exact: 8 bits x 11 bits
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- stage the activations: smoothed, summed per step of 128 --------------------------------------------------
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        if constexpr (SMOOTH) xv[j] = w8_smooth8<DT>(xv[j], cv[j % CVN]);
        // 16 consecutive lanes hold 128 consecutive elements of one row; whole groups of 16 lanes are valid or not
        float t = w8_sum8<DT>(xv[j]);
        t = t + __shfl_xor(t, 1);
        t = t + __shfl_xor(t, 2);
        t = t + __shfl_xor(t, 4);
        t = t + __shfl_xor(t, 8);
        if (v < n_xv) {
            *reinterpret_cast<uint4*>(xs + xrow[j] * xstride + xkv[j] * 16) = xv[j];
            if ((tid & 15) == 0) xsum[(xkv[j] >> 4) * 16 + xrow[j]] = t;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = FIRST; i < NLN; ++i) {
        wv[2 * i] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wlo + i * 128));
        wv[2 * i + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(whi + i * 128));
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // ---- follow the weights as they land ---------------------------------------------------------------------------
    // After the half swap, register 2 i of a pair holds, for row lane % 16, bytes 16 g .. 16 g + 15 of the first 64 of the
    // line, register 2 i + 1 the same of the second 64.  A register feeds two MFMAs of 32 elements of K: lane group g
    // brings elements 16 g .. 16 g + 7 to the first and 16 g + 8 .. 16 g + 15 to the second; the activation fragments are
    // read from the same places.
    w8f4 acc = {0.f, 0.f, 0.f, 0.f}, P = {0.f, 0.f, 0.f, 0.f}, X = {0.f, 0.f, 0.f, 0.f};
    const uint8_t* xlane = xs + (r16 < (int)M ? r16 : (int)M - 1) * xstride + (ks * kw + g * 16) * 2;
    int in_span = 0, span_idx = 0;
#pragma unroll
    for (int i = 0; i < NLN; ++i) {
        uint4 fa[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) fa[q] = *reinterpret_cast<const uint4*>(xlane + i * 256 + (q >> 1) * 128 + (q & 1) * 16);
        u4v b0, b1;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t lo = wv[2 * i][d], hi = wv[2 * i + 1][d];
            // row_ror:8 inside each row of 16 lanes; bank_mask picks the lanes that take the rotated value
            b0[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)hi, 0x128, 0xF, 0xC, false);
            b1[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)lo, 0x128, 0xF, 0x3, false);
        }
        P = W8Act<DT>::mfma(fa[0], w8_expand<DT>(b0.x, b0.y), P);
        P = W8Act<DT>::mfma(fa[1], w8_expand<DT>(b0.z, b0.w), P);
        P = W8Act<DT>::mfma(fa[2], w8_expand<DT>(b1.x, b1.y), P);
        P = W8Act<DT>::mfma(fa[3], w8_expand<DT>(b1.z, b1.w), P);
        {
            const w8f4 Xi = *reinterpret_cast<const w8f4*>(xsum + (ks * NLN + i) * 16 + 4 * g);
#pragma unroll
            for (int r = 0; r < 4; ++r) X[r] = X[r] + Xi[r];
        }
        if (++in_span == a.span) {                   // the span's scale ends here (the same for every wave of the launch)
            float sc = fs[0], c = fc[0];
#pragma unroll
            for (int q = 1; q < NLN; ++q)
                if (q == span_idx) { sc = fs[q]; c = fc[q]; }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(sc, P[r], __builtin_fmaf(c, X[r], acc[r]));
            P = w8f4{0.f, 0.f, 0.f, 0.f};
            X = w8f4{0.f, 0.f, 0.f, 0.f};
            in_span = 0;
            ++span_idx;
        }
    }
    w8f4 y = acc;

    // ---- add the four partial sums of a column group in wave order, write -------------------------------------------
    __syncthreads();                                  // every wave is done reading activations: their rows are reused
    float* red = reinterpret_cast<float*>(lds);
    if (ks > 0) *reinterpret_cast<w8f4*>(red + (((ks - 1) * CG + cg) * 64 + lane) * 4) = y;
    __syncthreads();
    if (ks == 0) {
#pragma unroll
        for (int w = 0; w < KS - 1; ++w) {
            const w8f4 o = *reinterpret_cast<const w8f4*>(red + ((w * CG + cg) * 64 + lane) * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = y[r] + o[r];
        }
        if (ncol < a.N) {
            const float b = a.bias ? a.bias[ncol] : 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                float v = y[r];
                if (a.bias) v = v + b;
                if (m < (int)M) a.out[(size_t)m * a.N + ncol] = (uint16_t)W8Act<DT>::out_bits(v);
            }
        }
    }
}

template <int DT, int CG, int NLN, bool SMOOTH>
static int stream16_launch_x(const Stream16Args& a, size_t lds_bytes, hipStream_t st) {
    constexpr int NT = 4 * CG * 64;
    const int n_xv = a.M * (a.K / 8);
    const int xj = (n_xv + NT - 1) / NT;
    const dim3 grid((unsigned)((a.N + CG * 16 - 1) / (CG * 16)));
#define AMCT_STREAM16_GO(XJ, CVN_)                                                                                    \
    {                                                                                                               \
        auto kern = &w8a16_stream<DT, CG, NLN, XJ, CVN_, SMOOTH>;                                                         \
        if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) { \
            (void)hipGetLastError();                                                                                \
            return AMCT_E_HIP;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, st, a);                                                 \
        return hip_status();                                                                                        \
    }
    const int kv = a.K / 8;
    if (NT % kv == 0) {
        if (xj <= 2) AMCT_STREAM16_GO(2, 1)
        if (xj <= 4) AMCT_STREAM16_GO(4, 1)
        if (xj <= 8) AMCT_STREAM16_GO(8, 1)
    } else if (kv == 2 * NT) {                       // K = 4096 in blocks of 256 threads: M = 1
        if constexpr (CG == 1 && NLN == 8) {
            if (xj <= 2) AMCT_STREAM16_GO(2, 2)
        }
    }
#undef AMCT_STREAM16_GO
    return AMCT_E_UNSUPPORTED;
}

template <int DT>
static int stream16_dispatch_dt(const Stream16Args& a, bool smooth, int cg, int nln, size_t lds_bytes, hipStream_t st) {
#define AMCT_STREAM16_SHAPE(CG_, NLN_)                                                                  \
    if (cg == CG_ && nln == NLN_)                                                                       \
        return smooth ? stream16_launch_x<DT, CG_, NLN_, true>(a, lds_bytes, st) : stream16_launch_x<DT, CG_, NLN_, false>(a, lds_bytes, st);
    AMCT_STREAM16_SHAPE(4, 8)
    AMCT_STREAM16_SHAPE(2, 8)
    AMCT_STREAM16_SHAPE(1, 8)
    AMCT_STREAM16_SHAPE(4, 4)
    AMCT_STREAM16_SHAPE(2, 4)
    AMCT_STREAM16_SHAPE(1, 4)
    AMCT_STREAM16_SHAPE(4, 2)
    AMCT_STREAM16_SHAPE(2, 2)
    AMCT_STREAM16_SHAPE(1, 2)
#undef AMCT_STREAM16_SHAPE
    return AMCT_E_UNSUPPORTED;
}

// Returns AMCT_E_UNSUPPORTED when the shape is not one this kernel takes (the caller then uses its other kernels).
int w8a16_stream_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                          const uint8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                          int dtype, hipStream_t st) {
    if (M < 1 || M > 16 || (K != 1024 && K != 2048 && K != 4096) || N > (int64_t(1) << 30)) return AMCT_E_UNSUPPORTED;
    if (group < 128 || (group & (group - 1)) != 0 || group > K) return AMCT_E_UNSUPPORTED;     // 128, 256, ..., K
    if (!aligned16(x) || !aligned16(wq) || (smooth && !aligned16(smooth)) || ((uintptr_t)scales & 1)) return AMCT_E_UNSUPPORTED;
    const int nln = (int)(K / 512);                  // lines of 128 per wave (a quarter of K)
    const int per_group = group / 128;               // steps that share a scale
    const int span = per_group < nln ? per_group : nln;
    Stream16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, (const uint16_t*)scales, offsets, bias, (uint16_t*)out,
                   (int)M, (int)N, (int)K, (int)(K / group), per_group, span, nln / span, scale_dtype == AMCT_F16 ? 1 : 0,
                   (uint32_t)(0x100000000ull / (uint64_t)(K / 8)) + 1u};
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16);
    const int cg = xbytes > 40 * 1024 ? 4 : xbytes > 12 * 1024 ? 2 : 1;
    const size_t red = (size_t)3 * cg * 64 * 16, img = xbytes + (size_t)(K / 128) * 64;
    const size_t lds_bytes = img > red ? img : red;
    if (lds_bytes > 160 * 1024) return AMCT_E_UNSUPPORTED;
    return dtype == AMCT_F16 ? stream16_dispatch_dt<AMCT_F16>(a, smooth != nullptr, cg, nln, lds_bytes, st)
                             : stream16_dispatch_dt<AMCT_BF16>(a, smooth != nullptr, cg, nln, lds_bytes, st);
}

}  // namespace amct
