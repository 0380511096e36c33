// Int8 weight-only Linear for M <= 16 (decode): the int8 weight is the only large traffic (59 MB for W[14336,4096])
// and is streamed the way the W8A8 and W4A16 kernels for a few rows stream theirs: every wave of the launch is resident
// at the same time and issues ALL its weight loads (whole 128-byte lines, 8 rows per instruction) before anything else
// waits; the activations are staged once per block through LDS with loads issued just before, smoothed on the way.
// A block owns CG groups of 16 output columns; 4 waves per column group split K.
// Arithmetic: x' = dt(x * smooth) as everywhere.  A weight enters the MFMA as the EXACT integer u = q + 128 in
// 0 .. 255 (one v_cvt_f32_ubyte per weight and one pack per pair; 255 needs 8 significant bits, which both 16-bit
// types have), and the offset leaves on the matrix pipe as well: behind every weight MFMA a second one multiplies the
// same activations with the constant -(128 + offset) of the lane's column (0 .. 255 too, exact), so the accumulators
// of a span of K that shares a scale hold P = sum x' * (q - offset) (fp32) and the fold is acc += s * P -- no sums of
// activations are needed anywhere.  That is sum x' * (q - offset) * s with the dequantised weight NOT rounded to 16
// bits -- the fp32 `weight * scale` of the reference's CPU stand-in for this operator
// (tests/amct_pytorch/mock_torch_npu.py:33-55) -- whereas the tile kernels for larger M feed dt((q - offset) * s) to the
// matrix pipe, which moves an output by up to 2^-8 (bf16; fp16: 2^-11) of sum |x' w|: amct_gemm_w8a16_weight_rounded tells
// which of the two a call takes.  Groups of 128, 256, ... up to the whole of K (per-channel and per-tensor factors) are
// spans of whole steps.
#include "amct_common.h"
#include "gemm_plan.h"

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
    // Rows longer than a slice (K above is the slice one block walks): blockIdx.y picks the slice; rows keep their full
    // length as stride; every slice leaves fp32 partial sums part[slice][M][N] that a second kernel adds in slice order
    int row_k;                                       // elements of a full row of x and of the weight
    int row_g;                                       // groups of a full row
    float* part;                                     // null: one slice, the result goes to `out`
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
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M;
    const uint32_t xstride = K * 2 + 16;             // 16 bytes of padding: the 16 rows of a fragment read hit different banks
    uint8_t* xs = lds;

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
        // (a last slice may reach beyond the row: those elements are staged as zeros, read from the row's start)
        const uint32_t xk = blockIdx.y * K + xkv[j] * 8;
        const bool inside = xk < (uint32_t)a.row_k;
        xv[j] = ldg16(a.x + (size_t)xrow[j] * a.row_k + (inside ? xk : 0u));
        if (!inside) xv[j] = make_uint4(0u, 0u, 0u, 0u);
        if constexpr (SMOOTH) {
            if (j < CVN) cv[j] = ldg16(a.smooth + (inside ? xk : 0u));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    // the factors of this lane's column for the spans of this wave (at most NLN), needed when the first span ends:
    // requested BEFORE the weights (a load issued behind the weight stream returns behind it) and kept as raw bits until
    // the fold that uses them, so that nothing waits for them here
    const int ncol = n0 + cg * 16 + r16;
    const int nc = ncol < a.N ? ncol : a.N - 1;
    const uint32_t g_first = (blockIdx.y * (K / 128) + (uint32_t)ks * NLN) / (uint32_t)a.per_group;   // the group of the wave's first span
    const uint32_t RG = (uint32_t)a.row_g;
    const float bias_v = (a.bias && ks == 0) ? a.bias[nc] : 0.f;    // with the factors: a load in the epilogue would cost a memory latency there
    uint32_t fs_raw[NLN];
    int fz_raw[NLN];
#pragma unroll
    for (int q = 0; q < NLN; ++q) {
        const uint32_t gi = q < a.spans ? g_first + q : g_first;
        const uint32_t gidx = gi < RG ? gi : RG - 1;
        fs_raw[q] = a.scales[(size_t)nc * RG + gidx];
        fz_raw[q] = a.offsets ? (int)reinterpret_cast<const int8_t*>(a.offsets)[(size_t)nc * RG + gidx] : 0;
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- the whole weight stream of this wave: NLN lines of 16 rows, two load instructions (rows 0 .. 7, 8 .. 15) each
    constexpr uint32_t kw = NLN * 128;               // elements (= bytes) of K of this wave
    const uint32_t oct = lane >> 3;
    const uint32_t chunk = (oct & 1) ? 4 + (oct >> 1) : (oct >> 1);
    const int rlo = n0 + cg * 16 + (lane & 7), rhi = rlo + 8;
    // (a wave whose part of a last, shorter slice lies beyond the row reads the row's first weights: its activations are zeros)
    const uint32_t kwave = blockIdx.y * K + ks * kw;
    const size_t woff = (size_t)(kwave < (uint32_t)a.row_k ? kwave : 0u) + chunk * 16;
    const uint8_t* wlo = a.wq + (size_t)(rlo < a.N ? rlo : a.N - 1) * (size_t)a.row_k + woff;
    const uint8_t* whi = a.wq + (size_t)(rhi < a.N ? rhi : a.N - 1) * (size_t)a.row_k + woff;
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
    // ---- stage the activations, smoothed ----------------------------------------------------------------------------
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        if constexpr (SMOOTH) xv[j] = w8_smooth8<DT>(xv[j], cv[j % CVN]);
        if (v < n_xv) *reinterpret_cast<uint4*>(xs + xrow[j] * xstride + xkv[j] * 16) = xv[j];
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
    // (two accumulator chains, so that an MFMA does not wait for the one just issued)
    w8f4 acc = {0.f, 0.f, 0.f, 0.f}, P0 = {0.f, 0.f, 0.f, 0.f}, P1 = {0.f, 0.f, 0.f, 0.f};
    const uint8_t* xlane = xs + (r16 < (int)M ? r16 : (int)M - 1) * xstride + (ks * kw + g * 16) * 2;
    int in_span = 0, span_idx = 0;
    uint4 nz = make_uint4(0u, 0u, 0u, 0u);           // -(128 + offset) of the lane's column in the current span, 8 times
#pragma unroll
    for (int i = 0; i < NLN; ++i) {
        if (in_span == 0) {                          // a span starts (the same for every wave of the launch)
            int zq = fz_raw[0];
#pragma unroll
            for (int q = 1; q < NLN; ++q)
                if (q == span_idx) zq = fz_raw[q];
            const float nf = -(float)(zq + 128);
            const uint32_t nb = W8Act<DT>::pack2(nf, nf);
            nz = make_uint4(nb, nb, nb, nb);
        }
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
        P0 = W8Act<DT>::mfma(fa[0], w8_expand<DT>(b0.x, b0.y), P0);
        P1 = W8Act<DT>::mfma(fa[1], w8_expand<DT>(b0.z, b0.w), P1);
        P0 = W8Act<DT>::mfma(fa[2], w8_expand<DT>(b1.x, b1.y), P0);
        P1 = W8Act<DT>::mfma(fa[3], w8_expand<DT>(b1.z, b1.w), P1);
        P0 = W8Act<DT>::mfma(fa[0], nz, P0);
        P1 = W8Act<DT>::mfma(fa[1], nz, P1);
        P0 = W8Act<DT>::mfma(fa[2], nz, P0);
        P1 = W8Act<DT>::mfma(fa[3], nz, P1);
        if (++in_span == a.span) {                   // the span's scale ends here
            uint32_t sbits = fs_raw[0];
#pragma unroll
            for (int q = 1; q < NLN; ++q)
                if (q == span_idx) sbits = fs_raw[q];
            const float sc = a.scale_f16 ? f16_bits_to_f32(sbits) : bf16_bits_to_f32(sbits);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(sc, P0[r] + P1[r], acc[r]);
            P0 = w8f4{0.f, 0.f, 0.f, 0.f};
            P1 = w8f4{0.f, 0.f, 0.f, 0.f};
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
        if (ncol < a.N && a.part) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                if (m < (int)M) a.part[((size_t)blockIdx.y * M + m) * a.N + ncol] = y[r];
            }
        } else if (ncol < a.N) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                float v = y[r];
                if (a.bias) v = v + bias_v;
                if (m < (int)M) a.out[(size_t)m * a.N + ncol] = (uint16_t)W8Act<DT>::out_bits(v);
            }
        }
    }
}

int splitk_reduce16_launch(const float* part, const float* bias, void* out, int64_t M, int64_t N, int splits, int dtype,
                           hipStream_t st);                          // gemm_w4a16.hip

template <int DT, int CG, int NLN, bool SMOOTH>
static int stream16_launch_x(const Stream16Args& a, size_t lds_bytes, hipStream_t st) {
    constexpr int NT = 4 * CG * 64;
    const int n_xv = a.M * (a.K / 8);
    const int xj = (n_xv + NT - 1) / NT;
    const dim3 grid((unsigned)((a.N + CG * 16 - 1) / (CG * 16)), (unsigned)((a.row_k + a.K - 1) / a.K));
#define AMCT_STREAM16_GO(XJ, CVN_)                                                                                    \
    {                                                                                                               \
        auto kern = &w8a16_stream<DT, CG, NLN, XJ, CVN_, SMOOTH>;                                                         \
        if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) { \
            (void)hipGetLastError();                                                                                \
            return AMCT_E_HIP;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, st, a);                                                 \
        if (a.part) return splitk_reduce16_launch(a.part, a.bias, a.out, a.M, a.N, (int)grid.y, DT, st);            \
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

// The slice of K one block walks: K itself when it is 1024, 2048 or 4096, else the largest of those that divides K into at
// most 16 slices; 0: none.
static int64_t stream16_slice(int64_t K) {
    if (K == 1024 || K == 2048 || K == 4096) return K;
    for (int64_t ks = 4096; ks >= 1024; ks /= 2)
        if (K % ks == 0 && K / ks <= 16) return ks;
    // other multiples of 256 (11008, 13824): slices of 1024 whose last one is shorter -- a wave walks 256 elements, so it
    // lies inside the row or beyond it as a whole
    if (K % 256 == 0 && K > 1024 && (K + 1023) / 1024 <= 16) return 1024;
    return 0;
}
// groups the kernel takes for slices of `ks`: 128, 256, ... up to the slice, whole slices, or the whole row (per-channel factors)
static bool stream16_group_ok(int64_t K_row, int64_t ks, int group) {
    if (group < 128 || K_row % group != 0) return false;
    if (group <= ks) return (group & (group - 1)) == 0;
    return group % ks == 0 || group == K_row;
}
// Sliced rows pay a second launch and stage the activations once per block: taken for long rows (K >= 12288), for four
// and more slices (slices of 1024), or while blocks of 64 columns per slice run in one round.  Measured against the
// kernels that served these shapes before (specialised waves with K split, shared kernel), us at M = 1 / 4 / 16,
// per-channel factors: W[8192,28672] 87 / 87 / 87 -> 58 / 65 / 77; W[8192,8192] 30 / 30 / 29 -> 21 / 29 / 23;
// W[13824,5120] 24 / 26 / 28 -> 19 / 20 / 25; not taken: W[28672,8192] 53 / 56 / 65 (sliced: 56 / 83 / 73),
// W[10240,8192] 27 / 29 / 33 (sliced: 25 / 35 / 38).
// (And whenever the activation image of a slice is small enough for the narrow blocks, several per CU: W[28672,8192] /
// W[57344,8192] at M = 1: 53 / 103 -> 40 / 73 us.)
static bool stream16_slices_pay(int64_t M, int64_t N, int64_t K, int64_t ks) {
    const int64_t S = (K + ks - 1) / ks, cus = current_cu_count();
    return K >= 12288 || S >= 4 || ((N + 63) / 64) * S <= cus || M * (ks * 2 + 16) <= 12 * 1024;
}
size_t w8a16_stream_part_bytes(int64_t M, int64_t N, int64_t K, int group) {
    const int64_t ks = stream16_slice(K);
    if (M < 1 || M > 16 || !ks || ks == K || N % 8 != 0 || !stream16_group_ok(K, ks, group) || !stream16_slices_pay(M, N, K, ks)) return 0;
    return (size_t)((K + ks - 1) / ks) * (size_t)M * (size_t)N * 4;
}

// Whether this kernel takes a call of this shape with a workspace of this size (operands suitably aligned): the one
// rule behind the dispatch below and behind amct_gemm_w8a16_weight_rounded.
bool w8a16_stream_takes(int64_t M, int64_t N, int64_t K_row, int group, size_t workspace_bytes) {
    const int64_t K = stream16_slice(K_row), S = K ? (K_row + K - 1) / K : 0;
    if (M < 1 || M > 16 || !K || N <= 0 || N > (int64_t(1) << 30)) return false;
    if (!stream16_group_ok(K_row, K, group)) return false;
    if (S > 1) {
        // rows of several slices: the partial sums go through the lent workspace
        const size_t need = w8a16_stream_part_bytes(M, N, K_row, group);
        if (!need || workspace_bytes < need) return false;
    }
    // the launch shapes below: threads whose staged vectors share a column (or M = 1 on K = 4096), at most 8 of them
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16);
    const int64_t cg = xbytes > 40 * 1024 ? 4 : xbytes > 12 * 1024 ? 2 : 1, nt = 256 * cg, kv = K / 8;
    const int64_t xj = (M * kv + nt - 1) / nt;
    if (xbytes > 160 * 1024) return false;
    if (nt % kv == 0) return xj <= 8;
    return kv == 2 * nt && cg == 1 && K / 512 == 8 && xj <= 2;
}

// Returns AMCT_E_UNSUPPORTED when the shape is not one this kernel takes (the caller then uses its other kernels).
int w8a16_stream_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                          const uint8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K_row, int group,
                          int dtype, void* workspace, size_t workspace_bytes, hipStream_t st) {
    if (!w8a16_stream_takes(M, N, K_row, group, workspace ? workspace_bytes : 0)) return AMCT_E_UNSUPPORTED;
    const int64_t K = stream16_slice(K_row), S = (K_row + K - 1) / K;
    if (!aligned16(x) || !aligned16(wq) || (smooth && !aligned16(smooth)) || ((uintptr_t)scales & 1)) return AMCT_E_UNSUPPORTED;
    float* part = nullptr;
    if (S > 1) {
        if (!aligned16(workspace) || !aligned16(out) || (bias && !aligned16(bias))) return AMCT_E_UNSUPPORTED;
        part = reinterpret_cast<float*>(workspace);
    }
    const int nln = (int)(K / 512);                  // lines of 128 per wave (a quarter of the slice)
    const int per_group = group / 128;               // steps that share a scale
    const int span = per_group < nln ? per_group : nln;
    Stream16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, (const uint16_t*)scales, offsets, bias, (uint16_t*)out,
                   (int)M, (int)N, (int)K, (int)(K_row / group), per_group, span, nln / span, scale_dtype == AMCT_F16 ? 1 : 0,
                   (uint32_t)(0x100000000ull / (uint64_t)(K / 8)) + 1u, (int)K_row, (int)(K_row / group), part};
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16);
    const int cg = xbytes > 40 * 1024 ? 4 : xbytes > 12 * 1024 ? 2 : 1;
    const size_t red = (size_t)3 * cg * 64 * 16, img = xbytes;
    const size_t lds_bytes = img > red ? img : red;
    if (lds_bytes > 160 * 1024) return AMCT_E_UNSUPPORTED;
    return dtype == AMCT_F16 ? stream16_dispatch_dt<AMCT_F16>(a, smooth != nullptr, cg, nln, lds_bytes, st)
                             : stream16_dispatch_dt<AMCT_BF16>(a, smooth != nullptr, cg, nln, lds_bytes, st);
}

}  // namespace amct
