// Weight-only quantised Linear for the combinations the int4 x bf16 kernels of gemm_w4a16.hip do not take:
// int8 weights with bf16 or fp16 activations (W8A16) and int4 weights with fp16 activations.
//   out[m,n] = dt( sum_k x'[m,k] * wdq[n,k] + bias[n] ), fp32 accumulate,
//   x'  = dt(x * smooth[k])                              (weight_npu_quant_module.py:113-114)
//   wdq = dt((q[n,k] - offset[n,k/g]) * scale[n,k/g])    (the operator called at :116-117, which adds the negated
//                                                         offset the module registers at :62-64)
// int4 weights are nibbles of u = q + 8 with zero-points offset + 8 (as amct_quant_int4_group_pack writes them);
// int8 weights are the signed codes, K contiguous, with int8 offsets (null = symmetric).  Internally both become
// an unsigned byte u and a zero-point z' with q - offset = u - z': one v_cvt_f32_ubyteN and one fma per weight
// ((u - z') * s == fma(u, s, -z' * s) exactly: |u - z'| < 2^9 and s has at most 11 significant bits).
//   tile kernel   : 128x128 block tile, 64 elements of K per step, 32x32x16 MFMA; activations (smoothed on the way)
//                   and dequantised weights double-buffered in LDS
//   decode kernel : M <= 64, weight streaming, 16x16x32 MFMA, K split over the waves of a block
//   general kernel: any shape, one output per thread
#include "amct_common.h"

namespace amct {

typedef float q4f __attribute__((ext_vector_type(4)));
typedef float q16f __attribute__((ext_vector_type(16)));
typedef float q2f __attribute__((ext_vector_type(2)));
typedef __bf16 q8bf __attribute__((ext_vector_type(8)));
typedef __bf16 q2bf __attribute__((ext_vector_type(2)));
typedef _Float16 q8h __attribute__((ext_vector_type(8)));
typedef _Float16 q2h __attribute__((ext_vector_type(2)));

// what differs between the two 16-bit activation types
template <int DT> struct Act16;
template <> struct Act16<AMCT_BF16> {
    typedef q8bf frag;
    static AMCT_DEV uint32_t pack2(float lo, float hi) {
        const q2f f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, q2bf));      // round-half-even
    }
    static AMCT_DEV float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static AMCT_DEV float hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
    static AMCT_DEV q16f mfma32(frag a, frag b, q16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static AMCT_DEV q4f mfma16(frag a, frag b, q4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Act16<AMCT_F16> {
    typedef q8h frag;
    static AMCT_DEV uint32_t pack2(float lo, float hi) {
        return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);                    // round-half-even
    }
    static AMCT_DEV float lo(uint32_t w) { return f16_bits_to_f32(w & 0xFFFFu); }
    static AMCT_DEV float hi(uint32_t w) { return f16_bits_to_f32(w >> 16); }
    static AMCT_DEV q16f mfma32(frag a, frag b, q16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static AMCT_DEV q4f mfma16(frag a, frag b, q4f c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

struct WqArgs {
    const uint16_t* x;
    const uint16_t* smooth;
    const uint8_t* wq;                               // int4: [N, K/2] nibbles of q + 8; int8: [N, K] signed codes
    const void* scales;                              // [N, K/group] of scale_dtype
    const uint8_t* zeros;                            // int4: q-offset + 8 (never null); int8: int8 offsets or null
    const float* bias;
    uint16_t* out;
    int64_t M, N, K;
    int group;
    int scale_dtype;
    uint32_t group_magic;                            // floor(2^32 / group) + 1: k / group == mulhi(k, magic) for k, group < 2^16
};

AMCT_DEV float wq_scale(const WqArgs& a, int64_t i) {
    const uint16_t h = reinterpret_cast<const uint16_t*>(a.scales)[i];
    return a.scale_dtype == AMCT_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}
// zero-point z' of the unsigned byte form
template <int WBITS> AMCT_DEV float wq_zero(const WqArgs& a, int64_t i) {
    if constexpr (WBITS == 4) return (float)a.zeros[i];
    else return a.zeros ? (float)((int)reinterpret_cast<const int8_t*>(a.zeros)[i] + 128) : 128.f;
}

// four bytes of `w` (opaque to the optimiser so that each becomes one v_cvt_f32_ubyteN) -> (u - z') * s
template <int DT> AMCT_DEV void dq_bytes(uint32_t w, float s, float nzs, float (&e)[4]) {
    asm("" : "+v"(w));
#pragma unroll
    for (int b = 0; b < 4; ++b) e[b] = __builtin_fmaf((float)((w >> (8 * b)) & 0xFFu), s, nzs);
}
// 8 consecutive int4 weights (element j in bits 4j..4j+3 of w) -> 8 values of DT as 4 packed words
template <int DT> AMCT_DEV uint4 dq8_int4(uint32_t w, float s, float nzs) {
    float lo[4], hi[4];
    dq_bytes<DT>(w & 0x0F0F0F0Fu, s, nzs, lo);                       // elements 0, 2, 4, 6
    dq_bytes<DT>((w >> 4) & 0x0F0F0F0Fu, s, nzs, hi);                // elements 1, 3, 5, 7
    return make_uint4(Act16<DT>::pack2(lo[0], hi[0]), Act16<DT>::pack2(lo[1], hi[1]), Act16<DT>::pack2(lo[2], hi[2]),
                      Act16<DT>::pack2(lo[3], hi[3]));
}
// 8 consecutive int8 weights (two words of signed bytes) -> 8 values of DT
template <int DT> AMCT_DEV uint4 dq8_int8(uint32_t w0, uint32_t w1, float s, float nzs) {
    float a[4], b[4];
    dq_bytes<DT>(w0 ^ 0x80808080u, s, nzs, a);                       // q + 128
    dq_bytes<DT>(w1 ^ 0x80808080u, s, nzs, b);
    return make_uint4(Act16<DT>::pack2(a[0], a[1]), Act16<DT>::pack2(a[2], a[3]), Act16<DT>::pack2(b[0], b[1]),
                      Act16<DT>::pack2(b[2], b[3]));
}
// 8 activations times 8 smoothing factors, each product rounded to DT
template <int DT> AMCT_DEV uint4 smooth8_dt(const uint4& x, const uint4& c) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, cs[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = Act16<DT>::pack2(Act16<DT>::lo(xs[i]) * Act16<DT>::lo(cs[i]), Act16<DT>::hi(xs[i]) * Act16<DT>::hi(cs[i]));
    return make_uint4(o[0], o[1], o[2], o[3]);
}
template <int DT> AMCT_DEV uint32_t to_bits16(float v) {
    return DT == AMCT_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v);
}

// 32 consecutive weights of one row starting at element k (k % 32 == 0) -> registers
template <int WBITS> struct Wchunk { uint4 v[WBITS == 4 ? 1 : 2]; };
template <int WBITS> AMCT_DEV Wchunk<WBITS> load_w32(const uint8_t* row, int64_t k) {
    Wchunk<WBITS> c;
    if constexpr (WBITS == 4) {
        c.v[0] = ldg16_nt(row + k / 2);
    } else {
        c.v[0] = ldg16_nt(row + k);
        c.v[1] = ldg16_nt(row + k + 16);
    }
    return c;
}
// weights 8 j .. 8 j + 7 of such a chunk, dequantised
template <int WBITS, int DT> AMCT_DEV uint4 dq_chunk8(const Wchunk<WBITS>& c, int j, float s, float nzs) {
    if constexpr (WBITS == 4) {
        const uint32_t ws[4] = {c.v[0].x, c.v[0].y, c.v[0].z, c.v[0].w};
        return dq8_int4<DT>(ws[j], s, nzs);
    } else {
        const uint32_t ws[8] = {c.v[0].x, c.v[0].y, c.v[0].z, c.v[0].w, c.v[1].x, c.v[1].y, c.v[1].z, c.v[1].w};
        return dq8_int8<DT>(ws[2 * j], ws[2 * j + 1], s, nzs);
    }
}

// ---------------------------------------------------------------------------
// tile kernel (K % 64 == 0, group % 32 == 0, 16-byte aligned operands)
// ---------------------------------------------------------------------------
constexpr int kGM = 128, kGN = 128, kGK = 64;
constexpr int kGRow = kGK * 2 + 16;                  // bytes per padded LDS row of 16-bit values

template <int WBITS, int DT>
__global__ __launch_bounds__(kBlock) void wq16_tile(WqArgs a) {
    using A = Act16<DT>;
    typedef typename A::frag frag;
    __shared__ __attribute__((aligned(16))) uint8_t As[2][kGM * kGRow];
    __shared__ __attribute__((aligned(16))) uint8_t Bs[2][kGN * kGRow];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * kGM, n0 = (int64_t)blockIdx.x * kGN;
    const int a_row = tid >> 3, a_chunk = tid & 7;              // activation tile: 8 chunks of 8 values per row
    const int b_row = tid >> 1, b_half = tid & 1;               // weight tile: 2 chunks of 32 weights per row
    const int nsteps = (int)(a.K / kGK);
    const int64_t G = a.K / a.group;
    const int64_t wrow = (n0 + b_row < a.N) ? n0 + b_row : a.N - 1;
    const uint8_t* wbase = a.wq + wrow * (WBITS == 4 ? a.K / 2 : a.K);

    uint4 ra[4], rc = make_uint4(0, 0, 0, 0);
    Wchunk<WBITS> rw;
    float s_cur = 0.f, nzs_cur = 0.f;
    auto load_global = [&](int step) {
        const int64_t k = (int64_t)step * kGK;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t m = m0 + a_row + 32 * i;
            ra[i] = ldg16(a.x + (m < a.M ? m : a.M - 1) * a.K + k + a_chunk * 8);
        }
        if (a.smooth) rc = ldg16(a.smooth + k + a_chunk * 8);
        const int64_t kw = k + b_half * 32;
        rw = load_w32<WBITS>(wbase, kw);
        const int64_t gi = wrow * G + kw / a.group;
        s_cur = wq_scale(a, gi);
        nzs_cur = -(wq_zero<WBITS>(a, gi) * s_cur);
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 v = ra[i];
            if (a.smooth) v = smooth8_dt<DT>(v, rc);
            *reinterpret_cast<uint4*>(&As[buf][(a_row + 32 * i) * kGRow + a_chunk * 16]) = v;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<uint4*>(&Bs[buf][b_row * kGRow + b_half * 64 + j * 16]) = dq_chunk8<WBITS, DT>(rw, j, s_cur, nzs_cur);
    };

    q16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    load_global(0);
    store_lds(0);
    __syncthreads();
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
    for (int step = 0; step < nsteps; ++step) {
        const int cur = step & 1;
        if (step + 1 < nsteps) load_global(step + 1);
#pragma unroll
        for (int ks = 0; ks < kGK / 16; ++ks) {
            frag fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const frag*>(&As[cur][(wm * 64 + i * 32 + frag_row) * kGRow + ks * 32 + frag_k]);
                fb[i] = *reinterpret_cast<const frag*>(&Bs[cur][(wn * 64 + i * 32 + frag_row) * kGRow + ks * 32 + frag_k]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = A::mfma32(fa[i], fb[j], acc[i][j]);
        }
        if (step + 1 < nsteps) store_lds(cur ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= a.N) continue;
        const float b = a.bias ? a.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < a.M) {
                    float v = acc[i][j][r];
                    if (a.bias) v = v + b;
                    a.out[m * a.N + n] = (uint16_t)to_bits16<DT>(v);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// decode kernel (M <= 16 * MT, K % 128 == 0, group % 32 == 0): a block owns 64 output columns, its waves split K
// in runs of 128.  Per iteration a lane fetches 32 weights of each of its 4 weight rows (row 16 t + lane % 16,
// k-slot lane / 16) and the matching 32 activations of its MT rows; all loads are unconditional (clamped) and
// issued one iteration ahead.
// ---------------------------------------------------------------------------
constexpr int kGDN = 64;

template <int WBITS, int DT, int MT, int WAVES, bool SMOOTH>
__global__ __launch_bounds__(WAVES * 64) void wq16_decode(WqArgs a) {
    using A = Act16<DT>;
    typedef typename A::frag frag;
    __shared__ float red[WAVES - 1 > 0 ? WAVES - 1 : 1][MT][4][64][4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * kGDN;
    const int64_t G = a.K / a.group;
    const int per_wave = (int)(a.K / 128) / WAVES;                 // host guarantees divisibility
    const int it0 = wave * per_wave;
    const bool scale_is_f16 = a.scale_dtype == AMCT_F16;
    const bool has_zeros = a.zeros != nullptr;
    // every load below is unconditional: without zero-points the bytes are fetched from the scales (in bounds) and
    // ignored
    const uint8_t* zbase = has_zeros ? a.zeros : reinterpret_cast<const uint8_t*>(a.scales);

    const uint8_t* wrow[4];
    const uint16_t* srow[4];
    const uint8_t* zrow[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int64_t n = n0 + t * 16 + r16;
        const int64_t nc = n < a.N ? n : a.N - 1;
        wrow[t] = a.wq + nc * (WBITS == 4 ? a.K / 2 : a.K);
        srow[t] = reinterpret_cast<const uint16_t*>(a.scales) + nc * G;
        zrow[t] = zbase + nc * G;
    }
    const uint16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int64_t m = mt * 16 + r16;
        xrow[mt] = a.x + (m < a.M ? m : a.M - 1) * a.K + g * 32;
    }
    q4f y[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) y[mt][t] = q4f{0.f, 0.f, 0.f, 0.f};

    Wchunk<WBITS> wv[2][4];
    uint4 xv[2][MT][4], cv[2][4];
    uint32_t sb[2][4], zb[2][4];
    auto load_it = [&](int buf, int it) {
        const int itc = it < it0 + per_wave ? it : it0 + per_wave - 1;      // clamped: loads are unconditional
        const uint32_t kb = (uint32_t)itc * 128u;
        const uint32_t gi = __umulhi(kb + (uint32_t)g * 32u, a.group_magic);
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
            if constexpr (SMOOTH) cv[buf][s4] = ldg16(a.smooth + kb + g * 32 + s4 * 8);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) xv[buf][mt][s4] = ldg16(xrow[mt] + kb + s4 * 8);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sb[buf][t] = srow[t][gi];
            zb[buf][t] = zrow[t][gi];
            wv[buf][t] = load_w32<WBITS>(wrow[t], (int64_t)kb + g * 32);
        }
    };
    auto compute = [&](int buf) {
        frag fa[MT][4];
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                uint4 v = xv[buf][mt][s4];
                if constexpr (SMOOTH) v = smooth8_dt<DT>(v, cv[buf][s4]);
                fa[mt][s4] = __builtin_bit_cast(frag, v);
            }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float s_h = f16_bits_to_f32(sb[buf][t]), s_b = bf16_bits_to_f32(sb[buf][t]);
            const float s = scale_is_f16 ? s_h : s_b;
            float z;                                                 // zero-point of the unsigned byte form
            if constexpr (WBITS == 4) z = (float)zb[buf][t];
            else z = has_zeros ? (float)((int)(int8_t)zb[buf][t] + 128) : 128.f;
            const float nz = -(z * s);
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const frag fb = __builtin_bit_cast(frag, dq_chunk8<WBITS, DT>(wv[buf][t], s4, s, nz));
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) y[mt][t] = A::mfma16(fa[mt][s4], fb, y[mt][t]);
            }
        }
    };

    load_it(0, it0);
    for (int i = 0; i < per_wave; i += 2) {
        load_it(1, it0 + i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(0);
        if (i + 1 >= per_wave) break;
        __builtin_amdgcn_sched_barrier(0);
        load_it(0, it0 + i + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(1);
        __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) red[wave - 1][mt][t][lane][r] = y[mt][t][r];
        }
        __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int64_t n = n0 + t * 16 + r16;
            const float b = (a.bias && n < a.N) ? a.bias[n] : 0.f;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = y[mt][t][r];
                    if constexpr (WAVES > 1) {
#pragma unroll
                        for (int w = 0; w < WAVES - 1; ++w) v = v + red[w][mt][t][lane][r];
                    }
                    if (a.bias) v = v + b;
                    const int64_t m = mt * 16 + 4 * g + r;
                    if (n < a.N && m < a.M) a.out[m * a.N + n] = (uint16_t)to_bits16<DT>(v);
                }
            }
        }
    }
}

// general kernel: one output per thread, sequential fp32 accumulation over k
template <int WBITS, int DT>
__global__ __launch_bounds__(kBlock) void wq16_general(WqArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= a.M * a.N) return;
    const int64_t m = idx / a.N, n = idx - m * a.N;
    const int64_t G = (a.K + a.group - 1) / a.group;
    float acc = 0.f;
    for (int64_t k = 0; k < a.K; ++k) {
        float xv = load_scalar<DT>(a.x, m * a.K + k);
        if (a.smooth) xv = round_to<DT>(xv * load_scalar<DT>(a.smooth, k));
        float u;
        if constexpr (WBITS == 4) {
            const uint32_t byte = a.wq[n * (a.K / 2) + k / 2];
            u = (float)((k & 1) ? (byte >> 4) : (byte & 0xFu));
        } else {
            u = (float)((int)reinterpret_cast<const int8_t*>(a.wq)[n * a.K + k] + 128);
        }
        const int64_t gi = n * G + k / a.group;
        const float w = round_to<DT>((u - wq_zero<WBITS>(a, gi)) * wq_scale(a, gi));
        acc = acc + xv * w;
    }
    if (a.bias) acc = acc + a.bias[n];
    a.out[m * a.N + n] = (uint16_t)to_bits16<DT>(acc);
}

template <int WBITS, int DT>
static int wq16_dispatch(WqArgs a, hipStream_t st) {
    const bool vec_ok = aligned16(a.x) && aligned16(a.wq) && (!a.smooth || aligned16(a.smooth)) && a.group % 32 == 0 &&
                        a.K % a.group == 0 && a.K < 65536 && a.group < 65536;
    if (vec_ok && a.M <= 64 && a.K % 128 == 0) {
        const dim3 grid((unsigned)((a.N + kGDN - 1) / kGDN));
        const int iters = (int)(a.K / 128);
#define AMCT_WQ_DEC2(MT, SM)                                                                                       \
    {                                                                                                              \
        if (iters % 4 == 0) hipLaunchKernelGGL((wq16_decode<WBITS, DT, MT, 4, SM>), grid, dim3(256), 0, st, a);   \
        else hipLaunchKernelGGL((wq16_decode<WBITS, DT, MT, 1, SM>), grid, dim3(64), 0, st, a);                    \
    }
#define AMCT_WQ_DEC(MT)                                                                                            \
    {                                                                                                              \
        if (a.smooth) AMCT_WQ_DEC2(MT, true) else AMCT_WQ_DEC2(MT, false)                                          \
    }
        if (a.M <= 16) AMCT_WQ_DEC(1)
        else if (a.M <= 32) AMCT_WQ_DEC(2)
        else AMCT_WQ_DEC(4)
#undef AMCT_WQ_DEC2
#undef AMCT_WQ_DEC
        return hip_status();
    }
    if (vec_ok && a.K % kGK == 0) {
        const dim3 grid((unsigned)((a.N + kGN - 1) / kGN), (unsigned)((a.M + kGM - 1) / kGM));
        if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
        hipLaunchKernelGGL((wq16_tile<WBITS, DT>), grid, dim3(kBlock), 0, st, a);
        return hip_status();
    }
    const int64_t nb = (a.M * a.N + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL((wq16_general<WBITS, DT>), dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    return hip_status();
}

// int4 weights with fp16 activations: called by amct_gemm_w4a16
int wq16_int4_f16(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                  const uint8_t* zeros, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                  hipStream_t st) {
    WqArgs a{(const uint16_t*)x, (const uint16_t*)smooth, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group,
             scale_dtype, (uint32_t)(0x100000000ull / (uint64_t)group) + 1u};
    return wq16_dispatch<4, AMCT_F16>(a, st);
}

}  // namespace amct

namespace amct {

// ---------------------------------------------------------------------------
// int8 weights, many rows: the weight is dequantised once into the caller's workspace, dt((q - offset) * scale) as the
// tile kernel above computes it per block, and the product is the plain 16-bit GEMM on the 256x256 tiles of the W8A8
// kernel (gemm_w8a8.hip: gemm16_tiles); the activations are smoothed into the workspace first when asked for.
// ---------------------------------------------------------------------------
// A thread takes 8 weights at a time (8 bytes in, 16 bytes out; group % 8 == 0, so they share a group), the threads of
// a block walk along kW8Rows rows at once: a wave reads 512 and writes 1024 contiguous bytes per row and step.  The
// first `wblocks` blocks of the launch dequantise; the others, if any, smooth the activations into `xs` (two independent
// passes in one launch: the short one runs beside the long one).
constexpr int kW8Rows = 4;
template <int DT>
AMCT_DEV void smooth_rows_dt_body(const uint16_t* x, const uint16_t* smooth, uint16_t* y, int64_t nvec, int kvec, unsigned block, unsigned nblocks) {
    const int64_t stride = (int64_t)nblocks * kBlock;
    for (int64_t v = (int64_t)block * kBlock + threadIdx.x; v < nvec; v += stride)
        stg16(y + v * 8, smooth8_dt<DT>(ldg16_nt(x + v * 8), ldg16(smooth + (v % kvec) * 8)));
}
template <int DT>
__global__ __launch_bounds__(kBlock) void w8_dequant_rows(WqArgs a, uint16_t* wdq, uint16_t* xs, unsigned wblocks) {
    if (blockIdx.x >= wblocks) {
        smooth_rows_dt_body<DT>(a.x, a.smooth, xs, a.M * a.K / 8, (int)(a.K / 8), blockIdx.x - wblocks, gridDim.x - wblocks);
        return;
    }
    const uint32_t kv = (uint32_t)(a.K >> 3), G = (uint32_t)(a.K / a.group);
    const bool small_k = a.K < 65536;                               // k / group by the multiply-high then
    const int64_t row0 = (int64_t)blockIdx.x * kW8Rows;
    for (uint32_t v = threadIdx.x; v < kv; v += kBlock) {
        const uint32_t k = v * 8;
        const uint32_t g = small_k ? __umulhi(k, a.group_magic) : k / (uint32_t)a.group;
        u2v w[kW8Rows];
        float sc[kW8Rows], nzs[kW8Rows];
#pragma unroll
        for (int r = 0; r < kW8Rows; ++r) {
            const int64_t row = row0 + r < a.N ? row0 + r : a.N - 1;
            const int64_t gi = row * G + g;
            w[r] = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(a.wq + row * a.K) + v);
            sc[r] = wq_scale(a, gi);
            nzs[r] = -(wq_zero<8>(a, gi) * sc[r]);
        }
#pragma unroll
        for (int r = 0; r < kW8Rows; ++r)
            if (row0 + r < a.N) stg16(wdq + (row0 + r) * a.K + k, dq8_int8<DT>(w[r].x, w[r].y, sc[r], nzs[r]));
    }
}

int gemm16_tiles(const void* x, const void* w, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int dtype,
                 void* workspace, size_t workspace_bytes, hipStream_t st);   // gemm_w8a8.hip
size_t gemm16_part_bytes(int64_t M, int64_t N, int64_t K);  // gemm_w8a8.hip: partial sums it wants lent for few tiles

static size_t w8a16_tiles_workspace(int64_t M, int64_t N, int64_t K, int group, int has_smooth) {
    if (M < 256 || N <= 0 || K <= 0 || group <= 0 || K % 64 != 0 || K % 16 != 0 || group % 16 != 0 || K % group != 0 || N % 8 != 0 ||
        N * K * 2 >= (int64_t(1) << 32) || M * K * 2 >= (int64_t(1) << 32))
        return 0;
    return (size_t)N * (size_t)K * 2 + (has_smooth ? (size_t)M * (size_t)K * 2 : 0) + gemm16_part_bytes(M, N, K);
}

int w8a16_stream_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                          const uint8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                          int dtype, void* workspace, size_t workspace_bytes, hipStream_t st);      // gemm_w8a16_stream.hip
size_t w8a16_stream_part_bytes(int64_t M, int64_t N, int64_t K, int group);   // partial sums of its launches over slices of K
bool w8a16_stream_takes(int64_t M, int64_t N, int64_t K, int group, size_t workspace_bytes);
int w8a16_spec_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                        const uint8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group, int dtype,
                        void* workspace, size_t workspace_bytes, hipStream_t st);   // gemm_w4a16.hip
size_t w8a16_spec_part_bytes(int64_t M, int64_t N, int64_t K, int group);         // gemm_w4a16.hip
}

using namespace amct;

extern "C" size_t amct_gemm_w8a16_workspace_bytes(int64_t M, int64_t N, int64_t K, int group, int has_smooth) {
    if (M <= 0 || N <= 0 || K <= 0 || group <= 0) return 0;
    // tile kernels: x * smooth done once; long rows on few column blocks: the partial sums of the K slices behind it
    const size_t part = w8a16_spec_part_bytes(M, N, K, group);
    const size_t spec = (has_smooth && (M > 16 || part) ? (size_t)M * (size_t)K * 2 : 0) + part;
    const size_t two = w8a16_tiles_workspace(M, N, K, group, has_smooth);   // many rows: the 16-bit weight as well
    const size_t stream = w8a16_stream_part_bytes(M, N, K, group);          // a few rows, K in slices: its partial sums
    const size_t most = two > spec ? two : spec;
    return most > stream ? most : stream;
}

extern "C" int amct_gemm_w8a16_weight_rounded(int64_t M, int64_t N, int64_t K, int group, int dtype, size_t workspace_bytes) {
    if (M < 0 || N <= 0 || K <= 0 || group <= 0) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    // the weight-streaming kernel is the only one that keeps the integer weight; amct_gemm_w8a16_ws tries it first
    return M <= 16 && w8a16_stream_takes(M, N, K, group, workspace_bytes) ? 0 : 1;
}

extern "C" int amct_gemm_w8a16(const void* x, const void* smooth, const int8_t* wq, const void* scales, int scale_dtype,
                               const int8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K,
                               int group, int dtype, amct_stream_t stream) {
    return amct_gemm_w8a16_ws(x, smooth, wq, scales, scale_dtype, offsets, bias, out, M, N, K, group, dtype, nullptr, 0, stream);
}

extern "C" int amct_gemm_w8a16_ws(const void* x, const void* smooth, const int8_t* wq, const void* scales, int scale_dtype,
                                  const int8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K,
                                  int group, int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream) {
    if (M < 0 || N <= 0 || K <= 0 || group <= 0) return AMCT_E_BADARG;
    if (M != 0 && (!x || !wq || !scales || !out)) return AMCT_E_BADARG;
    if (scale_dtype != AMCT_F16 && scale_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    if (K % group != 0) return AMCT_E_ALIGN;
    if (M == 0) return AMCT_OK;
    WqArgs a{(const uint16_t*)x, (const uint16_t*)smooth, reinterpret_cast<const uint8_t*>(wq), scales,
             reinterpret_cast<const uint8_t*>(offsets), bias, (uint16_t*)out, M, N, K, group, scale_dtype,
             (uint32_t)(0x100000000ull / (uint64_t)group) + 1u};
    hipStream_t st = (hipStream_t)stream;
    if (M <= 16) {                                   // K of 1024 / 2048 / 4096, groups of 128 .. K: the weight-streaming kernel
        const int rc = w8a16_stream_dispatch(x, smooth, reinterpret_cast<const uint8_t*>(wq), scales, scale_dtype,
                                             reinterpret_cast<const uint8_t*>(offsets), bias, out, M, N, K, group, dtype, workspace,
                                             workspace_bytes, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    if (M > 16 || w8a16_spec_part_bytes(M, N, K, group)) {   // the tile kernels with specialised waves (a few rows: only with K split)
        const int rc = w8a16_spec_dispatch(x, smooth, reinterpret_cast<const uint8_t*>(wq), scales, scale_dtype,
                                           reinterpret_cast<const uint8_t*>(offsets), bias, out, M, N, K, group, dtype, workspace,
                                           workspace_bytes, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    // many rows and a lent workspace: dequantise once, then the plain 16-bit GEMM on the large tiles
    const size_t full = w8a16_tiles_workspace(M, N, K, group, smooth != nullptr);
    const size_t need = full ? full - gemm16_part_bytes(M, N, K) : 0;      // the partial sums are optional
    if (need && workspace && workspace_bytes >= need && aligned16(workspace) && aligned16(x) && aligned16(wq) && aligned16(out) &&
        (!smooth || aligned16(smooth)) && (reinterpret_cast<uintptr_t>(scales) & 1u) == 0) {
        uint16_t* wdq = reinterpret_cast<uint16_t*>(workspace);
        uint16_t* xs = wdq + (size_t)N * (size_t)K;
        const int64_t wblocks = (N + kW8Rows - 1) / kW8Rows;
        int64_t sblocks = 0;
        if (smooth) {                                               // about 4 vectors of 16 bytes per thread
            sblocks = (M * K / 8 + 4 * kBlock - 1) / (4 * kBlock);
            if (sblocks > 16384) sblocks = 16384;
        }
        const dim3 grid((unsigned)(wblocks + sblocks));             // N * K < 2^31 (workspace check): far below the grid limit
        if (dtype == AMCT_BF16) hipLaunchKernelGGL((w8_dequant_rows<AMCT_BF16>), grid, dim3(kBlock), 0, st, a, wdq, xs, (unsigned)wblocks);
        else hipLaunchKernelGGL((w8_dequant_rows<AMCT_F16>), grid, dim3(kBlock), 0, st, a, wdq, xs, (unsigned)wblocks);
        const void* xa = smooth ? (const void*)xs : x;
        const int rc = gemm16_tiles(xa, wdq, bias, out, M, N, K, dtype, reinterpret_cast<char*>(workspace) + need, workspace_bytes - need, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
        // (the two preparatory kernels above only wrote the workspace: the call below starts from the caller's operands)
    }
    return dtype == AMCT_BF16 ? wq16_dispatch<8, AMCT_BF16>(a, st) : wq16_dispatch<8, AMCT_F16>(a, st);
}
