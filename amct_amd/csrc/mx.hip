// K4: microscaling block-32 quantise / dequantise (FP8 E4M3 and FP4 E2M1 elements,
// E8M0 shared exponents).  The reference has no such code; the format rules are:
//   byte  = clamp(biased_exp(amax) - emax_elem, 0, 254)   (0xFF when the block holds a NaN)
//   elem  = cast(x * 2^-(byte-127)), round-half-even, saturating to +-448 / +-6
//   fp4   : two codes per byte, even column in the low nibble
// Two element encoders are compiled: a bit-manipulation one and one using the gfx950
// v_cvt_scalef32_pk_* instructions (pre-clamped so that the result saturates).
#include "amct_common.h"

namespace amct {

typedef short v2i16 __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int kFmtE4M3 = 0, kFmtE2M1 = 1;

// ---- software element casts -------------------------------------------------------------
AMCT_DEV uint32_t sw_e4m3(float v) {
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;
    a = min(a, 0x43E00000u);                                   // 448.0f
    uint32_t code;
    if (a >= 0x3C800000u) {                                    // >= 2^-6: normal
        const uint32_t r = a + 0x7FFFFu + ((a >> 20) & 1u);
        code = (r >> 20) - (120u << 3);
    } else {                                                   // subnormal: units of 2^-9
        const float f = __uint_as_float(a) + 16384.0f;
        code = __float_as_uint(f) - 0x46800000u;
    }
    return sign | code;
}

AMCT_DEV uint32_t sw_e2m1(float v) {
    const uint32_t u = __float_as_uint(v);
    const uint32_t sign = (u >> 28) & 0x8u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 7u;
    a = min(a, 0x40C00000u);                                   // 6.0f
    uint32_t code;
    if (a >= 0x3F800000u) {                                    // >= 1.0: normal, 1 mantissa bit
        const uint32_t r = a + 0x1FFFFFu + ((a >> 22) & 1u);
        code = (r >> 22) - (126u << 1);
    } else {                                                   // units of 0.5
        const float f = __uint_as_float(a) + 4194304.0f;       // 2^22: ulp 0.5
        code = __float_as_uint(f) - 0x4A800000u;
    }
    return sign | code;
}

AMCT_DEV float sw_dec_e4m3(uint32_t c) {
    const uint32_t a = c & 0x7Fu;
    float f;
    if (a == 0x7Fu) f = __uint_as_float(0x7FC00000u);
    else if (a >= 8u) f = __uint_as_float((a << 20) + (120u << 23));
    else f = (float)a * 0.001953125f;                          // 2^-9
    return (c & 0x80u) ? -f : f;
}

AMCT_DEV float sw_dec_e2m1(uint32_t c) {
    const uint32_t a = c & 7u;
    float f;
    if (a >= 2u) f = __uint_as_float((a << 22) + (126u << 23));
    else f = (float)a * 0.5f;
    return (c & 8u) ? -f : f;
}

// 2^(byte-127) as fp32; byte 0 is the denormal 2^-127, byte 255 a NaN
AMCT_DEV float e8m0_to_f32(uint32_t byte) {
    if (byte == 0u) return __uint_as_float(0x00400000u);
    if (byte == 255u) return __uint_as_float(0x7FC00000u);
    return __uint_as_float(byte << 23);
}

// ---- quantise -------------------------------------------------------------------------------
// One 16-byte vector per lane and step; a block of 32 elements spans T = 32/VEC lanes.
template <int DT, int FMT, bool HW, int U>
__global__ __launch_bounds__(kBlock) void mx_quant_k(const void* x, uint8_t* el, uint8_t* e8, int64_t nvec, int scale_mode) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    constexpr int T = 32 / VEC;
    constexpr int EMAX = (FMT == kFmtE4M3) ? 8 : 2;
    constexpr uint32_t FMAX_MAN = (FMT == kFmtE4M3) ? 0x600000u : 0x400000u;
    constexpr float FMAX = (FMT == kFmtE4M3) ? 448.0f : 6.0f;
    const int tid = threadIdx.x;
    float v[U][VEC];
    int64_t gv[U];
    uint4 raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        gv[u] = ((int64_t)blockIdx.x * U + u) * kBlock + tid;
        // unconditional streaming load (index clamped; whole blocks of 32 are valid or not together)
        raw[u] = ldg16_nt(reinterpret_cast<const char*>(x) + (gv[u] < nvec ? gv[u] : nvec - 1) * 16);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        unpack16<DT>(raw[u], v[u]);
        uint32_t amax = 0;
#pragma unroll
        for (int j = 0; j < VEC; ++j) amax = max(amax, __float_as_uint(v[u][j]) & 0x7FFFFFFFu);
        amax = team_umax<T>(amax);
        const bool has_nan = amax > 0x7F800000u;
        int be = (int)(amax >> 23) - EMAX;
        if (scale_mode == 1) be += ((amax & 0x7FFFFFu) > FMAX_MAN) ? 1 : 0;
        be = has_nan ? 254 : min(max(be, 0), 254);             // a NaN block is cast at the largest scale
        const uint32_t byte = has_nan ? 255u : (uint32_t)be;
        // x * 2^-(be-127) as two exact power-of-two factors (a single one may not be representable)
        const int e = be - 127;
        const int h = e >> 1;                                  // floor(e / 2)
        const float f1 = __uint_as_float((uint32_t)(127 - h) << 23);
        const float f2 = __uint_as_float((uint32_t)(127 - (e - h)) << 23);
        uint32_t codes[VEC];
        if constexpr (HW) {
            // hardware cast of (value / scale); pre-clamp so that overflow saturates
            const float scale = 1.0f;
            float t[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                t[j] = v[u][j] * f1 * f2;
                t[j] = __builtin_amdgcn_fmed3f(t[j], -FMAX, FMAX);     // NaN handled below
            }
            if constexpr (FMT == kFmtE4M3) {
#pragma unroll
                for (int j = 0; j < VEC; j += 4) {
                    v2i16 o = {0, 0};
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, t[j], t[j + 1], scale, false);
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, t[j + 2], t[j + 3], scale, true);
                    const uint32_t w = __builtin_bit_cast(uint32_t, o);
                    codes[j] = w & 0xFFu; codes[j + 1] = (w >> 8) & 0xFFu; codes[j + 2] = (w >> 16) & 0xFFu; codes[j + 3] = w >> 24;
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j += 4) {
                    uint32_t w = 0;
                    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[j], t[j + 1], scale, 0);
                    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[j + 2], t[j + 3], scale, 1);
                    codes[j] = w & 0xFu; codes[j + 1] = (w >> 4) & 0xFu; codes[j + 2] = (w >> 8) & 0xFu; codes[j + 3] = (w >> 12) & 0xFu;
                }
            }
            if (has_nan) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float tt = v[u][j] * f1 * f2;
                    codes[j] = (FMT == kFmtE4M3) ? sw_e4m3(tt) : sw_e2m1(tt);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float tt = v[u][j] * f1 * f2;
                codes[j] = (FMT == kFmtE4M3) ? sw_e4m3(tt) : sw_e2m1(tt);
            }
        }
        if (gv[u] < nvec) {
            if constexpr (FMT == kFmtE4M3) {
                uint32_t w[VEC / 4];
#pragma unroll
                for (int j = 0; j < VEC / 4; ++j)
                    w[j] = codes[4 * j] | (codes[4 * j + 1] << 8) | (codes[4 * j + 2] << 16) | (codes[4 * j + 3] << 24);
                uint32_t* p = reinterpret_cast<uint32_t*>(el + gv[u] * VEC);
                if constexpr (VEC == 8) stg8_nt(p, w[0], w[1]);
                else stg4_nt(p, w[0]);
            } else {
                uint32_t w = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) w |= codes[j] << (4 * j);
                if constexpr (VEC == 8) stg4_nt(el + gv[u] * 4, w);
                else *reinterpret_cast<uint16_t*>(el + gv[u] * 2) = (uint16_t)w;
            }
            if ((tid & (T - 1)) == 0) e8[gv[u] / T] = (uint8_t)byte;
        }
    }
}

// ---- quantise, complete blocks of U * 256 vectors -------------------------------------------------
// Same results as mx_quant_k; what differs is the instruction count (about 4.5 vector instructions per bf16 element
// against 9.4, and no 64-bit address arithmetic).  The element cast is the hardware's scaled conversion
// (v_cvt_scalef32_pk_{fp8,fp4}_{bf16,f32}: cast(value / scale), scale a power of two taken from the block
// exponent), so nothing is multiplied.  Checked against the product form over every bf16 pattern and block
// exponents from -126 to 125: the FP4 conversion saturates by itself, the FP8 one turns magnitudes above the
// format's largest into NaN, hence the clamp to 448 * scale before it -- for bf16 input on the packed 16-bit
// magnitudes (v_pk_min_u16; sign-magnitude order equals unsigned order), with the block maximum found the same
// way (v_pk_max_u16).  Addresses are one wave-uniform base per block plus a 32-bit lane offset.
// A wave that holds a block with an infinity, a NaN or a block exponent of zero (maximum below 2^(emax-126): the
// scale is then a denormal) takes the general routine for all of its blocks.
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef unsigned short v2u16 __attribute__((ext_vector_type(2)));
AMCT_DEV uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2u16, a), __builtin_bit_cast(v2u16, b)));
}
AMCT_DEV uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(v2u16, a), __builtin_bit_cast(v2u16, b)));
}

// general routine for one vector per lane (every lane of the wave calls it): returns the block byte, fills the
// packed element codes (8, 4 or 2 bytes in w[0], w[1])
template <int DT, int FMT>
AMCT_DEV uint32_t mx_quant_vec_general(const uint4& raw, int scale_mode, uint32_t (&w)[2]) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int T = 32 / VEC;
    constexpr int EMAX = (FMT == kFmtE4M3) ? 8 : 2;
    constexpr uint32_t FMAX_MAN = (FMT == kFmtE4M3) ? 0x600000u : 0x400000u;
    float v[VEC];
    unpack16<DT>(raw, v);
    uint32_t amax = 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) amax = max(amax, __float_as_uint(v[j]) & 0x7FFFFFFFu);
    amax = team_umax<T>(amax);
    const bool has_nan = amax > 0x7F800000u;
    int be = (int)(amax >> 23) - EMAX;
    if (scale_mode == 1) be += ((amax & 0x7FFFFFu) > FMAX_MAN) ? 1 : 0;
    be = has_nan ? 254 : min(max(be, 0), 254);
    const int e = be - 127;
    const int h = e >> 1;
    const float f1 = __uint_as_float((uint32_t)(127 - h) << 23);
    const float f2 = __uint_as_float((uint32_t)(127 - (e - h)) << 23);
    w[0] = 0; w[1] = 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        const float tt = v[j] * f1 * f2;
        if constexpr (FMT == kFmtE4M3) w[j / 4] |= sw_e4m3(tt) << (8 * (j % 4));
        else w[0] |= sw_e2m1(tt) << (4 * j);
    }
    return has_nan ? 255u : (uint32_t)be;
}

template <int DT, int FMT, int U>
__global__ __launch_bounds__(kBlock) void mx_quant_full(const void* x, uint8_t* el, uint8_t* e8, int scale_mode, int64_t nchunks) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int T = 32 / VEC;
    constexpr int OB = (FMT == kFmtE4M3) ? VEC : VEC / 2;           // output bytes per vector
    constexpr int EMAX = (FMT == kFmtE4M3) ? 8 : 2;
    constexpr uint32_t FMAX_MAN = (FMT == kFmtE4M3) ? 0x600000u : 0x400000u;
    constexpr uint32_t FMAX_BITS = (FMT == kFmtE4M3) ? 0x43E00000u : 0x40C00000u;
    const uint32_t tid = threadIdx.x;
    uint4 nxt[U];
    if ((int64_t)blockIdx.x < nchunks) {
        const char* xb = reinterpret_cast<const char*>(x) + (int64_t)blockIdx.x * (U * kBlock * 16);
#pragma unroll
        for (int u = 0; u < U; ++u) nxt[u] = ldg16_nt(xb + (uint32_t)((u * kBlock + tid) * 16));
    }
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const int64_t v0 = c * (U * kBlock);
    uint8_t* eb = el + v0 * OB;
    uint8_t* sb = e8 + v0 / T;
    uint4 raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) raw[u] = nxt[u];
    if (c + gridDim.x < nchunks) {                   // the next chunk's loads fly while this one is converted
        const char* xb = reinterpret_cast<const char*>(x) + (c + gridDim.x) * (U * kBlock * 16);
#pragma unroll
        for (int u = 0; u < U; ++u) nxt[u] = ldg16_nt(xb + (uint32_t)((u * kBlock + tid) * 16));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t r[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
        uint32_t mag[4];
        uint32_t amax;
        if constexpr (DT == AMCT_BF16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) mag[j] = r[j] & 0x7FFF7FFFu;
            const uint32_t a = pk_max_u16(pk_max_u16(mag[0], mag[1]), pk_max_u16(mag[2], mag[3]));
            amax = team_umax<T>(max(a & 0xFFFFu, a >> 16)) << 16;
        } else {
            float v[VEC];
            unpack16<DT>(raw[u], v);
            amax = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) amax = max(amax, __float_as_uint(v[j]) & 0x7FFFFFFFu);
            amax = team_umax<T>(amax);
        }
        int be = (int)(amax >> 23) - EMAX;
        if (scale_mode == 1) be += ((amax & 0x7FFFFFu) > FMAX_MAN) ? 1 : 0;
        const bool special = amax >= 0x7F800000u || (be <= 0 && amax != 0u);
        uint32_t w[2] = {0u, 0u};
        uint32_t byte;
        if (__builtin_amdgcn_ballot_w64(special) != 0ull) {
            byte = mx_quant_vec_general<DT, FMT>(raw[u], scale_mode, w);
        } else {
            byte = (uint32_t)max(be, 0);                          // be <= 254 - EMAX here; 0 only for an all-zero block
            const uint32_t bs = (uint32_t)max(be, 1);
            const float scale = __uint_as_float(bs << 23);
            const uint32_t thr = FMAX_BITS + ((bs - 127u) << 23); // largest element magnitude times the scale
            if constexpr (DT == AMCT_BF16) {
                uint32_t q[4];
                if constexpr (FMT == kFmtE4M3) {
                    const uint32_t thr2 = (thr >> 16) * 0x10001u;
#pragma unroll
                    for (int j = 0; j < 4; ++j) q[j] = (r[j] & 0x80008000u) | pk_min_u16(mag[j], thr2);
                    v2i16 o0 = {0, 0}, o1 = {0, 0};
                    o0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o0, __builtin_bit_cast(v2bf, q[0]), scale, false);
                    o0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o0, __builtin_bit_cast(v2bf, q[1]), scale, true);
                    o1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o1, __builtin_bit_cast(v2bf, q[2]), scale, false);
                    o1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o1, __builtin_bit_cast(v2bf, q[3]), scale, true);
                    w[0] = __builtin_bit_cast(uint32_t, o0);
                    w[1] = __builtin_bit_cast(uint32_t, o1);
                } else {
                    uint32_t o = 0;
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(v2bf, r[0]), scale, 0);
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(v2bf, r[1]), scale, 1);
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(v2bf, r[2]), scale, 2);
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(v2bf, r[3]), scale, 3);
                    w[0] = o;
                }
            } else {
                float v[VEC];
                unpack16<DT>(raw[u], v);
                const float lim = __uint_as_float(thr);
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] = __builtin_amdgcn_fmed3f(v[j], -lim, lim);
                if constexpr (FMT == kFmtE4M3) {
#pragma unroll
                    for (int j = 0; j < VEC / 4; ++j) {
                        v2i16 o = {0, 0};
                        o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, v[4 * j], v[4 * j + 1], scale, false);
                        o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, v[4 * j + 2], v[4 * j + 3], scale, true);
                        w[j] = __builtin_bit_cast(uint32_t, o);
                    }
                } else {
                    uint32_t o = 0;
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, v[0], v[1], scale, 0);
                    o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, v[2], v[3], scale, 1);
                    if constexpr (VEC == 8) {
                        o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, v[4], v[5], scale, 2);
                        o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, v[6], v[7], scale, 3);
                    }
                    w[0] = o;
                }
            }
        }
        const uint32_t idx = u * kBlock + tid;
        if constexpr (OB == 8) stg8_nt(eb + idx * 8u, w[0], w[1]);
        else if constexpr (OB == 4) stg4_nt(eb + idx * 4u, w[0]);
        else *reinterpret_cast<uint16_t*>(eb + idx * 2u) = (uint16_t)w[0];
        if ((tid & (T - 1)) == 0) sb[idx / T] = (uint8_t)byte;
    }
    }
}

// ---- dequantise -------------------------------------------------------------------------------
// One lane produces one 16-byte output vector (VEC elements of the output dtype) per step, U steps in
// flight.  Element codes are decoded by the hardware conversions (v_cvt_pk_f32_fp8, v_cvt_scalef32_pk_f32_fp4
// with scale 1: two codes per instruction, exact; a table in LDS was 4 % slower); the product with the block
// scale is the same fp32 multiplication as in the element-wise form.
template <int DT, int FMT, int U>
__global__ __launch_bounds__(kBlock) void mx_dequant_k(const uint8_t* el, const uint8_t* e8, void* y, int64_t nvec) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int T = 32 / VEC;
    constexpr int EB = FMT == kFmtE4M3 ? VEC : VEC / 2;         // element bytes per output vector
    const int tid = threadIdx.x;
    const int64_t chunk = (int64_t)kBlock * U;
    const int64_t nchunks = (nvec + chunk - 1) / chunk;
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        uint32_t w[U][2];
        uint32_t sb[U];
        int64_t gv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            gv[u] = c * chunk + u * kBlock + tid;
            const int64_t g = gv[u] < nvec ? gv[u] : nvec - 1;  // clamped: loads are unconditional
            sb[u] = e8[g / T];
            w[u][1] = 0;
            if constexpr (EB == 8) {
                const u2v r = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(el + g * 8));
                w[u][0] = r.x; w[u][1] = r.y;
            } else if constexpr (EB == 4) {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(el + g * 4));
            } else {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(el + g * 2));
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float sc = e8m0_to_f32(sb[u]);
            float out[VEC];
            // the hardware conversions decode two codes per instruction, exactly; the product with the block
            // scale is then the same fp32 multiplication as in the element-wise form
            if constexpr (FMT == kFmtE4M3) {
#pragma unroll
                for (int j = 0; j < VEC / 2; ++j) {
                    const v2f p = (j & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u][j / 2], true)
                                          : __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u][j / 2], false);
                    out[2 * j] = p.x * sc;
                    out[2 * j + 1] = p.y * sc;
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC / 2; ++j) {
                    v2f p;
                    if (j == 0) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 0);
                    else if (j == 1) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 1);
                    else if (j == 2) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 2);
                    else p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 3);
                    out[2 * j] = p.x * sc;
                    out[2 * j + 1] = p.y * sc;
                }
            }
            if (gv[u] < nvec) stg16_nt(reinterpret_cast<char*>(y) + gv[u] * 16, pack16<DT>(out));
        }
    }
}

// Complete blocks of U * 256 vectors go to mx_quant_full; the rest (and everything, when the bit-manipulation cast is
// asked for) to mx_quant_k.  Both give the same codes.
// complete blocks of U * 256 output vectors: one wave-uniform base per block, 32-bit lane offsets, nothing clamped
template <int DT, int FMT, int U>
__global__ __launch_bounds__(kBlock) void mx_dequant_full(const uint8_t* el, const uint8_t* e8, void* y, int64_t nchunks) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int T = 32 / VEC;
    constexpr int EB = FMT == kFmtE4M3 ? VEC : VEC / 2;         // element bytes per output vector
    const uint32_t tid = threadIdx.x;
    auto load = [&](int64_t c, uint32_t (&w)[U][2], uint32_t (&sb)[U]) {
        const int64_t v0 = c * (U * kBlock);
        const uint8_t* eb = el + v0 * EB;
        const uint8_t* sbp = e8 + v0 / T;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t idx = u * kBlock + tid;
            sb[u] = sbp[idx / T];
            w[u][1] = 0;
            if constexpr (EB == 8) {
                const u2v r = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(eb + idx * 8u));
                w[u][0] = r.x; w[u][1] = r.y;
            } else if constexpr (EB == 4) {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(eb + idx * 4u));
            } else {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(eb + idx * 2u));
            }
        }
    };
    uint32_t wn[U][2], sn[U];
    if ((int64_t)blockIdx.x < nchunks) load(blockIdx.x, wn, sn);
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
    char* yb = reinterpret_cast<char*>(y) + c * (U * kBlock * 16);
    uint32_t w[U][2];
    uint32_t sb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) { w[u][0] = wn[u][0]; w[u][1] = wn[u][1]; sb[u] = sn[u]; }
    if (c + gridDim.x < nchunks) load(c + gridDim.x, wn, sn);    // the next chunk's loads fly while this one is decoded
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const float sc = e8m0_to_f32(sb[u]);
        float out[VEC];
        if constexpr (FMT == kFmtE4M3) {
#pragma unroll
            for (int j = 0; j < VEC / 2; ++j) {
                const v2f p = (j & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u][j / 2], true)
                                      : __builtin_amdgcn_cvt_pk_f32_fp8((int)w[u][j / 2], false);
                out[2 * j] = p.x * sc;
                out[2 * j + 1] = p.y * sc;
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC / 2; ++j) {
                v2f p;
                if (j == 0) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 0);
                else if (j == 1) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 1);
                else if (j == 2) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 2);
                else p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[u][0], 1.0f, 3);
                out[2 * j] = p.x * sc;
                out[2 * j + 1] = p.y * sc;
            }
        }
        stg16_nt(yb + (u * kBlock + tid) * 16u, pack16<DT>(out));
    }
    }
}

// Launch shapes of the complete-chunk kernels, measured on X[8192,4096] bf16 (kernels loop over chunks with the next
// chunk's loads in flight; a cap above the chunk count means one chunk per block).  Quantise, 2 vectors per lane and one
// chunk per block: 17.3 / 14.6 us (FP8 / FP4); 4 vectors: 17.65 / 14.7; 8 vectors, 4 blocks per CU looping: 19.3 / 16.3.
// Dequantise, 8 vectors per lane and 3 blocks per CU: 17.4 us; 4 vectors, one chunk per block: 17.95; 8 vectors and 2 / 4 / 5
// blocks per CU: 18.9 / 18.1 / 18.0.
constexpr int kMxQuantU = 2, kMxQuantBlocksPerCu = 32;
constexpr int kMxDequantU = 8, kMxDequantBlocksPerCu = 3;

template <int DT, int FMT>
static int launch_quant(const void* x, uint8_t* el, uint8_t* e8, int64_t nvec, int scale_mode, bool hw, hipStream_t st) {
    constexpr int U = 4, UF = kMxQuantU;
    constexpr int VEC = Tr<DT>::VEC;
    if (hw) {
        const int64_t full = nvec / ((int64_t)kBlock * UF), cap = (int64_t)kMxQuantBlocksPerCu * 256;
        if (full > 0) {
            hipLaunchKernelGGL((mx_quant_full<DT, FMT, UF>), dim3((unsigned)(full > cap ? cap : full)), dim3(kBlock), 0, st, x, el, e8, scale_mode, full);
            const int64_t done = full * kBlock * UF;
            x = reinterpret_cast<const char*>(x) + done * 16;
            el += done * (FMT == kFmtE4M3 ? VEC : VEC / 2);
            e8 += done / (32 / VEC);
            nvec -= done;
            if (nvec == 0) return hip_status();
        }
    }
    const int64_t nb = (nvec + (int64_t)kBlock * U - 1) / ((int64_t)kBlock * U);
    if (hw) hipLaunchKernelGGL((mx_quant_k<DT, FMT, true, U>), dim3((unsigned)nb), dim3(kBlock), 0, st, x, el, e8, nvec, scale_mode);
    else hipLaunchKernelGGL((mx_quant_k<DT, FMT, false, U>), dim3((unsigned)nb), dim3(kBlock), 0, st, x, el, e8, nvec, scale_mode);
    return hip_status();
}

template <int DT, int FMT>
static int launch_dequant(const uint8_t* el, const uint8_t* e8, void* y, int64_t nvec, hipStream_t st) {
    constexpr int U = 4, UF = kMxDequantU;
    constexpr int VEC = Tr<DT>::VEC;
    const int64_t full = nvec / ((int64_t)kBlock * UF), cap = (int64_t)kMxDequantBlocksPerCu * 256;
    if (full > 0) {
        hipLaunchKernelGGL((mx_dequant_full<DT, FMT, UF>), dim3((unsigned)(full > cap ? cap : full)), dim3(kBlock), 0, st, el, e8, y, full);
        const int64_t done = full * kBlock * UF;
        el += done * (FMT == kFmtE4M3 ? VEC : VEC / 2);
        e8 += done / (32 / VEC);
        y = reinterpret_cast<char*>(y) + done * 16;
        nvec -= done;
        if (nvec == 0) return hip_status();
    }
    int64_t nb = (nvec + (int64_t)kBlock * U - 1) / ((int64_t)kBlock * U);
    if (nb > 4096) nb = 4096;                                     // blocks loop over chunks
    hipLaunchKernelGGL((mx_dequant_k<DT, FMT, U>), dim3((unsigned)nb), dim3(kBlock), 0, st, el, e8, y, nvec);
    return hip_status();
}

}  // namespace amct

using namespace amct;

// scale_mode: bit 0 = 0 floor / 1 round-up; bit 8 set selects the bit-manipulation element cast
// instead of the hardware conversion instructions (both give identical codes).
extern "C" int amct_mx_quant(const void* x, uint8_t* elems, uint8_t* e8m0, int64_t rows, int64_t cols, int fmt,
                             int scale_mode, int dtype, amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || (rows != 0 && (!x || !elems || !e8m0))) return AMCT_E_BADARG;   // rows == 0 reads nothing
    if (fmt != kFmtE4M3 && fmt != kFmtE2M1) return AMCT_E_BADARG;
    if ((scale_mode & ~0x101) != 0) return AMCT_E_BADARG;
    if (cols % 32 != 0 || !aligned16(x) || (reinterpret_cast<uintptr_t>(elems) & 7u) != 0) return AMCT_E_ALIGN;
    if (rows == 0) return AMCT_OK;
    const bool hw = (scale_mode & 0x100) == 0;
    const int mode = scale_mode & 1;
    hipStream_t st = (hipStream_t)stream;
    const int64_t n = rows * cols;
#define AMCT_MXQ(DT)                                                                                   \
    return fmt == kFmtE4M3 ? launch_quant<DT, kFmtE4M3>(x, elems, e8m0, n / Tr<DT>::VEC, mode, hw, st) \
                           : launch_quant<DT, kFmtE2M1>(x, elems, e8m0, n / Tr<DT>::VEC, mode, hw, st);
    switch (dtype) {
        case AMCT_F32: AMCT_MXQ(AMCT_F32)
        case AMCT_F16: AMCT_MXQ(AMCT_F16)
        case AMCT_BF16: AMCT_MXQ(AMCT_BF16)
        default: return AMCT_E_BADARG;
    }
#undef AMCT_MXQ
}

extern "C" int amct_mx_dequant(const uint8_t* elems, const uint8_t* e8m0, void* y, int64_t rows, int64_t cols, int fmt,
                               int dtype, amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || (rows != 0 && (!elems || !e8m0 || !y))) return AMCT_E_BADARG;
    if (fmt != kFmtE4M3 && fmt != kFmtE2M1) return AMCT_E_BADARG;
    if (cols % 32 != 0 || !aligned16(y) || (reinterpret_cast<uintptr_t>(elems) & 7u) != 0) return AMCT_E_ALIGN;
    if (rows == 0) return AMCT_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t n = rows * cols;
#define AMCT_MXD(DT)                                                                           \
    return fmt == kFmtE4M3 ? launch_dequant<DT, kFmtE4M3>(elems, e8m0, y, n / Tr<DT>::VEC, st) \
                           : launch_dequant<DT, kFmtE2M1>(elems, e8m0, y, n / Tr<DT>::VEC, st);
    switch (dtype) {
        case AMCT_F32: AMCT_MXD(AMCT_F32)
        case AMCT_F16: AMCT_MXD(AMCT_F16)
        case AMCT_BF16: AMCT_MXD(AMCT_BF16)
        default: return AMCT_E_BADARG;
    }
#undef AMCT_MXD
}
