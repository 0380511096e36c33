// Shared device helpers for the gfx950 kernels: 16-byte vector I/O, dtype
// conversion, wave64 DPP reductions, and the scale/offset closed form.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/amct_hip.h"

namespace amct {

constexpr int kWave = 64;
constexpr int kBlock = 256;

#define AMCT_DEV __device__ __forceinline__

// ---------------------------------------------------------------------------
// dtype traits: VEC = elements in one 16-byte load
// ---------------------------------------------------------------------------
template <int DT> struct Tr;
template <> struct Tr<AMCT_F32> { static constexpr int VEC = 4; static constexpr int BYTES = 4; };
template <> struct Tr<AMCT_F16> { static constexpr int VEC = 8; static constexpr int BYTES = 2; };
template <> struct Tr<AMCT_BF16> { static constexpr int VEC = 8; static constexpr int BYTES = 2; };

AMCT_DEV float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
AMCT_DEV uint32_t f32_to_bf16_bits(float f) {
    // v_cvt_pk_bf16_f32: round-half-even
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
// The empty asm statements pin the fp16 conversions as separate instructions: without them the
// compiler folds "convert, then multiply" into v_fma_mix* with a +0 addend, which turns a -0.0
// product into +0.0.
AMCT_DEV float f16_bits_to_f32(uint32_t h) {
    float f = (float)__builtin_bit_cast(_Float16, (uint16_t)h);
    asm("" : "+v"(f));
    return f;
}
AMCT_DEV uint32_t f32_to_f16_bits(float f) {
    asm("" : "+v"(f));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// round a fp32 value to the precision of DT and back (identity for fp32)
template <int DT> AMCT_DEV float round_to(float f) {
    if constexpr (DT == AMCT_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(f));
    else if constexpr (DT == AMCT_F16) return f16_bits_to_f32(f32_to_f16_bits(f));
    else return f;
}

template <int DT> AMCT_DEV void unpack16(const uint4& v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (DT == AMCT_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(w[i]);
    } else if constexpr (DT == AMCT_BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = f16_bits_to_f32(w[i] & 0xFFFFu);
            f[2 * i + 1] = f16_bits_to_f32(w[i] >> 16);
        }
    }
}

template <int DT> AMCT_DEV uint4 pack16(const float* f) {
    uint32_t w[4];
    if constexpr (DT == AMCT_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = __float_as_uint(f[i]);
    } else if constexpr (DT == AMCT_BF16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = f32_to_bf16_bits(f[2 * i]) | (f32_to_bf16_bits(f[2 * i + 1]) << 16);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = f32_to_f16_bits(f[2 * i]) | (f32_to_f16_bits(f[2 * i + 1]) << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

template <int DT> AMCT_DEV float load_scalar(const void* p, int64_t i) {
    if constexpr (DT == AMCT_F32) return ((const float*)p)[i];
    else if constexpr (DT == AMCT_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    else return f16_bits_to_f32(((const uint16_t*)p)[i]);
}
template <int DT> AMCT_DEV void store_scalar(void* p, int64_t i, float f) {
    if constexpr (DT == AMCT_F32) ((float*)p)[i] = f;
    else if constexpr (DT == AMCT_BF16) ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(f);
    else ((uint16_t*)p)[i] = (uint16_t)f32_to_f16_bits(f);
}

AMCT_DEV uint4 ldg16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
AMCT_DEV void stg16(void* p, const uint4& v) { *reinterpret_cast<uint4*>(p) = v; }

// streaming (non-temporal) variants for data that is read or written exactly once: they bypass
// cache retention and measurably raise copy bandwidth on MI355X
typedef unsigned int u4v __attribute__((ext_vector_type(4)));
typedef unsigned int u2v __attribute__((ext_vector_type(2)));
AMCT_DEV uint4 ldg16_nt(const void* p) {
    const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
AMCT_DEV void stg16_nt(void* p, const uint4& v) {
    __builtin_nontemporal_store(u4v{v.x, v.y, v.z, v.w}, reinterpret_cast<u4v*>(p));
}
AMCT_DEV void stg8_nt(void* p, uint32_t a, uint32_t b) { __builtin_nontemporal_store(u2v{a, b}, reinterpret_cast<u2v*>(p)); }
AMCT_DEV void stg4_nt(void* p, uint32_t a) { __builtin_nontemporal_store(a, reinterpret_cast<uint32_t*>(p)); }

// NaN-propagating max / min (v_maximum3_f32 / v_minimum3_f32), as torch.max does
AMCT_DEV float fmax_nan(float a, float b) { return __builtin_elementwise_maximum(a, b); }
AMCT_DEV float fmin_nan(float a, float b) { return __builtin_elementwise_minimum(a, b); }

// ---------------------------------------------------------------------------
// wave64 reductions.  DPP for distances 1,2 (quad_perm), 4 (row_half_mirror),
// 8 (row_mirror); cross-row distances 16 and 32 go through ds_bpermute.
// All lanes of a team of T consecutive lanes end up with the team's result.
// ---------------------------------------------------------------------------
template <int CTRL> AMCT_DEV float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> AMCT_DEV uint32_t dpp_u(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, CTRL, 0xF, 0xF, true);
}

// value held by lane (lane & ~3) + Q of every quad
template <int Q> AMCT_DEV float quad_bcast(float v) { return dpp_f<Q * 0x55>(v); }

// all lanes of the wave agree that `p` holds
AMCT_DEV bool wave_all(bool p) { return __builtin_amdgcn_ballot_w64(p) == __builtin_amdgcn_ballot_w64(true); }

template <int T> AMCT_DEV void team_minmax(float& mn, float& mx) {
    if constexpr (T >= 2) { mx = fmax_nan(mx, dpp_f<0xB1>(mx)); mn = fmin_nan(mn, dpp_f<0xB1>(mn)); }
    if constexpr (T >= 4) { mx = fmax_nan(mx, dpp_f<0x4E>(mx)); mn = fmin_nan(mn, dpp_f<0x4E>(mn)); }
    if constexpr (T >= 8) { mx = fmax_nan(mx, dpp_f<0x141>(mx)); mn = fmin_nan(mn, dpp_f<0x141>(mn)); }
    if constexpr (T >= 16) { mx = fmax_nan(mx, dpp_f<0x140>(mx)); mn = fmin_nan(mn, dpp_f<0x140>(mn)); }
    if constexpr (T >= 32) { mx = fmax_nan(mx, __shfl_xor(mx, 16)); mn = fmin_nan(mn, __shfl_xor(mn, 16)); }
    if constexpr (T >= 64) { mx = fmax_nan(mx, __shfl_xor(mx, 32)); mn = fmin_nan(mn, __shfl_xor(mn, 32)); }
}

// Reduce 4 (min, max) pairs over a team of T lanes (T >= 4, a power of two) so that lane lt ends up
// with the pair of segment seg4_of_lane(lt), reduced over the whole team: two exchange steps that
// halve the data a lane carries, then plain butterflies.  About half the instructions of four
// independent all-reduces.
AMCT_DEV int seg4_of_lane(int lt) { return ((lt & 1) << 1) | ((lt >> 1) & 1); }

template <int T> AMCT_DEV void team_minmax_scatter4(const float* mn, const float* mx, int lt, float& mn_my, float& mx_my) {
    const bool b0 = lt & 1, b1 = lt & 2;
    // step 1 (partner lt^1): lanes with b0 = 0 keep segments {0,1}, the others {2,3}
    float kn0 = b0 ? mn[2] : mn[0], kn1 = b0 ? mn[3] : mn[1];
    float kx0 = b0 ? mx[2] : mx[0], kx1 = b0 ? mx[3] : mx[1];
    const float gn0 = b0 ? mn[0] : mn[2], gn1 = b0 ? mn[1] : mn[3];          // what the partner keeps
    const float gx0 = b0 ? mx[0] : mx[2], gx1 = b0 ? mx[1] : mx[3];
    kn0 = fmin_nan(kn0, dpp_f<0xB1>(gn0)); kn1 = fmin_nan(kn1, dpp_f<0xB1>(gn1));
    kx0 = fmax_nan(kx0, dpp_f<0xB1>(gx0)); kx1 = fmax_nan(kx1, dpp_f<0xB1>(gx1));
    // step 2 (partner lt^2): lanes with b1 = 0 keep the first of their two, the others the second
    float n = b1 ? kn1 : kn0, x = b1 ? kx1 : kx0;
    const float gn = b1 ? kn0 : kn1, gx = b1 ? kx0 : kx1;
    n = fmin_nan(n, dpp_f<0x4E>(gn));
    x = fmax_nan(x, dpp_f<0x4E>(gx));
    // remaining steps keep lt % 4: rotations by 4 and 8 inside a row of 16, then cross-row shuffles
    if constexpr (T == 8) { n = fmin_nan(n, __shfl_xor(n, 4)); x = fmax_nan(x, __shfl_xor(x, 4)); }
    if constexpr (T >= 16) {
        n = fmin_nan(n, dpp_f<0x124>(n)); x = fmax_nan(x, dpp_f<0x124>(x));      // row_ror:4
        n = fmin_nan(n, dpp_f<0x128>(n)); x = fmax_nan(x, dpp_f<0x128>(x));      // row_ror:8
    }
    if constexpr (T >= 32) { n = fmin_nan(n, __shfl_xor(n, 16)); x = fmax_nan(x, __shfl_xor(x, 16)); }
    if constexpr (T >= 64) { n = fmin_nan(n, __shfl_xor(n, 32)); x = fmax_nan(x, __shfl_xor(x, 32)); }
    mn_my = n;
    mx_my = x;
}

template <int T> AMCT_DEV uint32_t team_umax(uint32_t v) {
    if constexpr (T >= 2) v = max(v, dpp_u<0xB1>(v));
    if constexpr (T >= 4) v = max(v, dpp_u<0x4E>(v));
    if constexpr (T >= 8) v = max(v, dpp_u<0x141>(v));
    if constexpr (T >= 16) v = max(v, dpp_u<0x140>(v));
    if constexpr (T >= 32) v = max(v, (uint32_t)__shfl_xor((int)v, 16));
    if constexpr (T >= 64) v = max(v, (uint32_t)__shfl_xor((int)v, 32));
    return v;
}

// Correctly rounded x / s from a precomputed y = RN(1/s) (Markstein): q0 = RN(x*y); two rounds of
// "exact remainder by fma, correct by remainder*y".  After the first round q1 is within half an ulp
// (plus 2^-45 relative) of x/s; the second round's error, <= 2^-25 ulp, is below the smallest
// distance a quotient of two fp32 numbers can have from a rounding boundary (2^-47 relative), so q2
// equals the IEEE quotient.  Valid while no intermediate over/underflows: the callers use it only
// for |s| in [2^-60, 2^60], finite x, and results that are zero or at least 2^-60 in magnitude
// matter only through round(q + z) (smaller quotients round to the same integer whatever their ulp).
struct Divisor {
    float s;      // divisor
    float y;      // RN(1/s)
    bool fast;    // the fma sequence may be used
};
AMCT_DEV Divisor make_divisor(float s) {
    Divisor d;
    d.s = s;
    d.y = 1.0f / s;
    const uint32_t e = (__float_as_uint(s) >> 23) & 0xFFu;
    d.fast = (e >= 67u) && (e <= 187u) && s > 0.f;
    return d;
}
template <bool KEEP_ZERO_SIGN = true>
AMCT_DEV float div_fast(float x, const Divisor& d) {
    const float q0 = x * d.y;
    const float r0 = __builtin_fmaf(-q0, d.s, x);
    const float q1 = __builtin_fmaf(r0, d.y, q0);
    const float r1 = __builtin_fmaf(-q1, d.s, x);
    const float q2 = __builtin_fmaf(r1, d.y, q1);
    // the divisor is positive, so the quotient carries the sign of x; the fma chain loses it only
    // when the quotient is a zero (-0.0 + 0.0 = +0.0): put it back where a caller can see it
    if constexpr (KEEP_ZERO_SIGN) return __uint_as_float(__float_as_uint(q2) | (__float_as_uint(x) & 0x80000000u));
    else return q2;
}

// x / c for a compile-time-known positive constant through the same sequence
AMCT_DEV float div_const(float x, float c, float rc) {
    Divisor d;
    d.s = c;
    d.y = rc;
    d.fast = true;
    return div_fast<true>(x, d);
}

// ---------------------------------------------------------------------------
// (max, min) -> (scale, offset): the closed form of
// amct_pytorch/quantize_op/utils.py:75-108 with the eps guard of :26-51,
// every operation a separately rounded fp32 op as in the eager reference.
// `off` is returned as an integral float (after round-half-even).
// ---------------------------------------------------------------------------
constexpr float kEps = 1.1920928955078125e-7f;   // fp32(1.192092896e-7), utils.py:23

struct Factors {
    float s;
    float z;
    float y;      // RN(1 / s) of the final scale: computed once here, reused for the element divisions
    bool bad;     // scale, 1/scale or offset not finite (utils.py:54-72)
};

AMCT_DEV bool finite_f(float f) { return (__float_as_uint(f) & 0x7F800000u) != 0x7F800000u; }

template <int DT>
AMCT_DEV Factors make_factors(float vmax, float vmin, int bits, bool symmetric, int scope_rule) {
    Factors r;
    if (symmetric) {
        const float amax = __builtin_fabsf(vmax), amin = __builtin_fabsf(vmin);
        const float qpos = (float)((1 << (bits - 1)) - 1);
        if (scope_rule == AMCT_SCOPE_ABSMAX) {
            // deploy.py:128-137 -- torch.abs(t).max() / qmax: NaN propagates, no guard, and the
            // quotient of a tensor by a Python number keeps the tensor's dtype
            r.s = round_to<DT>(fmax_nan(amax, amin) / qpos);
            r.z = 0.f;
            r.y = 1.0f / r.s;
            r.bad = !finite_f(r.s) || !finite_f(r.y);
            return r;
        }
        const float scope = (amax < amin) ? qpos + 1.0f : qpos;
        const float bound = (amax > amin) ? amax : amin;
        const float s_raw = bound / scope;
        r.s = (s_raw < kEps) ? 1.0f : s_raw;
        r.z = 0.f;
        r.y = 1.0f / r.s;
    } else {
        // torch.clamp propagates NaN; (x < 0 ? 0 : x) keeps NaN as well
        vmax = (vmax < 0.f) ? 0.f : vmax;
        vmin = (vmin > 0.f) ? 0.f : vmin;
        const float scope = (float)((1 << bits) - 1);
        const float half = (float)(1 << (bits - 1));        // ceil(scope / 2)
        const float diff = vmax - vmin;
        const uint32_t ed = (__float_as_uint(diff) >> 23) & 0xFFu;
        const bool exact_fma = ed >= 67u && ed <= 187u;     // diff in [2^-60, 2^61)
        // both quotients by the exact fma sequence where it is valid (same results as '/')
        const float s_raw = exact_fma ? div_const(diff, scope, bits == 8 ? (1.0f / 255.0f) : (1.0f / 15.0f)) : diff / scope;
        const bool tiny = s_raw < kEps;
        r.s = tiny ? 1.0f : s_raw;
        r.y = 1.0f / r.s;                                   // the one reciprocal per segment
        float q;
        if (exact_fma) {
            Divisor ds;
            ds.s = r.s;
            ds.y = r.y;
            ds.fast = true;
            q = div_fast<true>(vmin, ds);                   // a tiny scale overrides the offset below
        } else {
            q = vmin / r.s;
        }
        r.z = (vmax != vmin) ? (-half - q) : -half;
        r.z = tiny ? -half : r.z;
    }
    r.bad = !finite_f(r.s) || !finite_f(r.y) || !finite_f(r.z);
    // round-half-even, then through int32 as the reference does: a rounded -0.0 becomes +0.0
    r.z = (float)(int)__builtin_rintf(r.z);
    return r;
}

// the element divisor of a segment from its factors (no second reciprocal)
AMCT_DEV Divisor divisor_of(const Factors& f) {
    Divisor d;
    d.s = f.s;
    d.y = f.y;
    const uint32_t e = (__float_as_uint(f.s) >> 23) & 0xFFu;
    d.fast = (e >= 67u) && (e <= 187u) && f.s > 0.f;
    return d;
}

// One element of the integer (fake-)quantiser.
//   t = x / s (+ z); [narrow to the source dtype]; q = clamp(rne(t), qmin, qmax)
// Returns q (integral float); *deq = (q - z) * s when requested.
template <int DT, bool VIA_SRC, bool FAST = false, bool KEEP_ZERO_SIGN = true>
AMCT_DEV float quant_elem(float x, const Divisor& d, float z, bool asym, float qmin, float qmax) {
    float t;
    if constexpr (FAST) t = div_fast<KEEP_ZERO_SIGN>(x, d);
    else t = x / d.s;
    if (asym) t = t + z;
    if constexpr (VIA_SRC) t = round_to<DT>(t);
    t = __builtin_rintf(t);
    // v_med3_f32 clamps in one op; it differs from torch.clamp only for a NaN t, which can
    // only come from NaN data or factors (reported through the bad-factor count)
    t = __builtin_amdgcn_fmed3f(t, qmin, qmax);
    return t;
}
template <int DT, bool VIA_SRC>
AMCT_DEV float quant_elem(float x, float s, float z, bool asym, float qmin, float qmax) {
    Divisor d;
    d.s = s;
    d.y = 0.f;
    d.fast = false;
    return quant_elem<DT, VIA_SRC, false>(x, d, z, asym, qmin, qmax);
}
AMCT_DEV float dequant_elem(float q, float s, float z, bool asym) {
    if (asym) q = q - z;
    return q * s;
}

inline int hip_status() { return hipGetLastError() == hipSuccess ? AMCT_OK : AMCT_E_HIP; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace amct
