// What the weight-streaming int4 kernels for a few rows share: the activation-type traits (pack, unpack, the bit
// pattern of the integer 16 + u, the MFMA) and the operand order of 8 activations that matches them.
#pragma once
#include "amct_common.h"

namespace amct {

typedef float s4f __attribute__((ext_vector_type(4)));
typedef __bf16 s8bf __attribute__((ext_vector_type(8)));
typedef __bf16 s2bf __attribute__((ext_vector_type(2)));
typedef float s2f __attribute__((ext_vector_type(2)));

typedef _Float16 s8h __attribute__((ext_vector_type(8)));

struct StreamArgs {
    const uint16_t* x;
    const uint16_t* smooth;
    const uint8_t* wq;
    const uint16_t* scales;
    const uint8_t* zeros;
    const float* bias;
    const float* bias_src;                           // bias, or any readable N floats when there is none
    uint16_t* out;
    int M, N, K, G;                                  // K: elements of a row one block walks (a slice); G = K / group
    int group;
    int scale_f16;
    uint32_t kv_magic;                               // floor(2^32 / (K / 8)) + 1: v / (K / 8) == mulhi(v, magic)
    // Rows longer than a slice: blockIdx.y picks the slice; rows keep their full length as stride; every slice leaves
    // fp32 partial sums part[slice][M][N] that a second kernel adds in slice order (plus bias, rounding to the output type)
    int row_k;                                       // elements of a full row of x and of the weight
    float* part;                                     // null: one slice, the result goes to `out`
};


// (x & m) | b in one instruction.  The compiler splits the expression into v_and + v_or when m and b are literals (a
// three-operand instruction takes no 32-bit literal here), so the callers keep both constants in registers.
AMCT_DEV uint32_t and_or(uint32_t x, uint32_t m, uint32_t b) { return (x & m) | b; }

// what differs between the two activation types: the pack, the unpack, the bit pattern of the integer 16 + u, the MFMA
template <int DT> struct StAct;
template <> struct StAct<AMCT_BF16> {
    static AMCT_DEV uint32_t pack2(float lo, float hi) {
        const s2f f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, s2bf));      // v_cvt_pk_bf16_f32, round-half-even
    }
    static AMCT_DEV float lo(uint32_t w) { return __uint_as_float(w << 16); }
    static AMCT_DEV float hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
    // 8 nibbles of w (nibble p = weight k0 + p) -> 4 words of two integers 16 + u each, word j = (weight j, weight j + 4)
    static AMCT_DEV uint4 int8x(uint32_t w) {
        constexpr uint32_t kMask = 0x00780078u, kBase = 0x41804180u;   // bf16(16 + u) = 0x4180 | u << 3
        return make_uint4(((w << 3) & kMask) | kBase, ((w >> 1) & kMask) | kBase, ((w >> 5) & kMask) | kBase,
                          ((w >> 9) & kMask) | kBase);
    }
    // the same in two instructions per word, with the mask and the base (kMask, kBase) held in registers by the caller
    static constexpr uint32_t kMask = 0x00780078u, kBase = 0x41804180u;
    static AMCT_DEV uint4 int8x(uint32_t w, uint32_t m, uint32_t b) {
        return make_uint4(and_or(w << 3, m, b), and_or(w >> 1, m, b), and_or(w >> 5, m, b), and_or(w >> 9, m, b));
    }
    static AMCT_DEV s4f mfma(const uint4& a, const uint4& b, s4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(s8bf, a), __builtin_bit_cast(s8bf, b), c, 0, 0, 0);
    }
    // two copies of -(16 + z), z in 0 .. 15: the operand that takes the zero-point out of a sum of x * (16 + u)
    static AMCT_DEV uint32_t neg16z(uint32_t z) { return (z * 0x00080008u) | 0xC180C180u; }
    static AMCT_DEV uint32_t out_bits(float v) { return f32_to_bf16_bits(v); }
};
template <> struct StAct<AMCT_F16> {
    static AMCT_DEV uint32_t pack2(float lo, float hi) { return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16); }
    static AMCT_DEV float lo(uint32_t w) { return f16_bits_to_f32(w & 0xFFFFu); }
    static AMCT_DEV float hi(uint32_t w) { return f16_bits_to_f32(w >> 16); }
    static AMCT_DEV uint4 int8x(uint32_t w) {
        constexpr uint32_t kMask = 0x03C003C0u, kBase = 0x4C004C00u;   // f16(16 + u) = 0x4C00 | u << 6
        return make_uint4(((w << 6) & kMask) | kBase, ((w << 2) & kMask) | kBase, ((w >> 2) & kMask) | kBase,
                          ((w >> 6) & kMask) | kBase);
    }
    static constexpr uint32_t kMask = 0x03C003C0u, kBase = 0x4C004C00u;
    static AMCT_DEV uint4 int8x(uint32_t w, uint32_t m, uint32_t b) {
        return make_uint4(and_or(w << 6, m, b), and_or(w << 2, m, b), and_or(w >> 2, m, b), and_or(w >> 6, m, b));
    }
    static AMCT_DEV s4f mfma(const uint4& a, const uint4& b, s4f c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(s8h, a), __builtin_bit_cast(s8h, b), c, 0, 0, 0);
    }
    static AMCT_DEV uint32_t neg16z(uint32_t z) { return (z * 0x00400040u) | 0xCC00CC00u; }
    static AMCT_DEV uint32_t out_bits(float v) { return f32_to_f16_bits(v); }
};
// the matching order of 8 activations: (k0, k4), (k1, k5), (k2, k6), (k3, k7)
AMCT_DEV uint4 st_interleave8(const uint4& x) {
    return make_uint4(__builtin_amdgcn_perm(x.z, x.x, 0x05040100u), __builtin_amdgcn_perm(x.z, x.x, 0x07060302u),
                      __builtin_amdgcn_perm(x.w, x.y, 0x05040100u), __builtin_amdgcn_perm(x.w, x.y, 0x07060302u));
}

}  // namespace amct
