// K5: HiFloat8 encode / decode by bit manipulation (gfx950 has no instruction for it; the
// reference has no such code).  Layout, MSB first: S | dot | exponent (D bits, sign-magnitude
// with a hidden leading one) | mantissa:
//   dot 11 -> D=4, 1 mantissa bit (|E| 8..15)     dot 10 -> D=3, 2 bits (|E| 4..7)
//   dot 01 -> D=2, 3 bits (|E| 2..3)              dot 001 -> D=1, 3 bits (|E| = 1)
//   dot 0001 -> D=0, 3 bits (E = 0)               dot 0000 -> denormal 2^(M-23), M = 1..7
// 0x00 zero, 0x80 NaN, 0x6F / 0xEF = +-Inf (E=15, M=1); largest finite 2^15.
// Encode rounds to nearest, ties away from zero; |x| < 2^-23 -> 0; overflow -> Inf or +-2^15.
#include "amct_common.h"

namespace amct {

// u: the fp32 bit pattern.  Integer arithmetic only, so the compiler can also evaluate it (the table below).
__host__ __device__ constexpr uint32_t hif8_enc_bits(uint32_t u, bool saturate) {
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x80u;
    const int E = (int)(a >> 23) - 127;
    if (E < -23) return 0u;                                   // |x| < 2^-23 (fp32 denormals included)
    const int absE = E < 0 ? -E : E;
    // mantissa bits kept in this binade
    int mb = (absE <= 3) ? 3 : (absE <= 7) ? 2 : (absE <= 15) ? 1 : 0;
    if (E > 15) mb = 1;                                       // overflows below anyway
    // ties away from zero: add half an ulp, truncate
    uint32_t r = a + (1u << (22 - mb));
    r &= ~((1u << (23 - mb)) - 1u);
    const int E2 = (int)(r >> 23) - 127;
    if (E2 < -23) return 0u;
    if (E2 < -15) {                                           // denormal range: powers of two only
        const int e = E2 < -22 ? -22 : E2;                    // [2^-23, 2^-22) rounds up to the smallest
        return sign | (uint32_t)(e + 23);
    }
    const int a2 = E2 < 0 ? -E2 : E2;
    if (E2 > 15 || (E2 == 15 && (r & 0x400000u))) return sign | (saturate ? 0x6Eu : 0x6Fu);
    const uint32_t es = E2 < 0 ? 1u : 0u;
    if (a2 == 0) return sign | 0x08u | ((r >> 20) & 7u);
    if (a2 == 1) return sign | 0x10u | (es << 3) | ((r >> 20) & 7u);
    if (a2 <= 3) return sign | 0x20u | (es << 4) | ((uint32_t)(a2 & 1) << 3) | ((r >> 20) & 7u);
    if (a2 <= 7) return sign | 0x40u | (es << 4) | ((uint32_t)(a2 & 3) << 2) | ((r >> 21) & 3u);
    return sign | 0x60u | (es << 4) | ((uint32_t)(a2 & 7) << 1) | ((r >> 22) & 1u);
}
AMCT_DEV uint32_t hif8_enc(float x, bool saturate) { return hif8_enc_bits(__float_as_uint(x), saturate); }

// The code of a bf16 value depends on its sign, its exponent and the first four bits of its mantissa only (at most
// three are kept and ties go away from zero, so the first dropped bit decides the rounding) -- except for exponent 255,
// where the last three bits tell a NaN from an infinity.  Table of the 8192 values with the last three bits zero, for
// overflow to infinity [0] and to the largest finite value [1], computed by the compiler.
struct Hif8Bf16Table {
    uint8_t code[2][8192];
    constexpr Hif8Bf16Table() : code{} {
        for (int s = 0; s < 2; ++s)
            for (uint32_t i = 0; i < 8192u; ++i) code[s][i] = (uint8_t)hif8_enc_bits(i << 19, s != 0);
    }
};
__device__ const Hif8Bf16Table kHif8Bf16{};

AMCT_DEV float hif8_dec(uint32_t c) {
    const uint32_t b = c & 0x7Fu;
    float f;
    int e;
    uint32_t man;      // mantissa aligned to the top of the fp32 fraction
    if (b >= 0x60u) { e = 8 + ((b >> 1) & 7); if (b & 0x10u) e = -e; man = (b & 1u) << 22; }
    else if (b >= 0x40u) { e = 4 + ((b >> 2) & 3); if (b & 0x10u) e = -e; man = (b & 3u) << 21; }
    else if (b >= 0x20u) { e = 2 + ((b >> 3) & 1); if (b & 0x10u) e = -e; man = (b & 7u) << 20; }
    else if (b >= 0x10u) { e = (b & 0x08u) ? -1 : 1; man = (b & 7u) << 20; }
    else if (b >= 0x08u) { e = 0; man = (b & 7u) << 20; }
    else {
        if (b == 0u) return (c & 0x80u) ? __uint_as_float(0x7FC00000u) : 0.f;
        e = (int)b - 23;
        man = 0;
    }
    if (b == 0x6Fu) f = __builtin_huge_valf();
    else f = __uint_as_float(((uint32_t)(e + 127) << 23) | man);
    return (c & 0x80u) ? -f : f;
}

// Encode through two small tables in LDS, indexed by sign and biased exponent (9 bits), which the block
// builds once and then uses for many elements:
//   rnd[se]  half an ulp of the HiF8 precision of that binade (0 where the result is 0 or the input is
//            Inf/NaN): r = bits + rnd is the magnitude rounded to nearest, ties away, before truncation;
//   par[se]  for the binade of r: shift, width and base packed into one word (a 16-byte entry made the kernel
//            LDS-bound: 26 us against 20 us); the code is base | bitfield(r, shift, width).  base
//            carries the sign, the dot field and the exponent field; zero results have base 0 (no sign:
//            0x80 is NaN), denormal and overflow results width 0.  Exponent 15 has base 0x6E and width 1,
//            so that mantissa bit 1 yields 0x6F, the Inf code (width 0 when saturating).
// A carry out of the mantissa moves r into the next binade with its top mantissa bits zero, which is why no
// truncation mask is needed before the lookup.  NaN is patched afterwards (one compare, one select).
struct Hif8Tables {
    uint32_t rnd[512];
    uint32_t par[512];                               // shift in bits 0..4, width in bits 8..12, base in bits 16..23
};

AMCT_DEV void hif8_build_tables(Hif8Tables& t, int tid, int nthreads, bool saturate) {
    for (int i = tid; i < 512; i += nthreads) {
        const uint32_t sign = (uint32_t)(i >> 8) << 7;
        const int eb = i & 255, E = eb - 127;
        const int absE = E < 0 ? -E : E;
        const int mb = (absE <= 3) ? 3 : (absE <= 7) ? 2 : (absE <= 15 || E > 15) ? 1 : 0;
        t.rnd[i] = (E < -23 || eb == 255) ? 0u : (1u << (22 - mb));
        uint32_t shift = 0, width = 0, base = 0;
        if (E < -23) {
            base = 0;
        } else if (E < -15) {
            base = sign | (uint32_t)((E < -22 ? -22 : E) + 23);   // [2^-23, 2^-22) rounds up to the smallest
        } else if (E > 15) {
            base = sign | (saturate ? 0x6Eu : 0x6Fu);
        } else {
            const uint32_t es = E < 0 ? 1u : 0u;
            if (absE == 0) { base = 0x08u; shift = 20; width = 3; }
            else if (absE == 1) { base = 0x10u | (es << 3); shift = 20; width = 3; }
            else if (absE <= 3) { base = 0x20u | (es << 4) | ((uint32_t)(absE & 1) << 3); shift = 20; width = 3; }
            else if (absE <= 7) { base = 0x40u | (es << 4) | ((uint32_t)(absE & 3) << 2); shift = 21; width = 2; }
            else { base = 0x60u | (es << 4) | ((uint32_t)(absE & 7) << 1); shift = 22; width = 1; }
            if (E == 15 && saturate) width = 0;
            base |= sign;
        }
        t.par[i] = shift | (width << 8) | (base << 16);
    }
}

AMCT_DEV uint32_t hif8_enc_lut(const Hif8Tables& t, float x) {
    const uint32_t u = __float_as_uint(x);
    const uint32_t r = u + t.rnd[u >> 23];
    const uint32_t p = t.par[r >> 23];
    // v_bfe_u32 looks at bits 0..4 of its offset and width operands only, so the packed word serves as both
    const uint32_t code = (p >> 16) | __builtin_amdgcn_ubfe(r, p, p >> 8);
    return __builtin_isnan(x) ? 0x80u : code;
}

template <int DT, int U>
__global__ __launch_bounds__(kBlock) void hif8_encode_k(const void* x, uint8_t* y, int64_t nvec, int64_t n, int saturate) {
    constexpr int VEC = Tr<DT>::VEC;
    __shared__ Hif8Tables tbl;
    const int tid = threadIdx.x;
    hif8_build_tables(tbl, tid, kBlock, saturate != 0);
    __syncthreads();
    const int64_t chunk = (int64_t)kBlock * U;
    const int64_t nchunks = (nvec + chunk - 1) / chunk;
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        uint4 raw[U];
        int64_t gv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            gv[u] = c * chunk + u * kBlock + tid;
            raw[u] = ldg16_nt(reinterpret_cast<const char*>(x) + ((gv[u] < nvec ? gv[u] : nvec - 1) * 16));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float v[VEC];
            unpack16<DT>(raw[u], v);
            uint32_t w[VEC / 4];
#pragma unroll
            for (int j = 0; j < VEC / 4; ++j)
                w[j] = hif8_enc_lut(tbl, v[4 * j]) | (hif8_enc_lut(tbl, v[4 * j + 1]) << 8) |
                       (hif8_enc_lut(tbl, v[4 * j + 2]) << 16) | (hif8_enc_lut(tbl, v[4 * j + 3]) << 24);
            if (gv[u] < nvec) {
                uint32_t* p = reinterpret_cast<uint32_t*>(y + gv[u] * VEC);
                if constexpr (VEC == 8) stg8_nt(p, w[0], w[1]);
                else stg4_nt(p, w[0]);
            }
        }
    }
    // tail (n % VEC elements), handled by block 0
    if (blockIdx.x == 0) {
        const int64_t e = nvec * VEC + tid;
        if (e < n) y[e] = (uint8_t)hif8_enc(load_scalar<DT>(x, e), saturate);
    }
}

// complete chunks of U * 256 vectors only: one wave-uniform base per chunk, 32-bit lane offsets, nothing clamped or
// predicated (the remainder goes to hif8_encode_k)
template <int DT, int U>
__global__ __launch_bounds__(kBlock) void hif8_encode_full(const void* x, uint8_t* y, int64_t nchunks, int saturate) {
    constexpr int VEC = Tr<DT>::VEC;
    __shared__ Hif8Tables tbl;
    const uint32_t tid = threadIdx.x;
    hif8_build_tables(tbl, (int)tid, kBlock, saturate != 0);
    __syncthreads();
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        const char* xb = reinterpret_cast<const char*>(x) + c * (U * kBlock * 16);
        uint8_t* yb = y + c * (U * kBlock * VEC);
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) raw[u] = ldg16_nt(xb + (u * kBlock + tid) * 16u);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float v[VEC];
            unpack16<DT>(raw[u], v);
            uint32_t w[VEC / 4];
#pragma unroll
            for (int j = 0; j < VEC / 4; ++j)
                w[j] = hif8_enc_lut(tbl, v[4 * j]) | (hif8_enc_lut(tbl, v[4 * j + 1]) << 8) |
                       (hif8_enc_lut(tbl, v[4 * j + 2]) << 16) | (hif8_enc_lut(tbl, v[4 * j + 3]) << 24);
            uint32_t* p = reinterpret_cast<uint32_t*>(yb + (u * kBlock + tid) * (uint32_t)VEC);
            if constexpr (VEC == 8) stg8_nt(p, w[0], w[1]);
            else stg4_nt(p, w[0]);
        }
    }
}

// bf16 input, complete chunks of U * BLK vectors: one look-up per element in the block's copy of the 8 KB table
// above (index = the first 13 bits of the value), four codes merged by one byte permute.  A wave that holds an infinity
// or a NaN (a magnitude of 0x7F80 or more in any lane, found with packed 16-bit maxima) encodes its vectors by the
// arithmetic routine instead.  The next chunk's loads are issued before this one is encoded.
typedef unsigned short h2u16 __attribute__((ext_vector_type(2)));
AMCT_DEV uint32_t hif8_pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(h2u16, a), __builtin_bit_cast(h2u16, b)));
}
// the two codes of a word of two bf16 values, zero-extended to 16 bits each
AMCT_DEV uint32_t hif8_lut2(const uint8_t* tbl, uint32_t w) {
    h2u16 p;
    p.x = tbl[__builtin_amdgcn_ubfe(w, 3, 13)];
    p.y = tbl[w >> 19];
    return __builtin_bit_cast(uint32_t, p);
}

template <int BLK, int U>
__global__ __launch_bounds__(BLK) void hif8_encode_bf16_lut(const void* x, uint8_t* y, int64_t nchunks, int saturate) {
    __shared__ __align__(16) uint8_t tbl[8192];
    const uint32_t tid = threadIdx.x;
    {
        const uint4* src = reinterpret_cast<const uint4*>(kHif8Bf16.code[saturate ? 1 : 0]);
        for (uint32_t i = tid; i < 512u; i += BLK) reinterpret_cast<uint4*>(tbl)[i] = src[i];
    }
    uint4 nxt[U];
    if ((int64_t)blockIdx.x < nchunks) {
        const char* xb = reinterpret_cast<const char*>(x) + (int64_t)blockIdx.x * (U * BLK * 16);
#pragma unroll
        for (int u = 0; u < U; ++u) nxt[u] = ldg16_nt(xb + (u * BLK + tid) * 16u);
    }
    __syncthreads();
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        uint8_t* yb = y + c * (U * BLK * 8);
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) raw[u] = nxt[u];
        if (c + gridDim.x < nchunks) {
            const char* xb = reinterpret_cast<const char*>(x) + (c + gridDim.x) * (U * BLK * 16);
#pragma unroll
            for (int u = 0; u < U; ++u) nxt[u] = ldg16_nt(xb + (u * BLK + tid) * 16u);
        }
        uint32_t m = 0;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            m = hif8_pk_max_u16(m, hif8_pk_max_u16(hif8_pk_max_u16(raw[u].x & 0x7FFF7FFFu, raw[u].y & 0x7FFF7FFFu),
                                                   hif8_pk_max_u16(raw[u].z & 0x7FFF7FFFu, raw[u].w & 0x7FFF7FFFu)));
        }
        const bool special = (m & 0xFFFFu) >= 0x7F80u || m >= 0x7F800000u;
        if (__builtin_amdgcn_ballot_w64(special) == 0) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t w0 = __builtin_amdgcn_perm(hif8_lut2(tbl, raw[u].y), hif8_lut2(tbl, raw[u].x), 0x06040200u);
                const uint32_t w1 = __builtin_amdgcn_perm(hif8_lut2(tbl, raw[u].w), hif8_lut2(tbl, raw[u].z), 0x06040200u);
                stg8_nt(yb + (u * BLK + tid) * 8u, w0, w1);
            }
        } else {
#pragma unroll                                       // (a rolled loop would index raw[] at run time: 64 KB of LDS)
            for (int u = 0; u < U; ++u) {
                float v[8];
                unpack16<AMCT_BF16>(raw[u], v);
                uint32_t w[2];
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    w[j] = hif8_enc(v[4 * j], saturate != 0) | (hif8_enc(v[4 * j + 1], saturate != 0) << 8) |
                           (hif8_enc(v[4 * j + 2], saturate != 0) << 16) | (hif8_enc(v[4 * j + 3], saturate != 0) << 24);
                stg8_nt(yb + (u * BLK + tid) * 8u, w[0], w[1]);
            }
        }
    }
}

// complete chunks of U * BLK vectors; the next chunk's codes are loaded before this one's are looked up
template <int DT, int BLK, int U>
__global__ __launch_bounds__(BLK) void hif8_decode_full(const uint8_t* x, void* y, int64_t nchunks) {
    constexpr int VEC = Tr<DT>::VEC;
    __shared__ float tbl[256];
    const uint32_t tid = threadIdx.x;
    if (tid < 256u) tbl[tid] = hif8_dec(tid);
    __syncthreads();
    auto load = [&](int64_t c, uint32_t (&w)[U][2]) {
        const uint8_t* xb = x + c * (U * BLK * VEC);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            w[u][1] = 0;
            if constexpr (VEC == 8) {
                const u2v r = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(xb + (u * BLK + tid) * 8u));
                w[u][0] = r.x; w[u][1] = r.y;
            } else {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(xb + (u * BLK + tid) * 4u));
            }
        }
    };
    uint32_t nxt[U][2];
    if ((int64_t)blockIdx.x < nchunks) load(blockIdx.x, nxt);
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        char* yb = reinterpret_cast<char*>(y) + c * (U * BLK * 16);
        uint32_t w[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u) { w[u][0] = nxt[u][0]; w[u][1] = nxt[u][1]; }
        if (c + gridDim.x < nchunks) load(c + gridDim.x, nxt);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float out[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) out[j] = tbl[(w[u][j / 4] >> (8 * (j % 4))) & 0xFFu];
            stg16_nt(yb + (u * BLK + tid) * 16u, pack16<DT>(out));
        }
    }
}

// decode through a 256-entry table in LDS built by the block itself; U vectors per lane in flight
template <int DT, int U>
__global__ __launch_bounds__(kBlock) void hif8_decode_k(const uint8_t* x, void* y, int64_t nvec, int64_t n) {
    constexpr int VEC = Tr<DT>::VEC;
    __shared__ float tbl[256];
    const int tid = threadIdx.x;
    tbl[tid] = hif8_dec((uint32_t)tid);
    __syncthreads();
    const int64_t chunk = (int64_t)kBlock * U;
    const int64_t nchunks = (nvec + chunk - 1) / chunk;
    for (int64_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
        uint32_t w[U][2];
        int64_t gv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            gv[u] = c * chunk + u * kBlock + tid;
            const int64_t g = gv[u] < nvec ? gv[u] : nvec - 1;      // clamped: loads are unconditional
            w[u][1] = 0;
            if constexpr (VEC == 8) {
                const u2v r = __builtin_nontemporal_load(reinterpret_cast<const u2v*>(x + g * 8));
                w[u][0] = r.x; w[u][1] = r.y;
            } else {
                w[u][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(x + g * 4));
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float out[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) out[j] = tbl[(w[u][j / 4] >> (8 * (j % 4))) & 0xFFu];
            if (gv[u] < nvec) stg16_nt(reinterpret_cast<char*>(y) + gv[u] * 16, pack16<DT>(out));
        }
    }
    if (blockIdx.x == 0) {
        const int64_t e = nvec * VEC + tid;
        if (e < n) store_scalar<DT>(y, e, tbl[x[e]]);
    }
}

// Launch shapes, measured on X[8192,4096] bf16: encoder 1024 threads x 1 vector, two blocks per CU, 17.3 us (512 x 4:
// 17.6; the two-table kernel 18.5); decoder 256 threads x 8 vectors, four blocks per CU, 17.3 us (256 x 4 with one
// chunk per block and no look-ahead 18.9; 1024 x 4: 19.5).
constexpr int kHif8LutBlock = 1024, kHif8LutU = 1, kHif8LutBlocksPerCu = 2;
constexpr int kHif8DecBlock = 256, kHif8DecU = 8, kHif8DecBlocksPerCu = 4;

}  // namespace amct

using namespace amct;

extern "C" int amct_hif8_encode(const void* x, uint8_t* y, int64_t n, int dtype, int saturate, amct_stream_t stream) {
    if (n < 0 || (n != 0 && (!x || !y))) return AMCT_E_BADARG;   // n == 0 reads nothing: null pointers are fine
    if (!aligned16(x) || (reinterpret_cast<uintptr_t>(y) & 7u) != 0) return AMCT_E_ALIGN;
    if (n == 0) return AMCT_OK;
    constexpr int U = 4;
    hipStream_t st = (hipStream_t)stream;
#define AMCT_HE(DT)                                                                                              \
    {                                                                                                            \
        constexpr int64_t per = (int64_t)kBlock * U * Tr<DT>::VEC;      /* elements of a complete chunk */       \
        const int64_t full = n / per;                                                                            \
        if (full > 0) {                                                                                          \
            /* blocks loop over chunks: the table build is paid 8 times per CU at most */                        \
            hipLaunchKernelGGL((hif8_encode_full<DT, U>), dim3((unsigned)(full > 2048 ? 2048 : full)), dim3(kBlock), 0, st, x, y, full, saturate); \
            x = reinterpret_cast<const char*>(x) + full * per * Tr<DT>::BYTES;                                   \
            y += full * per;                                                                                     \
            n -= full * per;                                                                                     \
        }                                                                                                        \
        if (n > 0) {                                                                                             \
            const int64_t nvec = n / Tr<DT>::VEC;                                                                \
            hipLaunchKernelGGL((hif8_encode_k<DT, U>), dim3(1), dim3(kBlock), 0, st, x, y, nvec, n, saturate);   \
        }                                                                                                        \
    }
    if (dtype == AMCT_BF16) {
        constexpr int BLK = kHif8LutBlock, UL = kHif8LutU;
        constexpr int64_t per = (int64_t)BLK * UL * 8;
        const int64_t full = n / per;
        if (full > 0) {
            const int64_t cap = (int64_t)kHif8LutBlocksPerCu * 256;
            hipLaunchKernelGGL((hif8_encode_bf16_lut<BLK, UL>), dim3((unsigned)(full > cap ? cap : full)), dim3(BLK), 0, st, x, y, full, saturate);
            x = reinterpret_cast<const char*>(x) + full * per * 2;
            y += full * per;
            n -= full * per;
        }
        if (n == 0) return hip_status();
    }
    switch (dtype) {
        case AMCT_F32: AMCT_HE(AMCT_F32) break;
        case AMCT_F16: AMCT_HE(AMCT_F16) break;
        case AMCT_BF16: AMCT_HE(AMCT_BF16) break;
        default: return AMCT_E_BADARG;
    }
#undef AMCT_HE
    return hip_status();
}

extern "C" int amct_hif8_decode(const uint8_t* x, void* y, int64_t n, int dtype, amct_stream_t stream) {
    if (n < 0 || (n != 0 && (!x || !y))) return AMCT_E_BADARG;   // n == 0 reads nothing: null pointers are fine
    if (!aligned16(y) || (reinterpret_cast<uintptr_t>(x) & 7u) != 0) return AMCT_E_ALIGN;
    if (n == 0) return AMCT_OK;
    hipStream_t st = (hipStream_t)stream;
#define AMCT_HD(DT)                                                                                   \
    {                                                                                                 \
        constexpr int64_t per = (int64_t)kHif8DecBlock * kHif8DecU * Tr<DT>::VEC;                     \
        const int64_t full = n / per, cap = (int64_t)kHif8DecBlocksPerCu * 256;                       \
        if (full > 0) {                                                                               \
            hipLaunchKernelGGL((hif8_decode_full<DT, kHif8DecBlock, kHif8DecU>), dim3((unsigned)(full > cap ? cap : full)), dim3(kHif8DecBlock), 0, st, x, y, full); \
            x += full * per;                                                                          \
            y = reinterpret_cast<char*>(y) + full * per * Tr<DT>::BYTES;                              \
            n -= full * per;                                                                          \
        }                                                                                             \
        if (n > 0) {                                                                                  \
            const int64_t nvec = n / Tr<DT>::VEC;                                                     \
            hipLaunchKernelGGL((hif8_decode_k<DT, 4>), dim3(1), dim3(kBlock), 0, st, x, y, nvec, n);  \
        }                                                                                             \
    }
    switch (dtype) {
        case AMCT_F32: AMCT_HD(AMCT_F32) break;
        case AMCT_F16: AMCT_HD(AMCT_F16) break;
        case AMCT_BF16: AMCT_HD(AMCT_BF16) break;
        default: return AMCT_E_BADARG;
    }
#undef AMCT_HD
    return hip_status();
}
