// GPTQ Hessian accumulation on the matrix pipe: H <- beta * H + alpha * X^T X, the update of
// amct_pytorch/quantize_op/gptq_module.py:176-181 (hessian *= n / (n + b); x = sqrt(2 / n) * x.float();
// hessian += x @ x.t()) for 16-bit calibration activations X [tokens, columns].
//
// The products of two bf16 (or fp16) values are exact in fp32 and the MFMA accumulates in fp32, so the matrix
// product of the 16-bit inputs is the reference's fp32 product up to the order of the sum; the factor 2 / n is
// applied once to the sum instead of sqrt(2 / n) to every element.
//
// Two kernels.  hess_transpose_k writes X^T, zero-padded to whole tiles, into the caller's workspace ([Cp, Tp], K
// contiguous), so that both MFMA operands are rows of one matrix.  hess_syrk_k owns one 128 x 128 tile of the lower
// triangle: 4 waves of 64 x 64 (2 x 2 MFMA 32x32x16), 64 tokens per step, one LDS stage (16-byte chunks of a row
// swizzled by the row so that fragment reads spread over the banks; the next step waits in registers), two barriers
// per step.  The epilogue reads the
// tile of H, applies beta and alpha, writes the tile and -- through LDS, as whole 256-byte rows -- its mirror image, so H
// stays exactly symmetric and only its lower triangle is ever read.
#include "amct_common.h"

namespace amct {

typedef float h16f __attribute__((ext_vector_type(16)));
typedef __bf16 h8bf __attribute__((ext_vector_type(8)));
typedef _Float16 h8h __attribute__((ext_vector_type(8)));

constexpr int kHsTile = 128;                         // rows / columns of H per block
constexpr int kHsK = 64;                             // tokens per step (128 bytes of a row of X^T)

// X [T, C] -> Xt [Cp, Tp], zeros beyond T and C.  64 x 64 tiles through LDS.
__global__ __launch_bounds__(kBlock) void hess_transpose_k(const uint16_t* x, uint16_t* xt, int64_t T, int64_t C, int64_t Tp) {
    __shared__ uint16_t tile[64][66];
    const int tid = threadIdx.x;
    const int64_t c0 = (int64_t)blockIdx.x * 64, t0 = (int64_t)blockIdx.y * 64;
    {
        const int c = tid & 63;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int t = (tid >> 6) + 4 * i;
            uint16_t v = 0;
            if (t0 + t < T && c0 + c < C) v = x[(t0 + t) * C + c0 + c];
            tile[t][c] = v;
        }
    }
    __syncthreads();
    {
        const int t = tid & 63;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = (tid >> 6) + 4 * i;
            xt[(c0 + c) * Tp + t0 + t] = tile[t][c];      // c0 + c < Cp and t0 + t < Tp by the grid
        }
    }
}

// The same for C % 8 == 0 and a 16-byte aligned x: 16-byte loads (8 columns of one token) and 16-byte stores (8
// tokens of one column); the tile is held column-major, a column 72 tokens apart (144 bytes: 16-byte aligned rows whose
// 16-byte reads by 8 lanes of consecutive columns fall into different banks).
__global__ __launch_bounds__(kBlock) void hess_transpose_vec_k(const uint16_t* x, uint16_t* xt, int64_t T, int64_t C, int64_t Tp) {
    __shared__ __align__(16) uint16_t tile[64][72];                           // [column][token]
    const int tid = threadIdx.x;
    const int64_t c0 = (int64_t)blockIdx.x * 64, t0 = (int64_t)blockIdx.y * 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int v = tid + 256 * i;                                          // 512 vectors: token v / 8, columns 8 (v % 8) ..
        const int t = v >> 3, cv = (v & 7) * 8;
        uint4 q = make_uint4(0, 0, 0, 0);
        if (t0 + t < T && c0 + cv < C) q = ldg16_nt(x + (t0 + t) * C + c0 + cv);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            tile[cv + 2 * j][t] = (uint16_t)(w[j] & 0xFFFFu);
            tile[cv + 2 * j + 1][t] = (uint16_t)(w[j] >> 16);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int v = tid + 256 * i;                                          // column v / 8, tokens 8 (v % 8) ..
        const int c = v >> 3, tv = (v & 7) * 8;
        const uint4 q = *reinterpret_cast<const uint4*>(&tile[c][tv]);
        stg16(xt + (c0 + c) * Tp + t0 + tv, q);                               // inside [Cp, Tp] by the grid
    }
}

struct SyrkArgs {
    const uint16_t* xt;                              // [Cp, Tp]
    float* h;                                        // [C, C]
    int64_t C, Tp;
    int nb;                                          // tiles per side
    int per_die;                                     // tiles of the lower triangle per die (rounded up)
    int64_t ntiles;                                  // nb (nb + 1) / 2
    float beta, alpha;
};

template <bool F16>
AMCT_DEV h16f hs_mfma(const uint4& a, const uint4& b, const h16f& c) {
    if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8h, a), __builtin_bit_cast(h8h, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(h8bf, a), __builtin_bit_cast(h8bf, b), c, 0, 0, 0);
}

template <bool F16>
__global__ __launch_bounds__(kBlock, 3) void hess_syrk_k(SyrkArgs a) {
    // one stage: two operands x 128 rows x 128 bytes = 32 KB (the next step waits in registers); the epilogue reuses it as
    // four 64 x 32 fp32 patches.  Three blocks fit a CU.
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // block -> tile (bi, bj) of the lower triangle, bi >= bj.  The chip hands consecutive blocks to its eight dies in
    // turn, and each die has an L2 of its own: block id works on tile (id % 8) * per + id / 8 of an order in which
    // consecutive tiles form compact patches (bands of 8 rows of tiles, inside a band column after column), so the 64
    // blocks that a die runs at a time share 8 + 8 operand tiles instead of fetching 64 + 64.
    const int per = a.per_die;
    const int64_t logical = (int64_t)(blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per || logical >= a.ntiles) return;         // whole block (before any barrier)
    int bi, bj;
    {
        // band b holds the rows 8 b .. min(8 b + 7, nb - 1); rows before it hold 8 b (8 b + 1) / 2 tiles
        int b = (int)((__builtin_sqrtf(8.0f * (float)logical + 1.0f) - 1.0f) * 0.5f) >> 3;
        while ((int64_t)(8 * (b + 1)) * (8 * (b + 1) + 1) / 2 <= logical) ++b;
        while ((int64_t)(8 * b) * (8 * b + 1) / 2 > logical) --b;
        const int r0 = 8 * b, r1 = min(8 * b + 7, a.nb - 1), H = r1 - r0 + 1;
        int o = (int)(logical - (int64_t)r0 * (r0 + 1) / 2);
        if (o < (r0 + 1) * H) {                      // the columns that every row of the band has
            bj = o / H;
            bi = r0 + o % H;
        } else {                                     // the triangle at the band's end: column r0 + 1 + c has H - 1 - c rows
            o -= (r0 + 1) * H;
            int c = 0;
            while (o >= H - 1 - c) { o -= H - 1 - c; ++c; }
            bj = r0 + 1 + c;
            bi = bj + o;
        }
    }
    const bool diag = bi == bj;
    const int64_t i0 = (int64_t)bi * kHsTile, j0 = (int64_t)bj * kHsTile;
    const int wi = wave >> 1, wj = wave & 1;         // 2 x 2 waves of 64 x 64

    // global -> LDS: a tile is 128 rows x 8 chunks of 16 bytes; thread t moves chunks t, t + 256, t + 512, t + 768
    const int ld_row = tid >> 3, ld_chunk = tid & 7; // + 32 rows per repeat
    const uint8_t* ga = reinterpret_cast<const uint8_t*>(a.xt) + ((i0 + ld_row) * a.Tp) * 2 + ld_chunk * 16;
    const uint8_t* gb = reinterpret_cast<const uint8_t*>(a.xt) + ((j0 + ld_row) * a.Tp) * 2 + ld_chunk * 16;
    const int64_t row_step = 32 * a.Tp * 2;          // bytes between the repeats
    // chunk c of row r sits at c ^ ((r >> 1) & 7): LDS has 64 banks of 4 bytes, two 128-byte rows cover them once, so 16
    // lanes reading the same logical chunk of 16 consecutive rows meet in no bank
    const uint32_t st_off = (uint32_t)ld_row * 128u + (uint32_t)((ld_chunk ^ ((ld_row >> 1) & 7)) * 16);   // rows 32 apart: same swizzle
    constexpr uint32_t kTileBytes = kHsTile * 128;

    // fragments: lane l holds row l % 32 of a 32-row tile, chunk 2 * slice + l / 32 of the step's 128 bytes
    const int fr = lane & 31, fh = lane >> 5;
    uint32_t fa_off[2], fb_off[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const uint32_t ra = (uint32_t)(wi * 64 + m * 32 + fr), rb = (uint32_t)(wj * 64 + m * 32 + fr);
        fa_off[m] = ra * 128u;
        fb_off[m] = rb * 128u + kTileBytes;
    }
    const uint32_t fsw = (uint32_t)((fr >> 1) & 7);  // rows of a fragment are 64 w + 32 m + fr: the swizzle depends on fr only

    h16f acc[2][2];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

    // (a tile on the diagonal loads its rows twice, as both operands: one block in nb + 1, and no special cases below)
    const int steps = (int)(a.Tp / kHsK);
    uint4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
#define AMCT_HS_GLOAD(S)                                                                  \
    {                                                                                     \
        const int64_t so = (int64_t)(S) * 128;                                            \
        ra0 = *reinterpret_cast<const uint4*>(ga + so);                                   \
        ra1 = *reinterpret_cast<const uint4*>(ga + row_step + so);                        \
        ra2 = *reinterpret_cast<const uint4*>(ga + 2 * row_step + so);                    \
        ra3 = *reinterpret_cast<const uint4*>(ga + 3 * row_step + so);                    \
        rb0 = *reinterpret_cast<const uint4*>(gb + so);                                   \
        rb1 = *reinterpret_cast<const uint4*>(gb + row_step + so);                        \
        rb2 = *reinterpret_cast<const uint4*>(gb + 2 * row_step + so);                    \
        rb3 = *reinterpret_cast<const uint4*>(gb + 3 * row_step + so);                    \
    }
#define AMCT_HS_LSTORE()                                                                  \
    {                                                                                     \
        uint8_t* base = lds + st_off;                                                     \
        *reinterpret_cast<uint4*>(base) = ra0;                                            \
        *reinterpret_cast<uint4*>(base + 32 * 128) = ra1;                                 \
        *reinterpret_cast<uint4*>(base + 64 * 128) = ra2;                                 \
        *reinterpret_cast<uint4*>(base + 96 * 128) = ra3;                                 \
        *reinterpret_cast<uint4*>(base + kTileBytes) = rb0;                               \
        *reinterpret_cast<uint4*>(base + kTileBytes + 32 * 128) = rb1;                    \
        *reinterpret_cast<uint4*>(base + kTileBytes + 64 * 128) = rb2;                    \
        *reinterpret_cast<uint4*>(base + kTileBytes + 96 * 128) = rb3;                    \
    }
    AMCT_HS_GLOAD(0)
    AMCT_HS_LSTORE()
    __syncthreads();
    for (int s = 0; s < steps; ++s) {
        if (s + 1 < steps) AMCT_HS_GLOAD(s + 1)      // in flight during this step's MFMAs
        const uint8_t* st = lds;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const uint32_t ch = ((uint32_t)(2 * ks + fh) ^ fsw) * 16u;
            uint4 fa[2], fb[2];
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                fa[m] = *reinterpret_cast<const uint4*>(st + fa_off[m] + ch);
                fb[m] = *reinterpret_cast<const uint4*>(st + fb_off[m] + ch);
            }
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int n = 0; n < 2; ++n) acc[m][n] = hs_mfma<F16>(fa[m], fb[n], acc[m][n]);
        }
        __syncthreads();                             // everyone has read this step's tiles
        if (s + 1 < steps) {
            AMCT_HS_LSTORE()
            __syncthreads();
        }
    }
#undef AMCT_HS_GLOAD
#undef AMCT_HS_LSTORE

    // ---- epilogue -------------------------------------------------------------------------------------------
    // acc[m][n][r]: row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32 of the 32 x 32 tile (m, n) of this wave
    // Addresses: one block-uniform base per wave plus 32-bit lane offsets (cols < 2^22 is checked by the host), so an
    // address costs one register and the compiler keeps none of them alive in 64 bits.
    const bool have = a.beta != 0.f;
    float* patch = reinterpret_cast<float*>(lds) + wave * (64 * 32);          // 8 KB per wave (after the last barrier)
    const uint32_t C32 = (uint32_t)a.C;
    const int64_t wi0 = i0 + wi * 64, wj0 = j0 + wj * 64;                     // the wave's first row and column
    float* hw = a.h + wi0 * a.C + wj0;                                        // H[wi0][wj0]
    float* hm = a.h + wj0 * a.C + wi0;                                        // its mirror image H[wj0][wi0]
    const int rows_left = (int)min((int64_t)64, a.C - wi0), cols_left = (int)min((int64_t)64, a.C - wj0);   // may be <= 0
    const uint32_t lane_off = (uint32_t)(4 * fh) * C32 + (uint32_t)fr;
#pragma unroll
    for (int n = 0; n < 2; ++n) {                    // the wave's columns 32 n .. 32 n + 31
        const bool col_ok = n * 32 + fr < cols_left;
        // all of the half's old values first (32 independent loads in flight; one at a time, each behind the store
        // before it, they cost a trip to memory each), then the arithmetic and the stores
        h16f old[2];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m * 32 + 8 * (r / 4) + (r % 4);               // + 4 fh
                const uint32_t idx = lane_off + (uint32_t)row * C32 + (uint32_t)(n * 32);
                old[m][r] = (have && col_ok && row + 4 * fh < rows_left) ? __builtin_nontemporal_load(hw + idx) : 0.f;
            }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m * 32 + 8 * (r / 4) + (r % 4);
                const int lr = row + 4 * fh;                                  // row inside the wave's 64 x 64
                const uint32_t idx = lane_off + (uint32_t)row * C32 + (uint32_t)(n * 32);
                float v = a.alpha * acc[m][n][r];
                if (have) v = old[m][r] * a.beta + v;
                if (col_ok && lr < rows_left) hw[idx] = v;
                patch[lr * 32 + (fr ^ (lr & 31))] = v;
            }
        }
        if (diag) continue;                          // the tile on the diagonal is its own mirror image
        // mirror image: H[gj][gi] = H[gi][gj]; lane = row lr of the patch, one column per instruction, so the wave
        // writes 64 consecutive floats of a row of H.  (The patch is the wave's own: no barrier.)
        const int lr = lane;
#pragma unroll 8
        for (int lc = 0; lc < 32; ++lc) {
            const float v = patch[lr * 32 + (lc ^ (lr & 31))];
            if (lr < rows_left && n * 32 + lc < cols_left) hm[(uint32_t)(n * 32 + lc) * C32 + (uint32_t)lr] = v;
        }
    }
}

}  // namespace amct

using namespace amct;

static int64_t hs_round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

extern "C" size_t amct_hessian_update_workspace_bytes(int64_t tokens, int64_t cols) {
    if (tokens <= 0 || cols <= 0) return 0;
    return (size_t)hs_round_up(cols, kHsTile) * (size_t)hs_round_up(tokens, kHsK) * 2;
}

extern "C" int amct_hessian_update(float* hessian, const void* x, int64_t tokens, int64_t cols, float beta, float alpha,
                                   int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream) {
    if (tokens < 0 || cols <= 0 || !hessian) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    if (tokens != 0 && !x) return AMCT_E_BADARG;
    const int64_t Cp = hs_round_up(cols, kHsTile), Tp = hs_round_up(tokens > 0 ? tokens : 1, kHsK);
    const int64_t nb = Cp / kHsTile;
    if (cols >= (int64_t(1) << 22)) return AMCT_E_TOO_LARGE;                  // 32-bit offsets inside a tile, block ids
    if (!workspace || workspace_bytes < (size_t)Cp * (size_t)Tp * 2) return AMCT_E_BADARG;
    if (!aligned16(workspace) || (reinterpret_cast<uintptr_t>(hessian) & 3u) != 0 || (reinterpret_cast<uintptr_t>(x) & 1u) != 0)
        return AMCT_E_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (cols % 8 == 0 && aligned16(x))
        hipLaunchKernelGGL(hess_transpose_vec_k, dim3((unsigned)(Cp / 64), (unsigned)(Tp / 64)), dim3(kBlock), 0, st,
                           reinterpret_cast<const uint16_t*>(x), reinterpret_cast<uint16_t*>(workspace), tokens, cols, Tp);
    else
        hipLaunchKernelGGL(hess_transpose_k, dim3((unsigned)(Cp / 64), (unsigned)(Tp / 64)), dim3(kBlock), 0, st,
                           reinterpret_cast<const uint16_t*>(x), reinterpret_cast<uint16_t*>(workspace), tokens, cols, Tp);
    const int64_t ntiles = nb * (nb + 1) / 2, per_die = (ntiles + 7) / 8;
    SyrkArgs a{reinterpret_cast<const uint16_t*>(workspace), hessian, cols, Tp, (int)nb, (int)per_die, ntiles, beta, alpha};
    constexpr size_t lds_bytes = 2 * kHsTile * 128;                           // 32 KB
    const dim3 grid((unsigned)(8 * per_die));
    if (dtype == AMCT_F16) hipLaunchKernelGGL((hess_syrk_k<true>), grid, dim3(kBlock), lds_bytes, st, a);
    else hipLaunchKernelGGL((hess_syrk_k<false>), grid, dim3(kBlock), lds_bytes, st, a);
    return hip_status();
}
