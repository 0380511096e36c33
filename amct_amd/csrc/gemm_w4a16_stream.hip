// K7 for M <= 16 (decode): the packed weights are the only large traffic, 29 MB for W[14336,4096], which the
// memory system delivers in a few microseconds only if all of it is requested at once.  So every wave of the launch
// is resident at the same time and issues ALL its weight loads (16 bytes per lane and 128 elements of K) before
// anything else waits; what it needs besides (activations, smoothing factors, scales, zero-points) is staged once
// per block through LDS with coalesced loads that were issued just before (waits are in issue order, so the staged
// data can be consumed while the weights are still arriving) and the dequantisation then follows the data as it
// lands.  A block owns CG groups of 16 output columns; KS waves per column group split K; a lane holds the 32
// consecutive weights k0 + 32 g .. of column n0 + lane % 16 per step (g = lane / 16), i.e. one MFMA 16x16x32 operand
// per 8 weights, and reads the matching activations of row lane % 16 from LDS.
// Arithmetic: x' = bf16(x * smooth) as everywhere.  The weights enter the MFMA as the EXACT integers 16 + u (a
// bf16 pattern 0x4180 | u << 3: two instructions per pair of weights instead of six for (u - z) * s rounded to bf16),
// each group of `group` columns is accumulated on its own (P = sum x' * (16 + u), fp32) and folded into the result
// as acc += s * P - s * (16 + z) * X with X = sum of the group's x' (computed once per block while staging).  That is
// sum x' * (u - z) * s with the dequantised weight NOT rounded to bf16 -- the fp32 `weight * scale` of the reference's
// CPU stand-in for this operator (tests/amct_pytorch/mock_torch_npu.py:33-55): within 1e-5 of the row's largest output
// (plus the rounding of the output) of the exact result.  The tile kernels for larger M feed bf16((u - z) * s) to the
// matrix pipe, which moves an output by up to 2^-8 * sum |x' w| (2.6e-3 of the row's largest output on W[14336,4096]
// with N(0,1) activations): the two readings are NOT within 1e-3 of each other at K = 4096, and
// amct_gemm_w4a16_weight_rounded says which one a call takes.
// The partial sums of the KS waves are added in wave order, so the result does not depend on the launch shape
// beyond KS.
#include "amct_common.h"
#include "gemm_plan.h"
#include "w4a16_stream_act.h"

namespace amct {

template <int DT>
AMCT_DEV float st_sum8(const uint4& x) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w};
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) t = t + (StAct<DT>::lo(xs[i]) + StAct<DT>::hi(xs[i]));
    return t;
}
template <int DT>
AMCT_DEV uint4 st_smooth8(const uint4& x, const uint4& c) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, cs[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = StAct<DT>::pack2(StAct<DT>::lo(xs[i]) * StAct<DT>::lo(cs[i]), StAct<DT>::hi(xs[i]) * StAct<DT>::hi(cs[i]));
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// What a wave holds of one tile of CG x 16 columns: its whole weight stream and the factors of its lane's column.
template <int NL>
struct StTile {
    u4v wv[NL];
    uint32_t fsw[NL / 2], fzw[(NL + 3) / 4];
    float bias;
};

// Issues every load of one tile (factors first, then the NL weight registers) and waits for none of them.
template <int KS, int CG, int NL>
AMCT_DEV void st_load_tile(const StreamArgs& a, StTile<NL>& t, int n0, int cg, int ks, int lane) {
    const uint32_t K = (uint32_t)a.K, G = (uint32_t)a.G;
    const int r16 = lane & 15;
    // the scales and zero-points of this lane's column for the NL groups of this wave: 2 NL and NL contiguous bytes.
    // They come from HBM like the weights and are only needed when the first group is folded, so they are loaded into
    // registers by every lane itself (a block-wide table in LDS would hold up the barrier below for as long as an
    // HBM access takes under the load of the whole launch's weight requests).
    const int fcol = n0 + cg * 16 + r16;
    const uint32_t slice = blockIdx.y;
    // (a wave whose part of a last, shorter slice lies beyond the row reads the row's last factors and its first weights:
    // its activations are zeros)
    const uint32_t row_g = (uint32_t)(a.row_k / a.group);
    const uint32_t gwave = slice * G + ks * NL;
    const size_t fidx = (size_t)(fcol < a.N ? fcol : a.N - 1) * (size_t)row_g + (gwave + NL <= row_g ? gwave : row_g - NL);
    // the bias too: a load issued in the epilogue would queue behind the next tile's weights
    // (unconditional, from `bias_src`, which is always readable: a branch here makes the wait counts of the two paths differ
    // and the compiler then waits for everything in flight)
    t.bias = a.bias_src[fcol < a.N ? fcol : a.N - 1];
#pragma unroll
    for (int q = 0; q < NL / 2; ++q) t.fsw[q] = *reinterpret_cast<const uint32_t*>(a.scales + fidx + 2 * q);
    if constexpr (NL >= 4) {
#pragma unroll
        for (int q = 0; q < NL / 4; ++q) t.fzw[q] = *reinterpret_cast<const uint32_t*>(a.zeros + fidx + 4 * q);
    } else {
        t.fzw[0] = *reinterpret_cast<const uint16_t*>(a.zeros + fidx);
    }
    __builtin_amdgcn_sched_barrier(0);
    // A load instruction fetches 8 weight rows x one whole 128-byte line (256 elements of K): lane l reads row l % 8
    // (the second instruction of a pair rows 8 .. 15) and the 16-byte chunk chunk_of(l / 8) of the line.  Whole lines per
    // instruction stream 1.3 us faster over W[14336,4096] than 16 rows x 64 bytes.  The MFMA wants 16 different rows in
    // lanes 0 .. 15 of a lane group, so the two registers of a pair swap halves afterwards (two DPP moves per word):
    // the first then holds chunks 0 .. 3 (one group of 128, chunk g in lane group g) for rows 0 .. 15, the second chunks
    // 4 .. 7 (the next group).
    const uint32_t kw = K / KS;                      // elements of K of this wave: NL steps of 128
    const uint32_t oct = lane >> 3;
    const uint32_t chunk = (oct & 1) ? 4 + (oct >> 1) : (oct >> 1);
    const int rlo = n0 + cg * 16 + (lane & 7), rhi = rlo + 8;
    const uint32_t kwave = slice * K + ks * kw;      // first element of K of this wave
    const size_t wrow = (size_t)(a.row_k / 2), woff = (size_t)(kwave < (uint32_t)a.row_k ? kwave / 2 : 0u) + chunk * 16;
    const uint8_t* wlo = a.wq + (size_t)(rlo < a.N ? rlo : a.N - 1) * wrow + woff;
    const uint8_t* whi = a.wq + (size_t)(rhi < a.N ? rhi : a.N - 1) * wrow + woff;
#pragma unroll
    for (int i = 0; i < NL; i += 2) {
        t.wv[i] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wlo + (i / 2) * 128));
        t.wv[i + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(whi + (i / 2) * 128));
    }
    __builtin_amdgcn_sched_barrier(0);
}

// Follows the weights of one tile as they land, adds the KS partial sums of a column group in wave order through
// `red` ((KS - 1) * CG * 64 * 16 bytes of LDS that nobody else touches until the next barrier but one), writes.
// FIRST_SYNC: `red` overlays the activations, so every wave has to be done reading them first.
template <int DT, int KS, int CG, int NL, bool FIRST_SYNC>
AMCT_DEV void st_compute_tile(const StreamArgs& a, StTile<NL>& t, int n0, int cg, int ks, int lane, const uint8_t* xlane,
                              const float* xsum, float* red) {
    const uint32_t kw = (uint32_t)a.K / KS;
    const int r16 = lane & 15, g = lane >> 4;
    const int M = a.M;
    s4f acc = {0.f, 0.f, 0.f, 0.f}, P = {0.f, 0.f, 0.f, 0.f};
    uint32_t km = StAct<DT>::kMask, kb = StAct<DT>::kBase;
    asm volatile("" : "+v"(km), "+v"(kb));           // in registers: (x & m) | b is then one instruction per word
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        // the loads retire in order: step i waits for wv[i] only, the younger ones stay in flight
        uint4 fa[4];
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) fa[s4] = *reinterpret_cast<const uint4*>(xlane + i * 256 + s4 * 16);
        if ((i & 1) == 0) {                          // both registers of the pair have landed: swap halves
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t lo = t.wv[i][d], hi = t.wv[i + 1][d];
                // row_ror:8 inside each row of 16 lanes; bank_mask picks the lanes that take the rotated value
                t.wv[i][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)hi, 0x128, 0xF, 0xC, false);
                t.wv[i + 1][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)lo, 0x128, 0xF, 0x3, false);
            }
        }
        const uint32_t ws[4] = {t.wv[i].x, t.wv[i].y, t.wv[i].z, t.wv[i].w};
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
            P = StAct<DT>::mfma(fa[s4], StAct<DT>::int8x(ws[s4], km, kb), P);
        {                                             // a step is one group of 128: fold it into the result
            const uint32_t gi = (ks * kw) / 128 + i;
            const uint32_t sbits = (t.fsw[i / 2] >> (16 * (i & 1))) & 0xFFFFu;
            const uint32_t zu = (t.fzw[i / 4] >> (8 * (i & 3))) & 0xFFu;
            const float s_h = f16_bits_to_f32(sbits), s_b = bf16_bits_to_f32(sbits);
            const float sc = a.scale_f16 ? s_h : s_b;
            const float c = -(sc * (float)(16u + zu));                        // exact: 5 bits x 11 bits
            const s4f X = *reinterpret_cast<const s4f*>(xsum + gi * 16 + 4 * g);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(sc, P[r], __builtin_fmaf(c, X[r], acc[r]));
            P = s4f{0.f, 0.f, 0.f, 0.f};
        }
    }
    s4f y = acc;
    if constexpr (KS > 1) {
        if constexpr (FIRST_SYNC) __syncthreads();
        if (ks > 0) *reinterpret_cast<s4f*>(red + (((ks - 1) * CG + cg) * 64 + lane) * 4) = y;
        __syncthreads();
        if (ks == 0) {
#pragma unroll
            for (int w = 0; w < KS - 1; ++w) {
                const s4f o = *reinterpret_cast<const s4f*>(red + ((w * CG + cg) * 64 + lane) * 4);
#pragma unroll
                for (int r = 0; r < 4; ++r) y[r] = y[r] + o[r];
            }
        }
    }
    const int ncol = n0 + cg * 16 + r16;
    if (ks == 0 && ncol < a.N) {
        int m0 = 4 * g;
        asm volatile("" : "+v"(m0));                  // the output addresses are computed here, per tile, not kept in registers
        if (a.part) {
            float* o = a.part + ((size_t)blockIdx.y * M + m0) * a.N + ncol;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (m0 + r < M) o[(size_t)r * a.N] = y[r];
        } else {
            uint16_t* o = a.out + (size_t)m0 * a.N + ncol;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = y[r];
                if (a.bias) v = v + t.bias;
                if (m0 + r < M) o[(size_t)r * a.N] = (uint16_t)StAct<DT>::out_bits(v);
            }
        }
    }
}

// XJ: 16-byte activation vectors a thread stages (clamped duplicates beyond the tensor).
// LOOP: a block walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ... on one staged copy of the activations, the
// next tile's loads issued before the current tile is consumed (two register sets); for weights with more tiles than
// the device runs blocks at once, where staging the activations per tile costs as much traffic as the tile's weights.
template <int DT, int KS, int CG, int NL, int XJ, bool SMOOTH, bool LOOP>
__global__ __launch_bounds__(KS * CG * 64) void w4a16_stream(StreamArgs a) {
    static_assert(NL % 2 == 0, "the weight loads come in pairs");
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int NT = KS * CG * 64;
    constexpr int COLS = CG * 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cg = wave / KS, ks = wave % KS;
    const int r16 = lane & 15, g = lane >> 4;
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M, G = (uint32_t)a.G;
    const uint32_t xstride = K * 2 + 16;             // 16 bytes of padding: the 16 rows of a fragment read hit different banks
    const uint32_t xbytes = M * xstride;
    constexpr uint32_t kRedBytes = (KS - 1) * CG * 64 * 16;
    uint8_t* xs = lds;
    float* xsum = reinterpret_cast<float*>(lds + xbytes);   // [G][16]: sum of x' per group and row

    // ---- staging loads (activations, smoothing factors) --------------------------------------------------------
    const uint32_t KV = K / 8, n_xv = M * KV;
    uint4 xv[XJ], cv[XJ];
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
        if constexpr (SMOOTH) cv[j] = ldg16(a.smooth + (inside ? xk : 0u));
    }
    // ---- the whole weight stream of this wave for its first tile -------------------------------------------------
    int tile = blockIdx.x;
    StTile<NL> ta;
    st_load_tile<KS, CG, NL>(a, ta, tile * COLS, cg, ks, lane);

    // ---- stage the activations: smoothed, interleaved to the operand order of st_int8x, summed per group ----------
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        if constexpr (SMOOTH) xv[j] = st_smooth8<DT>(xv[j], cv[j]);
        // 16 consecutive lanes hold 128 consecutive elements of one row; whole groups of 16 lanes are valid or not
        float t = st_sum8<DT>(xv[j]);
        t = t + __shfl_xor(t, 1);
        t = t + __shfl_xor(t, 2);
        t = t + __shfl_xor(t, 4);
        t = t + __shfl_xor(t, 8);
        if (v < n_xv) {
            *reinterpret_cast<uint4*>(xs + xrow[j] * xstride + xkv[j] * 16) = st_interleave8(xv[j]);
            if ((tid & 15) == 0) {
                xsum[(xkv[j] >> 4) * 16 + xrow[j]] = t;
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    const uint32_t kw = K / KS;
    const uint8_t* xlane = xs + (r16 < (int)M ? r16 : (int)M - 1) * xstride + (ks * kw + g * 32) * 2;
    if constexpr (!LOOP) {
        st_compute_tile<DT, KS, CG, NL, true>(a, ta, tile * COLS, cg, ks, lane, xlane, xsum, reinterpret_cast<float*>(lds));
    } else {
        // two reduction buffers behind the activation image, used in turn: a tile's partial sums are read before the
        // reading wave reaches the next tile's barrier, and written again only after that barrier
        float* red0 = reinterpret_cast<float*>(lds + xbytes + G * 64);
        float* red1 = red0 + kRedBytes / 4;
        const int tiles = (a.N + COLS - 1) / COLS, stride = gridDim.x;
        StTile<NL> tb;
        for (;;) {
            int next = tile + stride;
            if (next >= tiles) {
                st_compute_tile<DT, KS, CG, NL, false>(a, ta, tile * COLS, cg, ks, lane, xlane, xsum, red0);
                break;
            }
            st_load_tile<KS, CG, NL>(a, tb, next * COLS, cg, ks, lane);
            st_compute_tile<DT, KS, CG, NL, false>(a, ta, tile * COLS, cg, ks, lane, xlane, xsum, red0);
            tile = next;
            next = tile + stride;
            if (next >= tiles) {
                st_compute_tile<DT, KS, CG, NL, false>(a, tb, tile * COLS, cg, ks, lane, xlane, xsum, red1);
                break;
            }
            st_load_tile<KS, CG, NL>(a, ta, next * COLS, cg, ks, lane);
            st_compute_tile<DT, KS, CG, NL, false>(a, tb, tile * COLS, cg, ks, lane, xlane, xsum, red1);
            tile = next;
        }
    }
}

int splitk_reduce16_launch(const float* part, const float* bias, void* out, int64_t M, int64_t N, int splits, int dtype,
                           hipStream_t st);                          // gemm_w4a16.hip
bool w4a16_wave_fits(int64_t N, int64_t K_slice, int64_t slices);    // gemm_w4a16_wave.hip: the form with wave-private staging
int w4a16_wave_launch(const StreamArgs& a, int slices, int dtype, hipStream_t st);

template <int DT, int KS, int CG, int NL, bool SMOOTH, bool LOOP>
static int stream_launch_x(const StreamArgs& a, size_t lds_bytes, dim3 blocks, hipStream_t st) {
    constexpr int NT = KS * CG * 64;
    const int n_xv = a.M * (a.K / 8);
    const int xj = (n_xv + NT - 1) / NT;
    const dim3 grid = blocks;
#define AMCT_STREAM_GO(XJ)                                                                                          \
    {                                                                                                               \
        auto kern = &w4a16_stream<DT, KS, CG, NL, XJ, SMOOTH, LOOP>;                                                \
        if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess) { \
            (void)hipGetLastError();                                                                                \
            return AMCT_E_HIP;                                                                                      \
        }                                                                                                           \
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, st, a);                                                 \
        if (a.part) return splitk_reduce16_launch(a.part, a.bias, a.out, a.M, a.N, (int)grid.y, DT, st);            \
        return hip_status();                                                                                        \
    }
    if (xj <= 2) AMCT_STREAM_GO(2)
    if (xj <= 4) AMCT_STREAM_GO(4)
    if (xj <= 8) AMCT_STREAM_GO(8)
#undef AMCT_STREAM_GO
    return AMCT_E_UNSUPPORTED;
}

// The slice of K one block walks: K itself when it is 1024, 2048 or 4096, else the largest of those that divides K into at
// most 16 slices (8192 = 2 x 4096, 14336 = 7 x 2048, 5120 = 5 x 1024, 28672 = 7 x 4096); 0: none.
static int64_t stream_slice(int64_t K) {
    if (K == 1024 || K == 2048 || K == 4096) return K;
    for (int64_t ks = 4096; ks >= 1024; ks /= 2)
        if (K % ks == 0 && K / ks <= 16) return ks;
    // other multiples of 256 (11008, 13824): slices of 1024 whose last one is shorter -- a wave walks 256 elements, so it
    // lies inside the row or beyond it as a whole
    if (K % 256 == 0 && K > 1024 && (K + 1023) / 1024 <= 16) return 1024;
    return 0;
}
// Sliced rows pay a second launch: taken from 5 rows on, or for rows of 12288 elements and more (measured against the
// older kernels for a few rows, us: W[8192,8192] M = 1 / 4 / 16: 13.2 / 14.0 / 22.3 against 16.1 / 16.0 / 16.3 sliced;
// W[28672,8192]: 30.6 / 38.6 / 86.9 against 34.7 / 35.5 / 37.2; W[8192,28672]: 105 / 80 / 79 against 31 / 34 / 41).
// Rows whose 256-element units do not split evenly over the four waves of those older kernels (11008, 13824) come here for any M
// (W[4096,11008], us at M = 1 / 5 / 8 / 16: 18.6 / 18.1 / 18.1 / 18.2 on the split tile kernels against 16 / 16.1 / 15.0 / 17.7;
// W[5120,13824]: 34.5 against 18 - 24).
static bool stream_slices_pay(int64_t M, int64_t K) { return M >= 5 || K >= 12288 || (K / 256) % 4 != 0; }
size_t w4a16_stream_part_bytes(int64_t M, int64_t N, int64_t K, int group) {
    const int64_t ks = stream_slice(K);
    if (M < 1 || M > 16 || group != 128 || !ks || ks == K || N % 8 != 0 || !stream_slices_pay(M, K)) return 0;
    return (size_t)((K + ks - 1) / ks) * (size_t)M * (size_t)N * 4;
}

// Whether this kernel takes a call of this shape with a workspace of this size (operands suitably aligned): the one
// rule behind the dispatch below and behind amct_gemm_w4a16_weight_rounded.
bool w4a16_stream_takes(int64_t M, int64_t N, int64_t K_row, int group, size_t workspace_bytes) {
    // one group per step of 128 elements of K (the per-group partial sums of a step cannot be separated otherwise)
    const int64_t K = stream_slice(K_row), S = K ? (K_row + K - 1) / K : 0;
    if (M < 1 || M > 16 || !K || group != 128 || N <= 0 || N > (int64_t(1) << 30)) return false;
    if (S > 1) {
        // rows of several slices: the partial sums go through the lent workspace
        const size_t need = w4a16_stream_part_bytes(M, N, K_row, group);
        if (!need || workspace_bytes < need) return false;
    }
    // what the launch shapes below hold: an activation image of at most 160 KB, at most 8 vectors staged per thread
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16), img = xbytes + (size_t)(K / group) * 64;
    const int64_t cg = xbytes > 40 * 1024 ? 4 : xbytes > 12 * 1024 ? 2 : 1;
    return img <= 160 * 1024 && (M * (K / 8) + 256 * cg - 1) / (256 * cg) <= 8;
}

// Returns AMCT_E_UNSUPPORTED when the shape is not one this kernel takes (the caller then uses its other kernels).
int w4a16_stream_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                          const uint8_t* zeros, const float* bias, void* out, int64_t M, int64_t N, int64_t K_row, int group,
                          int dtype, void* workspace, size_t workspace_bytes, hipStream_t st) {
    if (!w4a16_stream_takes(M, N, K_row, group, workspace ? workspace_bytes : 0)) return AMCT_E_UNSUPPORTED;
    const int64_t K = stream_slice(K_row), S = (K_row + K - 1) / K;
    if (!aligned16(x) || !aligned16(wq) || (smooth && !aligned16(smooth)) || ((uintptr_t)scales & 3) || ((uintptr_t)zeros & 3))
        return AMCT_E_UNSUPPORTED;
    float* part = nullptr;
    if (S > 1) {
        if (!aligned16(workspace) || !aligned16(out) || (bias && !aligned16(bias))) return AMCT_E_UNSUPPORTED;
        part = reinterpret_cast<float*>(workspace);
    }
    StreamArgs a{(const uint16_t*)x, (const uint16_t*)smooth, wq, (const uint16_t*)scales, zeros, bias,
                 bias ? bias : reinterpret_cast<const float*>(scales),   // N * K / group * 2 >= N * 4 bytes (K >= 1024)
                 (uint16_t*)out, (int)M, (int)N, (int)K, (int)(K / group), group, scale_dtype == AMCT_F16 ? 1 : 0,
                 (uint32_t)(0x100000000ull / (uint64_t)(K / 8)) + 1u, (int)K_row, part};
    // launches whose blocks all run at once: every wave stages its own 256 elements of K (gemm_w4a16_wave.hip)
    // Taken where it measured faster than the form below (us on W[14336,4096] / W[4096,4096] / W[8192,8192], this form
    // against that one): with smoothing M = 5: 10.7 / 10.5 / 13.4 against 10.9 / 10.2 / 13.4, M = 8: 10.8 / 10.6 / 13.4
    // against 11.2 / 10.4 / 13.9, M = 16: 11.4 / 10.9 / 14.1 against 13.2 / 12.5 / 16.0; without smoothing M = 12:
    // 11.0 / 10.8 / 14.1 against 11.4 / 10.8 / 14.1, M = 16: 11.2 / 10.9 / 14.1 against 11.9 / 11.1 / 14.8.  Below that the
    // narrow blocks of the form below win (M = 1: 8.5 against 10.2 us: a block of this form is a whole CU's work however
    // few rows there are); slices shorter than 4096 (W[4096,14336]: 7 x 2048) stay below as well (M = 16: 15.2 against 15.9).
    if ((smooth ? M >= 5 : M >= 12) && (S == 1 || K == 4096) && w4a16_wave_fits(N, K, S))
        return w4a16_wave_launch(a, (int)S, dtype, st);
    // A wave streams K / 4 elements of 16 columns in NL = K / 512 steps, all of them in flight from the start.  Large
    // activation blocks are staged by few, wide blocks (16 waves share one copy in LDS); small ones by many narrow
    // blocks, several per CU.  Measured on W[14336,4096]: 8.8 us at M = 1 (11.0 us for the kernel this one replaced),
    // 12.9 us at M = 16 (17.3 us); preparing the activation image once in a kernel of its own instead of in every block
    // was slower for every M (the second launch costs more than the staging arithmetic it removes).
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16);
    const int cg = xbytes > 40 * 1024 ? 4 : xbytes > 12 * 1024 ? 2 : 1;
    const int64_t nl = K / 512;
    const size_t red = (size_t)3 * cg * 64 * 16, img = xbytes + (size_t)(K / group) * 64;
    // More tiles than CUs under a wide block (one per CU: its activation image fills most of the LDS): one block per CU
    // walks its share of the tiles on one staged copy of the activations.  W[128256,4096] at M = 8 / 16: 82 / 96 ->
    // 62 / 63 us; W[28672,4096]: 22.6 / 25.4 -> 19.1 / 20.0 us.  The narrower blocks for smaller activation images (several
    // per CU, which overlap one block's staging with another's stream) were 5 - 15 % slower in this form.
    const int64_t tiles = (N + cg * 16 - 1) / (cg * 16), cus = current_cu_count();
    const size_t loop_bytes = img + 2 * red;
    const bool loop = cg == 4 && cus > 0 && tiles * S > cus && tiles > 1 && loop_bytes <= 160 * 1024;
    const size_t lds_bytes = loop ? loop_bytes : img > red ? img : red;
    const int64_t per_slice = cus / S > 0 ? cus / S : 1;            // blocks per slice when they walk tiles
    const dim3 blocks((unsigned)(loop ? (tiles < per_slice ? tiles : per_slice) : tiles), (unsigned)S);
    if (lds_bytes > 160 * 1024) return AMCT_E_UNSUPPORTED;
#define AMCT_STREAM_DT(DT_, CG_, NL_, LOOP_)                                                              \
    return smooth ? stream_launch_x<DT_, 4, CG_, NL_, true, LOOP_>(a, lds_bytes, blocks, st)              \
                  : stream_launch_x<DT_, 4, CG_, NL_, false, LOOP_>(a, lds_bytes, blocks, st);
#define AMCT_STREAM_SHAPE(CG_, NL_)                                                                       \
    if (cg == CG_ && nl == NL_) {                                                                         \
        if (dtype == AMCT_F16) { AMCT_STREAM_DT(AMCT_F16, CG_, NL_, false) }                              \
        AMCT_STREAM_DT(AMCT_BF16, CG_, NL_, false)                                                        \
    }
#define AMCT_STREAM_SHAPE_LOOP(NL_)                                                                       \
    if (cg == 4 && nl == NL_ && loop) {                                                                   \
        if (dtype == AMCT_F16) { AMCT_STREAM_DT(AMCT_F16, 4, NL_, true) }                                 \
        AMCT_STREAM_DT(AMCT_BF16, 4, NL_, true)                                                           \
    }
    AMCT_STREAM_SHAPE_LOOP(8)
    AMCT_STREAM_SHAPE_LOOP(4)
    AMCT_STREAM_SHAPE_LOOP(2)
    AMCT_STREAM_SHAPE(4, 8)
    AMCT_STREAM_SHAPE(2, 8)
    AMCT_STREAM_SHAPE(1, 8)
    AMCT_STREAM_SHAPE(4, 4)
    AMCT_STREAM_SHAPE(2, 4)
    AMCT_STREAM_SHAPE(1, 4)
    AMCT_STREAM_SHAPE(4, 2)
    AMCT_STREAM_SHAPE(2, 2)
    AMCT_STREAM_SHAPE(1, 2)
#undef AMCT_STREAM_SHAPE_LOOP
#undef AMCT_STREAM_SHAPE
#undef AMCT_STREAM_DT
    return AMCT_E_UNSUPPORTED;                        // K / 512 steps per wave beyond 8: the other kernels
}

}  // namespace amct
