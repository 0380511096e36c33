// K2: int4 per-group quantise + nibble pack in one pass, and the int4 interchange layouts.
// Reference behaviour: amct_pytorch/deploy_op/weight_npu_quant_module.py:38-66 (weight preparation),
// amct_pytorch/utils/quant_util.py:76-93 (codes), amct_pytorch/quantize_op/utils.py:75-136 (factors).
#include <type_traits>

#include "amct_common.h"

namespace amct {

struct PackArgs {
    const void* w;
    uint8_t* packed;
    void* scales16;
    float* scales32;
    uint8_t* zeros;
    int32_t* bad;
    const void* col;
    int64_t nseg;
    int seg_len;
    int segs_per_row;
    int scale_dtype;
    int col_mode;
    int symmetric;
};

// A team of T lanes owns one group; each lane holds NV 16-byte vectors; U groups in flight.
template <int DT, int T, int NV, int U>
__global__ __launch_bounds__(kBlock) void int4_group_pack(PackArgs a) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    constexpr int TEAMS = kBlock / T;
    const int tid = threadIdx.x;
    const int team = tid / T, lt = tid % T;
    const int S = a.seg_len / VEC;
    const bool asym = !a.symmetric;
    const float inf = __builtin_huge_valf();

    float x[U][NV][VEC];
    int64_t seg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        seg[u] = ((int64_t)blockIdx.x * U + u) * TEAMS + team;
        const bool ok = seg[u] < a.nseg;
        uint4 raw[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = i * T + lt;
            raw[i] = make_uint4(0, 0, 0, 0);
            if (ok && v < S)
                raw[i] = ldg16(reinterpret_cast<const char*>(a.w) + (seg[u] * a.seg_len + (int64_t)v * VEC) * BYTES);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) unpack16<DT>(raw[i], x[u][i]);
    }

    if (a.col_mode != AMCT_COL_NONE) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t c0 = (seg[u] % a.segs_per_row) * (int64_t)a.seg_len;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = i * T + lt;
                if (seg[u] < a.nseg && v < S) {
                    float c[VEC];
                    unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.col) + (c0 + (int64_t)v * VEC) * BYTES), c);
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        x[u][i][j] = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x[u][i][j] / c[j] : x[u][i][j] * c[j]);
                }
            }
        }
    }

    float mx[U], mn[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        mx[u] = -inf;
        mn[u] = inf;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = i * T + lt;
            if (seg[u] < a.nseg && v < S) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    mx[u] = fmax_nan(mx[u], x[u][i][j]);
                    mn[u] = fmin_nan(mn[u], x[u][i][j]);
                }
            }
        }
        team_minmax<T>(mn[u], mx[u]);
    }

#pragma unroll
    for (int u = 0; u < U; ++u) {
        const bool ok = seg[u] < a.nseg;
        const Factors f = make_factors<AMCT_F32>(mx[u], mn[u], 4, a.symmetric != 0, AMCT_SCOPE_AMCT);
        if (ok && lt == 0) {
            if (a.scales32) a.scales32[seg[u]] = f.s;
            if (a.scales16) {
                if (a.scale_dtype == AMCT_F16) reinterpret_cast<uint16_t*>(a.scales16)[seg[u]] = (uint16_t)f32_to_f16_bits(f.s);
                else reinterpret_cast<uint16_t*>(a.scales16)[seg[u]] = (uint16_t)f32_to_bf16_bits(f.s);
            }
            if (a.zeros) a.zeros[seg[u]] = (uint8_t)((int)f.z + 8);
            if (f.bad && a.bad) atomicAdd(a.bad, 1);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = i * T + lt;
            if (ok && v < S) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float q = quant_elem<DT, false>(x[u][i][j], f.s, f.z, asym, -8.f, 7.f);
                    word |= (uint32_t)((int)q + 8) << (4 * j);
                }
                const int64_t b0 = (seg[u] * a.seg_len + (int64_t)v * VEC) / 2;
                if constexpr (VEC == 8) *reinterpret_cast<uint32_t*>(a.packed + b0) = word;
                else *reinterpret_cast<uint16_t*>(a.packed + b0) = (uint16_t)word;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// main kernel (groups of at most 64 vectors).  A team of T lanes owns 4 consecutive groups; lane lt
// holds vector lt of each, so 4 x 16 bytes per lane are in flight.  Loads are unconditional (indices
// are clamped, duplicates do not change a min/max), streaming, and issued before any use.
// The factors of group u are computed by the lanes with lt % 4 == u and shared inside each quad by
// DPP; the per-element division is the exact fma sequence when every group of the wave allows it.
// ---------------------------------------------------------------------------
// FULL: every block is complete (the group count is a multiple of the groups per block), every lane's vector exists
// (group length = T * NV vectors) and the tensor is below 2 GiB: addresses are then one wave-uniform 64-bit base per
// block plus 32-bit lane offsets and nothing is clamped or predicated, which removes 70 of the 560 vector
// instructions a wave executes for its 2048 elements (counted by the hardware).
template <int DT, int T, int NV, bool COL, bool FULL = false>
__global__ __launch_bounds__(kBlock) void int4_group_pack4(PackArgs a) {
    constexpr int U = 4;
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    constexpr int TEAMS = kBlock / T;
    const int tid = threadIdx.x;
    const int team = tid / T, lt = tid % T;
    const int S = a.seg_len / VEC;
    const bool asym = !a.symmetric;
    const int64_t seg0 = ((int64_t)blockIdx.x * TEAMS + team) * U;
    int vl[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) vl[v] = (lt + T * v < S) ? lt + T * v : S - 1;

    // one 64-bit base per lane (first group of the team, clamped into the tensor), then 32-bit offsets per group:
    // group u of the team is u groups further, or the last group of the tensor if the team hangs over its end
    uint4 raw[U][NV];
    int64_t segc[U];
    const uint32_t blk_bytes = (uint32_t)(TEAMS * U) * (uint32_t)a.seg_len * BYTES;      // input bytes of one block
    const uint32_t lane_off = (uint32_t)(team * U) * ((uint32_t)a.seg_len * BYTES) + (uint32_t)lt * 16u;
    if constexpr (FULL) {
        const char* blk = reinterpret_cast<const char*>(a.w) + (int64_t)blockIdx.x * blk_bytes;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            segc[u] = seg0 + u;
#pragma unroll
            for (int v = 0; v < NV; ++v)
                raw[u][v] = ldg16_nt(blk + (lane_off + (uint32_t)u * ((uint32_t)a.seg_len * BYTES) + (uint32_t)(v * T * 16)));
        }
    }
    const int64_t seg_first = seg0 < a.nseg ? seg0 : a.nseg - 1;
    const int64_t left = a.nseg - 1 - seg_first;                    // groups after the first one
    const int left32 = left < U ? (int)left : U - 1;
    const char* base = reinterpret_cast<const char*>(a.w) + seg_first * a.seg_len * BYTES;
    const uint32_t seg_bytes = (uint32_t)a.seg_len * BYTES;
    if constexpr (!FULL) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int uc = u < left32 ? u : left32;
            segc[u] = seg_first + uc;
#pragma unroll
            for (int v = 0; v < NV; ++v) raw[u][v] = ldg16_nt(base + (uint32_t)uc * seg_bytes + (uint32_t)vl[v] * 16u);
        }
    }
    float x[U][NV][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int v = 0; v < NV; ++v) unpack16<DT>(raw[u][v], x[u][v]);
    if constexpr (COL) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t c0 = (segc[u] % a.segs_per_row) * (int64_t)a.seg_len;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float c[VEC];
                unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.col) + (c0 + (int64_t)vl[v] * VEC) * BYTES), c);
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    x[u][v][j] = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x[u][v][j] / c[j] : x[u][v][j] * c[j]);
            }
        }
    }
    float mx[U], mn[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        mx[u] = x[u][0][0];
        mn[u] = x[u][0][0];
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int j = (v == 0 ? 1 : 0); j < VEC; ++j) {
                mx[u] = fmax_nan(mx[u], x[u][v][j]);
                mn[u] = fmin_nan(mn[u], x[u][v][j]);
            }
    }
    // lane lt ends up with the extrema of group seg4_of_lane(lt) and computes its factors
    const int my = seg4_of_lane(lt);
    float mx_my, mn_my;
    team_minmax_scatter4<T>(mn, mx, lt, mn_my, mx_my);
    const Factors f = make_factors<AMCT_F32>(mx_my, mn_my, 4, a.symmetric != 0, AMCT_SCOPE_AMCT);
    const Divisor dmy = divisor_of(f);
    const uint32_t big = max(__float_as_uint(mx_my) & 0x7FFFFFFFu, __float_as_uint(mn_my) & 0x7FFFFFFFu);
    const bool fast = wave_all(dmy.fast && big < 0x5D800000u);       // |x| < 2^60, finite
    if (lt < 4 && (FULL || seg0 + my < a.nseg)) {
        const int64_t sg = FULL ? (int64_t)blockIdx.x * (TEAMS * U) + (team * U + my) : seg0 + my;
        if (a.scales32) a.scales32[sg] = f.s;
        if (a.scales16) {
            reinterpret_cast<uint16_t*>(a.scales16)[sg] =
                (uint16_t)(a.scale_dtype == AMCT_F16 ? f32_to_f16_bits(f.s) : f32_to_bf16_bits(f.s));
        }
        if (a.zeros) a.zeros[sg] = (uint8_t)((int)f.z + 8);
        if (f.bad && a.bad) atomicAdd(a.bad, 1);
    }
    // quad lane holding segment u: u = 0 -> lane 0, 1 -> lane 2, 2 -> lane 1, 3 -> lane 3
    Divisor dv[U];
    float z[U];
    dv[0].s = quad_bcast<0>(f.s); dv[0].y = quad_bcast<0>(dmy.y); z[0] = quad_bcast<0>(f.z);
    dv[1].s = quad_bcast<2>(f.s); dv[1].y = quad_bcast<2>(dmy.y); z[1] = quad_bcast<2>(f.z);
    dv[2].s = quad_bcast<1>(f.s); dv[2].y = quad_bcast<1>(dmy.y); z[2] = quad_bcast<1>(f.z);
    dv[3].s = quad_bcast<3>(f.s); dv[3].y = quad_bcast<3>(dmy.y); z[3] = quad_bcast<3>(f.z);

    // codes u = q + 8 are gathered by exact fp32 arithmetic: sum (q_j + 8) * 16^j over 4 nibbles
    uint32_t word[U][NV];
    // keeps each variant's arithmetic inside its own branch: without it the optimiser computes the first product of
    // every division ahead of the four-way branch and holds 32 more registers live
    auto pinned = [](float v) {
        asm volatile("" : "+v"(v));
        return v;
    };
    auto encode = [&](auto fast_tag, auto asym_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
        constexpr bool ASYM = decltype(asym_tag)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float lo = 34952.0f, hi = 34952.0f;              // 8 * (1 + 16 + 256 + 4096)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float q = quant_elem<DT, false, FAST, false>(pinned(x[u][v][j]), dv[u], z[u], ASYM, -8.f, 7.f);
                    lo = __builtin_fmaf(q, (float)(1 << (4 * j)), lo);
                }
                if constexpr (VEC == 8) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float q = quant_elem<DT, false, FAST, false>(pinned(x[u][v][4 + j]), dv[u], z[u], ASYM, -8.f, 7.f);
                        hi = __builtin_fmaf(q, (float)(1 << (4 * j)), hi);
                    }
                    word[u][v] = (uint32_t)lo | ((uint32_t)hi << 16);
                } else {
                    word[u][v] = (uint32_t)lo;
                }
                // one word at a time: left alone, the scheduler interleaves all 32 elements of a lane; bounded, the
                // kernel needs fewer registers and runs 5 % faster (26.7 us against 28.1 us on W[14336,4096] bf16)
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if (fast && asym) encode(std::true_type{}, std::true_type{});
    else if (fast) encode(std::true_type{}, std::false_type{});
    else if (asym) encode(std::false_type{}, std::true_type{});
    else encode(std::false_type{}, std::false_type{});
    if constexpr (FULL) {
        // a 16-byte input vector becomes VEC / 2 output bytes: the output offsets are the input offsets / (2 * BYTES)
        uint8_t* oblk = a.packed + (int64_t)blockIdx.x * (blk_bytes / (2 * BYTES));
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t o = (lane_off + (uint32_t)u * ((uint32_t)a.seg_len * BYTES) + (uint32_t)(v * T * 16)) / (2 * BYTES);
                if constexpr (VEC == 8) stg4_nt(oblk + o, word[u][v]);
                else *reinterpret_cast<uint16_t*>(oblk + o) = (uint16_t)word[u][v];
            }
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            if (lt + T * v < S && seg0 + u < a.nseg) {
                const int64_t b0 = ((seg0 + u) * a.seg_len + (int64_t)(lt + T * v) * VEC) / 2;
                if constexpr (VEC == 8) stg4_nt(a.packed + b0, word[u][v]);
                else *reinterpret_cast<uint16_t*>(a.packed + b0) = (uint16_t)word[u][v];
            }
        }
    }
}

// general kernel: one block per row, scalar loads; cols % group == 0 and cols even.
template <int DT>
__global__ __launch_bounds__(kBlock) void int4_group_pack_general(PackArgs a, int64_t cols) {
    __shared__ float sm[2][kBlock / kWave];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const bool asym = !a.symmetric;
    const float inf = __builtin_huge_valf();
    for (int sg = 0; sg < a.segs_per_row; ++sg) {
        const int64_t c_begin = (int64_t)sg * a.seg_len, c_end = c_begin + a.seg_len;
        float mx = -inf, mn = inf;
        for (int64_t c = c_begin + tid; c < c_end; c += kBlock) {
            float x = load_scalar<DT>(a.w, row * cols + c);
            if (a.col_mode != AMCT_COL_NONE) {
                const float cs = load_scalar<DT>(a.col, c);
                x = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x / cs : x * cs);
            }
            mx = fmax_nan(mx, x);
            mn = fmin_nan(mn, x);
        }
        team_minmax<kWave>(mn, mx);
        __syncthreads();
        if ((tid & (kWave - 1)) == 0) {
            sm[0][tid / kWave] = mn;
            sm[1][tid / kWave] = mx;
        }
        __syncthreads();
#pragma unroll
        for (int wv = 0; wv < kBlock / kWave; ++wv) {
            mn = fmin_nan(mn, sm[0][wv]);
            mx = fmax_nan(mx, sm[1][wv]);
        }
        const Factors f = make_factors<AMCT_F32>(mx, mn, 4, a.symmetric != 0, AMCT_SCOPE_AMCT);
        const int64_t pi = row * a.segs_per_row + sg;
        if (tid == 0) {
            if (a.scales32) a.scales32[pi] = f.s;
            if (a.scales16) {
                if (a.scale_dtype == AMCT_F16) reinterpret_cast<uint16_t*>(a.scales16)[pi] = (uint16_t)f32_to_f16_bits(f.s);
                else reinterpret_cast<uint16_t*>(a.scales16)[pi] = (uint16_t)f32_to_bf16_bits(f.s);
            }
            if (a.zeros) a.zeros[pi] = (uint8_t)((int)f.z + 8);
            if (f.bad && a.bad) atomicAdd(a.bad, 1);
        }
        for (int64_t c = c_begin + 2 * tid; c < c_end; c += 2 * kBlock) {
            uint32_t byte = 0;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float x = load_scalar<DT>(a.w, row * cols + c + j);
                if (a.col_mode != AMCT_COL_NONE) {
                    const float cs = load_scalar<DT>(a.col, c + j);
                    x = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x / cs : x * cs);
                }
                const float q = quant_elem<DT, false>(x, f.s, f.z, asym, -8.f, 7.f);
                byte |= (uint32_t)((int)q + 8) << (4 * j);
            }
            a.packed[(row * cols + c) / 2] = (uint8_t)byte;
        }
    }
}

template <int DT, int T, int NV, int U>
static void launch_pack(const PackArgs& a, hipStream_t st) {
    const int64_t per_block = (int64_t)(kBlock / T) * U;
    const int64_t nb = (a.nseg + per_block - 1) / per_block;
    hipLaunchKernelGGL((int4_group_pack<DT, T, NV, U>), dim3((unsigned)nb), dim3(kBlock), 0, st, a);
}

template <int DT, int T, int NV>
static void launch_pack4(const PackArgs& a, hipStream_t st) {
    const int64_t per_block = (int64_t)(kBlock / T) * 4;
    const int64_t nb = (a.nseg + per_block - 1) / per_block;
    constexpr int BYTES = Tr<DT>::BYTES, VEC = Tr<DT>::VEC;
    const bool full = a.nseg % per_block == 0 && a.seg_len == T * NV * VEC && a.nseg * a.seg_len * BYTES < (int64_t(1) << 31);
    if (a.col_mode != AMCT_COL_NONE) hipLaunchKernelGGL((int4_group_pack4<DT, T, NV, true>), dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    else if (full) hipLaunchKernelGGL((int4_group_pack4<DT, T, NV, false, true>), dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((int4_group_pack4<DT, T, NV, false>), dim3((unsigned)nb), dim3(kBlock), 0, st, a);
}

template <int DT>
static int run_pack(const PackArgs& a, int64_t rows, int64_t cols, hipStream_t st) {
    constexpr int VEC = Tr<DT>::VEC;
    const int S = a.seg_len / VEC;
    const bool vec_ok = aligned16(a.w) && (reinterpret_cast<uintptr_t>(a.packed) & 3u) == 0 &&
                        (a.col_mode == AMCT_COL_NONE || aligned16(a.col));
    if (vec_ok && S <= 64) {
        // one vector per lane and group (NV = 1) measured fastest: 2 vectors per lane halve the per-lane
        // fixed work but cost occupancy (106 instead of 69 registers), 30.8 us against 29.6 us
        if (S <= 4) launch_pack4<DT, 4, 1>(a, st);
        else if (S <= 8) launch_pack4<DT, 8, 1>(a, st);
        else if (S <= 16) launch_pack4<DT, 16, 1>(a, st);
        else if (S <= 32) launch_pack4<DT, 32, 1>(a, st);
        else launch_pack4<DT, 64, 1>(a, st);
        return hip_status();
    }
    if (vec_ok && S <= 512) {
        if (S <= 128) launch_pack<DT, 64, 2, 2>(a, st);
        else if (S <= 256) launch_pack<DT, 64, 4, 1>(a, st);
        else launch_pack<DT, 64, 8, 1>(a, st);
        return hip_status();
    }
    if (rows > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL((int4_group_pack_general<DT>), dim3((unsigned)rows), dim3(kBlock), 0, st, a, cols);
    return hip_status();
}

// int32 [k, n] one signed int4 each -> int32 [k, n/8]
__global__ __launch_bounds__(kBlock) void pack_words_k(const int32_t* codes, int32_t* words, int64_t nwords) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= nwords) return;
    const int4 lo = *reinterpret_cast<const int4*>(codes + i * 8);
    const int4 hi = *reinterpret_cast<const int4*>(codes + i * 8 + 4);
    const uint32_t w = ((uint32_t)lo.x & 0xF) | (((uint32_t)lo.y & 0xF) << 4) | (((uint32_t)lo.z & 0xF) << 8) |
                       (((uint32_t)lo.w & 0xF) << 12) | (((uint32_t)hi.x & 0xF) << 16) | (((uint32_t)hi.y & 0xF) << 20) |
                       (((uint32_t)hi.z & 0xF) << 24) | (((uint32_t)hi.w & 0xF) << 28);
    words[i] = (int32_t)w;
}

// int32 [k, n/8] (column 8i+j in nibble j, signed) -> uint8 [n, k/2] (code+8, even k low).
// One thread per (word column i, k pair): reads two words, writes 8 bytes (strided by k/2).
__global__ __launch_bounds__(kBlock) void words_to_nibbles_k(const int32_t* words, uint8_t* packed, int64_t k, int64_t n8) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t kp = k / 2;
    if (idx >= kp * n8) return;
    const int64_t i = idx % n8, p = idx / n8;       // consecutive threads read consecutive words
    const uint32_t w0 = (uint32_t)words[(2 * p) * n8 + i] ^ 0x88888888u;        // +8 mod 16 on every nibble
    const uint32_t w1 = (uint32_t)words[(2 * p + 1) * n8 + i] ^ 0x88888888u;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t b = ((w0 >> (4 * j)) & 0xF) | (((w1 >> (4 * j)) & 0xF) << 4);
        packed[(i * 8 + j) * kp + p] = (uint8_t)b;
    }
}

// int8 codes [rows, cols] (signed int4 values) -> uint8 [rows, cols/2] (code+8, even column low)
__global__ __launch_bounds__(kBlock) void pack_nibbles_k(const int8_t* codes, uint8_t* packed, int64_t nbytes) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= nbytes) return;
    const uint32_t lo = ((uint32_t)codes[2 * i] + 8u) & 0xFu, hi = ((uint32_t)codes[2 * i + 1] + 8u) & 0xFu;
    packed[i] = (uint8_t)(lo | (hi << 4));
}

// uint8 [n, k/2] -> int32 [k, n] signed codes (the operand of the word packer)
__global__ __launch_bounds__(kBlock) void nibbles_to_codes_kn_k(const uint8_t* packed, int32_t* codes, int64_t k, int64_t n) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= k * n) return;
    const int64_t col = idx % n, row = idx / n;          // consecutive threads write consecutive n
    const uint32_t b = packed[col * (k / 2) + row / 2];
    const int32_t u = (row & 1) ? (int32_t)(b >> 4) : (int32_t)(b & 0xFu);
    codes[idx] = u - 8;
}

// ---- the same three conversions for aligned shapes: 16-byte accesses, transposes through an LDS tile ----
// (the kernels above touch one word or byte per thread with strided partners: 147 us, 41 us and 224 us for
// W[14336,4096])

// 128 k-rows x 16 words (128 columns) per block: coalesced word loads, then thread (column c, half h) gathers the
// nibbles of its column over 64 k-rows into 32 consecutive output bytes.  k % 128 == 0, n8 % 16 == 0.
__global__ __launch_bounds__(kBlock) void words_to_nibbles_tile_k(const int32_t* words, uint8_t* packed, int64_t k, int64_t n8) {
    __shared__ uint32_t tile[128][17];
    const int tid = threadIdx.x;
    const int64_t i0 = (int64_t)blockIdx.x * 16, k0 = (int64_t)blockIdx.y * 128;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int kr = tid / 16 + 16 * j, i = tid % 16;
        tile[kr][i] = (uint32_t)words[(k0 + kr) * n8 + i0 + i] ^ 0x88888888u;     // +8 mod 16 on every nibble
    }
    __syncthreads();
    const int c = tid >> 1, h = tid & 1;
    const int i = c >> 3, sh = 4 * (c & 7);
    uint32_t out[8];
#pragma unroll
    for (int wd = 0; wd < 8; ++wd) {
        uint32_t v = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int kr = 64 * h + 8 * wd + 2 * b;
            const uint32_t lo = (tile[kr][i] >> sh) & 0xFu, hi = (tile[kr + 1][i] >> sh) & 0xFu;
            v |= (lo | (hi << 4)) << (8 * b);
        }
        out[wd] = v;
    }
    uint8_t* dst = packed + (i0 * 8 + c) * (k / 2) + k0 / 2 + 32 * h;
    stg16_nt(dst, make_uint4(out[0], out[1], out[2], out[3]));
    stg16_nt(dst + 16, make_uint4(out[4], out[5], out[6], out[7]));
}

// 16 codes (16 bytes) -> 8 bytes per thread: (c + 8) mod 16 = (c & 15) ^ 8, pairs merged by shifts
__global__ __launch_bounds__(kBlock) void pack_nibbles_vec_k(const int8_t* codes, uint8_t* packed, int64_t nvec) {
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= nvec) return;
    const uint4 in = ldg16_nt(codes + v * 16);
    const uint32_t ws[4] = {in.x, in.y, in.z, in.w};
    uint32_t half[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t t = (ws[j] & 0x0F0F0F0Fu) ^ 0x08080808u;   // bytes t0 t1 t2 t3, each below 16
        const uint32_t u = t | (t >> 4);                           // byte 0 = t0 | t1 << 4, byte 2 = t2 | t3 << 4
        half[j] = (u & 0xFFu) | ((u >> 8) & 0xFF00u);
    }
    stg8_nt(packed + v * 8, half[0] | (half[1] << 16), half[2] | (half[3] << 16));
}

// 64 rows x 32 bytes (64 values of k) per block: 16-byte loads, then every k-row of the tile is written as 64
// consecutive int32 codes.  k % 64 == 0, n % 64 == 0.
__global__ __launch_bounds__(kBlock) void nibbles_to_codes_tile_k(const uint8_t* packed, int32_t* codes, int64_t k, int64_t n) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[64][48];  // 32 bytes used; rows 12 words apart
    const int tid = threadIdx.x;
    const int64_t n0 = (int64_t)blockIdx.x * 64, k0 = (int64_t)blockIdx.y * 64;
    if (tid < 128) {
        const int r = tid >> 1, h = tid & 1;
        *reinterpret_cast<uint4*>(&tile[r][16 * h]) = ldg16_nt(packed + (n0 + r) * (k / 2) + k0 / 2 + 16 * h);
    }
    __syncthreads();
    const int c = tid & 63, kq = tid >> 6;
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
        const int kr = 16 * kq + kk;
        const uint32_t b = tile[c][kr >> 1];
        const int32_t u = (kr & 1) ? (int32_t)(b >> 4) : (int32_t)(b & 0xFu);
        __builtin_nontemporal_store(u - 8, codes + (k0 + kr) * n + n0 + c);
    }
}

}  // namespace amct

using namespace amct;

extern "C" int amct_quant_int4_group_pack(const void* w, uint8_t* packed, void* scales16, int scale_dtype,
                                          float* scales32, uint8_t* zeros, int32_t* bad_count, const void* col_scale,
                                          int col_mode, int64_t rows, int64_t cols, int group, int symmetric, int dtype,
                                          amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || group <= 0) return AMCT_E_BADARG;
    if (scales16 && scale_dtype != AMCT_F16 && scale_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (col_mode < 0 || col_mode > 2) return AMCT_E_BADARG;
    if (rows != 0 && (!w || !packed || (col_mode != AMCT_COL_NONE && !col_scale))) return AMCT_E_BADARG;   // rows == 0 reads nothing
    if (cols % group != 0 || group % 32 != 0) return AMCT_E_ALIGN;
    if (rows == 0) return AMCT_OK;
    PackArgs a{};
    a.w = w; a.packed = packed; a.scales16 = scales16; a.scales32 = scales32; a.zeros = zeros; a.bad = bad_count;
    a.col = col_scale; a.col_mode = col_mode; a.seg_len = group; a.segs_per_row = (int)(cols / group);
    a.nseg = rows * a.segs_per_row; a.scale_dtype = scale_dtype; a.symmetric = symmetric;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case AMCT_F32: return run_pack<AMCT_F32>(a, rows, cols, st);
        case AMCT_F16: return run_pack<AMCT_F16>(a, rows, cols, st);
        case AMCT_BF16: return run_pack<AMCT_BF16>(a, rows, cols, st);
        default: return AMCT_E_BADARG;
    }
}

extern "C" int amct_pack_int4_words(const int32_t* codes, int32_t* words, int64_t k, int64_t n, amct_stream_t stream) {
    if (k < 0 || n < 0 || (k * n != 0 && (!codes || !words))) return AMCT_E_BADARG;
    if (n % 8 != 0 || !aligned16(codes)) return AMCT_E_ALIGN;
    const int64_t nwords = k * (n / 8);
    if (nwords == 0) return AMCT_OK;
    hipLaunchKernelGGL(pack_words_k, dim3((unsigned)((nwords + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, codes, words, nwords);
    return hip_status();
}

extern "C" int amct_words_to_nibbles_nk(const int32_t* words, uint8_t* packed, int64_t k, int64_t n, amct_stream_t stream) {
    if (k < 0 || n < 0 || (k * n != 0 && (!words || !packed))) return AMCT_E_BADARG;
    if (n % 8 != 0 || k % 2 != 0) return AMCT_E_ALIGN;
    const int64_t total = (k / 2) * (n / 8);
    if (total == 0) return AMCT_OK;
    if (k % 128 == 0 && (n / 8) % 16 == 0 && aligned16(packed) && k / 128 <= 65535) {
        hipLaunchKernelGGL(words_to_nibbles_tile_k, dim3((unsigned)(n / 128), (unsigned)(k / 128)), dim3(kBlock), 0,
                           (hipStream_t)stream, words, packed, k, n / 8);
        return hip_status();
    }
    hipLaunchKernelGGL(words_to_nibbles_k, dim3((unsigned)((total + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, words, packed, k, n / 8);
    return hip_status();
}

extern "C" int amct_pack_nibbles_nk(const int8_t* codes, uint8_t* packed, int64_t rows, int64_t cols, amct_stream_t stream) {
    if (rows < 0 || cols < 0 || (rows * cols != 0 && (!codes || !packed))) return AMCT_E_BADARG;
    if (cols % 2 != 0) return AMCT_E_ALIGN;
    const int64_t nbytes = rows * (cols / 2);
    if (nbytes == 0) return AMCT_OK;
    if (nbytes % 8 == 0 && aligned16(codes) && (reinterpret_cast<uintptr_t>(packed) & 7u) == 0) {
        const int64_t nvec = nbytes / 8;
        hipLaunchKernelGGL(pack_nibbles_vec_k, dim3((unsigned)((nvec + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                           (hipStream_t)stream, codes, packed, nvec);
        return hip_status();
    }
    hipLaunchKernelGGL(pack_nibbles_k, dim3((unsigned)((nbytes + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, codes, packed, nbytes);
    return hip_status();
}

extern "C" int amct_nibbles_nk_to_codes_kn(const uint8_t* packed, int32_t* codes, int64_t k, int64_t n, amct_stream_t stream) {
    if (k < 0 || n < 0 || (k * n != 0 && (!packed || !codes))) return AMCT_E_BADARG;
    if (k % 2 != 0) return AMCT_E_ALIGN;
    if (k * n == 0) return AMCT_OK;
    if (k % 64 == 0 && n % 64 == 0 && aligned16(packed) && k / 64 <= 65535) {
        hipLaunchKernelGGL(nibbles_to_codes_tile_k, dim3((unsigned)(n / 64), (unsigned)(k / 64)), dim3(kBlock), 0,
                           (hipStream_t)stream, packed, codes, k, n);
        return hip_status();
    }
    hipLaunchKernelGGL(nibbles_to_codes_kn_k, dim3((unsigned)((k * n + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, packed, codes, k, n);
    return hip_status();
}
