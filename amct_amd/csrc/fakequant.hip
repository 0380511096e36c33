// K1: integer (fake-)quantisation of weights.
//   fused path   : one read of w -> min/max per segment (row or group) in registers ->
//                  scale/offset -> quantise the cached registers -> write dq / codes.
//   params path  : flat elementwise kernel for given factors.
//   general path : scalar kernel for ragged / unaligned shapes (zero-pad semantics).
// Reference behaviour: amct_pytorch/quantize_op/utils.py:75-136,
// amct_pytorch/utils/quant_util.py:56-93,162-188, amct_pytorch/algorithm/awq.py:129-170.
#include <type_traits>

#include "amct_common.h"

namespace amct {

struct FqArgs {
    const void* w;
    void* dq;
    void* codes;
    float* scale;
    int32_t* offset;
    int32_t* bad;
    const void* col;
    const float* pscale;
    const int32_t* poffset;
    int64_t nseg;
    int64_t rows;
    int64_t cols;
    int seg_len;        // elements per segment
    int segs_per_row;
    int group;          // as given by the caller (params path indexing)
    int codes_kind;
    int col_mode;
    int bits;
    int symmetric;
    int scope_rule;
    int via_src;
    int stage;          // params path only: AMCT_STAGE_*
    float qmin, qmax;
};

template <int DT> AMCT_DEV void apply_col_pre(float* x, const float* c, int mode) {
    constexpr int VEC = Tr<DT>::VEC;
    if (mode == AMCT_COL_DIV) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[j] = round_to<DT>(x[j] / c[j]);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[j] = round_to<DT>(x[j] * c[j]);
    }
}

// Params path: the whole quantiser or one of the two halves the AWQ search calls separately.
//   FULL    : q = clamp(rne(x/s + z)); d = (q - z) * s
//   SCALE   : d = x/s + z                      (do_quant, amct_pytorch/algorithm/awq.py:129-149)
//   DEQUANT : d = (x - z [in x's dtype]) * s   (do_dequant, amct_pytorch/algorithm/awq.py:152-170)
//   COL     : d = x after the column scaling   (amct_pytorch/utils/quant_util.py:96-111,143-159)
template <int DT, bool VIA_SRC>
AMCT_DEV void staged_elem(int stage, float x, float s, float z, bool asym, float qmin, float qmax, float& q, float& d) {
    if (stage == AMCT_STAGE_SCALE) {
        float t = x / s;
        if (asym) t = t + z;
        q = 0.f;
        d = t;
    } else if (stage == AMCT_STAGE_DEQUANT) {
        const float t = asym ? round_to<DT>(x - z) : x;
        q = 0.f;
        d = t * s;
    } else if (stage == AMCT_STAGE_COL) {
        q = 0.f;
        d = x;                                  // the column scaling has already been applied
    } else {
        q = quant_elem<DT, VIA_SRC>(x, s, z, asym, qmin, qmax);
        d = dequant_elem(q, s, z, asym);
    }
}

template <int DT> AMCT_DEV void store_codes(void* codes, int kind, int64_t e0, const float* q) {
    constexpr int VEC = Tr<DT>::VEC;
    if (kind == AMCT_CODES_I8) {
        uint32_t pk[VEC / 4];
#pragma unroll
        for (int j = 0; j < VEC / 4; ++j) {
            pk[j] = ((uint32_t)(int)q[4 * j] & 0xFFu) | (((uint32_t)(int)q[4 * j + 1] & 0xFFu) << 8) |
                    (((uint32_t)(int)q[4 * j + 2] & 0xFFu) << 16) | (((uint32_t)(int)q[4 * j + 3] & 0xFFu) << 24);
        }
        uint32_t* p = reinterpret_cast<uint32_t*>(reinterpret_cast<int8_t*>(codes) + e0);
        if constexpr (VEC == 4) p[0] = pk[0];
        else *reinterpret_cast<uint2*>(p) = make_uint2(pk[0], pk[1]);
    } else if (kind == AMCT_CODES_I32) {
        int32_t* p = reinterpret_cast<int32_t*>(codes) + e0;
#pragma unroll
        for (int j = 0; j < VEC / 4; ++j)
            *reinterpret_cast<int4*>(p + 4 * j) = make_int4((int)q[4 * j], (int)q[4 * j + 1], (int)q[4 * j + 2], (int)q[4 * j + 3]);
    }
}

// ---------------------------------------------------------------------------
// fused kernel.  A team of T lanes owns U consecutive segments; every lane caches NV 16-byte
// vectors of each, all loaded up front (unconditional, streaming; indices are clamped and a
// duplicated vector cannot change a min/max).  With U == 4 the factors of segment u are computed by
// the lanes with lt % 4 == u and shared by DPP inside each quad.
// ---------------------------------------------------------------------------
template <int DT, int T, int NV, int U, bool VIA_SRC, bool COL>
__global__ __launch_bounds__(kBlock) void fq_fused(FqArgs a) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    constexpr int TEAMS = kBlock / T;
    const int tid = threadIdx.x;
    const int team = tid / T, lt = tid % T;
    const int S = a.seg_len / VEC;
    const bool asym = !a.symmetric;
    const int64_t seg0 = ((int64_t)blockIdx.x * TEAMS + team) * U;

    float x[U][NV][VEC];
    int64_t segc[U];
    {
        uint4 raw[U][NV];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            segc[u] = (seg0 + u < a.nseg) ? seg0 + u : a.nseg - 1;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = (i * T + lt < S) ? i * T + lt : S - 1;
                raw[u][i] = ldg16_nt(reinterpret_cast<const char*>(a.w) + (segc[u] * a.seg_len + (int64_t)v * VEC) * BYTES);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < NV; ++i) unpack16<DT>(raw[u][i], x[u][i]);
    }
    if constexpr (COL) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t c0 = (segc[u] % a.segs_per_row) * (int64_t)a.seg_len;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = (i * T + lt < S) ? i * T + lt : S - 1;
                float c[VEC];
                unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.col) + (c0 + (int64_t)v * VEC) * BYTES), c);
                apply_col_pre<DT>(x[u][i], c, a.col_mode);
            }
        }
    }

    float mx[U], mn[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        mx[u] = x[u][0][0];
        mn[u] = x[u][0][0];
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                mx[u] = fmax_nan(mx[u], x[u][i][j]);
                mn[u] = fmin_nan(mn[u], x[u][i][j]);
            }
    }
    if constexpr (U == 4) {
        // reduced further below by a scatter-reduction
    } else if constexpr (T <= kWave) {
#pragma unroll
        for (int u = 0; u < U; ++u) team_minmax<T>(mn[u], mx[u]);
    } else {
        __shared__ float sm[2][kBlock / kWave][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            team_minmax<kWave>(mn[u], mx[u]);
            if ((tid & (kWave - 1)) == 0) {
                sm[0][tid / kWave][u] = mn[u];
                sm[1][tid / kWave][u] = mx[u];
            }
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int wv = 0; wv < kBlock / kWave; ++wv) {
                mn[u] = fmin_nan(mn[u], sm[0][wv][u]);
                mx[u] = fmax_nan(mx[u], sm[1][wv][u]);
            }
        }
    }

    Divisor dv[U];
    float z[U];
    bool fast;
    if constexpr (U == 4) {
        const int my = seg4_of_lane(lt);
        float mx_my, mn_my;
        team_minmax_scatter4<T>(mn, mx, lt, mn_my, mx_my);
        const Factors f = make_factors<DT>(mx_my, mn_my, a.bits, a.symmetric != 0, a.scope_rule);
        const Divisor dmy = divisor_of(f);
        const uint32_t big = max(__float_as_uint(mx_my) & 0x7FFFFFFFu, __float_as_uint(mn_my) & 0x7FFFFFFFu);
        fast = wave_all(dmy.fast && big < 0x5D800000u);
        if (lt < 4 && seg0 + my < a.nseg) {
            a.scale[seg0 + my] = f.s;
            if (a.offset) a.offset[seg0 + my] = (int32_t)f.z;
            if (f.bad && a.bad) atomicAdd(a.bad, 1);
        }
        dv[0].s = quad_bcast<0>(f.s); dv[0].y = quad_bcast<0>(dmy.y); z[0] = quad_bcast<0>(f.z);
        dv[1].s = quad_bcast<2>(f.s); dv[1].y = quad_bcast<2>(dmy.y); z[1] = quad_bcast<2>(f.z);
        dv[2].s = quad_bcast<1>(f.s); dv[2].y = quad_bcast<1>(dmy.y); z[2] = quad_bcast<1>(f.z);
        dv[3].s = quad_bcast<3>(f.s); dv[3].y = quad_bcast<3>(dmy.y); z[3] = quad_bcast<3>(f.z);
    } else {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const Factors f = make_factors<DT>(mx[u], mn[u], a.bits, a.symmetric != 0, a.scope_rule);
            dv[u] = divisor_of(f);
            z[u] = f.z;
            const uint32_t big = max(__float_as_uint(mx[u]) & 0x7FFFFFFFu, __float_as_uint(mn[u]) & 0x7FFFFFFFu);
            ok = ok && dv[u].fast && big < 0x5D800000u;
            if (lt == 0 && seg0 + u < a.nseg) {
                a.scale[seg0 + u] = f.s;
                if (a.offset) a.offset[seg0 + u] = (int32_t)f.z;
                if (f.bad && a.bad) atomicAdd(a.bad, 1);
            }
        }
        fast = wave_all(ok);
    }

    auto emit = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool ok = seg0 + u < a.nseg;
            const int64_t c0 = (COL && a.col_mode == AMCT_COL_MUL_THEN_DIV) ? (segc[u] % a.segs_per_row) * (int64_t)a.seg_len : 0;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = i * T + lt;
                float q[VEC], d[VEC];
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    q[j] = quant_elem<DT, VIA_SRC, FAST>(x[u][i][j], dv[u], z[u], asym, a.qmin, a.qmax);
                    d[j] = dequant_elem(q[j], dv[u].s, z[u], asym);
                }
                if (ok && v < S) {
                    const int64_t e0 = (seg0 + u) * a.seg_len + (int64_t)v * VEC;
                    if (a.codes) store_codes<DT>(a.codes, a.codes_kind, e0, q);
                    if (a.dq) {
                        if constexpr (COL) {
                            if (a.col_mode == AMCT_COL_MUL_THEN_DIV) {
                                float c[VEC];
                                unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.col) + (c0 + (int64_t)v * VEC) * BYTES), c);
#pragma unroll
                                for (int j = 0; j < VEC; ++j) d[j] = round_to<DT>(d[j]) / c[j];
                            }
                        }
                        stg16_nt(reinterpret_cast<char*>(a.dq) + e0 * BYTES, pack16<DT>(d));
                    }
                }
            }
        }
    };
    if (fast) emit(std::true_type{});
    else emit(std::false_type{});
}

// ---------------------------------------------------------------------------
// params kernel: factors given; flat over 16-byte vectors (cols % VEC == 0).
// ---------------------------------------------------------------------------
template <int DT, bool VIA_SRC>
__global__ __launch_bounds__(kBlock) void fq_params(FqArgs a, int64_t nvec) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    const bool asym = a.poffset != nullptr;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride) {
        const int64_t e0 = v * VEC;
        const int64_t row = e0 / a.cols;
        const int64_t c0 = e0 - row * a.cols;
        int64_t pi = 0;
        if (a.group > 0) pi = row * a.segs_per_row + c0 / a.group;
        else if (a.group == 0) pi = row;
        const float s = a.pscale[pi];
        const float z = asym ? (float)a.poffset[pi] : 0.f;
        float x[VEC], q[VEC], d[VEC];
        unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.w) + e0 * BYTES), x);
        float c[VEC];
        if (a.col_mode != AMCT_COL_NONE) {
            unpack16<DT>(ldg16(reinterpret_cast<const char*>(a.col) + c0 * BYTES), c);
            apply_col_pre<DT>(x, c, a.col_mode);
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) staged_elem<DT, VIA_SRC>(a.stage, x[j], s, z, asym, a.qmin, a.qmax, q[j], d[j]);
        if (a.codes) store_codes<DT>(a.codes, a.codes_kind, e0, q);
        if (a.dq) {
            if (a.col_mode == AMCT_COL_MUL_THEN_DIV) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) d[j] = round_to<DT>(d[j]) / c[j];
            }
            stg16(reinterpret_cast<char*>(a.dq) + e0 * BYTES, pack16<DT>(d));
        }
    }
}

// ---------------------------------------------------------------------------
// general kernel: one block per row, scalar accesses, any cols / group / alignment.
// A ragged last group is zero-padded: the zeros take part in min/max
// (amct_pytorch/utils/quant_util.py:23-36).  With GIVEN factors the reduction is skipped.
// ---------------------------------------------------------------------------
template <int DT, bool VIA_SRC, bool GIVEN>
__global__ __launch_bounds__(kBlock) void fq_general(FqArgs a) {
    __shared__ float sm[2][kBlock / kWave];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t L = a.seg_len;
    const float inf = __builtin_huge_valf();
    for (int sg = 0; sg < a.segs_per_row; ++sg) {
        const int64_t c_begin = sg * L;
        const int64_t c_end = (c_begin + L < a.cols) ? c_begin + L : a.cols;
        float s, z;
        bool asym;
        if constexpr (GIVEN) {
            int64_t pi = 0;
            if (a.group > 0) pi = row * a.segs_per_row + sg;
            else if (a.group == 0) pi = row;
            s = a.pscale[pi];
            asym = a.poffset != nullptr;
            z = asym ? (float)a.poffset[pi] : 0.f;
        } else {
            asym = !a.symmetric;
            float mx = -inf, mn = inf;
            for (int64_t c = c_begin + tid; c < c_end; c += kBlock) {
                float x = load_scalar<DT>(a.w, row * a.cols + c);
                if (a.col_mode != AMCT_COL_NONE) {
                    const float cs = load_scalar<DT>(a.col, c);
                    x = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x / cs : x * cs);
                }
                mx = fmax_nan(mx, x);
                mn = fmin_nan(mn, x);
            }
            if (c_end - c_begin < L && tid == 0) {      // zero padding of the ragged group
                mx = fmax_nan(mx, 0.f);
                mn = fmin_nan(mn, 0.f);
            }
            team_minmax<kWave>(mn, mx);
            __syncthreads();                            // protect sm from the previous segment's readers
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
            const Factors f = make_factors<DT>(mx, mn, a.bits, a.symmetric != 0, a.scope_rule);
            s = f.s;
            z = f.z;
            if (tid == 0) {
                const int64_t pi = row * a.segs_per_row + sg;
                a.scale[pi] = f.s;
                if (a.offset) a.offset[pi] = (int32_t)f.z;
                if (f.bad && a.bad) atomicAdd(a.bad, 1);
            }
        }
        for (int64_t c = c_begin + tid; c < c_end; c += kBlock) {
            const int64_t e = row * a.cols + c;
            float x = load_scalar<DT>(a.w, e);
            float cs = 1.f;
            if (a.col_mode != AMCT_COL_NONE) {
                cs = load_scalar<DT>(a.col, c);
                x = round_to<DT>(a.col_mode == AMCT_COL_DIV ? x / cs : x * cs);
            }
            float q, d;
            if constexpr (GIVEN) {
                staged_elem<DT, VIA_SRC>(a.stage, x, s, z, asym, a.qmin, a.qmax, q, d);
            } else {
                q = quant_elem<DT, VIA_SRC>(x, s, z, asym, a.qmin, a.qmax);
                d = dequant_elem(q, s, z, asym);
            }
            if (a.codes) {
                if (a.codes_kind == AMCT_CODES_I8) reinterpret_cast<int8_t*>(a.codes)[e] = (int8_t)(int)q;
                else if (a.codes_kind == AMCT_CODES_I32) reinterpret_cast<int32_t*>(a.codes)[e] = (int)q;
            }
            if (a.dq) {
                if (a.col_mode == AMCT_COL_MUL_THEN_DIV) d = round_to<DT>(d) / cs;
                store_scalar<DT>(a.dq, e, d);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// min/max only (A1), groups of T vectors (cols % group == 0, so the tensor is one flat array of groups): a team of T
// lanes owns 4 consecutive groups, 4 x 16 bytes per lane in flight, extrema by lane exchange.  (The general kernel
// below walks the groups of a row one after another with 16 of its 256 threads busy for a group of 128 bf16 values:
// 189 us for W[14336,4096], against 18 us for the per-row case.)
// ---------------------------------------------------------------------------
template <int DT, int T>
__global__ __launch_bounds__(kBlock) void minmax_groups(const void* w, float* mn_out, float* mx_out, int64_t nseg) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int U = 4;
    const int tid = threadIdx.x;
    const int lt = tid % T;
    const int64_t seg0 = ((int64_t)blockIdx.x * (kBlock / T) + tid / T) * U;
    uint4 raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t sg = seg0 + u < nseg ? seg0 + u : nseg - 1;   // clamped: loads are unconditional
        raw[u] = ldg16_nt(reinterpret_cast<const char*>(w) + (sg * T + lt) * 16);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float x[VEC];
        unpack16<DT>(raw[u], x);
        float mx = x[0], mn = x[0];
#pragma unroll
        for (int j = 1; j < VEC; ++j) {
            mx = fmax_nan(mx, x[j]);
            mn = fmin_nan(mn, x[j]);
        }
        team_minmax<T>(mn, mx);
        if (lt == 0 && seg0 + u < nseg) {
            mn_out[seg0 + u] = mn;
            mx_out[seg0 + u] = mx;
        }
    }
}

// ---------------------------------------------------------------------------
// min/max only (A1) -- general block-per-row kernel with vector fast path
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kBlock) void minmax_rows(const void* w, float* mn_out, float* mx_out, int64_t cols,
                                                      int seg_len, int segs_per_row, int vec_ok) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    __shared__ float sm[2][kBlock / kWave];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const float inf = __builtin_huge_valf();
    for (int sg = 0; sg < segs_per_row; ++sg) {
        const int64_t c_begin = (int64_t)sg * seg_len;
        const int64_t c_end = (c_begin + seg_len < cols) ? c_begin + seg_len : cols;
        float mx = -inf, mn = inf;
        if (vec_ok) {
            const int64_t nv = (c_end - c_begin) / VEC;
            const char* base = reinterpret_cast<const char*>(w) + (row * cols + c_begin) * BYTES;
            for (int64_t v = tid; v < nv; v += kBlock) {
                float x[VEC];
                unpack16<DT>(ldg16(base + v * 16), x);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    mx = fmax_nan(mx, x[j]);
                    mn = fmin_nan(mn, x[j]);
                }
            }
        } else {
            for (int64_t c = c_begin + tid; c < c_end; c += kBlock) {
                const float x = load_scalar<DT>(w, row * cols + c);
                mx = fmax_nan(mx, x);
                mn = fmin_nan(mn, x);
            }
        }
        if (c_end - c_begin < seg_len && tid == 0) {
            mx = fmax_nan(mx, 0.f);
            mn = fmin_nan(mn, 0.f);
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
        if (tid == 0) {
            mn_out[row * segs_per_row + sg] = mn;
            mx_out[row * segs_per_row + sg] = mx;
        }
    }
}

template <int DT>
__global__ __launch_bounds__(kBlock) void scale_offset_k(const void* mx, const void* mn, float* scale, int32_t* offset,
                                                         int32_t* bad, int64_t n, int bits, int symmetric, int scope_rule) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const Factors f = make_factors<DT>(load_scalar<DT>(mx, i), load_scalar<DT>(mn, i), bits, symmetric != 0, scope_rule);
    scale[i] = f.s;
    if (offset && !symmetric) offset[i] = (int32_t)f.z;
    if (f.bad && bad) atomicAdd(bad, 1);
}

// ---------------------------------------------------------------------------
// host-side dispatch
// ---------------------------------------------------------------------------
template <int DT, int T, int NV, int U>
static void launch_fused(const FqArgs& a, hipStream_t st) {
    constexpr int TEAMS = kBlock / T;
    const int64_t per_block = (int64_t)TEAMS * U;
    const int64_t nb = (a.nseg + per_block - 1) / per_block;
    const dim3 grid((unsigned)nb), block(kBlock);
    const bool via = a.via_src && DT != AMCT_F32;
    const bool col = a.col_mode != AMCT_COL_NONE;
    if (via && col) hipLaunchKernelGGL((fq_fused<DT, T, NV, U, true, true>), grid, block, 0, st, a);
    else if (via) hipLaunchKernelGGL((fq_fused<DT, T, NV, U, true, false>), grid, block, 0, st, a);
    else if (col) hipLaunchKernelGGL((fq_fused<DT, T, NV, U, false, true>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((fq_fused<DT, T, NV, U, false, false>), grid, block, 0, st, a);
}

template <int DT>
static bool dispatch_fused(const FqArgs& a, hipStream_t st) {
    constexpr int VEC = Tr<DT>::VEC;
    const int S = a.seg_len / VEC;
    if (S <= 4) launch_fused<DT, 4, 1, 4>(a, st);
    else if (S <= 8) launch_fused<DT, 8, 1, 4>(a, st);
    else if (S <= 16) launch_fused<DT, 16, 1, 4>(a, st);
    else if (S <= 32) launch_fused<DT, 32, 1, 4>(a, st);
    else if (S <= 64) launch_fused<DT, 64, 1, 4>(a, st);
    else if (S <= 128) launch_fused<DT, 64, 2, 2>(a, st);
    else if (S <= 256) launch_fused<DT, 64, 4, 1>(a, st);
    else if (S <= 512) launch_fused<DT, 64, 8, 1>(a, st);
    else if (S <= 1024) launch_fused<DT, 256, 4, 1>(a, st);
    else if (S <= 2048) launch_fused<DT, 256, 8, 1>(a, st);
    else if (S <= 4096) launch_fused<DT, 256, 16, 1>(a, st);        // rows up to 16384 fp32 / 32768 16-bit elements (64 / 128 values per lane)
    else return false;
    return true;
}

template <int DT>
static int run_fused(FqArgs a, hipStream_t st) {
    constexpr int VEC = Tr<DT>::VEC;
    const bool vec_ok = (a.cols % VEC == 0) && (a.seg_len % VEC == 0) && (a.cols % a.seg_len == 0) && aligned16(a.w) &&
                        (!a.dq || aligned16(a.dq)) && (!a.codes || aligned16(a.codes)) &&
                        (a.col_mode == AMCT_COL_NONE || aligned16(a.col));
    if (vec_ok && dispatch_fused<DT>(a, st)) return hip_status();
    if (a.rows > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    if (a.via_src && DT != AMCT_F32)
        hipLaunchKernelGGL((fq_general<DT, true, false>), dim3((unsigned)a.rows), dim3(kBlock), 0, st, a);
    else
        hipLaunchKernelGGL((fq_general<DT, false, false>), dim3((unsigned)a.rows), dim3(kBlock), 0, st, a);
    return hip_status();
}

template <int DT>
static int run_params(FqArgs a, hipStream_t st) {
    constexpr int VEC = Tr<DT>::VEC;
    const bool vec_ok = (a.cols % VEC == 0) && (a.group <= 0 || a.group % VEC == 0) && aligned16(a.w) &&
                        (!a.dq || aligned16(a.dq)) && (!a.codes || aligned16(a.codes)) &&
                        (a.col_mode == AMCT_COL_NONE || aligned16(a.col));
    const bool via = a.via_src && DT != AMCT_F32;
    if (vec_ok) {
        const int64_t nvec = a.rows * a.cols / VEC;
        int64_t nb = (nvec + kBlock - 1) / kBlock;
        if (nb > 65536) nb = 65536;
        if (via) hipLaunchKernelGGL((fq_params<DT, true>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, nvec);
        else hipLaunchKernelGGL((fq_params<DT, false>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, nvec);
        return hip_status();
    }
    if (a.rows > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    if (via) hipLaunchKernelGGL((fq_general<DT, true, true>), dim3((unsigned)a.rows), dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((fq_general<DT, false, true>), dim3((unsigned)a.rows), dim3(kBlock), 0, st, a);
    return hip_status();
}

static bool fill_geometry(FqArgs& a, int64_t rows, int64_t cols, int group) {
    a.rows = rows;
    a.cols = cols;
    a.group = group;
    if (group > 0) {
        a.seg_len = group;
        a.segs_per_row = (int)((cols + group - 1) / group);
    } else {
        if (cols > 0x7FFFFFFF) return false;
        a.seg_len = (int)cols;
        a.segs_per_row = 1;
    }
    a.nseg = rows * a.segs_per_row;
    return true;
}

}  // namespace amct

using namespace amct;

extern "C" int amct_minmax(const void* w, float* mn, float* mx, int64_t rows, int64_t cols, int group, int dtype,
                           amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || group < 0) return AMCT_E_BADARG;
    if (rows == 0) return AMCT_OK;                                // nothing is read: null pointers are fine
    if (!w || !mn || !mx) return AMCT_E_BADARG;
    if (rows > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    const int seg_len = group > 0 ? group : (int)cols;
    const int spr = group > 0 ? (int)((cols + group - 1) / group) : 1;
    hipStream_t st = (hipStream_t)stream;
#define AMCT_MMG(DT, T)                                                                                          \
    case T:                                                                                                      \
        hipLaunchKernelGGL((minmax_groups<DT, T>), dim3(nbg), dim3(kBlock), 0, st, w, mn, mx, nseg);              \
        return hip_status();
#define AMCT_MM(DT)                                                                                              \
    {                                                                                                            \
        const int vec_ok = aligned16(w) && cols % Tr<DT>::VEC == 0 && seg_len % Tr<DT>::VEC == 0;               \
        if (vec_ok && group > 0 && cols % group == 0) {                                                          \
            const int64_t nseg = rows * spr;                                                                     \
            const int t = seg_len / Tr<DT>::VEC;                                                                 \
            const int64_t per_block = (int64_t)(kBlock / (t > 0 && t <= 64 ? t : 64)) * 4;                        \
            const int64_t nb64 = (nseg + per_block - 1) / per_block;                                             \
            if (nb64 <= 0x7FFFFFFF) {                                                                            \
                const unsigned nbg = (unsigned)nb64;                                                             \
                switch (t) {                                                                                     \
                    AMCT_MMG(DT, 1) AMCT_MMG(DT, 2) AMCT_MMG(DT, 4) AMCT_MMG(DT, 8) AMCT_MMG(DT, 16) AMCT_MMG(DT, 32)  \
                    AMCT_MMG(DT, 64)                                                                             \
                    default: break;                                                                              \
                }                                                                                                \
            }                                                                                                    \
        }                                                                                                        \
        hipLaunchKernelGGL((minmax_rows<DT>), dim3((unsigned)rows), dim3(kBlock), 0, st, w, mn, mx, cols, seg_len, \
                           spr, vec_ok);                                                                         \
    }
    switch (dtype) {
        case AMCT_F32: AMCT_MM(AMCT_F32) break;
        case AMCT_F16: AMCT_MM(AMCT_F16) break;
        case AMCT_BF16: AMCT_MM(AMCT_BF16) break;
        default: return AMCT_E_BADARG;
    }
#undef AMCT_MM
#undef AMCT_MMG
    return hip_status();
}

extern "C" int amct_scale_offset(const void* mx, const void* mn, float* scale, int32_t* offset, int32_t* bad_count,
                                 int64_t n, int bits, int symmetric, int scope_rule, int in_dtype,
                                 amct_stream_t stream) {
    if (n < 0 || (bits != 4 && bits != 8)) return AMCT_E_BADARG;
    if (n == 0) return AMCT_OK;
    if (!mx || !mn || !scale) return AMCT_E_BADARG;
    if (!symmetric && !offset) return AMCT_E_BADARG;
    const unsigned nb = (unsigned)((n + kBlock - 1) / kBlock);
    hipStream_t st = (hipStream_t)stream;
    switch (in_dtype) {
        case AMCT_F32:
            hipLaunchKernelGGL((scale_offset_k<AMCT_F32>), dim3(nb), dim3(kBlock), 0, st, mx, mn, scale, offset, bad_count, n, bits, symmetric, scope_rule);
            break;
        case AMCT_F16:
            hipLaunchKernelGGL((scale_offset_k<AMCT_F16>), dim3(nb), dim3(kBlock), 0, st, mx, mn, scale, offset, bad_count, n, bits, symmetric, scope_rule);
            break;
        case AMCT_BF16:
            hipLaunchKernelGGL((scale_offset_k<AMCT_BF16>), dim3(nb), dim3(kBlock), 0, st, mx, mn, scale, offset, bad_count, n, bits, symmetric, scope_rule);
            break;
        default: return AMCT_E_BADARG;
    }
    return hip_status();
}

extern "C" int amct_quant_with_params(const void* w, const float* scale, const int32_t* offset, void* dq, void* codes,
                                      int codes_kind, const void* col_scale, int col_mode, int64_t rows, int64_t cols,
                                      int group, int qmin, int qmax, int round_via_src_dtype, int stage, int dtype,
                                      amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || group < -1 || qmin > qmax) return AMCT_E_BADARG;
    if (stage < AMCT_STAGE_FULL || stage > AMCT_STAGE_COL) return AMCT_E_BADARG;
    if (codes && codes_kind != AMCT_CODES_I8 && codes_kind != AMCT_CODES_I32) return AMCT_E_BADARG;
    if (col_mode < 0 || col_mode > 3) return AMCT_E_BADARG;
    if (rows == 0) return AMCT_OK;
    if (!w || !scale) return AMCT_E_BADARG;
    if (stage != AMCT_STAGE_FULL && (codes || !dq)) return AMCT_E_BADARG;
    if (col_mode != AMCT_COL_NONE && !col_scale) return AMCT_E_BADARG;
    FqArgs a{};
    if (!fill_geometry(a, rows, cols, group)) return AMCT_E_UNSUPPORTED;
    a.w = w; a.dq = dq; a.codes = codes; a.codes_kind = codes ? codes_kind : AMCT_CODES_NONE;
    a.pscale = scale; a.poffset = offset; a.col = col_scale; a.col_mode = col_mode;
    a.qmin = (float)qmin; a.qmax = (float)qmax; a.via_src = round_via_src_dtype; a.stage = stage;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case AMCT_F32: return run_params<AMCT_F32>(a, st);
        case AMCT_F16: return run_params<AMCT_F16>(a, st);
        case AMCT_BF16: return run_params<AMCT_BF16>(a, st);
        default: return AMCT_E_BADARG;
    }
}

extern "C" int amct_fakequant_int(const void* w, void* dq, void* codes, int codes_kind, float* scale, int32_t* offset,
                                  int32_t* bad_count, const void* col_scale, int col_mode, int64_t rows, int64_t cols,
                                  int group, int bits, int symmetric, int scope_rule, int qmin, int qmax,
                                  int round_via_src_dtype, int dtype, amct_stream_t stream) {
    if (rows < 0 || cols <= 0 || group < 0 || qmin > qmax) return AMCT_E_BADARG;
    if (bits != 4 && bits != 8) return AMCT_E_BADARG;
    if (codes && codes_kind != AMCT_CODES_I8 && codes_kind != AMCT_CODES_I32) return AMCT_E_BADARG;
    if (col_mode < 0 || col_mode > 3) return AMCT_E_BADARG;
    if (scope_rule != AMCT_SCOPE_AMCT && scope_rule != AMCT_SCOPE_ABSMAX) return AMCT_E_BADARG;
    if (rows == 0) return AMCT_OK;
    if (!w || !scale) return AMCT_E_BADARG;
    if (!symmetric && !offset) return AMCT_E_BADARG;
    if (col_mode != AMCT_COL_NONE && !col_scale) return AMCT_E_BADARG;
    FqArgs a{};
    if (!fill_geometry(a, rows, cols, group)) return AMCT_E_UNSUPPORTED;
    a.w = w; a.dq = dq; a.codes = codes; a.codes_kind = codes ? codes_kind : AMCT_CODES_NONE;
    a.scale = scale; a.offset = symmetric ? nullptr : offset; a.bad = bad_count;
    a.col = col_scale; a.col_mode = col_mode; a.bits = bits; a.symmetric = symmetric; a.scope_rule = scope_rule;
    a.qmin = (float)qmin; a.qmax = (float)qmax; a.via_src = round_via_src_dtype;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case AMCT_F32: return run_fused<AMCT_F32>(a, st);
        case AMCT_F16: return run_fused<AMCT_F16>(a, st);
        case AMCT_BF16: return run_fused<AMCT_BF16>(a, st);
        default: return AMCT_E_BADARG;
    }
}
