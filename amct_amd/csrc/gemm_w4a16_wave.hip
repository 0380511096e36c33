// K7 for M <= 16 (decode), second form: every wave stages ITS OWN part of the activations.
//
// The first weight-streaming kernel (gemm_w4a16_stream.hip) stages the whole activation block once per block, all 16
// waves behind one barrier, and every block of the launch repeats that work: smoothing, group sums and the copy into LDS
// of 16 x 4096 activations are as many vector instructions as the dequantisation of the block's 64 weight columns, and
// nothing can be multiplied before the slowest wave has finished them.  Here a block of KS waves owns 64 output
// columns and a wave owns 256 elements of K (two groups of 128 = one 128-byte line of packed weights per column) for
// all 64 columns:
//   * its activations are 16 rows x 256 elements = 8 vectors of 16 bytes per lane, loaded coalesced (two rows of 512
//     bytes per instruction), smoothed with ONE smoothing vector per lane (a lane's 8 vectors share their position in
//     K), written to a piece of LDS only this wave touches, and read back as MFMA operands, which the wave keeps in
//     registers for its four column groups -- no block-wide barrier before the first MFMA, a quarter of the fragment
//     reads, and calls of fewer rows skip the load instructions of the missing row pairs (MR);
//   * the weights enter the MFMA as the exact integers 16 + u (see w4a16_stream_act.h) and the zero-point leaves on the
//     matrix pipe as well: a second MFMA multiplies the same activations with the constant -(16 + z) of the lane's
//     column, so the accumulator of a group holds sum x' * (u - z) and the fold is one fma with the group's scale per
//     accumulator -- no sums of activations are needed anywhere;
//   * all loads of a wave (activations, factors, bias, 8 x 16 bytes of weights per lane) are issued before anything
//     waits, in the order in which they are consumed.
// Arithmetic: x' = dt(x * smooth); y = sum_g s_g * (sum_{k in g} x'_k * (u_k - z_g)) with exact products, fp32
// accumulation, the KS partial sums added in wave order: the dequantised weight is NOT rounded to 16 bits.
#include "amct_common.h"
#include "gemm_plan.h"
#include "w4a16_stream_act.h"

namespace amct {

constexpr uint32_t kWvRow = 528;                     // bytes of a staged row: 256 elements + 16 (the 16 rows of a fragment read hit different banks)
constexpr uint32_t kWvRegion = 16 * kWvRow;          // LDS of one wave; later its 4 KB of partial sums

template <int DT>
AMCT_DEV uint4 wv_smooth8(const uint4& x, const float* cf) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = StAct<DT>::pack2(StAct<DT>::lo(xs[i]) * cf[2 * i], StAct<DT>::hi(xs[i]) * cf[2 * i + 1]);
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// MR: row pairs whose activations are loaded and staged (M <= 2 * MR); the rows beyond are never written nor read.
template <int DT, bool SF16, bool SMOOTH, int MR>
__global__ __launch_bounds__(1024) void w4a16_wave(StreamArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KS = (int)(blockDim.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int M = a.M, N = a.N;
    const int n0 = (int)blockIdx.x * 64;
    const uint32_t slice = blockIdx.y;
    // this wave's 256 elements of K; in a last, shorter slice a wave lies inside the row or beyond it as a whole (rows
    // are multiples of 256): beyond it, it reads the row's start and multiplies zeros
    const uint32_t k0 = slice * (uint32_t)a.K + (uint32_t)w * 256u;
    const bool inside = k0 < (uint32_t)a.row_k;
    const uint32_t kc = inside ? k0 : 0u;
    uint8_t* xs = lds + (uint32_t)w * kWvRegion;

    // ---- every load of the wave, in the order of use ---------------------------------------------------------------
    const uint32_t pv = lane & 31, half = lane >> 5;  // the lane's vector of 8 elements inside the 256, its row of a pair
    uint4 cv = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (SMOOTH) cv = ldg16(a.smooth + kc + 8 * pv);
    uint4 xv[MR];
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        int row = 2 * i + (int)half;
        row = row < M ? row : M - 1;
        xv[i] = ldg16(a.x + (size_t)row * a.row_k + kc + 8 * pv);
    }
    // scales (two adjacent 16-bit values) and zero-points (two adjacent bytes) of the lane's column in each column group
    const uint32_t row_g = (uint32_t)a.row_k / 128u, g0 = kc / 128u;
    uint32_t fs[4], fz[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int col = n0 + 16 * c + r16;
        const size_t fidx = (size_t)(col < N ? col : N - 1) * row_g + g0;
        fs[c] = *reinterpret_cast<const uint32_t*>(a.scales + fidx);
        fz[c] = *reinterpret_cast<const uint16_t*>(a.zeros + fidx);
    }
    // the bias of the column group this wave may write (waves 0 .. 3): loaded here, unconditionally, because a load in
    // the epilogue would wait for a trip to memory with nothing left to overlap it
    float bias_v;
    {
        const int col = n0 + 16 * (w & 3) + r16;
        bias_v = a.bias_src[col < N ? col : N - 1];
    }
    __builtin_amdgcn_sched_barrier(0);
    // weights: an instruction fetches 8 rows x one whole 128-byte line (this wave's 256 elements of K): lane l reads
    // row l % 8 (the second instruction of a pair rows 8 .. 15) and the 16-byte chunk chunk_of(l / 8) of the line
    u4v wv[8];
    {
        const uint32_t oct = lane >> 3;
        const uint32_t chunk = (oct & 1) ? 4 + (oct >> 1) : (oct >> 1);
        const size_t wrow = (size_t)(a.row_k / 2), woff = (size_t)(kc / 2) + chunk * 16;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int rlo = n0 + 16 * c + (lane & 7), rhi = rlo + 8;
            wv[2 * c] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(a.wq + (size_t)(rlo < N ? rlo : N - 1) * wrow + woff));
            wv[2 * c + 1] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(a.wq + (size_t)(rhi < N ? rhi : N - 1) * wrow + woff));
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- stage this wave's activations: smoothed, in the operand order of int8x --------------------------------------
    float cf[8];
    if constexpr (SMOOTH) {
        const uint32_t cs[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            cf[2 * i] = StAct<DT>::lo(cs[i]);
            cf[2 * i + 1] = StAct<DT>::hi(cs[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        uint4 v = xv[i];
        if (!inside) v = make_uint4(0u, 0u, 0u, 0u);
        if constexpr (SMOOTH) v = wv_smooth8<DT>(v, cf);
        *reinterpret_cast<uint4*>(xs + (2 * i + half) * kWvRow + pv * 16) = st_interleave8(v);
    }
    // the same wave reads them back as operands: lane (row r16, lane group g) takes elements 128 q + 32 g + 8 s .. + 7
    // for group q and MFMA s -- the elements its weight registers hold after the half swap below
    // (rows the call does not have read its last row: every operand of the MFMA is staged data)
    uint4 xf[2][4];
    const int rr = r16 < M ? r16 : M - 1;
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int s = 0; s < 4; ++s)
            xf[q][s] = *reinterpret_cast<const uint4*>(xs + rr * kWvRow + q * 256 + g * 64 + s * 16);
    __builtin_amdgcn_sched_barrier(0);

    // ---- four column groups, as their weights land -----------------------------------------------------------------
    s4f acc[4];
    uint32_t km = StAct<DT>::kMask, kb = StAct<DT>::kBase;
    asm volatile("" : "+v"(km), "+v"(kb));           // in registers: see and_or
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        // The MFMA wants 16 different rows in lanes 0 .. 15 of a lane group: the two registers of a pair swap halves (two
        // DPP moves per word); the first then holds chunks 0 .. 3 (the first group of 128, chunk g in lane group g) for
        // rows 0 .. 15, the second chunks 4 .. 7 (the second group).
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t lo = wv[2 * c][d], hi = wv[2 * c + 1][d];
            wv[2 * c][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)lo, (int)hi, 0x128, 0xF, 0xC, false);
            wv[2 * c + 1][d] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi, (int)lo, 0x128, 0xF, 0x3, false);
        }
        s4f P0 = {0.f, 0.f, 0.f, 0.f}, P1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            P0 = StAct<DT>::mfma(xf[0][s], StAct<DT>::int8x(wv[2 * c][s], km, kb), P0);
            P1 = StAct<DT>::mfma(xf[1][s], StAct<DT>::int8x(wv[2 * c + 1][s], km, kb), P1);
        }
        const uint32_t z0 = StAct<DT>::neg16z(fz[c] & 0xFFu), z1 = StAct<DT>::neg16z((fz[c] >> 8) & 0xFFu);
        const uint4 b0 = make_uint4(z0, z0, z0, z0), b1 = make_uint4(z1, z1, z1, z1);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            P0 = StAct<DT>::mfma(xf[0][s], b0, P0);
            P1 = StAct<DT>::mfma(xf[1][s], b1, P1);
        }
        const uint32_t sb0 = fs[c] & 0xFFFFu, sb1 = fs[c] >> 16;
        const float s0 = SF16 ? f16_bits_to_f32(sb0) : bf16_bits_to_f32(sb0);
        const float s1 = SF16 ? f16_bits_to_f32(sb1) : bf16_bits_to_f32(sb1);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[c][r] = __builtin_fmaf(s1, P1[r], s0 * P0[r]);
    }

    // ---- the KS partial sums of a column group, added in wave order by waves 0 .. 3 ----------------------------------
    // (a wave's partial sums go to its own piece of LDS, which only it has used so far: one barrier)
#pragma unroll
    for (int c = 0; c < 4; ++c) *reinterpret_cast<s4f*>(xs + (c * 64 + lane) * 16) = acc[c];
    __syncthreads();
    if (w < 4) {
        s4f y = *reinterpret_cast<const s4f*>(lds + (w * 64 + lane) * 16);
        for (int v = 1; v < KS; ++v) {
            const s4f o = *reinterpret_cast<const s4f*>(lds + (uint32_t)v * kWvRegion + (w * 64 + lane) * 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = y[r] + o[r];
        }
        const int ncol = n0 + 16 * w + r16, m0 = 4 * g;
        if (ncol < N) {
            if (a.part) {
                float* o = a.part + ((size_t)slice * M + m0) * N + ncol;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (m0 + r < M) o[(size_t)r * N] = y[r];
            } else {
                uint16_t* o = a.out + (size_t)m0 * N + ncol;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = y[r];
                    if (a.bias) v = v + bias_v;
                    if (m0 + r < M) o[(size_t)r * N] = (uint16_t)StAct<DT>::out_bits(v);
                }
            }
        }
    }
}

int splitk_reduce16_launch(const float* part, const float* bias, void* out, int64_t M, int64_t N, int splits, int dtype,
                           hipStream_t st);                          // gemm_w4a16.hip

template <int DT, bool SF16, bool SMOOTH, int MR>
static int wave_launch_mr(const StreamArgs& a, dim3 grid, int ks, hipStream_t st) {
    auto kern = &w4a16_wave<DT, SF16, SMOOTH, MR>;
    const size_t lds_bytes = (size_t)ks * kWvRegion;
    if (lds_bytes > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                     160 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return AMCT_E_HIP;
    }
    hipLaunchKernelGGL(kern, grid, dim3((unsigned)ks * 64), lds_bytes, st, a);
    if (a.part) return splitk_reduce16_launch(a.part, a.bias, a.out, a.M, a.N, (int)grid.y, DT, st);
    return hip_status();
}

template <int DT, bool SF16, bool SMOOTH>
static int wave_launch_sf(const StreamArgs& a, dim3 grid, int ks, hipStream_t st) {
    if (a.M <= 2) return wave_launch_mr<DT, SF16, SMOOTH, 1>(a, grid, ks, st);
    if (a.M <= 4) return wave_launch_mr<DT, SF16, SMOOTH, 2>(a, grid, ks, st);
    if (a.M <= 8) return wave_launch_mr<DT, SF16, SMOOTH, 4>(a, grid, ks, st);
    return wave_launch_mr<DT, SF16, SMOOTH, 8>(a, grid, ks, st);
}
template <int DT, bool SMOOTH>
static int wave_launch(const StreamArgs& a, dim3 grid, int ks, hipStream_t st) {
    return a.scale_f16 ? wave_launch_sf<DT, true, SMOOTH>(a, grid, ks, st) : wave_launch_sf<DT, false, SMOOTH>(a, grid, ks, st);
}

// Whether this form takes the shape: a slice of 1024 / 2048 / 4096 elements (4 / 8 / 16 waves), and blocks that all run
// at once (16 waves fill a CU) -- with more column tiles than that, the first form walks several tiles per block on one
// staged copy of the activations.
bool w4a16_wave_fits(int64_t N, int64_t K_slice, int64_t slices) {
    const int64_t cus = current_cu_count();
    if (K_slice != 1024 && K_slice != 2048 && K_slice != 4096) return false;
    const int64_t tiles = (N + 63) / 64, per_cu = 4096 / K_slice;
    return cus > 0 && tiles * slices <= cus * per_cu && tiles <= 0x7FFFFFFF && slices <= 65535;
}

// The arguments as the first form's dispatch has prepared and checked them (K: the slice one block walks).
int w4a16_wave_launch(const StreamArgs& a, int slices, int dtype, hipStream_t st) {
    const dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)slices);
    const int ks = a.K / 256;
    if (dtype == AMCT_F16) return a.smooth ? wave_launch<AMCT_F16, true>(a, grid, ks, st) : wave_launch<AMCT_F16, false>(a, grid, ks, st);
    return a.smooth ? wave_launch<AMCT_BF16, true>(a, grid, ks, st) : wave_launch<AMCT_BF16, false>(a, grid, ks, st);
}

}  // namespace amct
