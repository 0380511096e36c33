// GPTQ inner block: the column-by-column quantise / propagate-error loop of
// amct_pytorch/quantize_op/gptq_module.py:128-151 for one block of at most 128 columns, fused into one launch
// (the reference issues, per column, a fake-quant of an [N,1] slice, a division and a rank-1 update).
//
// Every row of the weight is independent inside the block:
//   for i in 0 .. count-1:
//       w    = W[n][i]
//       wq   = ((clamp(rne(w / s + z), qmin, qmax)) - z) * s                    (quant_dequant_weight)
//       err  = (w - wq) / Hinv[i][i]
//       W[n][j] -= err * Hinv[i][j]      for j = i .. count-1                   (one product, one subtraction)
//       E[n][i]  = err
// Two kernels.  Blocks of fewer than 128 columns (gptq_block_k):
// a wave owns four rows at a time with the columns across its lanes (2 per lane), so W[n][i] is a lane
// broadcast, the update is two multiplies and two subtractions per step, and the row's errors stay in
// registers until the row is done.  Full blocks of 128 columns (gptq_block_quad_k, described there): four lanes
// share a row.  The block of the inverse Hessian is read once per thread block into LDS.
// All arithmetic is fp32 with one rounding per operation, as in the eager reference: true divisions,
// round-half-even, product and subtraction rounded separately.
#include "amct_common.h"

namespace amct {

constexpr int kGqMax = 128;                         // columns per block at most
constexpr int kGqRows = 4;                          // rows a wave works on at the same time

struct GptqArgs {
    float* w;                                       // [rows][ld_w], the block starts at column 0 of this pointer
    float* err;                                     // [rows][ld_e]
    const float* hinv;                              // [count][ld_h]
    const float* scale;                             // [rows or 1][scale_stride or 0 ...]
    const int32_t* offset;                          // same layout, or null (symmetric)
    const int32_t* gidx;                            // [count] index of the scale column for each block column
    int64_t rows, ld_w, ld_e, ld_h, scale_stride;
    int count;
    int rows_per_wave;
    float qmin, qmax;
};

__global__ __launch_bounds__(kBlock) void gptq_block_k(GptqArgs a) {
    extern __shared__ float hs[];                   // [count][count]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int count = a.count;
    for (int i = tid; i < count * count; i += kBlock) {
        const int r = i / count, c = i - r * count;
        hs[i] = a.hinv[(int64_t)r * a.ld_h + c];
    }
    __syncthreads();
    const int c0 = lane, c1 = lane + 64;
    const bool v0 = c0 < count, v1 = c1 < count;
    const int64_t row_begin = ((int64_t)blockIdx.x * (kBlock / 64) + wave) * a.rows_per_wave;
    // kGqRows rows at a time: their chains of dependent operations (two divisions and ten more per step) are
    // independent of one another, so the wave issues one row's step while the others' results are on their way, and
    // the Hessian entries of a step are read from LDS once for all of them.  One row at a time ran at a fifth of the
    // vector-ALU issue rate.
    for (int rr = 0; rr < a.rows_per_wave; rr += kGqRows) {
        if (row_begin + rr >= a.rows) break;        // uniform for the wave
        float w0[kGqRows], w1[kGqRows], e0[kGqRows], e1[kGqRows], s0[kGqRows], s1[kGqRows], z0[kGqRows], z1[kGqRows];
        const int32_t g0 = v0 ? a.gidx[c0] : 0, g1 = v1 ? a.gidx[c1] : 0;
#pragma unroll
        for (int r = 0; r < kGqRows; ++r) {
            // rows beyond the matrix repeat its last row (loads stay unconditional; nothing is stored for them)
            const int64_t n = row_begin + rr + r < a.rows ? row_begin + rr + r : a.rows - 1;
            const float* wr = a.w + n * a.ld_w;
            w0[r] = v0 ? wr[c0] : 0.f;
            w1[r] = v1 ? wr[c1] : 0.f;
            e0[r] = 0.f;
            e1[r] = 0.f;
            // the factors of this row for every column of the block, one gather before the loop: lane j keeps
            // those of columns j and j + 64, and step i fetches them by lane broadcast like the weight itself
            const float* srow = a.scale + n * a.scale_stride;
            const int32_t* zrow = a.offset ? a.offset + n * a.scale_stride : nullptr;
            s0[r] = v0 ? srow[g0] : 1.f;
            s1[r] = v1 ? srow[g1] : 1.f;
            z0[r] = (zrow && v0) ? (float)zrow[g0] : 0.f;
            z1[r] = (zrow && v1) ? (float)zrow[g1] : 0.f;
        }
        const bool asym = a.offset != nullptr;
        for (int i = 0; i < count; ++i) {
            const int src = i & 63;                                // i is wave-uniform
            const float d = hs[i * count + i];
            const float h0 = v0 ? hs[i * count + c0] : 0.f;
            const float h1 = v1 ? hs[i * count + c1] : 0.f;
#pragma unroll
            for (int r = 0; r < kGqRows; ++r) {
                const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? w0[r] : w1[r]), src));
                const float s = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? s0[r] : s1[r]), src));
                const float z = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? z0[r] : z1[r]), src));
                float t = w / s;
                if (asym) t = t + z;
                t = __builtin_rintf(t);
                t = __builtin_amdgcn_fmed3f(t, a.qmin, a.qmax);
                const float wq = (t - z) * s;
                const float err = (w - wq) / d;
                const float p0 = err * h0, p1 = err * h1;
                if (c0 >= i) w0[r] = w0[r] - p0;
                if (c1 >= i) w1[r] = w1[r] - p1;
                if (c0 == i) e0[r] = err;
                if (c1 == i) e1[r] = err;
            }
        }
#pragma unroll
        for (int r = 0; r < kGqRows; ++r) {
            const int64_t n = row_begin + rr + r;
            if (n < a.rows) {
                float* wr = a.w + n * a.ld_w;
                float* er = a.err + n * a.ld_e;
                if (v0) { wr[c0] = w0[r]; er[c0] = e0[r]; }
                if (v1) { wr[c1] = w1[r]; er[c1] = e1[r]; }
            }
        }
    }
}

// Full blocks of 128 columns: four lanes share a row (16 rows per wave, 64 per thread block) and each keeps 32
// of the row's columns in registers, column 16 m + 4 q + e in slot [m][e] of quad lane q, so that loads and stores
// are 16 bytes per lane and the columns still to be updated stay spread over the four lanes as the step advances.
// The chain of a step (weight of column i by quad broadcast, quantise, error) is computed by the 4 lanes of the row
// instead of by all 64 lanes of a wave, and the update touches only the slots at or behind column i: about 60
// instructions per step for 16 rows instead of 40 per step and row.  The 128 steps are unrolled (the slots are
// registers); the factors of step i + 8 are fetched while step i runs.  Same operations per element as the kernel
// above, in the same order.
constexpr int kGqAhead = 8;

template <bool ASYM>
__global__ __launch_bounds__(kBlock) void gptq_block_quad_k(GptqArgs a) {
    __shared__ __attribute__((aligned(16))) float hs[kGqMax * kGqMax];           // [128][128]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < kGqMax * kGqMax; i += kBlock) hs[i] = a.hinv[(int64_t)(i >> 7) * a.ld_h + (i & 127)];
    __syncthreads();
    const int q = lane & 3;
    const int64_t n = (int64_t)blockIdx.x * 64 + wave * 16 + (lane >> 2);
    const int64_t nc = n < a.rows ? n : a.rows - 1;              // rows beyond the matrix repeat its last row; not stored
    const float* wr = a.w + nc * a.ld_w + 4 * q;
    const float* srow = a.scale + nc * a.scale_stride;
    const int32_t* zrow = ASYM ? a.offset + nc * a.scale_stride : nullptr;
    float w[8][4], eo[8][4];
#pragma unroll
    for (int m = 0; m < 8; ++m) {
        const float4 v = *reinterpret_cast<const float4*>(wr + 16 * m);
        w[m][0] = v.x; w[m][1] = v.y; w[m][2] = v.z; w[m][3] = v.w;
    }
    float sr[kGqAhead], zr[kGqAhead];
#pragma unroll
    for (int i = 0; i < kGqAhead; ++i) {
        const int g = a.gidx[i];
        sr[i] = srow[g];
        zr[i] = ASYM ? (float)zrow[g] : 0.f;
    }
    // Software pipeline: the chain of step i (broadcast, two divisions, quantisation: about 30 dependent operations) is
    // the critical path of the whole kernel -- a thread block takes the same 128 x chain whether the matrix has 64 rows
    // or 14336 -- and the updates of step i - 1 are independent of it except for the one slot that holds column i.  So
    // step i - 1 updates only that slot before step i starts (the "critical" slot: one product and one subtraction), and
    // the other slots of step i - 1 are updated INSIDE the chain of step i, a third of them in each of its three parts,
    // where they fill the issue slots the chain leaves empty.  Every element still receives its updates in step order:
    // the operations and their order per element are those of the loop above.
    float err_prev = 0.f;
    float hprev[8][4];                                              // row i - 1 of the block of Hinv, this lane's columns
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) hprev[m][e] = 0.f;
#pragma clang loop unroll(full)
    for (int i = 0; i < kGqMax; ++i) {
        const int mi = i >> 4, qi = (i >> 2) & 3, ei = i & 3;
        const int mp = (i - 1) >> 4;                                // slot row of column i - 1 (i >= 1)
        // the slots of step i - 1 that are still to be updated: (m, e) with m >= mp, except the slot of column i
        auto pending = [&](int part) {
            if (i == 0) return;
#pragma unroll
            for (int sl = 0; sl < 32; ++sl) {
                const int m = sl >> 2, e = sl & 3;
                if (sl % 3 != part || m < mp || (m == mi && e == ei)) continue;
                const float p = err_prev * hprev[m][e];
                if (m > mp) w[m][e] = w[m][e] - p;
                else if (4 * q + e >= ((i - 1) & 15)) w[m][e] = w[m][e] - p;
            }
        };
        // row i of the block of Hinv for the updates of this step: the diagonal, the critical slot, and (for the next
        // iteration) this lane's columns at and behind slot row mi
        const float hdiag = hs[i * kGqMax + i];
        const int inx = i + 1 < kGqMax ? i + 1 : i;                 // column i + 1, whose slot is updated before step i + 1
        const int mn = inx >> 4, en = inx & 3;
        const float hcrit = hs[i * kGqMax + 16 * mn + 4 * q + en];
        float hcur[8][4];
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if (m < mi) continue;
            const float4 h = *reinterpret_cast<const float4*>(&hs[i * kGqMax + 16 * m + 4 * q]);
            hcur[m][0] = h.x; hcur[m][1] = h.y; hcur[m][2] = h.z; hcur[m][3] = h.w;
        }
        float wi;
        if (qi == 0) wi = quad_bcast<0>(w[mi][ei]);
        else if (qi == 1) wi = quad_bcast<1>(w[mi][ei]);
        else if (qi == 2) wi = quad_bcast<2>(w[mi][ei]);
        else wi = quad_bcast<3>(w[mi][ei]);
        const float sc = sr[i % kGqAhead], z = zr[i % kGqAhead];
        if (i + kGqAhead < kGqMax) {
            const int g = a.gidx[i + kGqAhead];
            sr[i % kGqAhead] = srow[g];
            zr[i % kGqAhead] = ASYM ? (float)zrow[g] : 0.f;
        }
        float t = wi / sc;
        pending(0);
        __builtin_amdgcn_sched_barrier(0);
        if (ASYM) t = t + z;
        t = __builtin_rintf(t);
        t = __builtin_amdgcn_fmed3f(t, a.qmin, a.qmax);
        const float wq = (t - z) * sc;
        const float dlt = wi - wq;
        pending(1);
        __builtin_amdgcn_sched_barrier(0);
        const float err = dlt / hdiag;
        pending(2);
        __builtin_amdgcn_sched_barrier(0);
        if (q == qi) eo[mi][ei] = err;
        // the critical slot: the one that holds column i + 1 (column i itself -- the reference's update runs from j = i,
        // W[n][i] -= err * Hinv[i][i]: not read again, but what the caller gets back -- shares its slot with columns of
        // the other lanes and is updated with them, among the pending slots of the next iteration)
        if (i + 1 < kGqMax) {
            const float p = err * hcrit;
            if (mn > mi) w[mn][en] = w[mn][en] - p;
            else if (4 * q + en >= (i & 15)) w[mn][en] = w[mn][en] - p;
        }
        __builtin_amdgcn_sched_barrier(0);
        err_prev = err;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if (m < mi) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) hprev[m][e] = hcur[m][e];
        }
    }
    // what step 127 leaves pending: column 127 itself (slot (7, 3) of lane 3)
    if (q == 3) w[7][3] = w[7][3] - err_prev * hprev[7][3];
    if (n < a.rows) {
        float* wo = a.w + n * a.ld_w + 4 * q;
        float* er = a.err + n * a.ld_e + 4 * q;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            *reinterpret_cast<float4*>(wo + 16 * m) = make_float4(w[m][0], w[m][1], w[m][2], w[m][3]);
            *reinterpret_cast<float4*>(er + 16 * m) = make_float4(eo[m][0], eo[m][1], eo[m][2], eo[m][3]);
        }
    }
}

}  // namespace amct

using namespace amct;

extern "C" int amct_gptq_block(float* w, int64_t ld_w, float* err, int64_t ld_e, const float* hinv, int64_t ld_h,
                               const float* scale, const int32_t* offset, int64_t scale_stride, const int32_t* gidx,
                               int64_t rows, int count, int qmin, int qmax, amct_stream_t stream) {
    if (rows < 0 || count < 0 || count > kGqMax || qmin > qmax) return AMCT_E_BADARG;
    if (ld_w < count || ld_e < count || ld_h < count || scale_stride < 0) return AMCT_E_BADARG;
    if (rows == 0 || count == 0) return AMCT_OK;
    if (!w || !err || !hinv || !scale || !gidx) return AMCT_E_BADARG;
    GptqArgs a{};
    a.w = w; a.err = err; a.hinv = hinv; a.scale = scale; a.offset = offset; a.gidx = gidx;
    a.rows = rows; a.ld_w = ld_w; a.ld_e = ld_e; a.ld_h = ld_h; a.scale_stride = scale_stride;
    a.count = count; a.qmin = (float)qmin; a.qmax = (float)qmax;
    if (count == kGqMax && ld_w % 4 == 0 && ld_e % 4 == 0 && aligned16(w) && aligned16(err) && (rows + 63) / 64 <= 0x7FFFFFFF) {
        const unsigned nbq = (unsigned)((rows + 63) / 64);
        if (offset) hipLaunchKernelGGL(gptq_block_quad_k<true>, dim3(nbq), dim3(kBlock), 0, (hipStream_t)stream, a);
        else hipLaunchKernelGGL(gptq_block_quad_k<false>, dim3(nbq), dim3(kBlock), 0, (hipStream_t)stream, a);
        return hip_status();
    }
    // about 1024 thread blocks of 4 waves, each wave walking a few groups of kGqRows rows
    int64_t rpw = (rows + 4095) / 4096;
    rpw = (rpw + kGqRows - 1) / kGqRows * kGqRows;
    if (rpw < kGqRows) rpw = kGqRows;
    a.rows_per_wave = (int)rpw;
    const int64_t rows_per_block = rpw * (kBlock / 64);
    const int64_t nb = (rows + rows_per_block - 1) / rows_per_block;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    const size_t lds = (size_t)count * count * sizeof(float);
    if (lds > 64 * 1024) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(gptq_block_k, dim3((unsigned)nb), dim3(kBlock), lds, (hipStream_t)stream, a);
    return hip_status();
}
