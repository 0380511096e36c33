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
// A wave owns a row at a time with the columns across its lanes (2 per lane), so W[n][i] is a lane
// broadcast, the update is two multiplies and two subtractions per step, and the row's errors stay in
// registers until the row is done.  The block of the inverse Hessian is read once per thread block into LDS.
// All arithmetic is fp32 with one rounding per operation, as in the eager reference: true divisions,
// round-half-even, product and subtraction rounded separately.
#include "amct_common.h"

namespace amct {

constexpr int kGqMax = 128;                         // columns per block at most

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
    for (int rr = 0; rr < a.rows_per_wave; ++rr) {
        const int64_t n = row_begin + rr;
        if (n >= a.rows) break;                     // uniform for the wave
        float* wr = a.w + n * a.ld_w;
        float w0 = v0 ? wr[c0] : 0.f, w1 = v1 ? wr[c1] : 0.f;
        float e0 = 0.f, e1 = 0.f;
        // the factors of this row for every column of the block, one gather before the loop: lane j keeps
        // those of columns j and j + 64, and step i fetches them by lane broadcast like the weight itself
        const float* srow = a.scale + n * a.scale_stride;
        const int32_t* zrow = a.offset ? a.offset + n * a.scale_stride : nullptr;
        const int g0 = v0 ? a.gidx[c0] : 0, g1 = v1 ? a.gidx[c1] : 0;
        const float s0 = v0 ? srow[g0] : 1.f, s1 = v1 ? srow[g1] : 1.f;
        const float z0 = (zrow && v0) ? (float)zrow[g0] : 0.f, z1 = (zrow && v1) ? (float)zrow[g1] : 0.f;
        for (int i = 0; i < count; ++i) {
            const int src = i & 63;                                // i is wave-uniform
            const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? w0 : w1), src));
            const float s = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? s0 : s1), src));
            const float z = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < 64 ? z0 : z1), src));
            float t = w / s;
            if (zrow) t = t + z;
            t = __builtin_rintf(t);
            t = __builtin_amdgcn_fmed3f(t, a.qmin, a.qmax);
            const float wq = (t - z) * s;
            const float d = hs[i * count + i];
            const float err = (w - wq) / d;
            const float h0 = v0 ? hs[i * count + c0] : 0.f;
            const float h1 = v1 ? hs[i * count + c1] : 0.f;
            const float p0 = err * h0, p1 = err * h1;
            if (c0 >= i) w0 = w0 - p0;
            if (c1 >= i) w1 = w1 - p1;
            if (c0 == i) e0 = err;
            if (c1 == i) e1 = err;
        }
        float* er = a.err + n * a.ld_e;
        if (v0) { wr[c0] = w0; er[c0] = e0; }
        if (v1) { wr[c1] = w1; er[c1] = e1; }
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
    // about 1024 thread blocks of 4 waves, each wave walking a few rows
    int64_t rpw = (rows + 4095) / 4096;
    if (rpw < 1) rpw = 1;
    a.rows_per_wave = (int)rpw;
    const int64_t rows_per_block = rpw * (kBlock / 64);
    const int64_t nb = (rows + rows_per_block - 1) / rows_per_block;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    const size_t lds = (size_t)count * count * sizeof(float);
    if (lds > 64 * 1024) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(gptq_block_k, dim3((unsigned)nb), dim3(kBlock), lds, (hipStream_t)stream, a);
    return hip_status();
}
