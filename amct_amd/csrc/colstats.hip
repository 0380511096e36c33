// Column statistics over tokens: per input channel max / min (or max of |x|) of a [rows, cols] tensor.
// Replaces the calibration reductions of amct_pytorch/quantize_op/smooth_quant_module.py:79-80
// (batch amax / amin over all tokens), :88-91 (running update) and :121 (|W|.amax(dim=0)).
//
// The tensor is read once, 16 bytes per lane and instruction, rows in the outer loop:
//   pass 1: a block of 32 column vectors x 8 row lanes reduces a chunk of rows; its 8 row lanes meet in
//           LDS and one partial per (chunk, column) goes to the caller's workspace;
//   pass 2: one lane per column folds the chunks (coalesced across columns) and applies the update rule.
// max / min propagate NaN like torch.amax / amin; the running update `batch > old ? batch : old` then
// ignores a NaN batch value, exactly as torch.where does in the reference.
#include <atomic>

#include "amct_common.h"

namespace amct {

constexpr int kCsVecs = 32;            // column vectors per block
constexpr int kCsLanes = 8;            // row lanes per block
constexpr int kCsRows = 256;           // rows per chunk (before the chunk count is capped)
constexpr int kCsMaxChunks = 64;
constexpr int kCsUnroll = 16;          // rows in flight per lane (measured: 16.8 us against 17.5 us with 4)

struct ColArgs {
    const void* x;
    float* ws;                          // [chunks][2][cols]
    int64_t rows, cols;
    int64_t rows_per_chunk;
    int chunks;
};

template <int DT, bool ABS>
__global__ __launch_bounds__(kCsVecs * kCsLanes) void col_partial_k(ColArgs a) {
    constexpr int VEC = Tr<DT>::VEC;
    constexpr int BYTES = Tr<DT>::BYTES;
    __shared__ float red[2][kCsLanes][kCsVecs * VEC + 1];
    const int tid = threadIdx.x;
    const int cv = tid % kCsVecs, rl = tid / kCsVecs;
    const int64_t nvec = a.cols / VEC;
    const int64_t v = (int64_t)blockIdx.x * kCsVecs + cv;
    const int64_t vc = v < nvec ? v : nvec - 1;                     // clamped: loads are unconditional
    const int64_t r0 = (int64_t)blockIdx.y * a.rows_per_chunk;
    const int64_t r1 = r0 + a.rows_per_chunk < a.rows ? r0 + a.rows_per_chunk : a.rows;
    const char* base = reinterpret_cast<const char*>(a.x) + vc * 16;
    const int64_t row_bytes = a.cols * BYTES;

    float mx[VEC], mn[VEC];
    bool first = true;
    // rows r0 + rl, + 8, + 16, ... of the chunk, kCsUnroll per iteration; the first iteration always runs (a row
    // lane beyond a short chunk re-reads the chunk's last row, which changes nothing)
    int64_t r = r0 + rl;
    do {
        uint4 raw[kCsUnroll];
#pragma unroll
        for (int u = 0; u < kCsUnroll; ++u) {
            const int64_t rr = r + u * kCsLanes;
            raw[u] = ldg16_nt(base + (rr < r1 ? rr : r1 - 1) * row_bytes);   // duplicates do not change a max / min
        }
#pragma unroll
        for (int u = 0; u < kCsUnroll; ++u) {
            float x[VEC];
            unpack16<DT>(raw[u], x);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float e = ABS ? __builtin_fabsf(x[j]) : x[j];
                mx[j] = first ? e : fmax_nan(mx[j], e);
                mn[j] = first ? e : fmin_nan(mn[j], e);
            }
            first = false;
        }
        r += kCsUnroll * kCsLanes;
    } while (r < r1);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        red[0][rl][cv * VEC + j] = mx[j];
        red[1][rl][cv * VEC + j] = mn[j];
    }
    __syncthreads();
    // 32 * VEC columns, 2 statistics: one (statistic, column) per lane and pass
    for (int i = tid; i < 2 * kCsVecs * VEC; i += kCsVecs * kCsLanes) {
        const int which = i / (kCsVecs * VEC), c = i % (kCsVecs * VEC);
        float acc = red[which][0][c];
#pragma unroll
        for (int l = 1; l < kCsLanes; ++l) acc = which == 0 ? fmax_nan(acc, red[which][l][c]) : fmin_nan(acc, red[which][l][c]);
        const int64_t col = (int64_t)blockIdx.x * kCsVecs * VEC + c;
        if (col < a.cols) a.ws[((int64_t)blockIdx.y * 2 + which) * a.cols + col] = acc;
    }
}

// any shape / alignment: one lane per column walks the chunk's rows
template <int DT, bool ABS>
__global__ __launch_bounds__(kBlock) void col_partial_general_k(ColArgs a) {
    const int64_t col = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= a.cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * a.rows_per_chunk;
    const int64_t r1 = r0 + a.rows_per_chunk < a.rows ? r0 + a.rows_per_chunk : a.rows;
    float mx = 0.f, mn = 0.f;
    for (int64_t r = r0; r < r1; ++r) {
        float e = load_scalar<DT>(a.x, r * a.cols + col);
        if (ABS) e = __builtin_fabsf(e);
        mx = r == r0 ? e : fmax_nan(mx, e);
        mn = r == r0 ? e : fmin_nan(mn, e);
    }
    a.ws[((int64_t)blockIdx.y * 2 + 0) * a.cols + col] = mx;
    a.ws[((int64_t)blockIdx.y * 2 + 1) * a.cols + col] = mn;
}

// pass 2: four lanes per column, each folding every fourth chunk with all of its loads in flight (at most
// kCsMaxChunks / 4; an index beyond the last chunk re-reads the last one, which changes nothing), then the quad meets
// by DPP.  One lane per column and eight loads in flight took 3.8 us for 32 chunks of 4096 columns.
__global__ __launch_bounds__(kBlock) void col_final_k(const float* ws, float* col_max, float* col_min, int64_t cols,
                                                      int chunks, int accumulate) {
    constexpr int kPer = kCsMaxChunks / 4;
    const int cg = threadIdx.x & 3;
    const int64_t col = (int64_t)blockIdx.x * (kBlock / 4) + (threadIdx.x >> 2);
    const int64_t cc = col < cols ? col : cols - 1;
    float tx[kPer], tn[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const int c = cg + 4 * u < chunks ? cg + 4 * u : chunks - 1;
        tx[u] = ws[((int64_t)c * 2 + 0) * cols + cc];
        tn[u] = ws[((int64_t)c * 2 + 1) * cols + cc];
    }
    float mx = tx[0], mn = tn[0];
#pragma unroll
    for (int u = 1; u < kPer; ++u) {
        mx = fmax_nan(mx, tx[u]);
        mn = fmin_nan(mn, tn[u]);
    }
    mx = fmax_nan(mx, __uint_as_float(dpp_u<0xB1>(__float_as_uint(mx))));
    mn = fmin_nan(mn, __uint_as_float(dpp_u<0xB1>(__float_as_uint(mn))));
    mx = fmax_nan(mx, __uint_as_float(dpp_u<0x4E>(__float_as_uint(mx))));
    mn = fmin_nan(mn, __uint_as_float(dpp_u<0x4E>(__float_as_uint(mn))));
    if (cg != 0 || col >= cols) return;
    if (col_max) {
        const float old = col_max[col];
        col_max[col] = accumulate ? (mx > old ? mx : old) : mx;
    }
    if (col_min) {
        const float old = col_min[col];
        col_min[col] = accumulate ? (mn < old ? mn : old) : mn;
    }
}

static void chunking(int64_t rows, int64_t& rows_per_chunk, int& chunks) {
    int64_t n = (rows + kCsRows - 1) / kCsRows;
    if (n > kCsMaxChunks) n = kCsMaxChunks;
    if (n < 1) n = 1;
    rows_per_chunk = (rows + n - 1) / n;
    chunks = (int)((rows + rows_per_chunk - 1) / (rows_per_chunk > 0 ? rows_per_chunk : 1));
    if (chunks < 1) chunks = 1;
}

}  // namespace amct

using namespace amct;

extern "C" size_t amct_col_minmax_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    int64_t rpc;
    int chunks;
    chunking(rows, rpc, chunks);
    return (size_t)chunks * 2 * (size_t)cols * sizeof(float);
}

// shared by both entry points: `ws` holds chunks * 2 * cols floats and is fully overwritten by pass 1 before pass 2 reads it
static int col_minmax_launch(const void* x, float* col_max, float* col_min, int64_t rows, int64_t cols, int absolute,
                             int accumulate, int dtype, float* ws, hipStream_t st) {
    ColArgs a{};
    a.x = x; a.ws = ws; a.rows = rows; a.cols = cols;
    chunking(rows, a.rows_per_chunk, a.chunks);
#define AMCT_CS(DT)                                                                                              \
    {                                                                                                            \
        constexpr int VEC = Tr<DT>::VEC;                                                                         \
        if (aligned16(x) && cols % VEC == 0) {                                                                   \
            const dim3 grid((unsigned)((cols / VEC + kCsVecs - 1) / kCsVecs), (unsigned)a.chunks);               \
            if (absolute) hipLaunchKernelGGL((col_partial_k<DT, true>), grid, dim3(kCsVecs * kCsLanes), 0, st, a); \
            else hipLaunchKernelGGL((col_partial_k<DT, false>), grid, dim3(kCsVecs * kCsLanes), 0, st, a);       \
        } else {                                                                                                 \
            const dim3 grid((unsigned)((cols + kBlock - 1) / kBlock), (unsigned)a.chunks);                       \
            if (absolute) hipLaunchKernelGGL((col_partial_general_k<DT, true>), grid, dim3(kBlock), 0, st, a);   \
            else hipLaunchKernelGGL((col_partial_general_k<DT, false>), grid, dim3(kBlock), 0, st, a);           \
        }                                                                                                        \
    }
    switch (dtype) {
        case AMCT_F32: AMCT_CS(AMCT_F32) break;
        case AMCT_F16: AMCT_CS(AMCT_F16) break;
        default: AMCT_CS(AMCT_BF16) break;
    }
#undef AMCT_CS
    hipLaunchKernelGGL(col_final_k, dim3((unsigned)((cols + kBlock / 4 - 1) / (kBlock / 4))), dim3(kBlock), 0, st, a.ws, col_max,
                       col_min, cols, a.chunks, accumulate);
    return hip_status();
}

extern "C" int amct_col_minmax(const void* x, float* col_max, float* col_min, int64_t rows, int64_t cols, int absolute,
                               int accumulate, int dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream) {
    if (rows < 0 || cols <= 0) return AMCT_E_BADARG;
    if (dtype != AMCT_F32 && dtype != AMCT_F16 && dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (rows == 0) return AMCT_OK;                                  // no batch: the running values stay
    if (!x || (!col_max && !col_min) || !workspace) return AMCT_E_BADARG;
    if (workspace_bytes < amct_col_minmax_workspace_bytes(rows, cols)) return AMCT_E_BADARG;
    if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return AMCT_E_ALIGN;
    return col_minmax_launch(x, col_max, col_min, rows, cols, absolute, accumulate, dtype,
                             reinterpret_cast<float*>(workspace), (hipStream_t)stream);
}

// ---- the same reduction for callers that cannot allocate -----------------------------------------------------
// The per-chunk partials live in a fixed array in device memory that is part of the library's code object: every
// GPU the library runs on holds its own copy (4 MiB) until the process ends.  The array's name is only a host-side
// handle; its device address is asked for once per device and kept.
static __device__ __align__(256) float scratch[(size_t)kCsMaxChunks * 2 * AMCT_COL_MINMAX_NOALLOC_MAX_COLS];

constexpr int kMaxDevices = 64;
static std::atomic<float*> scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device (null on failure); first call per device asks the runtime
static float* scratch_on_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    float* p = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* q = nullptr;
        if (hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)) != hipSuccess || !q) {
            (void)hipGetLastError();
            return nullptr;
        }
        p = reinterpret_cast<float*>(q);
        scratch_ptr[dev].store(p, std::memory_order_release);       // racing first calls store the same address
    }
    return p;
}

extern "C" int amct_col_minmax_noalloc(const void* x, float* col_max, float* col_min, int64_t rows, int64_t cols,
                                       int absolute, int accumulate, int dtype, amct_stream_t stream) {
    if (rows < 0 || cols <= 0) return AMCT_E_BADARG;
    if (dtype != AMCT_F32 && dtype != AMCT_F16 && dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (cols > AMCT_COL_MINMAX_NOALLOC_MAX_COLS) return AMCT_E_TOO_LARGE;
    if (rows == 0) return AMCT_OK;
    if (!x || (!col_max && !col_min)) return AMCT_E_BADARG;
    float* ws = scratch_on_current_device();
    if (!ws) return AMCT_E_HIP;
    // pass 1 writes every partial that pass 2 reads, so nothing of an earlier call has to be cleared
    return col_minmax_launch(x, col_max, col_min, rows, cols, absolute, accumulate, dtype, ws, (hipStream_t)stream);
}
