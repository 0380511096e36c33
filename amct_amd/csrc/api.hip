// Library identity and error strings.
#include "amct_common.h"

extern "C" int amct_hip_version(void) { return 100; }

extern "C" const char* amct_hip_strerror(int code) {
    switch (code) {
        case AMCT_OK: return "ok";
        case AMCT_E_BADARG: return "bad argument (null pointer, negative size or unknown enum)";
        case AMCT_E_UNSUPPORTED: return "shape or combination not supported by the kernels";
        case AMCT_E_ALIGN: return "alignment or divisibility requirement violated";
        case AMCT_E_HIP: return "HIP runtime reported a launch error";
        case AMCT_E_TOO_LARGE: return "problem exceeds the fixed scratch buffer of the allocation-free entry point";
        default: return "unknown error code";
    }
}

namespace amct {
// plain streaming copy, 16 bytes per lane and 4 in flight: the yardstick the quantize kernels'
// bandwidth and hardware traffic counters are compared with
__global__ __launch_bounds__(kBlock) void copy_k(const uint4* src, uint4* dst, int64_t nvec) {
    constexpr int U = 4;
    const int64_t base = (int64_t)blockIdx.x * kBlock * U + threadIdx.x;
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {                      // unconditional streaming loads, index clamped
        const int64_t i = base + u * kBlock;
        v[u] = ldg16_nt(src + (i < nvec ? i : nvec - 1));
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (base + u * kBlock < nvec) stg16_nt(dst + base + u * kBlock, v[u]);
}

// Register-only MFMA loop: 8 waves per block, 8 independent accumulator tiles per wave, no memory traffic.
// With RANDOM the 8 operand pairs of a wave hold pseudo-random values (so consecutive instructions see different
// data); otherwise every operand byte is the same.  What this loop sustains is the ceiling of the matrix pipe
// under the power limit for that kind of data: a GEMM cannot be faster.
typedef int yv4i __attribute__((ext_vector_type(4)));
typedef int yv16i __attribute__((ext_vector_type(16)));
typedef float yv16f __attribute__((ext_vector_type(16)));
typedef __bf16 yv8bf __attribute__((ext_vector_type(8)));

AMCT_DEV uint32_t yard_hash(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

template <bool BF, bool RANDOM>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void mfma_yardstick_k(int32_t* sink, int iters) {
    const int tid = threadIdx.x;
    yv4i a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t ra = RANDOM ? yard_hash(tid * 64 + i * 8 + c + blockIdx.x * 7919u) : 0x01010101u;
            uint32_t rb = RANDOM ? yard_hash(tid * 64 + i * 8 + c + 4 + blockIdx.x * 104729u) : 0x02020202u;
            if (BF) {                                               // bf16 values in +-[0.5, 1)
                ra = (ra & 0x807F807Fu) | 0x3F003F00u;
                rb = (rb & 0x807F807Fu) | 0x3F003F00u;
            }
            a[i][c] = (int)ra;
            b[i][c] = (int)rb;
        }
    int s = 0;
    if constexpr (BF) {
        yv16f acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(yv8bf, a[i]), __builtin_bit_cast(yv8bf, b[i]), acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) s += (int)acc[i][0] + (int)acc[i][7];
    } else {
        yv16i acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][r] = 0;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[i], acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][7];
    }
    if (s == 0x12345678) sink[tid] = s;                             // keeps the loop alive; practically never taken
}
}  // namespace amct

extern "C" int amct_mfma_yardstick(int bf16, int random_operands, int iters, void* sink, int64_t* ops, amct_stream_t stream) {
    if (iters < 0 || !sink || !ops) return AMCT_E_BADARG;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0) {
        (void)hipGetLastError();
        return AMCT_E_HIP;
    }
    // one block of 8 waves per CU; a 32x32x32 int8 MFMA is 65536 operations, a 32x32x16 bf16 MFMA 32768
    *ops = (int64_t)cus * 8 * 8 * (int64_t)iters * (bf16 ? 32768 : 65536);
    if (iters == 0) return AMCT_OK;
    hipStream_t st = (hipStream_t)stream;
    int32_t* sk = reinterpret_cast<int32_t*>(sink);
    if (bf16 && random_operands) hipLaunchKernelGGL((amct::mfma_yardstick_k<true, true>), dim3(cus), dim3(512), 0, st, sk, iters);
    else if (bf16) hipLaunchKernelGGL((amct::mfma_yardstick_k<true, false>), dim3(cus), dim3(512), 0, st, sk, iters);
    else if (random_operands) hipLaunchKernelGGL((amct::mfma_yardstick_k<false, true>), dim3(cus), dim3(512), 0, st, sk, iters);
    else hipLaunchKernelGGL((amct::mfma_yardstick_k<false, false>), dim3(cus), dim3(512), 0, st, sk, iters);
    return amct::hip_status();
}

extern "C" int amct_copy_bytes(const void* src, void* dst, int64_t nbytes, amct_stream_t stream) {
    if (nbytes < 0 || (nbytes != 0 && (!src || !dst))) return AMCT_E_BADARG;
    if (nbytes % 16 != 0 || !amct::aligned16(src) || !amct::aligned16(dst)) return AMCT_E_ALIGN;
    const int64_t nvec = nbytes / 16;
    if (nvec == 0) return AMCT_OK;
    const int64_t nb = (nvec + amct::kBlock * 4 - 1) / (amct::kBlock * 4);
    hipLaunchKernelGGL(amct::copy_k, dim3((unsigned)nb), dim3(amct::kBlock), 0, (hipStream_t)stream,
                       (const uint4*)src, (uint4*)dst, nvec);
    return amct::hip_status();
}
