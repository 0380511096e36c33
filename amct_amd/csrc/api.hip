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
}  // namespace amct

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
