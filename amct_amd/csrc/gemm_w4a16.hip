// K7: W4A16 Linear.  out[m,n] = bf16( sum_k x'[m,k] * wdq[n,k] + bias[n] ), fp32 accumulate,
//   x'  = bf16(x * smooth[k])                         (weight_npu_quant_module.py:113-114)
//   wdq = bf16((u[n,k] - zero[n,k/g]) * scale[n,k/g]) (the operator called at :116-117)
// wq holds u = code + 8 as nibbles, even k in the low nibble.
//
//   large-tile kernel (M >= 256): 256x256 block tile, 8 waves, activations direct-to-LDS, packed weights
//                   fetched by asm loads four steps ahead, dequantised one step ahead into LDS.
//   tile kernel   : 128x128 block tile, BK = 64, bf16 MFMA 32x32x16; the weight tile is dequantised on its
//                   way from global memory to LDS (64 < M < 256 and shapes the large-tile kernel does not take).
//   decode kernels (M <= 16 with the activations staged in LDS, M <= 64 straight from L2): the weight is
//                   streamed once, dequantised in registers, bf16 MFMA 16x16x32, split-K over the waves.
//   general kernel: any shape, one output per thread.
// Dequantisation everywhere: byte-wise nibble split, v_cvt_f32_ubyteN, one fma per element
// ((u - z) * s == fma(u, s, -z*s) exactly), one v_cvt_pk_bf16_f32 per pair.
#include <type_traits>

#include "amct_common.h"
#include "gemm_plan.h"

namespace amct {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

struct W4A16Args {
    const uint16_t* x;
    const uint16_t* smooth;
    const uint8_t* wq;
    const void* scales;
    const uint8_t* zeros;
    const float* bias;
    uint16_t* out;
    int64_t M, N, K;
    int group;
    int scale_dtype;
    uint32_t group_magic;                            // floor(2^32 / group) + 1: k / group == mulhi(k, magic) for k, group < 2^16
    float* part;                                     // split-K launches (gridDim.z > 1): fp32 partial sums [gridDim.z, M, N]
};

AMCT_DEV float load_scale(const W4A16Args& a, int64_t i) {
    const uint16_t h = reinterpret_cast<const uint16_t*>(a.scales)[i];
    return a.scale_dtype == AMCT_F16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}

typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
// one v_cvt_pk_bf16_f32 for the pair (round-half-even); converting the halves separately costs four
// instructions instead
AMCT_DEV uint32_t pack_bf16x2(float lo, float hi) {
    const v2f f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2bf));
}

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
// the same for fp16: one v_cvt_pk_f16_f32
AMCT_DEV uint32_t pack_f16x2(float lo, float hi) {
    const v2f f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, v2h));
}
template <bool AF16> AMCT_DEV uint32_t pack_act2(float lo, float hi) { return AF16 ? pack_f16x2(lo, hi) : pack_bf16x2(lo, hi); }

// 8 signed bytes (two words) -> 8 values of (q - offset) * s in the activation type: the bytes as q + 128 (one
// v_cvt_f32_ubyteN each), z = offset + 128, one fma(u, s, -z s) per weight, as the other int8 weight-only kernels do
template <bool AF16>
AMCT_DEV uint4 dequant8_i8(uint32_t w0, uint32_t w1, float s, float nzs) {
    w0 ^= 0x80808080u;
    w1 ^= 0x80808080u;
    asm("" : "+v"(w0), "+v"(w1));
    float e[8];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        e[b] = __builtin_fmaf((float)((w0 >> (8 * b)) & 0xFFu), s, nzs);
        e[4 + b] = __builtin_fmaf((float)((w1 >> (8 * b)) & 0xFFu), s, nzs);
    }
    return make_uint4(pack_act2<AF16>(e[0], e[1]), pack_act2<AF16>(e[2], e[3]), pack_act2<AF16>(e[4], e[5]), pack_act2<AF16>(e[6], e[7]));
}

// 8 nibbles of `w` (element j in bits 4j..4j+3) -> 8 values of (u - z) * s in the activation type, as 4 packed dwords
template <bool AF16 = false>
AMCT_DEV uint4 dequant8(uint32_t w, float s, float nzs) {
    uint32_t lo = w & 0x0F0F0F0Fu;                  // elements 0,2,4,6 in bytes 0..3
    uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;           // elements 1,3,5,7
    // opaque to the optimiser: otherwise it rewrites the byte extraction below as one bit-field extract
    // per nibble followed by a conversion, two instructions per element instead of v_cvt_f32_ubyteN alone
    asm("" : "+v"(lo));
    asm("" : "+v"(hi));
    uint32_t o[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const float e0 = (float)((lo >> (8 * b)) & 0xFFu);
        const float e1 = (float)((hi >> (8 * b)) & 0xFFu);
        o[b] = pack_act2<AF16>(__builtin_fmaf(e0, s, nzs), __builtin_fmaf(e1, s, nzs));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// 8 bf16 activations times 8 bf16 smooth factors, each product rounded to bf16
AMCT_DEV uint4 smooth8(const uint4& x, const uint4& c) {
    const uint32_t xs[4] = {x.x, x.y, x.z, x.w}, cs[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(xs[i] << 16) * __uint_as_float(cs[i] << 16);
        const float hi = __uint_as_float(xs[i] & 0xFFFF0000u) * __uint_as_float(cs[i] & 0xFFFF0000u);
        o[i] = pack_bf16x2(lo, hi);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// ---------------------------------------------------------------------------
// tile kernel
// ---------------------------------------------------------------------------
constexpr int kTM = 128, kTN = 128, kTK = 64;       // BK in elements
constexpr int kTRow = kTK * 2 + 16;                 // bytes per padded LDS row of bf16

__global__ __launch_bounds__(kBlock) void w4a16_tile(W4A16Args a) {
    __shared__ __attribute__((aligned(16))) uint8_t As[2][kTM * kTRow];
    __shared__ __attribute__((aligned(16))) uint8_t Bs[2][kTN * kTRow];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * kTM, n0 = (int64_t)blockIdx.x * kTN;
    const int a_row = tid >> 3, a_chunk = tid & 7;              // activation tile: 8 chunks of 8 bf16 per row
    const int b_row = tid >> 1, b_half = tid & 1;               // weight tile: 2 chunks of 32 nibbles per row
    const int nsteps = (int)(a.K / kTK);
    const int64_t G = a.K / a.group;
    const int64_t wrow = (n0 + b_row < a.N) ? n0 + b_row : a.N - 1;

    uint4 ra[4], rw, rc;
    float s_cur = 0.f, nzs_cur = 0.f;
    auto load_global = [&](int step) {
        const int64_t k = (int64_t)step * kTK;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t m = m0 + a_row + 32 * i;
            ra[i] = ldg16(a.x + (m < a.M ? m : a.M - 1) * a.K + k + a_chunk * 8);
        }
        if (a.smooth) rc = ldg16(a.smooth + k + a_chunk * 8);
        const int64_t kw = k + b_half * 32;
        rw = ldg16(a.wq + wrow * (a.K / 2) + kw / 2);
        const int64_t gi = wrow * G + kw / a.group;
        s_cur = load_scale(a, gi);
        nzs_cur = -((float)a.zeros[gi] * s_cur);
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint4 v = a.smooth ? smooth8(ra[i], rc) : ra[i];
            *reinterpret_cast<uint4*>(&As[buf][(a_row + 32 * i) * kTRow + a_chunk * 16]) = v;
        }
        const uint32_t ws[4] = {rw.x, rw.y, rw.z, rw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<uint4*>(&Bs[buf][b_row * kTRow + b_half * 64 + j * 16]) = dequant8(ws[j], s_cur, nzs_cur);
    };

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    load_global(0);
    store_lds(0);
    __syncthreads();
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
    for (int step = 0; step < nsteps; ++step) {
        const int cur = step & 1;
        if (step + 1 < nsteps) load_global(step + 1);
#pragma unroll
        for (int ks = 0; ks < kTK / 16; ++ks) {
            v8bf fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const v8bf*>(&As[cur][(wm * 64 + i * 32 + frag_row) * kTRow + ks * 32 + frag_k]);
                fb[i] = *reinterpret_cast<const v8bf*>(&Bs[cur][(wn * 64 + i * 32 + frag_row) * kTRow + ks * 32 + frag_k]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (step + 1 < nsteps) store_lds(cur ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
        if (n >= a.N) continue;
        const float b = a.bias ? a.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < a.M) {
                    float v = acc[i][j][r];
                    if (a.bias) v = v + b;
                    a.out[m * a.N + n] = (uint16_t)f32_to_bf16_bits(v);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// large-tile kernel: 256x256 block tile, 8 waves (2 x 4) of 128x64, BK = 32 elements (64-byte rows of
// bf16), four LDS stages.  The activation tile arrives by direct global->LDS loads; the weight tile is
// fetched as packed nibbles into registers four K-steps ahead (8 bytes = 16 weights per thread and
// step), dequantised and written to its LDS stage one step before use.  All global loads and their
// s_waitcnt are inline asm so that the compiler never drains the queue of direct-to-LDS loads; a load
// issued in iteration t is guaranteed complete at the wait of iteration t+3 because the counter
// retires in order and every iteration issues the same number of operations.
// LDS layout as in the int8 kernel: unpadded [row][64 B], 16-byte chunk c of row r at c ^ ((r >> 2) & 3).
// ---------------------------------------------------------------------------
constexpr int kQK = 32;                                            // elements per K-step
constexpr int kQRow = 64;                                          // bytes per LDS row
constexpr int kQM = 256, kQN = 256, kQStages = 4, kQThreads = 512;
constexpr int kQStageBytes = (kQM + kQN) * kQRow;                  // 32 KiB
constexpr int kQPPW = (kQM / 16) / 8;                              // activation pieces per wave: 2
template <bool SMOOTH> constexpr int kQOps = kQPPW + 3 + (SMOOTH ? 1 : 0);   // vm operations per thread and iteration

AMCT_DEV void dma16(uint32_t lds_addr, const void* gptr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(gptr) : "memory");
}
AMCT_DEV void gload16(u4v& dst, const void* p) { asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory"); }
AMCT_DEV void gload8(uint64_t& dst, const void* p) { asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(dst) : "v"(p) : "memory"); }
AMCT_DEV void gload_u16(uint32_t& dst, const void* p) { asm volatile("global_load_ushort %0, %1, off" : "=v"(dst) : "v"(p) : "memory"); }
AMCT_DEV void gload_u8(uint32_t& dst, const void* p) { asm volatile("global_load_ubyte %0, %1, off" : "=v"(dst) : "v"(p) : "memory"); }

template <bool SMOOTH>
__global__ __launch_bounds__(kQThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void w4a16_tile_dma(W4A16Args a) {
    constexpr int OPS = kQOps<SMOOTH>;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[kQStages * kQStageBytes];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;
    const int64_t m0 = (int64_t)blockIdx.y * kQM, n0 = (int64_t)blockIdx.x * kQN;
    const int nsteps = (int)(a.K / kQK);
    const int last = nsteps - 1;
    const int64_t G = a.K / a.group;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

    // activation pieces of this wave (16 rows x 64 B each)
    const uint16_t* gp[kQPPW];
    const uint16_t* smp = nullptr;                                 // smooth factors of this lane's chunk
    {
        const int rin = lane >> 2;
        const int lc = (lane & 3) ^ ((rin >> 2) & 3);
        if constexpr (SMOOTH) smp = a.smooth + lc * 8;
#pragma unroll
        for (int j = 0; j < kQPPW; ++j) {
            const int64_t r = m0 + (wave * kQPPW + j) * 16 + rin;
            gp[j] = a.x + (r < a.M ? r : a.M - 1) * a.K + lc * 8;
        }
    }
    // weight row of this thread: row tid/2, 16 weights (8 bytes) per step, which half from tid%2
    const int brow = tid >> 1, bhalf = tid & 1;
    const int64_t wrow = (n0 + brow < a.N) ? n0 + brow : a.N - 1;
    const uint8_t* wp = a.wq + wrow * (a.K / 2) + bhalf * 8;
    const int bphys0 = (bhalf * 2) ^ ((brow >> 2) & 3), bphys1 = (bhalf * 2 + 1) ^ ((brow >> 2) & 3);
    const int boff0 = kQM * kQRow + brow * kQRow + bphys0 * 16, boff1 = kQM * kQRow + brow * kQRow + bphys1 * 16;
    const int sbytes = 2;
    const uint8_t* sp = reinterpret_cast<const uint8_t*>(a.scales) + wrow * G * sbytes;
    const uint8_t* zp = a.zeros + wrow * G;

    uint64_t wreg[4];
    uint32_t sreg[4], zreg[4];
    u4v mreg[4];
    auto issue = [&](int slot, int stage, int step) {              // the loads of K-step `step`
        const int st = step < last ? step : last;
        const uint32_t k = (uint32_t)st * kQK;
        // k / group without a division (k, group < 2^16); group % 32 == 0 keeps both halves of a step in one group
        const uint32_t gi = __umulhi(k, a.group_magic);
        gload8(wreg[slot], wp + k / 2);
        gload_u16(sreg[slot], sp + gi * sbytes);
        gload_u8(zreg[slot], zp + gi);
        if constexpr (SMOOTH) gload16(mreg[slot], smp + k);
        const uint32_t base = __builtin_amdgcn_readfirstlane(lds0 + stage * kQStageBytes + wave * kQPPW * 1024);
#pragma unroll
        for (int j = 0; j < kQPPW; ++j) dma16(base + j * 1024, gp[j] + k);
    };
    auto write_b = [&](int slot, int stage) {                      // dequantise 16 weights into LDS
        const float sc = a.scale_dtype == AMCT_F16 ? f16_bits_to_f32(sreg[slot]) : bf16_bits_to_f32(sreg[slot]);
        const float nzs = -((float)zreg[slot] * sc);
        uint8_t* st = smem + stage * kQStageBytes;
        *reinterpret_cast<uint4*>(st + boff0) = dequant8((uint32_t)wreg[slot], sc, nzs);
        *reinterpret_cast<uint4*>(st + boff1) = dequant8((uint32_t)(wreg[slot] >> 32), sc, nzs);
    };
    // x' = bf16(x * smooth) in place on the pieces this wave fetched itself (lane l owns bytes
    // 16 l .. 16 l + 15 of each piece).  Split in two so that the LDS read latency is not exposed: the
    // raw chunks are read in the second half of iteration t, multiplied and written back in the first
    // half of iteration t+1, one barrier before the stage is consumed.
    uint4 araw[kQPPW];
    auto smooth_read = [&](int stage) {
        const uint8_t* st = smem + stage * kQStageBytes + wave * kQPPW * 1024 + lane * 16;
#pragma unroll
        for (int j = 0; j < kQPPW; ++j) araw[j] = *reinterpret_cast<const uint4*>(st + j * 1024);
    };
    auto smooth_write = [&](int slot, int stage) {
        uint8_t* st = smem + stage * kQStageBytes + wave * kQPPW * 1024 + lane * 16;
        const uint4 c = make_uint4(mreg[slot].x, mreg[slot].y, mreg[slot].z, mreg[slot].w);
#pragma unroll
        for (int j = 0; j < kQPPW; ++j) *reinterpret_cast<uint4*>(st + j * 1024) = smooth8(araw[j], c);
    };
    // wait until at most N vm operations are outstanding and all LDS operations are done; the slot's
    // registers are tied to the statement so that their uses stay behind it
#define AMCT_WAIT_SLOT(N, slot) \
    asm volatile("s_waitcnt vmcnt(%3) lgkmcnt(0)" : "+v"(wreg[slot]), "+v"(sreg[slot]), "+v"(zreg[slot]) : "n"(N) : "memory")
#define AMCT_TIE_SMOOTH(slot) asm volatile("" : "+v"(mreg[slot]) : : "memory")

    int offA[2], offB[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int r = lane & 31;
        const int phys = (ks * 2 + (lane >> 5)) ^ ((r >> 2) & 3);
        offA[ks] = (wm * 128 + r) * kQRow + phys * 16;
        offB[ks] = kQM * kQRow + (wn * 64 + r) * kQRow + phys * 16;
    }
    v16f acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    auto read_frags = [&](int stage, int ks, v8bf (&fa)[4], v8bf (&fb)[2]) {
        const uint8_t* st = smem + stage * kQStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const v8bf*>(st + offA[ks] + i * 32 * kQRow);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = *reinterpret_cast<const v8bf*>(st + offB[ks] + j * 32 * kQRow);
    };
    auto mfma_half = [&](const v8bf (&fa)[4], const v8bf (&fb)[2]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };

    // prologue: the loads of steps 0..3; step 0 must have landed before its weights are dequantised
#pragma unroll
    for (int s = 0; s < 4; ++s) issue(s, s, s);
    if constexpr (SMOOTH) {
        AMCT_WAIT_SLOT(2 * OPS, 0);                                 // steps 0 and 1 have landed
        AMCT_TIE_SMOOTH(0);
        AMCT_TIE_SMOOTH(1);
        smooth_read(0);
        smooth_write(0, 0);
        smooth_read(1);                                             // written back in iteration 0
    } else {
        AMCT_WAIT_SLOT(3 * OPS, 0);
    }
    write_b(0, 0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v8bf fa0[4], fb0[2], fa1[4], fb1[2];
    read_frags(0, 0, fa0, fb0);

    // iteration t (stage/slot U = t % 4): second half of the fragments of step t, MFMAs of the first
    // half; wait for the loads of step t+1; dequantise the weights of step t+1 into their stage;
    // barrier; issue the loads of step t+4 into stage/slot U (both free now); first half of step t+1.
    // The dequantisation (and, with smoothing, the in-place multiply of the activations of step t+2)
    // sits in the same scheduling region as 8 MFMAs and is interleaved with them instruction by
    // instruction: a wave issues in order, so VALU work placed after a run of MFMAs would only start
    // once the matrix pipe has accepted all of them.
#define AMCT_INTERLEAVE()                                                   \
    _Pragma("unroll") for (int q_ = 0; q_ < 8; ++q_) {                      \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); /* 1 MFMA  */     \
        __builtin_amdgcn_sched_group_barrier(0x002, 8, 0); /* 8 VALU  */     \
        __builtin_amdgcn_sched_group_barrier(0x080, 1, 0); /* 1 DS    */     \
    }
#define AMCT_ITER(U, NX, NX2, step)                      \
    {                                                    \
        AMCT_WAIT_SLOT(2 * OPS, NX);                     \
        read_frags(U, 1, fa1, fb1);                      \
        write_b(NX, NX);                                 \
        if constexpr (SMOOTH) smooth_write(NX, NX);      \
        mfma_half(fa0, fb0);                             \
        AMCT_INTERLEAVE()                                \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); \
        __builtin_amdgcn_s_barrier();                    \
        asm volatile("" ::: "memory");                   \
        issue(U, U, (step) + 4);                         \
        if constexpr (SMOOTH) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(mreg[NX2]) : "n"(2 * OPS) : "memory"); \
        read_frags(NX, 0, fa0, fb0);                     \
        if constexpr (SMOOTH) smooth_read(NX2);          \
        mfma_half(fa1, fb1);                             \
        AMCT_INTERLEAVE()                                \
    }
    for (int step = 0; step < nsteps; step += 4) {
        AMCT_ITER(0, 1, 2, step)
        AMCT_ITER(1, 2, 3, step + 1)
        AMCT_ITER(2, 3, 0, step + 2)
        AMCT_ITER(3, 0, 1, step + 3)
    }
#undef AMCT_ITER
#undef AMCT_INTERLEAVE
#undef AMCT_WAIT_SLOT
#undef AMCT_TIE_SMOOTH
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // epilogue: + bias, narrow to bf16, transpose through a per-wave LDS patch, 16-byte stores
    constexpr int kPatchRow = 64 * 2 + 16;
    uint8_t* patch = smem + wave * 16384;
    float bs[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
        bs[j] = a.bias ? a.bias[n < a.N ? n : a.N - 1] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t mbase = m0 + wm * 128 + i * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int prow = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float v = acc[i][j][r];
                if (a.bias) v = v + bs[j];
                *reinterpret_cast<uint16_t*>(patch + prow * kPatchRow + (j * 32 + (lane & 31)) * 2) = (uint16_t)f32_to_bf16_bits(v);
            }
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int prow = it * 8 + (lane >> 3);
            const int chunk = lane & 7;
            const uint4 v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * 64 + chunk * 8;
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * 2, v);
        }
    }
}

// ---------------------------------------------------------------------------
// wide tile kernels (K % 128 == 0, group % 64 == 0, activations already smoothed): block tile (32*TI*WM) x
// (32*TJ*WN), WM x WN waves, STAGES LDS stages of 64 elements of K (128-byte rows: a direct-to-LDS load covers
// whole cache lines, one barrier per 64 elements).  256x256 with 8 waves of 128x64 and two stages for large M;
// 128x128 (4 waves of 64x64) and 128x256 (8 waves of 64x64) with three stages for medium M, where a short step
// would expose the load latency that two stages cover for the large tile.
//   activations : direct global->LDS loads issued by the upper half of the waves (one per SIMD) in one burst
//                 right after the barrier that frees the stage; a wave stalls at such a load while the memory
//                 pipeline is busy and the other wave of its SIMD keeps the matrix pipe fed meanwhile;
//   weights     : 16 bytes (32 nibbles) per thread and step into registers two steps ahead (two register slots,
//                 the loop is unrolled by two; the LDS stage index is a run-time value), with the scale and
//                 zero-point of their group; dequantised in the shadow of the MFMAs of the first two k-slices
//                 of the step before and written to the next LDS stage in MFMA operand order.
// The issue order is pinned: sched_group_barrier interleaves MFMA / VALU / LDS inside a k-slice, scheduling
// barriers separate the slices, and the MFMAs of the slices before the barrier are issued BEFORE the wait
// (left alone, the optimiser moves them behind the barrier and the matrix pipe idles while the waves meet).
// All global loads and their s_waitcnt are inline asm with SGPR bases and constant 32-bit lane offsets; the
// counter retires in order and every iteration issues the same number of operations per wave.
// LDS layout: unpadded [row][128 B], 16-byte chunk c of row r at c ^ ((r >> 1) & 7).
// ---------------------------------------------------------------------------
constexpr int kWK = 64;                                            // elements of K per stage
constexpr int kWRow = 128;                                         // bytes per LDS row
constexpr int kSpecThreads = 768;                                  // 4 matrix waves + 8 data-movement waves
constexpr int kSpecMaxG = 32;                                      // groups per weight row the specialised kernel's factor table holds

AMCT_DEV void dma16s(uint32_t lds_addr, const void* sbase, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
AMCT_DEV void gload16s(u4v& dst, const void* sbase, uint32_t voff) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
AMCT_DEV void gload16s(u2v& dst, const void* sbase, uint32_t voff) {   // 8 bytes: the quarter-row share of a step
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
AMCT_DEV void gload_u16s(uint32_t& dst, const void* sbase, uint32_t voff) {
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
AMCT_DEV void gload_u8s(uint32_t& dst, const void* sbase, uint32_t voff) {
    asm volatile("global_load_ubyte %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
template <int N> AMCT_DEV void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

// STAGES: LDS stages of the activation tile (filled by direct-to-LDS loads; a third stage gives a load two steps to
// land); SB: stages of the dequantised weight tile (written by the waves themselves one step ahead: two suffice)
template <int WM, int WN, int TI, int TJ, int STAGES, int SB = STAGES>
struct WideTile {
    static constexpr int kLM = 32 * TI * WM, kLN = 32 * TJ * WN, kWaves = WM * WN, kThreads = kWaves * 64;
    static constexpr int kABytes = kLM * kWRow, kBBytes = kLN * kWRow;     // one stage of each operand
    static constexpr int kBBase = STAGES * kABytes;                        // the weight stages follow the activation stages
    static constexpr int kLW = kWaves / 2;                         // waves that issue the direct-to-LDS loads
    static constexpr int kNA = (kLM * kWRow / 1024) / kLW;         // activation pieces (8 rows x 128 B) per loading wave
    static constexpr int kEpi = kWaves * 16384;
    static constexpr int kRing = STAGES * kABytes + SB * kBBytes;
    static constexpr int kSmem = kRing > kEpi ? kRing : kEpi;
    static constexpr int kQ = kThreads / kLN;                     // threads per weight row of the tile
    static constexpr int kBC = 8 / kQ;                             // 8-weight chunks a thread dequantises per step
    static_assert(kThreads == 2 * kLN || kThreads == 4 * kLN, "every thread dequantises a half or a quarter of a weight row of the tile per step");
    static_assert((kLM * kWRow / 1024) % kLW == 0 && kSmem <= 160 * 1024, "tile shape");
    static_assert(kNA < 64, "vmcnt range");
};

template <bool SF16, int WM, int WN, int TI, int TJ, int STAGES, int SB = STAGES, bool AF16 = false>
AMCT_DEV void w4a16_wide_body(const W4A16Args& a, uint8_t* smem, const int64_t m0, const int64_t n0) {
    using Sh = WideTile<WM, WN, TI, TJ, STAGES, SB>;
    constexpr int kABytes = Sh::kABytes, kBBytes = Sh::kBBytes, kBBase = Sh::kBBase;
    constexpr int kWaves = Sh::kWaves, kLW = Sh::kLW, kNA = Sh::kNA;
    constexpr int kNM = TI * TJ, kNR = TI + TJ;                    // MFMAs and fragment reads per k-slice
    constexpr int kRPM = (kNR + kNM - 1) / kNM;                    // fragment reads issued behind each MFMA
    static_assert((STAGES == 2 || STAGES == 3) && (SB == 2 || SB == 3) && SB <= STAGES, "2 or 3 stages");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int nsteps = (int)(a.K / kWK);
    const int last = nsteps - 1;
    const uint32_t G = (uint32_t)(a.K / a.group);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
    auto swz = [](int r) { return (r >> 1) & 7; };

    // activation pieces (8 rows x 128 B) of the loading waves
    const bool loader = wave >= kWaves - kLW;
    const int lw = loader ? wave - (kWaves - kLW) : 0;
    uint32_t goff[kNA];
    {
        const int rin = lane >> 3, pc = lane & 7;
#pragma unroll
        for (int j = 0; j < kNA; ++j) {
            const int lr = (lw * kNA + j) * 8 + rin;
            const int64_t r = m0 + lr < a.M ? m0 + lr : a.M - 1;
            goff[j] = (uint32_t)((r * a.K + (pc ^ swz(lr)) * 8) * 2);
        }
    }
    auto dma_a = [&](int stg, int step) {
        if (loader) {
            const int st = step < last ? step : last;
#pragma unroll
            for (int j = 0; j < kNA; ++j)
                dma16s(lds0 + stg * kABytes + (lw * kNA + j) * 1024, a.x + (int64_t)st * kWK, goff[j]);
        }
    };
    // weight row of this thread: row tid/kQ of the tile, 8*kBC weights (4*kBC bytes) per step, which part from tid%kQ
    constexpr int kQ = Sh::kQ, kBC = Sh::kBC;
    const int brow = tid / kQ, bpart = tid % kQ;
    const int64_t wrow = (n0 + brow < a.N) ? n0 + brow : a.N - 1;
    const uint32_t woff = (uint32_t)(wrow * (a.K / 2) + bpart * (4 * kBC));
    const uint32_t soff = (uint32_t)(wrow * G * 2), zoff = (uint32_t)(wrow * G);
    int bdst[kBC];
#pragma unroll
    for (int c = 0; c < kBC; ++c) bdst[c] = kBBase + brow * kWRow + ((kBC * bpart + c) ^ swz(brow)) * 16;

    typename std::conditional<kBC == 4, u4v, u2v>::type wreg[2];
    uint32_t sreg[2], zreg[2];
    auto issue_b = [&](int slot, int step) {                       // the weight loads of K-step `step`
        const int st = step < last ? step : last;
        const uint32_t k = (uint32_t)st * kWK;
        const uint32_t gi = __umulhi(k, a.group_magic);             // k / group (k, group < 2^16); group % 64 == 0
        gload16s(wreg[slot], a.wq + k / 2, woff);
        gload_u16s(sreg[slot], reinterpret_cast<const uint8_t*>(a.scales) + gi * 2, soff);
        gload_u8s(zreg[slot], a.zeros + gi, zoff);
    };
    float sc = 0.f, nzs = 0.f;
    auto factors = [&](int slot) {
        sc = SF16 ? f16_bits_to_f32(sreg[slot]) : bf16_bits_to_f32(sreg[slot]);
        nzs = -((float)zreg[slot] * sc);
    };
    auto write_b = [&](int slot, int stg, int c) {                 // dequantise 8 weights into LDS
        *reinterpret_cast<uint4*>(smem + stg * kBBytes + bdst[c]) = dequant8<AF16>(wreg[slot][c], sc, nzs);
    };
    // Wait until the weight loads of the previous iteration and the activation loads issued STAGES-1 iterations ago
    // have landed and this wave's LDS operations are done.  An iteration issues its 3 weight loads in the middle of the
    // step, as soon as their register slot has been dequantised (when the memory pipeline is idle: issued right after
    // the barrier they queued behind the loading waves' burst and both waves of a SIMD stood still), and, in a loading
    // wave, kNA direct-to-LDS loads right after the barrier.  The youngest weight loads may stay in flight, and with three
    // stages the youngest activation loads too, hence the wave-uniform choice of the count.  The slot's registers are tied to a statement behind the wait so that
    // their uses (and any copies the register allocator makes) stay behind it.
    auto wait_older = [&]() {
        if constexpr (STAGES == 2) {
            wait_vm<3>();
        } else {
            if (loader) wait_vm<kNA + 3>();
            else wait_vm<3>();
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
#define AMCT_TIE_SLOT(slot) asm volatile("" : "+v"(wreg[slot]), "+v"(sreg[slot]), "+v"(zreg[slot]) : : "memory")

    int offA[4], offB[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int r = lane & 31;
        const int phys = (ks * 2 + (lane >> 5)) ^ swz(r);
        offA[ks] = (wm * 32 * TI + r) * kWRow + phys * 16;
        offB[ks] = kBBase + (wn * 32 * TJ + r) * kWRow + phys * 16;
    }
    v16f acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // fragment q in the order the MFMAs need them: A0, B0, B1, .., A1, A2, ..
    auto read_one = [&](int sa, int sb, int ks, int q, v8bf (&fa)[TI], v8bf (&fb)[TJ]) {
        const uint8_t* pa = smem + sa * kABytes;
        const uint8_t* pb = smem + sb * kBBytes;
        if (q == 0) fa[0] = *reinterpret_cast<const v8bf*>(pa + offA[ks]);
        else if (q <= TJ) fb[q - 1] = *reinterpret_cast<const v8bf*>(pb + offB[ks] + (q - 1) * 32 * kWRow);
        else fa[q - TJ] = *reinterpret_cast<const v8bf*>(pa + offA[ks] + (q - TJ) * 32 * kWRow);
    };
    auto mfma_one = [&](int m, const v8bf (&fa)[TI], const v8bf (&fb)[TJ]) {
        const int i = m / TJ, j = m % TJ;
        if constexpr (AF16) {
            typedef _Float16 v8h __attribute__((ext_vector_type(8)));
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, fa[i]), __builtin_bit_cast(v8h, fb[j]), acc[i][j], 0, 0, 0);
        } else {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    // prologue: B(0), B(1) and A(0 .. STAGES-2); once B(0) is dequantised into stage 0 its slot takes B(2), and
    // A(STAGES-1) follows (weights first, as in the loop)
    v8bf fa[2][TI], fb[2][TJ];
    issue_b(0, 0);
    issue_b(1, 1);
#pragma unroll
    for (int j = 0; j < STAGES - 1; ++j) dma_a(j, j);
    wait_vm<0>();
    AMCT_TIE_SLOT(0);
    AMCT_TIE_SLOT(1);
    factors(0);
#pragma unroll
    for (int c = 0; c < kBC; ++c) write_b(0, 0, c);
    issue_b(0, 2);
    dma_a(STAGES - 1, STAGES - 1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int q = 0; q < kNR; ++q) read_one(0, 0, 0, q, fa[0], fb[0]);

    // iteration s (LDS stage cur, the next one nxt; register slot SL holds B(s+1), landed; the other slot B(s+2)):
    //   k-slices 0, 1 : MFMAs, fragment reads of the next slice, dequantisation of B(s+1) into stage nxt
    //   loads         : B(s+3) into slot SL (its old content is in LDS now)
    //   k-slice 2     : MFMAs, fragment reads of slice 3
    //   wait (A(s+1) and B(s+2) have landed; own LDS operations done), barrier: stage cur is free, nxt complete
    //   loads         : A(s+STAGES) into stage cur (loading waves)
    //   k-slice 3     : MFMAs, fragment reads of slice 0 of stage nxt
    int cur = 0, nxt = 1;                                           // activation stages
    int curb = 0, nxtb = 1;                                         // weight stages
#define AMCT_WSLICE_DQ(CUR, NXT, SL, KS)                                                 \
    {                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                             \
        _Pragma("unroll") for (int m_ = 0; m_ < kNM; ++m_) mfma_one(m_, fa[(KS) & 1], fb[(KS) & 1]); \
        _Pragma("unroll") for (int q_ = 0; q_ < kNR; ++q_) read_one(CUR, curb, (KS) + 1, q_, fa[((KS) + 1) & 1], fb[((KS) + 1) & 1]); \
        _Pragma("unroll") for (int c_ = 0; c_ < kBC / 2; ++c_) write_b(SL, nxtb, (kBC / 2) * (KS) + c_); \
        _Pragma("unroll") for (int g_ = 0; g_ < kNM; ++g_) {                           \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                      /* 1 MFMA */ \
            __builtin_amdgcn_sched_group_barrier(0x002, (14 * kBC + kNM - 1) / kNM, 0); /* VALU */ \
            __builtin_amdgcn_sched_group_barrier(0x080, (kNR + kBC / 2 + kNM - 1) / kNM, 0); /* DS */ \
        }                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                             \
    }
#define AMCT_WSLICE_PIN(STG, STGB, KSREAD, KS)                                         \
    {                                                                                  \
        _Pragma("unroll") for (int m_ = 0; m_ < kNM; ++m_) {                           \
            mfma_one(m_, fa[(KS) & 1], fb[(KS) & 1]);                                  \
            __builtin_amdgcn_sched_barrier(0);                                         \
            _Pragma("unroll") for (int q_ = m_ * kRPM; q_ < (m_ + 1) * kRPM && q_ < kNR; ++q_) { \
                read_one(STG, STGB, KSREAD, q_, fa[((KS) + 1) & 1], fb[((KS) + 1) & 1]); \
                __builtin_amdgcn_sched_barrier(0);                                     \
            }                                                                          \
        }                                                                              \
    }
#define AMCT_WITER(SL, step)                                                           \
    {                                                                                  \
        AMCT_TIE_SLOT(SL);                                                             \
        factors(SL);                                                                   \
        AMCT_WSLICE_DQ(cur, nxt, SL, 0)                                                \
        AMCT_WSLICE_DQ(cur, nxt, SL, 1)                                                \
        issue_b(SL, (step) + 3);                                                       \
        __builtin_amdgcn_sched_barrier(0);                                             \
        AMCT_WSLICE_PIN(cur, curb, 3, 2)                                               \
        wait_older();                                                                  \
        __builtin_amdgcn_s_barrier();                                                  \
        asm volatile("" ::: "memory");                                                 \
        __builtin_amdgcn_sched_barrier(0);                                             \
        dma_a(cur, (step) + STAGES);                                                   \
        __builtin_amdgcn_sched_barrier(0);                                             \
        AMCT_WSLICE_PIN(nxt, nxtb, 0, 3)                                               \
        cur = nxt;                                                                     \
        nxt = nxt + 1 == STAGES ? 0 : nxt + 1;                                         \
        curb = nxtb;                                                                   \
        nxtb = nxtb + 1 == SB ? 0 : nxtb + 1;                                          \
    }
    for (int step = 0; step < nsteps; step += 2) {                  // K % 128 == 0: an even number of steps
        AMCT_WITER(1, step)
        AMCT_WITER(0, step + 1)
    }
#undef AMCT_WITER
#undef AMCT_WSLICE_PIN
#undef AMCT_WSLICE_DQ
#undef AMCT_TIE_SLOT
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // epilogue: + bias (or + (-0.0f), which returns the value bit for bit), narrow to bf16, transpose through a
    // per-wave LDS patch of 32 rows x 32*TJ columns, 16-byte stores of full rows
    constexpr int kPW = 32 * TJ;                                   // patch width in columns
    constexpr int kPatchRow = kPW * 2 + 16;
    constexpr int CPR = kPW * 2 / 16;                              // 16-byte chunks per patch row
    static_assert(32 * kPatchRow <= 16384 && (32 * CPR) % 64 == 0, "patch");
    uint8_t* patch = smem + wave * 16384;
    float bs[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int64_t n = n0 + wn * kPW + j * 32 + (lane & 31);
        bs[j] = a.bias ? a.bias[n < a.N ? n : a.N - 1] : -0.0f;
    }
    uint8_t* wbase = patch + 4 * (lane >> 5) * kPatchRow + (lane & 31) * 2;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int64_t mbase = m0 + wm * 32 * TI + i * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int prow0 = 8 * (r >> 2) + (r & 3);
#pragma unroll
            for (int j = 0; j < TJ; ++j)
                *reinterpret_cast<uint16_t*>(wbase + prow0 * kPatchRow + j * 64) = (uint16_t)(AF16 ? f32_to_f16_bits(acc[i][j][r] + bs[j]) : f32_to_bf16_bits(acc[i][j][r] + bs[j]));
        }
#pragma unroll
        for (int it = 0; it < 32 * CPR / 64; ++it) {
            const int idx = it * 64 + lane;                        // 16-byte chunk of the patch, row-major
            const int prow = idx / CPR, chunk = idx % CPR;
            const uint4 v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * kPW + chunk * 8;
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * 2, v);
        }
    }
}

template <bool SF16, int WM, int WN, int TI, int TJ, int STAGES, int SB = STAGES, bool AF16 = false>
AMCT_DEV void w4a16_wide_body16(const W4A16Args& a, uint8_t* smem, const int64_t m0, const int64_t n0) {
    using Sh = WideTile<WM, WN, TI, TJ, STAGES, SB>;
    constexpr int kABytes = Sh::kABytes, kBBytes = Sh::kBBytes, kBBase = Sh::kBBase;
    constexpr int kWaves = Sh::kWaves, kLW = Sh::kLW, kNA = Sh::kNA;
    // v_mfma_f32_16x16x32_bf16: a stage (64 elements of K) is two k-slices of 32; each is done in two units (the upper
    // and the lower half of the wave's 16-row tiles), so a stage is four units u = 2 * slice + half, as many as the
    // 32x32x16 form has k-slices, and the schedule below is that form's with units in the place of slices.
    constexpr int TA = TI;                                         // 16-row tiles per unit
    constexpr int TB = 2 * TJ;                                     // 16-column tiles of the wave
    constexpr int kNM = TA * TB;                                   // MFMAs per unit
    constexpr int kDqGap = kNM / (4 * (Sh::kBC / 2));              // a dequantisation piece behind every kDqGap-th MFMA
    static_assert(kDqGap >= 1 && Sh::kBC >= 2, "a dequantising unit takes kBC / 2 chunks of four pieces");
    static_assert(TA >= 2 && TA * 2 >= TB, "the unit must have room for its fragment reads");
    static_assert((STAGES == 2 || STAGES == 3) && (SB == 2 || SB == 3) && SB <= STAGES, "2 or 3 stages");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int nsteps = (int)(a.K / kWK);
    const int last = nsteps - 1;
    const uint32_t G = (uint32_t)(a.K / a.group);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
    auto swz = [](int r) { return (r >> 1) & 7; };

    // activation pieces (8 rows x 128 B) of the loading waves
    const bool loader = wave >= kWaves - kLW;
    const int lw = loader ? wave - (kWaves - kLW) : 0;
    uint32_t goff[kNA];
    {
        const int rin = lane >> 3, pc = lane & 7;
#pragma unroll
        for (int j = 0; j < kNA; ++j) {
            const int lr = (lw * kNA + j) * 8 + rin;
            const int64_t r = m0 + lr < a.M ? m0 + lr : a.M - 1;
            goff[j] = (uint32_t)((r * a.K + (pc ^ swz(lr)) * 8) * 2);
        }
    }
    auto dma_a = [&](int stg, int step) {
        if (loader) {
            const int st = step < last ? step : last;
#pragma unroll
            for (int j = 0; j < kNA; ++j)
                dma16s(lds0 + stg * kABytes + (lw * kNA + j) * 1024, a.x + (int64_t)st * kWK, goff[j]);
        }
    };
    // weight row of this thread: row tid/kQ of the tile, 8*kBC weights (4*kBC bytes) per step, which part from tid%kQ
    constexpr int kQ = Sh::kQ, kBC = Sh::kBC;
    const int brow = tid / kQ, bpart = tid % kQ;
    const int64_t wrow = (n0 + brow < a.N) ? n0 + brow : a.N - 1;
    const uint32_t woff = (uint32_t)(wrow * (a.K / 2) + bpart * (4 * kBC));
    const uint32_t soff = (uint32_t)(wrow * G * 2), zoff = (uint32_t)(wrow * G);
    int bdst[kBC];
#pragma unroll
    for (int c = 0; c < kBC; ++c) bdst[c] = kBBase + brow * kWRow + ((kBC * bpart + c) ^ swz(brow)) * 16;

    typename std::conditional<kBC == 4, u4v, u2v>::type wreg[2];
    uint32_t sreg[2], zreg[2];
    auto issue_b = [&](int slot, int step) {                       // the weight loads of K-step `step`
        const int st = step < last ? step : last;
        const uint32_t k = (uint32_t)st * kWK;
        const uint32_t gi = __umulhi(k, a.group_magic);             // k / group (k, group < 2^16); group % 64 == 0
        gload16s(wreg[slot], a.wq + k / 2, woff);
        gload_u16s(sreg[slot], reinterpret_cast<const uint8_t*>(a.scales) + gi * 2, soff);
        gload_u8s(zreg[slot], a.zeros + gi, zoff);
    };
    float sc = 0.f, nzs = 0.f;
    auto factors = [&](int slot) {
        sc = SF16 ? f16_bits_to_f32(sreg[slot]) : bf16_bits_to_f32(sreg[slot]);
        nzs = -((float)zreg[slot] * sc);
    };
    auto write_b = [&](int slot, int stg, int c) {                 // dequantise 8 weights into LDS
        *reinterpret_cast<uint4*>(smem + stg * kBBytes + bdst[c]) = dequant8<AF16>(wreg[slot][c], sc, nzs);
    };
    // Wait until the weight loads of the previous iteration and the activation loads issued STAGES-1 iterations ago
    // have landed and this wave's LDS operations are done.  An iteration issues its 3 weight loads in the middle of the
    // step, as soon as their register slot has been dequantised (when the memory pipeline is idle: issued right after
    // the barrier they queued behind the loading waves' burst and both waves of a SIMD stood still), and, in a loading
    // wave, kNA direct-to-LDS loads right after the barrier.  The youngest weight loads may stay in flight, and with three
    // stages the youngest activation loads too, hence the wave-uniform choice of the count.  The slot's registers are tied to a statement behind the wait so that
    // their uses (and any copies the register allocator makes) stay behind it.
    auto wait_older = [&]() {
        if constexpr (STAGES == 2) {
            wait_vm<3>();
        } else {
            if (loader) wait_vm<kNA + 3>();
            else wait_vm<3>();
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
#define AMCT_TIE_SLOT(slot) asm volatile("" : "+v"(wreg[slot]), "+v"(sreg[slot]), "+v"(zreg[slot]) : : "memory")

    // fragment of unit u: lane reads row (tile base + lane % 16), logical chunk 4 * slice + lane / 16
    int offA[4], offB[2];
    {
        const int r = lane & 15;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            offA[u] = (wm * 32 * TI + (u & 1) * 16 * TA + r) * kWRow + ((4 * (u >> 1) + (lane >> 4)) ^ swz(r)) * 16;
#pragma unroll
        for (int sl = 0; sl < 2; ++sl)
            offB[sl] = kBBase + (wn * 32 * TJ + r) * kWRow + ((4 * sl + (lane >> 4)) ^ swz(r)) * 16;
    }
    typedef float v4f __attribute__((ext_vector_type(4)));
    v4f acc[2 * TI][TB];
#pragma unroll
    for (int i = 0; i < 2 * TI; ++i)
#pragma unroll
        for (int j = 0; j < TB; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // Row fragments live in ONE set of registers: a unit walks its MFMAs row tile by row tile, and the fragment of a row
    // tile is loaded again (for the next unit) right behind the last MFMA that used it.  Column fragments are used by
    // every row tile of both units of a slice, so they alternate between two sets per slice.
    v8bf fa[TA], fb[2][TB];
    auto read_a = [&](int sa, int u, int i) {                       // u, i: compile-time in every use
        fa[i] = *reinterpret_cast<const v8bf*>(smem + sa * kABytes + offA[u] + i * 16 * kWRow);
    };
    auto read_b = [&](int sb, int sl, int j) {
        fb[sl & 1][j] = *reinterpret_cast<const v8bf*>(smem + sb * kBBytes + offB[sl] + j * 16 * kWRow);
    };
    auto mfma_one = [&](int u, int m) {
        const int i = m / TB, j = m % TB;
        if constexpr (AF16) {
            typedef _Float16 v8h __attribute__((ext_vector_type(8)));
            acc[(u & 1) * TA + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, fa[i]), __builtin_bit_cast(v8h, fb[(u >> 1) & 1][j]),
                                                                          acc[(u & 1) * TA + i][j], 0, 0, 0);
        } else {
            acc[(u & 1) * TA + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[(u >> 1) & 1][j], acc[(u & 1) * TA + i][j], 0, 0, 0);
        }
    };
    // dequantisation of 8 weights in four pieces of two, so that the pieces can sit between MFMAs
    uint32_t dq_lo = 0, dq_hi = 0, dq_o[4];
    auto dq_piece = [&](int slot, int c, int bb) {                  // c, bb: compile-time
        if (bb == 0) {
            dq_lo = wreg[slot][c] & 0x0F0F0F0Fu;                   // elements 0, 2, 4, 6 in bytes 0 .. 3
            dq_hi = (wreg[slot][c] >> 4) & 0x0F0F0F0Fu;            // elements 1, 3, 5, 7
            asm("" : "+v"(dq_lo));                                  // keeps the byte conversions below as v_cvt_f32_ubyteN
            asm("" : "+v"(dq_hi));
        }
        const float e0 = (float)((dq_lo >> (8 * bb)) & 0xFFu);
        const float e1 = (float)((dq_hi >> (8 * bb)) & 0xFFu);
        dq_o[bb] = pack_act2<AF16>(__builtin_fmaf(e0, sc, nzs), __builtin_fmaf(e1, sc, nzs));
    };
    auto dq_write = [&](int stg, int c) {
        *reinterpret_cast<uint4*>(smem + stg * kBBytes + bdst[c]) = make_uint4(dq_o[0], dq_o[1], dq_o[2], dq_o[3]);
    };

    // prologue: B(0), B(1) and A(0 .. STAGES-2); once B(0) is dequantised into stage 0 its slot takes B(2), and
    // A(STAGES-1) follows (weights first, as in the loop)
    issue_b(0, 0);
    issue_b(1, 1);
#pragma unroll
    for (int j = 0; j < STAGES - 1; ++j) dma_a(j, j);
    wait_vm<0>();
    AMCT_TIE_SLOT(0);
    AMCT_TIE_SLOT(1);
    factors(0);
#pragma unroll
    for (int c = 0; c < kBC; ++c) write_b(0, 0, c);
    issue_b(0, 2);
    dma_a(STAGES - 1, STAGES - 1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int q = 0; q < TA; ++q) read_a(0, 0, q);
#pragma unroll
    for (int q = 0; q < TB; ++q) read_b(0, 0, q);

    // iteration s (LDS stage cur, the next one nxt; register slot SL holds B(s+1), landed; the other slot B(s+2)):
    //   k-slices 0, 1 : MFMAs, fragment reads of the next slice, dequantisation of B(s+1) into stage nxt
    //   loads         : B(s+3) into slot SL (its old content is in LDS now)
    //   k-slice 2     : MFMAs, fragment reads of slice 3
    //   wait (A(s+1) and B(s+2) have landed; own LDS operations done), barrier: stage cur is free, nxt complete
    //   loads         : A(s+STAGES) into stage cur (loading waves)
    //   k-slice 3     : MFMAs, fragment reads of slice 0 of stage nxt
    int cur = 0, nxt = 1;                                           // activation stages
    int curb = 0, nxtb = 1;                                         // weight stages
    // one unit, every instruction in its place: MFMA m; behind the last MFMA of a row tile the reload of its fragment for
    // unit UN (stage SA); when UN starts a slice, its column fragments (stage SBR) behind the second MFMA of each row
    // tile; in a dequantising unit a piece of two weights behind every second MFMA and the 16-byte LDS write of a chunk
    // behind its last piece
#define AMCT_WUNIT(U, UN, SA, SBR, DQ, SL)                                             \
    {                                                                                  \
        _Pragma("unroll") for (int m_ = 0; m_ < kNM; ++m_) {                           \
            mfma_one((U), m_);                                                         \
            __builtin_amdgcn_sched_barrier(0);                                         \
            if (m_ % TB == TB - 1) {                                                   \
                read_a((SA), (UN), m_ / TB);                                           \
                __builtin_amdgcn_sched_barrier(0);                                     \
            }                                                                          \
            if (((UN) & 1) == 0 && m_ % TA == 1 && m_ / TA < TB) {                     \
                read_b((SBR), (UN) >> 1, m_ / TA);                                     \
                __builtin_amdgcn_sched_barrier(0);                                     \
            }                                                                          \
            if ((DQ) && m_ % kDqGap == 0 && m_ / kDqGap < 4 * (kBC / 2)) {             \
                dq_piece((SL), (kBC / 2) * (U) + (m_ / kDqGap) / 4, (m_ / kDqGap) % 4); \
                __builtin_amdgcn_sched_barrier(0);                                     \
                if ((m_ / kDqGap) % 4 == 3) {                                          \
                    dq_write(nxtb, (kBC / 2) * (U) + (m_ / kDqGap) / 4);               \
                    __builtin_amdgcn_sched_barrier(0);                                 \
                }                                                                      \
            }                                                                          \
        }                                                                              \
    }
#define AMCT_WITER(SL, step)                                                           \
    {                                                                                  \
        AMCT_TIE_SLOT(SL);                                                             \
        factors(SL);                                                                   \
        __builtin_amdgcn_sched_barrier(0);                                             \
        AMCT_WUNIT(0, 1, cur, curb, true, SL)                                          \
        AMCT_WUNIT(1, 2, cur, curb, true, SL)                                          \
        issue_b(SL, (step) + 3);                                                       \
        __builtin_amdgcn_sched_barrier(0);                                             \
        AMCT_WUNIT(2, 3, cur, curb, false, SL)                                         \
        wait_older();                                                                  \
        __builtin_amdgcn_s_barrier();                                                  \
        asm volatile("" ::: "memory");                                                 \
        __builtin_amdgcn_sched_barrier(0);                                             \
        dma_a(cur, (step) + STAGES);                                                   \
        __builtin_amdgcn_sched_barrier(0);                                             \
        AMCT_WUNIT(3, 0, nxt, nxtb, false, SL)                                         \
        cur = nxt;                                                                     \
        nxt = nxt + 1 == STAGES ? 0 : nxt + 1;                                         \
        curb = nxtb;                                                                   \
        nxtb = nxtb + 1 == SB ? 0 : nxtb + 1;                                          \
    }
    for (int step = 0; step < nsteps; step += 2) {                  // K % 128 == 0: an even number of steps
        AMCT_WITER(1, step)
        AMCT_WITER(0, step + 1)
    }
#undef AMCT_WITER
#undef AMCT_WUNIT
#undef AMCT_TIE_SLOT
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // epilogue: + bias (or + (-0.0f), which returns the value bit for bit), narrow to bf16, transpose through a
    // per-wave LDS patch of 32 rows x 32*TJ columns, 16-byte stores of full rows
    constexpr int kPW = 32 * TJ;                                   // patch width in columns
    constexpr int kPatchRow = kPW * 2 + 16;
    constexpr int CPR = kPW * 2 / 16;                              // 16-byte chunks per patch row
    static_assert(32 * kPatchRow <= 16384 && (32 * CPR) % 64 == 0, "patch");
    uint8_t* patch = smem + wave * 16384;
    // accumulator tile (t, j), register r: row 16 t + 4 (lane / 16) + r, column 16 j + lane % 16 of the wave tile
    float bs[TB];
#pragma unroll
    for (int j = 0; j < TB; ++j) {
        const int64_t n = n0 + wn * kPW + j * 16 + (lane & 15);
        bs[j] = a.bias ? a.bias[n < a.N ? n : a.N - 1] : -0.0f;
    }
    uint8_t* wbase = patch + 4 * (lane >> 4) * kPatchRow + (lane & 15) * 2;
#pragma unroll
    for (int i = 0; i < TI; ++i) {                                  // 32 rows of the wave tile per pass: tiles 2 i and 2 i + 1
        const int64_t mbase = m0 + wm * 32 * TI + i * 32;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < TB; ++j)
                    *reinterpret_cast<uint16_t*>(wbase + (16 * hh + r) * kPatchRow + j * 32) =
                        (uint16_t)(AF16 ? f32_to_f16_bits(acc[2 * i + hh][j][r] + bs[j]) : f32_to_bf16_bits(acc[2 * i + hh][j][r] + bs[j]));
#pragma unroll
        for (int it = 0; it < 32 * CPR / 64; ++it) {
            const int idx = it * 64 + lane;                        // 16-byte chunk of the patch, row-major
            const int prow = idx / CPR, chunk = idx % CPR;
            const uint4 v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * kPW + chunk * 8;
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * 2, v);
        }
    }
}

// blockIdx.x: column tile, blockIdx.y: row tile
template <bool SF16, int WM, int WN, int TI, int TJ, int STAGES, int SB = STAGES, bool AF16 = false>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(WM * WN / 4, WM * WN / 4))) void w4a16_tile_wide(W4A16Args a) {
    using Sh = WideTile<WM, WN, TI, TJ, STAGES, SB>;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Sh::kSmem];
    w4a16_wide_body<SF16, WM, WN, TI, TJ, STAGES, SB, AF16>(a, smem, (int64_t)blockIdx.y * Sh::kLM, (int64_t)blockIdx.x * Sh::kLN);
}

template <bool SF16, int WM, int WN, int TI, int TJ, int STAGES, int SB = STAGES, bool AF16 = false>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(WM * WN / 4, WM * WN / 4))) void w4a16_tile_wide16(W4A16Args a) {
    using Sh = WideTile<WM, WN, TI, TJ, STAGES, SB>;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[Sh::kSmem];
    w4a16_wide_body16<SF16, WM, WN, TI, TJ, STAGES, SB, AF16>(a, smem, (int64_t)blockIdx.y * Sh::kLM, (int64_t)blockIdx.x * Sh::kLN);
}

// ---------------------------------------------------------------------------
// medium-M kernel with specialised waves: 128x128 block tile, 12 waves.  Waves 0..3 (2 x 2 of 64x64, one per
// SIMD) only read fragments and issue MFMAs; waves 4..11 (two per SIMD) only move data: the direct-to-LDS loads of
// the activation tile, the packed weights into registers (8 bytes per thread and step, four steps ahead), their
// dequantisation and the LDS writes.  The dequantisation then runs under the other waves' MFMAs instead of
// between a wave's own: a block of 4 waves that does both, alone on its CU (three 32 KiB stages), has nobody to
// overlap with.  Same LDS layout and stage protocol as w4a16_wide_body; every wave passes the same number of
// barriers (one per step, two before the loop, one behind it).  Measured on W[14336,4096], M = 128: 38 us (8
// data-movement waves), 43 us (4), 51 us (4 waves doing everything); of the 38 us, 22 us are the matrix waves and
// the barriers alone, the LDS writes of the dequantised weights add 8 us, the loads 7 us, the arithmetic 4 us.
// ---------------------------------------------------------------------------
// Tile (64*TI) x (64*TJ): 2 x 2 matrix waves of (32*TI) x (32*TJ) and 8 data-movement waves (512 / (64*TJ) threads per
// weight row of the tile); 128x128 as described above, 64x64 and 128x64 for small M (8 weights per thread and step).
// WBITS = 8: the weight is int8 [N, K] (a.wq), a.zeros the int8 offsets or null; everything but the weight loads (twice the
// bytes per thread and step) and the dequantisation is the int4 kernel.
template <bool SF16, int STAGES, int TI = 2, int TJ = 2, int kD = 4, bool AF16 = false, int WBITS = 4>
__global__ __launch_bounds__(kSpecThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void w4a16_tile_spec(W4A16Args a) {
    constexpr int kLM = 64 * TI, kLN = 64 * TJ, WN = 2;
    constexpr int kThreads = kSpecThreads;
    constexpr int kStageBytes = (kLM + kLN) * kWRow;                // 32 KiB for 128x128
    constexpr int kMW = kSpecThreads / 64 - 4;                      // data-movement waves: 8
    constexpr int kPPR = kMW * 64 / kLN;                            // threads per weight row: 4 or 8
    constexpr int kBC = 8 / kPPR;                                   // 8-weight chunks per thread and step: 2 or 1
    constexpr int kNA = (kLM * kWRow / 1024) / kMW;                 // activation pieces per moving wave
    constexpr int kNM = TI * TJ, kNR = TI + TJ;
    static_assert(STAGES == 2 || STAGES == 3, "stages");
    constexpr int kStages = STAGES * kStageBytes > 65536 ? STAGES * kStageBytes : 65536;
    // behind the stages: scale (low 16 bits) and zero-point of every (weight row of the tile, group), one row of
    // kSpecMaxG + 1 words per weight row (odd stride: the 32 rows a wave reads hit different banks)
    __shared__ __attribute__((aligned(1024))) uint8_t smem[kStages + kLN * (kSpecMaxG + 1) * 4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t m0 = (int64_t)blockIdx.y * kLM, n0 = (int64_t)blockIdx.x * kLN;
    // Split K (gridDim.z > 1): block z takes the units of 256 elements [units z / S, units (z + 1) / S) of every row and
    // leaves fp32 partial sums in a.part[z]; a second kernel adds them in order.  Rows keep their stride a.K.
    const uint32_t units = (uint32_t)(a.K >> 8);
    const uint32_t k0 = (units * blockIdx.z / gridDim.z) << 8;
    const uint32_t klen = ((units * (blockIdx.z + 1) / gridDim.z) << 8) - k0;
    const uint32_t gfirst = __umulhi(k0, a.group_magic);           // first group of the slice
    const int nsteps = (int)(klen / kWK);
    const int last = nsteps - 1;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
    auto swz = [](int r) { return (r >> 1) & 7; };
    uint32_t* const tab = reinterpret_cast<uint32_t*>(smem + kStages);
    {
        // Per-step loads of a 2-byte scale and a 1-byte zero-point per thread touch 48 cache lines per wave
        // instruction; all of the tile's factors are fetched once instead, by all 512 threads.
        const uint32_t G = (uint32_t)(a.K / a.group);
        const uint32_t Gs = __umulhi(k0 + klen - 1, a.group_magic) - gfirst + 1;   // groups the slice touches (<= kSpecMaxG: host)
        // kTPR threads share a row; all loads are issued before the first use (unconditional, clamped): a loop that
        // loads and stores entry by entry pays one memory latency per trip before the kernel's first MFMA
        constexpr int kTPR = kThreads / kLN, kIt = (kSpecMaxG + kTPR - 1) / kTPR;
        const uint32_t row = tid / kTPR, g0 = tid % kTPR;
        const int64_t wr = (n0 + row < a.N) ? n0 + row : a.N - 1;
        uint32_t sb[kIt], zb[kIt];
#pragma unroll
        for (int j = 0; j < kIt; ++j) {
            const uint32_t g = gfirst + (g0 + j * kTPR < Gs ? g0 + j * kTPR : Gs - 1);
            sb[j] = reinterpret_cast<const uint16_t*>(a.scales)[wr * G + g];
            if constexpr (WBITS == 4) zb[j] = a.zeros[wr * G + g];
            else zb[j] = a.zeros ? (uint32_t)((int)reinterpret_cast<const int8_t*>(a.zeros)[wr * G + g] + 128) : 128u;
        }
#pragma unroll
        for (int j = 0; j < kIt; ++j)
            if (g0 + j * kTPR < Gs) tab[row * (kSpecMaxG + 1) + g0 + j * kTPR] = sb[j] | (zb[j] << 16);
        __syncthreads();
    }

    if (wave >= 4) {
        // ---------------- data movement ----------------
        const int pw = wave - 4, ptid = tid - 256;
        const uint32_t G = (uint32_t)(a.K / a.group);
        uint32_t goff[kNA];
        {
            const int rin = lane >> 3, pc = lane & 7;
#pragma unroll
            for (int j = 0; j < kNA; ++j) {
                const int lr = (pw * kNA + j) * 8 + rin;
                const int64_t r = m0 + lr < a.M ? m0 + lr : a.M - 1;
                goff[j] = (uint32_t)((r * a.K + (pc ^ swz(lr)) * 8) * 2);
            }
        }
        auto dma_a = [&](int stg, int step) {
            const int st = step < last ? step : last;
#pragma unroll
            for (int j = 0; j < kNA; ++j)
                dma16s(lds0 + stg * kStageBytes + (pw * kNA + j) * 1024, a.x + k0 + (int64_t)st * kWK, goff[j]);
        };
        // weight row ptid/kPPR of the tile, 8*kBC weights (4*kBC bytes) per step, which part from ptid%kPPR
        const int brow = ptid / kPPR, bq = ptid % kPPR;
        const int64_t wrow = (n0 + brow < a.N) ? n0 + brow : a.N - 1;
        constexpr int kWB = WBITS == 4 ? 4 : 8;                     // bytes of 8 weights
        const uint32_t woff = (uint32_t)(wrow * (a.K * kWB / 8) + bq * (kWB * kBC));
        const uint32_t* const trow = tab + brow * (kSpecMaxG + 1);
        int bdst[kBC];
#pragma unroll
        for (int c = 0; c < kBC; ++c) bdst[c] = kLM * kWRow + brow * kWRow + ((kBC * bq + c) ^ swz(brow)) * 16;
        // The weights stream from HBM and a step of this small tile is shorter than that latency, so the packed
        // weights of a step are fetched kD steps ahead into kD register slots (the loop is unrolled by kD).
        typedef unsigned int wq4 __attribute__((ext_vector_type(4)));
        typename std::conditional<kWB * kBC == 16, wq4, typename std::conditional<kWB * kBC == 8, uint64_t, uint32_t>::type>::type wreg[kD];
        auto issue_b = [&](int slot, int step) {
            const int st = step < last ? step : last;
            const uint8_t* src = a.wq + (k0 + (uint32_t)st * kWK) * kWB / 8;
            if constexpr (kWB * kBC == 16)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(wreg[slot]) : "v"(woff), "s"(src) : "memory");
            else if constexpr (kWB * kBC == 8)
                asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(wreg[slot]) : "v"(woff), "s"(src) : "memory");
            else
                asm volatile("global_load_dword %0, %1, %2" : "=v"(wreg[slot]) : "v"(woff), "s"(src) : "memory");
        };
        // the factors of a step are read from the table one iteration before they are used (enext): the LDS latency
        // would otherwise head the chain table read -> arithmetic -> LDS write -> barrier that bounds a step
        auto factor_word = [&](int step) {
            const int st = step < last ? step : last;
            return trow[__umulhi(k0 + (uint32_t)st * kWK, a.group_magic) - gfirst];   // k / group (k, group < 2^16); group % 64 == 0
        };
        uint32_t enext = factor_word(0);
        auto dequant_into = [&](int slot, int step, int stg) {      // the weights of K-step `step` (in `slot`) -> stage stg
            const uint32_t e = enext;
            enext = factor_word(step + 1);                          // issued before this step's LDS writes (see the loop)
            __builtin_amdgcn_sched_barrier(0);                      // keeps the read in front of the writes
            const float sc = SF16 ? f16_bits_to_f32(e & 0xFFFFu) : bf16_bits_to_f32(e & 0xFFFFu);
            const float nzs = -((float)(e >> 16) * sc);
            if constexpr (WBITS == 4) {
                *reinterpret_cast<uint4*>(smem + stg * kStageBytes + bdst[0]) = dequant8<AF16>((uint32_t)wreg[slot], sc, nzs);
                if constexpr (kBC == 2)
                    *reinterpret_cast<uint4*>(smem + stg * kStageBytes + bdst[1]) = dequant8<AF16>((uint32_t)((uint64_t)wreg[slot] >> 32), sc, nzs);
            } else if constexpr (kBC == 2) {
                *reinterpret_cast<uint4*>(smem + stg * kStageBytes + bdst[0]) = dequant8_i8<AF16>(wreg[slot].x, wreg[slot].y, sc, nzs);
                *reinterpret_cast<uint4*>(smem + stg * kStageBytes + bdst[1]) = dequant8_i8<AF16>(wreg[slot].z, wreg[slot].w, sc, nzs);
            } else {
                *reinterpret_cast<uint4*>(smem + stg * kStageBytes + bdst[0]) =
                    dequant8_i8<AF16>((uint32_t)wreg[slot], (uint32_t)((uint64_t)wreg[slot] >> 32), sc, nzs);
            }
        };
#define AMCT_TIE_SLOT(slot) asm volatile("" : "+v"(wreg[slot]) : : "memory")
        // prologue: B(0 .. kD-1) into their slots and A(0 .. STAGES-2); everything lands; B(0), B(1) are dequantised into
        // stages 0, 1 and their slots take B(kD), B(kD+1); A(STAGES-1) follows (weights first, as in the loop)
#pragma unroll
        for (int j = 0; j < kD; ++j) issue_b(j, j);
#pragma unroll
        for (int j = 0; j < STAGES - 1; ++j) dma_a(j, j);
        wait_vm<0>();
#pragma unroll
        for (int j = 0; j < kD; ++j) AMCT_TIE_SLOT(j);
        dequant_into(0, 0, 0);
        dequant_into(1, 1, 1);
        issue_b(0, kD);
        issue_b(1, kD + 1);
        dma_a(STAGES - 1, STAGES - 1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // The dequantisation runs TWO steps ahead of the matrix waves, which need stage s+1 behind the barrier of
        // iteration s: that barrier then waits for the LDS writes of the iteration before (lgkmcnt leaves this
        // iteration's kBC writes in flight), so their latency is not part of the step's chain.
        // iteration s: wait for B(s+2) (slot SL; issued kD iterations ago: the kNA activation loads of that iteration
        // and the 1 + kNA operations of each iteration since may stay in flight; in iteration 2 the loads behind B(4)
        // are those of the prologue's tail, one activation group fewer); B(s+2) -> stage (s+2) % STAGES, free since the
        // barrier before; wait for A(s+1) (issued STAGES-1 iterations ago); barrier; B(s+2+kD) into slot SL,
        // A(s+STAGES) into stage cur
        int cur = 0, s2 = 2 % STAGES;
#define AMCT_MOVE_ITER(SL, step)                                                       \
    {                                                                                  \
        if ((step) == kD - 2) wait_vm<(kD - 1) * (1 + kNA)>();                         \
        else wait_vm<kNA + (kD - 1) * (1 + kNA)>();                                    \
        AMCT_TIE_SLOT(SL);                                                             \
        dequant_into(SL, (step) + 2, s2);                                              \
        wait_vm<(STAGES - 2) * (1 + kNA)>();                                           \
        asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(kBC) : "memory");                 \
        __builtin_amdgcn_s_barrier();                                                  \
        asm volatile("" ::: "memory");                                                 \
        issue_b(SL, (step) + 2 + kD);                                                  \
        dma_a(cur, (step) + STAGES);                                                   \
        cur = cur + 1 == STAGES ? 0 : cur + 1;                                         \
        s2 = s2 + 1 == STAGES ? 0 : s2 + 1;                                            \
    }
        for (int step = 0; step < nsteps; step += kD) {             // K % (64 * kD) == 0: a multiple of kD steps
#pragma unroll
            for (int u = 0; u < kD; ++u) AMCT_MOVE_ITER((u + 2) % kD, step + u)
        }
#undef AMCT_MOVE_ITER
#undef AMCT_TIE_SLOT
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        return;
    }

    // ---------------- matrix work ----------------
    const int wm = wave / WN, wn = wave % WN;
    int offA[4], offB[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int r = lane & 31;
        const int phys = (ks * 2 + (lane >> 5)) ^ swz(r);
        offA[ks] = (wm * 32 * TI + r) * kWRow + phys * 16;
        offB[ks] = kLM * kWRow + (wn * 32 * TJ + r) * kWRow + phys * 16;
    }
    v16f acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    auto read_one = [&](int stg, int ks, int q, v8bf (&fa)[TI], v8bf (&fb)[TJ]) {
        const uint8_t* st = smem + stg * kStageBytes;
        if (q == 0) fa[0] = *reinterpret_cast<const v8bf*>(st + offA[ks]);
        else if (q <= TJ) fb[q - 1] = *reinterpret_cast<const v8bf*>(st + offB[ks] + (q - 1) * 32 * kWRow);
        else fa[q - TJ] = *reinterpret_cast<const v8bf*>(st + offA[ks] + (q - TJ) * 32 * kWRow);
    };
    auto mfma_one = [&](int m, const v8bf (&fa)[TI], const v8bf (&fb)[TJ]) {
        const int i = m / TJ, j = m % TJ;
        if constexpr (AF16) {
            typedef _Float16 v8hs __attribute__((ext_vector_type(8)));
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8hs, fa[i]), __builtin_bit_cast(v8hs, fb[j]), acc[i][j], 0, 0, 0);
        } else {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };
    // One fragment buffer per k-slice: a 64x64 wave tile has only 4 MFMAs per slice, fewer cycles than an LDS read
    // takes, so the reads of slices 1..3 of a step are all issued behind the MFMAs of slice 0 (the stage is complete
    // when the step starts) and their latency is paid once per step instead of once per slice.
    v8bf fa[4][TI], fb[4][TJ];
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int q = 0; q < kNR; ++q) read_one(0, 0, q, fa[0], fb[0]);
    {
        int cur = 0, nxt = 1;
        constexpr int kRPM = (3 * kNR + kNM - 1) / kNM;             // reads behind each MFMA of slice 0
        constexpr int kRP0 = (kNR + kNM - 1) / kNM;                 // reads of the next step's slice 0 behind each MFMA of slice 3
        if constexpr (kNM == 2) {
            // 64x32 wave tiles: a whole step is 8 MFMAs, so ALL fragments of the next stage are read right behind the
            // barrier that completes it (after the last slice of the current step, which still uses the old registers)
            // and the step pays one LDS latency instead of two: 22.8 us against 24.0 us for the 128x64 block (the 64x64
            // block, 4 MFMAs per step, lost with this order: 20.5 us against 18.4 us)
#pragma unroll
            for (int ks = 1; ks < 4; ++ks)
#pragma unroll
                for (int q = 0; q < kNR; ++q) read_one(0, ks, q, fa[ks], fb[ks]);
            for (int step = 0; step < nsteps; ++step) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < 3; ++ks) {
#pragma unroll
                    for (int m = 0; m < kNM; ++m) {
                        mfma_one(m, fa[ks], fb[ks]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < kNM; ++m) {
                    mfma_one(m, fa[3], fb[3]);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                    for (int q = 0; q < kNR; ++q) {
                        read_one(nxt, ks, q, fa[ks], fb[ks]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                cur = nxt;
                nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
            }
        } else
        for (int step = 0; step < nsteps; ++step) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m < kNM; ++m) {
                mfma_one(m, fa[0], fb[0]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q = kRPM * m; q < kRPM * (m + 1); ++q) {
                    if (q < 3 * kNR) {
                        read_one(cur, 1 + q / kNR, q % kNR, fa[1 + q / kNR], fb[1 + q / kNR]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
#pragma unroll
            for (int ks = 1; ks < 3; ++ks) {
#pragma unroll
                for (int m = 0; m < kNM; ++m) {
                    mfma_one(m, fa[ks], fb[ks]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int m = 0; m < kNM; ++m) {
                mfma_one(m, fa[3], fb[3]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q = kRP0 * m; q < kRP0 * (m + 1) && q < kNR; ++q) {
                    read_one(nxt, 0, q, fa[0], fb[0]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            cur = nxt;
            nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    if (gridDim.z > 1) {
        // split K: the raw fp32 sums of this slice, row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32 of each 32x32 tile
        float* const part = a.part + (int64_t)blockIdx.z * a.M * a.N;
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m0 + wm * 32 * TI + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const int64_t n = n0 + wn * 32 * TJ + j * 32 + (lane & 31);
                    if (m < a.M && n < a.N) part[m * a.N + n] = acc[i][j][r];
                }
            }
        return;
    }
    // epilogue (matrix waves only): + bias (or + (-0.0f)), narrow to the activation type, transpose through a per-wave LDS patch
    constexpr int kPW = 32 * TJ, kPatchRow = kPW * 2 + 16, CPR = kPW * 2 / 16;
    uint8_t* patch = smem + wave * 16384;
    float bs[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int64_t n = n0 + wn * kPW + j * 32 + (lane & 31);
        bs[j] = a.bias ? a.bias[n < a.N ? n : a.N - 1] : -0.0f;
    }
    uint8_t* wbase = patch + 4 * (lane >> 5) * kPatchRow + (lane & 31) * 2;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int64_t mbase = m0 + wm * 32 * TI + i * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int prow0 = 8 * (r >> 2) + (r & 3);
#pragma unroll
            for (int j = 0; j < TJ; ++j)
                *reinterpret_cast<uint16_t*>(wbase + prow0 * kPatchRow + j * 64) = (uint16_t)(AF16 ? f32_to_f16_bits(acc[i][j][r] + bs[j]) : f32_to_bf16_bits(acc[i][j][r] + bs[j]));
        }
#pragma unroll
        for (int it = 0; it < 32 * CPR / 64; ++it) {
            const int idx = it * 64 + lane;
            const int prow = idx / CPR, chunk = idx % CPR;
            const uint4 v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * kPW + chunk * 8;
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * 2, v);
        }
    }
}

// x' = bf16(x * smooth[k]) over the whole activation matrix (K % 8 == 0): used when the caller lends a
// workspace, so that the multiply is done once instead of once per column tile.  Block `block` of `nblocks`.
AMCT_DEV void smooth_rows_body(const uint16_t* x, const uint16_t* smooth, uint16_t* y, int64_t nvec, int kvec, unsigned block, unsigned nblocks) {
    const int64_t stride = (int64_t)nblocks * kBlock;
    for (int64_t v = (int64_t)block * kBlock + threadIdx.x; v < nvec; v += stride) {
        const uint4 c = ldg16(smooth + (v % kvec) * 8);
        stg16(y + v * 8, smooth8(ldg16_nt(x + v * 8), c));
    }
}
__global__ __launch_bounds__(kBlock) void smooth_rows(const uint16_t* x, const uint16_t* smooth, uint16_t* y, int64_t nvec, int kvec) {
    smooth_rows_body(x, smooth, y, nvec, kvec, blockIdx.x, gridDim.x);
}
// the same for fp16 activations: x' = fp16(x * smooth[k])
AMCT_DEV void smooth_rows_f16_body(const uint16_t* x, const uint16_t* smooth, uint16_t* y, int64_t nvec, int kvec, unsigned block, unsigned nblocks) {
    const int64_t stride = (int64_t)nblocks * kBlock;
    for (int64_t v = (int64_t)block * kBlock + threadIdx.x; v < nvec; v += stride) {
        const uint4 c = ldg16(smooth + (v % kvec) * 8), xv = ldg16_nt(x + v * 8);
        const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w}, cs[4] = {c.x, c.y, c.z, c.w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = pack_f16x2(f16_bits_to_f32(xs[i] & 0xFFFFu) * f16_bits_to_f32(cs[i] & 0xFFFFu),
                              f16_bits_to_f32(xs[i] >> 16) * f16_bits_to_f32(cs[i] >> 16));
        stg16(y + v * 8, make_uint4(o[0], o[1], o[2], o[3]));
    }
}
__global__ __launch_bounds__(kBlock) void smooth_rows_f16(const uint16_t* x, const uint16_t* smooth, uint16_t* y, int64_t nvec, int kvec) {
    smooth_rows_f16_body(x, smooth, y, nvec, kvec, blockIdx.x, gridDim.x);
}

// The whole weight dequantised once, dt((u - z) * s) as the tile kernels compute it per block: for so many rows that
// dequantising inside every row tile costs more than writing and re-reading the 16-bit weight (the product is then the
// plain 16-bit GEMM on the large tiles of the W8A8 kernel, gemm_w8a8.hip: gemm16_tiles).  A thread takes 8 weights at a
// time (4 bytes of nibbles in, 16 bytes out), the threads of a block walk along a row: a wave reads 256 and writes 1024
// contiguous bytes per step.  group % 8 == 0, so the 8 weights share a group.
constexpr int kDqRows = 4;      // rows of the weight per block, their loads in flight together (1 / 2 / 4 / 8: 209 / 206 / 205.6 / 206.8 us at M = 2048)
// out = dt(part[0] + part[1] + ... + part[S - 1] + bias), the slices added in that order; 8 columns per thread (N % 8 == 0)
template <bool AF16>
__global__ __launch_bounds__(kBlock) void splitk_reduce16(const float* part, const float* bias, uint16_t* out, int64_t M, int64_t N, int S) {
    const int64_t nvec = M * N / 8, stride = (int64_t)gridDim.x * kBlock;
    for (int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride) {
        const int64_t e = v * 8;
        float4 lo = *reinterpret_cast<const float4*>(part + e), hi = *reinterpret_cast<const float4*>(part + e + 4);
        for (int z = 1; z < S; ++z) {
            const float4 a0 = *reinterpret_cast<const float4*>(part + (int64_t)z * M * N + e);
            const float4 a1 = *reinterpret_cast<const float4*>(part + (int64_t)z * M * N + e + 4);
            lo.x += a0.x, lo.y += a0.y, lo.z += a0.z, lo.w += a0.w;
            hi.x += a1.x, hi.y += a1.y, hi.z += a1.z, hi.w += a1.w;
        }
        if (bias) {
            const int64_t n = e % N;
            const float4 b0 = *reinterpret_cast<const float4*>(bias + n), b1 = *reinterpret_cast<const float4*>(bias + n + 4);
            lo.x += b0.x, lo.y += b0.y, lo.z += b0.z, lo.w += b0.w;
            hi.x += b1.x, hi.y += b1.y, hi.z += b1.z, hi.w += b1.w;
        }
        stg16_nt(out + e, make_uint4(pack_act2<AF16>(lo.x, lo.y), pack_act2<AF16>(lo.z, lo.w), pack_act2<AF16>(hi.x, hi.y), pack_act2<AF16>(hi.z, hi.w)));
    }
}

// The first `wblocks` blocks of the launch dequantise (kDqRows rows each); the others, if any, smooth the activations
// into `xs` (two independent passes in one launch: the short one runs beside the long one).
template <bool AF16>
__global__ __launch_bounds__(kBlock) void w4_dequant_rows(W4A16Args a, uint16_t* wdq, uint16_t* xs, unsigned wblocks) {
    if (blockIdx.x >= wblocks) {
        const int64_t nvec = a.M * a.K / 8;
        if constexpr (AF16) smooth_rows_f16_body(a.x, a.smooth, xs, nvec, (int)(a.K / 8), blockIdx.x - wblocks, gridDim.x - wblocks);
        else smooth_rows_body(a.x, a.smooth, xs, nvec, (int)(a.K / 8), blockIdx.x - wblocks, gridDim.x - wblocks);
        return;
    }
    const uint32_t kv = (uint32_t)(a.K >> 3), G = (uint32_t)(a.K / a.group);
    const bool small_k = a.K < 65536;                               // k / group by the multiply-high then
    const int64_t row0 = (int64_t)blockIdx.x * kDqRows;
    for (uint32_t v = threadIdx.x; v < kv; v += kBlock) {
        const uint32_t k = v * 8;
        const uint32_t g = small_k ? __umulhi(k, a.group_magic) : k / (uint32_t)a.group;
        uint32_t w[kDqRows];
        float sc[kDqRows], nzs[kDqRows];
#pragma unroll
        for (int r = 0; r < kDqRows; ++r) {
            const int64_t row = row0 + r < a.N ? row0 + r : a.N - 1;
            const int64_t gi = row * G + g;
            w[r] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(a.wq + row * (a.K >> 1)) + v);
            sc[r] = load_scale(a, gi);
            nzs[r] = -((float)a.zeros[gi] * sc[r]);
        }
#pragma unroll
        for (int r = 0; r < kDqRows; ++r)
            if (row0 + r < a.N) stg16(wdq + (row0 + r) * a.K + k, dequant8<AF16>(w[r], sc[r], nzs[r]));
    }
}

// ---------------------------------------------------------------------------
// decode kernel (M <= 16 * MT, K % 128 == 0, group % 32 == 0): weight streaming.
// A block owns 64 output columns; its waves split K in runs of 128 (one iteration = 4 MFMA k-slots of
// 32).  Per iteration a lane fetches 16 bytes of each of its 4 weight rows (row 16 t + lane % 16,
// k-slot lane / 16): 64 bytes per lane, twice that in flight with the prefetch of the next iteration.
// All loads are unconditional (indices clamped), so none forces a full wait.  The activation fragments
// of an iteration (smoothed once) are shared by the 4 column tiles; the weights are dequantised to bf16
// exactly as in the large-tile kernel, so both produce the same operand bits.
// ---------------------------------------------------------------------------
constexpr int kDN = 64;                                           // output columns per block

template <int MT, int WAVES, bool SMOOTH>
__global__ __launch_bounds__(WAVES * 64) void w4a16_decode(W4A16Args a) {
    __shared__ float red[WAVES - 1 > 0 ? WAVES - 1 : 1][MT][4][64][4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * kDN;
    const int64_t G = a.K / a.group;
    const int iters_total = (int)(a.K / 128);
    const int per_wave = iters_total / WAVES;                      // host guarantees divisibility
    const int it0 = wave * per_wave;
    const bool scale_is_f16 = a.scale_dtype == AMCT_F16;

    const uint8_t* wrow[4];
    const uint8_t* srow[4];
    const uint8_t* zrow[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int64_t n = n0 + t * 16 + r16;
        const int64_t nc = n < a.N ? n : a.N - 1;
        wrow[t] = a.wq + nc * (a.K / 2) + g * 16;
        srow[t] = reinterpret_cast<const uint8_t*>(a.scales) + nc * G * 2;
        zrow[t] = a.zeros + nc * G;
    }
    const uint16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int64_t m = mt * 16 + r16;
        xrow[mt] = a.x + (m < a.M ? m : a.M - 1) * a.K + g * 32;
    }

    v4f y[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t) y[mt][t] = v4f{0.f, 0.f, 0.f, 0.f};

    // one iteration's loads, all issued together and all consumed one iteration later: the waits the
    // compiler derives (in issue order) then never cover the batch that was just issued
    uint4 wv[2][4], xv[2][MT][4], cv[2][4];
    uint32_t sb[2][4], zb[2][4];
    auto load_w = [&](int buf, int it) {
        const int itc = it < it0 + per_wave ? it : it0 + per_wave - 1;      // clamped: loads are unconditional
        const uint32_t kb = (uint32_t)itc * 128u;
        const uint32_t gi = __umulhi(kb + (uint32_t)g * 32u, a.group_magic);   // (kb + 32 g) / group
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
            if constexpr (SMOOTH) cv[buf][s4] = ldg16(a.smooth + kb + g * 32 + s4 * 8);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) xv[buf][mt][s4] = ldg16(xrow[mt] + kb + s4 * 8);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sb[buf][t] = *reinterpret_cast<const uint16_t*>(srow[t] + gi * 2);
            zb[buf][t] = zrow[t][gi];
            wv[buf][t] = ldg16_nt(wrow[t] + kb / 2);
        }
    };
    auto compute = [&](int buf) {
        v8bf fa[MT][4];
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                fa[mt][s4] = __builtin_bit_cast(v8bf, SMOOTH ? smooth8(xv[buf][mt][s4], cv[buf][s4]) : xv[buf][mt][s4]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float sc_h = f16_bits_to_f32(sb[buf][t]), sc_b = bf16_bits_to_f32(sb[buf][t]);
            const float sc = scale_is_f16 ? sc_h : sc_b;
            const float nzs = -((float)zb[buf][t] * sc);
            const uint32_t ws[4] = {wv[buf][t].x, wv[buf][t].y, wv[buf][t].z, wv[buf][t].w};
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const v8bf fb = __builtin_bit_cast(v8bf, dequant8(ws[s4], sc, nzs));
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    y[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[mt][s4], fb, y[mt][t], 0, 0, 0);
            }
        }
    };

    load_w(0, it0);
    for (int i = 0; i < per_wave; i += 2) {
        load_w(1, it0 + i + 1);
        __builtin_amdgcn_sched_barrier(0);                        // keep the prefetch ahead of the arithmetic
        compute(0);
        if (i + 1 >= per_wave) break;
        __builtin_amdgcn_sched_barrier(0);
        load_w(0, it0 + i + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(1);
        __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r) red[wave - 1][mt][t][lane][r] = y[mt][t][r];
        }
        __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int64_t n = n0 + t * 16 + r16;
            const float b = (a.bias && n < a.N) ? a.bias[n] : 0.f;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = y[mt][t][r];
                    if constexpr (WAVES > 1) {
#pragma unroll
                        for (int w = 0; w < WAVES - 1; ++w) v = v + red[w][mt][t][lane][r];
                    }
                    if (a.bias) v = v + b;
                    const int64_t m = mt * 16 + 4 * g + r;
                    if (n < a.N && m < a.M) a.out[m * a.N + n] = (uint16_t)f32_to_bf16_bits(v);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// decode kernel with the block's activations in LDS (M <= 16, K % 256 == 0, M * K small enough).
// Everything that is not the weight stream is fetched once per block with coalesced loads: the
// activations (smoothed on the way, rows padded by 16 bytes so that the 16 rows of a fragment read fall
// into different banks) and the block's 64 x G scales and zero-points.  The weight stream is the only
// per-lane traffic left; a lane's loads come in pairs that cover both 64-byte halves of a 128-byte
// line back to back (k-slots h = 0, 1 of a 256-wide iteration), two iterations are in flight.
// ---------------------------------------------------------------------------
// SMOOTH: 0 no smoothing; 1 every vector a thread stages has the same k position (the thread count is a multiple
// of the vectors per row), so one smoothing vector serves them all; 2 one smoothing vector per staged vector
template <int WAVES, int SMOOTH, int XJ, int TN>
__global__ __launch_bounds__(WAVES * 64) void w4a16_decode_lds(W4A16Args a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    constexpr int NT = WAVES * 64;
    constexpr int DN = 16 * TN;                                   // output columns per block
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * DN;
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M;
    const uint32_t G = K / (uint32_t)a.group;
    const uint32_t xstride = K * 2 + 16;                          // bytes per staged activation row
    const uint32_t xbytes = M * xstride;
    const uint32_t red_bytes = (WAVES - 1) * TN * 64 * 16;
    uint8_t* xs = lds_raw;
    uint16_t* sc_lds = reinterpret_cast<uint16_t*>(lds_raw + (xbytes > red_bytes ? xbytes : red_bytes));
    uint8_t* z_lds = reinterpret_cast<uint8_t*>(sc_lds + DN * G);
    const bool scale_is_f16 = a.scale_dtype == AMCT_F16;
    const int per_wave = (int)(K / 256) / WAVES;
    const int it0 = wave * per_wave;

    // ---- staging loads first, the weight stream after them: waits are in issue order, so the staged data
    // can be consumed (and the block barrier passed) while the weights are still arriving
    // scales: DN rows x G u16 = 2 TN G vectors of 16 bytes; zero-points: TN G vectors.  Rows past N read the last
    // vectors of the tensors (in bounds, never used for a stored output).
    constexpr int SJ = (2 * TN * 128 + NT - 1) / NT;              // G <= 128
    constexpr int ZJ = (TN * 128 + NT - 1) / NT;
    const int64_t sv_total = a.N * (int64_t)G / 8, zv_total = a.N * (int64_t)G / 16;
    const int64_t sv0 = n0 * (int64_t)G / 8, zv0 = n0 * (int64_t)G / 16;
    uint4 sv[SJ], zv[ZJ];
#pragma unroll
    for (int j = 0; j < SJ; ++j) {
        const int64_t i = sv0 + tid + NT * j;
        sv[j] = ldg16(reinterpret_cast<const uint8_t*>(a.scales) + (i < sv_total ? i : sv_total - 1) * 16);
    }
#pragma unroll
    for (int j = 0; j < ZJ; ++j) {
        const int64_t i = zv0 + tid + NT * j;
        zv[j] = ldg16(a.zeros + (i < zv_total ? i : zv_total - 1) * 16);
    }
    const uint32_t KV = K / 8, n_xv = M * KV;
    uint4 xv[XJ], cv[SMOOTH == 2 ? XJ : 1];
    uint32_t xdst[XJ];
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        const uint32_t vc = v < n_xv ? v : n_xv - 1;
        const uint32_t row = vc / KV, kv = vc - row * KV;
        xv[j] = ldg16(a.x + (int64_t)row * K + kv * 8);
        if constexpr (SMOOTH == 2) cv[j] = ldg16(a.smooth + kv * 8);
        if constexpr (SMOOTH == 1) {
            if (j == 0) cv[0] = ldg16(a.smooth + kv * 8);
        }
        xdst[j] = row * xstride + kv * 16;
    }
    __builtin_amdgcn_sched_barrier(0);

    const uint8_t* wrow[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const int64_t n = n0 + t * 16 + r16;
        wrow[t] = a.wq + (n < a.N ? n : a.N - 1) * (int64_t)(K / 2) + g * 16;
    }
    uint4 wv[2][TN * 2];
    auto load_w = [&](int buf, int it) {
        const int itc = it < it0 + per_wave ? it : it0 + per_wave - 1;      // clamped: loads are unconditional
        const uint32_t kb2 = (uint32_t)itc * 128u;                          // byte offset of the iteration
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int h = 0; h < 2; ++h) wv[buf][t * 2 + h] = ldg16(wrow[t] + kb2 + h * 64);
    };
    load_w(0, it0);
    load_w(1, it0 + 1);
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int j = 0; j < SJ; ++j) {
        const uint32_t i = tid + NT * j;
        if (i < 2 * TN * G) *reinterpret_cast<uint4*>(reinterpret_cast<uint8_t*>(sc_lds) + i * 16) = sv[j];
    }
#pragma unroll
    for (int j = 0; j < ZJ; ++j) {
        const uint32_t i = tid + NT * j;
        if (i < TN * G) *reinterpret_cast<uint4*>(z_lds + i * 16) = zv[j];
    }
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        if constexpr (SMOOTH != 0) xv[j] = smooth8(xv[j], cv[SMOOTH == 2 ? j : 0]);
        if (v < n_xv) *reinterpret_cast<uint4*>(xs + xdst[j]) = xv[j];
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    v4f y[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) y[t] = v4f{0.f, 0.f, 0.f, 0.f};
    const uint8_t* xlane = xs + (r16 < (int)M ? r16 : (int)M - 1) * xstride + g * 64;

    auto compute = [&](int buf, int it) {
        const uint32_t kb = (uint32_t)it * 256u;
        v8bf fa[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4)
                fa[h][s4] = *reinterpret_cast<const v8bf*>(xlane + (kb + h * 128) * 2 + s4 * 16);
#pragma unroll
        for (int t = 0; t < TN; ++t) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t k0 = kb + h * 128 + g * 32;
                const uint32_t gi = __umulhi(k0, a.group_magic);  // k0 / group
                const uint32_t sbits = sc_lds[(t * 16 + r16) * G + gi];
                const float sc_h = f16_bits_to_f32(sbits), sc_b = bf16_bits_to_f32(sbits);
                const float sc = scale_is_f16 ? sc_h : sc_b;
                const float nzs = -((float)z_lds[(t * 16 + r16) * G + gi] * sc);
                const uint4 w4 = wv[buf][t * 2 + h];
                const uint32_t ws[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int s4 = 0; s4 < 4; ++s4) {
                    const v8bf fb = __builtin_bit_cast(v8bf, dequant8(ws[s4], sc, nzs));
                    y[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[h][s4], fb, y[t], 0, 0, 0);
                }
            }
        }
    };

    for (int i = 0; i < per_wave; i += 2) {
        compute(0, it0 + i);
        __builtin_amdgcn_sched_barrier(0);
        if (i + 1 >= per_wave) break;
        load_w(0, it0 + i + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute(1, it0 + i + 1);
        __builtin_amdgcn_sched_barrier(0);
        load_w(1, it0 + i + 3);
        __builtin_amdgcn_sched_barrier(0);
    }

    float* red = reinterpret_cast<float*>(lds_raw);               // reuses the activation rows
    if constexpr (WAVES > 1) {
        __syncthreads();                                          // every wave is done reading activations
        if (wave > 0) {
#pragma unroll
            for (int t = 0; t < TN; ++t)
                *reinterpret_cast<v4f*>(red + (((wave - 1) * TN + t) * 64 + lane) * 4) = y[t];
        }
        __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            const int64_t n = n0 + t * 16 + r16;
            const float b = (a.bias && n < a.N) ? a.bias[n] : 0.f;
            v4f acc = y[t];
            if constexpr (WAVES > 1) {
#pragma unroll
                for (int w = 0; w < WAVES - 1; ++w) {
                    const v4f o = *reinterpret_cast<const v4f*>(red + ((w * TN + t) * 64 + lane) * 4);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[r] = acc[r] + o[r];
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = acc[r];
                if (a.bias) v = v + b;
                const int64_t m = 4 * g + r;
                if (n < a.N && m < a.M) a.out[m * a.N + n] = (uint16_t)f32_to_bf16_bits(v);
            }
        }
    }
}

// LDS bytes of w4a16_decode_lds, 0 if the shape does not fit
static size_t decode_lds_bytes(int64_t M, int64_t K, int group, int waves, int tn) {
    const size_t xbytes = (size_t)M * ((size_t)K * 2 + 16);
    const size_t red = (size_t)(waves - 1) * tn * 64 * 16;
    const size_t G = (size_t)(K / group);
    const size_t total = (xbytes > red ? xbytes : red) + (size_t)tn * 16 * G * 3;
    return total <= 150 * 1024 ? total : 0;
}

template <int WAVES, int SMOOTH, int XJ, int TN>
static int launch_decode_lds(const W4A16Args& a, size_t lds, hipStream_t st) {
    // only launches above the default 64 KiB of dynamic LDS need the attribute; it is per device and cheap,
    // so it is simply set on every such launch and no state is kept in the library
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(&w4a16_decode_lds<WAVES, SMOOTH, XJ, TN>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return AMCT_E_HIP;
    }
    const dim3 grid((unsigned)((a.N + 16 * TN - 1) / (16 * TN)));
    hipLaunchKernelGGL((w4a16_decode_lds<WAVES, SMOOTH, XJ, TN>), grid, dim3(WAVES * 64), lds, st, a);
    return hip_status();
}

template <int WAVES, int SMOOTH, int TN>
static int launch_decode_lds_sm(const W4A16Args& a, size_t lds, hipStream_t st) {
    const int64_t per_thread = (a.M * (a.K / 8) + WAVES * 64 - 1) / (WAVES * 64);
    if (per_thread <= 1) return launch_decode_lds<WAVES, SMOOTH, 1, TN>(a, lds, st);
    if (per_thread <= 4) return launch_decode_lds<WAVES, SMOOTH, 4, TN>(a, lds, st);
    if (per_thread <= 16) return launch_decode_lds<WAVES, SMOOTH, 16, TN>(a, lds, st);
    return AMCT_E_UNSUPPORTED;                                    // caller falls through to the register kernel
}

template <int WAVES, bool SMOOTH, int TN>
static int launch_decode_lds_xj(const W4A16Args& a, size_t lds, hipStream_t st) {
    if constexpr (!SMOOTH) return launch_decode_lds_sm<WAVES, 0, TN>(a, lds, st);
    else if ((WAVES * 64) % (a.K / 8) == 0) return launch_decode_lds_sm<WAVES, 1, TN>(a, lds, st);
    else return launch_decode_lds_sm<WAVES, 2, TN>(a, lds, st);
}

template <bool SMOOTH, int TN>
static int launch_decode_lds_w(const W4A16Args& a, int waves, size_t lds, hipStream_t st) {
    if constexpr (TN == 4) {
        if (waves == 8) return launch_decode_lds_xj<8, SMOOTH, TN>(a, lds, st);
    }
    return waves == 4 ? launch_decode_lds_xj<4, SMOOTH, TN>(a, lds, st) : launch_decode_lds_xj<1, SMOOTH, TN>(a, lds, st);
}

// general kernel: one output per thread, sequential fp32 accumulation over k
__global__ __launch_bounds__(kBlock) void w4a16_general(W4A16Args a) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= a.M * a.N) return;
    const int64_t m = idx / a.N, n = idx - m * a.N;
    const int64_t G = a.K / a.group;
    float acc = 0.f;
    for (int64_t k = 0; k < a.K; ++k) {
        float xv = bf16_bits_to_f32(a.x[m * a.K + k]);
        if (a.smooth) xv = round_to<AMCT_BF16>(xv * bf16_bits_to_f32(a.smooth[k]));
        const uint32_t byte = a.wq[n * (a.K / 2) + k / 2];
        const float u = (float)((k & 1) ? (byte >> 4) : (byte & 0xFu));
        const int64_t gi = n * G + k / a.group;
        const float w = round_to<AMCT_BF16>((u - (float)a.zeros[gi]) * load_scale(a, gi));
        acc = acc + xv * w;
    }
    if (a.bias) acc = acc + a.bias[n];
    a.out[m * a.N + n] = (uint16_t)f32_to_bf16_bits(acc);
}

int wq16_int4_f16(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                  const uint8_t* zeros, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                  hipStream_t st);                                 // gemm_wq16.hip
int w4a16_stream_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                          const uint8_t* zeros, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group,
                          int dtype, void* workspace, size_t workspace_bytes, hipStream_t st);
size_t w4a16_stream_part_bytes(int64_t M, int64_t N, int64_t K, int group);   // partial sums of its launches over slices of K
bool w4a16_stream_takes(int64_t M, int64_t N, int64_t K, int group, size_t workspace_bytes);   // gemm_w4a16_stream.hip

int gemm16_tiles(const void* x, const void* w, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int dtype,
                 void* workspace, size_t workspace_bytes, hipStream_t st);   // gemm_w8a8.hip
size_t gemm16_part_bytes(int64_t M, int64_t N, int64_t K);         // gemm_w8a8.hip: partial sums it wants lent for few tiles

// From this many rows on, dequantising the weight once into a lent workspace and running the plain 16-bit GEMM beats
// dequantising inside every row tile.  Measured on W[14336,4096] with smoothing, fused kernel / two passes: M = 1024
// 132 / 132 us, 1088 209 / 187, 1280 209 / 188, 1536 214 / 206, 2048 222 / 209, 3072 333 / 321, 4096 439 / 384: the
// weight pass costs 26 us, a row of the plain GEMM 0.083 us against 0.107 us for the fused kernel, and up to 1024 rows
// the fused kernel's tiles fit the CUs in one round.
constexpr int64_t kTwoPassFrom = 1025;

static size_t two_pass_workspace(int64_t M, int64_t N, int64_t K, int group, int has_smooth) {
    if (M < kTwoPassFrom || K % 64 != 0 || N % 8 != 0 || group % 32 != 0 || K % group != 0 || N * K * 2 >= (int64_t(1) << 32) ||
        M * K * 2 >= (int64_t(1) << 32))
        return 0;
    return (size_t)N * (size_t)K * 2 + (has_smooth ? (size_t)M * (size_t)K * 2 : 0) + gemm16_part_bytes(M, N, K);
}

// dequantise, smooth, multiply; AMCT_E_UNSUPPORTED when the shape or the workspace does not allow it
static int two_pass(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype, const uint8_t* zeros,
                    const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group, int dtype, void* workspace,
                    size_t workspace_bytes, hipStream_t st) {
    const size_t part = gemm16_part_bytes(M, N, K);
    const size_t need = two_pass_workspace(M, N, K, group, smooth != nullptr) - part;   // the partial sums are optional
    if (!two_pass_workspace(M, N, K, group, smooth != nullptr) || !workspace || workspace_bytes < need || !aligned16(workspace) || !aligned16(x) || !aligned16(wq) || !aligned16(out) ||
        (smooth && !aligned16(smooth)))
        return AMCT_E_UNSUPPORTED;
    W4A16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group, scale_dtype,
                (uint32_t)(0x100000000ull / (uint64_t)group) + 1u};
    uint16_t* wdq = reinterpret_cast<uint16_t*>(workspace);
    uint16_t* xs = wdq + (size_t)N * (size_t)K;
    const int64_t wblocks = (N + kDqRows - 1) / kDqRows;
    int64_t sblocks = 0;
    if (smooth) {                                                   // about 4 vectors of 16 bytes per thread
        sblocks = (M * K / 8 + 4 * kBlock - 1) / (4 * kBlock);
        if (sblocks > 16384) sblocks = 16384;
    }
    if (wblocks + sblocks > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    const dim3 grid((unsigned)(wblocks + sblocks));
    if (dtype == AMCT_F16) hipLaunchKernelGGL((w4_dequant_rows<true>), grid, dim3(kBlock), 0, st, a, wdq, xs, (unsigned)wblocks);
    else hipLaunchKernelGGL((w4_dequant_rows<false>), grid, dim3(kBlock), 0, st, a, wdq, xs, (unsigned)wblocks);
    const void* xa = smooth ? (const void*)xs : x;
    char* const rest = reinterpret_cast<char*>(workspace) + need;
    return gemm16_tiles(xa, wdq, bias, out, M, N, K, dtype, rest, workspace_bytes - need, st);
}

// Block shape of the kernels with specialised waves (3: 64x64, 4: 128x64, 1: 128x128; 0: they do not apply) and the number
// of K slices of the launch.  K is split over blocks when the tiles alone would leave CUs idle (few output columns, long
// rows: the down projection of an MLP) or when a row has more groups than the kernel's factor table holds; a slice is
// at least 2048 elements.  max_rounds: 1 = only launches whose 128x128 blocks run at once; 2 = the rule for int8 weights below.
struct SpecPlan {
    int shape;
    int splits;
};
static SpecPlan spec_plan(int64_t M, int64_t N, int64_t K, int group, int64_t cus, int max_rounds) {
    SpecPlan p{0, 1};
    if (M <= 0 || cus <= 0 || K % 256 != 0 || K >= 65536 || group % 64 != 0 || group <= 0 || K % group != 0) return p;
    const int64_t mt = (M + 127) / 128, nt64 = (N + 63) / 64, nt128 = (N + 127) / 128;
    int64_t blocks;
    if (M <= 64 && nt64 <= cus) p.shape = 3, blocks = nt64;
    else if (mt * nt64 <= cus) p.shape = 4, blocks = mt * nt64;
    else if (mt * nt128 <= cus ||
             (max_rounds > 1 && (M <= 384 || (M <= 512 && (mt * nt128 <= max_rounds * cus || mt * nt128 > 4 * cus)))))
        // (int8 weights: any number of rounds up to 384 rows -- dequantising the weight once costs more than the rounds --
        // and up to 512 rows unless the last round of three or four would run half empty)
        p.shape = 1, blocks = mt * nt128;
    else return p;
    const int64_t units = K / 256;
    auto fits = [&](int64_t S) {                                    // the groups of every slice fit the factor table
        for (int64_t z = 0; z < S; ++z) {
            const int64_t k0 = units * z / S * 256, k1 = units * (z + 1) / S * 256;
            if (k1 <= k0 || (k1 - 1) / group - k0 / group + 1 > kSpecMaxG) return false;
        }
        return true;
    };
    int64_t S = cus / blocks;
    if (S > 8) S = 8;
    while (S > 1 && K / S < 2048) --S;
    if (S < 1) S = 1;
    while (S <= 16 && S <= units && !fits(S)) ++S;
    if (S > 16 || S > units || mt > 65535) return SpecPlan{0, 1};
    p.splits = (int)S;
    return p;
}
static size_t spec_part_bytes(const SpecPlan& p, int64_t M, int64_t N) {
    return p.shape && p.splits > 1 ? (size_t)p.splits * (size_t)M * (size_t)N * 4 : 0;
}

// The kernels with specialised waves for int4 (WB = 4) or int8 (WB = 8) weights, with the plan above.  `smooth`: the
// activations go through the pre-pass into the workspace first (M * K * 2 bytes; the partial sums of a split launch
// follow).  only_split: serve only shapes whose plan splits K (the caller has its own kernels otherwise).
// AMCT_E_UNSUPPORTED when the shape, the operands or the workspace do not allow it (nothing has been launched then).
template <int WB>
static int spec_launch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype, const uint8_t* zeros,
                       const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group, int dtype, void* workspace,
                       size_t workspace_bytes, hipStream_t st, int max_rounds, bool only_split) {
    const int64_t G = group > 0 ? K / group : 0, cus = current_cu_count();
    SpecPlan p = spec_plan(M, N, K, group, cus, max_rounds);
    if (!p.shape || N % 8 != 0 || !aligned16(x) || !aligned16(wq) || !aligned16(out) || (reinterpret_cast<uintptr_t>(scales) & 1u) != 0 ||
        M * K * 2 >= (int64_t(1) << 32) || N * K * WB / 8 >= (int64_t(1) << 32) || N * G * 2 >= (int64_t(1) << 32))
        return AMCT_E_UNSUPPORTED;
    const size_t xs_bytes = smooth ? (size_t)(M * K * 2) : 0;
    const bool ws_ok = workspace && aligned16(workspace);
    if (smooth && !(ws_ok && workspace_bytes >= xs_bytes && aligned16(smooth))) return AMCT_E_UNSUPPORTED;
    if (p.splits > 1 && !(ws_ok && workspace_bytes >= xs_bytes + spec_part_bytes(p, M, N) && (!bias || aligned16(bias)))) {
        // no room for the partial sums: the unsplit launch, if the factor table allows it
        if (G > kSpecMaxG) return AMCT_E_UNSUPPORTED;
        p.splits = 1;
    }
    if (only_split && p.splits == 1) return AMCT_E_UNSUPPORTED;
    W4A16Args a{(const uint16_t*)x, nullptr, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group, scale_dtype,
                (uint32_t)(0x100000000ull / (uint64_t)group) + 1u, nullptr};
    if (smooth) {
        const int64_t nvec = M * K / 8;
        int64_t nb = (nvec + kBlock - 1) / kBlock;
        if (nb > 16384) nb = 16384;
        if (dtype == AMCT_F16) hipLaunchKernelGGL(smooth_rows_f16, dim3((unsigned)nb), dim3(kBlock), 0, st, a.x, (const uint16_t*)smooth, (uint16_t*)workspace, nvec, (int)(K / 8));
        else hipLaunchKernelGGL(smooth_rows, dim3((unsigned)nb), dim3(kBlock), 0, st, a.x, (const uint16_t*)smooth, (uint16_t*)workspace, nvec, (int)(K / 8));
        a.x = (const uint16_t*)workspace;
    }
    if (p.splits > 1) a.part = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + xs_bytes);
    const unsigned mt = (unsigned)((M + 127) / 128), nt64 = (unsigned)((N + 63) / 64), nt128 = (unsigned)((N + 127) / 128), S = (unsigned)p.splits;
#define AMCT_LAUNCH_SPEC(SF, AF)                                                                                       \
    {                                                                                                                  \
        if (p.shape == 3) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 1, 1, 4, AF, WB>), dim3(nt64, 1, S), dim3(kSpecThreads), 0, st, a); \
        else if (p.shape == 4) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 2, 1, 4, AF, WB>), dim3(nt64, mt, S), dim3(kSpecThreads), 0, st, a); \
        else hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 2, 2, 4, AF, WB>), dim3(nt128, mt, S), dim3(kSpecThreads), 0, st, a); \
    }
    if (dtype == AMCT_F16) {
        if (scale_dtype == AMCT_F16) AMCT_LAUNCH_SPEC(true, true) else AMCT_LAUNCH_SPEC(false, true)
    } else {
        if (scale_dtype == AMCT_F16) AMCT_LAUNCH_SPEC(true, false) else AMCT_LAUNCH_SPEC(false, false)
    }
#undef AMCT_LAUNCH_SPEC
    if (p.splits > 1) {
        int64_t nb = (M * N / 8 + kBlock - 1) / kBlock;
        if (nb > 8192) nb = 8192;
        if (dtype == AMCT_F16) hipLaunchKernelGGL((splitk_reduce16<true>), dim3((unsigned)nb), dim3(kBlock), 0, st, a.part, bias, (uint16_t*)out, M, N, p.splits);
        else hipLaunchKernelGGL((splitk_reduce16<false>), dim3((unsigned)nb), dim3(kBlock), 0, st, a.part, bias, (uint16_t*)out, M, N, p.splits);
    }
    return hip_status();
}

// out = dt(part[0] + ... + part[splits - 1] + bias) for the other files' split launches (N % 8 == 0; part, bias and out
// 16-byte aligned)
int splitk_reduce16_launch(const float* part, const float* bias, void* out, int64_t M, int64_t N, int splits, int dtype, hipStream_t st) {
    int64_t nb = (M * N / 8 + kBlock - 1) / kBlock;
    if (nb > 8192) nb = 8192;
    if (dtype == AMCT_F16) hipLaunchKernelGGL((splitk_reduce16<true>), dim3((unsigned)nb), dim3(kBlock), 0, st, part, bias, (uint16_t*)out, M, N, splits);
    else hipLaunchKernelGGL((splitk_reduce16<false>), dim3((unsigned)nb), dim3(kBlock), 0, st, part, bias, (uint16_t*)out, M, N, splits);
    return hip_status();
}

// The int8 weight-only Linear (gemm_wq16.hip) on the kernels with specialised waves: up to 384 rows, and up to 512 rows
// unless the last of three or four rounds of 128x128 blocks would run half empty (W[14336, 4096]: 74 / 81 us at 384 / 512 rows
// against 98 us for the dequantise-once form, which wins from there on: 640 rows 115 against 111 us; W[57344, 4096] at
// 256 / 384 / 512 rows: 167 / 245 / 313 us against 285 / 347 / 357 us); any number of rows when K is split.
int w8a16_spec_dispatch(const void* x, const void* smooth, const uint8_t* wq, const void* scales, int scale_dtype,
                        const uint8_t* offsets, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int group, int dtype,
                        void* workspace, size_t workspace_bytes, hipStream_t st) {
    return spec_launch<8>(x, smooth, wq, scales, scale_dtype, offsets, bias, out, M, N, K, group, dtype, workspace, workspace_bytes, st, 2, false);
}
// what that path wants lent beyond the smoothed activations: the partial sums of a split launch
size_t w8a16_spec_part_bytes(int64_t M, int64_t N, int64_t K, int group) {
    return spec_part_bytes(spec_plan(M, N, K, group, current_cu_count(), 2), M, N);
}

}  // namespace amct

using namespace amct;

extern "C" size_t amct_gemm_w4a16_workspace_bytes(int64_t M, int64_t N, int64_t K, int group, int has_smooth) {
    if (M <= 0 || N <= 0 || K <= 0 || group <= 0) return 0;
    const size_t two = two_pass_workspace(M, N, K, group, has_smooth);    // many rows: the dequantised weight as well
    if (two) return two;
    // tile kernels: x * smooth done once; long rows on few column blocks: the partial sums of the K slices behind it
    const size_t part = spec_part_bytes(spec_plan(M, N, K, group, current_cu_count(), 1), M, N);
    const size_t tiles = (has_smooth && (M > 16 || part) ? (size_t)M * (size_t)K * 2 : 0) + part;
    const size_t stream = w4a16_stream_part_bytes(M, N, K, group);     // a few rows, K in slices: its partial sums only
    return tiles > stream ? tiles : stream;
}

extern "C" int amct_gemm_w4a16_weight_rounded(int64_t M, int64_t N, int64_t K, int group, int dtype, size_t workspace_bytes) {
    if (M < 0 || N <= 0 || K <= 0 || group <= 0) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    // the weight-streaming kernel is the only one that keeps the integer weight; amct_gemm_w4a16 tries it first
    return M <= 16 && w4a16_stream_takes(M, N, K, group, workspace_bytes) ? 0 : 1;
}

extern "C" int amct_gemm_w4a16(const void* x, const void* smooth, const uint8_t* wq, const void* scales,
                               int scale_dtype, const uint8_t* zeros, const float* bias, void* out, int64_t M,
                               int64_t N, int64_t K, int group, int dtype, void* workspace, size_t workspace_bytes,
                               amct_stream_t stream) {
    if (M < 0 || N <= 0 || K <= 0 || group <= 0) return AMCT_E_BADARG;
    if (M != 0 && (!x || !wq || !scales || !zeros || !out)) return AMCT_E_BADARG;   // M == 0 reads nothing
    if (scale_dtype != AMCT_F16 && scale_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    if (K % group != 0 || K % 2 != 0) return AMCT_E_ALIGN;
    if (M == 0) return AMCT_OK;
    if (M <= 16) {                                                 // K of 1024 / 2048 / 4096, group 128: the weight-streaming kernel
        const int rc = w4a16_stream_dispatch(x, smooth, wq, scales, scale_dtype, zeros, bias, out, M, N, K, group, dtype,
                                             workspace, workspace_bytes, (hipStream_t)stream);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    // long rows on few column blocks: specialised waves, K split over blocks.  Measured on W[4096, 14336] / W[4096, 8192]
    // (us, the older kernels for a few rows / this path): M = 2: 17.3 / 20.5 and 12.2 / 14.1; M = 4: 29.3 / 20.9 and
    // 12.7 / 14.4; M = 8: 52.6 / 20.8 and 21.4 / 14.5; M = 32: 78.7 / 21.3 and 46.1 / 15.3.
    // Rows whose 256-element units do not split evenly over four waves leave the older kernels one wave per block
    // (W[4096, 11008], M = 1: 43 us), so they come here for any M; many rows come here too while the 128x128 blocks fit
    // the CUs in one round (W[1024, 4096], M = 2048: 27 us against 51 us for the dequantise-once form).
    if (M >= 8 || (M >= 4 && K >= 12288) || (K / 256) % 4 != 0) {
        // (below kTwoPassFrom rows only launches that split K: the dispatch further down takes the unsplit ones)
        const int rc = spec_launch<4>(x, smooth, wq, scales, scale_dtype, zeros, bias, out, M, N, K, group, dtype, workspace,
                                      workspace_bytes, (hipStream_t)stream, 1, M < kTwoPassFrom);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    // fp16 activations: otherwise the tile kernels below or the kernels shared with the int8-weight path (gemm_wq16.hip),
    // which smooth in the tile
    if (dtype == AMCT_F16) {
        if (M >= kTwoPassFrom) {
            const int rc = two_pass(x, smooth, wq, scales, scale_dtype, zeros, bias, out, M, N, K, group, dtype, workspace,
                                    workspace_bytes, (hipStream_t)stream);
            if (rc != AMCT_E_UNSUPPORTED) return rc;
        }
        // more than 16 rows: the tile kernels with fp16 operands (the same bodies: the dequantised weight and the smoothed
        // activations are rounded to fp16 instead of bf16, one v_cvt_pk_f16_f32 per pair, and the MFMAs are the f16 ones);
        // the same conditions and block shapes as for bf16 below (up to 64 rows only the kernels with specialised waves,
        // i.e. K % 256 == 0), and the caller's workspace when the activations are to be smoothed
        {
            hipStream_t st = (hipStream_t)stream;
            const int64_t cus = current_cu_count();
            const int64_t mt = (M + 127) / 128, nt64 = (N + 63) / 64, nt128 = (N + 127) / 128, nt256 = (N + 255) / 256, G = K / group;
            const bool ok = aligned16(x) && aligned16(wq) && (!smooth || aligned16(smooth)) && aligned16(out) && K % 128 == 0 &&
                            K < 65536 && N % 8 == 0 && group % 64 == 0 && M * K * 2 < (int64_t(1) << 32) &&
                            N * (K / 2) < (int64_t(1) << 32) && N * G * 2 < (int64_t(1) << 32) && cus > 0 &&
                            (M > 64 || (M > 16 && K % 256 == 0 && G <= kSpecMaxG)) &&   // few rows: only the kernels with specialised waves
                            mt <= 65535 && (!smooth || (workspace && workspace_bytes >= (size_t)(M * K * 2) && aligned16(workspace)));
            if (ok) {
                W4A16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group,
                            scale_dtype, (uint32_t)(0x100000000ull / (uint64_t)group) + 1u};
                if (smooth) {
                    const int64_t nvec = M * K / 8;
                    int64_t nb = (nvec + kBlock - 1) / kBlock;
                    if (nb > 16384) nb = 16384;
                    hipLaunchKernelGGL(smooth_rows_f16, dim3((unsigned)nb), dim3(kBlock), 0, st, a.x, a.smooth, (uint16_t*)workspace, nvec, (int)(K / 8));
                    a.x = (const uint16_t*)workspace;
                    a.smooth = nullptr;
                }
                int shape = 0;
                if (M <= 64 && nt64 <= cus) shape = 3;
                else if (mt * nt64 <= cus) shape = 4;
                else if (mt * nt128 <= cus) shape = 1;
                else if (mt * nt256 <= cus || M < 256) shape = 2;
                const bool spec = K % 256 == 0 && G <= kSpecMaxG;   // 4 matrix + 8 data-movement waves, as for bf16
                const dim3 grid((unsigned)((N + kQN - 1) / kQN), (unsigned)((M + kQM - 1) / kQM));
#define AMCT_LAUNCH_WIDE_F16(SF)                                                                                       \
    {                                                                                                                  \
        if (shape == 3 && spec) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 1, 1, 4, true>), dim3((unsigned)nt64, 1), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 4 && spec) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 2, 1, 4, true>), dim3((unsigned)nt64, (unsigned)mt), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 1 && spec) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 2, 2, 4, true>), dim3((unsigned)nt128, (unsigned)mt), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 3) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 1, 1, 3, 3, true>), dim3((unsigned)nt64, 1), dim3(256), 0, st, a); \
        else if (shape == 4) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 2, 1, 3, 3, true>), dim3((unsigned)nt64, (unsigned)mt), dim3(256), 0, st, a); \
        else if (shape == 1) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 2, 2, 3, 3, true>), dim3((unsigned)nt128, (unsigned)mt), dim3(256), 0, st, a); \
        else if (shape == 2 && M > 256 && (M + 255) / 256 * nt128 <= cus) hipLaunchKernelGGL((w4a16_tile_wide<SF, 4, 2, 2, 2, 3, 3, true>), dim3((unsigned)nt128, (unsigned)((M + 255) / 256)), dim3(512), 0, st, a); \
        else if (shape == 2) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 4, 2, 2, 3, 3, true>), dim3((unsigned)nt256, (unsigned)mt), dim3(512), 0, st, a); \
        else hipLaunchKernelGGL((w4a16_tile_wide16<SF, 2, 4, 4, 2, 2, 2, true>), grid, dim3(kQThreads), 0, st, a);     \
    }
                if (scale_dtype == AMCT_F16) AMCT_LAUNCH_WIDE_F16(true)
                else AMCT_LAUNCH_WIDE_F16(false)
#undef AMCT_LAUNCH_WIDE_F16
                return hip_status();
            }
        }
        return wq16_int4_f16(x, smooth, wq, scales, scale_dtype, zeros, bias, out, M, N, K, group, (hipStream_t)stream);
    }
    W4A16Args a{(const uint16_t*)x, (const uint16_t*)smooth, wq, scales, zeros, bias, (uint16_t*)out, M, N, K, group, scale_dtype,
                (uint32_t)(0x100000000ull / (uint64_t)group) + 1u};
    hipStream_t st = (hipStream_t)stream;
    if (M >= kTwoPassFrom) {                                       // many rows and a workspace for the dequantised weight
        const int rc = two_pass(x, smooth, wq, scales, scale_dtype, zeros, bias, out, M, N, K, group, dtype, workspace,
                                workspace_bytes, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    const bool vec_ok = aligned16(x) && aligned16(wq) && (!smooth || aligned16(smooth)) && group % 32 == 0;
    if (vec_ok && M <= 16 && K % 256 == 0 && K < 65536 && group % 32 == 0 && K / group <= 128 && (N * (K / group)) % 16 == 0 &&
        aligned16(scales) && aligned16(zeros)) {
        // Few activations (M * K small): narrow blocks of 4 waves, several per CU, so that one block's start-up
        // and reduction overlap with another's streaming.  More activations: wide blocks, which stage the
        // activations fewer times.
        const int iters = (int)(K / 256);
        const bool few = M * K <= 32768;
        const int waves = (!few && iters % 8 == 0) ? 8 : iters % 4 == 0 ? 4 : 1;
        const int tn = M * K <= 8192 ? 1 : few ? 2 : 4;
        const size_t lds = decode_lds_bytes(M, K, group, waves, tn);
        int rc = AMCT_E_UNSUPPORTED;
        if (lds) {
            if (tn == 1) rc = smooth ? launch_decode_lds_w<true, 1>(a, waves, lds, st) : launch_decode_lds_w<false, 1>(a, waves, lds, st);
            else if (tn == 2) rc = smooth ? launch_decode_lds_w<true, 2>(a, waves, lds, st) : launch_decode_lds_w<false, 2>(a, waves, lds, st);
            else rc = smooth ? launch_decode_lds_w<true, 4>(a, waves, lds, st) : launch_decode_lds_w<false, 4>(a, waves, lds, st);
        }
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    // The weight-streaming kernel below serves 16 < M <= 24 (25 us on W[14336,4096] at M = 17, 29 us at M = 32, 40 us
    // at M = 64; 64x64 tiles take 26 us for any M <= 64, 22 us with specialised waves, which then start at M = 17), and
    // larger M up to 64 where the tile kernels do not apply; when the activations are to be smoothed the tile path pays
    // a pre-pass, so the switch of the plain tiles comes later.
    const bool tiles_apply = vec_ok && K % 128 == 0 && K < 65536 && N % 8 == 0 && aligned16(out) && group % 64 == 0 &&
                             M * K * 2 < (int64_t(1) << 32) && N * (K / 2) < (int64_t(1) << 32) &&
                             N * (K / group) * 2 < (int64_t(1) << 32) &&
                             (!smooth || (workspace && workspace_bytes >= (size_t)(M * K * 2) && aligned16(workspace)));
    const bool spec_small = K % 256 == 0 && K / group <= kSpecMaxG;   // the 22 us kernel serves this shape
    const int64_t small_tiles_from = spec_small ? 17 : smooth ? 41 : 25;
    if (vec_ok && M <= 64 && K % 128 == 0 && K < 65536 && group % 32 == 0 && !(tiles_apply && M >= small_tiles_from)) {
        const dim3 grid((unsigned)((N + kDN - 1) / kDN));
        const int iters = (int)(K / 128);
#define AMCT_DEC2(MT, SM)                                                                                    \
    {                                                                                                        \
        if (iters % 8 == 0 && MT < 4) hipLaunchKernelGGL((w4a16_decode<MT, (MT < 4 ? 8 : 4), SM>), grid, dim3(512), 0, st, a); \
        else if (iters % 4 == 0) hipLaunchKernelGGL((w4a16_decode<MT, 4, SM>), grid, dim3(256), 0, st, a);   \
        else if (iters % 2 == 0) hipLaunchKernelGGL((w4a16_decode<MT, 2, SM>), grid, dim3(128), 0, st, a);   \
        else hipLaunchKernelGGL((w4a16_decode<MT, 1, SM>), grid, dim3(64), 0, st, a);                        \
    }
#define AMCT_DEC(MT)                                                                                         \
    {                                                                                                        \
        if (smooth) AMCT_DEC2(MT, true) else AMCT_DEC2(MT, false)                                            \
    }
        if (M <= 16) AMCT_DEC(1)
        else if (M <= 32) AMCT_DEC(2)
        else AMCT_DEC(4)
#undef AMCT_DEC2
#undef AMCT_DEC
        return hip_status();
    }
    if (vec_ok && (M > 64 || (tiles_apply && M >= small_tiles_from)) && K % 128 == 0 && K < 65536 && N % 8 == 0 && aligned16(out)) {
        const dim3 grid((unsigned)((N + kQN - 1) / kQN), (unsigned)((M + kQM - 1) / kQM));
        if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
        const int64_t G = K / group;
        const bool fits = group % 64 == 0 && M * K * 2 < (int64_t(1) << 32) && N * (K / 2) < (int64_t(1) << 32) &&
                          N * G * 2 < (int64_t(1) << 32);
        if (smooth && workspace && workspace_bytes >= (size_t)(M * K * 2) && aligned16(workspace)) {
            // smoothing once into the lent workspace, then the kernel without the in-tile multiply
            const int64_t nvec = M * K / 8;
            int64_t nb = (nvec + kBlock - 1) / kBlock;
            if (nb > 16384) nb = 16384;
            hipLaunchKernelGGL(smooth_rows, dim3((unsigned)nb), dim3(kBlock), 0, st, a.x, a.smooth, (uint16_t*)workspace, nvec, (int)(K / 8));
            a.x = (const uint16_t*)workspace;
            a.smooth = nullptr;
            smooth = nullptr;
        }
        const bool wide = !smooth && fits;
        if (wide) {
            // Block shape: as long as all tiles of a launch run at once, small tiles on many CUs beat large tiles on
            // few (the weight stream is the bulk of the traffic for medium M): 128x128 blocks (with specialised waves
            // when K % 256 == 0: 38 us against 51 us on W[14336,4096], M = 129 .. 256; the first-generation kernel took
            // 97 us; 64-column blocks of 4 waves, a quarter of a weight row per thread and step, while they still fit the
            // CUs in one round: 64x64 for M <= 64, 26 us, and 128x64 for M <= 128, 34 us; with 4 matrix and 8 data-movement
            // waves when K % 256 == 0: 20 us and 24 us; fetching the weights 8 steps ahead instead of 4 changed nothing, and two
            // row tiles of 128x64 blocks lose to one 128x128 block for 128 < M <= 256: 46 us against 39 us), then blocks of 8 waves: 256x128 for 256 < M <= 512 (65 us; half the
            // dequantisation of 128x256 blocks, which take 72 .. 75 us; the first-generation kernel took 96 us), 128x256 where those do not fit the CUs, each with three LDS
            // stages; 256x256 with two stages otherwise.  (Mixing in 256x192
            // blocks as the W8A8 launch does was measured neutral here: the narrow tile dequantises as many weights.)
            const int64_t cus = current_cu_count();
            const int64_t mt = (M + 127) / 128, nt64 = (N + 63) / 64, nt128 = (N + 127) / 128, nt256 = (N + 255) / 256;
            int shape = 0;
            if (cus > 0 && M <= 64 && nt64 <= cus) shape = 3;
            else if (cus > 0 && mt * nt64 <= cus) shape = 4;
            else if (cus > 0 && mt * nt128 <= cus) shape = 1;
            else if (cus > 0 && (mt * nt256 <= cus || M < 256)) shape = 2;
            if (mt > 65535) return AMCT_E_UNSUPPORTED;
            // 256x256 tiles run on v_mfma_f32_16x16x32_bf16: under the part's power limit it sustains more than the
            // 32x32x16 form on non-constant operands (register-only loops: 1.81 - 1.97 against 1.67 - 1.81 PFLOP/s) at equal
            // LDS traffic per wave tile: 217.5 against 225.2 us on M = 2048, N = 14336, K = 4096 (pre-pass included).
            constexpr bool mi16 = true;
#define AMCT_LAUNCH_WIDE(SF)                                                                                           \
    {                                                                                                                  \
        if (shape == 3 && K % 256 == 0 && G <= kSpecMaxG) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 1, 1>), dim3((unsigned)nt64, 1), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 4 && K % 256 == 0 && G <= kSpecMaxG) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3, 2, 1>), dim3((unsigned)nt64, (unsigned)mt), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 3) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 1, 1, 3>), dim3((unsigned)nt64, 1), dim3(256), 0, st, a);          \
        else if (shape == 4) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 2, 1, 3>), dim3((unsigned)nt64, (unsigned)mt), dim3(256), 0, st, a); \
        else if (shape == 1 && K % 256 == 0 && G <= kSpecMaxG) hipLaunchKernelGGL((w4a16_tile_spec<SF, 3>), dim3((unsigned)nt128, (unsigned)mt), dim3(kSpecThreads), 0, st, a); \
        else if (shape == 1) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 2, 2, 2, 3>), dim3((unsigned)nt128, (unsigned)mt), dim3(256), 0, st, a); \
        else if (shape == 2 && M > 256 && (M + 255) / 256 * nt128 <= cus) hipLaunchKernelGGL((w4a16_tile_wide<SF, 4, 2, 2, 2, 3>), dim3((unsigned)nt128, (unsigned)((M + 255) / 256)), dim3(512), 0, st, a); \
        else if (shape == 2) hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 4, 2, 2, 3>), dim3((unsigned)nt256, (unsigned)mt), dim3(512), 0, st, a); \
        else if (mi16) hipLaunchKernelGGL((w4a16_tile_wide16<SF, 2, 4, 4, 2, 2>), grid, dim3(kQThreads), 0, st, a);    \
        else hipLaunchKernelGGL((w4a16_tile_wide<SF, 2, 4, 4, 2, 2>), grid, dim3(kQThreads), 0, st, a);                \
    }
            if (scale_dtype == AMCT_F16) AMCT_LAUNCH_WIDE(true)
            else AMCT_LAUNCH_WIDE(false)
#undef AMCT_LAUNCH_WIDE
            return hip_status();
        }
        if (M >= 256) {
            if (smooth) hipLaunchKernelGGL((w4a16_tile_dma<true>), grid, dim3(kQThreads), 0, st, a);
            else hipLaunchKernelGGL((w4a16_tile_dma<false>), grid, dim3(kQThreads), 0, st, a);
            return hip_status();
        }
    }
    if (vec_ok && K % kTK == 0) {
        const dim3 grid((unsigned)((N + kTN - 1) / kTN), (unsigned)((M + kTM - 1) / kTM));
        if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
        hipLaunchKernelGGL(w4a16_tile, grid, dim3(kBlock), 0, st, a);
        return hip_status();
    }
    const int64_t nb = (M * N + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(w4a16_general, dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    return hip_status();
}
