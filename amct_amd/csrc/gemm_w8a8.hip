// K6: W8A8 Linear.  out[m,n] = cast(fp32(sum_k xq[m,k]*wq[n,k] + ibias[n]) * s_ch[n] * s_tok[m] + fbias[n])
// Reference call site: amct_pytorch/deploy_op/npu_quantization_linear.py:100-102.
//
// Both operands are K-contiguous, which is the natural operand order of the gfx950 int8 MFMAs
// (v_mfma_i32_32x32x32_i8: lane l supplies 16 consecutive k-bytes of row l%32, k-half l/32;
//  v_mfma_i32_16x16x64_i8: row l%16, k-quarter l/16).
//   large tiles   : 256x256 block tile, 8 waves of 128x64, LDS stages of 128 bytes of K filled by direct
//                   global->LDS loads, fragment reads software-pipelined against the MFMAs in a pinned
//                   issue order; when the tile count does not fill the CUs evenly, one launch mixes in
//                   256x192 tiles.  With K a multiple of 128 the 16x16x64 form runs (w8a8_dma_body16), else the
//                   32x32x32 form with 64-byte rows (w8a8_dma_body).
//   tile kernel   : 128x128 block tile, 4 waves of 64x64, BK = 128 bytes, two register stages of
//                   prefetch (shapes the large-tile kernel does not take).
//   decode kernels: M <= 16: activations staged once per block in LDS, the weight streamed once straight
//                   from HBM into MFMA operands (v_mfma_i32_16x16x64_i8), split-K across the waves; for K of 1024,
//                   2048 or 4096 the variant in gemm_w8a8_stream.hip (all weight loads of the launch in flight at
//                   once, whole 128-byte lines per load instruction).
//   medium tiles  : 16 < M up to a few hundred rows: the large-tile body with 128x128 (4 waves) or 128x256 blocks and
//                   three LDS stages, chosen so that all blocks of the launch run at once.
//   skinny kernel : 16 < M <= 32 when K is not a multiple of 128 (and M <= 16 shapes the decode kernel does not
//                   take): as above with the activations read from L2 per MFMA.
//   general kernel: any shape, one output per thread.
#include "amct_common.h"

#include <type_traits>
#include "gemm_plan.h"

namespace amct {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct W8A8Args {
    const int8_t* xq;
    const int8_t* wq;
    const float* s_tok;
    const float* s_ch;
    const void* bias;
    void* out;
    int32_t* acc_out;
    int64_t M, N, K;
    int bias_kind;
    int out_dtype;
    int32_t* part;                                   // split-K launches (gridDim.z > 1): int32 partial sums [gridDim.z, M, N]
};

AMCT_DEV void w8a8_epilogue(const W8A8Args& a, int64_t m, int64_t n, int32_t acc) {
    if (a.bias_kind == 1) acc += reinterpret_cast<const int32_t*>(a.bias)[n];
    if (a.acc_out) a.acc_out[m * a.N + n] = acc;
    float f = (float)acc;
    f = f * a.s_ch[n];
    if (a.s_tok) f = f * a.s_tok[m];
    if (a.bias_kind == 2) f = f + reinterpret_cast<const float*>(a.bias)[n];
    const int64_t o = m * a.N + n;
    if (a.out_dtype == AMCT_BF16) store_scalar<AMCT_BF16>(a.out, o, f);
    else if (a.out_dtype == AMCT_F16) store_scalar<AMCT_F16>(a.out, o, f);
    else store_scalar<AMCT_F32>(a.out, o, f);
}

// ---------------------------------------------------------------------------
// tile kernel
// ---------------------------------------------------------------------------
constexpr int kBM = 128, kBN = 128, kBK = 128;      // BK in bytes (= int8 elements)
constexpr int kRow = kBK + 16;                      // padded LDS row: conflict-free ds_read_b128
constexpr int kLoads = (kBM * kBK / 16) / kBlock;   // 16-byte chunks per thread and operand: 4

AMCT_DEV uint4 ld_chunk_or_zero(const int8_t* base, int64_t row, int64_t rows, int64_t K, int64_t k) {
    // rows beyond the matrix are clamped (their results are never stored); k beyond K reads zero
    // (the load itself is unconditional: a predicated load would force a wait on every load)
    const int64_t r = row < rows ? row : rows - 1;
    const int64_t kk = k < K ? k : K - 16;
    uint4 v = ldg16(base + r * K + kk);
    if (k >= K) v = make_uint4(0, 0, 0, 0);
    return v;
}

template <int ODT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2, 2))) void w8a8_tile(W8A8Args a) {
    __shared__ __attribute__((aligned(16))) int8_t As[2][kBM * kRow];
    __shared__ __attribute__((aligned(16))) int8_t Bs[2][kBN * kRow];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * kBM, n0 = (int64_t)blockIdx.x * kBN;
    const int ld_row = tid >> 3, ld_chunk = tid & 7;            // 8 chunks of 16 B per row
    const int nsteps = (int)((a.K + kBK - 1) / kBK);

    // two register stages: the loads of step s+2 are issued while step s is computed and the
    // registers of step s+1 (loaded one iteration earlier) are moved to the free LDS buffer, so two
    // K-steps of global traffic are in flight behind the MFMAs
    uint4 ra[2][kLoads], rb[2][kLoads];
    auto load_global = [&](int step, uint4* pa, uint4* pb) {
        const int64_t k = (int64_t)step * kBK + ld_chunk * 16;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            pa[i] = ld_chunk_or_zero(a.xq, m0 + ld_row + 32 * i, a.M, a.K, k);
            pb[i] = ld_chunk_or_zero(a.wq, n0 + ld_row + 32 * i, a.N, a.K, k);
        }
    };
    auto store_lds = [&](int buf, const uint4* pa, const uint4* pb) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            *reinterpret_cast<uint4*>(&As[buf][(ld_row + 32 * i) * kRow + ld_chunk * 16]) = pa[i];
            *reinterpret_cast<uint4*>(&Bs[buf][(ld_row + 32 * i) * kRow + ld_chunk * 16]) = pb[i];
        }
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
    auto compute = [&](int cur) {
#pragma unroll
        for (int ks = 0; ks < kBK / 32; ++ks) {
            v4i fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const v4i*>(&As[cur][(wm * 64 + i * 32 + frag_row) * kRow + ks * 32 + frag_k]);
                fb[i] = *reinterpret_cast<const v4i*>(&Bs[cur][(wn * 64 + i * 32 + frag_row) * kRow + ks * 32 + frag_k]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    // loads past the last step re-read the last step (never used) instead of branching around the load
    const int last = nsteps - 1;
    load_global(0, ra[0], rb[0]);
    load_global(1 < last ? 1 : last, ra[1], rb[1]);
    store_lds(0, ra[0], rb[0]);
    __syncthreads();
    for (int step = 0; step < nsteps; step += 2) {
        // even step: LDS buffer 0 holds step, registers 1 hold step+1, registers 0 are free
        load_global(step + 2 < last ? step + 2 : last, ra[0], rb[0]);
        compute(0);
        store_lds(1, ra[1], rb[1]);
        __syncthreads();
        if (step + 1 >= nsteps) break;
        // odd step: LDS buffer 1 holds step+1, registers 0 hold step+2, registers 1 are free
        load_global(step + 3 < last ? step + 3 : last, ra[1], rb[1]);
        compute(1);
        store_lds(0, ra[0], rb[0]);
        __syncthreads();
    }

    // epilogue: register r of a 32x32 tile holds row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
    // Per-column and per-row factors are fetched once; fp32(acc + ibias) * s_ch * s_tok + fbias.
    float sc[2], fb[2];
    int32_t ib[2];
    int64_t ncol[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        ncol[j] = n0 + wn * 64 + j * 32 + (lane & 31);
        const int64_t nc = ncol[j] < a.N ? ncol[j] : a.N - 1;
        sc[j] = a.s_ch[nc];
        ib[j] = a.bias_kind == 1 ? reinterpret_cast<const int32_t*>(a.bias)[nc] : 0;
        fb[j] = a.bias_kind == 2 ? reinterpret_cast<const float*>(a.bias)[nc] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (m >= a.M) continue;
            const float tk = a.s_tok ? a.s_tok[m] : 1.0f;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (ncol[j] >= a.N) continue;
                const int32_t v = acc[i][j][r] + ib[j];
                const int64_t o = m * a.N + ncol[j];
                if (a.acc_out) a.acc_out[o] = v;
                float f = (float)v * sc[j];
                if (a.s_tok) f = f * tk;
                if (a.bias_kind == 2) f = f + fb[j];
                store_scalar<ODT>(a.out, o, f);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// large-tile kernel: 256x256 (or 256x192) block tile, 8 waves, LDS stages of 128 (or 64) bytes of K filled by
// direct global->LDS loads (global_load_lds_dwordx4: no VGPR staging, no ds_write), one barrier per stage,
// epilogue transposed through LDS so that every lane stores 16 contiguous bytes.
//
// A direct-to-LDS load writes the 64 lanes' 16-byte pieces to 1024 contiguous LDS bytes, so the LDS layout is
// unpadded [row][LK bytes]; bank conflicts are avoided by a swizzle instead (measured conflict-free with
// SQ_LDS_BANK_CONFLICT), applied by choosing which global chunk a lane fetches.  The loads and their s_waitcnt
// are inline asm: the compiler would otherwise wait for ALL outstanding direct-to-LDS loads before every LDS read.
// ---------------------------------------------------------------------------
constexpr int kLK = 64;                                             // smallest K granule of the large-tile kernel

// one direct-to-LDS load: a wave-uniform 64-bit base in SGPRs and a 32-bit byte offset per lane (no vector ALU
// work per load); lane l's 16 bytes land at lds_addr + 16 * l
AMCT_DEV void dma16s(uint32_t lds_addr, const void* sbase, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
template <int N> AMCT_DEV void wait_dma_lds() { asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(N) : "memory"); }

// WM x WN waves of (32*TI) x (32*TJ) each: block tile (32*TI*WM) x (32*TJ*WN); STAGES LDS stages of LK bytes
// of K (64 or 128).  The body is a device function so that one launch can mix block shapes (see w8a8_tile_mix).
template <int WM, int WN, int TI, int TJ, int STAGES, int LK>
struct DmaTile {
    static constexpr int kLM = 32 * TI * WM, kLN = 32 * TJ * WN, kWaves = WM * WN;
    static constexpr int kLStageBytes = (kLM + kLN) * LK;
    static constexpr int kRP = 1024 / LK;                          // rows per 1 KiB piece
    static constexpr int kLW = kWaves / 2;                         // waves that issue the direct-to-LDS loads
    static constexpr int kNA = kLM / kRP / kLW;                    // A pieces per loading wave and stage
    static constexpr int kNB = (kLN / kRP + kLW - 1) / kLW;        // B pieces per loading wave (the last ones may repeat)
    static constexpr int kPPW = kNA + kNB;
    static constexpr int kEpiBytes = kWaves * 16384;
    static constexpr int kSmem = STAGES * kLStageBytes > kEpiBytes ? STAGES * kLStageBytes : kEpiBytes;
    static constexpr int kSmemFac = kSmem + 3 * 256 * 4;           // with the epilogue's factor table behind it
    static_assert((kLM / kRP) % kLW == 0, "the A pieces must divide evenly among the loading waves");
    static_assert(kSmemFac <= 160 * 1024, "LDS");
};

template <int ODT, int WM, int WN, int TI, int TJ, int STAGES, int LK>
AMCT_DEV void w8a8_dma_body(const W8A8Args& a, int8_t* smem, const int64_t m0, const int64_t n0) {
    using Sh = DmaTile<WM, WN, TI, TJ, STAGES, LK>;
    constexpr int kLM = Sh::kLM, kLN = Sh::kLN, kRP = Sh::kRP, kNA = Sh::kNA, kNB = Sh::kNB, kPPW = Sh::kPPW;
    constexpr int kLStageBytes = Sh::kLStageBytes, kWaves = Sh::kWaves, kLW = Sh::kLW;
    constexpr int kCH = LK / 16;                                    // 16-byte chunks per row
    constexpr int kKS = LK / 32;                                    // MFMA k-slices per stage
    static_assert(LK == 64 || LK == 128, "row length");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    // Split K (gridDim.z > 1): block z takes the steps [steps z / S, steps (z + 1) / S) of every row and leaves its int32
    // sums in a.part[z]; w8a8_splitk_reduce adds them (exactly) and applies the epilogue.  Rows keep their stride a.K.
    const uint32_t steps_all = (uint32_t)(a.K / LK);
    const uint32_t step0 = steps_all * blockIdx.z / gridDim.z;
    const int nsteps = (int)(steps_all * (blockIdx.z + 1) / gridDim.z - step0);
    const int last = nsteps - 1;
    const int8_t* const xk = a.xq + (int64_t)step0 * LK;
    const int8_t* const wk = a.wq + (int64_t)step0 * LK;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t*)smem;
    // Rows are LK bytes, unpadded (a direct-to-LDS load writes the 64 lanes' 16-byte pieces to 1024 contiguous
    // bytes); 16-byte chunk c of row r lives at chunk position c ^ swz(r), which spreads the 16 rows that one
    // phase of a 16-byte fragment read touches over all banks.
    auto swz = [](int r) { return LK == 64 ? (r >> 2) & 3 : (r >> 1) & 7; };

    // this wave's 1 KiB pieces of a stage: kNA pieces of A rows, then kNB pieces of B rows.  A load is addressed
    // as (operand base + LK * step) in SGPRs plus a constant 32-bit byte offset per lane and piece (the host
    // admits only operands below 4 GiB to this kernel).
    const bool loader = wave >= kWaves - kLW;                       // the last kLW waves: one per SIMD when kLW = 4
    const int lw = loader ? wave - (kWaves - kLW) : 0;
    uint32_t goff[kPPW];
    {
        const int rin = lane / kCH;                                 // row inside the piece
        const int pc = lane % kCH;                                  // physical chunk this lane fills
#pragma unroll
        for (int j = 0; j < kPPW; ++j) {
            int64_t r;
            int lr;                                                 // row inside the operand's LDS tile
            if (j < kNA) {
                lr = (lw * kNA + j) * kRP + rin;
                r = m0 + lr < a.M ? m0 + lr : a.M - 1;
            } else {
                // a wave beyond the last piece fetches the last piece again: same bytes to the same place
                const int pb = lw * kNB + (j - kNA) < kLN / kRP ? lw * kNB + (j - kNA) : kLN / kRP - 1;
                lr = pb * kRP + rin;
                r = n0 + lr < a.N ? n0 + lr : a.N - 1;
            }
            goff[j] = (uint32_t)(r * a.K + (pc ^ swz(lr)) * 16);
        }
    }
    auto dma_one = [&](int stg, int step, int j) {
        if (j < kNA) {
            dma16s(lds0 + stg * kLStageBytes + (lw * kNA + j) * 1024, xk + (int64_t)step * LK, goff[j]);
        } else {
            const int pb = lw * kNB + (j - kNA) < kLN / kRP ? lw * kNB + (j - kNA) : kLN / kRP - 1;
            dma16s(lds0 + stg * kLStageBytes + kLM * LK + pb * 1024, wk + (int64_t)step * LK, goff[j]);
        }
    };
    auto dma_stage = [&](int stage, int step) {
        if (loader) {
#pragma unroll
            for (int j = 0; j < kPPW; ++j) dma_one(stage, step, j);
        }
    };

    // fragment offsets of k-slice ks: lane reads row (tile base + lane%32), logical chunk 2*ks + lane/32
    int offA[kKS], offB[kKS];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
        const int r = lane & 31;
        const int phys = (ks * 2 + (lane >> 5)) ^ swz(r);
        offA[ks] = (wm * 32 * TI + r) * LK + phys * 16;
        offB[ks] = kLM * LK + (wn * 32 * TJ + r) * LK + phys * 16;
    }

    v16i acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) dma_stage(s, s < last ? s : last);

    // The factors of the epilogue (per column: s_ch and the float bias; per row: s_tok; absent ones replaced by their
    // neutral elements) are fetched now, one or two per thread, and parked in an LDS table behind the stages: read at the
    // end of the tile they would cost a round trip to memory with nothing to hide it.  An integer bias is where the
    // accumulators start (its loads wait together with the first stage's), so the epilogue never sees it.
    static_assert(kLN + kLM <= kWaves * 64 && kLN <= 256 && kLM <= 256, "one factor per thread");
    float fac0 = 1.0f, fac1 = -0.0f;
    if (tid < kLN) {
        const int64_t n = n0 + tid < a.N ? n0 + tid : a.N - 1;
        if (a.s_ch) fac0 = a.s_ch[n];
        if (a.bias_kind == 2) fac1 = reinterpret_cast<const float*>(a.bias)[n];
    } else if (tid - kLN < kLM) {
        const int64_t m = m0 + (tid - kLN) < a.M ? m0 + (tid - kLN) : a.M - 1;
        if (a.s_tok) fac0 = a.s_tok[m];
    }
    if (a.bias_kind == 1 && gridDim.z == 1) {
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const int64_t n = n0 + wn * 32 * TJ + j * 32 + (lane & 31);
            const int32_t b = reinterpret_cast<const int32_t*>(a.bias)[n < a.N ? n : a.N - 1];
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = b;
        }
    }

    // Software pipeline over k-slices of 32 bytes: while the MFMAs of one slice run, the fragments of the next
    // slice are read from LDS.  Before the last slice of a stage the waves meet: every wave then holds that
    // slice's fragments in registers (lgkmcnt(0)), so the stage is free for the loads of step s + STAGES, and
    // the loads of step s + 1 have landed (those of the STAGES-2 steps after it stay in flight).
    // The direct-to-LDS loads of a step are issued by half of the waves (the last WM*WN/2, one per SIMD with
    // the usual round-robin placement) in one burst right after the barrier: a wave stalls at such a load while
    // the memory pipeline is busy, and the other wave of its SIMD keeps the matrix pipe fed meanwhile (3 %
    // faster than every wave issuing its share between its MFMAs).
    // The issue order is pinned instruction by instruction (a scheduling barrier after each): fragment reads
    // in the shadow of the MFMAs, the MFMAs of the slices before the barrier issued BEFORE the wait, the first
    // MFMA of the last slice right after the barrier (and the loads).  Left alone, the optimiser moves MFMAs behind the
    // barrier (the matrix pipe then idles while the waves meet) and, with a conditional read at the end of the
    // loop, waits for the youngest LDS reads too early.  The loop is therefore branch-free: the last iteration
    // reads one stage too far (valid LDS, values unused).
    constexpr int kNM = TI * TJ, kNR = TI + TJ;
    constexpr int kRPM = (kNR + kNM - 1) / kNM;                     // fragment reads behind each MFMA
    // fragment q in the order the MFMAs need them: A0, B0, B1, .., A1, A2, ..
    auto read_one = [&](int stg, int ks, int q, v4i (&fa)[TI], v4i (&fb)[TJ]) {
        const int8_t* st = smem + stg * kLStageBytes;
        if (q == 0) fa[0] = *reinterpret_cast<const v4i*>(st + offA[ks]);
        else if (q <= TJ) fb[q - 1] = *reinterpret_cast<const v4i*>(st + offB[ks] + (q - 1) * 32 * LK);
        else fa[q - TJ] = *reinterpret_cast<const v4i*>(st + offA[ks] + (q - TJ) * 32 * LK);
    };
    auto mfma_one = [&](int m, const v4i (&fa)[TI], const v4i (&fb)[TJ]) {
        const int i = m / TJ, j = m % TJ;
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };
    v4i fa[2][TI], fb[2][TJ];
    wait_dma_lds<(STAGES - 2) * kPPW>();
    float* ftab = reinterpret_cast<float*>(smem + Sh::kSmem);       // [0, 256) s_ch, [256, 512) float bias, [512, 768) s_tok
    if (tid < kLN) {
        ftab[tid] = fac0;
        ftab[256 + tid] = fac1;
    } else if (tid - kLN < kLM) {
        ftab[512 + tid - kLN] = fac0;
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    dma_stage(STAGES - 1, STAGES - 1 < last ? STAGES - 1 : last);
#pragma unroll
    for (int q = 0; q < kNR; ++q) read_one(0, 0, q, fa[0], fb[0]);
    int stage = 0;
    for (int step = 0; step < nsteps; ++step) {
        const int next = stage + 1 == STAGES ? 0 : stage + 1;
        const int refill = step + STAGES < last ? step + STAGES : last;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < kKS - 1; ++ks) {
#pragma unroll
            for (int m = 0; m < kNM; ++m) {
                mfma_one(m, fa[ks & 1], fb[ks & 1]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q = kRPM * m; q < kRPM * (m + 1); ++q) {
                    if (q < kNR) {
                        read_one(stage, ks + 1, q, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
        wait_dma_lds<(STAGES - 2) * kPPW>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        dma_stage(stage, refill);                                   // loading waves only
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < kNM; ++m) {
            mfma_one(m, fa[(kKS - 1) & 1], fb[(kKS - 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = kRPM * m; q < kRPM * (m + 1); ++q) {
                if (q < kNR) {
                    read_one(next, 0, q, fa[0], fb[0]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        stage = next;
    }
    // all loads landed and every wave is done with the stages before LDS is reused
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // epilogue: fp32(acc, integer bias included) * s_ch * s_tok + fbias, narrowed, transposed through a per-wave LDS
    // patch of 32 rows x 32*TJ columns, stored as 16-byte pieces of full rows.  Branch-free per element:
    // absent factors are replaced by their neutral elements (x * 1.0f and x + (-0.0f) return x bit for bit),
    // the factors come from the block's LDS table, every LDS address is base + immediate.
    constexpr int ES = (ODT == AMCT_F32) ? 4 : 2;                   // bytes per output element
    constexpr int kPW = 32 * TJ;                                   // patch width in columns
    constexpr int kPatchRow = kPW * ES + 16;                       // padded patch row
    constexpr int CPR = kPW * ES / 16;                             // 16-byte chunks per patch row
    static_assert(32 * kPatchRow <= 16384 && (32 * CPR) % 64 == 0 && TI <= 4,
                  "the patch must fit the wave's 16 KiB and split into wave-wide reads");
    int8_t* patch = smem + wave * 16384;
    const float* tokl = ftab + 512 + wm * 32 * TI;                  // the row factors of this wave
    float sc[TJ], fb2[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        sc[j] = ftab[wn * kPW + j * 32 + (lane & 31)];
        fb2[j] = ftab[256 + wn * kPW + j * 32 + (lane & 31)];
    }
    int32_t* const raw = gridDim.z > 1 ? a.part + (int64_t)blockIdx.z * a.M * a.N : a.acc_out;
    if (raw) {                                                      // a slice's partial sums, or the accumulators on request (tests): plain stores
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r)
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const int64_t m = m0 + wm * 32 * TI + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                    const int64_t n = n0 + wn * kPW + j * 32 + (lane & 31);
                    if (m < a.M && n < a.N) raw[m * a.N + n] = acc[i][j][r];
                }
        if (gridDim.z > 1) return;
    }
    const int h4 = 4 * (lane >> 5);
    int8_t* wbase = patch + h4 * kPatchRow + (lane & 31) * ES;      // this lane's element of patch row h4
    const int8_t* rbase = patch + (lane / CPR) * kPatchRow + (lane % CPR) * 16;
    constexpr int RPI = 64 / CPR;                                   // patch rows per wave-wide read when CPR divides 64
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        const int64_t mbase = m0 + wm * 32 * TI + i * 32;
        float tks[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {                               // rows 8q + h4 .. + 3 are registers 4q .. 4q + 3
            const float4 t4 = *reinterpret_cast<const float4*>(tokl + i * 32 + 8 * q + h4);
            tks[4 * q] = t4.x; tks[4 * q + 1] = t4.y; tks[4 * q + 2] = t4.z; tks[4 * q + 3] = t4.w;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int prow0 = 8 * (r >> 2) + (r & 3);               // patch row minus h4
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                float f = (float)acc[i][j][r] * sc[j];
                f = f * tks[r];
                f = f + fb2[j];
                int8_t* dst = wbase + prow0 * kPatchRow + j * 32 * ES;
                if constexpr (ODT == AMCT_F32) *reinterpret_cast<float*>(dst) = f;
                else if constexpr (ODT == AMCT_BF16) *reinterpret_cast<uint16_t*>(dst) = (uint16_t)f32_to_bf16_bits(f);
                else *reinterpret_cast<uint16_t*>(dst) = (uint16_t)f32_to_f16_bits(f);
            }
        }
        // LDS operations of one wave complete in order: the reads below see the writes above
#pragma unroll
        for (int it = 0; it < 32 * CPR / 64; ++it) {
            int prow, chunk;
            uint4 v;
            if constexpr (64 % CPR == 0) {
                prow = it * RPI + lane / CPR;
                chunk = lane % CPR;
                v = *reinterpret_cast<const uint4*>(rbase + it * RPI * kPatchRow);
            } else {
                const int idx = it * 64 + lane;                    // 16-byte chunk of the patch, row-major
                prow = idx / CPR;
                chunk = idx % CPR;
                v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            }
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * kPW + chunk * (16 / ES);
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * ES, v);
        }
    }
}

constexpr int kFacOff = 128 * 1024;                                 // the epilogue's factor table behind the LDS stages
constexpr int kFacBytes = 3 * 256 * 4;

// MODE 0: int8 operands (v_mfma_i32_16x16x64_i8).  MODE 1 / 2: bf16 / fp16 operands with fp32 accumulation
// (v_mfma_f32_16x16x32_bf16 / _f16): the same 64 bytes of K per row and MFMA and the same fragment layout in bytes, so
// the body is that of the int8 kernel with a.K counted in BYTES of a row; s_ch and s_tok are null then (factor 1).
template <int ODT, int WM, int WN, int TI, int TJ, int STAGES, int MODE = 0>
AMCT_DEV void w8a8_dma_body16(const W8A8Args& a, int8_t* smem, const int64_t m0, const int64_t n0) {
    constexpr int LK = 128;
    using Sh = DmaTile<WM, WN, TI, TJ, STAGES, LK>;
    constexpr int kLM = Sh::kLM, kLN = Sh::kLN, kRP = Sh::kRP, kNA = Sh::kNA, kNB = Sh::kNB, kPPW = Sh::kPPW;
    constexpr int kLStageBytes = Sh::kLStageBytes, kWaves = Sh::kWaves, kLW = Sh::kLW;
    constexpr int kCH = LK / 16;                                    // 16-byte chunks per row
    constexpr int kKS = LK / 32;                                    // MFMA k-slices per stage
    static_assert(LK == 64 || LK == 128, "row length");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    // Split K (gridDim.z > 1): block z takes the steps [steps z / S, steps (z + 1) / S) of every row and leaves its sums
    // (int32, or fp32 in the 16-bit modes) in a.part[z]; a second kernel adds them and applies the epilogue.
    const uint32_t steps_all = (uint32_t)(a.K / LK);
    const uint32_t step0 = steps_all * blockIdx.z / gridDim.z;
    const int nsteps = (int)(steps_all * (blockIdx.z + 1) / gridDim.z - step0);
    const int last = nsteps - 1;
    const int8_t* const xk = a.xq + (int64_t)step0 * LK;
    const int8_t* const wk = a.wq + (int64_t)step0 * LK;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t*)smem;
    // Rows are LK bytes, unpadded (a direct-to-LDS load writes the 64 lanes' 16-byte pieces to 1024 contiguous
    // bytes); 16-byte chunk c of row r lives at chunk position c ^ swz(r), which spreads the 16 rows that one
    // phase of a 16-byte fragment read touches over all banks.
    auto swz = [](int r) { return LK == 64 ? (r >> 2) & 3 : (r >> 1) & 7; };

    // this wave's 1 KiB pieces of a stage: kNA pieces of A rows, then kNB pieces of B rows.  A load is addressed
    // as (operand base + LK * step) in SGPRs plus a constant 32-bit byte offset per lane and piece (the host
    // admits only operands below 4 GiB to this kernel).
    const bool loader = wave >= kWaves - kLW;                       // the last kLW waves: one per SIMD when kLW = 4
    const int lw = loader ? wave - (kWaves - kLW) : 0;
    uint32_t goff[kPPW];
    {
        const int rin = lane / kCH;                                 // row inside the piece
        const int pc = lane % kCH;                                  // physical chunk this lane fills
#pragma unroll
        for (int j = 0; j < kPPW; ++j) {
            int64_t r;
            int lr;                                                 // row inside the operand's LDS tile
            if (j < kNA) {
                lr = (lw * kNA + j) * kRP + rin;
                r = m0 + lr < a.M ? m0 + lr : a.M - 1;
            } else {
                // a wave beyond the last piece fetches the last piece again: same bytes to the same place
                const int pb = lw * kNB + (j - kNA) < kLN / kRP ? lw * kNB + (j - kNA) : kLN / kRP - 1;
                lr = pb * kRP + rin;
                r = n0 + lr < a.N ? n0 + lr : a.N - 1;
            }
            goff[j] = (uint32_t)(r * a.K + (pc ^ swz(lr)) * 16);
        }
    }
    auto dma_one = [&](int stg, int step, int j) {
        if (j < kNA) {
            dma16s(lds0 + stg * kLStageBytes + (lw * kNA + j) * 1024, xk + (int64_t)step * LK, goff[j]);
        } else {
            const int pb = lw * kNB + (j - kNA) < kLN / kRP ? lw * kNB + (j - kNA) : kLN / kRP - 1;
            dma16s(lds0 + stg * kLStageBytes + kLM * LK + pb * 1024, wk + (int64_t)step * LK, goff[j]);
        }
    };
    auto dma_stage = [&](int stage, int step) {
        if (loader) {
#pragma unroll
            for (int j = 0; j < kPPW; ++j) dma_one(stage, step, j);
        }
    };

    // A stage holds two k-slices of 64 bytes; each is done in two units (the upper and the lower half of the wave's
    // 16-row tiles), so a stage is four units u = 2 * slice + half, as many as the 32x32x32 form has k-slices.
    // Fragment of unit u: lane reads row (tile base + lane % 16), logical chunk 4 * slice + lane / 16.
    constexpr int TA = TI;                                          // 16-row tiles per unit
    constexpr int TB = 2 * TJ;                                      // 16-column tiles of the wave
    int offA[4], offB[2];
    {
        const int r = lane & 15;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            offA[u] = (wm * 32 * TI + (u & 1) * 16 * TA + r) * LK + ((4 * (u >> 1) + (lane >> 4)) ^ swz(r)) * 16;
#pragma unroll
        for (int sl = 0; sl < 2; ++sl)
            offB[sl] = kLM * LK + (wn * 32 * TJ + r) * LK + ((4 * sl + (lane >> 4)) ^ swz(r)) * 16;
    }

    typedef float v4fa __attribute__((ext_vector_type(4)));
    typedef typename std::conditional<MODE == 0, v4i, v4fa>::type acc_t;
    acc_t acc[2 * TI][TB];
#pragma unroll
    for (int i = 0; i < 2 * TI; ++i)
#pragma unroll
        for (int j = 0; j < TB; ++j) {
            if constexpr (MODE == 0) acc[i][j] = v4i{0, 0, 0, 0};
            else acc[i][j] = v4fa{0.f, 0.f, 0.f, 0.f};
        }

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) dma_stage(s, s < last ? s : last);

    // The factors of the epilogue (per column: s_ch and the float bias; per row: s_tok; absent ones replaced by their
    // neutral elements) are fetched now, one or two per thread, and parked in an LDS table behind the stages: read at the
    // end of the tile they would cost a round trip to memory with nothing to hide it.
    float fac0 = 1.0f, fac1 = -0.0f;
    if (tid < kLN) {
        const int64_t n = n0 + tid < a.N ? n0 + tid : a.N - 1;
        if (a.s_ch) fac0 = a.s_ch[n];
        if (a.bias_kind == 2) fac1 = reinterpret_cast<const float*>(a.bias)[n];
    } else if (tid - kLN < kLM) {
        const int64_t m = m0 + (tid - kLN) < a.M ? m0 + (tid - kLN) : a.M - 1;
        if (a.s_tok) fac0 = a.s_tok[m];
    }
    // The weight fragment is the MFMA's first operand, so a lane's four accumulator registers of tile (t, j) are four
    // ADJACENT COLUMNS 16 j + 4 (lane / 16) + r of row 16 t + lane % 16 of the wave tile: the epilogue converts them in pairs
    // and moves them with one LDS write.  An integer bias is where the accumulators start (its loads wait together with
    // the first stage's), so the epilogue never sees it.
    if constexpr (MODE == 0) {
        if (a.bias_kind == 1 && gridDim.z == 1) {
#pragma unroll
            for (int j = 0; j < TB; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t n = n0 + wn * 32 * TJ + j * 16 + 4 * (lane >> 4) + r;
                    const int32_t b = reinterpret_cast<const int32_t*>(a.bias)[n < a.N ? n : a.N - 1];
#pragma unroll
                    for (int i = 0; i < 2 * TI; ++i) acc[i][j][r] = b;
                }
        }
    }

    // The schedule of w8a8_dma_body with units in the place of its k-slices: while the MFMAs of a unit run, the fragments
    // of the next one are read (TA row fragments, plus the TB column fragments when the next unit starts a slice); before
    // the last unit of a stage the waves meet, the refill loads follow, and the last unit reads the first fragments of the
    // next stage.  Row fragments alternate between two buffers per unit, column fragments per slice.
    constexpr int kNM = TA * TB;                                    // MFMAs per unit
    constexpr int kNRmax = TA + TB;
    constexpr int kGap = kNM / kNRmax;                              // one fragment read behind every kGap-th MFMA
    static_assert(kGap >= 1, "fewer MFMAs than fragment reads per unit");
    v4i fa[2][TA], fb[2][TB];
    auto read_one = [&](int stg, int u, int q) {                    // u, q: compile-time in every use
        const int8_t* st = smem + stg * kLStageBytes;
        if (q < TA) fa[u & 1][q] = *reinterpret_cast<const v4i*>(st + offA[u] + q * 16 * LK);
        else if ((u & 1) == 0 && q < TA + TB) fb[(u >> 1) & 1][q - TA] = *reinterpret_cast<const v4i*>(st + offB[u >> 1] + (q - TA) * 16 * LK);
    };
    auto mfma_one = [&](int u, int m) {
        const int i = m / TB, j = m % TB;
        if constexpr (MODE == 0) {
            acc[(u & 1) * TA + i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[(u >> 1) & 1][j], fa[u & 1][i], acc[(u & 1) * TA + i][j], 0, 0, 0);
        } else if constexpr (MODE == 1) {
            typedef __bf16 v8bfm __attribute__((ext_vector_type(8)));
            acc[(u & 1) * TA + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bfm, fb[(u >> 1) & 1][j]), __builtin_bit_cast(v8bfm, fa[u & 1][i]),
                                                                           acc[(u & 1) * TA + i][j], 0, 0, 0);
        } else {
            typedef _Float16 v8hm __attribute__((ext_vector_type(8)));
            acc[(u & 1) * TA + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8hm, fb[(u >> 1) & 1][j]), __builtin_bit_cast(v8hm, fa[u & 1][i]),
                                                                          acc[(u & 1) * TA + i][j], 0, 0, 0);
        }
    };
    wait_dma_lds<(STAGES - 2) * kPPW>();
    {
        float* ftab = reinterpret_cast<float*>(smem + kFacOff);     // [0, 256) s_ch, [256, 512) float bias, [512, 768) s_tok
        if (tid < kLN) {
            ftab[tid] = fac0;
            ftab[256 + tid] = fac1;
        } else if (tid - kLN < kLM) {
            ftab[512 + tid - kLN] = fac0;
        }
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    dma_stage(STAGES - 1, STAGES - 1 < last ? STAGES - 1 : last);
#pragma unroll
    for (int q = 0; q < kNRmax; ++q) read_one(0, 0, q);
    int stage = 0;
    for (int step = 0; step < nsteps; ++step) {
        const int next = stage + 1 == STAGES ? 0 : stage + 1;
        const int refill = step + STAGES < last ? step + STAGES : last;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 3; ++u) {
#pragma unroll
            for (int m = 0; m < kNM; ++m) {
                mfma_one(u, m);
                __builtin_amdgcn_sched_barrier(0);
                if (m % kGap == 0 && m / kGap < kNRmax) {
                    read_one(stage, u + 1, m / kGap);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        wait_dma_lds<(STAGES - 2) * kPPW>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        dma_stage(stage, refill);                                   // loading waves only
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < kNM; ++m) {
            mfma_one(3, m);
            __builtin_amdgcn_sched_barrier(0);
            if (m % kGap == 0 && m / kGap < kNRmax) {
                read_one(next, 0, m / kGap);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        stage = next;
    }
    // all loads landed and every wave is done with the stages before LDS is reused
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    if (gridDim.z > 1) {
        // the raw sums of this slice: a lane's four adjacent columns of row 16 t + lane % 16 as one 16-byte store
        int32_t* const part = a.part + (int64_t)blockIdx.z * a.M * a.N;
#pragma unroll
        for (int t = 0; t < 2 * TI; ++t)
#pragma unroll
            for (int j = 0; j < TB; ++j) {
                const int64_t m = m0 + wm * 32 * TI + t * 16 + (lane & 15);
                const int64_t n = n0 + wn * 32 * TJ + j * 16 + 4 * (lane >> 4);
                if (m < a.M && n < a.N) *reinterpret_cast<acc_t*>(part + m * a.N + n) = acc[t][j];
            }
        return;
    }
    // epilogue: fp32(acc, integer bias included) * s_ch * s_tok + fbias, narrowed, through a per-wave LDS patch of 32 rows x
    // 32*TJ columns, stored as 16-byte pieces of full rows.  Branch-free per element: absent factors are replaced by
    // their neutral elements (x * 1.0f and x + (-0.0f) return x bit for bit).  A lane holds the factors of its 4 TB
    // columns and of its 2 TI rows in registers.
    constexpr int ES = (ODT == AMCT_F32) ? 4 : 2;                   // bytes per output element
    constexpr int kPW = 32 * TJ;                                   // patch width in columns
    constexpr int kPatchRow = kPW * ES + 16;                       // padded patch row
    constexpr int CPR = kPW * ES / 16;                             // 16-byte chunks per patch row
    static_assert(32 * kPatchRow <= 16384 && (32 * CPR) % 64 == 0 && TI <= 4,
                  "the patch must fit the wave's 16 KiB and split into wave-wide reads");
    int8_t* patch = smem + wave * 16384;
    const int q4 = 4 * (lane >> 4);
    float sc[TB][4], fb2[TB][4], tks[2 * TI];
    {
        const float* ftab = reinterpret_cast<const float*>(smem + kFacOff);
#pragma unroll
        for (int j = 0; j < TB; ++j) {
            const float4 s4 = *reinterpret_cast<const float4*>(ftab + wn * kPW + j * 16 + q4);
            const float4 b4 = *reinterpret_cast<const float4*>(ftab + 256 + wn * kPW + j * 16 + q4);
            sc[j][0] = s4.x, sc[j][1] = s4.y, sc[j][2] = s4.z, sc[j][3] = s4.w;
            fb2[j][0] = b4.x, fb2[j][1] = b4.y, fb2[j][2] = b4.z, fb2[j][3] = b4.w;
        }
#pragma unroll
        for (int t = 0; t < 2 * TI; ++t) tks[t] = ftab[512 + wm * 32 * TI + t * 16 + (lane & 15)];
    }
    if constexpr (MODE == 0) if (a.acc_out) {                       // accumulators on request (tests): plain stores
#pragma unroll
        for (int t = 0; t < 2 * TI; ++t)
#pragma unroll
            for (int j = 0; j < TB; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t m = m0 + wm * 32 * TI + t * 16 + (lane & 15);
                    const int64_t n = n0 + wn * kPW + j * 16 + q4 + r;
                    if (m < a.M && n < a.N) a.acc_out[m * a.N + n] = acc[t][j][r];
                }
    }
    int8_t* wbase = patch + (lane & 15) * kPatchRow + q4 * ES;      // this lane's first element of patch row lane % 16
    const int8_t* rbase = patch + (lane / CPR) * kPatchRow + (lane % CPR) * 16;
    constexpr int RPI = 64 / CPR;                                   // patch rows per wave-wide read when CPR divides 64
#pragma unroll
    for (int i = 0; i < TI; ++i) {                                  // 32 rows of the wave tile per pass: tiles 2 i and 2 i + 1
        const int64_t mbase = m0 + wm * 32 * TI + i * 32;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int t = 2 * i + hh;
#pragma unroll
            for (int j = 0; j < TB; ++j) {
                float f[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    f[r] = (float)acc[t][j][r] * sc[j][r];
                    f[r] = f[r] * tks[t];
                    f[r] = f[r] + fb2[j][r];
                }
                int8_t* dst = wbase + 16 * hh * kPatchRow + j * 16 * ES;
                if constexpr (ODT == AMCT_F32) {
                    *reinterpret_cast<float4*>(dst) = make_float4(f[0], f[1], f[2], f[3]);
                } else {
                    // one packed conversion per pair; the empty asm keeps it a conversion of the rounded fp32 sum
#pragma unroll
                    for (int r = 0; r < 4; ++r) asm("" : "+v"(f[r]));
                    typedef float v2fe __attribute__((ext_vector_type(2)));
                    uint2 w;
                    if constexpr (ODT == AMCT_BF16) {
                        typedef __bf16 v2be __attribute__((ext_vector_type(2)));
                        w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((v2fe{f[0], f[1]}), v2be));
                        w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((v2fe{f[2], f[3]}), v2be));
                    } else {
                        typedef _Float16 v2he __attribute__((ext_vector_type(2)));
                        w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((v2fe{f[0], f[1]}), v2he));
                        w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((v2fe{f[2], f[3]}), v2he));
                    }
                    *reinterpret_cast<uint2*>(dst) = w;
                }
            }
        }
        // LDS operations of one wave complete in order: the reads below see the writes above
#pragma unroll
        for (int it = 0; it < 32 * CPR / 64; ++it) {
            int prow, chunk;
            uint4 v;
            if constexpr (64 % CPR == 0) {
                prow = it * RPI + lane / CPR;
                chunk = lane % CPR;
                v = *reinterpret_cast<const uint4*>(rbase + it * RPI * kPatchRow);
            } else {
                const int idx = it * 64 + lane;                    // 16-byte chunk of the patch, row-major
                prow = idx / CPR;
                chunk = idx % CPR;
                v = *reinterpret_cast<const uint4*>(patch + prow * kPatchRow + chunk * 16);
            }
            const int64_t m = mbase + prow;
            const int64_t n = n0 + wn * kPW + chunk * (16 / ES);
            if (m < a.M && n < a.N) stg16_nt(reinterpret_cast<char*>(a.out) + (m * a.N + n) * ES, v);
        }
    }
}

template <int ODT, int WM, int WN, int STAGES, int LK>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void w8a8_tile_dma(W8A8Args a) {
    using Sh = DmaTile<WM, WN, 4, 2, STAGES, LK>;
    __shared__ __attribute__((aligned(1024))) int8_t smem[Sh::kSmemFac];
    w8a8_dma_body<ODT, WM, WN, 4, 2, STAGES, LK>(a, smem, (int64_t)blockIdx.y * Sh::kLM, (int64_t)blockIdx.x * Sh::kLN);
}

template <int ODT, int STAGES, int LK>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void w8a8_tile_mix(W8A8Args a, MixPlan p) {
    using Big = DmaTile<2, 4, 4, 2, STAGES, LK>;
    using Small = DmaTile<4, 2, 2, 3, STAGES, LK>;
    static_assert(Big::kSmem == Small::kSmem, "one place for the factor table");
    __shared__ __attribute__((aligned(1024))) int8_t smem[Big::kSmemFac];
    const int b = blockIdx.x;
    if (b < p.big) {
        w8a8_dma_body<ODT, 2, 4, 4, 2, STAGES, LK>(a, smem, (int64_t)(b / p.nbig) * 256, (int64_t)(b % p.nbig) * 256);
    } else {
        const int s = b - p.big;
        w8a8_dma_body<ODT, 4, 2, 2, 3, STAGES, LK>(a, smem, (int64_t)(s / p.nsmall) * 256,
                                                   (int64_t)p.nbig * 256 + (int64_t)(s % p.nsmall) * 192);
    }
}

// the same two launches on v_mfma_i32_16x16x64_i8 (K a multiple of 128)
template <int ODT, int MODE = 0>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void w8a8_tile_dma16(W8A8Args a) {
    using Sh = DmaTile<2, 4, 4, 2, 2, 128>;
    static_assert(Sh::kSmem <= kFacOff, "the factor table lies behind the stages");
    __shared__ __attribute__((aligned(1024))) int8_t smem[kFacOff + kFacBytes];
    w8a8_dma_body16<ODT, 2, 4, 4, 2, 2, MODE>(a, smem, (int64_t)blockIdx.y * Sh::kLM, (int64_t)blockIdx.x * Sh::kLN);
}

template <int ODT, int MODE = 0>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void w8a8_tile_mix16(W8A8Args a, MixPlan p) {
    using Big = DmaTile<2, 4, 4, 2, 2, 128>;
    using Small = DmaTile<4, 2, 2, 3, 2, 128>;
    static_assert(Big::kSmem <= kFacOff && Small::kSmem <= kFacOff, "the factor table lies behind the stages");
    __shared__ __attribute__((aligned(1024))) int8_t smem[kFacOff + kFacBytes];
    const int b = blockIdx.x;
    if (b < p.big) {
        w8a8_dma_body16<ODT, 2, 4, 4, 2, 2, MODE>(a, smem, (int64_t)(b / p.nbig) * 256, (int64_t)(b % p.nbig) * 256);
    } else {
        const int s = b - p.big;
        w8a8_dma_body16<ODT, 4, 2, 2, 3, 2, MODE>(a, smem, (int64_t)(s / p.nsmall) * 256,
                                            (int64_t)p.nbig * 256 + (int64_t)(s % p.nsmall) * 192);
    }
}

// any block shape the body supports, uniform over the launch (blockIdx.x: column tile, blockIdx.y: row tile)
template <int ODT, int WM, int WN, int TI, int TJ, int STAGES, int LK>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(WM * WN / 4, WM * WN / 4))) void w8a8_tile_shape(W8A8Args a) {
    using Sh = DmaTile<WM, WN, TI, TJ, STAGES, LK>;
    __shared__ __attribute__((aligned(1024))) int8_t smem[Sh::kSmemFac];
    w8a8_dma_body<ODT, WM, WN, TI, TJ, STAGES, LK>(a, smem, (int64_t)blockIdx.y * Sh::kLM, (int64_t)blockIdx.x * Sh::kLN);
}

// ---------------------------------------------------------------------------
// skinny kernel: M <= 16 * MT.  One block = 16 output columns; its 4 waves split K.
// Lane l of a wave streams row n0 + l%16 of the weight, 16 bytes per MFMA, k-slot l/16.
// ---------------------------------------------------------------------------
template <int MT>
__global__ __launch_bounds__(kBlock) void w8a8_skinny(W8A8Args a) {
    __shared__ int32_t red[3][MT][64][4];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int64_t nrow = (n0 + (lane & 15) < a.N) ? n0 + (lane & 15) : a.N - 1;
    const int8_t* wrow = a.wq + nrow * a.K;
    const int kslot = (lane >> 4) * 16;
    // K is split into 4 contiguous spans, one per wave, each a multiple of 64 bytes
    const int64_t steps_total = (a.K + 63) / 64;
    const int64_t steps_per_wave = (steps_total + 3) / 4;
    const int64_t s_begin = wave * steps_per_wave;
    const int64_t s_end = (s_begin + steps_per_wave < steps_total) ? s_begin + steps_per_wave : steps_total;

    v4i acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = v4i{0, 0, 0, 0};
    const int8_t* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int64_t m = t * 16 + (lane & 15);
        xrow[t] = a.xq + (m < a.M ? m : a.M - 1) * a.K;
    }
    constexpr int UN = 4;
    for (int64_t s = s_begin; s < s_end; s += UN) {
        // every load is unconditional (a predicated load forces a full wait): out-of-range positions read
        // the last 16 bytes of the row instead and the weight fragment is zeroed afterwards
        uint4 wv[UN], xv[UN][MT];
        bool ok[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int64_t k = (s + u) * 64 + kslot;
            ok[u] = (s + u < s_end) && k < a.K;
            const int64_t kc = ok[u] ? k : a.K - 16;
            wv[u] = ldg16(wrow + kc);
#pragma unroll
            for (int t = 0; t < MT; ++t) xv[u][t] = ldg16(xrow[t] + kc);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const uint4 w4 = ok[u] ? wv[u] : make_uint4(0, 0, 0, 0);
            const v4i fb = v4i{(int)w4.x, (int)w4.y, (int)w4.z, (int)w4.w};
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const v4i fa = v4i{(int)xv[u][t].x, (int)xv[u][t].y, (int)xv[u][t].z, (int)xv[u][t].w};
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, fb, acc[t], 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave - 1][t][lane][r] = acc[t][r];
    }
    __syncthreads();
    if (wave == 0) {
        // register r of a 16x16 tile holds row 4*(lane/16) + r, column lane%16
        const int64_t n = n0 + (lane & 15);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int32_t v = acc[t][r] + red[0][t][lane][r] + red[1][t][lane][r] + red[2][t][lane][r];
                const int64_t m = t * 16 + 4 * (lane >> 4) + r;
                if (n < a.N && m < a.M) w8a8_epilogue(a, m, n, v);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// decode kernel (M <= 16, K % 256 == 0): the weight matrix is streamed once, nothing else is expensive.
// A block owns 16 * TN output columns, its waves split K in runs of 256.  The block's activations are
// staged in LDS once (rows padded by 16 bytes: the 16 rows of a fragment read fall into different
// banks).  The staging loads are issued before the weight loads: waits follow issue order, so the staged
// data is consumed, and the block barrier passed, while the weights are still arriving.  A lane's weight
// loads cover the 64-byte quarters of a row's 256-byte run back to back; two iterations are in flight.
// All loads are unconditional (indices clamped).
// ---------------------------------------------------------------------------
template <int WAVES, int XJ, int TN>
__global__ __launch_bounds__(WAVES * 64) void w8a8_decode_lds(W8A8Args a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    constexpr int NT = WAVES * 64;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * (16 * TN);
    const uint32_t K = (uint32_t)a.K, M = (uint32_t)a.M;
    const uint32_t xstride = K + 16;
    const int per_wave = (int)(K / 256) / WAVES;
    const int it0 = wave * per_wave;

    const uint32_t KV = K / 16, n_xv = M * KV;
    uint4 xv[XJ];
    uint32_t xdst[XJ];
#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        const uint32_t vc = v < n_xv ? v : n_xv - 1;
        const uint32_t row = vc / KV, kv = vc - row * KV;
        xv[j] = ldg16(a.xq + (int64_t)row * K + kv * 16);
        xdst[j] = row * xstride + kv * 16;
    }
    __builtin_amdgcn_sched_barrier(0);

    const int8_t* wrow[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const int64_t n = n0 + t * 16 + r16;
        wrow[t] = a.wq + (n < a.N ? n : a.N - 1) * (int64_t)K + g * 16;
    }
    uint4 wv[2][TN * 4];
    auto load_w = [&](int buf, int it) {
        const int itc = it < it0 + per_wave ? it : it0 + per_wave - 1;
        const uint32_t kb = (uint32_t)itc * 256u;
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) wv[buf][t * 4 + q] = ldg16(wrow[t] + kb + q * 64);
    };
    load_w(0, it0);
    load_w(1, it0 + 1);
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int j = 0; j < XJ; ++j) {
        const uint32_t v = tid + NT * j;
        if (v < n_xv) *reinterpret_cast<uint4*>(lds_raw + xdst[j]) = xv[j];
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    v4i acc[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) acc[t] = v4i{0, 0, 0, 0};
    const uint8_t* xlane = lds_raw + (r16 < (int)M ? r16 : (int)M - 1) * xstride + g * 16;

    auto compute = [&](int buf, int it) {
        const uint32_t kb = (uint32_t)it * 256u;
        v4i fa[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) fa[q] = *reinterpret_cast<const v4i*>(xlane + kb + q * 64);
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint4 w4 = wv[buf][t * 4 + q];
                const v4i fb = v4i{(int)w4.x, (int)w4.y, (int)w4.z, (int)w4.w};
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[q], fb, acc[t], 0, 0, 0);
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

    int32_t* red = reinterpret_cast<int32_t*>(lds_raw);           // reuses the activation rows
    if constexpr (WAVES > 1) {
        __syncthreads();                                          // every wave is done reading activations
        if (wave > 0) {
#pragma unroll
            for (int t = 0; t < TN; ++t)
                *reinterpret_cast<v4i*>(red + (((wave - 1) * TN + t) * 64 + lane) * 4) = acc[t];
        }
        __syncthreads();
    }
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            const int64_t n = n0 + t * 16 + r16;
            v4i v = acc[t];
            if constexpr (WAVES > 1) {
#pragma unroll
                for (int w = 0; w < WAVES - 1; ++w) {
                    const v4i o = *reinterpret_cast<const v4i*>(red + ((w * TN + t) * 64 + lane) * 4);
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] += o[r];
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t m = 4 * g + r;                      // register r of a 16x16 tile: row 4*(lane/16) + r
                if (n < a.N && m < a.M) w8a8_epilogue(a, m, n, v[r]);
            }
        }
    }
}

// LDS bytes of w8a8_decode_lds, 0 if the shape does not fit
static size_t w8a8_decode_lds_bytes(int64_t M, int64_t K, int waves, int tn) {
    const size_t xbytes = (size_t)M * ((size_t)K + 16);
    const size_t red = (size_t)(waves - 1) * tn * 64 * 16;
    const size_t total = xbytes > red ? xbytes : red;
    return total <= 150 * 1024 ? total : 0;
}

template <int WAVES, int XJ, int TN>
static int launch_w8a8_decode(const W8A8Args& a, size_t lds, hipStream_t st) {
    // only launches above the default 64 KiB of dynamic LDS need the attribute; it is per device and cheap,
    // so it is simply set on every such launch and no state is kept in the library
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(&w8a8_decode_lds<WAVES, XJ, TN>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return AMCT_E_HIP;
    }
    const dim3 grid((unsigned)((a.N + 16 * TN - 1) / (16 * TN)));
    hipLaunchKernelGGL((w8a8_decode_lds<WAVES, XJ, TN>), grid, dim3(WAVES * 64), lds, st, a);
    return hip_status();
}

template <int WAVES, int TN>
static int launch_w8a8_decode_xj(const W8A8Args& a, size_t lds, hipStream_t st) {
    const int64_t per_thread = (a.M * (a.K / 16) + WAVES * 64 - 1) / (WAVES * 64);
    if (per_thread <= 1) return launch_w8a8_decode<WAVES, 1, TN>(a, lds, st);
    if (per_thread <= 4) return launch_w8a8_decode<WAVES, 4, TN>(a, lds, st);
    if (per_thread <= 16) return launch_w8a8_decode<WAVES, 16, TN>(a, lds, st);
    return AMCT_E_UNSUPPORTED;
}

template <int TN>
static int launch_w8a8_decode_w(const W8A8Args& a, int waves, size_t lds, hipStream_t st) {
    return waves == 4   ? launch_w8a8_decode_xj<4, TN>(a, lds, st)
           : waves == 2 ? launch_w8a8_decode_xj<2, TN>(a, lds, st)
                        : launch_w8a8_decode_xj<1, TN>(a, lds, st);
}

// general kernel: any M, N, K; one output per thread.
__global__ __launch_bounds__(kBlock) void w8a8_general(W8A8Args a) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= a.M * a.N) return;
    const int64_t m = idx / a.N, n = idx - m * a.N;
    const int8_t* xr = a.xq + m * a.K;
    const int8_t* wr = a.wq + n * a.K;
    int32_t acc = 0;
    for (int64_t k = 0; k < a.K; ++k) acc += (int32_t)xr[k] * (int32_t)wr[k];
    w8a8_epilogue(a, m, n, acc);
}

// out = dt(fp32(part[0] + ... + part[S - 1] + ibias) * s_ch * s_tok + fbias): the tile kernels' epilogue, operation for
// operation, on the exact sum of the K slices; four columns per thread (N % 8 == 0)
template <int ODT>
__global__ __launch_bounds__(kBlock) void w8a8_splitk_reduce(W8A8Args a, int S) {
    const int64_t nvec = a.M * a.N / 4, stride = (int64_t)gridDim.x * kBlock;
    for (int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride) {
        const int64_t e = v * 4, m = e / a.N, n = e - m * a.N;
        int4 sum = *reinterpret_cast<const int4*>(a.part + e);
        for (int z = 1; z < S; ++z) {
            const int4 p = *reinterpret_cast<const int4*>(a.part + (int64_t)z * a.M * a.N + e);
            sum.x += p.x, sum.y += p.y, sum.z += p.z, sum.w += p.w;
        }
        int32_t acc[4] = {sum.x, sum.y, sum.z, sum.w};
        const float tk = a.s_tok ? a.s_tok[m] : 1.0f;
        float f[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (a.bias_kind == 1) acc[c] += reinterpret_cast<const int32_t*>(a.bias)[n + c];
            f[c] = (float)acc[c] * (a.s_ch ? a.s_ch[n + c] : 1.0f);
            f[c] = f[c] * tk;
            f[c] = f[c] + (a.bias_kind == 2 ? reinterpret_cast<const float*>(a.bias)[n + c] : -0.0f);
        }
        if (a.acc_out) {
#pragma unroll
            for (int c = 0; c < 4; ++c) a.acc_out[e + c] = acc[c];
        }
        if constexpr (ODT == AMCT_F32) {
            *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.out) + e) = make_float4(f[0], f[1], f[2], f[3]);
        } else {
            uint32_t h[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) h[c] = ODT == AMCT_BF16 ? f32_to_bf16_bits(f[c]) : f32_to_f16_bits(f[c]);
            *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.out) + e) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
        }
    }
}

// the same for the 16-bit GEMM: out = dt(part[0] + ... + part[S - 1] + bias), fp32 partial sums added in that order
template <int ODT>
__global__ __launch_bounds__(kBlock) void gemm16_splitk_reduce(W8A8Args a, int S) {
    const int64_t nvec = a.M * a.N / 4, stride = (int64_t)gridDim.x * kBlock;
    const float* part = reinterpret_cast<const float*>(a.part);
    for (int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride) {
        const int64_t e = v * 4, n = e % a.N;
        float4 sum = *reinterpret_cast<const float4*>(part + e);
        for (int z = 1; z < S; ++z) {
            const float4 p = *reinterpret_cast<const float4*>(part + (int64_t)z * a.M * a.N + e);
            sum.x += p.x, sum.y += p.y, sum.z += p.z, sum.w += p.w;
        }
        float f[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) f[c] = f[c] + (a.bias_kind == 2 ? reinterpret_cast<const float*>(a.bias)[n + c] : -0.0f);
        uint32_t h[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) h[c] = ODT == AMCT_BF16 ? f32_to_bf16_bits(f[c]) : f32_to_f16_bits(f[c]);
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(a.out) + e) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    }
}

// K slices of a launch of `blocks` tile blocks: as many as fill the CUs, at most 8, a slice of at least 2048 bytes of K
static int w8a8_splits(int64_t blocks, int64_t K, int64_t cus) {
    if (blocks <= 0 || cus <= 0) return 1;
    int64_t S = cus / blocks;
    if (S > 8) S = 8;
    while (S > 1 && K / S < 2048) --S;
    return S < 1 ? 1 : (int)S;
}

int w8a8_stream_dispatch(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch, const void* bias,
                         int bias_kind, void* out, int32_t* acc_out, int64_t M, int64_t N, int64_t K, int out_dtype,
                         hipStream_t st);

// out [M, N] of dtype = x [M, K] @ w [N, K]^T + bias (fp32 [N] or null), fp32 accumulation, both operands of dtype (bf16 or
// fp16), K contiguous: the 256x256 / 256x192 tiles of the W8A8 kernel on the 16-bit MFMAs.  Returns AMCT_E_UNSUPPORTED
// for shapes the tiles do not take (fewer than 256 rows, K not a multiple of 64, N not a multiple of 8, unaligned or
// 4 GiB operands).  Used by the int8 weight-only Linear, which dequantises its weight into a workspace first.
// K slices of the uniform 256x256 launch of the 16-bit GEMM (1: not split), and the bytes of their fp32 partial sums
static int gemm16_splits(int64_t M, int64_t N, int64_t Kb, int cus) {
    return w8a8_splits(((M + 255) / 256) * ((N + 255) / 256), Kb, cus);
}
size_t gemm16_part_bytes(int64_t M, int64_t N, int64_t K) {
    const int S = M >= 256 ? gemm16_splits(M, N, K * 2, current_cu_count()) : 1;
    return S > 1 ? (size_t)S * (size_t)M * (size_t)N * 4 : 0;
}

int gemm16_tiles(const void* x, const void* w, const float* bias, void* out, int64_t M, int64_t N, int64_t K, int dtype,
                 void* workspace, size_t workspace_bytes, hipStream_t st) {
    const int64_t Kb = K * 2;                                       // bytes of a row
    if (dtype != AMCT_BF16 && dtype != AMCT_F16) return AMCT_E_UNSUPPORTED;
    if (M < 256 || Kb % 128 != 0 || N % 8 != 0 || !aligned16(x) || !aligned16(w) || !aligned16(out) ||
        M * Kb >= (int64_t(1) << 32) || N * Kb >= (int64_t(1) << 32))
        return AMCT_E_UNSUPPORTED;
    const dim3 grid((unsigned)((N + 255) / 256), (unsigned)((M + 255) / 256));
    if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
    W8A8Args a{reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), nullptr, nullptr, bias, out, nullptr,
               M, N, Kb, bias ? 2 : 0, dtype};
    const int cus = current_cu_count();
    // few tiles (half the CUs or fewer: few output columns): K split over S blocks per uniform tile, fp32 partial sums in
    // the lent workspace; otherwise the plan that mixes in narrower tiles where that fills the CUs better
    unsigned S = (unsigned)gemm16_splits(M, N, Kb, cus);
    if (S > 1 && !(workspace && aligned16(workspace) && workspace_bytes >= (size_t)S * (size_t)M * (size_t)N * 4)) S = 1;
    const MixPlan plan = plan_mix(M, N, cus);
    if (S == 1 && plan.nbig >= 0) {
        const dim3 g1((unsigned)(plan.big + plan.mtiles * plan.nsmall));
        if (dtype == AMCT_BF16) hipLaunchKernelGGL((w8a8_tile_mix16<AMCT_BF16, 1>), g1, dim3(512), 0, st, a, plan);
        else hipLaunchKernelGGL((w8a8_tile_mix16<AMCT_F16, 2>), g1, dim3(512), 0, st, a, plan);
    } else {
        if (S > 1) a.part = reinterpret_cast<int32_t*>(workspace);
        const dim3 g(grid.x, grid.y, S);
        if (dtype == AMCT_BF16) hipLaunchKernelGGL((w8a8_tile_dma16<AMCT_BF16, 1>), g, dim3(512), 0, st, a);
        else hipLaunchKernelGGL((w8a8_tile_dma16<AMCT_F16, 2>), g, dim3(512), 0, st, a);
        if (S > 1) {
            int64_t nb = (M * N / 4 + kBlock - 1) / kBlock;
            if (nb > 8192) nb = 8192;
            if (dtype == AMCT_BF16) hipLaunchKernelGGL((gemm16_splitk_reduce<AMCT_BF16>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, (int)S);
            else hipLaunchKernelGGL((gemm16_splitk_reduce<AMCT_F16>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, (int)S);
        }
    }
    return hip_status();
}

}  // namespace amct

using namespace amct;

// block shape of the small and medium tile launches (1: 64x64, 2: 128x64, 3: 128x128, 4: 128x256; 0: none of them) and
// the number of blocks it takes
static int w8a8_mid_shape(int64_t M, int64_t N, int64_t cus, int64_t* blocks) {
    const int64_t mt = (M + 127) / 128, nt64 = (N + 63) / 64, nt128 = (N + 127) / 128, nt256 = (N + 255) / 256;
    int shape = 0;
    if (cus > 0 && M <= 64 && nt64 <= cus) shape = 1, *blocks = nt64;
    else if (cus > 0 && mt * nt64 <= cus) shape = 2, *blocks = mt * nt64;
    else if (cus > 0 && mt * nt128 <= cus) shape = 3, *blocks = mt * nt128;
    else if (cus > 0 && (mt * nt256 <= cus || M < 256)) shape = 4, *blocks = mt * nt256;
    return shape;
}

extern "C" size_t amct_gemm_w8a8_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 2 || N <= 0 || K <= 0 || K % 128 != 0 || N % 8 != 0) return 0;
    if (M <= 16 && (K == 1024 || K == 2048 || K == 4096)) return 0;      // the weight-streaming kernel
    int64_t blocks = 0;
    const int64_t cus = current_cu_count();
    if (!w8a8_mid_shape(M, N, cus, &blocks)) {                      // the large tiles, when their launch is uniform
        if (M < 256 || plan_mix(M, N, (int)cus).nbig >= 0) return 0;
        blocks = ((M + 255) / 256) * ((N + 255) / 256);
    }
    const int S = w8a8_splits(blocks, K, cus);
    return S > 1 ? (size_t)S * (size_t)M * (size_t)N * 4 : 0;
}

namespace amct {
int w8a8_stream_quant_dispatch(const void* x, int x_dtype, const void* smooth, const void* act_scale, const void* act_zp,
                               int per_token, const int8_t* wq, const float* s_tok, const float* s_ch, const void* bias,
                               int bias_kind, void* out, int64_t M, int64_t N, int64_t K, int out_dtype, hipStream_t st);   // gemm_w8a8_stream.hip
}

// the int8 activations of the two-kernel form (rounded up to 16 bytes), then what the GEMM asks for
extern "C" size_t amct_linear_w8a8_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return (((size_t)M * (size_t)K + 15) & ~(size_t)15) + amct_gemm_w8a8_workspace_bytes(M, N, K);
}

extern "C" int amct_linear_w8a8(const void* x, int x_dtype, const void* smooth, const void* act_scale, const void* act_offset,
                                int64_t n_scales, int per_token, const int8_t* wq, const float* s_tok, const float* s_ch,
                                const void* bias, int bias_kind, void* out, int64_t M, int64_t N, int64_t K, int out_dtype,
                                void* workspace, size_t workspace_bytes, amct_stream_t stream) {
    if (M < 0 || N <= 0 || K <= 0 || bias_kind < 0 || bias_kind > 2) return AMCT_E_BADARG;
    if (x_dtype != AMCT_F32 && x_dtype != AMCT_F16 && x_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (out_dtype != AMCT_F32 && out_dtype != AMCT_F16 && out_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (per_token ? (n_scales != M) : (n_scales != 1 && n_scales != K)) return AMCT_E_BADARG;
    if (M == 0) return AMCT_OK;
    if (!x || !act_scale || !wq || !s_ch || !out || (bias_kind != 0 && !bias)) return AMCT_E_BADARG;
    if (per_token || n_scales == 1) {
        const int rc = w8a8_stream_quant_dispatch(x, x_dtype, smooth, act_scale, act_offset, per_token, wq, s_tok, s_ch, bias,
                                                  bias_kind, out, M, N, K, out_dtype, (hipStream_t)stream);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    const size_t xq_bytes = ((size_t)M * (size_t)K + 15) & ~(size_t)15;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0 || workspace_bytes < xq_bytes) return AMCT_E_BADARG;
    int8_t* xq = reinterpret_cast<int8_t*>(workspace);
    const int rc = amct_quantize(x, smooth, act_scale, act_offset, xq, M, K, n_scales, per_token, x_dtype, stream);
    if (rc != AMCT_OK) return rc;
    return amct_gemm_w8a8_ws(xq, wq, s_tok, s_ch, bias, bias_kind, out, nullptr, M, N, K, out_dtype,
                             reinterpret_cast<char*>(workspace) + xq_bytes, workspace_bytes - xq_bytes, stream);
}

extern "C" int amct_gemm_w8a8(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch,
                              const void* bias, int bias_kind, void* out, int32_t* acc_out, int64_t M, int64_t N,
                              int64_t K, int out_dtype, amct_stream_t stream) {
    return amct_gemm_w8a8_ws(xq, wq, s_tok, s_ch, bias, bias_kind, out, acc_out, M, N, K, out_dtype, nullptr, 0, stream);
}

extern "C" int amct_gemm_w8a8_ws(const int8_t* xq, const int8_t* wq, const float* s_tok, const float* s_ch,
                                 const void* bias, int bias_kind, void* out, int32_t* acc_out, int64_t M, int64_t N,
                                 int64_t K, int out_dtype, void* workspace, size_t workspace_bytes, amct_stream_t stream) {
    if (M < 0 || N <= 0 || K <= 0 || bias_kind < 0 || bias_kind > 2) return AMCT_E_BADARG;
    if (M != 0 && (!xq || !wq || !s_ch || !out || (bias_kind != 0 && !bias))) return AMCT_E_BADARG;   // M == 0 reads nothing
    if (out_dtype != AMCT_F32 && out_dtype != AMCT_F16 && out_dtype != AMCT_BF16) return AMCT_E_BADARG;
    if (M == 0) return AMCT_OK;
    W8A8Args a{xq, wq, s_tok, s_ch, bias_kind ? bias : nullptr, out, acc_out, M, N, K, bias_kind, out_dtype};
    hipStream_t st = (hipStream_t)stream;
    const bool vec_ok = (K % 16 == 0) && aligned16(xq) && aligned16(wq);
    // the tile kernels (direct-to-LDS loads, MFMA 32x32x32): K a multiple of 128, 16-byte pieces of whole output rows,
    // operands below 4 GiB (32-bit lane offsets)
    const bool tile_ok = vec_ok && K % 128 == 0 && N % 8 == 0 && aligned16(out) && M * K < (int64_t(1) << 32) &&
                         N * K < (int64_t(1) << 32);
    if (M <= 16) {                                              // weight-streaming kernel (K of 1024, 2048 or 4096)
        const int rc = w8a8_stream_dispatch(xq, wq, s_tok, s_ch, bias, bias_kind, out, acc_out, M, N, K, out_dtype, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    if (vec_ok && M <= 16 && K % 256 == 0 && (M <= 2 || !tile_ok)) {
        const int iters = (int)(K / 256);
        // measured: blocks of 2 or 4 waves, several per CU, stream best (one block's start-up and reduction
        // overlap with another's loads); wider blocks only pay when the activations are large
        const int64_t mk = M * K;
        int waves = mk <= 8192 ? 2 : 4;
        while (iters % waves != 0) waves >>= 1;
        const int tn = (mk <= 8192 || mk > 32768) ? 2 : 1;
        const size_t lds = w8a8_decode_lds_bytes(M, K, waves, tn);
        int rc = AMCT_E_UNSUPPORTED;
        if (lds) rc = tn == 1 ? launch_w8a8_decode_w<1>(a, waves, lds, st) : launch_w8a8_decode_w<2>(a, waves, lds, st);
        if (rc != AMCT_E_UNSUPPORTED) return rc;
    }
    // Small and medium M: as long as all tiles of a launch run at once, small tiles on many CUs beat large tiles on
    // few, and a short step exposes the load latency that two LDS stages cover for a 256x256 tile.  The smallest block
    // shape whose blocks fit the CUs in one round is taken (measured on W[14336,4096], us per call):
    //   64x64,   4 waves of 32x32, 4 stages : M = 3 .. 64   15.2 .. 16.1  (weight-streaming decode kernel: 16.4 .. 19.5 at
    //                                                        M = 3 .. 16; it stays for M <= 2: 14.4 against 15.1)
    //   128x64,  4 waves of 64x32, 4 stages : M = 65 .. 128 17.5 .. 19.3
    //   128x128, 4 waves of 64x64, 3 stages : M <= 256      25     (first-generation 128x128 kernel: 39 .. 42)
    //   128x256, 8 waves of 64x64, 3 stages : M <= 512      32     (256x256 tiles: 43)
    if (tile_ok) {
        const int64_t cus = current_cu_count();
        const int64_t mt = (M + 127) / 128, nt64 = (N + 63) / 64, nt128 = (N + 127) / 128, nt256 = (N + 255) / 256;
        int64_t blocks = 0;
        const int shape = w8a8_mid_shape(M, N, cus, &blocks);
        if (shape && mt <= 65535) {
            // Few blocks and long rows (the down projection of an MLP): K is split over S blocks per tile, which leave
            // int32 partial sums in the lent workspace; a second kernel adds them - exactly - and applies the epilogue,
            // so the result is that of the unsplit launch bit for bit.
            unsigned S = (unsigned)w8a8_splits(blocks, K, cus);
            if (S > 1 && !(workspace && aligned16(workspace) && workspace_bytes >= (size_t)S * (size_t)M * (size_t)N * 4)) S = 1;
            if (S > 1) a.part = reinterpret_cast<int32_t*>(workspace);
#define AMCT_LAUNCH_MID(ODT)                                                                                          \
    {                                                                                                                 \
        if (shape == 1) hipLaunchKernelGGL((w8a8_tile_shape<ODT, 2, 2, 1, 1, 4, 128>), dim3((unsigned)nt64, 1, S), dim3(256), 0, st, a);             \
        else if (shape == 2) hipLaunchKernelGGL((w8a8_tile_shape<ODT, 2, 2, 2, 1, 4, 128>), dim3((unsigned)nt64, (unsigned)mt, S), dim3(256), 0, st, a);  \
        else if (shape == 3) hipLaunchKernelGGL((w8a8_tile_shape<ODT, 2, 2, 2, 2, 3, 128>), dim3((unsigned)nt128, (unsigned)mt, S), dim3(256), 0, st, a); \
        else hipLaunchKernelGGL((w8a8_tile_shape<ODT, 2, 4, 2, 2, 3, 128>), dim3((unsigned)nt256, (unsigned)mt, S), dim3(512), 0, st, a);            \
        if (S > 1) {                                                                                                  \
            int64_t nb = (M * N / 4 + kBlock - 1) / kBlock;                                                           \
            if (nb > 8192) nb = 8192;                                                                                 \
            hipLaunchKernelGGL((w8a8_splitk_reduce<ODT>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, (int)S);        \
        }                                                                                                             \
    }
            if (out_dtype == AMCT_BF16) AMCT_LAUNCH_MID(AMCT_BF16)
            else if (out_dtype == AMCT_F16) AMCT_LAUNCH_MID(AMCT_F16)
            else AMCT_LAUNCH_MID(AMCT_F32)
#undef AMCT_LAUNCH_MID
            return hip_status();
        }
    }
    // measured on W[14336,4096]: the skinny kernel re-reads the activations once per 16 output columns and
    // loses to the 128x128 tile kernel from M = 48 on (33.9 us against 30.5 us; M = 64: 41.7 against 32.9)
    if (vec_ok && M <= 32) {
        const dim3 grid((unsigned)((N + 15) / 16));
        if (M <= 16) hipLaunchKernelGGL((w8a8_skinny<1>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((w8a8_skinny<2>), grid, dim3(kBlock), 0, st, a);
        return hip_status();
    }
    if (vec_ok && M >= 256 && K % kLK == 0 && K >= kLK && N % 8 == 0 && aligned16(out) && M * K < (int64_t(1) << 32) &&
        N * K < (int64_t(1) << 32)) {
        // 256x256 tiles, 8 waves, 4 stages (measured faster than 256x128 with two blocks per CU:
        // the traffic from L2 into LDS matters more than decoupling the barriers)
        const dim3 grid((unsigned)((N + 255) / 256), (unsigned)((M + 255) / 256));
        if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
        const int cus = current_cu_count();
        const MixPlan plan = plan_mix(M, N, cus);
        // 128-byte LDS rows and 2 stages when K allows (whole cache lines per load, one barrier per 128 bytes of K:
        // 7 % faster), else 64-byte rows and 4 stages
        const bool wide = K % 128 == 0;
        // Under the part's power limit v_mfma_i32_16x16x64_i8 sustains more than v_mfma_i32_32x32x32_i8 on non-constant
        // operands (register-only loops: 3.74 against 3.24 POP/s; with the large tile's fragment reads interleaved 3.8
        // against 3.4), at equal LDS traffic per wave tile: 98 against 105 us on M = 2048, N = 14336, K = 4096.
        constexpr bool mi16 = true;
        // few tiles (few output columns): K split over S blocks per tile, int32 partial sums in the lent workspace
        unsigned S = 1;
        if (wide && mi16 && plan.nbig < 0) {
            S = (unsigned)w8a8_splits((int64_t)grid.x * grid.y, K, cus);
            if (S > 1 && !(workspace && aligned16(workspace) && workspace_bytes >= (size_t)S * (size_t)M * (size_t)N * 4)) S = 1;
            if (S > 1) a.part = reinterpret_cast<int32_t*>(workspace);
        }
#define AMCT_LAUNCH_DMA(ODT)                                                                                        \
    {                                                                                                               \
        if (plan.nbig >= 0) {                                                                                       \
            const dim3 g1((unsigned)(plan.big + plan.mtiles * plan.nsmall));                                        \
            if (wide && mi16) hipLaunchKernelGGL((w8a8_tile_mix16<ODT>), g1, dim3(512), 0, st, a, plan);            \
            else if (wide) hipLaunchKernelGGL((w8a8_tile_mix<ODT, 2, 128>), g1, dim3(512), 0, st, a, plan);         \
            else hipLaunchKernelGGL((w8a8_tile_mix<ODT, 4, 64>), g1, dim3(512), 0, st, a, plan);                    \
        } else {                                                                                                    \
            if (wide && mi16) hipLaunchKernelGGL((w8a8_tile_dma16<ODT>), dim3(grid.x, grid.y, S), dim3(512), 0, st, a); \
            else if (wide) hipLaunchKernelGGL((w8a8_tile_dma<ODT, 2, 4, 2, 128>), grid, dim3(512), 0, st, a);       \
            else hipLaunchKernelGGL((w8a8_tile_dma<ODT, 2, 4, 4, 64>), grid, dim3(512), 0, st, a);                  \
            if (S > 1) {                                                                                            \
                int64_t nb = (M * N / 4 + kBlock - 1) / kBlock;                                                     \
                if (nb > 8192) nb = 8192;                                                                           \
                hipLaunchKernelGGL((w8a8_splitk_reduce<ODT>), dim3((unsigned)nb), dim3(kBlock), 0, st, a, (int)S);  \
            }                                                                                                       \
        }                                                                                                           \
    }
        if (out_dtype == AMCT_BF16) AMCT_LAUNCH_DMA(AMCT_BF16)
        else if (out_dtype == AMCT_F16) AMCT_LAUNCH_DMA(AMCT_F16)
        else AMCT_LAUNCH_DMA(AMCT_F32)
#undef AMCT_LAUNCH_DMA
        return hip_status();
    }
    if (vec_ok) {
        const dim3 grid((unsigned)((N + kBN - 1) / kBN), (unsigned)((M + kBM - 1) / kBM));
        if (grid.y > 65535) return AMCT_E_UNSUPPORTED;
        if (out_dtype == AMCT_BF16) hipLaunchKernelGGL((w8a8_tile<AMCT_BF16>), grid, dim3(kBlock), 0, st, a);
        else if (out_dtype == AMCT_F16) hipLaunchKernelGGL((w8a8_tile<AMCT_F16>), grid, dim3(kBlock), 0, st, a);
        else hipLaunchKernelGGL((w8a8_tile<AMCT_F32>), grid, dim3(kBlock), 0, st, a);
        return hip_status();
    }
    const int64_t nb = (M * N + kBlock - 1) / kBlock;
    if (nb > 0x7FFFFFFF) return AMCT_E_UNSUPPORTED;
    hipLaunchKernelGGL(w8a8_general, dim3((unsigned)nb), dim3(kBlock), 0, st, a);
    return hip_status();
}
