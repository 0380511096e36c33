// Block-shape plan of the large-tile GEMM launches (host side) and its kernel argument.
#pragma once
#include <cstdint>
#include <map>

namespace amct {

// One launch, two block shapes: the first `big` blocks compute 256x256 tiles of the first `nbig` column tiles,
// the rest 256x192 tiles of the columns after them.  The host picks the split so that the blocks fill the
// CUs evenly (a 256x192 tile costs 3/4 of a 256x256 one): with uniform tiles the last round of a launch
// leaves CUs idle, e.g. 448 tiles on 256 CUs take two rounds for 1.75 rounds of work.
struct MixPlan {
    int mtiles;                                                     // row tiles (256 rows each)
    int nbig;                                                       // 256-column tiles, columns [0, 256*nbig)
    int big;                                                        // mtiles * nbig
    int nsmall;                                                     // 192-column tiles after them
};

// Finish time, in quarters of a 256x256 tile, of `big` blocks of cost 4 followed by `small` blocks of cost 3
// handed in that order to `cus` CUs holding one block each (the hardware gives the next block to the first
// CU that becomes free).  CUs that become free at the same time are handled together, so the cost is a few
// map operations per round of blocks, not per block.
inline int64_t mix_makespan(int64_t big, int64_t small, int cus) {
    std::map<int64_t, int64_t> free_at;                            // time -> number of CUs free from then on
    const int64_t q = big / cus, rem = big % cus;
    free_at[4 * q] = cus - rem;
    if (rem) free_at[4 * (q + 1)] = rem;
    int64_t end = big ? (rem ? 4 * (q + 1) : 4 * q) : 0;
    while (small > 0) {
        const auto it = free_at.begin();
        const int64_t t = it->first, n = it->second < small ? it->second : small;
        if (n == it->second) free_at.erase(it);
        else it->second -= n;
        free_at[t + 3] += n;
        if (t + 3 > end) end = t + 3;
        small -= n;
    }
    return end;
}

// Split of the N columns into 256-wide and 192-wide column tiles that finishes first; nbig = -1 when plain
// 256x256 tiles are as good (or the launch is so large that its last round does not matter).
inline MixPlan plan_mix_search(int64_t M, int64_t N, int cus) {
    MixPlan best{(int)((M + 255) / 256), -1, 0, 0};
    const int64_t mt = best.mtiles;
    const int64_t uniform_tiles = mt * ((N + 255) / 256);
    if (cus <= 0 || uniform_tiles > 16 * (int64_t)cus) return best;
    int64_t best_t = mix_makespan(uniform_tiles, 0, cus);
    for (int64_t nb = (N + 255) / 256 - 1; nb >= 0; --nb) {         // nb big column tiles, the rest 192 wide
        const int64_t ns = (N - 256 * nb + 191) / 192;
        const int64_t t = mix_makespan(mt * nb, mt * ns, cus);
        if (t < best_t) {
            best_t = t;
            best.nbig = (int)nb;
            best.big = (int)(mt * nb);
            best.nsmall = (int)ns;
        }
    }
    return best;
}

inline MixPlan plan_mix(int64_t M, int64_t N, int cus) {
    // the last answer is kept per host thread: a layer is called with the same shape again and again
    struct Last { int64_t M, N; int cus; MixPlan plan; };
    static thread_local Last last_plan{-1, -1, -1, {}};
    if (last_plan.M == M && last_plan.N == N && last_plan.cus == cus) return last_plan.plan;
    const MixPlan fresh = plan_mix_search(M, N, cus);
    last_plan = Last{M, N, cus, fresh};
    return fresh;
}

// number of CUs of the current device, 0 if it cannot be read (the plan then keeps uniform tiles)
inline int current_cu_count() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return cus;
}

}  // namespace amct
