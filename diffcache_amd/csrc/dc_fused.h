// State, workspace layout and helpers of the streaming select kernels (fused.hip).
#pragma once
#include "dc_common.h"
#include "dc_select.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlockStep = 256;
constexpr int kBigSteps = 8;       // 2048 rows per large block
constexpr int kSmallChunks = 16;   // leading 256-row blocks per unit
constexpr int kStage = kBigSteps * kRowsPerBlockStep;
constexpr int kCandLds = 16384;    // candidates the finish kernel keeps in LDS (128 KB of the CU's 160)
constexpr int kSharedPollUnits = 8;   // sketch scan: up to this many units, one wave per block polls
constexpr int kPqThreads = 512;    // PQ scan: threads per block = keys per step
constexpr int kPqBigSteps = 8;     // PQ scan: 4096 keys per large block
constexpr int kBinsPerThread = DC_HIST_BINS / kThreads;  // bins a thread owns when a block scans a histogram
static_assert(kBinsPerThread % 4 == 0 && kBinsPerThread * kThreads == DC_HIST_BINS, "bin split");

// tb_run is polled by every wave of the scan while surv_cnt takes returning
// atomics; they sit in separate 128-byte lines because polling a line that is
// being updated atomically serialises both at the memory side.
struct UnitState {
    uint32_t tb_run;    // running threshold bucket (only decreases)
    uint32_t sync_cnt;  // one-kernel route (small.hip): arrivals of the unit's blocks at its barriers; zero between launches
    uint32_t pad0[30];
    uint32_t surv_cnt;  // survivors appended so far
    uint32_t win_cnt;   // certain members written to idx_out (select phase)
    uint32_t cand_cnt;  // candidates of the threshold bucket (select phase)
    uint32_t c_less;    // keys in buckets better than the threshold bucket
    uint32_t margin;    // sketch scan only: float bits of the score margin of the unit
    // the one-kernel route for short contexts (small.hip)
    uint32_t sync_err;  // a bounded wait ran out (never expected)
    uint32_t cut_key;   // the cutoff (key, id) when a unit's candidates are too many to rank in LDS
    uint32_t cut_id;
    uint32_t pad1[24];
};
static_assert(sizeof(UnitState) == 256, "UnitState is two 128-byte lines");
static_assert(kRadixBins * 4 >= kFinalThreads * 8, "lh doubles as the packed candidate list");

__device__ __forceinline__ uint32_t load_relaxed(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Exact threshold bucket of a unit from its complete histogram: the bucket that
// holds the k-th best key, and how many keys sit in better buckets.  Called by
// all kThreads threads; the result is uniform.  `wtot`, `sres`: LDS scratch.
__device__ __forceinline__ void unit_threshold(const uint32_t *__restrict__ hu, uint32_t kk,
                                               uint32_t *wtot, uint32_t *sres, uint32_t &tb,
                                               uint32_t &c_less) {
    const int tid = threadIdx.x;
    if (tid == 0) {
        sres[0] = DC_HIST_BINS;
        sres[1] = 0;
    }
    uint32_t bins[kBinsPerThread];
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kBinsPerThread / 4; ++i) {
        const uint4 t = reinterpret_cast<const uint4 *>(hu)[tid * (kBinsPerThread / 4) + i];
        bins[4 * i + 0] = t.x;
        bins[4 * i + 1] = t.y;
        bins[4 * i + 2] = t.z;
        bins[4 * i + 3] = t.w;
        sum += t.x + t.y + t.z + t.w;
    }
    uint32_t total;
    const uint32_t excl = block_excl_scan<kThreads>(sum, wtot, &total);
    if (excl < kk && kk <= excl + sum) {
        uint32_t run = excl;
        bool done = false;
#pragma unroll
        for (int i = 0; i < kBinsPerThread; ++i) {
            if (!done && run + bins[i] >= kk) {
                sres[0] = tid * kBinsPerThread + i;
                sres[1] = run;
                done = true;
            }
            run += bins[i];
        }
    }
    __syncthreads();
    tb = sres[0];
    c_less = sres[1];
}

struct FusedWs {
    uint32_t *hist;
    UnitState *state;
    uint2 *surv;
    uint32_t *cand_key, *cand_idx, *sel_keys;
    unsigned long long *sort_scratch;
    size_t bytes;
};

int fused_pow2(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

FusedWs carve_fused(void *base, int n_units, int n_rows, int k) {
    FusedWs w;
    char *p = (char *)base;
    size_t off = 0;
    const size_t nu = n_units > 0 ? n_units : 0, nr = n_rows > 0 ? n_rows : 0;
    const int keff = k < n_rows ? k : n_rows;
    w.hist = (uint32_t *)(p + off);
    off += dc_align_up(nu * DC_HIST_BINS * 4, 256);
    w.state = (UnitState *)(p + off);
    off += dc_align_up(nu * sizeof(UnitState), 256);
    w.surv = (uint2 *)(p + off);
    off += dc_align_up(nu * nr * 8, 256);
    w.cand_key = (uint32_t *)(p + off);
    off += dc_align_up(nu * nr * 4, 256);
    w.cand_idx = (uint32_t *)(p + off);
    off += dc_align_up(nu * nr * 4, 256);
    w.sel_keys = (uint32_t *)(p + off);
    off += dc_align_up(nu * (size_t)(keff > 0 ? keff : 0) * 4, 256);
    w.sort_scratch = (unsigned long long *)(p + off);
    if (keff > 4096) off += dc_align_up(nu * (size_t)fused_pow2(keff) * 8, 256);
    w.bytes = off;
    return w;
}

}  // namespace
