// Streaming score + exact top-k in two kernels, without a dense score array.
// Same result as dc_score_bf16 followed by dc_topk_select (the set a size-k heap
// scan keeps, diffcache_cpu/src/nsw.rs:600-621), built for the case where the
// scores themselves are not wanted.
//
// Why: on MI355X every byte the scan writes costs several read bytes' worth of
// HBM time, so the 4 bytes/row of a dense score array are the main overhead of
// a kernel that otherwise streams 256 bytes/row at the read ceiling.
//
// score_prune_kernel streams the key rows like score_kernel, bins every key in
// the unit's bucket histogram, and keeps a row only if its bucket is not
// worse than the unit's running threshold bucket tb_run.  tb_run is the bucket
// of the k-th best key among the rows histogrammed so far; rows can only be
// added, so tb_run never undershoots the final threshold bucket and no member
// of the final top-k is ever dropped, however stale the value a block reads.
// Survivors are staged in LDS and appended to the unit's list as (id, score)
// with one atomic per block.  Blocks are ordered chunk-major so that all units
// advance together, and the first chunks of every unit are small so that a
// threshold exists early.
//
// classify_kernel (several blocks per unit) derives the exact threshold bucket
// from the complete histogram and splits the survivors into certain members and
// candidates; select_finish_kernel (one block per unit) finishes with the same
// radix select as finalize_kernel.
//
// The sketch route reads half the bytes for the same result: sketch_prune_kernel
// is the same scan over an 8-bit sketch of the keys (one byte per element, see
// sketch.hip) with a margin that makes its pruning safe, rescore_kernel computes
// the exact scores of the rows that survive it and lists them as candidates, and
// select_finish_kernel picks the k best of that list.
#include <type_traits>
#include "dc_common.h"
#include "dc_select.h"
#include "dc_fused.h"
#include "dc_pq.h"

namespace {

__global__ void init_state_kernel(uint32_t *hist, UnitState *state, int n_units) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t n_hist = (int64_t)n_units * DC_HIST_BINS;
    if (i < n_hist) hist[i] = 0;
    if (i < n_units) {
        state[i].tb_run = DC_HIST_BINS;  // nothing is pruned until a threshold exists
        state[i].surv_cnt = 0;
        state[i].win_cnt = 0;
        state[i].cand_cnt = 0;
        state[i].c_less = 0;
        state[i].margin = 0;
        state[i].sync_cnt = 0;
        state[i].sync_err = 0;
        state[i].cut_key = 0;
        state[i].cut_id = 0;
    }
}

// A block's copy of its unit's running threshold bucket, in LDS.  The poll of the unit's
// value crosses the chip (agent scope) and every younger load of the polling wave returns
// after it, so one wave of the block polls and the others read the copy.
__device__ __forceinline__ uint32_t lds_load_relaxed(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void lds_store_relaxed(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// End of a scan block: append the block's survivors (staged per wave in LDS) to
// the unit's list with one returning atomic, flush the block's histogram, and in
// the blocks chosen by the caller refresh the unit's running threshold from
// whatever part of the histogram is visible.  Staleness only loosens the bound.
template <int kT = kThreads, typename E = uint2>
__device__ __forceinline__ void prune_block_finish(uint32_t *lhist, const E *wstage, uint32_t wcnt,
                                                   uint32_t *s_wcnt, uint32_t *s_base, uint32_t *wtot,
                                                   UnitState *st, uint32_t *hu, E *surv_unit,
                                                   bool refresh, uint32_t kk) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    if (lane == 0) s_wcnt[wave] = wcnt;
    __syncthreads();

    // the atomic is in flight while the histogram is flushed
    uint32_t wbase = 0, cnt = 0;
#pragma unroll
    for (int w2 = 0; w2 < kT / 64; ++w2) {
        if (w2 < wave) wbase += s_wcnt[w2];
        cnt += s_wcnt[w2];
    }
    if (tid == 0) *s_base = cnt ? atomicAdd(&st->surv_cnt, cnt) : 0;
    for (int i = tid; i < DC_HIST_BINS; i += kT) {
        const uint32_t c = lhist[i];
        if (c) atomicAdd(&hu[i], c);
    }
    __syncthreads();
    {
        E *dst = surv_unit + *s_base + wbase;
        for (uint32_t i = lane; i < wcnt; i += 64) dst[i] = wstage[i];
    }
    if (!refresh) return;

    // Coalesced, L2-bypassing read of the unit's histogram into LDS (lhist is
    // free again), then kBinsPerThread adjacent bins per thread.
    {
        const unsigned long long *h64 = reinterpret_cast<const unsigned long long *>(hu);
        unsigned long long *l64 = reinterpret_cast<unsigned long long *>(lhist);
        for (int i = tid; i < DC_HIST_BINS / 2; i += kT)
            l64[i] = __hip_atomic_load(h64 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    constexpr int kBins = DC_HIST_BINS / kT;  // adjacent bins a thread owns
    static_assert(kBins * kT == DC_HIST_BINS, "bin split");
    uint32_t bins[kBins];
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < kBins; ++i) {
        bins[i] = lhist[tid * kBins + i];
        sum += bins[i];
    }
    uint32_t total;
    const uint32_t excl = block_excl_scan<kT>(sum, wtot, &total);
    if (excl < kk && kk <= excl + sum) {
        uint32_t run = excl;
        bool done = false;
#pragma unroll
        for (int i = 0; i < kBins; ++i) {
            if (!done && run + bins[i] >= kk) {
                atomicMin(&st->tb_run, (uint32_t)(tid * kBins + i));
                done = true;
            }
            run += bins[i];
        }
    }
}

template <int HD>
__global__ __launch_bounds__(kThreads) void score_prune_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ Q, uint32_t *__restrict__ hist,
    UnitState *__restrict__ state, uint2 *__restrict__ surv, int n_units, int n_h, int n_cap,
    int64_t sb, int64_t sh, int64_t sr, int q_group, int mode, int k_eff, int small_chunks,
    int big_steps, const int32_t *__restrict__ hi_dev, int lo_row) {
    constexpr int LPR = HD / 8;
    constexpr int CH = LPR < 16 ? LPR : 16;
    __shared__ uint32_t lhist[DC_HIST_BINS];
    __shared__ uint2 stage[kStage];
    __shared__ uint32_t wtot[kThreads / 64 + 1];
    __shared__ uint32_t s_wcnt[kThreads / 64];
    __shared__ uint32_t s_base;
    const int n_rows = dc_live_rows(n_cap, hi_dev, lo_row);

    const int unit = blockIdx.x % n_units;
    const int chunk = blockIdx.x / n_units;
    const int b = unit / n_h, h = unit % n_h;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int grp = lane / LPR, col = lane % LPR;

    const bool small = chunk < small_chunks;
    // Units sit a power of two apart in memory; rotating each unit's order of large
    // chunks keeps blocks that run together from walking the same address offsets.
    const int big_chunks = (int)(gridDim.x / n_units) - small_chunks;
    const int big_id = small ? 0 : (int)(((int64_t)(chunk - small_chunks) + (int64_t)unit * 7) % big_chunks);
    const int64_t block_row0 =
        small ? (int64_t)chunk * kRowsPerBlockStep
              : (int64_t)small_chunks * kRowsPerBlockStep + (int64_t)big_id * big_steps * kRowsPerBlockStep;
    const int steps = small ? 1 : big_steps;

    if (block_row0 >= n_rows) return;  // the grid is laid out for n_cap rows
    for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;

    const uint16_t *Ku = K + b * sb + h * sh + col * 8;
    UnitState *st = state + unit;
    const int last = n_rows - 1;
    uint32_t tb = load_relaxed(&st->tb_run);

    float q[8];
    dc_load_query<HD>(Q, unit, q_group, col, q);
    __syncthreads();

    // Each wave stages its survivors in its own slice of `stage` (at most 64 per
    // step), so the cursor is a wave-uniform register and no LDS atomic is needed.
    uint2 *wstage = stage + wave * (kBigSteps * 64);
    uint32_t wcnt = 0;
    const unsigned long long lt = (1ull << lane) - 1ull;

    for (int step = 0; step < steps; ++step) {
        const int64_t row0 = block_row0 + (int64_t)step * kRowsPerBlockStep + wave * 64;
        if (row0 >= n_rows) break;  // wave-uniform; no barrier inside the loop
        float mine = 0.f;
        uint32_t tb_next = tb;
#pragma unroll
        for (int c0 = 0; c0 < LPR; c0 += CH) {
            uint4 w[CH];
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                int64_t r = row0 + grp * LPR + c0 + j;
                r = r > last ? last : r;
                w[j] = dc_load_stream16(Ku + r * sr);
            }
            // the threshold for the next step queues up behind this step's rows
            if (c0 + CH >= LPR && step + 1 < steps) tb_next = load_relaxed(&st->tb_run);
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float p = dc_group_sum<LPR>(dc_dot8(w[j], q, 0.f));
                mine = (col == c0 + j) ? p : mine;
            }
        }
        const int64_t myrow = row0 + lane;
        const bool valid = myrow < n_rows;
        uint32_t key = 0, bucket = 0xffffffffu;
        if (valid) dc_key_bucket(mine, mode, key, bucket);
        // Only rows that can still matter are kept and counted: the final threshold
        // bucket is never worse than tb, so it is fixed by the counts of buckets <= tb.
        const bool keep = valid && bucket <= tb;
        if (keep) atomicAdd(&lhist[bucket], 1u);
        const unsigned long long mask = __ballot(keep);
        if (keep) wstage[wcnt + __popcll(mask & lt)] = make_uint2((uint32_t)myrow, __float_as_uint(mine));
        wcnt += (uint32_t)__popcll(mask);
        tb = tb_next;
    }
    // every 4th small block and every 8th large one refresh the running threshold
    const bool refresh = small ? (chunk & 3) == 3 : ((chunk - small_chunks) & 7) == 7;
    prune_block_finish(lhist, wstage, wcnt, s_wcnt, &s_base, wtot, st, hist + (int64_t)unit * DC_HIST_BINS,
                       surv + (int64_t)unit * n_cap, refresh, (uint32_t)k_eff);
}

// sum over aligned groups of LPR lanes (4, 8 or 16)
template <int LPR>
__device__ __forceinline__ float sketch_group_sum(float v) {
    if (LPR == 4) {
        v += __builtin_amdgcn_update_dpp(0.0f, v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
        v += __builtin_amdgcn_update_dpp(0.0f, v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
        return v;
    }
    return dc_group_sum<(LPR == 8 ? 8 : 16)>(v);
}

// 16 code bytes (value + 128) times 16 weights, added to acc
__device__ __forceinline__ float sketch_dot16(const uint4 &c, const float (&w)[16], float acc) {
    const uint32_t x[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = fmaf((float)(x[i] & 0xffu), w[4 * i + 0], acc);
        acc = fmaf((float)((x[i] >> 8) & 0xffu), w[4 * i + 1], acc);
        acc = fmaf((float)((x[i] >> 16) & 0xffu), w[4 * i + 2], acc);
        acc = fmaf((float)(x[i] >> 24), w[4 * i + 3], acc);
    }
    return acc;
}

// Scan of the 8-bit sketch of the keys.  Row i of a unit is stored as codes
// u_id = c_id + 128 with k_id = a_d * c_id + e_id, |e_id| <= r_d (a: `scale`,
// r: `resid`, both per unit and channel).  The scan computes
//   approx_i = sum_d (q_d a_d) c_id,   |s_i - approx_i| <= E' for every row,
//   E' = sum_d |q_d| r_d + fp32 slack,
// where s_i is the fp32 score the exact kernels produce.  With A_k the k-th
// largest approx, every member of the exact top-k has approx_i >= A_k - 2E' - Q
// (Q: one quantisation step of the reference key in DC_MODE_REF_DIST, where equal
// keys of unequal scores tie).  So rows are histogrammed by bucket(approx_i), which
// yields the bucket of A_k exactly as in score_prune_kernel, and a row is kept when
// bucket(approx_i + margin) is not worse than the running threshold bucket,
// margin = 2E' + Q.  The kept rows are rescored exactly by rescore_kernel.
constexpr uint32_t kBulkKeep = 96;      // of the 128 rows of a wave's first two steps
// What the sketch scan keeps of a row: the row, and the bucket of (approximation + margin), which
// is all the exact pass asks of it (the exact pass keeps the row when that bucket is not worse
// than the final threshold bucket).  One word instead of (row, approximation): a byte the scan
// writes costs it several bytes read.  Rows of a unit beyond 2^22 do not fit: the callers send
// such regions down the bf16 route.
constexpr int kSketchRowBits = 22;
constexpr int kSketchMaxRows = 1 << kSketchRowBits;
static_assert(kSketchMaxRows == DC_SKETCH_MAX_ROWS && DC_HIST_BINS <= (1 << (32 - kSketchRowBits)), "row and bucket share a word");
__device__ __forceinline__ uint32_t sketch_entry(uint32_t bucket, uint32_t row) { return (bucket << kSketchRowBits) | row; }

template <int HD, bool SHARED_POLL>
__global__ __launch_bounds__(kThreads, HD <= 128 ? 4 : 1) void sketch_prune_kernel(
    const uint8_t *__restrict__ C, const uint16_t *__restrict__ Q, const float *__restrict__ scale,
    const float *__restrict__ resid, uint32_t *__restrict__ hist, UnitState *__restrict__ state,
    uint2 *__restrict__ surv, int n_units, int n_h, int n_cap, int64_t cb, int64_t ch, int64_t cr,
    int q_group, int mode, int k_eff, int small_chunks, int big_steps, const int32_t *__restrict__ hi_dev,
    int lo_row) {
    constexpr int LPR = HD / 16;  // lanes per row, 16 code bytes each
    const int n_rows = dc_live_rows(n_cap, hi_dev, lo_row);
    __shared__ uint32_t lhist[DC_HIST_BINS];
    __shared__ uint32_t stage[kStage];  // kept rows as kSketchEntry words
    __shared__ uint32_t s_tb;  // the block's copy of the unit's running threshold bucket
    __shared__ uint32_t wtot[kThreads / 64 + 1];
    __shared__ uint32_t s_wcnt[kThreads / 64];
    __shared__ uint32_t s_base;

    const int unit = blockIdx.x % n_units;
    const int chunk = blockIdx.x / n_units;
    const int b = unit / n_h, h = unit % n_h;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int grp = lane / LPR, col = lane % LPR;

    const bool small = chunk < small_chunks;
    const int big_chunks = (int)(gridDim.x / n_units) - small_chunks;
    const int big_id = small ? 0 : (int)(((int64_t)(chunk - small_chunks) + (int64_t)unit * 7) % big_chunks);
    const int64_t block_row0 =
        small ? (int64_t)chunk * kRowsPerBlockStep
              : (int64_t)small_chunks * kRowsPerBlockStep + (int64_t)big_id * big_steps * kRowsPerBlockStep;
    const int steps = small ? 1 : big_steps;

    if (block_row0 >= n_rows) return;  // the grid is laid out for n_cap rows
    for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;

    const uint8_t *Cu = C + b * cb + h * ch + col * 16;
    UnitState *st = state + unit;
    const int last = n_rows - 1;
    uint32_t tb = load_relaxed(&st->tb_run);

    // this lane's 16 weights q_d * a_d, the bias of the +128 code offset, and the margin
    float w[16];
    float bias, margin;
    {
        float qv[16];
        {
            float t[8];
            dc_load_query<HD>(Q, unit, q_group, 2 * col, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) qv[i] = t[i];
            dc_load_query<HD>(Q, unit, q_group, 2 * col + 1, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) qv[8 + i] = t[i];
        }
        const float4 *ap = reinterpret_cast<const float4 *>(scale + (int64_t)unit * HD + col * 16);
        const float4 *rp = reinterpret_cast<const float4 *>(resid + (int64_t)unit * HD + col * 16);
        float wsum = 0.f, wabs = 0.f, e = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 a4 = ap[i], r4 = rp[i];
            const float av[4] = {a4.x, a4.y, a4.z, a4.w}, rv[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float ww = qv[4 * i + j] * av[j];
                w[4 * i + j] = ww;
                wsum += ww;
                wabs += fabsf(ww);
                e += fabsf(qv[4 * i + j]) * rv[j];
            }
        }
        bias = -128.0f * wsum;
        wabs = sketch_group_sum<LPR>(wabs);
        e = sketch_group_sum<LPR>(e);
        margin = dc_sketch_margin(e, wabs, mode);
    }
    if (chunk == 0 && tid == 0) st->margin = __float_as_uint(margin);
    if (tid == 0) s_tb = tb;
    __syncthreads();

    uint32_t *wstage = stage + wave * (kBigSteps * 64);
    uint32_t wcnt = 0, marginal = 0;
    const unsigned long long lt = (1ull << lane) - 1ull;

    // Double buffering: the loads of the next step are issued before the current step is
    // worked on, so a wave always has a step's worth of bytes in flight.  The loads are
    // unconditional (past the block's end they repeat its last row), which lets the
    // compiler wait for exactly the older buffer instead of for every load in flight.
    const int64_t blk_end = block_row0 + (int64_t)steps * kRowsPerBlockStep - 1;
    const int64_t blk_last = blk_end < (int64_t)last ? blk_end : (int64_t)last;
    auto load_step = [&](int step, uint4 (&cv)[LPR]) __attribute__((always_inline)) {
        const int64_t row0 = block_row0 + (int64_t)step * kRowsPerBlockStep + wave * 64;
#pragma unroll
        for (int j = 0; j < LPR; ++j) {
            int64_t r = row0 + grp * LPR + j;
            r = r > blk_last ? blk_last : r;
            cv[j] = dc_load_stream16(Cu + r * cr);
        }
    };
    // COUNT: also count the rows kept although their own bucket is not better than the
    // threshold's (ties and near-ties); only the first two steps of a wave do.
    auto work_step = [&](int step, const uint4 (&cv)[LPR], auto count) __attribute__((always_inline)) {
        const int64_t row0 = block_row0 + (int64_t)step * kRowsPerBlockStep + wave * 64;
        float mine = 0.f;
#pragma unroll
        for (int j = 0; j < LPR; ++j) {
            const float p = sketch_group_sum<LPR>(sketch_dot16(cv[j], w, bias));
            mine = (col == j) ? p : mine;
        }
        const int64_t myrow = row0 + lane;
        const bool valid = myrow < n_rows;
        const uint32_t lb = dc_score_bucket(mine), kb = dc_score_bucket(mine + margin);
        const bool keep = valid && kb <= tb;
        if (keep) atomicAdd(&lhist[lb], 1u);
        const unsigned long long mask = __ballot(keep);
        if (keep) wstage[wcnt + __popcll(mask & lt)] = sketch_entry(kb, (uint32_t)myrow);
        wcnt += (uint32_t)__popcll(mask);
        if (decltype(count)::value) marginal += (uint32_t)__popcll(__ballot(keep && lb >= tb));
    };
    // steps of this wave that hold rows (wave-uniform)
    int my_steps = 0;
    {
        const int64_t first = block_row0 + wave * 64;
        if (first < n_rows) {
            const int64_t left = (int64_t)n_rows - first;
            my_steps = (int)((left + kRowsPerBlockStep - 1) / kRowsPerBlockStep);
            my_steps = my_steps < steps ? my_steps : steps;
        }
    }
    uint4 ca[LPR], cb2[LPR];
    load_step(0, ca);
    bool bulk = false;
    const bool had_tb = tb < (uint32_t)DC_HIST_BINS;  // the first steps are judged against a real threshold
    // The threshold poll is issued before the prefetch: loads return in order, so waiting
    // for a poll that was issued last would also wait for the whole prefetch.
    int step = 0;
    // With few units the whole chip polls a handful of lines, and every poll holds back
    // the younger loads of its wave (the poll is an agent-scope load): then only wave 0
    // polls and passes the value on through LDS.  With many units every wave polls for
    // itself, which keeps its threshold one step fresher.
    // (SHARED_POLL is a template parameter: as a run-time choice it costs registers.)
    auto two_steps = [&](auto count) __attribute__((always_inline)) {
        uint32_t tb_next = tb;
        if (!SHARED_POLL || wave == 0) tb_next = load_relaxed(&st->tb_run);
        load_step(step + 1, cb2);
        work_step(step, ca, count);
        if (SHARED_POLL) {
            if (wave == 0 && lane == 0) lds_store_relaxed(&s_tb, tb_next);
            tb = lds_load_relaxed(&s_tb);
        } else {
            tb = tb_next;
        }
        if (!SHARED_POLL || wave == 0) tb_next = load_relaxed(&st->tb_run);
        load_step(step + 2, ca);
        work_step(step + 1, cb2, count);
        if (SHARED_POLL) {
            if (wave == 0 && lane == 0) lds_store_relaxed(&s_tb, tb_next);
            tb = lds_load_relaxed(&s_tb);
        } else {
            tb = tb_next;
        }
        step += 2;
    };
    if (my_steps >= 2) {
        two_steps(std::true_type{});
        // Degenerate data (rows that nearly all tie with the k-th best: the sketch prunes nothing):
        // a wave that kept three quarters of the rows of its first two steps without any of them
        // being better than the threshold stops reading codes and keeps the rest of its rows unseen.
        // An unseen row carries the best possible approximation, so the exact rescoring takes it
        // in any case, and it is left out of the histogram, which only loosens the threshold: the
        // selected ids are the same, the scan costs a quarter.
        bulk = had_tb && marginal >= kBulkKeep;
    }
    while (!bulk && step + 1 < my_steps) two_steps(std::false_type{});
    if (bulk) {
        for (; step < my_steps; ++step) {
            const int64_t myrow = block_row0 + (int64_t)step * kRowsPerBlockStep + wave * 64 + lane;
            const bool keep = myrow < n_rows;
            const unsigned long long mask = __ballot(keep);
            if (keep) wstage[wcnt + __popcll(mask & lt)] = sketch_entry(0u, (uint32_t)myrow);  // passes any threshold
            wcnt += (uint32_t)__popcll(mask);
        }
    } else if (step < my_steps) {
        work_step(step, ca, std::false_type{});  // an odd last step; its rows are already on the way
    }
    const bool refresh = small ? (chunk & 3) == 3 : ((chunk - small_chunks) & 7) == 7;
    prune_block_finish<kThreads, uint32_t>(lhist, wstage, wcnt, s_wcnt, &s_base, wtot, st,
                                           hist + (int64_t)unit * DC_HIST_BINS,
                                           reinterpret_cast<uint32_t *>(surv) + (int64_t)unit * n_cap, refresh,
                                           (uint32_t)k_eff);
}

// The same scan for the PQ baseline: a key's score is its ADC score (dc_pq.h), read
// from M code bytes per key, in DC_MODE_IP order.  One key per lane.  The unit's
// tables are staged per block, so blocks are large: 512 threads, 512 keys per step.
template <int M>
__global__ __launch_bounds__(kPqThreads) void pq_prune_kernel(
    const uint8_t *__restrict__ codes, const float *__restrict__ lut, uint32_t *__restrict__ hist,
    UnitState *__restrict__ state, uint2 *__restrict__ surv, int n_units, int n_rows, int k_eff,
    int small_chunks, int big_steps) {
    constexpr int NW = M / 4;
    constexpr int kWaves = kPqThreads / 64;
    __shared__ float s_lut[kPqLutWords];
    __shared__ uint32_t lhist[DC_HIST_BINS];
    __shared__ uint2 stage[kWaves * kPqBigSteps * 64];
    __shared__ uint32_t s_tb;  // the block's copy of the unit's running threshold bucket
    __shared__ uint32_t wtot[kWaves + 1];
    __shared__ uint32_t s_wcnt[kWaves];
    __shared__ uint32_t s_base;

    const int unit = blockIdx.x % n_units;
    const int chunk = blockIdx.x / n_units;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const bool small = chunk < small_chunks;
    const int big_chunks = (int)(gridDim.x / n_units) - small_chunks;
    const int big_id = small ? 0 : (int)(((int64_t)(chunk - small_chunks) + (int64_t)unit * 7) % big_chunks);
    const int64_t block_row0 =
        small ? (int64_t)chunk * kPqThreads
              : (int64_t)small_chunks * kPqThreads + (int64_t)big_id * big_steps * kPqThreads;
    const int steps = small ? 1 : big_steps;

    for (int i = tid; i < DC_HIST_BINS; i += kPqThreads) lhist[i] = 0;
    pq_stage_lut<M>(s_lut, lut + (int64_t)unit * M * 256, tid, kPqThreads);
    PqLane<M> ln;
    ln.init(lane);
    UnitState *st = state + unit;
    const int64_t last = n_rows - 1;
    uint32_t tb = load_relaxed(&st->tb_run);
    const uint8_t *cu = codes + (int64_t)unit * n_rows * M;
    // rows are a multiple of 64 from the start of the unit: lane = key mod 64, as pq_adc_score expects
    const int64_t blk_end = block_row0 + (int64_t)steps * kPqThreads - 1;
    const int64_t blk_last = blk_end < last ? blk_end : last;
    auto load_row = [&](int64_t row0, uint32_t(&w)[NW]) {
        int64_t r = row0 + lane;
        r = r > blk_last ? blk_last : r;
        // plain loads: the two halves of a 32-byte row come from the same cache line
        const uint4 *cp = reinterpret_cast<const uint4 *>(cu + r * M);
#pragma unroll
        for (int i = 0; i < NW / 4; ++i) {
            const uint4 t = cp[i];
            w[4 * i + 0] = t.x;
            w[4 * i + 1] = t.y;
            w[4 * i + 2] = t.z;
            w[4 * i + 3] = t.w;
        }
    };
    // A wave keeps the codes of kAhead steps in flight beyond the one it scores: 32 bytes
    // per lane and step are too few to cover the memory latency otherwise.  Loads return
    // in order, so the threshold polled before the rows of step s + kAhead is first looked
    // at when those rows are, and never makes the wave wait for younger loads.  The
    // requests are issued unconditionally (past the block's end they repeat its last
    // row) so that the number of loads in flight is the same on every path.
    constexpr int kAhead = 3, kRing = kAhead + 1;
    uint32_t buf[kRing][NW];
    const int64_t wave_row0 = block_row0 + wave * 64;
    const int64_t rows_left = (int64_t)n_rows - wave_row0;
    const int64_t steps_left = (rows_left + kPqThreads - 1) / kPqThreads;
    const int my_steps = rows_left <= 0 ? 0 : (int)(steps_left < steps ? steps_left : steps);
    uint32_t tb_polled = tb;
    if (tid == 0) s_tb = tb;
#pragma unroll
    for (int j = 0; j < kAhead; ++j) load_row(wave_row0 + (int64_t)j * kPqThreads, buf[j]);
    __syncthreads();

    // each wave stages its survivors in its own slice (at most 64 per step)
    uint2 *wstage = stage + wave * (kPqBigSteps * 64);
    uint32_t wcnt = 0;
    const unsigned long long lt = (1ull << lane) - 1ull;

    for (int s0 = 0; s0 < my_steps; s0 += kRing) {
#pragma unroll
        for (int j = 0; j < kRing; ++j) {
            const int step = s0 + j;
            const int64_t row0 = wave_row0 + (int64_t)step * kPqThreads;
            // The poll crosses the chip (agent scope) and every younger load of the wave
            // queues behind it, so only wave 0 polls, once per kRing steps, and hands the
            // value to the other waves through LDS when it has arrived.
            if (wave == 0 && j == 0) tb_polled = load_relaxed(&st->tb_run);
            load_row(row0 + (int64_t)kAhead * kPqThreads, buf[(j + kAhead) % kRing]);
            if (wave == 0 && j == kAhead && lane == 0) lds_store_relaxed(&s_tb, tb_polled);
            if (step < my_steps) {  // wave-uniform; no barrier inside the loop
                const float mine = pq_adc_score<M>(buf[j], s_lut, ln);
                tb = lds_load_relaxed(&s_tb);
                const int64_t myrow = row0 + lane;
                const bool valid = myrow < n_rows;
                uint32_t key = 0, bucket = 0xffffffffu;
                if (valid) dc_key_bucket(mine, DC_MODE_IP, key, bucket);
                const bool keep = valid && bucket <= tb;
                if (keep) atomicAdd(&lhist[bucket], 1u);
                const unsigned long long mask = __ballot(keep);
                if (keep)
                    wstage[wcnt + __popcll(mask & lt)] = make_uint2((uint32_t)myrow, __float_as_uint(mine));
                wcnt += (uint32_t)__popcll(mask);
            }
        }
    }
    // every 4th small block and every 2nd large one refresh the running threshold
    const bool refresh = small ? (chunk & 3) == 3 : ((chunk - small_chunks) & 1) == 1;
    prune_block_finish<kPqThreads>(lhist, wstage, wcnt, s_wcnt, &s_base, wtot, st,
                                   hist + (int64_t)unit * DC_HIST_BINS, surv + (int64_t)unit * n_rows,
                                   refresh, (uint32_t)k_eff);
}

// Several blocks per unit split the unit's survivor list: rows in buckets better
// than the threshold bucket are certain members and go straight to idx_out, rows
// in the threshold bucket become candidates.  Each block reserves its output
// ranges with one returning atomic per list.
constexpr int kClassifyBatch = 4;

__global__ __launch_bounds__(kThreads) void classify_kernel(
    const uint32_t *__restrict__ hist, UnitState *__restrict__ state, const uint2 *__restrict__ surv,
    uint32_t *__restrict__ cand_key, uint32_t *__restrict__ cand_idx, uint32_t *__restrict__ idx_out,
    int64_t idx_stride, uint32_t *__restrict__ sel_keys, int n_units, int n_rows, int k_eff, int mode,
    int nblk) {
    __shared__ uint32_t wtot[kThreads / 64 + 1];
    __shared__ uint32_t sres[2];
    __shared__ uint32_t sbase[2];
    const int unit = blockIdx.x % n_units;
    const int blk = blockIdx.x / n_units;
    const int tid = threadIdx.x;
    UnitState *st = state + unit;
    const uint2 *su = surv + (int64_t)unit * n_rows;
    const uint32_t cap = (uint32_t)n_rows;
    uint32_t n_s = st->surv_cnt;
    if (n_s > cap) n_s = cap;
    // every block takes one contiguous slice of whole batches
    constexpr uint32_t kPer = kClassifyBatch * kThreads;
    const uint32_t per = ((n_s + (uint32_t)nblk - 1) / (uint32_t)nblk + kPer - 1) / kPer * kPer;
    const uint32_t lo = (uint32_t)blk * per;
    uint32_t hi = lo + per;
    if (hi > n_s) hi = n_s;
    if (lo >= n_s && blk != 0) return;

    const uint32_t kk = (uint32_t)k_eff;
    uint32_t tb, c_less;
    unit_threshold(hist + (int64_t)unit * DC_HIST_BINS, kk, wtot, sres, tb, c_less);
    if (blk == 0 && tid == 0) st->c_less = c_less;

    uint32_t *ck = cand_key + (int64_t)unit * n_rows;
    uint32_t *ci = cand_idx + (int64_t)unit * n_rows;
    uint32_t *io = idx_out + (int64_t)unit * idx_stride;
    uint32_t *ko = sel_keys ? sel_keys + (int64_t)unit * k_eff : nullptr;

    for (uint32_t i0 = lo; i0 < hi; i0 += kPer) {
        uint2 p[kClassifyBatch];
#pragma unroll
        for (int j = 0; j < kClassifyBatch; ++j) {
            const uint32_t i = i0 + j * kThreads + tid;
            p[j] = make_uint2(0u, 0u);
            if (i < hi) p[j] = su[i];
        }
        uint32_t keys[kClassifyBatch];
        uint32_t wmask = 0, cmask = 0;
#pragma unroll
        for (int j = 0; j < kClassifyBatch; ++j) {
            const uint32_t i = i0 + j * kThreads + tid;
            uint32_t key = 0, bucket = 0xffffffffu;
            if (i < hi) dc_key_bucket(__uint_as_float(p[j].y), mode, key, bucket);
            keys[j] = key;
            if (bucket < tb) wmask |= 1u << j;
            else if (bucket == tb) cmask |= 1u << j;
        }
        uint32_t tot;
        const uint32_t ex = block_excl_scan<kThreads>(__popc(wmask) | (__popc(cmask) << 16), wtot, &tot);
        if (tid == 0) {
            const uint32_t nw = tot & 0xffffu, nc = tot >> 16;
            sbase[0] = nw ? atomicAdd(&st->win_cnt, nw) : 0u;
            sbase[1] = nc ? atomicAdd(&st->cand_cnt, nc) : 0u;
        }
        __syncthreads();
        uint32_t wpos = sbase[0] + (ex & 0xffffu), cpos = sbase[1] + (ex >> 16);
#pragma unroll
        for (int j = 0; j < kClassifyBatch; ++j) {
            if (wmask & (1u << j)) {
                if (wpos < kk) {
                    io[wpos] = p[j].x;
                    if (ko) ko[wpos] = keys[j];
                }
                ++wpos;
            } else if (cmask & (1u << j)) {
                if (cpos < cap) {
                    ck[cpos] = keys[j];
                    ci[cpos] = p[j].x;
                }
                ++cpos;
            }
        }
        __syncthreads();  // sbase is rewritten by the next batch
    }
}

// Second pass of the sketch path.  Several blocks per unit split the list the
// sketch scan left ((id, approx) pairs): a row stays a candidate when
// bucket(approx + margin) is not worse than the exact bucket of the k-th largest
// approx; candidates get their exact fp32 score from the bf16 row, computed lane for
// lane as score_kernel computes it, and their (key, id) go to the unit's candidate
// list, from which select_finish_kernel picks the k best (c_less = 0: the list
// holds every member of the top-k).
constexpr int kRescoreBatch = 4;

template <int HD>
__global__ __launch_bounds__(kThreads) void rescore_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ Q, const uint32_t *__restrict__ hist,
    UnitState *__restrict__ state, const uint2 *__restrict__ surv, uint32_t *__restrict__ cand_key,
    uint32_t *__restrict__ cand_idx, int n_units, int n_h, int n_rows, int64_t sb, int64_t sh,
    int64_t sr, int q_group, int mode, int k_eff, int nblk) {
    constexpr int LPR = HD / 8;
    constexpr int GROUPS = kThreads / LPR;
    constexpr uint32_t kPer = kRescoreBatch * kThreads;
    __shared__ uint32_t cid[kPer];
    __shared__ uint32_t ckey[kPer];
    __shared__ uint32_t wtot[kThreads / 64 + 1];
    __shared__ uint32_t sres[2];
    __shared__ uint32_t s_base;
    const int unit = blockIdx.x % n_units;
    const int blk = blockIdx.x / n_units;
    const int b = unit / n_h, h = unit % n_h;
    const int tid = threadIdx.x;
    const int grp = tid / LPR, col = tid % LPR;
    UnitState *st = state + unit;
    uint32_t opaque_zero = 0;
    asm volatile("" : "+v"(opaque_zero));
    // The list is dealt to the unit's blocks in tiles of kThreads entries, round robin:
    // the scan appends in the order its blocks finish, and the entries of late blocks
    // (tight threshold) pass the filter far more often than those of early ones, so
    // contiguous slices would leave a few blocks with most of the gathers.
    auto entry = [&](uint32_t t) { return ((uint32_t)blk + t * (uint32_t)nblk) * kThreads + (uint32_t)tid; };

    // The block's first batch of the list is requested before its length is known (what lies
    // beyond the length is stale and is masked below), together with the length, the histogram
    // and the query: one memory round trip for all of them.
    const uint32_t *su = reinterpret_cast<const uint32_t *>(surv) + (int64_t)unit * n_rows;
    uint32_t p[kRescoreBatch];
#pragma unroll
    for (int j = 0; j < kRescoreBatch; ++j) {
        const uint32_t i = entry((uint32_t)j);
        p[j] = 0xffffffffu;
        if (i < (uint32_t)n_rows) p[j] = su[i];
    }
    uint32_t n_s = st->surv_cnt;
    float q[8];
    dc_load_query<HD>(Q, unit, q_group, col, q);
    uint32_t tb, c_less;
    unit_threshold(hist + (int64_t)unit * DC_HIST_BINS, (uint32_t)k_eff, wtot, sres, tb, c_less);
    if (n_s > (uint32_t)n_rows) n_s = n_rows;
    const uint32_t n_tiles = (n_s + kThreads - 1) / kThreads;
    if ((uint32_t)blk >= n_tiles) return;
    const uint32_t my_tiles = (n_tiles - (uint32_t)blk + (uint32_t)nblk - 1) / (uint32_t)nblk;
    if (blk == 0 && tid == 0) st->c_less = 0;
    const uint16_t *Ku = K + b * sb + h * sh + col * 8;
    uint32_t *ck = cand_key + (int64_t)unit * n_rows;
    uint32_t *ci = cand_idx + (int64_t)unit * n_rows;

    for (uint32_t t0 = 0; t0 < my_tiles; t0 += kRescoreBatch) {
        uint32_t pass = 0;
#pragma unroll
        for (int j = 0; j < kRescoreBatch; ++j) {
            const uint32_t t = t0 + (uint32_t)j;
            const uint32_t i = entry(t);
            const bool in = t < my_tiles && i < n_s;
            if (t0 != 0) {
                p[j] = 0xffffffffu;
                if (in) p[j] = su[i];
            }
            if (in && (p[j] >> kSketchRowBits) <= tb) pass |= 1u << j;
        }
        uint32_t n_c;
        uint32_t pos = block_excl_scan<kThreads>(__popc(pass), wtot, &n_c);
#pragma unroll
        for (int j = 0; j < kRescoreBatch; ++j)
            if (pass & (1u << j)) cid[pos++] = p[j] & (uint32_t)(kSketchMaxRows - 1);
        // The list slot is reserved now and looked at after the rows are scored.  (Through an address
        // the compiler cannot prove uniform: it turns an atomic on a uniform address into one atomic
        // per wave plus a broadcast of the result and waits for that on the spot, a memory round
        // trip in front of the barrier below and of every row request behind it.)
        uint32_t base_reg = 0;
        if (tid == 0 && n_c) base_reg = atomicAdd(&st->cand_cnt + opaque_zero, n_c);
        __syncthreads();
        // exact scores: one LPR-lane group per row, kRowsInFlight rows of a group in flight
        constexpr int kRowsInFlight = 8;
        for (uint32_t j0 = 0; j0 < n_c; j0 += GROUPS * kRowsInFlight) {
            uint4 wv[kRowsInFlight];
#pragma unroll
            for (int u = 0; u < kRowsInFlight; ++u) {
                uint32_t j = j0 + u * GROUPS + grp;
                j = j < n_c ? j : n_c - 1;
                wv[u] = *reinterpret_cast<const uint4 *>(Ku + (int64_t)cid[j] * sr);
            }
#pragma unroll
            for (int u = 0; u < kRowsInFlight; ++u) {
                const uint32_t j = j0 + u * GROUPS + grp;
                const float sc = dc_group_sum<LPR>(dc_dot8(wv[u], q, 0.f));
                if (col == 0 && j < n_c) {
                    uint32_t key, bucket;
                    dc_key_bucket(sc, mode, key, bucket);
                    ckey[j] = key;
                }
            }
        }
        if (tid == 0) s_base = base_reg;
        __syncthreads();
        for (uint32_t i = tid; i < n_c; i += kThreads) {
            const uint32_t slot = s_base + i;
            if (slot < (uint32_t)n_rows) {
                ck[slot] = ckey[i];
                ci[slot] = cid[i];
            }
        }
        __syncthreads();  // cid, ckey and s_base are rewritten by the next batch
    }
}

// Exact scores of the rows the PQ scan selected: one LPR-lane group per row, the
// arithmetic of score_gathered_kernel.  Their (key, id) become the unit's candidate
// list, from which select_finish_kernel picks the best (c_less = 0).
template <int HD>
__global__ __launch_bounds__(kThreads) void pq_rescore_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ Q, const uint32_t *__restrict__ idx,
    UnitState *__restrict__ state, uint32_t *__restrict__ cand_key, uint32_t *__restrict__ cand_idx,
    int n_h, int n_idx, int64_t idx_stride, int n_rows, int64_t sb, int64_t sh, int64_t sr,
    int blocks_per_unit) {
    constexpr int LPR = HD / 8;
    constexpr int GROUPS = kThreads / LPR;
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int grp = threadIdx.x / LPR, col = threadIdx.x % LPR;
    if (chunk == 0 && threadIdx.x == 0) {
        state[unit].cand_cnt = (uint32_t)n_idx;
        state[unit].c_less = 0;
    }
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = dc_bf16_to_f32(Q[(int64_t)unit * HD + col * 8 + i]);
    const int j = chunk * GROUPS + grp;
    const int jj = j < n_idx ? j : n_idx - 1;
    const uint32_t id = idx[(int64_t)unit * idx_stride + jj];
    const uint4 w = *reinterpret_cast<const uint4 *>(K + b * sb + h * sh + (int64_t)id * sr + col * 8);
    const float p = dc_group_sum<LPR>(dc_dot8(w, q, 0.f));
    if (j < n_idx && col == 0) {
        uint32_t key, bucket;
        dc_key_bucket(p, DC_MODE_IP, key, bucket);
        cand_key[(int64_t)unit * n_rows + j] = key;
        cand_idx[(int64_t)unit * n_rows + j] = id;
    }
}

// One block per unit: radix select among the candidates of the threshold bucket
// fills idx_out[c_less, k).  Leaves the unit's list cursors at zero.
__global__ __launch_bounds__(kFinalThreads) void select_finish_kernel(
    uint32_t *__restrict__ hist, UnitState *__restrict__ state, uint32_t *__restrict__ cand_key,
    uint32_t *__restrict__ cand_idx, uint32_t *__restrict__ idx_out, int64_t idx_stride,
    uint32_t *__restrict__ sel_keys, int n_rows, int k_eff, int reinit) {
    __shared__ uint32_t lh[kRadixBins];
    __shared__ uint32_t wtot[kFinalThreads / 64 + 1];
    __shared__ uint32_t sres[4];
    __shared__ uint32_t smisc[2];
    __shared__ uint32_t lck[kCandLds], lci[kCandLds];  // candidates are staged in LDS when they fit
    const int unit = blockIdx.x;
    const int tid = threadIdx.x;
    UnitState *st = state + unit;
    uint32_t *ck = cand_key + (int64_t)unit * n_rows;
    uint32_t *ci = cand_idx + (int64_t)unit * n_rows;
    // the head of the candidate list (what a list of ordinary length holds) is fetched before
    // its length is known: one memory round trip less
    constexpr int kHead = 4;
    uint32_t hk[kHead], hi[kHead];
#pragma unroll
    for (int j = 0; j < kHead; ++j) {
        const int i = tid + j * kFinalThreads;
        hk[j] = hi[j] = 0;
        if (i < n_rows) {
            hk[j] = ck[i];
            hi[j] = ci[i];
        }
    }
    uint32_t n_c = st->cand_cnt;
    const uint32_t c_less = st->c_less;
    if (n_c > (uint32_t)n_rows) n_c = n_rows;
    const uint32_t kk = (uint32_t)k_eff;
    uint32_t *io = idx_out + (int64_t)unit * idx_stride;
    uint32_t *ko = sel_keys ? sel_keys + (int64_t)unit * k_eff : nullptr;
    const bool staged = n_c <= (uint32_t)kCandLds;
    if (staged) {
#pragma unroll
        for (int j = 0; j < kHead; ++j) {
            const uint32_t i = (uint32_t)(tid + j * kFinalThreads);
            if (i < n_c) {
                lck[i] = hk[j];
                lci[i] = hi[j];
            }
        }
        for (uint32_t i = tid + kHead * kFinalThreads; i < n_c; i += kFinalThreads) {
            lck[i] = ck[i];
            lci[i] = ci[i];
        }
    }
    __syncthreads();  // every thread has read the counters
    if (reinit) {
        // leave the unit's histogram and threshold ready for the next scan
        uint4 *hz = reinterpret_cast<uint4 *>(hist + (int64_t)unit * DC_HIST_BINS);
        if (tid < DC_HIST_BINS / 4) hz[tid] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (tid == 0) {
        if (reinit) {
            st->tb_run = DC_HIST_BINS;
            st->surv_cnt = 0;
        }
        st->win_cnt = 0;
        st->cand_cnt = 0;
    }
    if (c_less >= kk) return;
    uint32_t need = kk - c_less;
    if (need > n_c) need = n_c;
    if (n_c <= 128u) {
        // Short list: every thread ranks its own candidate among all of them by
        // (key, id).  The packed pairs sit in lh, padded with a sentinel to a multiple
        // of 8; the reads in the loop are wave-uniform 16-byte broadcasts.
        unsigned long long *comp = reinterpret_cast<unsigned long long *>(lh);
        const unsigned long long mine = ((unsigned long long)hk[0] << 32) | hi[0];
        comp[tid] = (uint32_t)tid < n_c ? mine : ~0ull;
        __syncthreads();
        if ((uint32_t)tid < n_c) {
            const ulonglong2 *c2 = reinterpret_cast<const ulonglong2 *>(comp);
            const uint32_t n8 = (n_c + 7u) / 8u;
            uint32_t rank = 0;
            for (uint32_t j = 0; j < n8; ++j) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const ulonglong2 t = c2[4 * j + u];
                    rank += (t.x < mine ? 1u : 0u) + (t.y < mine ? 1u : 0u);
                }
            }
            if (rank < need) {
                io[c_less + rank] = hi[0];
                if (ko) ko[c_less + rank] = hk[0];
            }
        }
        return;
    }
    // Two calls, so that the staged list is read with LDS instructions: through a pointer chosen
    // at run time every access would be a flat one, and waiting for a flat load also waits for
    // the stores issued above.
    if (staged) dc_finalize_unit<true>(lck, lci, n_c, need, io + c_less, n_rows, lh, wtot, sres, smisc, ko ? ko + c_less : nullptr);
    else dc_finalize_unit(ck, ci, n_c, need, io + c_less, n_rows, lh, wtot, sres, smisc, ko ? ko + c_less : nullptr);
}

}  // namespace

extern "C" size_t dc_score_select_workspace_bytes(int n_units, int n_rows, int k) {
    return carve_fused(nullptr, n_units, n_rows, k).bytes;
}

extern "C" size_t dc_sketch_select_workspace_bytes(int n_units, int n_rows, int k) {
    return carve_fused(nullptr, n_units, n_rows, k).bytes;  // the same lists serve both paths
}

namespace {

constexpr int kSketchFillBlocks = 512;  // see plan_fused

struct FusedPlan {
    int n_units, k_eff, small_chunks, big_steps;
    int64_t blocks;
};

int plan_fused(const char *who, int n_b, int n_h, int n_rows, int budget, FusedPlan *p,
               int big_steps = kBigSteps, int rows_per_step = kRowsPerBlockStep, int fill_div = 2048) {
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_rows >= 0 && budget >= 0, "%s: bad sizes", who);
    const int64_t n_units64 = (int64_t)n_b * n_h;
    DC_REQUIRE(n_units64 < (1 << 20), "%s: too many units", who);
    p->n_units = (int)n_units64;
    p->k_eff = budget < n_rows ? budget : n_rows;
    // chunks per unit: up to kSmallChunks blocks of one step, then blocks of big_steps steps.
    // Short scans take fewer steps per block so that the grid still has fill_div blocks or
    // more: a block's steps run one after the other, and with few blocks the kernel
    // lasts as long as its longest block.  (2048 for the bf16 and PQ scans; the sketch scan,
    // whose blocks cost more to start and to end than their steps cost, does better with 512:
    // 34 against 42 us at 8 units x 131072 rows, 37 against 46 us at 32 units x 32768 rows.)
    const int64_t tiles = ((int64_t)n_rows + rows_per_step - 1) / rows_per_step;
    const int64_t fill = n_units64 * tiles / fill_div;
    if (fill < big_steps) big_steps = fill < 1 ? 1 : (int)fill;
    p->big_steps = big_steps;
    p->small_chunks = (int)(tiles < kSmallChunks ? tiles : kSmallChunks);
    const int64_t rest = (int64_t)n_rows - (int64_t)p->small_chunks * rows_per_step;
    const int64_t big_rows = (int64_t)p->big_steps * rows_per_step;
    const int64_t big_chunks = rest > 0 ? (rest + big_rows - 1) / big_rows : 0;
    p->blocks = n_units64 * (p->small_chunks + big_chunks);
    DC_REQUIRE(p->blocks < (1ll << 31), "%s: grid too large", who);
    return DC_OK;
}

int check_ws(const char *who, void *workspace, size_t workspace_bytes, int n_units, int n_rows,
             int budget, FusedWs *w) {
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "%s: workspace must be non-null and 256-byte aligned", who);
    *w = carve_fused(workspace, n_units, n_rows, budget);
    if (workspace_bytes < w->bytes) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, workspace_bytes, w->bytes);
        return DC_ENOMEM;
    }
    return DC_OK;
}

}  // namespace

extern "C" int dc_select_state_init(int n_units, int n_rows, int budget, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    DC_REQUIRE(n_units >= 0 && n_rows >= 0 && budget >= 0, "dc_select_state_init: bad sizes");
    if (n_units == 0) return DC_OK;
    FusedWs w;
    int rc = check_ws("dc_select_state_init", workspace, workspace_bytes, n_units, n_rows, budget, &w);
    if (rc) return rc;
    const int64_t n = (int64_t)n_units * DC_HIST_BINS;
    hipLaunchKernelGGL(init_state_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, w.hist, w.state, n_units);
    DC_CHECK_LAUNCH("dc_select_state_init");
    return DC_OK;
}

extern "C" int dc_score_prune_bf16(const void *k, const void *q, int n_b, int n_h, int n_rows, int hd,
                                   int64_t sb, int64_t sh, int64_t sr, int q_group, int budget,
                                   int mode, void *workspace, size_t workspace_bytes, void *stream) {
    return dc_score_prune_launch(k, q, n_b, n_h, n_rows, hd, sb, sh, sr, q_group, budget, mode, workspace,
                                 workspace_bytes, stream, nullptr, 0);
}

// hi_dev: null, or a device word holding the row at which the region ends at the time the kernel
// runs (lo_row: its first row); n_rows is then the capacity that the grid and the lists are laid
// out for.
int dc_score_prune_launch(const void *k, const void *q, int n_b, int n_h, int n_rows, int hd, int64_t sb, int64_t sh,
                          int64_t sr, int q_group, int budget, int mode, void *workspace, size_t workspace_bytes,
                          void *stream, const int32_t *hi_dev, int lo_row) {
    DC_REQUIRE(k && q, "dc_score_prune_bf16: null pointer");
    DC_REQUIRE(q_group >= 1, "dc_score_prune_bf16: bad q_group");
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "dc_score_prune_bf16: head_dim %d not in {64,128,256}", hd);
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "dc_score_prune_bf16: bad mode %d", mode);
    DC_REQUIRE(dc_aligned16(k), "dc_score_prune_bf16: k must be 16-byte aligned");
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0 && sr >= hd,
               "dc_score_prune_bf16: strides must be multiples of 8 elements and row_stride >= hd");
    FusedPlan p;
    // (short scans of up to 32 units: eight steps per block down to 512 blocks, like the sketch scan)
    int rc = plan_fused("dc_score_prune_bf16", n_b, n_h, n_rows, budget, &p, kBigSteps, kRowsPerBlockStep,
                        (int64_t)n_b * n_h <= 32 ? kSketchFillBlocks : 2048);
    if (rc) return rc;
    if (p.n_units == 0 || p.k_eff == 0) return DC_OK;
    FusedWs w;
    rc = check_ws("dc_score_prune_bf16", workspace, workspace_bytes, p.n_units, n_rows, budget, &w);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
#define DC_LAUNCH_SP(HD)                                                                           \
    hipLaunchKernelGGL(score_prune_kernel<HD>, dim3((unsigned)p.blocks), dim3(kThreads), 0, st,    \
                       (const uint16_t *)k, (const uint16_t *)q, w.hist, w.state, w.surv,          \
                       p.n_units, n_h, n_rows, sb, sh, sr, q_group, mode, p.k_eff, p.small_chunks,  \
                       p.big_steps, hi_dev, lo_row)
    if (hd == 64) DC_LAUNCH_SP(64);
    else if (hd == 128) DC_LAUNCH_SP(128);
    else DC_LAUNCH_SP(256);
#undef DC_LAUNCH_SP
    DC_CHECK_LAUNCH("dc_score_prune_bf16");
    return DC_OK;
}

namespace {

// finish (+ sort): picks min(k, candidates) from the unit's candidate list
int launch_finish(const char *who, const FusedWs &w, uint32_t *idx_out, int64_t idx_unit_stride, int n_units,
                  int n_rows, int k_eff, int mode, int order, int reinit, hipStream_t st) {
    uint32_t *sel_keys = order == DC_ORDER_BEST ? w.sel_keys : nullptr;
    hipLaunchKernelGGL(select_finish_kernel, dim3(n_units), dim3(kFinalThreads), 0, st, w.hist, w.state,
                       w.cand_key, w.cand_idx, idx_out, idx_unit_stride, sel_keys, n_rows, k_eff, reinit);
    DC_CHECK_LAUNCH(who);
    if (order != DC_ORDER_ANY)
        return dc_sort_selected(nullptr, 0, sel_keys, idx_out, idx_unit_stride, w.sort_scratch, n_units,
                                k_eff, mode, order, st, n_rows);
    return DC_OK;
}

// classify + finish (+ sort) on the survivor list of score_prune_kernel
int launch_select(const char *who, const FusedWs &w, uint32_t *idx_out, int64_t idx_unit_stride, int n_units,
                  int n_rows, int k_eff, int mode, int order, int reinit, hipStream_t st) {
    uint32_t *sel_keys = order == DC_ORDER_BEST ? w.sel_keys : nullptr;
    // blocks per unit for the classify pass: one per 4096 rows of context, as long as
    // the grid stays near 2048 blocks
    // one block per 4096 rows and at most 2048 blocks; below 3 Mi rows in all, one per 1024 rows
    // and at most 1024 blocks (8 x 131072 rows: 5.5 us against 7.1 us)
    const bool few = (int64_t)n_units * n_rows < (3ll << 20);
    int nblk = few ? (n_rows + 1023) / 1024 : (n_rows + 4095) / 4096;
    const int grid = few ? 1024 : 2048;
    const int cap = n_units >= grid ? 1 : grid / n_units;
    if (nblk > cap) nblk = cap;
    if (nblk < 1) nblk = 1;
    hipLaunchKernelGGL(classify_kernel, dim3((unsigned)n_units * (unsigned)nblk), dim3(kThreads), 0, st,
                       w.hist, w.state, w.surv, w.cand_key, w.cand_idx, idx_out, idx_unit_stride, sel_keys,
                       n_units, n_rows, k_eff, mode, nblk);
    DC_CHECK_LAUNCH(who);
    return launch_finish(who, w, idx_out, idx_unit_stride, n_units, n_rows, k_eff, mode, order, reinit, st);
}

}  // namespace

extern "C" int dc_sparse_select(uint32_t *idx_out, int64_t idx_unit_stride, int n_units, int n_rows,
                                int budget, int mode, int order, int reinit, void *workspace,
                                size_t workspace_bytes, void *stream) {
    DC_REQUIRE(idx_out, "dc_sparse_select: null pointer");
    DC_REQUIRE(n_units >= 0 && n_rows >= 0 && budget >= 0, "dc_sparse_select: bad sizes");
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "dc_sparse_select: bad mode %d", mode);
    DC_REQUIRE(order >= DC_ORDER_ANY && order <= DC_ORDER_INDEX, "dc_sparse_select: bad order %d", order);
    const int k_eff = budget < n_rows ? budget : n_rows;
    if (n_units == 0 || k_eff == 0) return DC_OK;
    DC_REQUIRE(idx_unit_stride >= k_eff, "dc_sparse_select: idx_unit_stride < min(budget, n_rows)");
    FusedWs w;
    int rc = check_ws("dc_sparse_select", workspace, workspace_bytes, n_units, n_rows, budget, &w);
    if (rc) return rc;
    return launch_select("dc_sparse_select", w, idx_out, idx_unit_stride, n_units, n_rows, k_eff, mode, order,
                         reinit, (hipStream_t)stream);
}

extern "C" int dc_score_select_bf16(const void *k, const void *q, uint32_t *idx_out,
                                    int64_t idx_unit_stride, int n_b, int n_h, int n_rows, int hd,
                                    int64_t sb, int64_t sh, int64_t sr, int q_group, int budget,
                                    int mode, int order, void *workspace, size_t workspace_bytes,
                                    void *stream) {
    DC_REQUIRE(n_b >= 0 && n_h >= 1, "dc_score_select_bf16: bad sizes");
    const int n_units = n_b * n_h;
    int rc = dc_select_state_init(n_units, n_rows, budget, workspace, workspace_bytes, stream);
    if (rc) return rc;
    rc = dc_score_prune_bf16(k, q, n_b, n_h, n_rows, hd, sb, sh, sr, q_group, budget, mode, workspace,
                             workspace_bytes, stream);
    if (rc) return rc;
    return dc_sparse_select(idx_out, idx_unit_stride, n_units, n_rows, budget, mode, order, 0, workspace,
                            workspace_bytes, stream);
}

extern "C" int dc_sketch_select_state_init(int n_units, int n_rows, int budget, void *workspace,
                                           size_t workspace_bytes, void *stream) {
    return dc_select_state_init(n_units, n_rows, budget, workspace, workspace_bytes, stream);
}

// Checks, state initialisation and the scan kernel of the sketch route; what follows the scan
// (exact pass, selection) is enqueued by the caller.
int dc_sketch_scan_launch(const char *who, const void *k, const uint8_t *codes, const float *scale,
                          const float *resid, const void *q, int n_b, int n_h, int n_rows, int hd, int64_t sb,
                          int64_t sh, int64_t sr, int64_t cb, int64_t ch, int64_t cr, int q_group, int budget,
                          int mode, int state_ready, void *workspace, size_t workspace_bytes,
                          void *ev_scan_begin, void *ev_scan_end, void *stream, const int32_t *hi_dev, int lo_row) {
    DC_REQUIRE(k && codes && scale && resid && q, "%s: null pointer", who);
    DC_REQUIRE(q_group >= 1, "%s: bad q_group", who);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d not in {64,128,256}", who, hd);
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "%s: bad mode %d", who, mode);
    DC_REQUIRE(dc_aligned16(k) && dc_aligned16(codes) && dc_aligned16(scale) && dc_aligned16(resid),
               "%s: k, codes, scale and resid must be 16-byte aligned", who);
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0 && sr >= hd,
               "%s: key strides must be multiples of 8 elements and row_stride >= hd", who);
    DC_REQUIRE(cb % 16 == 0 && ch % 16 == 0 && cr % 16 == 0 && cr >= hd,
               "%s: code strides must be multiples of 16 bytes and row_stride >= hd", who);
    DC_REQUIRE(n_rows <= kSketchMaxRows, "%s: %d rows per unit; the sketch scan takes at most %d (use the bf16 scan)", who,
               n_rows, kSketchMaxRows);
    FusedPlan p;
    int rc = plan_fused(who, n_b, n_h, n_rows, budget, &p, kBigSteps, kRowsPerBlockStep, kSketchFillBlocks);
    if (rc) return rc;
    if (p.n_units == 0 || p.k_eff == 0) return DC_OK;
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "%s: workspace must be non-null and 256-byte aligned", who);
    const FusedWs w = carve_fused(workspace, p.n_units, n_rows, budget);
    if (workspace_bytes < w.bytes) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, workspace_bytes, w.bytes);
        return DC_ENOMEM;
    }
    hipStream_t st = (hipStream_t)stream;
    if (!state_ready) {
        rc = dc_sketch_select_state_init(p.n_units, n_rows, budget, workspace, workspace_bytes, stream);
        if (rc) return rc;
    }
    if (ev_scan_begin) (void)hipEventRecord((hipEvent_t)ev_scan_begin, st);
#define DC_LAUNCH_SK(HD, SP)                                                                        \
    hipLaunchKernelGGL((sketch_prune_kernel<HD, SP>), dim3((unsigned)p.blocks), dim3(kThreads), 0, st,  \
                       codes, (const uint16_t *)q, scale, resid, w.hist, w.state, w.surv, p.n_units,    \
                       n_h, n_rows, cb, ch, cr, q_group, mode, p.k_eff, p.small_chunks, p.big_steps, hi_dev, lo_row)
    const bool shared_poll = p.n_units <= kSharedPollUnits;
    if (hd == 64 && shared_poll) DC_LAUNCH_SK(64, true);
    else if (hd == 64) DC_LAUNCH_SK(64, false);
    else if (hd == 128 && shared_poll) DC_LAUNCH_SK(128, true);
    else if (hd == 128) DC_LAUNCH_SK(128, false);
    else if (shared_poll) DC_LAUNCH_SK(256, true);
    else DC_LAUNCH_SK(256, false);
#undef DC_LAUNCH_SK
    DC_CHECK_LAUNCH(who);
    if (ev_scan_end) (void)hipEventRecord((hipEvent_t)ev_scan_end, st);
    return DC_OK;
}

extern "C" int dc_score_select_sketch_bf16(const void *k, const uint8_t *codes, const float *scale,
                                           const float *resid, const void *q, uint32_t *idx_out,
                                           int64_t idx_unit_stride, int n_b, int n_h, int n_rows, int hd,
                                           int64_t sb, int64_t sh, int64_t sr, int64_t cb, int64_t ch,
                                           int64_t cr, int q_group, int budget, int mode, int order,
                                           int state_ready, void *workspace, size_t workspace_bytes,
                                           void *ev_scan_begin, void *ev_scan_end, void *stream) {
    return dc_sketch_select_impl(k, codes, scale, resid, q, idx_out, idx_unit_stride, n_b, n_h, n_rows, hd, sb, sh, sr,
                                 cb, ch, cr, q_group, budget, mode, order, state_ready, workspace, workspace_bytes,
                                 ev_scan_begin, ev_scan_end, stream, nullptr, 0);
}

// hi_dev, lo_row: as in dc_score_prune_launch.  Only the scan needs the live length: the passes
// after it work on the lists the scan left, whose capacity is n_rows.
int dc_sketch_select_impl(const void *k, const uint8_t *codes, const float *scale, const float *resid, const void *q,
                          uint32_t *idx_out, int64_t idx_unit_stride, int n_b, int n_h, int n_rows, int hd,
                          int64_t sb, int64_t sh, int64_t sr, int64_t cb, int64_t ch, int64_t cr, int q_group,
                          int budget, int mode, int order, int state_ready, void *workspace, size_t workspace_bytes,
                          void *ev_scan_begin, void *ev_scan_end, void *stream, const int32_t *hi_dev, int lo_row) {
    const char *who = "dc_score_select_sketch_bf16";
    DC_REQUIRE(idx_out, "%s: null pointer", who);
    DC_REQUIRE(order >= DC_ORDER_ANY && order <= DC_ORDER_INDEX, "%s: bad order %d", who, order);
    int rc = dc_sketch_scan_launch(who, k, codes, scale, resid, q, n_b, n_h, n_rows, hd, sb, sh, sr, cb, ch, cr,
                                   q_group, budget, mode, state_ready, workspace, workspace_bytes,
                                   ev_scan_begin, ev_scan_end, stream, hi_dev, lo_row);
    if (rc) return rc;
    FusedPlan p;
    rc = plan_fused(who, n_b, n_h, n_rows, budget, &p);
    if (rc) return rc;
    if (p.n_units == 0 || p.k_eff == 0) return DC_OK;
    DC_REQUIRE(idx_unit_stride >= p.k_eff, "%s: idx_unit_stride < min(budget, n_rows)", who);
    const FusedWs w = carve_fused(workspace, p.n_units, n_rows, budget);
    hipStream_t st = (hipStream_t)stream;
    // Blocks per unit of the exact pass: one per 1024 rows of context, but a grid of at most 2048
    // blocks when the units hold 3 Mi rows or more between them and of 1024 below that (measured
    // at 8 to 128 units: 8 x 131072 rows 7.5 us against 9.1 us with half and 10.4 us with twice the
    // blocks; 64 x 131072 rows 18.9 us at 2048 blocks against 20.8 us at 1024 and 23.9 us at 4096).
    int nblk = (n_rows + 1023) / 1024;
    const int grid = (int64_t)p.n_units * n_rows >= (3ll << 20) ? 2048 : 1024;
    const int cap = p.n_units >= grid ? 1 : grid / p.n_units;
    if (nblk > cap) nblk = cap;
    if (nblk < 1) nblk = 1;
#define DC_LAUNCH_RS(HD)                                                                              \
    hipLaunchKernelGGL(rescore_kernel<HD>, dim3((unsigned)p.n_units * (unsigned)nblk), dim3(kThreads), 0, \
                       st, (const uint16_t *)k, (const uint16_t *)q, w.hist, w.state, w.surv, w.cand_key, \
                       w.cand_idx, p.n_units, n_h, n_rows, sb, sh, sr, q_group, mode, p.k_eff, nblk)
    if (hd == 64) DC_LAUNCH_RS(64);
    else if (hd == 128) DC_LAUNCH_RS(128);
    else DC_LAUNCH_RS(256);
#undef DC_LAUNCH_RS
    DC_CHECK_LAUNCH(who);
    return launch_finish(who, w, idx_out, idx_unit_stride, p.n_units, n_rows, p.k_eff, mode, order, 1, st);
}

extern "C" size_t dc_pq_search_workspace_bytes(int n_units, int n_rows, int n_cand) {
    const FusedWs w = carve_fused(nullptr, n_units, n_rows, n_cand);
    const size_t nu = n_units > 0 ? n_units : 0;
    const size_t kc = (size_t)(n_cand < n_rows ? n_cand : n_rows);
    return w.bytes + dc_align_up(nu * (n_cand > 0 && n_rows > 0 ? kc : 0) * 4, 256);
}

extern "C" int dc_pq_search_bf16(const void *k, const uint8_t *codes, const float *lut, const void *q,
                                 uint32_t *idx_out, int64_t idx_unit_stride, int n_b, int n_h, int n_rows,
                                 int hd, int m, int64_t sb, int64_t sh, int64_t sr, int n_cand, int topk,
                                 int state_ready, void *workspace, size_t workspace_bytes,
                                 void *ev_scan_begin, void *ev_scan_end, void *stream) {
    const char *who = "dc_pq_search_bf16";
    DC_REQUIRE(k && codes && lut && q && idx_out, "%s: null pointer", who);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d not in {64,128,256}", who, hd);
    DC_REQUIRE(m == 16 || m == 32, "%s: m = %d subspaces unsupported (16 or 32)", who, m);
    DC_REQUIRE(n_cand >= 0 && topk >= 0 && topk <= n_cand, "%s: need 0 <= topk <= n_cand", who);
    DC_REQUIRE(dc_aligned16(k) && dc_aligned16(codes) && dc_aligned16(lut),
               "%s: k, codes and lut must be 16-byte aligned", who);
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0 && sr >= hd,
               "%s: key strides must be multiples of 8 elements and row_stride >= hd", who);
    FusedPlan p;
    int rc = plan_fused(who, n_b, n_h, n_rows, n_cand, &p, kPqBigSteps, kPqThreads);
    if (rc) return rc;
    const int k1 = p.k_eff;                   // candidates per unit
    const int k2 = topk < k1 ? topk : k1;     // results per unit
    if (p.n_units == 0 || k2 == 0) return DC_OK;
    DC_REQUIRE(idx_unit_stride >= k2, "%s: idx_unit_stride < min(topk, n_rows)", who);
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "%s: workspace must be non-null and 256-byte aligned", who);
    const FusedWs w = carve_fused(workspace, p.n_units, n_rows, n_cand);
    const size_t need = dc_pq_search_workspace_bytes(p.n_units, n_rows, n_cand);
    if (workspace_bytes < need) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, workspace_bytes, need);
        return DC_ENOMEM;
    }
    uint32_t *cand = (uint32_t *)((char *)workspace + w.bytes);
    hipStream_t st = (hipStream_t)stream;
    if (!state_ready) {
        rc = dc_select_state_init(p.n_units, n_rows, n_cand, workspace, workspace_bytes, stream);
        if (rc) return rc;
    }
    if (ev_scan_begin) (void)hipEventRecord((hipEvent_t)ev_scan_begin, st);
    if (m == 16)
        hipLaunchKernelGGL(pq_prune_kernel<16>, dim3((unsigned)p.blocks), dim3(kPqThreads), 0, st, codes, lut,
                           w.hist, w.state, w.surv, p.n_units, n_rows, k1, p.small_chunks, p.big_steps);
    else
        hipLaunchKernelGGL(pq_prune_kernel<32>, dim3((unsigned)p.blocks), dim3(kPqThreads), 0, st, codes, lut,
                           w.hist, w.state, w.surv, p.n_units, n_rows, k1, p.small_chunks, p.big_steps);
    DC_CHECK_LAUNCH(who);
    if (ev_scan_end) (void)hipEventRecord((hipEvent_t)ev_scan_end, st);
    // the k1 best ADC scores of every unit, in no particular order
    rc = launch_select(who, w, cand, k1, p.n_units, n_rows, k1, DC_MODE_IP, DC_ORDER_ANY, 1, st);
    if (rc) return rc;
    const int lpr = hd / 8, groups = kThreads / lpr;
    const int64_t bpu = ((int64_t)k1 + groups - 1) / groups;
    DC_REQUIRE((int64_t)p.n_units * bpu < (1ll << 31), "%s: grid too large", who);
#define DC_LAUNCH_PR(HD)                                                                              \
    hipLaunchKernelGGL(pq_rescore_kernel<HD>, dim3((unsigned)(p.n_units * bpu)), dim3(kThreads), 0, st, \
                       (const uint16_t *)k, (const uint16_t *)q, cand, w.state, w.cand_key, w.cand_idx, \
                       n_h, k1, (int64_t)k1, n_rows, sb, sh, sr, (int)bpu)
    if (hd == 64) DC_LAUNCH_PR(64);
    else if (hd == 128) DC_LAUNCH_PR(128);
    else DC_LAUNCH_PR(256);
#undef DC_LAUNCH_PR
    DC_CHECK_LAUNCH(who);
    return launch_finish(who, w, idx_out, idx_unit_stride, p.n_units, n_rows, k2, DC_MODE_IP, DC_ORDER_BEST, 1,
                         st);
}
