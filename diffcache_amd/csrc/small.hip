// A whole decode layer in ONE kernel, for short contexts.
//
// With a few hundred thousand key rows in all, the four-to-six kernel chain of the long-context
// routes is bound by memory latency between its phases, not by bytes: benchmark configuration 2
// (8 units x 32700 rows) moves 72 MB -- 9 us of HBM time -- in about 50 us.  Here every block of
// the grid is resident at once (the grid is sized to what the chip holds), so the phases of a
// unit hand over through memory instead of a kernel boundary:
//
//   1  every block scores its slice of the unit's rows against the GQA-mean query (the
//      arithmetic of dc_score_bf16, nsw.rs:129-139), keeps the scores in LDS and adds its
//      histogram of ordering-key buckets to the unit's          -- barrier (arrival counter) --
//   2  every block derives the threshold bucket from the complete histogram, emits the ids of
//      its rows in better buckets and writes its rows of the threshold bucket into slots of
//      the unit's candidate list.  No slot is reserved through a counter: what the block's
//      addition to a bucket of the histogram returned is its place among the unit's rows of
//      that bucket.  The histogram also says how many candidates there are, and an unwritten
//      slot reads "empty", so the list itself tells a reader when it is complete
//   3  every block ranks its own candidates among all of the unit's: those among the
//      k - (rows in better buckets) smallest (key, id) pairs are in (ties to the lower id: the
//      kept set of search_bruteforce, nsw.rs:592-630).  (Candidates by the thousand -- equal
//      keys -- take two more barriers and a radix select by one block instead.)
//   4  every block attends to its own selected rows and to its share of the sinks, the recent
//      window and the current token (base.py:134-142) and leaves a softmax partial; the last
//      block of the unit to finish merges the partials, writes the output and puts the
//      shared state (histogram, counters, candidate slots) back to its initial values.
//
// A block that waits, waits for blocks that are resident too, so the wait ends; it is bounded
// all the same, and a wait that runs out cannot go unnoticed: the block sets the unit's error word
// (which stays set until the host initialises the state again), tells the host through a word of
// pinned host memory, and writes NaN over the unit's output rows and 0xffffffff over its ids; every
// block of a later launch that finds the error word set does the same.  The host side keeps two
// such launches from overlapping (they would starve each other of CUs): see dc_small_try.
// Data that crosses blocks goes through agent-scope loads, stores and atomics: the L2 caches
// of the eight XCDs are not coherent inside a kernel.  One such hand-over costs
// about 1.5 to 2 us, and a layer is a chain of about ten of them after the 10 us of scoring.
#include "dc_attn.h"
#include "dc_fused.h"
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <unordered_map>

namespace {

constexpr int kSmallRows = 4096;     // rows a block scores at most (their scores stay in LDS)
constexpr int kSmallCand = 4096;     // candidates of a unit that are ranked in LDS
constexpr int kSmallBlocks = 512;    // blocks of a launch at most: two per CU
constexpr int64_t kSmallTotalRows = 640 * 1024;  // rows of all units that the route takes on (measured crossover)
// ... and rows per unit when the caller brings a sketch (measured: 8 units, 43.3 us against 41.6 us
// for the sketch chain at 49152 rows, 37.3 against 40.6 at 32768; 16 units: 53.4 against 50.8 at 40960)
constexpr int kSmallSketchRows = 40 * 1024;
constexpr int kSmallMl = 2048;       // floats of (m, l) the merge keeps in LDS: blocks per unit * G * 2

struct SmallArgs {
    const uint16_t *Q, *K, *V;  // K, V: row 0 of unit (0, 0)
    const uint16_t *new_k, *new_v;
    uint32_t *hist;
    UnitState *state;
    unsigned long long *cand;  // per unit n_rows packed (key << 32 | id) entries, kEmpty between launches
    uint32_t *idx_out;
    int64_t idx_stride;
    float *ws_acc, *ws_ml;
    uint16_t *out;
    float *lse;
    const int32_t *n_recent_dev;
    int n_units, n_h, n_rows, rows_per_block, bpu, k_eff, mode;
    int n_sink;
    int64_t recent_lo;
    int n_recent;
    int64_t sb, sh, sr;  // K and V share their strides
    float scale;
    int spin_limit;
    uint32_t *mailbox;    // one word of pinned host memory (device address), or null: receives launch_seq when a wait runs out
    uint32_t launch_seq;  // never zero
};

__device__ __forceinline__ void stores_done() {
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt, expcnt and lgkmcnt at zero: stores and atomics are acknowledged
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

constexpr unsigned long long kEmpty = ~0ull;  // a slot of the candidate list that nobody has written (no row has id 2^32 - 1)

__device__ __forceinline__ unsigned long long ld_agent_u64(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent_u64(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A bounded wait ran out.  The unit's error word is sticky (only the host's initialisation clears
// it), the block remembers that its results are void, and the host is told through pinned memory
// (a system-scope store: this path is never taken in a healthy run).
constexpr uint32_t kSyncErrBit = 0x80000000u;  // of sync_cnt: a wait of this launch ran out
__device__ __forceinline__ void give_up(UnitState *st, uint32_t *s_bad, uint32_t *mailbox, uint32_t seq) {
    dc_st_agent(&st->sync_err, 1u);
    // also in the arrival counter, where the block that merges finds it in what its own arrival
    // returns, at no extra memory round trip
    atomicOr(&st->sync_cnt, kSyncErrBit);
    __hip_atomic_store(s_bad, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (mailbox) __hip_atomic_store(mailbox, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Every block of the unit has arrived `target` times in all.  Called by all threads.
__device__ __forceinline__ void unit_barrier(UnitState *st, uint32_t target, const SmallArgs &a, uint32_t *s_bad) {
    stores_done();
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(&st->sync_cnt, 1u);
        int spins = 0;
        while ((dc_ld_agent(&st->sync_cnt) & ~kSyncErrBit) < target && spins < a.spin_limit) {
            __builtin_amdgcn_s_sleep(1);
            ++spins;
        }
        if (spins >= a.spin_limit) give_up(st, s_bad, a.mailbox, a.launch_seq);
    }
    __syncthreads();
}

// 16-byte agent-scope load: a raw buffer load with the sc1 cache policy, which is what an
// agent-scope atomic load compiles to, four words at a time.
__device__ __forceinline__ float4 ld_agent_f4(const float *base, uint32_t byte_offset) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, 0x7fffffff, 0x00020000);
    const f32x4 v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 16));
    return make_float4(v.x, v.y, v.z, v.w);
}

// A lane group's running softmax over the rows it has seen: every lane of the group knows the
// logits of the group's rows and accumulates its 8 output columns.  absorb() takes RR rows:
// x[t][g] logits (-inf for a missing row), vw[t] the 16 bytes of the V row this lane owns.
template <int G>
struct GroupSoftmax {
    float m[G], l[G], acc[G][8];
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            m[g] = -INFINITY;
            l[g] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
        }
    }
    template <int RR>
    __device__ __forceinline__ void absorb(const float (&x)[RR][G], const uint4 (&vw)[RR]) {
        float m_new[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float mx = m[g];
#pragma unroll
            for (int t = 0; t < RR; ++t) mx = fmaxf(mx, x[t][g]);
            m_new[g] = mx;
            const float resc = (m[g] > -INFINITY) ? __expf(m[g] - mx) : 0.f;
            l[g] *= resc;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] *= resc;
            m[g] = mx;
        }
#pragma unroll
        for (int t = 0; t < RR; ++t) {
            const float v[8] = {dc_bf16_lo(vw[t].x), dc_bf16_hi(vw[t].x), dc_bf16_lo(vw[t].y),
                                dc_bf16_hi(vw[t].y), dc_bf16_lo(vw[t].z), dc_bf16_hi(vw[t].z),
                                dc_bf16_lo(vw[t].w), dc_bf16_hi(vw[t].w)};
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float pw = (x[t][g] > -INFINITY) ? __expf(x[t][g] - m_new[g]) : 0.f;
                l[g] += pw;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(pw, v[i], acc[g][i]);
            }
        }
    }
};

template <int HD, int G>
constexpr int small_lds_bytes() {
    // [scores of the block's rows, later the unit's candidates as packed (key, id)] [own selected ids]
    constexpr int a = kSmallCand * 8 > kSmallRows * 4 ? kSmallCand * 8 : kSmallRows * 4;
    constexpr int red = (kAttnWaves * G * 2 + kAttnWaves * G * HD) * 4;  // block reduction, aliases the first part
    constexpr int first = a > red ? a : red;
    return first + kSmallRows * 4;
}

template <int HD, int G>
__global__ __launch_bounds__(kThreads) void small_layer_kernel(SmallArgs a) {
    constexpr int LPR = HD / 8;
    constexpr int CH = LPR < 16 ? LPR : 16;
    constexpr int NG = kThreads / LPR;  // row groups per block in the attention phase
    constexpr int R = rows_per_group(G);
    __shared__ __align__(16) unsigned char smem[small_lds_bytes<HD, G>()];
    __shared__ uint32_t lhist[DC_HIST_BINS];
    __shared__ uint32_t lbase[DC_HIST_BINS];  // what this block's additions to the unit's histogram returned
    __shared__ uint32_t lpre[DC_HIST_BINS];   // exclusive prefix of the unit's histogram
    __shared__ uint32_t wtot[kThreads / 64 + 1];
    __shared__ uint32_t sres[3];
    __shared__ uint32_t s_cnt[4];   // [2]: this block's selected rows so far
    __shared__ uint32_t s_base[2];  // scratch of the radix select
    __shared__ uint32_t s_flag;
    __shared__ uint32_t s_bad;  // this block's results are void: a wait ran out, here or in an earlier launch
    float *s_scores = reinterpret_cast<float *>(smem);
    unsigned long long *s_cand = reinterpret_cast<unsigned long long *>(smem);
    constexpr int kFirst = small_lds_bytes<HD, G>() - kSmallRows * 4;
    uint32_t *own_win = reinterpret_cast<uint32_t *>(smem + kFirst);

    const int unit = blockIdx.x % a.n_units;
    const int blk = blockIdx.x / a.n_units;
    const int b = unit / a.n_h, h = unit % a.n_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    UnitState *st = a.state + unit;
    uint32_t *hu = a.hist + (int64_t)unit * DC_HIST_BINS;
    const uint16_t *Kb = a.K + b * a.sb + h * a.sh;
    const uint16_t *Vb = a.V + b * a.sb + h * a.sh;
    const int64_t r0 = (int64_t)blk * a.rows_per_block;
    const int64_t r1 = r0 + a.rows_per_block < a.n_rows ? r0 + a.rows_per_block : a.n_rows;
    const int n_own = r1 > r0 ? (int)(r1 - r0) : 0;
    const uint32_t bpu = (uint32_t)a.bpu;
    uint32_t *io = a.idx_out + (int64_t)unit * a.idx_stride;
    // A unit in which a wait ran out has no valid result: NaN over its output rows and 0xffffffff
    // over its ids, so that the step cannot pass for a good one downstream.
    auto poison = [&]() {
        for (int o = tid; o < G * HD; o += kThreads) a.out[(int64_t)unit * G * HD + o] = 0x7fc0;
        if (a.lse && tid < G) a.lse[unit * G + tid] = __uint_as_float(0x7fc00000u);
        for (int i = tid; i < a.k_eff; i += kThreads) io[i] = 0xffffffffu;
    };
    // ---------------- 1: scores of this block's rows ----------------
    for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;
    if (tid < 4) s_cnt[tid] = 0;
    // The unit's error word, set by an earlier launch and not cleared since: the shared state
    // cannot be trusted until the host has initialised it again.  (The load returns while the
    // rows are scored; it is looked at before the block first touches the shared state.)
    // A plain load: the word was written by an earlier kernel.
    uint32_t err0 = 0u;
    if (tid == 0) err0 = st->sync_err;
    __syncthreads();
    {
        const int grp = lane / LPR, col = lane % LPR;
        float q[8];
        dc_load_query<HD>(a.Q, unit, G, col, q);
        const uint16_t *Ku = Kb + (int64_t)a.n_sink * a.sr + col * 8;  // the region starts after the sinks
        const int64_t last = r1 - 1;
        for (int64_t row0 = r0 + wave * 64; row0 < r1; row0 += kRowsPerBlockStep) {
            float mine = 0.f;
#pragma unroll
            for (int c0 = 0; c0 < LPR; c0 += CH) {
                uint4 w[CH];
#pragma unroll
                for (int j = 0; j < CH; ++j) {
                    int64_t r = row0 + grp * LPR + c0 + j;
                    r = r > last ? last : r;
                    w[j] = *reinterpret_cast<const uint4 *>(Ku + r * a.sr);
                }
#pragma unroll
                for (int j = 0; j < CH; ++j) {
                    const float p = dc_group_sum<LPR>(dc_dot8(w[j], q, 0.f));
                    mine = (col == c0 + j) ? p : mine;
                }
            }
            const int64_t myrow = row0 + lane;
            if (myrow < r1) {
                s_scores[myrow - r0] = mine;
                uint32_t key, bucket;
                dc_key_bucket(mine, a.mode, key, bucket);
                atomicAdd(&lhist[bucket], 1u);
            }
        }
    }
    if (tid == 0) s_bad = err0;
    __syncthreads();
    if (s_bad != 0u) {  // every block of the unit sees the same word: none of them goes on
        poison();
        return;
    }
    // What an addition returns -- the rows of that bucket counted before this block's -- is the
    // block's place among the unit's rows of the bucket: every selected id and every candidate
    // gets its slot from the histogram, and no other counter is needed.
    // (All of a thread's additions are issued before the first result is looked at: written as one
    // loop over the bins the compiler waits for each addition before it issues the next, a memory
    // round trip per bin and thread on the unit's critical path.)
    {
        constexpr int kPer = DC_HIST_BINS / kThreads;
        static_assert(kPer * kThreads == DC_HIST_BINS, "bins per thread");
        uint32_t before[kPer];
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
            const int i = tid + u * kThreads;
            const uint32_t c = lhist[i];
            before[u] = 0u;
            if (c) before[u] = atomicAdd(&hu[i], c);
        }
#pragma unroll
        for (int u = 0; u < kPer; ++u) lbase[tid + u * kThreads] = before[u];
    }

    // ---------------- 2: threshold bucket; ids of better buckets, candidates of the threshold bucket ----------------
    unit_barrier(st, bpu, a, &s_bad);  // the unit's histogram is complete
    uint32_t tb, c_less, n_cand;
    {
        uint32_t bins[kBinsPerThread];
        uint32_t sum = 0, total;
#pragma unroll
        for (int i = 0; i < kBinsPerThread; ++i) {
            bins[i] = dc_ld_agent(hu + tid * kBinsPerThread + i);
            sum += bins[i];
        }
        const uint32_t excl = block_excl_scan<kThreads>(sum, wtot, &total);
        if (tid == 0) {
            sres[0] = DC_HIST_BINS;
            sres[1] = 0;
            sres[2] = 0;
        }
        __syncthreads();
        const uint32_t kk = (uint32_t)a.k_eff;
        uint32_t run = excl;
        bool done = !(excl < kk && kk <= excl + sum);
#pragma unroll
        for (int i = 0; i < kBinsPerThread; ++i) {
            lpre[tid * kBinsPerThread + i] = run;  // rows of the unit in better buckets
            if (!done && run + bins[i] >= kk) {
                sres[0] = tid * kBinsPerThread + i;
                sres[1] = run;
                sres[2] = bins[i];
                done = true;
            }
            run += bins[i];
        }
        __syncthreads();
        tb = sres[0];
        c_less = sres[1];
        n_cand = sres[2];  // rows of the threshold bucket in the whole unit
    }
    const uint32_t n_oc = tb < (uint32_t)DC_HIST_BINS ? lhist[tb] : 0u;    // this block's rows of that bucket
    const uint32_t base_c = tb < (uint32_t)DC_HIST_BINS ? lbase[tb] : 0u;  // and their first slot in the list
    __syncthreads();
    for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;  // from here on: rows of a bucket placed so far
    __syncthreads();
    unsigned long long *cl = a.cand + (int64_t)unit * a.n_rows;
    for (int i = tid; i < n_own; i += kThreads) {
        uint32_t key, bucket;
        dc_key_bucket(s_scores[i], a.mode, key, bucket);
        const uint32_t id = (uint32_t)(r0 + i);
        if (bucket < tb) {
            own_win[atomicAdd(&s_cnt[2], 1u)] = id;
            const uint32_t slot = lpre[bucket] + lbase[bucket] + atomicAdd(&lhist[bucket], 1u);
            if (slot < (uint32_t)a.k_eff) io[slot] = id;
        } else if (bucket == tb) {
            const uint32_t slot = base_c + atomicAdd(&lhist[bucket], 1u);
            if (slot < n_cand) st_agent_u64(cl + slot, ((unsigned long long)key << 32) | id);
        }
    }

    // ---------------- 3: which of this block's candidates are in ----------------
    // (the scores in LDS are dead from here on)
    const uint32_t need = (uint32_t)a.k_eff - c_less;  // 1 .. n_cand candidates are in
    uint32_t arrivals = 1u;  // barriers passed so far
    if (n_cand < (uint32_t)kSmallCand) {
        // The unit's candidates as packed (key, id) into LDS.  A slot that still reads kEmpty has
        // not been written yet: read it again (the list itself says when it is complete).
        __syncthreads();
        for (uint32_t i0 = tid; i0 < n_cand; i0 += 8 * kThreads) {
            unsigned long long v8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t i = i0 + (uint32_t)j * kThreads;
                v8[j] = i < n_cand ? ld_agent_u64(cl + i) : 0ull;
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t i = i0 + (uint32_t)j * kThreads;
                int spins = 0;
                while (v8[j] == kEmpty && spins < a.spin_limit) {
                    __builtin_amdgcn_s_sleep(1);
                    v8[j] = ld_agent_u64(cl + i);
                    ++spins;
                }
                if (v8[j] == kEmpty) give_up(st, &s_bad, a.mailbox, a.launch_seq);
                if (i < n_cand) s_cand[i] = v8[j];
            }
        }
        if (tid == 0 && (n_cand & 1u)) s_cand[n_cand] = ~0ull;  // pad to whole 16-byte reads
        __syncthreads();
        const ulonglong2 *s_cand2 = reinterpret_cast<const ulonglong2 *>(s_cand);
        const uint32_t n_pair = (n_cand + 1u) / 2u;
        // T lanes share one candidate, each counting over a T-th of the list
        uint32_t T = 1;
        while (T < 64u && n_oc * (T * 2u) <= (uint32_t)kThreads) T *= 2u;
        const uint32_t per_pass = (uint32_t)kThreads / T, sub = (uint32_t)tid % T;
        for (uint32_t e0 = 0; e0 < n_oc; e0 += per_pass) {
            const uint32_t e = e0 + (uint32_t)tid / T;
            const uint32_t slot = base_c + e;
            // (a slot that still reads empty after a wait that ran out is nobody's candidate)
            const unsigned long long mine = (e < n_oc && slot < n_cand) ? s_cand[slot] : kEmpty;
            const bool active = mine != kEmpty && (uint32_t)mine < (uint32_t)a.n_rows;
            uint32_t rank = 0;
#pragma unroll 4
            for (uint32_t j = sub; j < n_pair; j += T) {
                const ulonglong2 t = s_cand2[j];
                rank += (t.x < mine ? 1u : 0u) + (t.y < mine ? 1u : 0u);
            }
            for (uint32_t off = 1; off < T; off <<= 1) rank += __shfl_xor(rank, (int)off, 64);
            if (active && sub == 0 && rank < need) {  // ranks are distinct: the rank is the slot
                const uint32_t id = (uint32_t)mine;
                own_win[atomicAdd(&s_cnt[2], 1u)] = id;
                io[c_less + rank] = id;
            }
        }
    } else {
        // Too many candidates to rank in LDS (equal keys by the thousand): once every block has
        // written its candidates, block 0 of the unit finds the cutoff, the need-th smallest
        // (key, id) pair, with a radix select over the list.
        unit_barrier(st, 2u * bpu, a, &s_bad);
        if (blk == 0) {
            uint32_t *lh = reinterpret_cast<uint32_t *>(smem);  // kRadixBins words
            uint32_t prefix = 0u, rem = need, eq = n_cand;
            auto radix_pass = [&](auto get, uint32_t &pfx, uint32_t &rm, uint32_t &e_q, int &top) {
                constexpr int kBins = kRadixBins / kThreads;
                const int width = top < kRadixBits ? top : kRadixBits;
                const int shift = top - width;
                for (int i = tid; i < kRadixBins; i += kThreads) lh[i] = 0;
                __syncthreads();
                const uint32_t himask = (top >= 32) ? 0u : (0xffffffffu << top);
                for (uint32_t i = tid; i < n_cand; i += kThreads) {
                    uint32_t v;
                    const unsigned long long c = ld_agent_u64(cl + i);
                    if (get((uint32_t)(c >> 32), (uint32_t)c, &v) && ((v & himask) == (pfx & himask)))
                        atomicAdd(&lh[(v >> shift) & ((1u << width) - 1u)], 1u);
                }
                __syncthreads();
                uint32_t hh[kBins];
                uint32_t sum = 0;
#pragma unroll
                for (int j = 0; j < kBins; ++j) {
                    hh[j] = lh[kBins * tid + j];
                    sum += hh[j];
                }
                uint32_t total;
                const uint32_t excl = block_excl_scan<kThreads>(sum, wtot, &total);
                if (excl < rm && rm <= excl + sum) {
                    uint32_t run = excl;
                    bool done = false;
#pragma unroll
                    for (int j = 0; j < kBins; ++j) {
                        if (!done && run + hh[j] >= rm) {
                            s_base[0] = kBins * tid + j;
                            s_base[1] = run;
                            sres[0] = hh[j];
                            done = true;
                        }
                        run += hh[j];
                    }
                }
                __syncthreads();
                pfx |= s_base[0] << shift;
                rm -= s_base[1];
                e_q = sres[0];
                top = shift;
                __syncthreads();
            };
            int top = 32;
            auto get_key = [](uint32_t key, uint32_t, uint32_t *v) {
                *v = key;
                return true;
            };
            while (top > 0) radix_pass(get_key, prefix, rem, eq, top);
            const uint32_t t_key = prefix;
            uint32_t t_idx = 0xffffffffu;
            if (rem < eq) {  // only the lowest ids of the tie group fit
                const uint32_t span = (uint32_t)(a.n_rows - 1) | 1u;
                int top2 = 32 - __clz(span);
                auto get_idx = [t_key](uint32_t key, uint32_t id, uint32_t *v) {
                    *v = id;
                    return key == t_key;
                };
                uint32_t p2 = 0u, r2 = rem, e2 = eq;
                while (top2 > 0) radix_pass(get_idx, p2, r2, e2, top2);
                t_idx = p2;
            }
            if (tid == 0) {
                dc_st_agent(&st->cut_key, t_key);
                dc_st_agent(&st->cut_id, t_idx);
            }
        }
        unit_barrier(st, 3u * bpu, a, &s_bad);
        arrivals = 3u;
        const uint32_t cut_key = dc_ld_agent(&st->cut_key), cut_id = dc_ld_agent(&st->cut_id);
        for (uint32_t e = tid; e < n_oc; e += kThreads) {
            const uint32_t slot = base_c + e;
            if (slot >= n_cand) continue;
            const unsigned long long c = ld_agent_u64(cl + slot);
            const uint32_t key = (uint32_t)(c >> 32), id = (uint32_t)c;
            if (id < (uint32_t)a.n_rows && (key < cut_key || (key == cut_key && id <= cut_id))) {
                own_win[atomicAdd(&s_cnt[2], 1u)] = id;
                const uint32_t gs = c_less + atomicAdd(&st->win_cnt, 1u);
                if (gs < (uint32_t)a.k_eff) io[gs] = id;
            }
        }
    }
    __syncthreads();
    const uint32_t n_ow = s_cnt[2];  // this block's selected rows (ids relative to the region)

    // ---------------- 4: attention over this block's selected rows ----------------
    const int gid = tid / LPR, col = tid % LPR;
    GroupSoftmax<G> sm;
    sm.init();
    uint4 qh[G];  // the G heads as packed bf16, unpacked inside the dot product
#pragma unroll
    for (int g = 0; g < G; ++g)
        qh[g] = *reinterpret_cast<const uint4 *>(a.Q + ((int64_t)unit * G + g) * HD + col * 8);
    auto dot_q = [&](const uint4 &w, int g) {
        // the products and the order of additions of dc_dot8 over the unpacked head
        float acc = 0.f;
        acc = fmaf(dc_bf16_lo(w.x), dc_bf16_lo(qh[g].x), acc);
        acc = fmaf(dc_bf16_hi(w.x), dc_bf16_hi(qh[g].x), acc);
        acc = fmaf(dc_bf16_lo(w.y), dc_bf16_lo(qh[g].y), acc);
        acc = fmaf(dc_bf16_hi(w.y), dc_bf16_hi(qh[g].y), acc);
        acc = fmaf(dc_bf16_lo(w.z), dc_bf16_lo(qh[g].z), acc);
        acc = fmaf(dc_bf16_hi(w.z), dc_bf16_hi(qh[g].z), acc);
        acc = fmaf(dc_bf16_lo(w.w), dc_bf16_lo(qh[g].w), acc);
        acc = fmaf(dc_bf16_hi(w.w), dc_bf16_hi(qh[g].w), acc);
        return dc_group_sum<LPR>(acc) * a.scale;
    };
    const uint16_t *Ku = Kb + col * 8, *Vu = Vb + col * 8;
    // The always-kept rows (sinks, recent window, current token: base.py:134-142) are dealt out
    // over the unit's blocks and follow the block's selected rows in one list of items.
    int n_recent = a.n_recent;
    if (a.n_recent_dev) {  // the window's length may live on the device (cache_seqlens, base.py:134-142)
        const int c = *a.n_recent_dev;
        n_recent = c < 0 ? 0 : (c < n_recent ? c : n_recent);
    }
    const int n_fix = a.n_sink + n_recent + (a.new_k ? 1 : 0);
    const uint32_t n_myfix = n_fix > blk ? (uint32_t)((n_fix - blk + a.bpu - 1) / a.bpu) : 0u;
    const uint32_t n_items = n_ow + n_myfix;
    for (uint32_t w0 = 0; w0 < n_items; w0 += NG * R) {
        float x[R][G];
        uint4 kw[R], vw[R];
        bool ok[R];
#pragma unroll
        for (int t = 0; t < R; ++t) {
            const uint32_t w = w0 + (uint32_t)(t * NG + gid);
            ok[t] = w < n_items;
            const uint16_t *pk = Ku, *pv = Vu;
            if (w < n_ow) {
                const int64_t off = ((int64_t)a.n_sink + own_win[w]) * a.sr;
                pk = Ku + off, pv = Vu + off;
            } else if (ok[t]) {
                const int f = blk + (int)(w - n_ow) * a.bpu;
                if (f < a.n_sink + n_recent) {
                    const int64_t off = (f < a.n_sink ? (int64_t)f : a.recent_lo + (f - a.n_sink)) * a.sr;
                    pk = Ku + off, pv = Vu + off;
                } else {
                    pk = a.new_k + (int64_t)unit * HD + col * 8;
                    pv = a.new_v + (int64_t)unit * HD + col * 8;
                }
            }
            kw[t] = *reinterpret_cast<const uint4 *>(pk);
            vw[t] = *reinterpret_cast<const uint4 *>(pv);
        }
#pragma unroll
        for (int t = 0; t < R; ++t)
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float v = dot_q(kw[t], g);
                x[t][g] = ok[t] ? v : -INFINITY;
            }
        sm.template absorb<R>(x, vw);
    }

    // the block's partial: combine its lane groups (the candidate list in LDS is dead)
    __syncthreads();
    float *s_red = reinterpret_cast<float *>(smem);  // [kAttnWaves][G]
    float *s_l = s_red + kAttnWaves * G;             // [kAttnWaves][G]
    float *s_acc = s_l + kAttnWaves * G;             // [kAttnWaves][G * HD]
    float m_blk[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = sm.m[g];
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
        if (lane == 0) s_red[wave * G + g] = v;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = s_red[g];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) v = fmaxf(v, s_red[w2 * G + g]);
        m_blk[g] = v;
        const float sc = (sm.m[g] > -INFINITY) ? __expf(sm.m[g] - v) : 0.f;
        sm.l[g] *= sc;
#pragma unroll
        for (int i = 0; i < 8; ++i) sm.acc[g][i] *= sc;
    }
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            sm.l[g] += __shfl_xor(sm.l[g], off, 64);
#pragma unroll
            for (int i = 0; i < 8; ++i) sm.acc[g][i] += __shfl_xor(sm.acc[g][i], off, 64);
        }
    if (lane < LPR) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (col == 0) s_l[wave * G + g] = sm.l[g];
#pragma unroll
            for (int i = 0; i < 8; ++i) s_acc[wave * (G * HD) + g * HD + col * 8 + i] = sm.acc[g][i];
        }
    }
    __syncthreads();
    const int n_splits = a.bpu;
    const int64_t slot = (int64_t)unit * n_splits + blk;
    for (int o = tid; o < G * HD; o += kThreads) {
        float s = s_acc[o];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) s += s_acc[w2 * (G * HD) + o];
        dc_st_agent(a.ws_acc + slot * (G * HD) + o, s);
    }
    if (tid < G) {
        float l = s_l[tid];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) l += s_l[w2 * G + tid];
        dc_st_agent(a.ws_ml + (slot * G + tid) * 2 + 0, m_blk[tid]);
        dc_st_agent(a.ws_ml + (slot * G + tid) * 2 + 1, l);
    }
    stores_done();
    __syncthreads();
    if (tid == 0) s_flag = atomicAdd(&st->sync_cnt, 1u);
    __syncthreads();
    // A wait that ran out in this launch: the outputs are marked by every block whose own wait ran
    // out and by the merging block, which finds the error bit of any block that arrived before it
    // in the counter (a block sets the bit before its next arrival, and counts that do not add up
    // -- the only way a block could be taken for the last one too early -- come from a wait that
    // ran out earlier).
    const bool bad_self = s_bad != 0u;
    if ((s_flag & ~kSyncErrBit) != (arrivals + 1u) * bpu - 1u) {
        if (bad_self) poison();
        return;
    }

    // ---------------- merge of the unit's partials (the last block to arrive) ----------------
    // Every block of the unit is done with the shared state: leave it ready for the next call
    // (stores that nothing here waits for; the end of the kernel does).
    for (int i = tid; i < DC_HIST_BINS; i += kThreads) dc_st_agent(hu + i, 0u);
    for (uint32_t i = tid; i < n_cand; i += kThreads) st_agent_u64(cl + i, kEmpty);
    if (tid == 0) {
        dc_st_agent(&st->win_cnt, 0u);
        dc_st_agent(&st->sync_cnt, 0u);
    }
    if (bad_self || (s_flag & kSyncErrBit) != 0u) {
        poison();
        return;
    }
    // Four adjacent output columns per thread, the partials read 16 bytes at a time and a batch
    // of them in flight at once.  With fewer column quads than threads the partials are dealt
    // out over kParts thread groups, whose sums (all relative to the same maximum M) are added
    // through LDS.  (The sum over the partials runs in a different order than in the attention
    // kernels' merge: same result within float rounding.)
    constexpr int NC = G * HD / 4;
    constexpr int kParts = NC >= kThreads ? 1 : kThreads / NC;
    constexpr int kBatch = 32;
    float *ml = reinterpret_cast<float *>(smem);
    float *s_part = ml + kSmallMl;  // [kParts - 1][NC][4]: the sums of the other thread groups
    float *s_ML = s_part + kThreads * 4;  // [2][G]: M and L of every head
    const float *gml = a.ws_ml + (int64_t)unit * n_splits * G * 2;
    const float *pa = a.ws_acc + (int64_t)unit * n_splits * (G * HD);
    for (int c0 = 0; c0 < NC; c0 += kThreads) {
        const int o4 = c0 + tid % (kParts > 1 ? NC : kThreads), part = kParts > 1 ? tid / NC : 0;
        const bool live = o4 < NC && part < kParts;
        const int o = o4 * 4, g = live ? o / HD : 0;
        float4 v[kBatch];
        auto issue = [&](int s0) {
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int sp = s0 + j * kParts;
                v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (live && sp < n_splits) v[j] = ld_agent_f4(pa, (uint32_t)((sp * (G * HD) + o) * 4));
            }
        };
        issue(part);  // in flight while the weights of the partials are worked out
        if (c0 == 0) {
            // (m, l) of every partial -> its weight exp(m - M) and weight * l, with M and L per head
            // found by one wave each (fixed reduction trees: the result does not depend on timing)
            const int n_pairs = n_splits * G;
            for (int i = tid; i < 2 * n_pairs; i += kThreads) ml[i] = dc_ld_agent(gml + i);
            __syncthreads();
            for (int g = wave; g < G; g += kThreads / 64) {
                float mx = -INFINITY;
                for (int sp = lane; sp < n_splits; sp += 64) {
                    const float m = ml[(sp * G + g) * 2], l = ml[(sp * G + g) * 2 + 1];
                    if (l > 0.f) mx = fmaxf(mx, m);
                }
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
                if (lane == 0) s_ML[g] = mx;
            }
            __syncthreads();
            for (int i = tid; i < n_pairs; i += kThreads) {
                const float m = ml[2 * i], l = ml[2 * i + 1];
                const float w = (l > 0.f) ? __expf(m - s_ML[i % G]) : 0.f;
                ml[2 * i] = w;
                ml[2 * i + 1] = w * l;
            }
            __syncthreads();
            for (int g = wave; g < G; g += kThreads / 64) {
                float sum = 0.f;
                for (int sp = lane; sp < n_splits; sp += 64) sum += ml[(sp * G + g) * 2 + 1];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
                if (lane == 0) s_ML[G + g] = sum;
            }
            __syncthreads();
        }
        const float M = s_ML[g], L = s_ML[G + g];
        float4 acc_o = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s0 = part; s0 < n_splits; s0 += kParts * kBatch) {
            if (s0 != part) issue(s0);
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int sp = s0 + j * kParts;
                if (live && sp < n_splits) {
                    const float w = ml[(sp * G + g) * 2];
                    acc_o.x = fmaf(w, v[j].x, acc_o.x);
                    acc_o.y = fmaf(w, v[j].y, acc_o.y);
                    acc_o.z = fmaf(w, v[j].z, acc_o.z);
                    acc_o.w = fmaf(w, v[j].w, acc_o.w);
                }
            }
        }
        if (kParts > 1) {
            if (live && part > 0) {
                float *d = s_part + ((part - 1) * NC + o4) * 4;
                d[0] = acc_o.x, d[1] = acc_o.y, d[2] = acc_o.z, d[3] = acc_o.w;
            }
            __syncthreads();
            if (live && part == 0) {
                for (int pp = 1; pp < kParts; ++pp) {  // in a fixed order: the result does not depend on timing
                    const float *d = s_part + ((pp - 1) * NC + o4) * 4;
                    acc_o.x += d[0], acc_o.y += d[1], acc_o.z += d[2], acc_o.w += d[3];
                }
            }
        }
        if (live && part == 0) {
            uint16_t *po = a.out + (int64_t)unit * G * HD + o;
            po[0] = dc_f32_to_bf16(L > 0.f ? acc_o.x / L : 0.f);
            po[1] = dc_f32_to_bf16(L > 0.f ? acc_o.y / L : 0.f);
            po[2] = dc_f32_to_bf16(L > 0.f ? acc_o.z / L : 0.f);
            po[3] = dc_f32_to_bf16(L > 0.f ? acc_o.w / L : 0.f);
            if (a.lse && (o % HD) == 0) a.lse[unit * G + g] = L > 0.f ? M + logf(L) : -INFINITY;
        }
    }
}

struct SmallPlan {
    int bpu, rows_per_block;
    bool ok;
};

SmallPlan plan_small(int n_units, int region) {
    SmallPlan p;
    p.ok = false;
    p.bpu = p.rows_per_block = 0;
    if (n_units < 1 || n_units > kSmallBlocks || region < 1) return p;
    int bpu = kSmallBlocks / n_units;
    const int steps = (region + kRowsPerBlockStep - 1) / kRowsPerBlockStep;
    if (bpu > steps) bpu = steps;
    int rpb = (region + bpu - 1) / bpu;
    rpb = (rpb + kRowsPerBlockStep - 1) / kRowsPerBlockStep * kRowsPerBlockStep;
    p.bpu = (region + rpb - 1) / rpb;
    p.rows_per_block = rpb;
    // beyond this many rows in all, the routes that scan the 8-bit sketch are faster (half the bytes)
    p.ok = rpb <= kSmallRows && (int64_t)n_units * region <= kSmallTotalRows;
    return p;
}

std::atomic<int> g_small_wait_limit{0};  // polls a block's wait may take (0: the default)

// What the host keeps per device for this route.
//   occ       blocks of small_layer_kernel<HD, G> that the device holds at once (0: not asked yet,
//             -1: unknown), per (hd, group)
//   last      the stream that the last launch of the kernel outside stream capture went to.  A
//             call on ANOTHER stream asks whether that stream has run dry (hipStreamQuery: no
//             wait, nothing enqueued); while it has not, a launch here could overlap with the
//             last one.  (An event behind every launch would say the same a little more
//             precisely, but an event is a packet of its own in the queue: 5 us on a 36 us layer.)
//   mail      one word of pinned, mapped host memory: a block whose wait runs out stores its
//             launch number there, and the host looks at it (a plain read) at every later call
constexpr int kMaxDevices = 64;
struct SmallDev {
    int occ[3][9];
    hipStream_t last;
    bool have;
    volatile uint32_t *mail_host;
    uint32_t *mail_dev;
    bool mail_tried;
};
SmallDev g_dev[kMaxDevices];
std::mutex g_small_mutex;
uint32_t g_launch_seq = 0;
// Failures seen so far in this process.  Every workspace remembers the count at which its select
// state was last initialised; a call on a workspace that lags behind initialises the state
// again whatever the caller says about it (any workspace may have been the one that failed).
std::atomic<uint32_t> g_err_epoch{0};
std::unordered_map<const void *, uint32_t> g_ws_epoch;

// Looks at the mailbox of device `dev` (under g_small_mutex).
void observe_mailbox(int dev) {
    SmallDev &d = g_dev[dev];
    if (!d.mail_host) return;
    if (*d.mail_host != 0u) {
        *d.mail_host = 0u;  // a store of the device that lands between the two lines reports a launch that
                            // was enqueued before anything this observation leads to, so nothing is lost
        g_err_epoch.fetch_add(1u);
    }
}

int current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return -1;
    }
    return dev;
}

template <int HD, int G>
int small_occupancy() {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, small_layer_kernel<HD, G>, kThreads, 0) != hipSuccess) n = 0;
    (void)hipGetLastError();
    return n;
}

template <int HD>
int small_occupancy_g(int group) {
    switch (group) {
        case 1: return small_occupancy<HD, 1>();
        case 2: return small_occupancy<HD, 2>();
        case 3: return small_occupancy<HD, 3>();
        case 4: return small_occupancy<HD, 4>();
        case 5: return small_occupancy<HD, 5>();
        case 6: return small_occupancy<HD, 6>();
        case 7: return small_occupancy<HD, 7>();
        case 8: return small_occupancy<HD, 8>();
    }
    return 0;
}

template <int HD>
int launch_small(int group, dim3 grid, hipStream_t st, const SmallArgs &a) {
#define DC_CASE(GG)                                                                          \
    case GG:                                                                                 \
        hipLaunchKernelGGL((small_layer_kernel<HD, GG>), grid, dim3(kThreads), 0, st, a);     \
        return 0;
    switch (group) {
        DC_CASE(1)
        DC_CASE(2)
        DC_CASE(3)
        DC_CASE(4)
        DC_CASE(5)
        DC_CASE(6)
        DC_CASE(7)
        DC_CASE(8)
    }
#undef DC_CASE
    return -1;
}

}  // namespace

extern "C" void dc_set_wait_limit(int polls) { g_small_wait_limit.store(polls > 0 ? polls : 0); }

// The rule that keeps two launches of the kernel from overlapping, as a pure function (1: the
// kernel may be launched now, 0: the call takes the chain of kernels instead).
extern "C" int dc_one_kernel_guard(int policy, int capturing, int have_prev, int same_stream, int prev_done) {
    if (policy == DC_ONE_KERNEL_NEVER) return 0;
    if (policy == DC_ONE_KERNEL_EXCLUSIVE) return 1;  // the caller vouches that nothing else holds CUs
    if (capturing) return 0;   // a graph is replayed at times and on streams the library never sees
    if (!have_prev || same_stream) return 1;  // no earlier launch, or the stream orders the two
    return prev_done ? 1 : 0;
}

extern "C" unsigned dc_decode_layer_errors(void) {
    const int dev = current_device();
    if (dev >= 0) {
        std::lock_guard<std::mutex> lock(g_small_mutex);
        observe_mailbox(dev);
    }
    return g_err_epoch.load();
}

// Whether the caller's "the select state is ready" still holds for this workspace: not after a
// failure that was seen since the state was last initialised.  Looks at the mailbox first.
bool dc_ws_state_trusted(const void *workspace) {
    const int dev = current_device();
    std::lock_guard<std::mutex> lock(g_small_mutex);
    if (dev >= 0) observe_mailbox(dev);
    const uint32_t now = g_err_epoch.load();
    if (now == 0u) return true;  // nothing ever failed: nothing is kept per workspace
    const auto it = g_ws_epoch.find(workspace);
    return (it == g_ws_epoch.end() ? 0u : it->second) == now;
}

// The select state of this workspace is being initialised by the current call.
void dc_ws_state_initialised(const void *workspace) {
    const uint32_t now = g_err_epoch.load();
    if (now == 0u) return;
    std::lock_guard<std::mutex> lock(g_small_mutex);
    g_ws_epoch[workspace] = now;
}

// Whether a layer of these sizes can take the one-kernel route: every block must be resident at
// once (the blocks of a unit wait for each other), a block's rows must fit its LDS, and the
// merge must hold the (m, l) pairs of a unit's blocks.
bool dc_small_supported(int n_units, int region, int k_eff, int group, int hd, bool has_sketch) {
    // DIFFCACHE_ONE_KERNEL=0 in the environment (read once) switches the route off, for processes
    // that share the GPU with kernels that never leave their CUs
    static const bool enabled = [] {
        const char *e = std::getenv("DIFFCACHE_ONE_KERNEL");
        return !(e && e[0] == '0' && e[1] == 0);
    }();
    if (!enabled) return false;
    if (k_eff < 1 || group < 1 || group > 8 || !(hd == 64 || hd == 128 || hd == 256)) return false;
    const SmallPlan p = plan_small(n_units, region);
    if (!p.ok || p.bpu * group * 2 > kSmallMl) return false;
    // a caller with a sketch has the faster chain: there the kernel only wins up to 40 Ki rows per unit
    if (has_sketch && region > kSmallSketchRows) return false;
    const int hi = hd == 64 ? 0 : (hd == 128 ? 1 : 2);
    const int dev = current_device();
    if (dev < 0) return false;
    int occ;
    {
        std::lock_guard<std::mutex> lock(g_small_mutex);
        occ = g_dev[dev].occ[hi][group];
        if (occ == 0) {  // first use on this device: blocks per CU times its CUs
            occ = hd == 64 ? small_occupancy_g<64>(group) : (hd == 128 ? small_occupancy_g<128>(group) : small_occupancy_g<256>(group));
            int cus = 0;
            if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
                (void)hipGetLastError();
                cus = 0;
            }
            occ = occ > 0 && cus > 0 ? occ * cus : -1;
            g_dev[dev].occ[hi][group] = occ;
        }
    }
    if (occ <= 0) return false;
    return (int64_t)n_units * p.bpu <= (int64_t)occ;
}

size_t dc_small_workspace_bytes(int n_units, int region, int group, int hd) {
    const SmallPlan p = plan_small(n_units, region);
    if (!p.ok) return 0;
    return carve_attn(nullptr, n_units, group, hd, p.bpu).bytes;
}

// The route's own candidate lists: one packed (key, id) word per region row.  They are not shared
// with the lists of the other routes, so a workspace whose state is ready stays ready for this
// route whichever route the calls in between took.
size_t dc_small_cand_bytes(int n_units, int region) {
    const SmallPlan p = plan_small(n_units, region);
    if (!p.ok) return 0;
    return dc_align_up((size_t)n_units * (size_t)region * 8, 256);
}

namespace {
__global__ void small_list_init_kernel(unsigned long long *list, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) list[i] = kEmpty;
}
}  // namespace

// What the one-kernel route needs beyond dc_select_state_init: every slot of the candidate
// lists empty.  The kernel leaves them so.
int dc_small_state_init(int n_units, int region, void *cand, void *stream) {
    const int64_t n = (int64_t)n_units * region;
    if (n <= 0) return DC_OK;
    hipLaunchKernelGGL(small_list_init_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<unsigned long long *>(cand), n);
    DC_CHECK_LAUNCH("dc_decode_layer(one kernel, init)");
    return DC_OK;
}

// The whole layer on `stream`, unless the launch could overlap with an earlier one of this kernel
// on another stream (or sits in a graph under capture, whose replays the library never sees): two
// such launches would each hold part of the CUs and wait for blocks that cannot start.  Returns
// 1 when the kernel was launched, 0 when the caller has to take the chain of kernels, or a
// negative DC_E* code.  sel_ws: the select part of the layer workspace, its state initialised or
// left ready by the previous call; cand: dc_small_cand_bytes(...) bytes, every slot empty;
// attn_ws: dc_small_workspace_bytes(...) bytes.
int dc_small_try(const dc_layer_args *a, int region, int k_eff, void *sel_ws, void *cand, void *attn_ws,
                 size_t attn_ws_bytes, void *stream) {
    const char *who = "dc_decode_layer(one kernel)";
    const int n_units = a->n_b * a->n_h;
    const SmallPlan p = plan_small(n_units, region);
    DC_REQUIRE(p.ok, "%s: shape not supported", who);
    DC_REQUIRE((a->new_k == nullptr) == (a->new_v == nullptr), "%s: new_k and new_v must both be set or both be null", who);
    DC_REQUIRE(dc_aligned16(a->q) && dc_aligned16(a->k) && dc_aligned16(a->v) &&
                   (!a->new_k || (dc_aligned16(a->new_k) && dc_aligned16(a->new_v))),
               "%s: pointers must be 16-byte aligned", who);
    DC_REQUIRE(a->kv_batch_stride % 8 == 0 && a->kv_head_stride % 8 == 0 && a->kv_row_stride % 8 == 0 &&
                   a->kv_row_stride >= a->hd,
               "%s: strides must be multiples of 8 elements and row_stride >= hd", who);
    DC_REQUIRE(a->mode == DC_MODE_IP || a->mode == DC_MODE_REF_DIST, "%s: bad mode %d", who, a->mode);
    DC_REQUIRE(a->idx_unit_stride >= k_eff, "%s: idx_unit_stride < min(budget, region rows)", who);
    DC_REQUIRE(a->recent_lo + a->n_recent < 0xffffffffll, "%s: row numbers out of range", who);
    DC_REQUIRE(a->one_kernel >= DC_ONE_KERNEL_NEVER && a->one_kernel <= DC_ONE_KERNEL_EXCLUSIVE,
               "%s: bad one_kernel policy %d", who, a->one_kernel);
    const FusedWs w = carve_fused(sel_ws, n_units, region, a->budget);
    const AttnWs aw = carve_attn(attn_ws, n_units, a->group, a->hd, p.bpu);
    if (attn_ws_bytes < aw.bytes) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, attn_ws_bytes, aw.bytes);
        return DC_ENOMEM;
    }
    hipStream_t st = (hipStream_t)stream;
    const int dev = current_device();
    DC_REQUIRE(dev >= 0, "%s: no current device (or device number >= %d)", who, kMaxDevices);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusNone;
    }
    const bool capturing = cap != hipStreamCaptureStatusNone;

    std::lock_guard<std::mutex> lock(g_small_mutex);
    SmallDev &d = g_dev[dev];
    bool prev_done = true;
    const bool same = d.have && d.last == st;
    if (a->one_kernel == DC_ONE_KERNEL_AUTO && !capturing && d.have && !same) {
        // Has the last launch, on the other stream, ended?  (A stream under capture cannot be
        // asked; a handle that is no longer a stream has nothing in flight that we know of.)
        prev_done = false;
        hipStreamCaptureStatus lc = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(d.last, &lc) == hipSuccess && lc == hipStreamCaptureStatusNone) {
            const hipError_t e = hipStreamQuery(d.last);
            prev_done = e == hipSuccess;
            if (e == hipErrorInvalidHandle || e == hipErrorInvalidResourceHandle || e == hipErrorContextIsDestroyed) {
                d.have = false;
                prev_done = true;
            }
        }
        (void)hipGetLastError();
    }
    if (!dc_one_kernel_guard(a->one_kernel, capturing ? 1 : 0, d.have ? 1 : 0, same ? 1 : 0, prev_done ? 1 : 0))
        return 0;
    if (!capturing && !d.mail_tried) {  // (no allocation inside a capture)
        d.mail_tried = true;
        void *hp = nullptr, *dp = nullptr;
        if (hipHostMalloc(&hp, 64, hipHostMallocMapped | hipHostMallocCoherent) == hipSuccess && hp &&
            hipHostGetDevicePointer(&dp, hp, 0) == hipSuccess && dp) {
            d.mail_host = static_cast<volatile uint32_t *>(hp);
            *d.mail_host = 0u;
            d.mail_dev = static_cast<uint32_t *>(dp);
        } else {
            (void)hipGetLastError();  // no mailbox: failures are still marked in the outputs and in the status call
        }
    }
    SmallArgs s;
    s.Q = (const uint16_t *)a->q;
    s.K = (const uint16_t *)a->k;
    s.V = (const uint16_t *)a->v;
    s.new_k = (const uint16_t *)a->new_k;
    s.new_v = (const uint16_t *)a->new_v;
    s.hist = w.hist;
    s.state = w.state;
    s.cand = reinterpret_cast<unsigned long long *>(cand);
    s.idx_out = a->idx_out;
    s.idx_stride = a->idx_unit_stride;
    s.ws_acc = aw.acc;
    s.ws_ml = aw.ml;
    s.out = (uint16_t *)a->out;
    s.lse = a->lse;
    s.n_recent_dev = a->n_recent_dev;
    s.n_units = n_units;
    s.n_h = a->n_h;
    s.n_rows = region;
    s.rows_per_block = p.rows_per_block;
    s.bpu = p.bpu;
    s.k_eff = k_eff;
    s.mode = a->mode;
    s.n_sink = a->n_sink;
    s.recent_lo = a->recent_lo;
    s.n_recent = a->n_recent;
    s.sb = a->kv_batch_stride, s.sh = a->kv_head_stride, s.sr = a->kv_row_stride;
    s.scale = a->scale;
    s.spin_limit = g_small_wait_limit.load() > 0 ? g_small_wait_limit.load() : (1 << 20);
    s.mailbox = d.mail_dev;
    if (++g_launch_seq == 0u) g_launch_seq = 1u;
    s.launch_seq = g_launch_seq;
    dim3 grid((unsigned)(n_units * p.bpu));
    int rc;
    if (a->hd == 64) rc = launch_small<64>(a->group, grid, st, s);
    else if (a->hd == 128) rc = launch_small<128>(a->group, grid, st, s);
    else rc = launch_small<256>(a->group, grid, st, s);
    DC_REQUIRE(rc == 0, "%s: unsupported group %d", who, a->group);
    DC_CHECK_LAUNCH(who);
    if (!capturing) {
        d.last = st;
        d.have = true;
    }
    return 1;
}
