// Block-level scan and radix-select helpers shared by the select kernels.
#pragma once
#include "dc_common.h"

namespace {

constexpr int kFinalThreads = 1024;
constexpr int kRadixBits = 11;
constexpr int kRadixBins = 1 << kRadixBits;
constexpr int kScanBatch = 8;  // items of a list that a thread fetches before it looks at any
constexpr int kScanShort = 8192;  // lists in global memory up to this length are read with plain loops

// inclusive scan over the lanes of a wave: four shifts inside the rows of 16 lanes, then the
// last lane of row 0 (2) is added to row 1 (3), and the last lane of row 1 to rows 2 and 3
// (data-parallel primitives on the ALU; a shuffle through the LDS crossbar per step costs more)
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v, int) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, true);   // row_shr:1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, true);   // row_shr:2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, true);   // row_shr:4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, true);   // row_shr:8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
    return v;
}

// Block-wide exclusive scan for NT threads (NT a multiple of 64, <= 1024).
// `wtot` is LDS scratch of at least NT/64 + 1 words.  Returns the exclusive
// prefix; *total receives the block sum.  Contains two barriers.
template <int NT>
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t *wtot, uint32_t *total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int NW = NT / 64;
    uint32_t incl = wave_incl_scan(v, lane);
    if (lane == 63) wtot[wave] = incl;
    __syncthreads();
    uint32_t off = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        uint32_t t = wtot[w];
        if (w < wave) off += t;
        tot += t;
    }
    __syncthreads();
    *total = tot;
    return off + incl - v;
}

// Slots of a list in LDS for the lanes of a wave that ask for one: one addition per wave instead
// of one per lane (additions of a whole wave to one LDS word are served one after the other).
// Must be called by all lanes of the wave; returns the slot of a lane with `want`.
__device__ __forceinline__ uint32_t wave_reserve(bool want, uint32_t *counter) {
    const unsigned long long mask = __ballot(want);
    if (mask == 0ull) return 0u;
    const int lane = threadIdx.x & 63, leader = (int)__builtin_ctzll(mask);
    uint32_t base = 0u;
    if (lane == leader) base = atomicAdd(counter, (uint32_t)__popcll(mask));
    base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
    return base + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
}

// f(key, id, valid) for every entry of a (key, id) list, by ALL threads the same number of times
// (valid: the thread has an entry this time), so that f may use wave-wide operations.
template <int NT, bool IN_LDS = false, typename F>
__device__ __forceinline__ void dc_for_each_pair_uniform(const uint32_t *ck, const uint32_t *ci, uint32_t n, F f) {
    if (IN_LDS || n <= (uint32_t)kScanShort) {
        for (uint32_t i0 = 0; i0 < n; i0 += NT) {
            const uint32_t i = i0 + threadIdx.x;
            const bool in = i < n;
            f(in ? ck[i] : 0u, in ? ci[i] : 0u, in);
        }
        return;
    }
    for (uint32_t i0 = 0; i0 < n; i0 += kScanBatch * NT) {
        uint32_t key[kScanBatch], id[kScanBatch];
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const uint32_t i = i0 + (uint32_t)u * NT + threadIdx.x;
            key[u] = id[u] = 0u;
            if (i < n) {
                key[u] = ck[i];
                id[u] = ci[i];
            }
        }
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) f(key[u], id[u], i0 + (uint32_t)u * NT + threadIdx.x < n);
    }
}

// f(key, id) for every entry of a (key, id) list, kScanBatch entries of a thread in flight.
template <int NT, typename F>
__device__ __forceinline__ void dc_for_each_pair(const uint32_t *ck, const uint32_t *ci, uint32_t n, F f) {
    if (n <= (uint32_t)kScanShort) {
        for (uint32_t i = threadIdx.x; i < n; i += NT) f(ck[i], ci[i]);
        return;
    }
    for (uint32_t i0 = threadIdx.x; i0 < n; i0 += kScanBatch * NT) {
        uint32_t key[kScanBatch], id[kScanBatch];
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const uint32_t i = i0 + (uint32_t)u * NT;
            key[u] = id[u] = 0u;
            if (i < n) {
                key[u] = ck[i];
                id[u] = ci[i];
            }
        }
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u)
            if (i0 + (uint32_t)u * NT < n) f(key[u], id[u]);
    }
}

// One radix pass of a select: among the items whose bits [31, top) equal those of
// `prefix`, histogram bits [top-1, top-width) and find the bin that holds the
// rem-th smallest (1-based).  Updates prefix (bin bits filled in), rem (rank inside
// the bin), eq (bin size) and top (= the lowest decided bit).  Uniform over the block.
template <bool IN_LDS = false, typename Get>
__device__ __forceinline__ void block_radix_pass(Get get, uint32_t n, uint32_t &prefix, uint32_t &rem,
                                                 uint32_t &eq, int &top, uint32_t *lh, uint32_t *wtot,
                                                 uint32_t *sres) {
    const int tid = threadIdx.x;
    const int width = top < kRadixBits ? top : kRadixBits;
    const int shift = top - width;
    for (int i = tid; i < kRadixBins; i += kFinalThreads) lh[i] = 0;
    __syncthreads();
    const uint32_t himask = (top >= 32) ? 0u : (0xffffffffu << top);
    constexpr bool kPlain = IN_LDS;  // a list that the caller keeps in LDS: nothing to hide
    if (kPlain || n <= (uint32_t)kScanShort) {
        for (uint32_t i = tid; i < n; i += kFinalThreads) {
            uint32_t v;
            if (get(i, &v) && ((v & himask) == (prefix & himask)))
                atomicAdd(&lh[(v >> shift) & ((1u << width) - 1u)], 1u);
        }
    }
    // kScanBatch items of a thread are fetched before any is looked at: with one load per
    // iteration a long list costs a memory round trip per item and thread.  A wave whose lanes
    // all hit one bin (long runs of equal keys) adds its count once.
    for (uint32_t i0 = tid; !kPlain && n > (uint32_t)kScanShort && i0 < n; i0 += kScanBatch * kFinalThreads) {
        uint32_t v[kScanBatch];
        bool in[kScanBatch];
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const uint32_t i = i0 + (uint32_t)u * kFinalThreads;
            v[u] = 0u;
            in[u] = i < n && get(i, &v[u]);
        }
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const bool hit = in[u] && ((v[u] & himask) == (prefix & himask));
            const uint32_t bin = (v[u] >> shift) & ((1u << width) - 1u);
            const unsigned long long hits = __ballot(hit);
            if (hits == 0ull) continue;
            const int leader = (int)__builtin_ctzll(hits);
            const uint32_t lead = (uint32_t)__builtin_amdgcn_readlane((int)bin, leader);
            if (__ballot(hit && bin != lead) == 0ull) {
                if ((tid & 63) == leader) atomicAdd(&lh[lead], (uint32_t)__popcll(hits));
            } else if (hit) {
                atomicAdd(&lh[bin], 1u);
            }
        }
    }
    __syncthreads();
    // kRadixBins == 2 * kFinalThreads: each thread owns two adjacent bins
    const uint32_t h0 = lh[2 * tid], h1 = lh[2 * tid + 1];
    uint32_t total;
    const uint32_t excl = block_excl_scan<kFinalThreads>(h0 + h1, wtot, &total);
    if (excl < rem && rem <= excl + h0 + h1) {
        if (excl + h0 >= rem) {
            sres[0] = 2 * tid;
            sres[1] = excl;
            sres[2] = h0;
        } else {
            sres[0] = 2 * tid + 1;
            sres[1] = excl + h0;
            sres[2] = h1;
        }
    }
    __syncthreads();
    prefix |= sres[0] << shift;
    rem -= sres[1];
    eq = sres[2];
    top = shift;
    __syncthreads();
}

// Among `n` values v(i), find the rem-th smallest (1-based) by radix passes over
// bits [top-1, 0], the bits above being those of `prefix` for every item of the
// subset.  get(i, &value) returns false for items outside the subset.  Returns the
// threshold value; *rem_out = how many items equal to it are needed (rank of the
// threshold inside its tie group), *n_eq = size of the tie group.
template <bool IN_LDS = false, typename Get>
__device__ __forceinline__ uint32_t block_radix_select(Get get, uint32_t n, uint32_t rem, int top, uint32_t prefix,
                                       uint32_t eq, uint32_t *lh, uint32_t *wtot, uint32_t *sres,
                                       uint32_t *rem_out, uint32_t *n_eq) {
    while (top > 0) block_radix_pass<IN_LDS>(get, n, prefix, rem, eq, top, lh, wtot, sres);
    *rem_out = rem;
    *n_eq = eq;
    return prefix;
}

// Choose the `need` smallest (key, id) pairs among n_c candidates and write
// their ids to io[0, need).  Must be called by all kFinalThreads threads of a
// block with uniform arguments.  lh: kRadixBins words, wtot: kFinalThreads/64+1
// words, sres: 4 words, smisc: 2 words of LDS.  kout (optional) receives the
// key of each id written.  IN_LDS: ck and ci point into LDS (any length); lists in global
// memory longer than kScanShort are read kScanBatch entries per thread at a time.
template <bool IN_LDS = false>
__device__ __forceinline__ void dc_finalize_unit(const uint32_t *ck, const uint32_t *ci, uint32_t n_c, uint32_t need,
                                 uint32_t *io, int n_rows, uint32_t *lh, uint32_t *wtot,
                                 uint32_t *sres, uint32_t *smisc, uint32_t *kout = nullptr) {
    const int tid = threadIdx.x;
    if (need == n_c) {  // the whole candidate list is selected
#pragma unroll 4
        for (uint32_t i = tid; i < n_c; i += kFinalThreads) {
            io[i] = ci[i];
            if (kout) kout[i] = ck[i];
        }
        return;
    }
    // bits in which the candidate keys differ
    if (tid == 0) {
        smisc[0] = 0;  // OR of key differences, later the length of the tie list
        smisc[1] = 0;  // output slot counter
    }
    __syncthreads();
    const uint32_t k0 = ck[0];
    uint32_t diff = 0;
    const bool plain = IN_LDS || n_c <= (uint32_t)kScanShort;
    if (plain)
        for (uint32_t i = tid; i < n_c; i += kFinalThreads) diff |= ck[i] ^ k0;
    for (uint32_t i0 = tid; !plain && i0 < n_c; i0 += kScanBatch * kFinalThreads) {
        uint32_t v[kScanBatch];
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) {
            const uint32_t i = i0 + (uint32_t)u * kFinalThreads;
            v[u] = i < n_c ? ck[i] : k0;
        }
#pragma unroll
        for (int u = 0; u < kScanBatch; ++u) diff |= v[u] ^ k0;
    }
    // one addition per wave: a thousand lanes updating one LDS word are served one after the other
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) diff |= (uint32_t)__shfl_xor((int)diff, d, 64);
    if ((tid & 63) == 0 && diff) atomicOr(&smisc[0], diff);
    __syncthreads();
    diff = smisc[0];
    const int hb = diff ? 31 - __clz(diff) : -1;
    uint32_t prefix = (hb >= 31) ? 0u : (k0 & (0xffffffffu << (hb + 1)));
    int top = hb + 1;
    uint32_t rem = need, eq = n_c;
    auto get_key = [&](uint32_t i, uint32_t *v) {
        *v = ck[i];
        return true;
    };
    if (top > 0) block_radix_pass<IN_LDS>(get_key, n_c, prefix, rem, eq, top, lh, wtot, sres);

    if (eq <= (uint32_t)kFinalThreads) {
        // The keys whose decided bits equal the threshold bin's are few: they are
        // listed in LDS as packed (key, id) and ranked against each other, which
        // settles the remaining key bits and the ties by id at once.
        unsigned long long *tie = reinterpret_cast<unsigned long long *>(lh);
        __syncthreads();  // smisc[0] has been read by every thread
        if (tid == 0) smisc[0] = 0;
        __syncthreads();
        const uint32_t himask = (top >= 32) ? 0u : (0xffffffffu << top);
        const uint32_t base = need - rem;  // members from the bins below the threshold bin
        dc_for_each_pair_uniform<kFinalThreads, IN_LDS>(ck, ci, n_c, [&](uint32_t key, uint32_t id, bool in) {
            const uint32_t hi = key & himask, ph = prefix & himask;
            const bool member = in && hi < ph, tied = in && hi == ph;
            const uint32_t slot = wave_reserve(member, &smisc[1]);
            if (member && slot < base) {
                io[slot] = id;
                if (kout) kout[slot] = key;
            }
            const uint32_t e = wave_reserve(tied, &smisc[0]);
            if (tied && e < (uint32_t)kFinalThreads) tie[e] = ((unsigned long long)key << 32) | id;
        });
        __syncthreads();
        const uint32_t n_t = smisc[0] < (uint32_t)kFinalThreads ? smisc[0] : (uint32_t)kFinalThreads;
        if ((uint32_t)tid < n_t) {
            const unsigned long long mine = tie[tid];
            uint32_t rank = 0;
            for (uint32_t j = 0; j < n_t; ++j) rank += tie[j] < mine ? 1u : 0u;
            if (rank < rem) {
                io[base + rank] = (uint32_t)mine;
                if (kout) kout[base + rank] = (uint32_t)(mine >> 32);
            }
        }
        return;
    }

    uint32_t need_eq, n_eq;
    const uint32_t t_key =
        block_radix_select<IN_LDS>(get_key, n_c, rem, top, prefix, eq, lh, wtot, sres, &need_eq, &n_eq);

    uint32_t t_idx = 0xffffffffu;
    if (need_eq < n_eq) {  // only the lowest ids of the tie group fit
        const uint32_t span = (uint32_t)(n_rows - 1) | 1u;
        const int hbi = 31 - __clz(span);
        auto get_idx = [&](uint32_t i, uint32_t *v) {
            *v = ci[i];
            return ck[i] == t_key;
        };
        uint32_t r2, e2;
        t_idx = block_radix_select<IN_LDS>(get_idx, n_c, need_eq, hbi + 1, 0u, n_eq, lh, wtot, sres, &r2, &e2);
    }

    dc_for_each_pair_uniform<kFinalThreads, IN_LDS>(ck, ci, n_c, [&](uint32_t key, uint32_t id, bool in) {
        const bool member = in && (key < t_key || (key == t_key && id <= t_idx));
        const uint32_t slot = wave_reserve(member, &smisc[1]);
        if (member && slot < need) {
            io[slot] = id;
            if (kout) kout[slot] = key;
        }
    });
}

}  // namespace
