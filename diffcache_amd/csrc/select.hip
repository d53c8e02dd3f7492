// Exact top-k selection on fp32 scores.  Replaces the bounded max-heap of
// search_bruteforce (diffcache_cpu/src/nsw.rs:600-621): the result is the k
// smallest (ordering key, id) pairs, i.e. the set a size-k heap with the
// reference's strict "replace on smaller distance" rule ends with (ties go to
// the lower id), which is also what DualHeap keeps (dualheap.rs:4-87).
//
// Three stages, all streaming or tiny:
//   1. a DC_HIST_BINS-bucket histogram of a monotone function of the key (filled
//      by the scoring kernel's epilogue, or by hist_kernel here);
//   2. filter_kernel: every block finds the bucket tb holding the k-th key,
//      emits all ids in buckets < tb (certain members) and the (key, id) pairs
//      of bucket tb (candidates), one atomic per block for each list;
//   3. finalize_kernel (one block per unit): radix select among the candidates
//      on the 32-bit key, then on the id among keys equal to the threshold.
// An optional sort_kernel orders the k ids (best first, or by id).
#include "dc_common.h"
#include "dc_select.h"

namespace {

constexpr int kFilterThreads = 256;
constexpr int kFilterPerThread = 32;
constexpr int kFilterChunk = kFilterThreads * kFilterPerThread;  // 8192 scores per block
constexpr int kSortLds = 4096;

struct UnitMeta {
    uint32_t tb;        // threshold bucket
    uint32_t c_less;    // keys in buckets < tb
    uint32_t win_cnt;   // running count of emitted certain members
    uint32_t cand_cnt;  // running count of emitted candidates
};

__global__ void zero_u32_kernel(uint32_t *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

__global__ __launch_bounds__(kFilterThreads) void hist_kernel(
    const float *__restrict__ scores, int64_t scores_stride, uint32_t *__restrict__ hist,
    int n_rows, int mode, int blocks_per_unit) {
    __shared__ uint32_t lhist[DC_HIST_BINS];
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int tid = threadIdx.x;
    for (int i = tid; i < DC_HIST_BINS; i += kFilterThreads) lhist[i] = 0;
    __syncthreads();
    const float *su = scores + (int64_t)unit * scores_stride;
    const int64_t base = (int64_t)chunk * kFilterChunk;
#pragma unroll 8
    for (int it = 0; it < kFilterPerThread; ++it) {
        int64_t i = base + it * kFilterThreads + tid;
        if (i < n_rows) {
            uint32_t key, bucket;
            dc_key_bucket(su[i], mode, key, bucket);
            atomicAdd(&lhist[bucket], 1u);
        }
    }
    __syncthreads();
    uint32_t *hu = hist + (int64_t)unit * DC_HIST_BINS;
    for (int i = tid; i < DC_HIST_BINS; i += kFilterThreads) {
        uint32_t c = lhist[i];
        if (c) atomicAdd(&hu[i], c);
    }
}

__global__ __launch_bounds__(kFilterThreads) void filter_kernel(
    const float *__restrict__ scores, int64_t scores_stride, const uint32_t *__restrict__ hist,
    UnitMeta *__restrict__ meta, uint32_t *__restrict__ idx_out, int64_t idx_stride,
    uint32_t *__restrict__ cand_key, uint32_t *__restrict__ cand_idx, int n_rows, int k_eff,
    int mode, int blocks_per_unit) {
    __shared__ uint32_t wtot[kFilterThreads / 64 + 1];
    __shared__ uint32_t s_tb, s_cless, s_wbase, s_cbase;
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int tid = threadIdx.x;

    if (tid == 0) {
        s_tb = DC_HIST_BINS;  // "everything is a certain member" unless a crossing is found
        s_cless = 0;
    }
    // ---- threshold bucket: the bucket holding the k_eff-th smallest key ----
    constexpr int kBinsPerThread = DC_HIST_BINS / kFilterThreads;
    static_assert(kBinsPerThread % 4 == 0 && kBinsPerThread * kFilterThreads == DC_HIST_BINS, "bin split");
    uint32_t bins[kBinsPerThread];
    uint32_t sum = 0;
    {
        const uint4 *hp =
            reinterpret_cast<const uint4 *>(hist + (int64_t)unit * DC_HIST_BINS) + tid * (kBinsPerThread / 4);
#pragma unroll
        for (int i = 0; i < kBinsPerThread / 4; ++i) {
            uint4 t = hp[i];
            bins[4 * i + 0] = t.x;
            bins[4 * i + 1] = t.y;
            bins[4 * i + 2] = t.z;
            bins[4 * i + 3] = t.w;
        }
#pragma unroll
        for (int i = 0; i < kBinsPerThread; ++i) sum += bins[i];
    }
    uint32_t total;
    uint32_t excl = block_excl_scan<kFilterThreads>(sum, wtot, &total);
    const uint32_t kk = (uint32_t)k_eff;
    if (excl < kk && kk <= excl + sum) {
        uint32_t run = excl;
        bool done = false;
#pragma unroll
        for (int i = 0; i < kBinsPerThread; ++i) {
            if (!done && run + bins[i] >= kk) {
                s_tb = tid * kBinsPerThread + i;
                s_cless = run;
                done = true;
            }
            run += bins[i];
        }
    }
    __syncthreads();
    const uint32_t tb = s_tb, c_less = s_cless;
    if (chunk == 0 && tid == 0) {
        meta[unit].tb = tb;
        meta[unit].c_less = c_less;
    }

    // ---- classify this block's scores ----
    const float *su = scores + (int64_t)unit * scores_stride;
    const int64_t base = (int64_t)chunk * kFilterChunk;
    uint32_t wmask = 0, cmask = 0;
    uint32_t keys[kFilterPerThread];
#pragma unroll
    for (int it = 0; it < kFilterPerThread; ++it) {
        int64_t i = base + it * kFilterThreads + tid;
        uint32_t key = 0xffffffffu, bucket = 0xffffffffu;
        if (i < n_rows) dc_key_bucket(su[i], mode, key, bucket);
        keys[it] = key;
        if (i < n_rows) {
            if (bucket < tb) wmask |= 1u << it;
            else if (bucket == tb) cmask |= 1u << it;
        }
    }
    const uint32_t nw = __popc(wmask), nc = __popc(cmask);
    uint32_t tot2;
    uint32_t ex2 = block_excl_scan<kFilterThreads>(nw | (nc << 16), wtot, &tot2);
    if (tid == 0) {
        uint32_t tw = tot2 & 0xffffu, tc = tot2 >> 16;
        s_wbase = tw ? atomicAdd(&meta[unit].win_cnt, tw) : 0;
        s_cbase = tc ? atomicAdd(&meta[unit].cand_cnt, tc) : 0;
    }
    __syncthreads();
    uint32_t wpos = s_wbase + (ex2 & 0xffffu);
    uint32_t cpos = s_cbase + (ex2 >> 16);
    uint32_t *io = idx_out + (int64_t)unit * idx_stride;
    uint32_t *ck = cand_key + (int64_t)unit * n_rows;
    uint32_t *ci = cand_idx + (int64_t)unit * n_rows;
#pragma unroll
    for (int it = 0; it < kFilterPerThread; ++it) {
        uint32_t i = (uint32_t)(base + it * kFilterThreads + tid);
        if (wmask & (1u << it)) {
            if (wpos < kk) io[wpos] = i;
            ++wpos;
        } else if (cmask & (1u << it)) {
            if (cpos < (uint32_t)n_rows) {
                ck[cpos] = keys[it];
                ci[cpos] = i;
            }
            ++cpos;
        }
    }
}

__global__ __launch_bounds__(kFinalThreads) void finalize_kernel(
    const UnitMeta *__restrict__ meta, const uint32_t *__restrict__ cand_key,
    const uint32_t *__restrict__ cand_idx, uint32_t *__restrict__ idx_out, int64_t idx_stride,
    int n_rows, int k_eff) {
    __shared__ uint32_t lh[kRadixBins];
    __shared__ uint32_t wtot[kFinalThreads / 64 + 1];
    __shared__ uint32_t sres[4];
    __shared__ uint32_t smisc[2];
    const int unit = blockIdx.x;
    const uint32_t c_less = meta[unit].c_less;
    uint32_t n_c = meta[unit].cand_cnt;
    if (n_c > (uint32_t)n_rows) n_c = n_rows;
    if (c_less >= (uint32_t)k_eff) return;
    uint32_t need = (uint32_t)k_eff - c_less;
    if (need > n_c) need = n_c;
    dc_finalize_unit(cand_key + (int64_t)unit * n_rows, cand_idx + (int64_t)unit * n_rows, n_c, need,
                     idx_out + (int64_t)unit * idx_stride + c_less, n_rows, lh, wtot, sres, smisc);
}

// Bitonic sort of each unit's k ids by (key, id) or by id.
template <bool IN_LDS>
__global__ __launch_bounds__(kFinalThreads) void sort_kernel(
    const float *__restrict__ scores, int64_t scores_stride, const uint32_t *__restrict__ sel_keys,
    uint32_t *__restrict__ idx_out, int64_t idx_stride, unsigned long long *__restrict__ scratch,
    int k_eff, int pow2, int mode, int order) {
    __shared__ unsigned long long lbuf[IN_LDS ? kSortLds : 1];
    const int unit = blockIdx.x;
    const int tid = threadIdx.x;
    unsigned long long *buf = IN_LDS ? lbuf : scratch + (int64_t)unit * pow2;
    uint32_t *io = idx_out + (int64_t)unit * idx_stride;
    const float *su = scores ? scores + (int64_t)unit * scores_stride : nullptr;
    for (int i = tid; i < pow2; i += kFinalThreads) {
        unsigned long long v = ~0ull;
        if (i < k_eff) {
            uint32_t id = io[i];
            if (order == DC_ORDER_BEST) {
                uint32_t key, bucket;
                if (sel_keys) key = sel_keys[(int64_t)unit * k_eff + i];
                else dc_key_bucket(su[id], mode, key, bucket);
                v = ((unsigned long long)key << 32) | id;
            } else {
                v = id;
            }
        }
        buf[i] = v;
    }
    if (IN_LDS) {
        // The list is padded to at least 128 elements, one block of a wave (the padding
        // sorts to the end).  Stages with a stride of at most 64 stay inside such a block:
        // the wave keeps the block in registers, two elements per lane, exchanges across
        // lanes with shuffles and touches LDS once per run of those stages.  Only the
        // stages that cross waves (stride >= 128) go through LDS with a block barrier.
        const int n = pow2 < 128 ? 128 : pow2;
        for (int i = pow2 + tid; i < n; i += kFinalThreads) buf[i] = ~0ull;
        __syncthreads();
        const int lane = tid & 63;
        auto local_stages = [&](int size_lo, int size_hi) {
            for (int blk = tid >> 6; blk * 128 < n; blk += kFinalThreads / 64) {  // wave-uniform
                const int i0 = blk * 128 + lane, i1 = i0 + 64;
                unsigned long long a = buf[i0], b = buf[i1];
                for (int size = size_lo; size <= size_hi; size <<= 1) {
                    int s = size >> 1;
                    if (s >= 64) {  // the two elements of the lane meet; both sort the same way
                        const bool asc = (i0 & size) == 0;
                        const unsigned long long lo = a < b ? a : b, hi = a < b ? b : a;
                        a = asc ? lo : hi;
                        b = asc ? hi : lo;
                        s = 32;
                    }
                    const bool asc_a = (i0 & size) == 0, asc_b = (i1 & size) == 0;
                    for (; s >= 1; s >>= 1) {
                        const unsigned long long pa = __shfl_xor(a, s, 64), pb = __shfl_xor(b, s, 64);
                        const bool lower = (lane & s) == 0;
                        a = ((lower == asc_a) == (a < pa)) ? a : pa;  // keep the smaller iff lower == asc
                        b = ((lower == asc_b) == (b < pb)) ? b : pb;
                    }
                }
                buf[i0] = a;
                buf[i1] = b;
            }
        };
        local_stages(2, 128);
        __syncthreads();
        for (int size = 256; size <= n; size <<= 1) {
            for (int stride = size >> 1, ls = __ffs(size) - 2; stride >= 128; stride >>= 1, --ls) {
                for (int t = tid; t < (n >> 1); t += kFinalThreads) {
                    const int i = ((t >> ls) << (ls + 1)) | (t & (stride - 1));
                    const int j = i + stride;
                    const bool asc = (i & size) == 0;
                    unsigned long long a = buf[i], b = buf[j];
                    if ((a > b) == asc) {
                        buf[i] = b;
                        buf[j] = a;
                    }
                }
                __syncthreads();
            }
            local_stages(size, size);
            __syncthreads();
        }
    } else {
        __syncthreads();
        for (int size = 2; size <= pow2; size <<= 1) {
            for (int stride = size >> 1, ls = __ffs(size) - 2; stride > 0; stride >>= 1, --ls) {
                for (int t = tid; t < (pow2 >> 1); t += kFinalThreads) {
                    const int i = ((t >> ls) << (ls + 1)) | (t & (stride - 1));
                    const int j = i + stride;
                    const bool asc = (i & size) == 0;
                    unsigned long long a = buf[i], b = buf[j];
                    if ((a > b) == asc) {
                        buf[i] = b;
                        buf[j] = a;
                    }
                }
                __syncthreads();
            }
        }
    }
    __syncthreads();
    for (int i = tid; i < k_eff; i += kFinalThreads) io[i] = (uint32_t)(buf[i] & 0xffffffffull);
}

// DC_ORDER_INDEX without a sort: the unit's ids are marked in an LDS bitmap of the
// context (one bit per row) and read back in ascending order.  One block per unit;
// used while the bitmap fits in LDS (2^20 rows = 128 KB).
constexpr int kBitmapMaxRows = 1 << 20;

__global__ __launch_bounds__(kFinalThreads) void index_order_kernel(uint32_t *__restrict__ idx_out,
                                                                    int64_t idx_stride, int k_eff,
                                                                    int n_words) {
    extern __shared__ uint32_t bitmap[];
    __shared__ uint32_t wtot[kFinalThreads / 64 + 1];
    const int unit = blockIdx.x;
    const int tid = threadIdx.x;
    uint32_t *io = idx_out + (int64_t)unit * idx_stride;
    // word w lives at w + w/32: the runs of 32 words the threads sweep below then start in
    // different banks
    auto slot = [](int w) { return w + (w >> 5); };
    const int n_slots = slot(n_words - 1) + 1;
    for (int i = tid; i < n_slots; i += kFinalThreads) bitmap[i] = 0;
    __syncthreads();
    for (int i = tid; i < k_eff; i += kFinalThreads) {
        const uint32_t id = io[i];
        atomicOr(&bitmap[slot((int)(id >> 5))], 1u << (id & 31u));
    }
    __syncthreads();
    // every thread owns a contiguous run of words
    const int per = (n_words + kFinalThreads - 1) / kFinalThreads;
    const int w0 = tid * per;
    const int w1 = w0 + per < n_words ? w0 + per : n_words;
    uint32_t cnt = 0;
    for (int w = w0; w < w1; ++w) cnt += __popc(bitmap[slot(w)]);
    uint32_t total;
    uint32_t pos = block_excl_scan<kFinalThreads>(cnt, wtot, &total);
    for (int w = w0; w < w1; ++w) {
        uint32_t bits = bitmap[slot(w)];
        while (bits) {
            const int b = __ffs((int)bits) - 1;
            io[pos++] = (uint32_t)w * 32u + (uint32_t)b;
            bits &= bits - 1u;
        }
    }
}

__global__ void compose_idx_kernel(const uint32_t *__restrict__ outer, int64_t outer_stride,
                                   const uint32_t *__restrict__ inner, int64_t inner_stride,
                                   uint32_t *__restrict__ out, int64_t out_stride, int n_inner,
                                   int64_t total) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total) return;
    int64_t u = t / n_inner, j = t % n_inner;
    out[u * out_stride + j] = outer[u * outer_stride + inner[u * inner_stride + j]];
}

struct SelectWs {
    uint32_t *hist;
    UnitMeta *meta;
    uint32_t *cand_key, *cand_idx;
    unsigned long long *sort_scratch;
    size_t bytes;
};

int next_pow2(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

SelectWs carve(void *base, int n_units, int n_rows, int k) {
    SelectWs w;
    size_t off = 0;
    char *p = (char *)base;
    w.hist = (uint32_t *)(p + off);
    off += dc_align_up((size_t)n_units * DC_HIST_BINS * 4, 256);
    w.meta = (UnitMeta *)(p + off);
    off += dc_align_up((size_t)n_units * sizeof(UnitMeta), 256);
    w.cand_key = (uint32_t *)(p + off);
    off += dc_align_up((size_t)n_units * (size_t)n_rows * 4, 256);
    w.cand_idx = (uint32_t *)(p + off);
    off += dc_align_up((size_t)n_units * (size_t)n_rows * 4, 256);
    w.sort_scratch = (unsigned long long *)(p + off);
    int keff = k < n_rows ? k : n_rows;
    if (keff > kSortLds) off += dc_align_up((size_t)n_units * next_pow2(keff) * 8, 256);
    w.bytes = off;
    return w;
}

}  // namespace

// Sort each unit's k_eff selected ids: DC_ORDER_BEST by (key, id) with the key
// taken from sel_keys (n_units, k_eff) when given, else recomputed from the dense
// scores; DC_ORDER_INDEX by id.  scratch is needed when k_eff > 4096.
int dc_sort_selected(const float *scores, int64_t scores_stride, const uint32_t *sel_keys,
                     uint32_t *idx_out, int64_t idx_stride, unsigned long long *scratch, int n_units,
                     int k_eff, int mode, int order, hipStream_t st, int n_rows) {
    if (order == DC_ORDER_INDEX && n_rows > 0 && n_rows <= kBitmapMaxRows && k_eff >= 512) {
        // the ids are distinct and below n_rows: mark and sweep beats a bitonic sort
        const int n_words = (n_rows + 31) / 32;
        const size_t lds = (size_t)(n_words + (n_words >> 5) + 1) * 4;
        // more than the default 64 KB of dynamic LDS has to be asked for; the attribute
        // belongs to the current device, so it is set on every such call (a host-side
        // store), always to the same value so that concurrent callers cannot undercut it
        if (lds > 64 * 1024) {
            constexpr int kMaxLds = (kBitmapMaxRows / 32 + kBitmapMaxRows / 1024 + 1) * 4;
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(index_order_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
            if (e != hipSuccess) {
                dc_set_error("dc_sort_selected: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
                return DC_ELAUNCH;
            }
        }
        hipLaunchKernelGGL(index_order_kernel, dim3(n_units), dim3(kFinalThreads), lds, st, idx_out,
                           idx_stride, k_eff, n_words);
        DC_CHECK_LAUNCH("dc_sort_selected(index)");
        return DC_OK;
    }
    const int p2 = next_pow2(k_eff);
    if (p2 <= kSortLds)
        hipLaunchKernelGGL(sort_kernel<true>, dim3(n_units), dim3(kFinalThreads), 0, st, scores,
                           scores_stride, sel_keys, idx_out, idx_stride,
                           (unsigned long long *)nullptr, k_eff, p2, mode, order);
    else
        hipLaunchKernelGGL(sort_kernel<false>, dim3(n_units), dim3(kFinalThreads), 0, st, scores,
                           scores_stride, sel_keys, idx_out, idx_stride, scratch, k_eff, p2, mode, order);
    DC_CHECK_LAUNCH("dc_sort_selected");
    return DC_OK;
}

extern "C" size_t dc_topk_workspace_bytes(int n_units, int n_rows, int k) {
    if (n_units <= 0 || n_rows <= 0 || k <= 0) return 256;
    return carve(nullptr, n_units, n_rows, k).bytes;
}

extern "C" int dc_topk_select(const float *scores, int64_t scores_unit_stride, uint32_t *idx_out,
                              int64_t idx_unit_stride, int n_units, int n_rows, int k, int mode,
                              int order, const uint32_t *hist, void *workspace,
                              size_t workspace_bytes, void *stream) {
    DC_REQUIRE(scores && idx_out, "dc_topk_select: null pointer");
    DC_REQUIRE(n_units >= 0 && n_rows >= 0 && k >= 0, "dc_topk_select: bad sizes");
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "dc_topk_select: bad mode %d", mode);
    DC_REQUIRE(order >= DC_ORDER_ANY && order <= DC_ORDER_INDEX, "dc_topk_select: bad order %d", order);
    const int k_eff = k < n_rows ? k : n_rows;
    if (n_units == 0 || k_eff == 0) return DC_OK;
    DC_REQUIRE(scores_unit_stride >= n_rows, "dc_topk_select: scores_unit_stride < n_rows");
    DC_REQUIRE(idx_unit_stride >= k_eff, "dc_topk_select: idx_unit_stride < min(k, n_rows)");
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "dc_topk_select: workspace must be non-null and 256-byte aligned");
    DC_REQUIRE(!hist || dc_aligned16(hist), "dc_topk_select: hist must be 16-byte aligned");
    SelectWs w = carve(workspace, n_units, n_rows, k);
    if (workspace_bytes < w.bytes) {
        dc_set_error("dc_topk_select: workspace %zu bytes < %zu needed", workspace_bytes, w.bytes);
        return DC_ENOMEM;
    }
    hipStream_t st = (hipStream_t)stream;
    const int64_t bpu = ((int64_t)n_rows + kFilterChunk - 1) / kFilterChunk;
    DC_REQUIRE((int64_t)n_units * bpu < (1ll << 31), "dc_topk_select: grid too large");

    // clear the running counters (and the histogram if it is computed here)
    {
        uint32_t *z = hist ? (uint32_t *)w.meta : w.hist;
        int64_t n = ((char *)w.cand_key - (char *)z) / 4;
        hipLaunchKernelGGL(zero_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, z, n);
        DC_CHECK_LAUNCH("dc_topk_select(zero)");
    }
    if (!hist) {
        hipLaunchKernelGGL(hist_kernel, dim3((unsigned)(n_units * bpu)), dim3(kFilterThreads), 0, st,
                           scores, scores_unit_stride, w.hist, n_rows, mode, (int)bpu);
        DC_CHECK_LAUNCH("dc_topk_select(hist)");
        hist = w.hist;
    }
    hipLaunchKernelGGL(filter_kernel, dim3((unsigned)(n_units * bpu)), dim3(kFilterThreads), 0, st,
                       scores, scores_unit_stride, hist, w.meta, idx_out, idx_unit_stride,
                       w.cand_key, w.cand_idx, n_rows, k_eff, mode, (int)bpu);
    DC_CHECK_LAUNCH("dc_topk_select(filter)");
    hipLaunchKernelGGL(finalize_kernel, dim3(n_units), dim3(kFinalThreads), 0, st, w.meta,
                       w.cand_key, w.cand_idx, idx_out, idx_unit_stride, n_rows, k_eff);
    DC_CHECK_LAUNCH("dc_topk_select(finalize)");
    if (order != DC_ORDER_ANY)
        return dc_sort_selected(scores, scores_unit_stride, nullptr, idx_out, idx_unit_stride,
                                w.sort_scratch, n_units, k_eff, mode, order, st, n_rows);
    return DC_OK;
}

extern "C" int dc_compose_idx(const uint32_t *outer, int64_t outer_unit_stride,
                              const uint32_t *inner, int64_t inner_unit_stride, uint32_t *out,
                              int64_t out_unit_stride, int n_units, int n_inner, void *stream) {
    DC_REQUIRE(outer && inner && out, "dc_compose_idx: null pointer");
    DC_REQUIRE(n_units >= 0 && n_inner >= 0, "dc_compose_idx: bad sizes");
    int64_t total = (int64_t)n_units * n_inner;
    if (total == 0) return DC_OK;
    hipLaunchKernelGGL(compose_idx_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, outer, outer_unit_stride, inner, inner_unit_stride, out,
                       out_unit_stride, n_inner, total);
    DC_CHECK_LAUNCH("dc_compose_idx");
    return DC_OK;
}
