// Decode attention over gathered K/V rows: the per-split body and the merge of the splits,
// used by the attention kernels (attn.hip).  Replaces flash_attn_with_kvcache over the assembled buffer
// (src/diffcache/base.py:134-142, src/diffcache/kvcache/diffcache.py:196-209).
//
// A split is a slice of rows_per_group * NG consecutive positions of a unit's attended list
// [selected | sinks | recent | current token] (128 rows at head_dim 128 and a GQA group of 4).
// A group of LPR = HD/8 lanes owns one row at a time (one 16-byte load per lane covers the
// row) and the G query heads of the GQA group share every row that is loaded.  All K and V
// rows of the slice are requested up front, the logits stay in registers, the block agrees
// on a per-head maximum, and each split leaves (m, l, acc) in the workspace.
#pragma once
#include "dc_common.h"
#include <math.h>

namespace {

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;
// rows a lane group takes per block: 8 while the GQA group is small, 4 when the per-head
// registers (queries, logits, accumulators) leave less room
__host__ __device__ constexpr int rows_per_group(int group) { return group <= 4 ? 8 : 4; }
constexpr uint32_t kNewToken = 0xffffffffu;

struct AttnPlan {
    int rows_per_split;
    int n_splits;
};

inline AttnPlan plan_attn(int hd, int group, int n_total) {
    AttnPlan p;
    p.rows_per_split = (kAttnThreads / (hd / 8)) * rows_per_group(group);
    p.n_splits = n_total > 0 ? (n_total + p.rows_per_split - 1) / p.rows_per_split : 1;
    return p;
}

struct AttnWs {
    float *acc, *ml;
    size_t bytes;
};

inline AttnWs carve_attn(void *base, int n_units, int group, int hd, int n_splits) {
    AttnWs w;
    char *p = (char *)base;
    size_t off = 0;
    const size_t slots = (size_t)(n_units > 0 ? n_units : 0) * (size_t)n_splits;
    w.acc = (float *)(p + off);
    off += dc_align_up(slots * group * hd * 4, 256);
    w.ml = (float *)(p + off);
    off += dc_align_up(slots * group * 2 * 4, 256);
    w.bytes = off;
    return w;
}

// Loads and stores of data that another block of the SAME kernel has written or will read.
// The L2 caches of the eight XCDs are not coherent with each other, so such data goes
// through agent-scope accesses (they are served at the memory side); plain accesses are only
// safe across a kernel boundary.
__device__ __forceinline__ uint32_t dc_ld_agent(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float dc_ld_agent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void dc_st_agent(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void dc_st_agent(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct AttnArgs {
    const uint16_t *Q, *K, *V;
    const uint32_t *idx;
    const uint16_t *new_k, *new_v;
    float *ws_acc, *ws_ml;
    const uint32_t *n_idx_unit;
    const int32_t *n_recent_dev;
    int n_h, n_idx;
    int64_t idx_stride, region_lo;
    int n_sink;
    int64_t recent_lo;
    int n_recent, n_total, n_splits;
    int64_t ksb, ksh, ksr, vsb, vsh, vsr;
    float scale;
};

struct AttnShared {
    float *red;  // [kAttnWaves][G]
    float *l;    // [kAttnWaves][G]
    float *acc;  // [kAttnWaves][G * HD]
};
template <int HD, int G>
constexpr int attn_shared_floats() { return kAttnWaves * G * 2 + kAttnWaves * G * HD; }

// One split of one unit.
template <int HD, int G>
__device__ __forceinline__ void dc_attn_split(const AttnArgs &a, int unit, int split, const AttnShared &sh) {
    constexpr int LPR = HD / 8;
    constexpr int NG = kAttnThreads / LPR;  // row groups per block
    constexpr int R = rows_per_group(G);
    constexpr int ROWS = NG * R;
    float(*s_red)[G] = reinterpret_cast<float(*)[G]>(sh.red);
    float(*s_l)[G] = reinterpret_cast<float(*)[G]>(sh.l);
    float(*s_acc)[G * HD] = reinterpret_cast<float(*)[G * HD]>(sh.acc);

    const int b = unit / a.n_h, h = unit % a.n_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gid = tid / LPR, col = tid % LPR;
    const int r0 = split * ROWS;
    const int n_idx = a.n_idx, n_sink = a.n_sink;
    int n_recent = a.n_recent, n_total = a.n_total;

    // The length of the recent window may live on the device (the role of cache_seqlens in
    // base.py:134-142): n_recent is then its capacity, which sized the grid, and the rows
    // beyond the actual length are masked like any position past the end of the list.
    if (a.n_recent_dev) {
        int c = *a.n_recent_dev;
        c = c < 0 ? 0 : (c < n_recent ? c : n_recent);
        n_total -= n_recent - c;
        n_recent = c;
    }

    // only the first n_eff selected ids of the unit count when per-unit sizes are given
    int n_eff = n_idx;
    if (a.n_idx_unit) {
        const uint32_t ne = a.n_idx_unit[unit];
        n_eff = ne < (uint32_t)n_idx ? (int)ne : n_idx;
    }

    // physical rows of this group's list positions
    uint32_t row[R];
    bool ok[R];
#pragma unroll
    for (int t = 0; t < R; ++t) {
        const int vj = r0 + t * NG + gid;
        ok[t] = vj < n_total && (vj < n_eff || vj >= n_idx);
        uint32_t r = 0;
        if (ok[t]) {
            if (vj < n_idx) {
                const uint32_t *ip = a.idx + (int64_t)unit * a.idx_stride + vj;
                r = (uint32_t)(a.region_lo + *ip);
            } else if (vj < n_idx + n_sink) {
                r = (uint32_t)(vj - n_idx);
            } else if (vj < n_idx + n_sink + n_recent) {
                r = (uint32_t)(a.recent_lo + (vj - n_idx - n_sink));
            } else {
                r = kNewToken;
            }
        }
        row[t] = r;
    }
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const uint4 w = *reinterpret_cast<const uint4 *>(a.Q + ((int64_t)unit * G + g) * HD + col * 8);
        qf[g][0] = dc_bf16_lo(w.x);
        qf[g][1] = dc_bf16_hi(w.x);
        qf[g][2] = dc_bf16_lo(w.y);
        qf[g][3] = dc_bf16_hi(w.y);
        qf[g][4] = dc_bf16_lo(w.z);
        qf[g][5] = dc_bf16_hi(w.z);
        qf[g][6] = dc_bf16_lo(w.w);
        qf[g][7] = dc_bf16_hi(w.w);
    }
    const uint16_t *Ku = a.K + b * a.ksb + h * a.ksh + col * 8;
    const uint16_t *Vu = a.V + b * a.vsb + h * a.vsh + col * 8;
    const uint16_t *nk = a.new_k ? a.new_k + (int64_t)unit * HD + col * 8 : Ku;
    const uint16_t *nv = a.new_v ? a.new_v + (int64_t)unit * HD + col * 8 : Vu;

    // every K and V row of the slice is requested before any is used
    uint4 kw[R], vw[R];
#pragma unroll
    for (int t = 0; t < R; ++t) {
        const uint16_t *pk = (row[t] == kNewToken) ? nk : Ku + (int64_t)row[t] * a.ksr;
        kw[t] = *reinterpret_cast<const uint4 *>(pk);
    }
#pragma unroll
    for (int t = 0; t < R; ++t) {
        const uint16_t *pv = (row[t] == kNewToken) ? nv : Vu + (int64_t)row[t] * a.vsr;
        vw[t] = *reinterpret_cast<const uint4 *>(pv);
    }

    // scaled logits, in registers: x[t][g] is known to every lane of the group
    float x[R][G];
    float mloc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) mloc[g] = -INFINITY;
#pragma unroll
    for (int t = 0; t < R; ++t)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float v = dc_group_sum<LPR>(dc_dot8(kw[t], qf[g], 0.f)) * a.scale;
            x[t][g] = ok[t] ? v : -INFINITY;
            mloc[g] = fmaxf(mloc[g], x[t][g]);
        }
    // per-head maximum over the block
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = mloc[g];
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
        if (lane == 0) s_red[wave][g] = v;
    }
    __syncthreads();
    float m[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = s_red[0][g];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) v = fmaxf(v, s_red[w2][g]);
        m[g] = v;
    }

    // p = exp(x - m), acc[g] += p * V
    float acc[G][8];
    float lloc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        lloc[g] = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < R; ++t) {
        const float v[8] = {dc_bf16_lo(vw[t].x), dc_bf16_hi(vw[t].x), dc_bf16_lo(vw[t].y),
                            dc_bf16_hi(vw[t].y), dc_bf16_lo(vw[t].z), dc_bf16_hi(vw[t].z),
                            dc_bf16_lo(vw[t].w), dc_bf16_hi(vw[t].w)};
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float p = ok[t] ? __expf(x[t][g] - m[g]) : 0.f;
            lloc[g] += p;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p, v[i], acc[g][i]);
        }
    }

    // reduce over the row groups: inside the wave, then across waves
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            lloc[g] += __shfl_xor(lloc[g], off, 64);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] += __shfl_xor(acc[g][i], off, 64);
        }
    if (lane < LPR) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (col == 0) s_l[wave][g] = lloc[g];
#pragma unroll
            for (int i = 0; i < 8; ++i) s_acc[wave][g * HD + col * 8 + i] = acc[g][i];
        }
    }
    __syncthreads();
    const int64_t slot = (int64_t)unit * a.n_splits + split;
    for (int o = tid; o < G * HD; o += kAttnThreads) {
        float s = s_acc[0][o];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) s += s_acc[w2][o];
        a.ws_acc[slot * (G * HD) + o] = s;
    }
    if (tid < G) {
        float l = s_l[0][tid];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) l += s_l[w2][tid];
        float mm = s_red[0][tid];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) mm = fmaxf(mm, s_red[w2][tid]);
        float *ml = a.ws_ml + (slot * G + tid) * 2;
        ml[0] = mm;
        ml[1] = l;
    }
}

}  // namespace
