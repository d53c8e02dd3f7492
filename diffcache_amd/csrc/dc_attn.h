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

// mfma: the split runs on the matrix cores (dc_attn_split_mfma), whose slice does not depend on the group
inline AttnPlan plan_attn(int hd, int group, int n_total, bool mfma) {
    AttnPlan p;
    p.rows_per_split = mfma ? kAttnWaves * 16 * (hd <= 128 ? 2 : 1) : (kAttnThreads / (hd / 8)) * rows_per_group(group);
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
    const int32_t *recent_lo_dev;  // null, or the first row of the suffix as a device word (recent_lo: its largest value)
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
    const int64_t recent_lo = a.recent_lo_dev ? (int64_t)*a.recent_lo_dev : a.recent_lo;

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
                r = (uint32_t)(recent_lo + (vj - n_idx - n_sink));
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


// ---------------------------------------------------------------------------------------------
// The same split on the matrix cores.
//
// QK^T and PV of a decode step are thin products (G query heads against 16 or 32 gathered rows),
// far from filling an MFMA tile, but the VALU version spends most of its instructions unpacking
// bf16, multiplying 8 columns at a time and summing over the 16 lanes of a row; on the matrix
// cores the packed rows are operands as loaded.  A wave owns TILES tiles of 16 list positions.
//
//   S = K Q^T   v_mfma_f32_16x16x32_bf16, M = the tile's 16 rows, N = 16 query heads (G used, the
//               rest zero), K = 32 of the HD columns per instruction.  Lane (q, c) = (lane / 16,
//               lane % 16) supplies columns 32 ch + 8 q .. + 7 of row c: one 16-byte load per ch.
//               The result leaves S[row 4q + i][head c], i < 4, in lane (q, c).
//   O = P V     M = query heads, N = 16 of the HD output columns, K = the rows.  That lane's four
//               logits per tile are, as they stand, its part of the A operand (head c, rows 4q + i)
//               once exponentiated and split into two bf16 values (flash_attn_with_kvcache,
//               base.py:134-142, rounds P to one; that alone misses the 2e-3 bar on short
//               slices).  The B operand wants, per lane, the values of ITS rows 4q + i
//               in one output column; column n of instruction j is taken to be d = (HD/16) c + j,
//               so lane (q, c) loads HD/16 adjacent columns of each of its rows (16 bytes at
//               HD 128) and picks element j of every loaded vector with v_perm_b32: no transpose
//               through LDS and no data crossing lanes.  acc[j][i] = O[head 4q + i][(HD/16) c + j].
//
// Row ids are resolved once per position (by the lane that loads the K row) and handed to the
// lanes that load the V rows by a wave shuffle.  Rows are fetched with buffer loads relative to
// the unit's first row (32-bit offsets), so a load costs one multiply, not a 64-bit address.
typedef __bf16 dc_bf16x8 __attribute__((ext_vector_type(8)));
typedef short dc_s16x4 __attribute__((ext_vector_type(4)));
typedef float dc_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dc_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dc_u32x2 __attribute__((ext_vector_type(2)));

constexpr int kMfmaMaxGroup = 16;
__host__ __device__ constexpr int mfma_tiles(int hd) { return hd <= 128 ? 2 : 1; }
__host__ __device__ constexpr int mfma_rows_per_split(int hd) { return kAttnWaves * 16 * mfma_tiles(hd); }
// floats of LDS: per-wave maxima and sums of 16 heads, per-wave partial outputs of G heads
inline size_t mfma_shared_bytes(int hd, int group) {
    return (size_t)(2 * kAttnWaves * 16 + kAttnWaves * group * hd) * sizeof(float);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t dc_rows_rsrc(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);  // 4 GiB window, no stride
}

// two finite floats rounded to nearest even, packed
__device__ __forceinline__ uint32_t dc_pack_bf16(float lo, float hi) {
    const uint32_t a = __float_as_uint(lo), b = __float_as_uint(hi);
    const uint32_t ra = a + 0x7fffu + ((a >> 16) & 1u), rb = b + 0x7fffu + ((b >> 16) & 1u);
    return __builtin_amdgcn_perm(rb, ra, 0x07060302u);  // (rb & 0xffff0000) | (ra >> 16)
}

template <int HD>
__device__ __forceinline__ void dc_attn_split_mfma(const AttnArgs &a, int G, int unit, int split, float *s_mem) {
    constexpr int TILES = mfma_tiles(HD);
    constexpr int EPL = HD / 16;   // columns of a V row per lane
    constexpr int VW = EPL / 2;    // the same in 32-bit words
    constexpr int CH = HD / 32;    // instructions of one tile's QK^T
    constexpr int ROWS_W = 16 * TILES;
    constexpr int ROWS = kAttnWaves * ROWS_W;
    static_assert(HD == 64 || HD == 128 || HD == 256, "head_dim");
    float *s_red = s_mem;                          // [kAttnWaves][16]
    float *s_l = s_mem + kAttnWaves * 16;          // [kAttnWaves][16]
    float *s_acc = s_mem + 2 * kAttnWaves * 16;    // [kAttnWaves][G * HD]

    const int b = unit / a.n_h, h = unit % a.n_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane >> 4, c = lane & 15;
    const int n_idx = a.n_idx, n_sink = a.n_sink;
    int n_recent = a.n_recent, n_total = a.n_total;
    const int64_t recent_lo = a.recent_lo_dev ? (int64_t)*a.recent_lo_dev : a.recent_lo;
    if (a.n_recent_dev) {  // the window's length may live on the device (cache_seqlens, base.py:134-142)
        int cur = *a.n_recent_dev;
        cur = cur < 0 ? 0 : (cur < n_recent ? cur : n_recent);
        n_total -= n_recent - cur;
        n_recent = cur;
    }
    int n_eff = n_idx;  // only the first n_eff selected ids of the unit count when per-unit sizes are given
    if (a.n_idx_unit) {
        const uint32_t ne = a.n_idx_unit[unit];
        n_eff = ne < (uint32_t)n_idx ? (int)ne : n_idx;
    }
    const int p0 = split * ROWS + wave * ROWS_W;
    auto live = [&](int vj) { return vj < n_total && (vj < n_eff || vj >= n_idx); };

    // the store row of this lane's K position of every tile (row 0 for positions that do not count)
    uint32_t rowk[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int vj = p0 + t * 16 + c;
        uint32_t r = 0;
        if (live(vj)) {
            if (vj < n_idx) r = (uint32_t)(a.region_lo + a.idx[(int64_t)unit * a.idx_stride + vj]);
            else if (vj < n_idx + n_sink) r = (uint32_t)(vj - n_idx);
            else if (vj < n_idx + n_sink + n_recent) r = (uint32_t)(recent_lo + (vj - n_idx - n_sink));
            else r = kNewToken;
        }
        rowk[t] = r;
    }
    // the query heads as the B operand: head c, columns 32 ch + 8 q .. + 7
    dc_u32x4 bq[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        bq[ch] = dc_u32x4{0u, 0u, 0u, 0u};
        if (c < G) bq[ch] = *reinterpret_cast<const dc_u32x4 *>(a.Q + ((int64_t)unit * G + c) * HD + ch * 32 + q * 8);
    }
    const __amdgpu_buffer_rsrc_t rk = dc_rows_rsrc(a.K + b * a.ksb + h * a.ksh);
    const __amdgpu_buffer_rsrc_t rv = dc_rows_rsrc(a.V + b * a.vsb + h * a.vsh);
    const uint32_t k_row_bytes = (uint32_t)a.ksr * 2u, v_row_bytes = (uint32_t)a.vsr * 2u;

    // every K and V row of the slice is requested before any is used
    dc_u32x4 kw[TILES][CH];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const bool tok = rowk[t] == kNewToken;
        const uint32_t off = (tok ? 0u : rowk[t] * k_row_bytes) + (uint32_t)q * 16u;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch)
            kw[t][ch] = __builtin_bit_cast(dc_u32x4, __builtin_amdgcn_raw_buffer_load_b128(rk, (int)(off + ch * 64u), 0, 0));
        if (tok) {  // the current token's key comes from its own buffer (one position of the whole list)
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
                kw[t][ch] = *reinterpret_cast<const dc_u32x4 *>(a.new_k + (int64_t)unit * HD + ch * 32 + q * 8);
        }
    }
    uint32_t vwd[TILES * 4][VW];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t r = (uint32_t)__shfl((int)rowk[t], 4 * q + i, 64);
            const bool tok = r == kNewToken;
            const uint32_t off = (tok ? 0u : r * v_row_bytes) + (uint32_t)c * (EPL * 2u);
            uint32_t *dst = vwd[t * 4 + i];
            if constexpr (VW == 2) {
                const dc_u32x2 v2 = __builtin_bit_cast(dc_u32x2, __builtin_amdgcn_raw_buffer_load_b64(rv, (int)off, 0, 0));
                dst[0] = v2.x, dst[1] = v2.y;
            } else {
#pragma unroll
                for (int w4 = 0; w4 < VW / 4; ++w4) {
                    const dc_u32x4 v4 = __builtin_bit_cast(dc_u32x4, __builtin_amdgcn_raw_buffer_load_b128(rv, (int)(off + w4 * 16u), 0, 0));
                    dst[4 * w4 + 0] = v4.x, dst[4 * w4 + 1] = v4.y, dst[4 * w4 + 2] = v4.z, dst[4 * w4 + 3] = v4.w;
                }
            }
            if (tok) {
                const uint32_t *src = reinterpret_cast<const uint32_t *>(a.new_v + (int64_t)unit * HD + c * EPL);
#pragma unroll
                for (int w2 = 0; w2 < VW; ++w2) dst[w2] = src[w2];
            }
        }

    // S = K Q^T, scaled; positions that do not count get -inf
    float x[TILES][4];
    float mloc = -INFINITY;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        dc_f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ch = 0; ch < CH; ++ch)
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dc_bf16x8, kw[t][ch]),
                                                        __builtin_bit_cast(dc_bf16x8, bq[ch]), s, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[t][i] = live(p0 + t * 16 + 4 * q + i) ? s[i] * a.scale : -INFINITY;
            mloc = fmaxf(mloc, x[t][i]);
        }
    }
    // maximum of head c over the block
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    if (q == 0) s_red[wave * 16 + c] = mloc;
    __syncthreads();
    float m = s_red[c];
#pragma unroll
    for (int w2 = 1; w2 < kAttnWaves; ++w2) m = fmaxf(m, s_red[w2 * 16 + c]);

    // P = exp(S - m): this lane's part of the A operand of P V, as the sum of two bf16 values
    // (p = hi + lo to 2^-17 of p: with P rounded to one bf16 a slice of a few rows misses the
    // 2e-3 bar where the terms cancel), so P V takes two instructions per 16 output columns
    float p[TILES * 4];
    uint32_t pa[TILES * 2], pb[TILES * 2];
    float lloc = 0.f;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[t * 4 + i] = x[t][i] > -INFINITY ? __expf(x[t][i] - m) : 0.f;
            lloc += p[t * 4 + i];
        }
#pragma unroll
    for (int k2 = 0; k2 < TILES * 2; ++k2) {
        pa[k2] = dc_pack_bf16(p[2 * k2], p[2 * k2 + 1]);
        pb[k2] = dc_pack_bf16(p[2 * k2] - dc_bf16_lo(pa[k2]), p[2 * k2 + 1] - dc_bf16_hi(pa[k2]));
    }
    dc_f32x4 acc[EPL];
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;  // the high or the low halves of two words
        uint32_t bv[TILES * 2];
#pragma unroll
        for (int k2 = 0; k2 < TILES * 2; ++k2)
            bv[k2] = __builtin_amdgcn_perm(vwd[2 * k2 + 1][j / 2], vwd[2 * k2][j / 2], sel);
        const dc_f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        if constexpr (TILES == 2) {
            const dc_u32x4 ah = {pa[0], pa[1], pa[TILES * 2 - 2], pa[TILES * 2 - 1]};
            const dc_u32x4 al = {pb[0], pb[1], pb[TILES * 2 - 2], pb[TILES * 2 - 1]};
            const dc_bf16x8 bw = __builtin_bit_cast(dc_bf16x8, dc_u32x4{bv[0], bv[1], bv[TILES * 2 - 2], bv[TILES * 2 - 1]});
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dc_bf16x8, al), bw, zero, 0, 0, 0);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dc_bf16x8, ah), bw, acc[j], 0, 0, 0);
        } else {
            const dc_s16x4 bw = __builtin_bit_cast(dc_s16x4, dc_u32x2{bv[0], bv[1]});
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(dc_s16x4, dc_u32x2{pb[0], pb[1]}), bw, zero, 0, 0, 0);
            acc[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(dc_s16x4, dc_u32x2{pa[0], pa[1]}), bw, acc[j], 0, 0, 0);
        }
    }

    // the wave's partial output and sums, then the block's
    lloc += __shfl_xor(lloc, 16, 64);
    lloc += __shfl_xor(lloc, 32, 64);
    if (q == 0) s_l[wave * 16 + c] = lloc;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int head = 4 * q + i;
        if (head < G) {
            float *dst = s_acc + (wave * G + head) * HD + c * EPL;
#pragma unroll
            for (int j = 0; j < EPL; ++j) dst[j] = acc[j][i];
        }
    }
    __syncthreads();
    const int64_t slot = (int64_t)unit * a.n_splits + split;
    for (int o = tid; o < G * HD; o += kAttnThreads) {
        float s = s_acc[o];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) s += s_acc[w2 * G * HD + o];
        a.ws_acc[slot * (G * HD) + o] = s;
    }
    if (tid < G) {
        float l = s_l[tid], mm = s_red[tid];
#pragma unroll
        for (int w2 = 1; w2 < kAttnWaves; ++w2) {
            l += s_l[w2 * 16 + tid];
            mm = fmaxf(mm, s_red[w2 * 16 + tid]);
        }
        float *ml = a.ws_ml + (slot * G + tid) * 2;
        ml[0] = mm;
        ml[1] = l;
    }
}

}  // namespace
