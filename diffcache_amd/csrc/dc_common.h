// Shared device helpers and host-side error plumbing for libdiffcache_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/diffcache_hip.h"

#define DC_WAVE 64

// ---- host side -------------------------------------------------------------
void dc_set_error(const char *fmt, ...);

#define DC_REQUIRE(cond, ...)            \
    do {                                 \
        if (!(cond)) {                   \
            dc_set_error(__VA_ARGS__);   \
            return DC_EINVAL;            \
        }                                \
    } while (0)

#define DC_CHECK_LAUNCH(name)                                              \
    do {                                                                   \
        hipError_t e_ = hipGetLastError();                                 \
        if (e_ != hipSuccess) {                                            \
            dc_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return DC_ELAUNCH;                                             \
        }                                                                  \
    } while (0)

// select.hip: sort the selected ids of every unit (see the definition); n_rows = rows of
// the context the ids index into
int dc_sort_selected(const float *scores, int64_t scores_stride, const uint32_t *sel_keys,
                     uint32_t *idx_out, int64_t idx_stride, unsigned long long *scratch, int n_units,
                     int k_eff, int mode, int order, hipStream_t st, int n_rows);

// fused.hip: argument checks, state initialisation and the scan kernel of the sketch route
int dc_sketch_scan_launch(const char *who, const void *k, const uint8_t *codes, const float *scale,
                          const float *resid, const void *q, int n_b, int n_h, int n_rows, int hd, int64_t sb,
                          int64_t sh, int64_t sr, int64_t cb, int64_t ch, int64_t cr, int q_group, int budget,
                          int mode, int state_ready, void *workspace, size_t workspace_bytes,
                          void *ev_scan_begin, void *ev_scan_end, void *stream, const int32_t *hi_dev = nullptr,
                          int lo_row = 0);
// fused.hip: the bf16 scan of the streaming route (dc_score_prune_bf16 with an optional device-side region end)
int dc_score_prune_launch(const void *k, const void *q, int n_b, int n_h, int n_rows, int hd, int64_t sb, int64_t sh,
                          int64_t sr, int q_group, int budget, int mode, void *workspace, size_t workspace_bytes,
                          void *stream, const int32_t *hi_dev, int lo_row);
// fused.hip: dc_score_select_sketch_bf16 with an optional device-side region end
int dc_sketch_select_impl(const void *k, const uint8_t *codes, const float *scale, const float *resid, const void *q,
                          uint32_t *idx_out, int64_t idx_unit_stride, int n_b, int n_h, int n_rows, int hd,
                          int64_t sb, int64_t sh, int64_t sr, int64_t cb, int64_t ch, int64_t cr, int q_group,
                          int budget, int mode, int order, int state_ready, void *workspace, size_t workspace_bytes,
                          void *ev_scan_begin, void *ev_scan_end, void *stream, const int32_t *hi_dev, int lo_row);
// attn.hip: dc_gather_attn_bf16 with an optional device-side start of the suffix
int dc_gather_attn_common(const char *who, const void *q, const void *k, const void *v, const uint32_t *idx,
                          const void *new_k, const void *new_v, void *out, float *lse, int n_b, int n_h, int group,
                          int hd, int n_idx, int64_t idx_unit_stride, const uint32_t *n_idx_unit, int64_t region_lo,
                          int n_sink, int64_t recent_lo, int n_recent, const int32_t *n_recent_dev, int64_t ksb,
                          int64_t ksh, int64_t ksr, int64_t vsb, int64_t vsh, int64_t vsr, float scale,
                          void *workspace, size_t workspace_bytes, void *stream, const int32_t *recent_lo_dev);
// small.hip: a whole decode layer in one kernel, for short contexts
bool dc_small_supported(int n_units, int region, int k_eff, int group, int hd, bool has_sketch);
size_t dc_small_workspace_bytes(int n_units, int region, int group, int hd);
size_t dc_small_cand_bytes(int n_units, int region);
int dc_small_state_init(int n_units, int region, void *cand, void *stream);
int dc_small_try(const dc_layer_args *a, int region, int k_eff, void *sel_ws, void *cand, void *attn_ws,
                 size_t attn_ws_bytes, void *stream);
bool dc_ws_state_trusted(const void *workspace);
void dc_ws_state_initialised(const void *workspace);

static inline bool dc_aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
static inline size_t dc_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- device side -----------------------------------------------------------
// 16-byte load of data that is read once (the scans stream gigabytes through the
// caches): the non-temporal hint keeps the lines from displacing what is reused, and the
// streaming kernels reach the plain read rate of the part with it (about 8 % faster).
__device__ __forceinline__ uint4 dc_load_stream16(const void *p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}

// the matching stores, for bulk data that the writing kernel does not read back
__device__ __forceinline__ void dc_store_stream16(void *p, uint4 v) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ void dc_store_stream8(void *p, uint2 v) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 t = {v.x, v.y};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x2 *>(p));
}

__device__ __forceinline__ float dc_bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float dc_bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float dc_bf16_to_f32(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even; NaN -> canonical quiet NaN
__device__ __forceinline__ uint16_t dc_f32_to_bf16(float f) {
    uint32_t b = __float_as_uint(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    uint32_t lsb = (b >> 16) & 1u;
    return (uint16_t)((b + 0x7fffu + lsb) >> 16);
}

// order-preserving map f32 -> u32 (ascending)
__device__ __forceinline__ uint32_t dc_f2ord(float x) {
    uint32_t b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Histogram bucket of a score (larger score = better = smaller bucket), a monotone
// map onto [0, DC_HIST_BINS).  Positive scores from 2^-20 up to 2^20 get 8 buckets
// per binade (the top-k of an attention scan lives there: a finer grid leaves
// fewer rows in the threshold bucket, a coarser one costs the scan fewer histogram
// atomics); smaller positives share the last fine bucket, larger ones the first;
// negative scores get two buckets per binade.
constexpr uint32_t kPosBinades = 40u, kSubBits = 3u;
constexpr uint32_t kPosBuckets = kPosBinades << kSubBits;
__device__ __forceinline__ uint32_t dc_score_bucket(float s) {
    const uint32_t b = __float_as_uint(s + 0.0f);  // -0 -> +0
    const uint32_t mag = b & 0x7fffffffu;
    if (b & 0x80000000u) return kPosBuckets + (mag >> 22);
    constexpr uint32_t lo = (127u - 20u) << 23, hi = ((127u - 20u + kPosBinades) << 23) - 1u;
    const uint32_t m = mag < lo ? lo : (mag > hi ? hi : mag);
    return (kPosBuckets - 1u) - ((m - lo) >> (23u - kSubBits));
}
static_assert(kPosBuckets + 512u <= DC_HIST_BINS, "bucket map exceeds the histogram");

// 32-bit ordering key (smaller = better) and its histogram bucket.  The bucket is
// a monotone function of the key, so equal keys share a bucket.
// DC_MODE_IP:       key = ord(-(s + 0)),            bucket from s
// DC_MODE_REF_DIST: key = ord(d), d = f32(65536-s); bucket from s' = 65536 - d,
//                   which is exact and is s rounded onto d's grid.
__device__ __forceinline__ void dc_key_bucket(float s, int mode, uint32_t &key, uint32_t &bucket) {
    if (mode == DC_MODE_REF_DIST) {
        float d = 65536.0f - s;
        key = dc_f2ord(d);
        bucket = dc_score_bucket(65536.0f - d);
    } else {
        key = dc_f2ord(-(s + 0.0f));
        bucket = dc_score_bucket(s);
    }
}

// Margin of the sketch scan: a row can belong to the exact top-k only if
// approx + margin reaches the k-th largest approx.  e = sum_d |q_d| r_d bounds the
// quantisation error of one score, wabs = sum_d |q_d a_d| scales the fp32 rounding
// of both the approximate and the exact evaluation (128-term dots of values up to
// 127 a_d: below 1.5e-3 wabs together).  In DC_MODE_REF_DIST keys f32(65536 - s)
// of unequal scores can tie, within one ulp of the key: 2^-23 (65536 + |s|).
__device__ __forceinline__ float dc_sketch_margin(float e, float wabs, int mode) {
    const float ep = 1.02f * e + 4.0e-3f * wabs;
    float m = 2.0f * ep;
    if (mode == DC_MODE_REF_DIST) m += (65536.0f + 128.0f * wabs + e) * 4.8e-7f;
    return m;
}

// sum over the 16 lanes of a DPP row; every lane of the row receives the sum
__device__ __forceinline__ float dc_row16_sum(float v) {
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0x141, 0xF, 0xF, true);  // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0x140, 0xF, 0xF, true);  // row_mirror
    return v;
}

// sum over aligned groups of 8 lanes
__device__ __forceinline__ float dc_row8_sum(float v) {
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0xB1, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0x4E, 0xF, 0xF, true);
    v += __builtin_amdgcn_update_dpp(0.0f, v, 0x141, 0xF, 0xF, true);
    return v;
}

// sum over aligned groups of LPR lanes (8, 16 or 32)
template <int LPR>
__device__ __forceinline__ float dc_group_sum(float v) {
    if (LPR == 8) return dc_row8_sum(v);
    v = dc_row16_sum(v);
    if (LPR == 32) v += __shfl_xor(v, 16, 64);
    return v;
}

// Rows of a retrieval region that are live.  The kernels' grids and lists are laid out for
// n_cap rows; with hi_dev the region ends at the row that device word names (it moves up when the
// recent window is rolled over, between replays of a captured step), lo_row being its first row.
__device__ __forceinline__ int dc_live_rows(int n_cap, const int32_t *hi_dev, int lo_row) {
    if (!hi_dev) return n_cap;
    const int v = *hi_dev - lo_row;
    return v < 0 ? 0 : (v < n_cap ? v : n_cap);
}

// 8 bf16 (one 16-byte load) dotted with 8 fp32 query values, added to acc
__device__ __forceinline__ float dc_dot8(const uint4 &w, const float (&q)[8], float acc) {
    acc = fmaf(dc_bf16_lo(w.x), q[0], acc);
    acc = fmaf(dc_bf16_hi(w.x), q[1], acc);
    acc = fmaf(dc_bf16_lo(w.y), q[2], acc);
    acc = fmaf(dc_bf16_hi(w.y), q[3], acc);
    acc = fmaf(dc_bf16_lo(w.z), q[4], acc);
    acc = fmaf(dc_bf16_hi(w.z), q[5], acc);
    acc = fmaf(dc_bf16_lo(w.w), q[6], acc);
    acc = fmaf(dc_bf16_hi(w.w), q[7], acc);
    return acc;
}

// This lane's 8 query values (columns col*8 .. col*8+7) of one unit.  A GQA
// group (q_group > 1) is averaged in fp32 in ascending head order, divided once
// and rounded to bf16, as torch's bf16 mean does (diffcache.py:193).  The loads
// of up to 8 heads are issued together; a serial loop covers larger groups.
template <int HD>
__device__ __forceinline__ void dc_load_query(const uint16_t *__restrict__ Q, int64_t unit,
                                              int q_group, int col, float (&q)[8]) {
    const uint16_t *qp = Q + unit * q_group * HD + col * 8;
    uint4 raw[8];
#pragma unroll
    for (int g = 0; g < 8; ++g) {
        raw[g] = make_uint4(0u, 0u, 0u, 0u);
        if (g < q_group) raw[g] = *reinterpret_cast<const uint4 *>(qp + (int64_t)g * HD);
    }
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
#pragma unroll
    for (int g = 0; g < 8; ++g) {
        if (g < q_group) {
            acc[0] += dc_bf16_lo(raw[g].x);
            acc[1] += dc_bf16_hi(raw[g].x);
            acc[2] += dc_bf16_lo(raw[g].y);
            acc[3] += dc_bf16_hi(raw[g].y);
            acc[4] += dc_bf16_lo(raw[g].z);
            acc[5] += dc_bf16_hi(raw[g].z);
            acc[6] += dc_bf16_lo(raw[g].w);
            acc[7] += dc_bf16_hi(raw[g].w);
        }
    }
    for (int g = 8; g < q_group; ++g) {
        const uint4 r = *reinterpret_cast<const uint4 *>(qp + (int64_t)g * HD);
        acc[0] += dc_bf16_lo(r.x);
        acc[1] += dc_bf16_hi(r.x);
        acc[2] += dc_bf16_lo(r.y);
        acc[3] += dc_bf16_hi(r.y);
        acc[4] += dc_bf16_lo(r.z);
        acc[5] += dc_bf16_hi(r.z);
        acc[6] += dc_bf16_lo(r.w);
        acc[7] += dc_bf16_hi(r.w);
    }
    if (q_group == 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = acc[i];
    } else {
        const float n = (float)q_group;
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = dc_bf16_to_f32(dc_f32_to_bf16(acc[i] / n));
    }
}
