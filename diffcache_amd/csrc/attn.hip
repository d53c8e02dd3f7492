// Decode attention over gathered K/V rows.  Replaces the buffer assembly of
// src/diffcache/kvcache/diffcache.py:196-209 and the flash_attn_with_kvcache
// call of src/diffcache/base.py:134-142: the selected rows are read straight
// from the HBM-resident store instead of being copied into a dense buffer.
//
// Grid: one block per (unit, split); a split is a contiguous slice of the
// unit's attended list [selected | sinks | recent | current token].  Inside a
// block a group of LPR = HD/8 lanes owns one row at a time (one 16-byte load
// per lane covers the row) and the G query heads of the GQA group share every
// row that is loaded.  Three passes over the slice: logits into LDS, a
// block-wide max / exp / sum per head, then the V accumulation without any
// rescaling.  Each split writes (m, l, acc) and merge_kernel combines the
// splits through their log-sum-exp.  Bound by HBM: 2 * HD*2 bytes per row.
#include "dc_common.h"
#include <math.h>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxRowsPerSplit = 512;
constexpr uint32_t kNewToken = 0xffffffffu;
constexpr int kInflight = 4;

struct AttnPlan {
    int rows_per_split;
    int n_splits;
};

AttnPlan plan_attn(int n_units, int n_total) {
    AttnPlan p;
    if (n_total <= 0) {
        p.rows_per_split = 16;
        p.n_splits = 1;
        return p;
    }
    int want = (1024 + n_units - 1) / (n_units > 0 ? n_units : 1);
    if (want < 1) want = 1;
    int rps = (n_total + want - 1) / want;
    if (rps < 16) rps = 16;
    if (rps > kMaxRowsPerSplit) rps = kMaxRowsPerSplit;
    rps = (rps + 15) / 16 * 16;
    p.rows_per_split = rps;
    p.n_splits = (n_total + rps - 1) / rps;
    return p;
}

template <int HD, int G>
__global__ __launch_bounds__(kThreads) void gather_attn_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    const uint32_t *__restrict__ idx, const uint16_t *__restrict__ new_k,
    const uint16_t *__restrict__ new_v, float *__restrict__ ws_acc, float *__restrict__ ws_ml,
    int n_h, int n_idx, int64_t idx_stride, int64_t region_lo, int n_sink, int64_t recent_lo,
    int n_recent, int n_total, int rows_per_split, int n_splits, int64_t ksb, int64_t ksh,
    int64_t ksr, int64_t vsb, int64_t vsh, int64_t vsr, float scale) {
    constexpr int LPR = HD / 8;
    constexpr int NG = kThreads / LPR;  // row groups per block
    __shared__ uint32_t s_rows[kMaxRowsPerSplit];
    __shared__ float s_logit[G][kMaxRowsPerSplit];
    __shared__ float s_red[kWaves][G];
    __shared__ float s_acc[kWaves][G * HD];

    const int unit = blockIdx.x / n_splits;
    const int split = blockIdx.x % n_splits;
    const int b = unit / n_h, h = unit % n_h;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int gid = tid / LPR, col = tid % LPR;

    const int r0 = split * rows_per_split;
    int n = n_total - r0;
    n = n < rows_per_split ? n : rows_per_split;
    n = n < 0 ? 0 : n;

    // ---- pass 0: physical row of every list position of this slice ----
    for (int j = tid; j < n; j += kThreads) {
        const int vj = r0 + j;
        uint32_t row;
        if (vj < n_idx) row = (uint32_t)(region_lo + idx[(int64_t)unit * idx_stride + vj]);
        else if (vj < n_idx + n_sink) row = (uint32_t)(vj - n_idx);
        else if (vj < n_idx + n_sink + n_recent) row = (uint32_t)(recent_lo + (vj - n_idx - n_sink));
        else row = kNewToken;
        s_rows[j] = row;
    }

    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const uint16_t *qp = Q + ((int64_t)unit * G + g) * HD + col * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[g][i] = dc_bf16_to_f32(qp[i]);
    }
    __syncthreads();

    const uint16_t *Ku = K + b * ksb + h * ksh + col * 8;
    const uint16_t *Vu = V + b * vsb + h * vsh + col * 8;
    const uint16_t *nk = new_k ? new_k + (int64_t)unit * HD + col * 8 : nullptr;
    const uint16_t *nv = new_v ? new_v + (int64_t)unit * HD + col * 8 : nullptr;

    // ---- pass 1: scaled logits of every (head, row) into LDS ----
    for (int base = 0; base < n; base += kInflight * NG) {
        uint4 w[kInflight];
#pragma unroll
        for (int t = 0; t < kInflight; ++t) {
            int j = base + t * NG + gid;
            j = j < n ? j : n - 1;
            const uint32_t row = s_rows[j];
            const uint16_t *p = (row == kNewToken) ? nk : Ku + (int64_t)row * ksr;
            w[t] = *reinterpret_cast<const uint4 *>(p);
        }
#pragma unroll
        for (int t = 0; t < kInflight; ++t) {
            const int j = base + t * NG + gid;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float p = dc_group_sum<LPR>(dc_dot8(w[t], qf[g], 0.f));
                if (col == g % LPR && j < n) s_logit[g][j] = p * scale;
            }
        }
    }
    __syncthreads();

    // ---- pass 2: per-head max, exponentials, sum ----
    float m[G], l[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = -INFINITY;
        for (int j = tid; j < n; j += kThreads) v = fmaxf(v, s_logit[g][j]);
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
        if (lane == 0) s_red[wave][g] = v;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float v = s_red[0][g];
#pragma unroll
        for (int w2 = 1; w2 < kWaves; ++w2) v = fmaxf(v, s_red[w2][g]);
        m[g] = v;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float s = 0.f;
        for (int j = tid; j < n; j += kThreads) {
            float p = __expf(s_logit[g][j] - m[g]);
            s_logit[g][j] = p;
            s += p;
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) s += __shfl_xor(s, d, 64);
        if (lane == 0) s_red[wave][g] = s;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float s = s_red[0][g];
#pragma unroll
        for (int w2 = 1; w2 < kWaves; ++w2) s += s_red[w2][g];
        l[g] = s;
    }

    // ---- pass 3: acc[g] += p[g][row] * V[row] ----
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.f;
    for (int base = 0; base < n; base += kInflight * NG) {
        uint4 w[kInflight];
#pragma unroll
        for (int t = 0; t < kInflight; ++t) {
            int j = base + t * NG + gid;
            j = j < n ? j : n - 1;
            const uint32_t row = s_rows[j];
            const uint16_t *p = (row == kNewToken) ? nv : Vu + (int64_t)row * vsr;
            w[t] = *reinterpret_cast<const uint4 *>(p);
        }
#pragma unroll
        for (int t = 0; t < kInflight; ++t) {
            const int j = base + t * NG + gid;
            const bool ok = j < n;
            const int jj = ok ? j : 0;
            float v[8] = {dc_bf16_lo(w[t].x), dc_bf16_hi(w[t].x), dc_bf16_lo(w[t].y),
                          dc_bf16_hi(w[t].y), dc_bf16_lo(w[t].z), dc_bf16_hi(w[t].z),
                          dc_bf16_lo(w[t].w), dc_bf16_hi(w[t].w)};
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float p = ok ? s_logit[g][jj] : 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p, v[i], acc[g][i]);
            }
        }
    }

    // ---- reduce over the row groups: inside the wave, then across waves ----
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] += __shfl_xor(acc[g][i], off, 64);
    if (lane < LPR) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 8; ++i) s_acc[wave][g * HD + col * 8 + i] = acc[g][i];
    }
    __syncthreads();
    const int64_t slot = (int64_t)unit * n_splits + split;
    for (int o = tid; o < G * HD; o += kThreads) {
        float s = s_acc[0][o];
#pragma unroll
        for (int w2 = 1; w2 < kWaves; ++w2) s += s_acc[w2][o];
        ws_acc[slot * (G * HD) + o] = s;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if (tid == g) {
            ws_ml[(slot * G + g) * 2 + 0] = m[g];
            ws_ml[(slot * G + g) * 2 + 1] = l[g];
        }
    }
}

// out[u, g, :] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s
__global__ void merge_kernel(const float *__restrict__ ws_acc, const float *__restrict__ ws_ml,
                             uint16_t *__restrict__ out, float *__restrict__ lse, int group, int hd,
                             int n_splits) {
    const int ug = blockIdx.x;  // unit * group + g
    const int unit = ug / group, g = ug % group;
    float M = -INFINITY;
    for (int s = 0; s < n_splits; ++s)
        M = fmaxf(M, ws_ml[(((int64_t)unit * n_splits + s) * group + g) * 2]);
    float L = 0.f;
    for (int s = 0; s < n_splits; ++s) {
        const float *ml = ws_ml + (((int64_t)unit * n_splits + s) * group + g) * 2;
        if (ml[1] > 0.f) L += __expf(ml[0] - M) * ml[1];
    }
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float a = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const int64_t slot = (int64_t)unit * n_splits + s;
            const float *ml = ws_ml + (slot * group + g) * 2;
            if (ml[1] > 0.f) a += __expf(ml[0] - M) * ws_acc[(slot * group + g) * hd + d];
        }
        out[(int64_t)ug * hd + d] = dc_f32_to_bf16(L > 0.f ? a / L : 0.f);
    }
    if (lse && threadIdx.x == 0) lse[ug] = L > 0.f ? M + logf(L) : -INFINITY;
}

template <int HD>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ V, const uint32_t *__restrict__ idx,
    uint16_t *__restrict__ out_k, uint16_t *__restrict__ out_v, int n_h, int n_idx,
    int64_t idx_stride, int64_t row_offset, int64_t ssb, int64_t ssh, int64_t ssr, int64_t dsb,
    int64_t dsh, int64_t dsr, int blocks_per_unit) {
    constexpr int LPR = HD / 8;
    constexpr int NG = 256 / LPR;
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int gid = threadIdx.x / LPR, col = threadIdx.x % LPR;
    const int j = chunk * NG + gid;
    if (j >= n_idx) return;
    const int64_t r = row_offset + idx[(int64_t)unit * idx_stride + j];
    const int64_t src = b * ssb + h * ssh + r * ssr + col * 8;
    const int64_t dst = b * dsb + h * dsh + (int64_t)j * dsr + col * 8;
    if (out_k) *reinterpret_cast<uint4 *>(out_k + dst) = *reinterpret_cast<const uint4 *>(K + src);
    if (out_v) *reinterpret_cast<uint4 *>(out_v + dst) = *reinterpret_cast<const uint4 *>(V + src);
}

template <int HD>
int launch_attn(int group, dim3 grid, hipStream_t st, const uint16_t *q, const uint16_t *k,
                const uint16_t *v, const uint32_t *idx, const uint16_t *new_k,
                const uint16_t *new_v, float *ws_acc, float *ws_ml, int n_h, int n_idx,
                int64_t idx_stride, int64_t region_lo, int n_sink, int64_t recent_lo, int n_recent,
                int n_total, AttnPlan plan, int64_t ksb, int64_t ksh, int64_t ksr, int64_t vsb,
                int64_t vsh, int64_t vsr, float scale) {
#define DC_ATTN_CASE(GG)                                                                           \
    case GG:                                                                                       \
        hipLaunchKernelGGL((gather_attn_kernel<HD, GG>), grid, dim3(kThreads), 0, st, q, k, v, idx, \
                           new_k, new_v, ws_acc, ws_ml, n_h, n_idx, idx_stride, region_lo, n_sink, \
                           recent_lo, n_recent, n_total, plan.rows_per_split, plan.n_splits, ksb,  \
                           ksh, ksr, vsb, vsh, vsr, scale);                                        \
        return 0;
    switch (group) {
        DC_ATTN_CASE(1)
        DC_ATTN_CASE(2)
        DC_ATTN_CASE(3)
        DC_ATTN_CASE(4)
        DC_ATTN_CASE(5)
        DC_ATTN_CASE(6)
        DC_ATTN_CASE(7)
        DC_ATTN_CASE(8)
    }
#undef DC_ATTN_CASE
    return -1;
}

}  // namespace

// Upper bound of plan_attn(n_units, n).n_splits over every n <= n_total, so that a
// workspace sized for the longest attended list also serves shorter ones.
static int max_splits(int n_units, int n_total) {
    int want = (1024 + n_units - 1) / (n_units > 0 ? n_units : 1);
    int by_cap = (n_total + kMaxRowsPerSplit - 1) / kMaxRowsPerSplit;
    int m = want > by_cap ? want : by_cap;
    return m < 1 ? 1 : m;
}

extern "C" size_t dc_attn_workspace_bytes(int n_units, int group, int hd, int n_rows_attended) {
    if (n_units <= 0 || group <= 0 || hd <= 0) return 256;
    size_t slots = (size_t)n_units * max_splits(n_units, n_rows_attended);
    return dc_align_up(slots * group * hd * 4, 256) + dc_align_up(slots * group * 2 * 4, 256);
}

extern "C" int dc_gather_attn_bf16(const void *q, const void *k, const void *v, const uint32_t *idx,
                                   const void *new_k, const void *new_v, void *out, float *lse,
                                   int n_b, int n_h, int group, int hd, int n_idx,
                                   int64_t idx_unit_stride, int64_t region_lo, int n_sink,
                                   int64_t recent_lo, int n_recent, int64_t ksb, int64_t ksh,
                                   int64_t ksr, int64_t vsb, int64_t vsh, int64_t vsr, float scale,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    DC_REQUIRE(q && k && v && out, "dc_gather_attn_bf16: null pointer");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_idx >= 0 && n_sink >= 0 && n_recent >= 0,
               "dc_gather_attn_bf16: bad sizes");
    DC_REQUIRE(n_idx == 0 || idx, "dc_gather_attn_bf16: idx is null but n_idx > 0");
    DC_REQUIRE((new_k == nullptr) == (new_v == nullptr),
               "dc_gather_attn_bf16: new_k and new_v must both be set or both be null");
    DC_REQUIRE(group >= 1 && group <= 8, "dc_gather_attn_bf16: group %d not in [1,8]", group);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "dc_gather_attn_bf16: head_dim %d unsupported", hd);
    DC_REQUIRE(dc_aligned16(k) && dc_aligned16(v) && dc_aligned16(q) &&
                   (!new_k || (dc_aligned16(new_k) && dc_aligned16(new_v))),
               "dc_gather_attn_bf16: pointers must be 16-byte aligned");
    DC_REQUIRE(ksb % 8 == 0 && ksh % 8 == 0 && ksr % 8 == 0 && vsb % 8 == 0 && vsh % 8 == 0 &&
                   vsr % 8 == 0,
               "dc_gather_attn_bf16: strides must be multiples of 8 elements");
    DC_REQUIRE(idx_unit_stride >= n_idx, "dc_gather_attn_bf16: idx_unit_stride < n_idx");
    DC_REQUIRE(region_lo >= 0 && recent_lo >= 0 && recent_lo + n_recent < 0xffffffffll,
               "dc_gather_attn_bf16: row numbers out of range");
    const int n_units = n_b * n_h;
    if (n_units == 0) return DC_OK;
    const int n_total = n_idx + n_sink + n_recent + (new_k ? 1 : 0);
    AttnPlan plan = plan_attn(n_units, n_total);
    const size_t slots = (size_t)n_units * plan.n_splits;
    const size_t need = dc_align_up(slots * group * hd * 4, 256) + dc_align_up(slots * group * 2 * 4, 256);
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "dc_gather_attn_bf16: workspace must be non-null and 256-byte aligned");
    if (workspace_bytes < need) {
        dc_set_error("dc_gather_attn_bf16: workspace %zu bytes < %zu needed", workspace_bytes, need);
        return DC_ENOMEM;
    }
    float *ws_acc = (float *)workspace;
    float *ws_ml = (float *)((char *)workspace + dc_align_up(slots * group * hd * 4, 256));
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)slots);
    int rc;
    const uint16_t *q16 = (const uint16_t *)q, *k16 = (const uint16_t *)k, *v16 = (const uint16_t *)v;
    const uint16_t *nk16 = (const uint16_t *)new_k, *nv16 = (const uint16_t *)new_v;
    if (hd == 64)
        rc = launch_attn<64>(group, grid, st, q16, k16, v16, idx, nk16, nv16, ws_acc, ws_ml, n_h, n_idx,
                             idx_unit_stride, region_lo, n_sink, recent_lo, n_recent, n_total, plan,
                             ksb, ksh, ksr, vsb, vsh, vsr, scale);
    else if (hd == 128)
        rc = launch_attn<128>(group, grid, st, q16, k16, v16, idx, nk16, nv16, ws_acc, ws_ml, n_h,
                              n_idx, idx_unit_stride, region_lo, n_sink, recent_lo, n_recent, n_total,
                              plan, ksb, ksh, ksr, vsb, vsh, vsr, scale);
    else
        rc = launch_attn<256>(group, grid, st, q16, k16, v16, idx, nk16, nv16, ws_acc, ws_ml, n_h,
                              n_idx, idx_unit_stride, region_lo, n_sink, recent_lo, n_recent, n_total,
                              plan, ksb, ksh, ksr, vsb, vsh, vsr, scale);
    DC_REQUIRE(rc == 0, "dc_gather_attn_bf16: unsupported group %d", group);
    DC_CHECK_LAUNCH("dc_gather_attn_bf16(attn)");
    hipLaunchKernelGGL(merge_kernel, dim3((unsigned)(n_units * group)), dim3(hd < 256 ? hd : 256), 0,
                       st, ws_acc, ws_ml, (uint16_t *)out, lse, group, hd, plan.n_splits);
    DC_CHECK_LAUNCH("dc_gather_attn_bf16(merge)");
    return DC_OK;
}

extern "C" int dc_gather_rows_bf16(const void *k, const void *v, const uint32_t *idx, void *out_k,
                                   void *out_v, int n_b, int n_h, int n_idx,
                                   int64_t idx_unit_stride, int hd, int64_t row_offset, int64_t ssb,
                                   int64_t ssh, int64_t ssr, int64_t dsb, int64_t dsh, int64_t dsr,
                                   void *stream) {
    DC_REQUIRE(idx && (out_k || out_v), "dc_gather_rows_bf16: null pointer");
    DC_REQUIRE((!out_k || k) && (!out_v || v), "dc_gather_rows_bf16: source missing for an output");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_idx >= 0, "dc_gather_rows_bf16: bad sizes");
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "dc_gather_rows_bf16: head_dim %d unsupported", hd);
    DC_REQUIRE((!k || dc_aligned16(k)) && (!v || dc_aligned16(v)) && (!out_k || dc_aligned16(out_k)) &&
                   (!out_v || dc_aligned16(out_v)),
               "dc_gather_rows_bf16: pointers must be 16-byte aligned");
    DC_REQUIRE(ssb % 8 == 0 && ssh % 8 == 0 && ssr % 8 == 0 && dsb % 8 == 0 && dsh % 8 == 0 &&
                   dsr % 8 == 0,
               "dc_gather_rows_bf16: strides must be multiples of 8 elements");
    DC_REQUIRE(idx_unit_stride >= n_idx, "dc_gather_rows_bf16: idx_unit_stride < n_idx");
    const int64_t n_units = (int64_t)n_b * n_h;
    if (n_units == 0 || n_idx == 0) return DC_OK;
    const int ng = 256 / (hd / 8);
    const int64_t bpu = (n_idx + ng - 1) / ng;
    dim3 grid((unsigned)(n_units * bpu));
    hipStream_t st = (hipStream_t)stream;
#define DC_LAUNCH_GR(HD)                                                                           \
    hipLaunchKernelGGL(gather_rows_kernel<HD>, grid, dim3(256), 0, st, (const uint16_t *)k,        \
                       (const uint16_t *)v, idx, (uint16_t *)out_k, (uint16_t *)out_v, n_h, n_idx, \
                       idx_unit_stride, row_offset, ssb, ssh, ssr, dsb, dsh, dsr, (int)bpu)
    if (hd == 64) DC_LAUNCH_GR(64);
    else if (hd == 128) DC_LAUNCH_GR(128);
    else DC_LAUNCH_GR(256);
#undef DC_LAUNCH_GR
    DC_CHECK_LAUNCH("dc_gather_rows_bf16");
    return DC_OK;
}
