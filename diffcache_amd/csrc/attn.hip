// Decode attention over gathered K/V rows.  Replaces the buffer assembly of
// src/diffcache/kvcache/diffcache.py:196-209 and the flash_attn_with_kvcache
// call of src/diffcache/base.py:134-142: the selected rows are read straight
// from the HBM-resident store instead of being copied into a dense buffer.
//
// Grid: one block per (unit, split); a split is a slice of rows_per_group * NG
// consecutive positions of the unit's attended list [selected | sinks | recent |
// current token] (128 rows at head_dim 128 and a GQA group of 4).  A group of LPR = HD/8 lanes owns one
// row at a time (one 16-byte load per lane covers the row) and the G query heads
// of the GQA group share every row that is loaded.  All K and V rows of the
// slice are requested up front (one memory round trip after the id lookup), the
// logits stay in registers, the block agrees on a per-head maximum, and each
// split leaves (m, l, acc) in the workspace; merge_kernel combines the splits
// through their log-sum-exp.  (Merging in the last block to arrive was tried:
// the device-scope fence it needs costs far more than a second launch here.)
// Bound by HBM: 2 * HD*2 bytes per row.
#include "dc_attn.h"
#include <cstdlib>
#include <mutex>

namespace {

constexpr int kThreads = kAttnThreads;

template <int HD, int G>
__global__ __launch_bounds__(kThreads) void gather_attn_kernel(AttnArgs a) {
    __shared__ float s_mem[attn_shared_floats<HD, G>()];
    AttnShared sh;
    sh.red = s_mem;
    sh.l = s_mem + kAttnWaves * G;
    sh.acc = s_mem + 2 * kAttnWaves * G;
    dc_attn_split<HD, G>(a, blockIdx.x / a.n_splits, blockIdx.x % a.n_splits, sh);
}

// The same split on the matrix cores (dc_attn_split_mfma); the group is a run-time value here
// because the products are padded to 16 heads anyway.
template <int HD>
__global__ __launch_bounds__(kThreads) void gather_attn_mfma_kernel(AttnArgs a, int group) {
    extern __shared__ float s_dyn[];
    // Split-major: a grid a little larger than what the device holds at once (config 3: 1088
    // blocks on 1024 places) then ends on every unit's last, partial split instead of on the last
    // units' full ones.
    const int n_units = (int)(gridDim.x / (unsigned)a.n_splits);
    dc_attn_split_mfma<HD>(a, group, blockIdx.x % n_units, blockIdx.x / n_units, s_dyn);
}

// out[u, g, :] = sum_s w_s acc_s / sum_s w_s l_s with w_s = exp(m_s - max m): one block
// per (unit, head), one thread per output column.
__global__ __launch_bounds__(256) void merge_kernel(const float *__restrict__ ws_acc,
                                                    const float *__restrict__ ws_ml,
                                                    uint16_t *__restrict__ out, float *__restrict__ lse,
                                                    int group, int hd, int n_splits) {
    __shared__ float s_w[256];
    __shared__ float s_red[4];
    const int ug = blockIdx.x;  // unit * group + g
    const int unit = ug / group, g = ug % group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const float *ml = ws_ml + ((int64_t)unit * n_splits * group + g) * 2;  // split s at ml + s*group*2
    float acc = 0.f, M = -INFINITY, L = 0.f;
    // splits are folded in chunks of at most blockDim.x with a running maximum
    for (int s0 = 0; s0 < n_splits; s0 += blockDim.x) {
        const int sp = s0 + tid;
        float m = -INFINITY, l = 0.f;
        if (sp < n_splits) {
            m = ml[(int64_t)sp * group * 2];
            l = ml[(int64_t)sp * group * 2 + 1];
            if (!(l > 0.f)) m = -INFINITY;
        }
        float cm = m;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) cm = fmaxf(cm, __shfl_xor(cm, d, 64));
        if (lane == 0) s_red[wave] = cm;
        __syncthreads();
        cm = s_red[0];
        for (int w = 1; w < nw; ++w) cm = fmaxf(cm, s_red[w]);
        __syncthreads();
        const float Mn = fmaxf(M, cm);
        const float rescale = (M > -INFINITY) ? __expf(M - Mn) : 0.f;
        const float w = (m > -INFINITY) ? __expf(m - Mn) : 0.f;
        s_w[tid] = w;
        float cl = w * l;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) cl += __shfl_xor(cl, d, 64);
        if (lane == 0) s_red[wave] = cl;
        __syncthreads();
        cl = s_red[0];
        for (int w2 = 1; w2 < nw; ++w2) cl += s_red[w2];
        L = L * rescale + cl;
        acc *= rescale;
        M = Mn;
        const int cnt = (n_splits - s0) < (int)blockDim.x ? (n_splits - s0) : (int)blockDim.x;
        for (int d = tid; d < hd; d += blockDim.x) {
            // every thread owns one column when hd <= blockDim.x (the launch guarantees it)
            float a = 0.f;
            const float *pa = ws_acc + (((int64_t)unit * n_splits + s0) * group + g) * hd + d;
#pragma unroll 8
            for (int j = 0; j < cnt; ++j) a = fmaf(s_w[j], pa[(int64_t)j * group * hd], a);
            acc += a;
        }
        __syncthreads();
    }
    if (tid < hd) out[(int64_t)ug * hd + tid] = dc_f32_to_bf16(L > 0.f ? acc / L : 0.f);
    if (lse && tid == 0) lse[ug] = L > 0.f ? M + logf(L) : -INFINITY;
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
int launch_attn(int group, dim3 grid, hipStream_t st, const AttnArgs &a) {
#define DC_ATTN_CASE(GG)                                                                      \
    case GG:                                                                                  \
        hipLaunchKernelGGL((gather_attn_kernel<HD, GG>), grid, dim3(kThreads), 0, st, a);      \
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

// Which split body a call runs.  The matrix-core version takes any group up to 16; the VALU
// version (groups up to 8) stays for comparison: DIFFCACHE_ATTN_VALU=1 in the environment of the
// process (read once) selects it wherever it applies.
static bool attn_use_mfma(int group, int64_t max_row, int64_t ksr, int64_t vsr) {
    static const bool valu = [] {
        const char *e = std::getenv("DIFFCACHE_ATTN_VALU");
        return e && e[0] == '1' && e[1] == 0;
    }();
    if (group > 8) return true;
    if (valu) return false;
    // rows are addressed with 32-bit byte offsets from the unit's first row
    const int64_t sr = ksr > vsr ? ksr : vsr;
    return (max_row + 1) * sr * 2 <= 0xffffffffll;
}

extern "C" size_t dc_attn_workspace_bytes(int n_units, int group, int hd, int n_rows_attended) {
    if (n_units <= 0 || group <= 0 || hd < 8) return 256;
    // room for either split body (the slices of the VALU version are shorter for large groups)
    const size_t a = carve_attn(nullptr, n_units, group, hd, plan_attn(hd, group, n_rows_attended, false).n_splits).bytes;
    const size_t b = carve_attn(nullptr, n_units, group, hd, plan_attn(hd, group, n_rows_attended, true).n_splits).bytes;
    return a > b ? a : b;
}

// Argument checks and the two launches shared by dc_gather_attn_bf16 (caller's workspace),
// dc_gather_attn_static_bf16 (the library's static scratch array) and dc_decode_layer.
// recent_lo_dev: null, or a device word holding the first row of the suffix at the time the
// kernels run (recent_lo is then its largest value).
int dc_gather_attn_common(const char *who, const void *q, const void *k, const void *v, const uint32_t *idx,
                       const void *new_k, const void *new_v, void *out, float *lse, int n_b, int n_h,
                       int group, int hd, int n_idx, int64_t idx_unit_stride, const uint32_t *n_idx_unit,
                       int64_t region_lo, int n_sink, int64_t recent_lo, int n_recent,
                       const int32_t *n_recent_dev, int64_t ksb, int64_t ksh, int64_t ksr, int64_t vsb,
                       int64_t vsh, int64_t vsr, float scale, void *workspace, size_t workspace_bytes,
                       void *stream, const int32_t *recent_lo_dev) {
    DC_REQUIRE(q && k && v && out, "%s: null pointer", who);
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_idx >= 0 && n_sink >= 0 && n_recent >= 0,
               "%s: bad sizes", who);
    DC_REQUIRE(n_idx == 0 || idx, "%s: idx is null but n_idx > 0", who);
    DC_REQUIRE((new_k == nullptr) == (new_v == nullptr),
               "%s: new_k and new_v must both be set or both be null", who);
    DC_REQUIRE(group >= 1 && group <= kMfmaMaxGroup, "%s: group %d not in [1,%d]", who, group, kMfmaMaxGroup);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d unsupported", who, hd);
    DC_REQUIRE(dc_aligned16(k) && dc_aligned16(v) && dc_aligned16(q) &&
                   (!new_k || (dc_aligned16(new_k) && dc_aligned16(new_v))),
               "%s: pointers must be 16-byte aligned", who);
    DC_REQUIRE(ksb % 8 == 0 && ksh % 8 == 0 && ksr % 8 == 0 && vsb % 8 == 0 && vsh % 8 == 0 &&
                   vsr % 8 == 0,
               "%s: strides must be multiples of 8 elements", who);
    DC_REQUIRE(idx_unit_stride >= n_idx, "%s: idx_unit_stride < n_idx", who);
    DC_REQUIRE(region_lo >= 0 && recent_lo >= 0 && recent_lo + n_recent < 0xffffffffll,
               "%s: row numbers out of range", who);
    const int n_units = n_b * n_h;
    if (n_units == 0) return DC_OK;
    const int n_total = n_idx + n_sink + n_recent + (new_k ? 1 : 0);
    DC_REQUIRE(workspace && (((uintptr_t)workspace) & 255u) == 0,
               "%s: workspace must be non-null and 256-byte aligned", who);
    const bool mfma = attn_use_mfma(group, recent_lo + n_recent, ksr, vsr);
    DC_REQUIRE(mfma || group <= 8, "%s: group %d needs rows within 4 GiB of the unit's first row", who, group);
    const AttnPlan plan = plan_attn(hd, group, n_total, mfma);
    const AttnWs w = carve_attn(workspace, n_units, group, hd, plan.n_splits);
    if (workspace_bytes < w.bytes) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, workspace_bytes, w.bytes);
        return DC_ENOMEM;
    }
    DC_REQUIRE((int64_t)n_units * plan.n_splits < (1ll << 31), "%s: grid too large", who);
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)((size_t)n_units * plan.n_splits));
    AttnArgs aa;
    aa.Q = (const uint16_t *)q;
    aa.K = (const uint16_t *)k;
    aa.V = (const uint16_t *)v;
    aa.idx = idx;
    aa.new_k = (const uint16_t *)new_k;
    aa.new_v = (const uint16_t *)new_v;
    aa.ws_acc = w.acc;
    aa.ws_ml = w.ml;
    aa.n_idx_unit = n_idx_unit;
    aa.n_recent_dev = n_recent_dev;
    aa.recent_lo_dev = recent_lo_dev;
    aa.n_h = n_h;
    aa.n_idx = n_idx;
    aa.idx_stride = idx_unit_stride;
    aa.region_lo = region_lo;
    aa.n_sink = n_sink;
    aa.recent_lo = recent_lo;
    aa.n_recent = n_recent;
    aa.n_total = n_total;
    aa.n_splits = plan.n_splits;
    aa.ksb = ksb, aa.ksh = ksh, aa.ksr = ksr, aa.vsb = vsb, aa.vsh = vsh, aa.vsr = vsr;
    aa.scale = scale;
    uint16_t *o16 = (uint16_t *)out;
    int rc = 0;
    if (mfma) {
        const size_t lds = mfma_shared_bytes(hd, group);
        if (hd == 64) hipLaunchKernelGGL(gather_attn_mfma_kernel<64>, grid, dim3(kThreads), lds, st, aa, group);
        else if (hd == 128) hipLaunchKernelGGL(gather_attn_mfma_kernel<128>, grid, dim3(kThreads), lds, st, aa, group);
        else hipLaunchKernelGGL(gather_attn_mfma_kernel<256>, grid, dim3(kThreads), lds, st, aa, group);
    } else if (hd == 64) rc = launch_attn<64>(group, grid, st, aa);
    else if (hd == 128) rc = launch_attn<128>(group, grid, st, aa);
    else rc = launch_attn<256>(group, grid, st, aa);
    DC_REQUIRE(rc == 0, "%s: unsupported group %d", who, group);
    DC_CHECK_LAUNCH(who);
    hipLaunchKernelGGL(merge_kernel, dim3((unsigned)(n_units * group)), dim3(hd), 0, st, w.acc, w.ml, o16,
                       lse, group, hd, plan.n_splits);
    DC_CHECK_LAUNCH(who);
    return DC_OK;
}

namespace {

// Scratch of the allocation-free entry point: the per-split (m, l, acc) partials.  One copy
// per GPU, held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address is looked up once per device and kept.
constexpr size_t kStaticScratchBytes = (size_t)DC_ATTN_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

}  // namespace

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

extern "C" int dc_gather_attn_bf16(const void *q, const void *k, const void *v, const uint32_t *idx,
                                   const void *new_k, const void *new_v, void *out, float *lse,
                                   int n_b, int n_h, int group, int hd, int n_idx,
                                   int64_t idx_unit_stride, const uint32_t *n_idx_unit,
                                   int64_t region_lo, int n_sink,
                                   int64_t recent_lo, int n_recent, const int32_t *n_recent_dev,
                                   int64_t ksb, int64_t ksh,
                                   int64_t ksr, int64_t vsb, int64_t vsh, int64_t vsr, float scale,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    return dc_gather_attn_common("dc_gather_attn_bf16", q, k, v, idx, new_k, new_v, out, lse, n_b, n_h, group,
                                 hd, n_idx, idx_unit_stride, n_idx_unit, region_lo, n_sink, recent_lo,
                                 n_recent, n_recent_dev, ksb, ksh, ksr, vsb, vsh, vsr, scale, workspace, workspace_bytes,
                                 stream, nullptr);
}

extern "C" int dc_gather_attn_static_bf16(const void *q, const void *k, const void *v, const uint32_t *idx,
                                          const void *new_k, const void *new_v, void *out, float *lse,
                                          int n_b, int n_h, int group, int hd, int n_idx,
                                          int64_t idx_unit_stride, const uint32_t *n_idx_unit,
                                          int64_t region_lo, int n_sink, int64_t recent_lo, int n_recent,
                                          const int32_t *n_recent_dev, int64_t ksb, int64_t ksh, int64_t ksr, int64_t vsb, int64_t vsh,
                                          int64_t vsr, float scale, void *stream) {
    const char *who = "dc_gather_attn_static_bf16";
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && group >= 1 && group <= kMfmaMaxGroup && n_idx >= 0 && n_sink >= 0 && n_recent >= 0,
               "%s: bad sizes", who);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d unsupported", who, hd);
    const int64_t n_units = (int64_t)n_b * n_h;
    DC_REQUIRE(n_units < (1 << 20), "%s: too many units", who);
    const int64_t n_total = (int64_t)n_idx + n_sink + n_recent + (new_k ? 1 : 0);
    DC_REQUIRE(n_total < (1ll << 31), "%s: too many rows", who);
    const size_t need = dc_attn_workspace_bytes((int)n_units, group, hd, (int)n_total);
    if (need > kStaticScratchBytes) {
        dc_set_error("%s: %lld units x %lld attended rows (group %d, head_dim %d) need %zu bytes of scratch; "
                     "the static scratch holds %zu (use dc_gather_attn_bf16 with a workspace)",
                     who, (long long)n_units, (long long)n_total, group, hd, need, kStaticScratchBytes);
        return DC_ENOMEM;
    }
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        dc_set_error("%s: no current device (or device number >= %d)", who, kMaxDevices);
        return DC_EINVAL;
    }
    void *ptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ptr = g_scratch_ptr[dev];
        if (!ptr) {
            // once per device, with that device current: every GPU has its own copy of the array
            const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !ptr) {
                dc_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev,
                             hipGetErrorString(e));
                return DC_ELAUNCH;
            }
            g_scratch_ptr[dev] = ptr;
        }
    }
    // Every split slot the merge reads is written by the attention kernel of the same call, so
    // nothing has to start at zero; the contents of the previous call are simply overwritten.
    return dc_gather_attn_common(who, q, k, v, idx, new_k, new_v, out, lse, n_b, n_h, group, hd, n_idx,
                                 idx_unit_stride, n_idx_unit, region_lo, n_sink, recent_lo, n_recent, n_recent_dev,
                                 ksb, ksh, ksr, vsb, vsh, vsr, scale, ptr, kStaticScratchBytes, stream, nullptr);
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
