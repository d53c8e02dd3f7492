// Error plumbing, version, and the fused per-layer call chain of the C ABI.
#include "dc_common.h"
#include <vector>
#include "dc_fused.h"
#include <stdarg.h>
#include <string.h>

static thread_local char g_err[512] = "";
static thread_local int g_last_route = DC_ROUTE_ATTEND_ONLY;

void dc_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" int dc_version(void) { return DC_VERSION; }

extern "C" const char *dc_last_error(void) { return g_err; }

extern "C" int dc_last_route(void) { return g_last_route; }

namespace {

__global__ void fill_zero_kernel(uint32_t *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

struct LayerWs {
    uint32_t *hist;
    void *topk;
    size_t topk_bytes;
    void *attn;
    size_t attn_bytes;
    void *small_cand;  // candidate lists of the one-kernel route (shapes it can take only)
    size_t bytes;
};

LayerWs carve_layer(void *base, int n_units, int n_region, int budget, int group, int hd,
                    int n_attended) {
    LayerWs w;
    char *p = (char *)base;
    size_t off = 0;
    w.hist = (uint32_t *)(p + off);
    off += dc_align_up((size_t)(n_units > 0 ? n_units : 0) * DC_HIST_BINS * 4, 256);
    w.topk = p + off;
    {   // room for any select path: dense scores + dc_topk_select, or a streaming one
        size_t a = dc_topk_workspace_bytes(n_units, n_region, budget);
        size_t b = dc_sketch_select_workspace_bytes(n_units, n_region, budget);
        w.topk_bytes = dc_align_up(a > b ? a : b, 256);
    }
    off += w.topk_bytes;
    w.attn = p + off;
    {   // split partials of the attention kernels, or of the one-kernel route for short contexts
        size_t a = dc_attn_workspace_bytes(n_units, group, hd, n_attended);
        size_t b = dc_small_workspace_bytes(n_units, n_region, group, hd);
        w.attn_bytes = dc_align_up(a > b ? a : b, 256);
    }
    off += w.attn_bytes;
    w.small_cand = p + off;
    off += dc_small_cand_bytes(n_units, n_region);
    w.bytes = off;
    return w;
}

}  // namespace

extern "C" size_t dc_layer_workspace_bytes(int n_units, int n_region_rows, int budget, int group,
                                           int hd, int n_rows_attended) {
    return carve_layer(nullptr, n_units, n_region_rows, budget, group, hd, n_rows_attended).bytes;
}

extern "C" int dc_decode_layer(const dc_layer_args *a, void *stream) {
    DC_REQUIRE(a, "dc_decode_layer: null args");
    DC_REQUIRE(a->q && a->k && a->v && a->out && a->idx_out, "dc_decode_layer: null pointer in args");
    DC_REQUIRE(a->n_b >= 0 && a->n_h >= 1 && a->group >= 1 && a->n_sink >= 0 && a->n_recent >= 0 &&
                   a->budget >= 0,
               "dc_decode_layer: bad sizes");
    DC_REQUIRE(!(a->sketch_codes && a->scores), "dc_decode_layer: the sketch path needs scores == NULL");
    DC_REQUIRE(a->recent_lo >= a->n_sink, "dc_decode_layer: recent_lo %lld < n_sink %d",
               (long long)a->recent_lo, a->n_sink);
    DC_REQUIRE(!(a->region_hi_dev && a->scores), "dc_decode_layer: region_hi_dev needs scores == NULL");
    const int n_units = a->n_b * a->n_h;
    if (n_units == 0) return DC_OK;
    const int64_t region64 = a->recent_lo - a->n_sink;
    DC_REQUIRE(region64 < (1ll << 31), "dc_decode_layer: region too long");
    const int region = (int)region64;
    const int k_eff = a->budget < region ? a->budget : region;
    const int has_new = a->new_k ? 1 : 0;
    const int attended = k_eff + a->n_sink + a->n_recent + has_new;
    DC_REQUIRE(a->workspace && (((uintptr_t)a->workspace) & 255u) == 0,
               "dc_decode_layer: workspace must be non-null and 256-byte aligned");
    LayerWs w = carve_layer(a->workspace, n_units, region, a->budget, a->group, a->hd, attended);
    if (a->workspace_bytes < w.bytes) {
        dc_set_error("dc_decode_layer: workspace %zu bytes < %zu needed", a->workspace_bytes, w.bytes);
        return DC_ENOMEM;
    }
    hipStream_t st = (hipStream_t)stream;
    int rc;
    const uint16_t *k_region = (const uint16_t *)a->k + (int64_t)a->n_sink * a->kv_row_stride;
    // The caller's word that the select state is ready counts unless a kernel of the one-kernel
    // route has reported a failure since this workspace was last initialised.
    int ready = a->select_state_ready;
    if (k_eff > 0 && !a->scores) {
        if (ready && !dc_ws_state_trusted(a->workspace)) ready = 0;
        if (!ready) dc_ws_state_initialised(a->workspace);
    }
    g_last_route = k_eff <= 0 ? DC_ROUTE_ATTEND_ONLY
                              : (a->scores ? DC_ROUTE_DENSE
                                           : (a->sketch_codes && region <= DC_SKETCH_MAX_ROWS ? DC_ROUTE_SKETCH
                                                                                             : DC_ROUTE_STREAM));
    if (k_eff > 0 && !a->scores && a->order == DC_ORDER_ANY && !a->region_hi_dev &&
        dc_small_supported(n_units, region, k_eff, a->group, a->hd, a->sketch_codes != nullptr)) {
        // short context: the whole layer in one kernel whose blocks are all resident (ids in no
        // particular order); reads the bf16 keys, with or without a sketch.  The state is set up
        // for this route even when the call is sent down the chain below (another launch of the
        // kernel is in flight on another stream, or the stream is being captured): the next call
        // with these sizes may take the kernel and be told that the state is ready.
        if (!ready) {
            rc = dc_select_state_init(n_units, region, a->budget, w.topk, w.topk_bytes, stream);
            if (rc) return rc;
            rc = dc_small_state_init(n_units, region, w.small_cand, stream);
            if (rc) return rc;
            ready = 1;
        }
        if (a->ev_scan_begin) (void)hipEventRecord((hipEvent_t)a->ev_scan_begin, st);
        rc = dc_small_try(a, region, k_eff, w.topk, w.small_cand, w.attn, w.attn_bytes, stream);
        if (rc < 0) return rc;
        if (rc == 1) {
            if (a->ev_scan_end) (void)hipEventRecord((hipEvent_t)a->ev_scan_end, st);
            g_last_route = DC_ROUTE_ONE_KERNEL;
            return DC_OK;
        }
    }
    if (k_eff > 0 && !a->scores && a->sketch_codes && region <= DC_SKETCH_MAX_ROWS) {
        // streaming select over the 8-bit sketch, exact rescoring of the kept rows
        DC_REQUIRE(a->sketch_scale && a->sketch_resid, "dc_decode_layer: sketch_scale / sketch_resid missing");
        rc = dc_sketch_select_impl(
            k_region, a->sketch_codes + (int64_t)a->n_sink * a->sketch_row_stride, a->sketch_scale,
            a->sketch_resid, a->q, a->idx_out, a->idx_unit_stride, a->n_b, a->n_h, region, a->hd,
            a->kv_batch_stride, a->kv_head_stride, a->kv_row_stride, a->sketch_batch_stride,
            a->sketch_head_stride, a->sketch_row_stride, a->group, a->budget, a->mode, a->order,
            ready, w.topk, w.topk_bytes, a->ev_scan_begin, a->ev_scan_end, stream, a->region_hi_dev, a->n_sink);
        if (rc) return rc;
    } else if (k_eff > 0 && !a->scores) {
        // no dense scores wanted: streaming score + select
        if (!ready) {
            rc = dc_select_state_init(n_units, region, a->budget, w.topk, w.topk_bytes, stream);
            if (rc) return rc;
        }
        if (a->ev_scan_begin) (void)hipEventRecord((hipEvent_t)a->ev_scan_begin, st);
        rc = dc_score_prune_launch(k_region, a->q, a->n_b, a->n_h, region, a->hd, a->kv_batch_stride,
                                   a->kv_head_stride, a->kv_row_stride, a->group, a->budget, a->mode, w.topk,
                                   w.topk_bytes, stream, a->region_hi_dev, a->n_sink);
        if (rc) return rc;
        if (a->ev_scan_end) (void)hipEventRecord((hipEvent_t)a->ev_scan_end, st);
        rc = dc_sparse_select(a->idx_out, a->idx_unit_stride, n_units, region, a->budget, a->mode, a->order,
                              1, w.topk, w.topk_bytes, stream);
        if (rc) return rc;
    } else if (k_eff > 0) {
        const int64_t n = (int64_t)n_units * DC_HIST_BINS;
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                           w.hist, n);
        DC_CHECK_LAUNCH("dc_decode_layer(zero)");
        if (a->ev_scan_begin) (void)hipEventRecord((hipEvent_t)a->ev_scan_begin, st);
        rc = dc_score_bf16(k_region, a->q, a->scores, w.hist, a->n_b, a->n_h, region, a->hd,
                           a->kv_batch_stride, a->kv_head_stride, a->kv_row_stride,
                           a->scores_unit_stride, a->group, a->mode, stream);
        if (rc) return rc;
        if (a->ev_scan_end) (void)hipEventRecord((hipEvent_t)a->ev_scan_end, st);
        rc = dc_topk_select(a->scores, a->scores_unit_stride, a->idx_out, a->idx_unit_stride, n_units,
                            region, a->budget, a->mode, a->order, w.hist, w.topk, w.topk_bytes, stream);
        if (rc) return rc;
    }
    rc = dc_gather_attn_common("dc_decode_layer", a->q, a->k, a->v, a->idx_out, a->new_k, a->new_v, a->out, a->lse,
                               a->n_b, a->n_h, a->group, a->hd, k_eff, a->idx_unit_stride, nullptr, a->n_sink,
                               a->n_sink, a->recent_lo, a->n_recent, a->n_recent_dev, a->kv_batch_stride,
                               a->kv_head_stride, a->kv_row_stride, a->kv_batch_stride, a->kv_head_stride,
                               a->kv_row_stride, a->scale, w.attn, w.attn_bytes, stream, a->region_hi_dev);
    return rc;
}

extern "C" int dc_decode_layer_route(const dc_layer_args *a) {
    DC_REQUIRE(a, "dc_decode_layer_route: null args");
    const int n_units = a->n_b * a->n_h;
    const int64_t region64 = a->recent_lo - a->n_sink;
    DC_REQUIRE(n_units >= 0 && region64 >= 0 && region64 < (1ll << 31), "dc_decode_layer_route: bad sizes");
    const int region = (int)region64;
    const int k_eff = a->budget < region ? a->budget : region;
    if (n_units == 0 || k_eff <= 0) return DC_ROUTE_ATTEND_ONLY;
    if (a->scores) return DC_ROUTE_DENSE;
    if (a->order == DC_ORDER_ANY && a->one_kernel != DC_ONE_KERNEL_NEVER && !a->region_hi_dev &&
        dc_small_supported(n_units, region, k_eff, a->group, a->hd, a->sketch_codes != nullptr))
        return DC_ROUTE_ONE_KERNEL;
    return a->sketch_codes && region <= DC_SKETCH_MAX_ROWS ? DC_ROUTE_SKETCH : DC_ROUTE_STREAM;
}

extern "C" int dc_decode_layer_status(const dc_layer_args *a, void *stream) {
    DC_REQUIRE(a && a->workspace, "dc_decode_layer_status: null args or workspace");
    const int n_units = a->n_b * a->n_h;
    if (n_units <= 0) return DC_OK;
    const int region = (int)(a->recent_lo - a->n_sink);
    const int k_eff = a->budget < region ? a->budget : region;
    const LayerWs w = carve_layer(a->workspace, n_units, region, a->budget, a->group, a->hd,
                                  k_eff + a->n_sink + a->n_recent + (a->new_k ? 1 : 0));
    DC_REQUIRE(a->workspace_bytes >= w.bytes, "dc_decode_layer_status: workspace too small");
    const FusedWs f = carve_fused(w.topk, n_units, region, a->budget);
    std::vector<uint32_t> err((size_t)n_units, 0u);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = hipMemcpy2DAsync(err.data(), sizeof(uint32_t), &f.state[0].sync_err, sizeof(UnitState),
                                    sizeof(uint32_t), (size_t)n_units, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) {
        dc_set_error("dc_decode_layer_status: %s", hipGetErrorString(e));
        return DC_ELAUNCH;
    }
    for (int u = 0; u < n_units; ++u)
        if (err[(size_t)u]) {
            dc_set_error("dc_decode_layer_status: unit %d gave up a bounded wait between its blocks", u);
            return DC_EDEVICE;
        }
    return DC_OK;
}
