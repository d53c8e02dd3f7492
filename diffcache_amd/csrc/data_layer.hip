// Host-side mirror of the reference's data layer (struct DataLayer,
// diffcache_cpu/src/lib.rs:189-197, with new 292-327, prefill 329-347, insert 352-369
// and query 373-404) for callers that are not Python: a handle that keeps the
// bookkeeping the Rust struct keeps (shape, capacity, context length) over device
// buffers the caller owns, and turns each of its methods into calls of the kernels'
// entry points.  Nothing here allocates device memory or synchronises.
//
// Differences from the reference that a caller sees: one handle covers all
// bsz x kv_heads units (the reference holds one Index per unit and fans out with
// rayon); errors come back as negative codes where the reference panics; the scan is
// always the exact one (use_bruteforce); a context shorter than ef is not an error.
#include "dc_common.h"
#include <new>

struct dc_data_layer {
    int bsz, kv_heads, hd, mode, use_sketch;
    int64_t n_max;    // rows per unit the store can hold (max_ctx_len, lib.rs:297)
    int64_t ctx_len;  // rows held (lib.rs:196)
    // device buffers, bound by the caller
    uint16_t *k, *v;
    uint8_t *codes;
    float *scale, *resid;
    uint32_t *idx;
    void *ws;
    size_t ws_bytes;
    int max_ef;
    int bound;
};

namespace {

int64_t units_of(const dc_data_layer *dl) { return (int64_t)dl->bsz * dl->kv_heads; }

// element strides of the (bsz, kv_heads, n_max, hd) store and byte strides of the codes
void strides_of(const dc_data_layer *dl, int64_t *sb, int64_t *sh, int64_t *sr) {
    *sr = dl->hd;
    *sh = dl->n_max * dl->hd;
    *sb = (int64_t)dl->kv_heads * *sh;
}

}  // namespace

extern "C" int dc_data_layer_create(dc_data_layer **out, int bsz, int kv_heads, int hd, int64_t max_ctx_len,
                                    int mode, int use_sketch) {
    const char *who = "dc_data_layer_create";
    DC_REQUIRE(out, "%s: null pointer", who);
    *out = nullptr;
    DC_REQUIRE(bsz >= 1 && kv_heads >= 1, "%s: bad sizes", who);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d not in {64,128,256}", who, hd);
    DC_REQUIRE(max_ctx_len >= 1 && max_ctx_len < (1ll << 31), "%s: max_ctx_len out of range", who);
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "%s: bad mode %d", who, mode);
    DC_REQUIRE((int64_t)bsz * kv_heads < (1 << 20), "%s: too many units", who);
    dc_data_layer *dl = new (std::nothrow) dc_data_layer();
    if (!dl) {
        dc_set_error("%s: out of host memory", who);
        return DC_ENOMEM;
    }
    dl->bsz = bsz;
    dl->kv_heads = kv_heads;
    dl->hd = hd;
    dl->mode = mode;
    dl->use_sketch = use_sketch ? 1 : 0;
    dl->n_max = max_ctx_len;
    dl->ctx_len = 0;
    dl->bound = 0;
    *out = dl;
    return DC_OK;
}

extern "C" void dc_data_layer_destroy(dc_data_layer *dl) { delete dl; }

extern "C" int64_t dc_data_layer_ctx_len(const dc_data_layer *dl) { return dl ? dl->ctx_len : -1; }

extern "C" int dc_data_layer_sizes(const dc_data_layer *dl, int max_ef, size_t *store_bytes, size_t *codes_bytes,
                                   size_t *scale_bytes, size_t *idx_bytes, size_t *workspace_bytes) {
    const char *who = "dc_data_layer_sizes";
    DC_REQUIRE(dl && store_bytes && codes_bytes && scale_bytes && idx_bytes && workspace_bytes,
               "%s: null pointer", who);
    DC_REQUIRE(max_ef >= 1, "%s: max_ef must be positive", who);
    const size_t nu = (size_t)units_of(dl);
    *store_bytes = nu * (size_t)dl->n_max * dl->hd * 2;               // each of K and V
    *codes_bytes = dl->use_sketch ? nu * (size_t)dl->n_max * dl->hd : 0;
    *scale_bytes = dl->use_sketch ? nu * (size_t)dl->hd * 4 : 0;      // each of scale and resid
    *idx_bytes = nu * (size_t)max_ef * 4;
    // the sketch route and the bf16 route share one workspace layout
    *workspace_bytes = dc_sketch_select_workspace_bytes((int)nu, (int)dl->n_max, max_ef);
    return DC_OK;
}

extern "C" int dc_data_layer_bind(dc_data_layer *dl, void *k_store, void *v_store, void *codes, void *scale,
                                  void *resid, void *idx, void *workspace, size_t workspace_bytes, int max_ef) {
    const char *who = "dc_data_layer_bind";
    DC_REQUIRE(dl && k_store && v_store && idx && workspace, "%s: null pointer", who);
    DC_REQUIRE(!dl->use_sketch || (codes && scale && resid), "%s: the sketch buffers are missing", who);
    DC_REQUIRE(max_ef >= 1, "%s: max_ef must be positive", who);
    DC_REQUIRE(dc_aligned16(k_store) && dc_aligned16(v_store) && dc_aligned16(idx) &&
                   (!dl->use_sketch || (dc_aligned16(codes) && dc_aligned16(scale) && dc_aligned16(resid))),
               "%s: buffers must be 16-byte aligned", who);
    DC_REQUIRE((((uintptr_t)workspace) & 255u) == 0, "%s: workspace must be 256-byte aligned", who);
    const size_t need = dc_sketch_select_workspace_bytes((int)units_of(dl), (int)dl->n_max, max_ef);
    if (workspace_bytes < need) {
        dc_set_error("%s: workspace %zu bytes < %zu needed", who, workspace_bytes, need);
        return DC_ENOMEM;
    }
    dl->k = (uint16_t *)k_store;
    dl->v = (uint16_t *)v_store;
    dl->codes = (uint8_t *)codes;
    dl->scale = (float *)scale;
    dl->resid = (float *)resid;
    dl->idx = (uint32_t *)idx;
    dl->ws = workspace;
    dl->ws_bytes = workspace_bytes;
    dl->max_ef = max_ef;
    dl->bound = 1;
    return DC_OK;
}

// lib.rs:329-347: keys, vals (bsz, kv_heads, n_rows, hd) bf16, host or device memory
// true for a pointer the runtime does not know: ordinary (pageable) host memory
static bool pageable_host(const void *p) {
    hipPointerAttribute_t attr;
    const hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();  // older runtimes report an unknown pointer as an error
        return true;
    }
    return attr.type == hipMemoryTypeUnregistered;
}

extern "C" int dc_data_layer_prefill(dc_data_layer *dl, const void *keys, const void *vals, int64_t n_rows,
                                     void *stream) {
    const char *who = "dc_data_layer_prefill";
    DC_REQUIRE(dl && dl->bound, "%s: no buffers bound", who);
    DC_REQUIRE(keys && vals, "%s: null pointer", who);
    DC_REQUIRE(n_rows >= 0 && n_rows <= dl->n_max, "%s: %lld rows do not fit max_ctx_len %lld", who,
               (long long)n_rows, (long long)dl->n_max);
    hipStream_t st = (hipStream_t)stream;
    int64_t sb, sh, sr;
    strides_of(dl, &sb, &sh, &sr);
    if (n_rows > 0) {
        // one strided copy per tensor: unit u's rows are contiguous on both sides
        const size_t width = (size_t)n_rows * dl->hd * 2, height = (size_t)units_of(dl);
        hipError_t e = hipMemcpy2DAsync(dl->k, (size_t)sh * 2, keys, width, width, height, hipMemcpyDefault, st);
        if (e == hipSuccess)
            e = hipMemcpy2DAsync(dl->v, (size_t)sh * 2, vals, width, width, height, hipMemcpyDefault, st);
        // A source in pageable host memory (not allocated by HIP) cannot be read by the copy
        // engine behind the caller's back: the runtime stages it, and the caller may free or
        // reuse it as soon as this call returns only if the copy is complete by then.
        if (e == hipSuccess && (pageable_host(keys) || pageable_host(vals))) e = hipStreamSynchronize(st);
        if (e != hipSuccess) {
            dc_set_error("%s: copy failed: %s", who, hipGetErrorString(e));
            return DC_ELAUNCH;
        }
        if (dl->use_sketch) {
            const int rc = dc_sketch_build_bf16(dl->k, dl->codes, dl->scale, dl->resid, dl->bsz, dl->kv_heads,
                                                (int)n_rows, dl->hd, sb, sh, sr, sb, sh, sr, 0, stream);
            if (rc) return rc;
        }
    }
    dl->ctx_len = n_rows;
    return DC_OK;
}

// lib.rs:352-369: keys, vals (bsz, kv_heads, hd) bf16 in device memory; one token per unit
extern "C" int dc_data_layer_insert(dc_data_layer *dl, const void *keys, const void *vals, void *stream) {
    const char *who = "dc_data_layer_insert";
    DC_REQUIRE(dl && dl->bound, "%s: no buffers bound", who);
    DC_REQUIRE(keys && vals, "%s: null pointer", who);
    DC_REQUIRE(dl->ctx_len < dl->n_max, "%s: the store is full (%lld rows)", who, (long long)dl->n_max);
    int64_t sb, sh, sr;
    strides_of(dl, &sb, &sh, &sr);
    int rc = dc_append_kv_bf16(dl->k, dl->v, keys, vals, dl->bsz, dl->kv_heads, dl->hd, dl->ctx_len, nullptr,
                               dl->n_max, sb, sh, sr, stream);
    if (rc) return rc;
    if (dl->use_sketch) {
        // the first row fits the scales; later rows keep them and can only raise the residual bounds
        const int64_t pos = dl->ctx_len;
        rc = dc_sketch_build_bf16(dl->k + pos * sr, dl->codes + pos * sr, dl->scale, dl->resid, dl->bsz,
                                  dl->kv_heads, 1, dl->hd, sb, sh, sr, sb, sh, sr, pos > 0 ? 1 : 0, stream);
        if (rc) return rc;
    }
    dl->ctx_len += 1;
    return DC_OK;
}

// lib.rs:373-404: queries (bsz, kv_heads, hd); the min(ef, ctx_len) best K and V rows of
// every unit, best first (nsw.rs:621-629), into out_keys / out_vals (bsz, kv_heads,
// out_rows, hd) in device memory.  Returns the number of rows written per unit in *n_out.
extern "C" int dc_data_layer_query(dc_data_layer *dl, void *out_keys, void *out_vals, int64_t out_rows,
                                   const void *queries, int ef, int *n_out, void *stream) {
    const char *who = "dc_data_layer_query";
    if (n_out) *n_out = 0;
    DC_REQUIRE(dl && dl->bound, "%s: no buffers bound", who);
    DC_REQUIRE(out_keys && out_vals && queries, "%s: null pointer", who);
    DC_REQUIRE(ef >= 0 && ef <= dl->max_ef, "%s: ef %d outside [0, max_ef %d]", who, ef, dl->max_ef);
    DC_REQUIRE(dc_aligned16(out_keys) && dc_aligned16(out_vals) && dc_aligned16(queries),
               "%s: pointers must be 16-byte aligned", who);
    const int ef_eff = (int64_t)ef < dl->ctx_len ? ef : (int)dl->ctx_len;   // lib.rs:374
    DC_REQUIRE(out_rows >= ef_eff, "%s: out buffers hold %lld rows per unit, %d needed", who,
               (long long)out_rows, ef_eff);
    if (ef_eff == 0) return DC_OK;
    int64_t sb, sh, sr;
    strides_of(dl, &sb, &sh, &sr);
    const int n_rows = (int)dl->ctx_len;
    int rc;
    if (dl->use_sketch)
        rc = dc_score_select_sketch_bf16(dl->k, dl->codes, dl->scale, dl->resid, queries, dl->idx, dl->max_ef,
                                         dl->bsz, dl->kv_heads, n_rows, dl->hd, sb, sh, sr, sb, sh, sr, 1,
                                         ef_eff, dl->mode, DC_ORDER_BEST, 0, dl->ws, dl->ws_bytes, nullptr,
                                         nullptr, stream);
    else
        rc = dc_score_select_bf16(dl->k, queries, dl->idx, dl->max_ef, dl->bsz, dl->kv_heads, n_rows, dl->hd,
                                  sb, sh, sr, 1, ef_eff, dl->mode, DC_ORDER_BEST, dl->ws, dl->ws_bytes, stream);
    if (rc) return rc;
    rc = dc_gather_rows_bf16(dl->k, dl->v, dl->idx, out_keys, out_vals, dl->bsz, dl->kv_heads, ef_eff,
                             dl->max_ef, dl->hd, 0, sb, sh, sr, (int64_t)dl->kv_heads * out_rows * dl->hd,
                             out_rows * dl->hd, dl->hd, stream);
    if (rc) return rc;
    if (n_out) *n_out = ef_eff;
    return DC_OK;
}
