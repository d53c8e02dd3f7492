/*
 * diffcache_hip.h -- C ABI of libdiffcache_hip.so: the decode-time retrieval
 * path of DiffCache on one MI355X (gfx950), K/V resident in HBM as bf16.
 *
 * Every entry point
 *   - takes plain device pointers, sizes and element strides (no torch types);
 *   - enqueues its kernels on `stream` (a hipStream_t passed as void*) and
 *     returns without synchronising; nothing is allocated or freed, so the
 *     calls can sit between the two captured graph halves of a decode layer;
 *   - returns 0 on success or a negative DC_E* code, with a message kept for
 *     dc_last_error() (the reference panics instead: lib.rs:294,332,353,376,579).
 *
 * bf16 crosses the boundary as raw 16-bit words, as in the reference
 * (diffcache_cpu/src/lib.rs:529-544).  A "unit" is one (batch, kv-head) pair:
 * the reference keeps one independent index per unit (lib.rs:189-197,296-313).
 * Row r of unit (b, h) of a K or V store starts at element
 *   b * batch_stride + h * head_stride + r * row_stride
 * with head_dim contiguous bf16 values; all strides are in elements, must be
 * multiples of 8 and the base pointers 16-byte aligned.
 *
 * Paths in comments are relative to the reference checkout.
 */
#ifndef DIFFCACHE_HIP_H
#define DIFFCACHE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DC_VERSION 1

/* ordering-key modes */
#define DC_MODE_IP 0       /* highest inner product first, ties -> lower index */
#define DC_MODE_REF_DIST 1 /* order by f32(65536 - ip) as nsw.rs:138 does, ties -> lower index */

/* order of the selected ids */
#define DC_ORDER_ANY 0    /* unspecified (fastest) */
#define DC_ORDER_BEST 1   /* ascending (key, id): the order nsw.rs:621-629 writes rows in */
#define DC_ORDER_INDEX 2  /* ascending id */

/* error codes */
#define DC_OK 0
#define DC_EINVAL (-22)
#define DC_ENOMEM (-12)   /* workspace too small */
#define DC_ELAUNCH (-5)   /* hipLaunchKernel failed */
#define DC_EDEVICE (-6)   /* a kernel gave up a bounded wait: the outputs of that call are not valid */

#define DC_HIST_BINS 1024 /* histogram bins per unit used by the select */
#define DC_SKETCH_MAX_ROWS (1 << 22) /* rows of a unit the sketch scan takes (its lists name a row in 22 bits) */

/* Library version (DC_VERSION).  Replaces nothing; added for binding checks. */
int dc_version(void);

/* Message of the last failing call on this thread ("" if none).
 * Replaces the Rust panic text surfaced as PanicException (lib.rs:294-579). */
const char *dc_last_error(void);

/*
 * GQA-group mean query, rounded to bf16.
 * q (n_units, group, hd) bf16 -> q_mean (n_units, hd) bf16: fp32 sum over the
 * group, one division, round to nearest even.
 * Replaces src/diffcache/kvcache/diffcache.py:191-194 (view(b,Hkv,G,hd).mean(2)).
 */
int dc_group_mean_bf16(const void *q, void *q_mean, int n_units, int group, int hd, void *stream);

/*
 * Inner-product scores of one query per unit against n_rows key rows.
 *   k       first row to score of unit (0,0)
 *   q       (n_b*n_h, q_group, hd) bf16.  q_group == 1: the query itself;
 *           q_group > 1: the GQA group, averaged as dc_group_mean_bf16 does
 *   scores  out, fp32, unit u at scores + u*scores_unit_stride, n_rows each
 *   hist    NULL, or (n_b*n_h, DC_HIST_BINS) uint32 zeroed by the caller: receives
 *           the coarse histogram of the ordering keys that dc_topk_select needs
 * Products of bf16 values are exact in fp32; accumulation is fp32.
 * Replaces Index::distance(QKDist) over the scan of search_bruteforce
 * (diffcache_cpu/src/nsw.rs:129-139,601-607; simsimd dot, lib.rs:65-69).
 */
int dc_score_bf16(const void *k, const void *q, float *scores, uint32_t *hist, int n_b, int n_h,
                  int n_rows, int hd, int64_t k_batch_stride, int64_t k_head_stride,
                  int64_t k_row_stride, int64_t scores_unit_stride, int q_group, int mode,
                  void *stream);

/* Bytes of workspace dc_topk_select needs for these sizes. */
size_t dc_topk_workspace_bytes(int n_units, int n_rows, int k);

/*
 * Exact top-k of each unit's scores: the min(k, n_rows) smallest
 * (ordering key, id) pairs, where the key is given by `mode`.
 *   idx_out (n_units, idx_unit_stride) uint32: ids in [0, n_rows); the first
 *           min(k, n_rows) entries of each unit are written, in `order`
 *   hist    NULL (computed here) or the histogram dc_score_bf16 filled
 *   workspace  dc_topk_workspace_bytes(...) bytes, 256-byte aligned
 * Replaces the bounded max-heap scan and ascending collect of
 * search_bruteforce (diffcache_cpu/src/nsw.rs:600-621), the u64 key packing
 * (nsw.rs:74-91) and the kept-set semantic of DualHeap (dualheap.rs:4-87).
 */
int dc_topk_select(const float *scores, int64_t scores_unit_stride, uint32_t *idx_out,
                   int64_t idx_unit_stride, int n_units, int n_rows, int k, int mode, int order,
                   const uint32_t *hist, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Streaming score + exact top-k without a dense score array: the same ids as
 * dc_score_bf16 followed by dc_topk_select (identical arithmetic), for callers
 * that do not want the scores.  The scan writes only the rows that can still
 * reach the top-k, which matters because HBM writes are far dearer than reads
 * on this part.  Arguments as in dc_score_bf16 / dc_topk_select; `budget` is k.
 * Three steps that may also be called one by one on the same workspace:
 *   dc_select_state_init   clears the per-unit histogram and counters
 *   dc_score_prune_bf16    the scan (the HBM-bound kernel)
 *   dc_sparse_select       exact selection among the surviving rows; with reinit != 0
 *                          it also leaves the workspace as dc_select_state_init does, so
 *                          the next dc_score_prune_bf16 of the same sizes on it needs no
 *                          init call
 * Replaces the same reference code as the two calls it stands for
 * (diffcache_cpu/src/nsw.rs:129-139,600-621).
 */
size_t dc_score_select_workspace_bytes(int n_units, int n_rows, int budget);
int dc_select_state_init(int n_units, int n_rows, int budget, void *workspace,
                         size_t workspace_bytes, void *stream);
int dc_score_prune_bf16(const void *k, const void *q, int n_b, int n_h, int n_rows, int hd,
                        int64_t k_batch_stride, int64_t k_head_stride, int64_t k_row_stride,
                        int q_group, int budget, int mode, void *workspace, size_t workspace_bytes,
                        void *stream);
int dc_sparse_select(uint32_t *idx_out, int64_t idx_unit_stride, int n_units, int n_rows, int budget,
                     int mode, int order, int reinit, void *workspace, size_t workspace_bytes,
                     void *stream);
int dc_score_select_bf16(const void *k, const void *q, uint32_t *idx_out, int64_t idx_unit_stride,
                         int n_b, int n_h, int n_rows, int hd, int64_t k_batch_stride,
                         int64_t k_head_stride, int64_t k_row_stride, int q_group, int budget,
                         int mode, int order, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same selection from an 8-bit sketch of the keys: half the HBM bytes of the
 * bf16 scan, identical ids.  The sketch of a store is one byte per key element
 * plus, per unit and channel d, a scale a_d and a residual bound r_d with
 *   k[i, d] = a_d * (codes[i, d] - 128) + e,  |e| <= r_d  for every sketched row.
 * dc_score_select_sketch_bf16 scans the codes, keeps every row whose approximate
 * score plus a margin derived from q, a, r and the fp32 rounding of both
 * evaluations can still reach the k-th best, recomputes the exact fp32 score of
 * those rows from the bf16 keys with the arithmetic of dc_score_bf16, and selects
 * among them as dc_sparse_select does: the result is the exact top-k of the bf16
 * keys (ties -> lower index) whatever the data; only the running time depends on
 * how well the sketch fits.  No counterpart in the reference, whose exact scan
 * (diffcache_cpu/src/nsw.rs:592-630) reads every key; same results as that scan.
 *
 *   dc_sketch_build_bf16   sketches rows [0, n_rows) of every unit starting at `k`
 *     (pass pointers to the first row to sketch; codes has its own byte strides,
 *     multiples of 16, base 16-byte aligned; scale and resid are (n_b*n_h, hd) fp32).
 *     keep_scale == 0: scales are fitted to these rows (per-channel max / 127) and
 *     the residual bounds start from zero -- call it on the whole region at prefill.
 *     keep_scale != 0: the existing scales are used (values outside their range are
 *     clamped) and the residual bounds are raised where needed -- call it on rows
 *     appended later (replaces nothing in the reference; goes with lib.rs:352-369).
 *   dc_score_select_sketch_bf16   arguments as dc_score_select_bf16 plus the sketch; n_rows at most
 *     DC_SKETCH_MAX_ROWS (dc_decode_layer streams the bf16 keys of a longer region instead);
 *     state_ready as in dc_layer_args.select_state_ready; the optional event pair is
 *     recorded around the scan of the codes.
 */
int dc_sketch_build_bf16(const void *k, uint8_t *codes, float *scale, float *resid, int n_b, int n_h,
                         int n_rows, int hd, int64_t k_batch_stride, int64_t k_head_stride,
                         int64_t k_row_stride, int64_t c_batch_stride, int64_t c_head_stride,
                         int64_t c_row_stride, int keep_scale, void *stream);
size_t dc_sketch_select_workspace_bytes(int n_units, int n_rows, int budget);
int dc_sketch_select_state_init(int n_units, int n_rows, int budget, void *workspace,
                                size_t workspace_bytes, void *stream);
int dc_score_select_sketch_bf16(const void *k, const uint8_t *codes, const float *scale,
                                const float *resid, const void *q, uint32_t *idx_out,
                                int64_t idx_unit_stride, int n_b, int n_h, int n_rows, int hd,
                                int64_t k_batch_stride, int64_t k_head_stride, int64_t k_row_stride,
                                int64_t c_batch_stride, int64_t c_head_stride, int64_t c_row_stride,
                                int q_group, int budget, int mode, int order, int state_ready,
                                void *workspace, size_t workspace_bytes, void *ev_scan_begin,
                                void *ev_scan_end, void *stream);

/*
 * Copy selected K and V rows into dense output buffers.
 * For unit (b, h) and j < n_idx:
 *   out_k[b, h, j, :] = k[b, h, row_offset + idx[u, j], :]   (same for v)
 * idx unit u = b*n_h + h at idx + u*idx_unit_stride.
 * Replaces the row gather of search_bruteforce (nsw.rs:621-629) together with
 * the pinned-buffer hop and H2D copies of
 * src/diffcache/kvcache/diffcache.py:196-209.
 */
int dc_gather_rows_bf16(const void *k, const void *v, const uint32_t *idx, void *out_k, void *out_v,
                        int n_b, int n_h, int n_idx, int64_t idx_unit_stride, int hd,
                        int64_t row_offset, int64_t src_batch_stride, int64_t src_head_stride,
                        int64_t src_row_stride, int64_t dst_batch_stride, int64_t dst_head_stride,
                        int64_t dst_row_stride, void *stream);

/* Bytes of workspace dc_gather_attn_bf16 needs. */
size_t dc_attn_workspace_bytes(int n_units, int group, int hd, int n_rows_attended);

/*
 * Decode attention over a gathered set of rows, for the `group` query heads
 * that share each kv-head.  For unit (b, h) the attended rows are
 *   region_lo + idx[u, j]        j < n_idx     (the retrieved rows)
 *   [0, n_sink)                                 (prefix, always kept)
 *   [recent_lo, recent_lo + n_recent)           (suffix, always kept)
 *   new_k/new_v[u, :]            if not NULL    (the current token)
 * q, out: (n_b, n_h*group, hd) bf16, query head h*group + g belongs to kv-head h.
 * out = softmax(q . K^T * scale) . V, fp32 softmax and accumulation, bf16 out;
 * lse (n_b, n_h*group) fp32 log-sum-exp of the scaled logits, or NULL.
 * n_idx_unit: NULL, or (n_b*n_h) uint32: unit u attends only to its first
 * min(n_idx_unit[u], n_idx) retrieved rows (the output of dc_kcheck_f32 on ids in
 * DC_ORDER_BEST order); the always-kept rows are unaffected.
 * n_recent_dev: NULL, or one int32 in device memory holding the current length of the
 * suffix: the kernels then attend to min(*n_recent_dev, n_recent) suffix rows and n_recent
 * is the capacity that sizes the launch and the workspace.  This is what keeps a call that
 * was captured in a graph valid on later replays, as the cache_seqlens tensor does for
 * flash_attn_with_kvcache (src/diffcache/base.py:134-142,150-152); dc_step_advance moves it.
 * Replaces flash_attn_with_kvcache over the assembled buffer
 * (src/diffcache/base.py:134-142) and the buffer assembly it reads
 * (src/diffcache/kvcache/diffcache.py:48-66,186-209).
 */
int dc_gather_attn_bf16(const void *q, const void *k, const void *v, const uint32_t *idx,
                        const void *new_k, const void *new_v, void *out, float *lse, int n_b,
                        int n_h, int group, int hd, int n_idx, int64_t idx_unit_stride,
                        const uint32_t *n_idx_unit, int64_t region_lo, int n_sink, int64_t recent_lo,
                        int n_recent, const int32_t *n_recent_dev, int64_t k_batch_stride,
                        int64_t k_head_stride, int64_t k_row_stride, int64_t v_batch_stride,
                        int64_t v_head_stride, int64_t v_row_stride, float scale, void *workspace,
                        size_t workspace_bytes, void *stream);

/*
 * dc_gather_attn_bf16 for callers that cannot allocate device memory or bring a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * the same kernels, the same arguments without `workspace`, the same results bit for
 * bit.  The per-split softmax partials live in a static device array of
 * DC_ATTN_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the
 * process ends); a call that needs more -- dc_attn_workspace_bytes(n_b*n_h, group, hd,
 * n_idx + n_sink + n_recent + 1) -- returns DC_ENOMEM and launches nothing.  The call
 * allocates and frees nothing.  All calls on one GPU share the array: calls that overlap
 * on one GPU (two streams, two threads) race; order them on one stream.  The array's
 * device address is looked up on the first call on each device (a runtime query, no
 * allocation); make that first call outside graph capture.
 * No counterpart in the reference, which always allocates through torch.
 */
#define DC_ATTN_STATIC_SCRATCH_BYTES (32u << 20)
int dc_gather_attn_static_bf16(const void *q, const void *k, const void *v, const uint32_t *idx,
                               const void *new_k, const void *new_v, void *out, float *lse, int n_b,
                               int n_h, int group, int hd, int n_idx, int64_t idx_unit_stride,
                               const uint32_t *n_idx_unit, int64_t region_lo, int n_sink,
                               int64_t recent_lo, int n_recent, const int32_t *n_recent_dev,
                               int64_t k_batch_stride, int64_t k_head_stride, int64_t k_row_stride,
                               int64_t v_batch_stride, int64_t v_head_stride, int64_t v_row_stride,
                               float scale, void *stream);

/*
 * k-check (diffcache_cpu/src/nsw.rs:198-296): how many of a unit's best rows are
 * worth attending to.  scores (n_units, scores_unit_stride) fp32: the exact scores of
 * the n_sel selected rows, best first (dc_score_gathered_bf16 on ids in DC_ORDER_BEST
 * order).  The logit of a row is (65536 - f32(65536 - score)) / sqrt(hd) as in
 * nsw.rs:282-286 (score / sqrt(hd) in DC_MODE_IP).  For each size H of k_check_seq
 * (a host array of at most 16 ints), in order, while H < n_sel: a power law is
 * fitted to the logits of ranks 5..H (nsw.rs:198-241), the share of the softmax mass
 * held by the top H is estimated (nsw.rs:243-278), and the first H whose share
 * reaches attn_mass_threshold is written to n_eff[u]; if none does, n_eff[u] = n_sel.
 * alpha_out, mass_out: NULL or (n_units, n_seq) fp32, NaN where a size was not
 * evaluated or the reference returns None.  The reference only reports the outcome
 * of the check (nsw.rs:367-379); feeding n_eff to dc_gather_attn_bf16 is what acts
 * on it.
 */
int dc_kcheck_f32(const float *scores, int64_t scores_unit_stride, int n_units, int n_sel, int hd,
                  int mode, const int *k_check_seq, int n_seq, float attn_mass_threshold,
                  uint32_t *n_eff, float *alpha_out, float *mass_out, void *stream);

/*
 * Append one token: k_store[b, h, row, :] = new_k[b, h, :] (same for v), row = pos, or
 * pos + *pos_dev when pos_dev (one int32 in device memory) is not NULL -- the position
 * then moves with the device-side step count, so a captured call stays valid across
 * replays.  Rows outside [0, pos_end) are never written (pos itself must be inside).
 * new_k/new_v (n_b, n_h, hd) contiguous.
 * Replaces DataLayer::insert / Index::insert's row write
 * (diffcache_cpu/src/lib.rs:352-369, nsw.rs:551-557); no graph is built.
 */
int dc_append_kv_bf16(void *k_store, void *v_store, const void *new_k, const void *new_v, int n_b,
                      int n_h, int hd, int64_t pos, const int32_t *pos_dev, int64_t pos_end,
                      int64_t batch_stride, int64_t head_stride, int64_t row_stride, void *stream);

/*
 * *counter = clamp(*counter + delta, 0, limit), enqueued on `stream` (one thread).  The
 * device-side step count that dc_append_kv_bf16 (pos_dev) and the attention entry points
 * (n_recent_dev) read: advance it once per decoded token, after the last layer, as the
 * reference advances kvbuf_suffix_len (src/diffcache/kvcache/diffcache.py:221-223) and
 * its cache_seqlens (src/diffcache/base.py:150-152).
 */
int dc_step_advance(int32_t *counter, int delta, int limit, void *stream);

/*
 * The whole per-sequence step state as four device words, for a decode step that is captured
 * once and replayed for the whole generation (the reference captures its per-layer graphs once,
 * src/diffcache/base.py:46-55,116-148, and its data layer takes every decoded token as it comes,
 * diffcache_cpu/src/lib.rs:352-369):
 *   n_recent    rows of the recent window        -> n_recent_dev of the attention / layer calls
 *   region_hi   first row of the recent window = end of the retrieval region
 *                                                 -> dc_layer_args.region_hi_dev
 *   append_pos  region_hi + n_recent             -> pos_dev of dc_append_kv_bf16 (with pos = 0)
 *   overflow    set (and left set) when a step was counted although the window was full: that
 *               token's row was not stored; the caller did not roll the window over in time
 * dc_step_state_advance: n_recent = clamp(n_recent + delta, 0, limit), append_pos follows; once
 * per decoded token, after the last layer (src/diffcache/kvcache/diffcache.py:221-223).
 * dc_step_state_rollover: the oldest `moved` rows of the window join the region: region_hi +=
 * moved, n_recent = keep, append_pos follows.  Stream-ordered, may sit between two replays of a
 * captured step; the caller sketches the moved rows first (dc_sketch_build_bf16, keep_scale).
 */
typedef struct dc_step_state {
    int32_t n_recent, region_hi, append_pos, overflow;
} dc_step_state;
int dc_step_state_advance(int32_t *state, int delta, int limit, void *stream);
int dc_step_state_rollover(int32_t *state, int moved, int keep, void *stream);

/*
 * Prefill ingest: src (n_b, seq, n_h, hd) -> store[b, h, dst_pos + s, :].
 * Replaces the permute(0,2,1,3).contiguous() + host copy + Index::prefill memcpy
 * (src/diffcache/kvcache/diffcache.py:142-147, diffcache_cpu/src/nsw.rs:503-508).
 */
int dc_ingest_kv_bf16(void *store, const void *src, int n_b, int seq, int n_h, int hd,
                      int64_t dst_pos, int64_t batch_stride, int64_t head_stride,
                      int64_t row_stride, void *stream);

/*
 * One decode layer of the path: score -> select -> attend, enqueued back to back.
 * All pointers are device pointers; see the single-step calls for the meaning
 * of each field.  n_ctx rows are valid per unit; the retrieval region is
 * [n_sink, recent_lo); ids written to idx_out are relative to n_sink (the
 * reference's node ids are relative to the region too: diffcache.py:175-181).
 * Replaces the call sequence of BaseModel.layer_decode
 * (src/diffcache/base.py:150-155) between the two captured graph halves.
 */
typedef struct dc_layer_args {
    const void *q;        /* (n_b, n_h*group, hd) bf16 */
    const void *k;        /* K store */
    const void *v;        /* V store */
    const void *new_k;    /* (n_b, n_h, hd) bf16 or NULL */
    const void *new_v;
    void *out;            /* (n_b, n_h*group, hd) bf16 */
    float *lse;           /* (n_b, n_h*group) or NULL */
    float *scores;        /* (n_units, scores_unit_stride) fp32 output, or NULL: scores are
                             not materialised and the streaming select is used */
    uint32_t *idx_out;    /* (n_units, idx_unit_stride) */
    void *workspace;      /* dc_layer_workspace_bytes(...) bytes, 256-byte aligned */
    size_t workspace_bytes;
    int64_t kv_batch_stride, kv_head_stride, kv_row_stride; /* same for K and V */
    int64_t scores_unit_stride, idx_unit_stride;
    int64_t recent_lo;    /* first row of the always-kept suffix */
    int n_b, n_h, group, hd;
    int n_sink, n_recent; /* rows [0,n_sink) and [recent_lo, recent_lo+n_recent) always kept */
    int budget;           /* k */
    int mode, order;
    float scale;          /* softmax scale, 1/sqrt(hd) in the reference (of the TRUE head dim when the rows
                             are zero-padded to a supported one) */
    int select_state_ready; /* streaming select only (scores == NULL).  0: the workspace is
                             initialised first.  1: the caller vouches that the last call on this
                             workspace was a dc_decode_layer with the same n_b, n_h, group, hd,
                             region length, budget and order and scores == NULL (with or without
                             a sketch, whichever route it took), which leaves the select state
                             ready; the init kernels are skipped */
    void *ev_scan_begin;  /* optional hipEvent_t pair recorded on `stream` right before and */
    void *ev_scan_end;    /* right after the scan kernel (for timing it in place), or NULL */
    const uint8_t *sketch_codes; /* NULL, or the sketch of the K store (row 0 = store row 0): the
                             streaming select then scans the codes (dc_score_select_sketch_bf16);
                             needs scores == NULL */
    const float *sketch_scale;   /* (n_b*n_h, hd) */
    const float *sketch_resid;   /* (n_b*n_h, hd) */
    int64_t sketch_batch_stride, sketch_head_stride, sketch_row_stride; /* bytes */
    const int32_t *n_recent_dev; /* NULL, or the device-side length of the suffix (see
                             dc_gather_attn_bf16): n_recent is then its capacity */
    int one_kernel;       /* a DC_ONE_KERNEL_* value: when a short context may run as one kernel
                             (see "Short contexts" below); 0 = DC_ONE_KERNEL_AUTO */
    const int32_t *region_hi_dev; /* NULL, or a device word holding the first row of the suffix
                             (= the end of the retrieval region) at the time the kernels run;
                             recent_lo is then its LARGEST value, which sizes the launches and the
                             workspace, so that a call captured in a graph stays valid when the
                             recent window is rolled over (dc_step_state).  Needs scores == NULL; the
                             region must hold at least `budget` rows; takes the sketch or streaming
                             route */
} dc_layer_args;

size_t dc_layer_workspace_bytes(int n_units, int n_region_rows, int budget, int group, int hd,
                                int n_rows_attended);
int dc_decode_layer(const dc_layer_args *args, void *stream);
/*
 * Short contexts.  With scores == NULL, order == DC_ORDER_ANY and at most 640 Ki region rows
 * over all units (and, when a sketch is passed, whose chain of kernels is the faster one, at most
 * 40 Ki region rows per unit), dc_decode_layer runs the layer as ONE kernel whose blocks are all resident
 * (two per CU) and hand their phases over through the workspace (same results; the event pair
 * then brackets that kernel).  No counterpart in the reference, whose layers run on the CPU pool
 * (lib.rs:352-369); what it has to match is that one layer call is always right
 * (src/diffcache/base.py:150-155).
 *
 * The kernel counts on all its blocks running at the same time.  It may share the GPU with
 * short kernels of other streams, which only delay it, but not with a second launch of itself
 * on another stream (two DiffCache objects, two sequences decoded side by side: each launch
 * would get part of the CUs and wait for blocks that cannot start), nor with kernels that keep
 * CUs occupied for good.  What the library does about it:
 *   - it remembers, per device, the stream of the last launch of the kernel; a dc_decode_layer
 *     on ANOTHER stream while that stream still has work in flight (hipStreamQuery, never a
 *     wait) takes the chain of kernels of the long contexts instead (same ids, same attention
 *     within rounding).
 *     A call on a stream that is being captured takes the chain too, because a graph is replayed
 *     at times the library never sees.  dc_layer_args.one_kernel overrides this:
 *     DC_ONE_KERNEL_EXCLUSIVE: the caller vouches that no other launch of the kernel and no
 *     long-lived kernel shares the GPU (the kernel is then launched under capture as well);
 *     DC_ONE_KERNEL_NEVER: always the chain.  dc_last_route() says what the last call took;
 *   - the waits between blocks are bounded (about a second each).  If one runs out all the
 *     same, the call's results are void and say so: the out rows (and lse) of the unit are NaN
 *     and its ids 0xffffffff (do not gather with them), the unit's error word in the workspace
 *     stays set, and every later one-kernel call on that workspace returns NaN as well until the
 *     select state is initialised again;
 *   - it initialises that state again by itself: the failing kernel also stores into a word of
 *     pinned host memory, which every dc_decode_layer call reads (no copy, no wait); from then
 *     on the first call on every workspace ignores select_state_ready == 1 once.  Calls that
 *     were enqueued before the failure was seen return NaN; a captured graph cannot be mended
 *     this way (its launches are fixed): capture it again, or take it out of use, when
 *     dc_decode_layer_errors() has moved.
 * dc_decode_layer_errors: the number of failures seen so far in this process (reads the
 * pinned word of the current device, waits for nothing).
 * dc_decode_layer_status waits for `stream` and returns DC_EDEVICE if the error word of a unit
 * of this workspace is set, DC_OK otherwise.  `args` as in the call it checks.
 * DIFFCACHE_ONE_KERNEL=0 in the environment of the process switches the route off.
 */
#define DC_ONE_KERNEL_AUTO 0
#define DC_ONE_KERNEL_EXCLUSIVE 1
#define DC_ONE_KERNEL_NEVER (-1)
int dc_decode_layer_status(const dc_layer_args *args, void *stream);
unsigned dc_decode_layer_errors(void);
/*
 * Which kernels a dc_decode_layer call with these arguments runs when no other launch of the
 * one-kernel route is in the way (pointers are not followed): a DC_ROUTE_* value, or a negative
 * DC_E* code.  dc_last_route: the route that the last dc_decode_layer call of this thread took.
 */
#define DC_ROUTE_ATTEND_ONLY 0 /* nothing to select (empty region or budget 0) */
#define DC_ROUTE_DENSE 1       /* fp32 scores materialised: dc_score_bf16 + dc_topk_select */
#define DC_ROUTE_STREAM 2      /* dc_score_prune_bf16 + dc_sparse_select */
#define DC_ROUTE_SKETCH 3      /* dc_score_select_sketch_bf16 */
#define DC_ROUTE_ONE_KERNEL 4  /* short context: the whole layer in one kernel */
int dc_decode_layer_route(const dc_layer_args *args);
int dc_last_route(void);
/*
 * The rule by which a call is kept off the one-kernel route, as a function of what the library
 * knows at the call (exposed so that the rule can be tested without a GPU): 1 = launch the
 * kernel, 0 = take the chain.  policy: dc_layer_args.one_kernel; capturing: the stream is under
 * capture; have_prev: the kernel was launched on this device before; same_stream: on this very
 * stream; prev_done: that launch's stream has nothing in flight any more.
 */
int dc_one_kernel_guard(int policy, int capturing, int have_prev, int same_stream, int prev_done);
/*
 * For tests of that error path: the number of polls after which a block of the one-kernel
 * route gives up a wait (0: the default, about a second).  With a tiny limit the kernel still
 * runs to its end and behaves as described above for a wait that ran out.  Process-wide.
 */
void dc_set_wait_limit(int polls);

/*
 * PQ asymmetric-distance baseline.  The reference's PQ baseline directory
 * (evaluation/impl/pqcache) is empty, so these replace no reference code; the
 * shapes follow the benchmark configuration (M subspaces x 256 centroids).
 *   dc_pq_build_lut: lut[u, m, c] = q[u, m*ds:(m+1)*ds] . books[h(u), m, c, :]
 *     q (n_b*n_h, hd) bf16, books (n_h, M, 256, ds) fp32, lut (n_b*n_h, M, 256) fp32
 *   dc_pq_adc_scan: scores[u, i] = sum_m lut[u, m, codes[u, i, m]]
 *     codes (n_units, n_rows, M) uint8; the fp32 adds of key i run over
 *     m = i mod M, (i mod M) + 1, ... cyclically (the order that keeps the LDS
 *     table reads of a wave in different banks);
 *     hist as in dc_score_bf16 (keys in DC_MODE_IP order), or NULL
 *   dc_score_gathered_bf16: scores[u, j] = q[u] . k[row_offset + idx[u, j]]  (exact rerank)
 *   dc_compose_idx: out[u, j] = outer[u, inner[u, j]]
 */
int dc_pq_build_lut(const void *q, const float *books, float *lut, int n_b, int n_h, int hd, int m,
                    void *stream);
int dc_pq_adc_scan(const uint8_t *codes, const float *lut, float *scores, uint32_t *hist,
                   int n_units, int n_rows, int m, int64_t scores_unit_stride, void *stream);
int dc_score_gathered_bf16(const void *k, const void *q, const uint32_t *idx, float *scores,
                           int n_b, int n_h, int n_idx, int64_t idx_unit_stride, int hd,
                           int64_t row_offset, int64_t k_batch_stride, int64_t k_head_stride,
                           int64_t k_row_stride, int64_t scores_unit_stride, void *stream);
int dc_compose_idx(const uint32_t *outer, int64_t outer_unit_stride, const uint32_t *inner,
                   int64_t inner_unit_stride, uint32_t *out, int64_t out_unit_stride, int n_units,
                   int n_inner, void *stream);

/*
 * The whole PQ search in one call, without a dense ADC score array:
 *   candidates = the min(n_cand, n_rows) keys of every unit with the largest ADC
 *                scores (ties to the lower id), scores as dc_pq_adc_scan computes them;
 *   idx_out[u, 0 .. min(topk, n_rows)) = the candidates with the largest exact scores
 *                q[u] . k[id] (as dc_score_gathered_bf16 computes them), best first,
 *                ties to the lower id.
 * Same ids as dc_pq_adc_scan -> dc_topk_select(DC_ORDER_INDEX) ->
 * dc_score_gathered_bf16 -> dc_topk_select(DC_ORDER_BEST) -> dc_compose_idx.
 * q (n_b*n_h, hd) bf16, lut from dc_pq_build_lut, codes (n_b*n_h, n_rows, M) uint8,
 * k the bf16 key store with element strides; workspace from dc_pq_search_workspace_bytes.
 * state_ready: 0 = the call initialises the selection state of the workspace itself;
 * 1 = the previous call on this workspace was a dc_pq_search_bf16 with the same
 * n_units, n_rows and n_cand, returned 0 and had work to do (n_rows > 0, topk > 0):
 * every such call leaves the state ready for the next.
 * ev_scan_begin / ev_scan_end: optional hipEvent_t recorded on the stream around the
 * scan kernel (NULL: none).
 */
size_t dc_pq_search_workspace_bytes(int n_units, int n_rows, int n_cand);
int dc_pq_search_bf16(const void *k, const uint8_t *codes, const float *lut, const void *q,
                      uint32_t *idx_out, int64_t idx_unit_stride, int n_b, int n_h, int n_rows,
                      int hd, int m, int64_t k_batch_stride, int64_t k_head_stride,
                      int64_t k_row_stride, int n_cand, int topk, int state_ready,
                      void *workspace, size_t workspace_bytes, void *ev_scan_begin,
                      void *ev_scan_end, void *stream);

/*
 * The reference's data layer as a handle (struct DataLayer, diffcache_cpu/src/lib.rs:189-197):
 * shape, capacity and context length on the host, over device buffers the caller owns.
 * For hosts that are not Python (the Python mirror is diffcache_amd.DiffCacheHIP).
 *   create   DataLayer::new, lib.rs:292-327.  mode: DC_MODE_*; use_sketch: keep the 8-bit
 *            sketch of the keys and query through it (same results).
 *   sizes    bytes of the buffers to bind: store_bytes for EACH of the K and V stores
 *            (bsz, kv_heads, max_ctx_len, hd) bf16, codes_bytes, scale_bytes for EACH of
 *            scale and resid (0 without the sketch), idx_bytes, workspace_bytes; max_ef =
 *            the largest ef a query will ask for.
 *   bind     hands the buffers over (16-byte aligned, the workspace 256-byte aligned).
 *   prefill  lib.rs:329-347: keys, vals (bsz, kv_heads, n_rows, hd) bf16 replace the
 *            contents; n_rows <= max_ctx_len.  From device memory or pinned host memory
 *            (hipHostMalloc) the copy is enqueued and the source must stay unchanged until
 *            `stream` has passed it; from ordinary pageable host memory (a numpy array, a
 *            malloc'd block) the call waits for `stream` and returns with the copy done, so
 *            the source may be reused at once -- at the price of a synchronisation.
 *   insert   lib.rs:352-369: keys, vals (bsz, kv_heads, hd) bf16 in device memory, one
 *            token per unit, appended at ctx_len; an error when the store is full.
 *   query    lib.rs:373-404 with nsw.rs:592-630: queries (bsz, kv_heads, hd) bf16; the
 *            min(ef, ctx_len) best K and V rows of every unit, best first, ties to the
 *            lower id, into out_keys / out_vals (bsz, kv_heads, out_rows, hd) in device
 *            memory; *n_out (may be NULL) = rows written per unit.
 * prefill (from device or pinned memory), insert and query only enqueue work on `stream`;
 * calls on one handle must not overlap.  destroy frees the handle, never the buffers.
 */
typedef struct dc_data_layer dc_data_layer;
int dc_data_layer_create(dc_data_layer **out, int bsz, int kv_heads, int hd, int64_t max_ctx_len,
                         int mode, int use_sketch);
void dc_data_layer_destroy(dc_data_layer *dl);
int64_t dc_data_layer_ctx_len(const dc_data_layer *dl);
int dc_data_layer_sizes(const dc_data_layer *dl, int max_ef, size_t *store_bytes, size_t *codes_bytes,
                        size_t *scale_bytes, size_t *idx_bytes, size_t *workspace_bytes);
int dc_data_layer_bind(dc_data_layer *dl, void *k_store, void *v_store, void *codes, void *scale,
                       void *resid, void *idx, void *workspace, size_t workspace_bytes, int max_ef);
int dc_data_layer_prefill(dc_data_layer *dl, const void *keys, const void *vals, int64_t n_rows,
                          void *stream);
int dc_data_layer_insert(dc_data_layer *dl, const void *keys, const void *vals, void *stream);
int dc_data_layer_query(dc_data_layer *dl, void *out_keys, void *out_vals, int64_t out_rows,
                        const void *queries, int ef, int *n_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DIFFCACHE_HIP_H */
