/*
 * cpu_ref.c -- C restatement of the reference's exact-scan decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker and the timed CPU
 * baseline; nothing in the shipped library links or loads it.
 *
 * The reference's CPU path is a Rust crate that cannot be built here (no
 * cargo/rustc, crates not vendored), so this file follows it function by
 * function (paths relative to the reference checkout):
 *
 *   dcref_dot_bf16           diffcache_cpu/src/lib.rs:65-69 (simsimd 6.5.3 bf16
 *                            dot: fp32 accumulate, order unspecified -- bit-level
 *                            accumulation order is PARITY UNPINNED; checked to
 *                            1e-5 relative against a float64 dot)
 *   dcref_distance_qk        diffcache_cpu/src/nsw.rs:129-139  (65536.0f - dot)
 *   dcref_pack               diffcache_cpu/src/nsw.rs:74-80    (dist bits<<32 | id)
 *   dcref_search_bruteforce  diffcache_cpu/src/nsw.rs:592-630  (scan, max-heap of
 *                            size ef, replace on strictly smaller distance,
 *                            ascending output, row gather)
 *   dcref_query              diffcache_cpu/src/lib.rs:373-404  (ef clamp, one task
 *                            per (batch, kv-head); rayon -> pthreads here)
 *   dcref_group_mean         src/diffcache/kvcache/diffcache.py:191-194
 *   dcref_sparse_attention   src/diffcache/base.py:134-142 (flash-attn decode call
 *                            restated as an fp32 softmax . V; library absent from
 *                            the reference tree -> PARITY UNPINNED, checked against
 *                            a float64 softmax)
 *   dcref_decode_layer       src/diffcache/base.py:150-155 +
 *                            src/diffcache/kvcache/diffcache.py:196-223
 *   dcref_dualheap_*         diffcache_cpu/src/dualheap.rs:4-87
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t v) {
    uint32_t b = (uint32_t)v << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    if ((b & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    uint32_t lsb = (b >> 16) & 1u;
    return (uint16_t)((b + 0x7fffu + lsb) >> 16);
}

static inline uint32_t f32_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

static inline float bits_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

/* fp32-accumulated bf16 dot, 16 independent partial sums (SIMD friendly). */
__attribute__((target_clones("default", "avx2", "avx512f")))
float dcref_dot_bf16(const uint16_t *a, const uint16_t *b, int n) {
    float acc[16] = {0};
    int i = 0;
    for (; i + 16 <= n; i += 16)
        for (int j = 0; j < 16; ++j)
            acc[j] += bf16_to_f32(a[i + j]) * bf16_to_f32(b[i + j]);
    float s = 0.f;
    for (int j = 0; j < 16; ++j) s += acc[j];
    for (; i < n; ++i) s += bf16_to_f32(a[i]) * bf16_to_f32(b[i]);
    return s;
}

float dcref_distance_qk(const uint16_t *q, const uint16_t *k, int dim) {
    return 65536.0f - dcref_dot_bf16(q, k, dim);
}

uint64_t dcref_pack(float dist, uint32_t node) {
    return ((uint64_t)f32_bits(dist) << 32) | (uint64_t)node;
}

/* ---- binary max-heap on u64, the operations std::collections::BinaryHeap
 *      performs for push / replace-top / into_sorted_vec ---- */
static void heap_sift_up(uint64_t *h, size_t pos) {
    uint64_t v = h[pos];
    while (pos > 0) {
        size_t parent = (pos - 1) / 2;
        if (h[parent] >= v) break;
        h[pos] = h[parent];
        pos = parent;
    }
    h[pos] = v;
}

static void heap_sift_down(uint64_t *h, size_t len, size_t pos) {
    uint64_t v = h[pos];
    for (;;) {
        size_t child = 2 * pos + 1;
        if (child >= len) break;
        if (child + 1 < len && h[child + 1] > h[child]) child++;
        if (h[child] <= v) break;
        h[pos] = h[child];
        pos = child;
    }
    h[pos] = v;
}

static void heap_sort_ascending(uint64_t *h, size_t len) {
    for (size_t end = len; end > 1; --end) {
        uint64_t t = h[0];
        h[0] = h[end - 1];
        h[end - 1] = t;
        heap_sift_down(h, end - 1, 0);
    }
}

/*
 * Exact scan for one (batch, kv-head) index.
 * keys/vals: n_valid rows of `dim` bf16; out rows written best first.
 * Optional outputs (may be NULL): out_ids[ef], out_scores[n_valid].
 * `pre_scores` (may be NULL) replaces the computed dot products, so the
 * selection can be replayed on scores measured elsewhere.
 * Returns the number of rows written = min(ef, n_valid).
 */
int dcref_search_bruteforce(const uint16_t *keys, const uint16_t *vals, int n_valid, int dim,
                            const uint16_t *query, int ef, uint16_t *out_keys,
                            uint16_t *out_vals, uint32_t *out_ids, float *out_scores,
                            const float *pre_scores) {
    if (ef <= 0) return 0;
    uint64_t *heap = (uint64_t *)malloc(sizeof(uint64_t) * (size_t)ef);
    size_t len = 0;
    for (int node = 0; node < n_valid; ++node) {
        float dot = pre_scores ? pre_scores[node]
                               : dcref_dot_bf16(query, keys + (size_t)node * dim, dim);
        if (out_scores) out_scores[node] = dot;
        float dist = 65536.0f - dot;
        if (len < (size_t)ef) {
            heap[len] = dcref_pack(dist, (uint32_t)node);
            heap_sift_up(heap, len);
            len++;
        } else if (dist < bits_f32((uint32_t)(heap[0] >> 32))) {
            heap[0] = dcref_pack(dist, (uint32_t)node);
            heap_sift_down(heap, len, 0);
        }
    }
    heap_sort_ascending(heap, len);
    for (size_t i = 0; i < len; ++i) {
        uint32_t node = (uint32_t)(heap[i] & 0xffffffffu);
        if (out_ids) out_ids[i] = node;
        if (out_keys) memcpy(out_keys + i * dim, keys + (size_t)node * dim, 2 * (size_t)dim);
        if (out_vals) memcpy(out_vals + i * dim, vals + (size_t)node * dim, 2 * (size_t)dim);
    }
    free(heap);
    return (int)len;
}

/* ---- fan-out over (batch, kv-head) units ---- */
typedef struct {
    const uint16_t *keys, *vals, *queries;
    uint16_t *out_keys, *out_vals;
    uint32_t *out_ids;
    int n_units, ctx_len, n_max, dim, ef;
    int next;
    pthread_mutex_t mu;
} query_job;

static void *query_worker(void *arg) {
    query_job *j = (query_job *)arg;
    for (;;) {
        pthread_mutex_lock(&j->mu);
        int u = j->next++;
        pthread_mutex_unlock(&j->mu);
        if (u >= j->n_units) break;
        size_t base = (size_t)u * j->n_max * j->dim;
        size_t obase = (size_t)u * j->ef * j->dim;
        dcref_search_bruteforce(j->keys + base, j->vals + base, j->ctx_len, j->dim,
                                j->queries + (size_t)u * j->dim, j->ef,
                                j->out_keys ? j->out_keys + obase : NULL,
                                j->out_vals ? j->out_vals + obase : NULL,
                                j->out_ids ? j->out_ids + (size_t)u * j->ef : NULL, NULL, NULL);
    }
    return NULL;
}

/*
 * keys/vals (n_units, n_max, dim) with ctx_len valid rows per unit,
 * queries (n_units, dim), outputs (n_units, ef', dim) with ef' = min(ef, ctx_len).
 * Returns ef'.
 */
int dcref_query(const uint16_t *keys, const uint16_t *vals, const uint16_t *queries,
                uint16_t *out_keys, uint16_t *out_vals, uint32_t *out_ids, int n_units,
                int ctx_len, int n_max, int dim, int ef, int n_threads) {
    if (ef > ctx_len) ef = ctx_len;
    query_job j = {keys, vals, queries, out_keys, out_vals, out_ids,
                   n_units, ctx_len, n_max, dim, ef, 0, PTHREAD_MUTEX_INITIALIZER};
    if (n_threads > n_units) n_threads = n_units;
    if (n_threads <= 1) {
        query_worker(&j);
        return ef;
    }
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)n_threads);
    for (int t = 0; t < n_threads; ++t) pthread_create(&th[t], NULL, query_worker, &j);
    for (int t = 0; t < n_threads; ++t) pthread_join(th[t], NULL);
    free(th);
    return ef;
}

/* queries (n_units, group, dim) bf16 -> (n_units, dim) bf16: fp32 sum, one divide. */
void dcref_group_mean(const uint16_t *q, uint16_t *out, int n_units, int group, int dim) {
    for (int u = 0; u < n_units; ++u)
        for (int d = 0; d < dim; ++d) {
            float acc = 0.f;
            for (int g = 0; g < group; ++g) acc += bf16_to_f32(q[((size_t)u * group + g) * dim + d]);
            out[(size_t)u * dim + d] = f32_to_bf16(acc / (float)group);
        }
}

/*
 * fp32 softmax(q.K^T * scale).V over `n_rows` gathered rows, for `group` query
 * heads that share the rows.  out (group, dim) bf16.
 */
void dcref_sparse_attention(const uint16_t *q, const uint16_t *k_rows, const uint16_t *v_rows,
                            int n_rows, int group, int dim, float scale, uint16_t *out) {
    float *logit = (float *)malloc(sizeof(float) * (size_t)(n_rows > 0 ? n_rows : 1));
    float *acc = (float *)malloc(sizeof(float) * (size_t)dim);
    for (int g = 0; g < group; ++g) {
        const uint16_t *qg = q + (size_t)g * dim;
        float m = -INFINITY;
        for (int i = 0; i < n_rows; ++i) {
            logit[i] = dcref_dot_bf16(qg, k_rows + (size_t)i * dim, dim) * scale;
            if (logit[i] > m) m = logit[i];
        }
        float l = 0.f;
        memset(acc, 0, sizeof(float) * (size_t)dim);
        for (int i = 0; i < n_rows; ++i) {
            float p = expf(logit[i] - m);
            l += p;
            const uint16_t *vr = v_rows + (size_t)i * dim;
            for (int d = 0; d < dim; ++d) acc[d] += p * bf16_to_f32(vr[d]);
        }
        for (int d = 0; d < dim; ++d)
            out[(size_t)g * dim + d] = f32_to_bf16(n_rows > 0 ? acc[d] / l : 0.f);
    }
    free(logit);
    free(acc);
}

/* ---- one decode layer for a batch of units: the timed CPU baseline ---- */
typedef struct {
    const uint16_t *q, *k, *v, *new_k, *new_v;
    uint16_t *out;
    uint32_t *out_ids;
    int n_units, group, dim, n_ctx, n_max, budget, prefix, suffix;
    int next;
    pthread_mutex_t mu;
} layer_job;

static void layer_unit(layer_job *j, int u) {
    int dim = j->dim, g = j->group;
    int p_len = j->prefix < j->n_ctx ? j->prefix : j->n_ctx;
    int s_len = j->suffix < j->n_ctx - p_len ? j->suffix : j->n_ctx - p_len;
    int lo = p_len, hi = j->n_ctx - s_len, region = hi - lo;
    int ef = j->budget < region ? j->budget : region;
    const uint16_t *K = j->k + (size_t)u * j->n_max * dim;
    const uint16_t *V = j->v + (size_t)u * j->n_max * dim;
    int extra = j->new_k ? 1 : 0;
    int rows = ef + p_len + s_len + extra;
    uint16_t *kb = (uint16_t *)malloc(2 * (size_t)(rows > 0 ? rows : 1) * dim);
    uint16_t *vb = (uint16_t *)malloc(2 * (size_t)(rows > 0 ? rows : 1) * dim);
    uint16_t qmean[1024];
    dcref_group_mean(j->q + (size_t)u * g * dim, qmean, 1, g, dim);
    /* retrieved rows first (diffcache.py:202-209), then prefix, then suffix */
    dcref_search_bruteforce(K + (size_t)lo * dim, V + (size_t)lo * dim, region, dim, qmean, ef,
                            kb, vb, j->out_ids ? j->out_ids + (size_t)u * j->budget : NULL,
                            NULL, NULL);
    memcpy(kb + (size_t)ef * dim, K, 2 * (size_t)p_len * dim);
    memcpy(vb + (size_t)ef * dim, V, 2 * (size_t)p_len * dim);
    memcpy(kb + (size_t)(ef + p_len) * dim, K + (size_t)hi * dim, 2 * (size_t)s_len * dim);
    memcpy(vb + (size_t)(ef + p_len) * dim, V + (size_t)hi * dim, 2 * (size_t)s_len * dim);
    if (extra) {
        memcpy(kb + (size_t)(rows - 1) * dim, j->new_k + (size_t)u * dim, 2 * (size_t)dim);
        memcpy(vb + (size_t)(rows - 1) * dim, j->new_v + (size_t)u * dim, 2 * (size_t)dim);
    }
    dcref_sparse_attention(j->q + (size_t)u * g * dim, kb, vb, rows, g, dim,
                           1.0f / sqrtf((float)dim), j->out + (size_t)u * g * dim);
    free(kb);
    free(vb);
}

static void *layer_worker(void *arg) {
    layer_job *j = (layer_job *)arg;
    for (;;) {
        pthread_mutex_lock(&j->mu);
        int u = j->next++;
        pthread_mutex_unlock(&j->mu);
        if (u >= j->n_units) break;
        layer_unit(j, u);
    }
    return NULL;
}

/*
 * q (n_units, group, dim); k, v (n_units, n_max, dim) with n_ctx valid rows;
 * new_k/new_v (n_units, dim) or NULL; out (n_units, group, dim);
 * out_ids (n_units, budget) region-relative ids, or NULL.  dim <= 1024.
 */
void dcref_decode_layer(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                        const uint16_t *new_k, const uint16_t *new_v, uint16_t *out,
                        uint32_t *out_ids, int n_units, int group, int dim, int n_ctx, int n_max,
                        int budget, int prefix, int suffix, int n_threads) {
    layer_job j = {q, k, v, new_k, new_v, out, out_ids, n_units, group, dim, n_ctx, n_max,
                   budget, prefix, suffix, 0, PTHREAD_MUTEX_INITIALIZER};
    if (n_threads > n_units) n_threads = n_units;
    if (n_threads <= 1) {
        layer_worker(&j);
        return;
    }
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)n_threads);
    for (int t = 0; t < n_threads; ++t) pthread_create(&th[t], NULL, layer_worker, &j);
    for (int t = 0; t < n_threads; ++t) pthread_join(th[t], NULL);
    free(th);
}

/* ---- DualHeap on int64 items (dualheap.rs:4-87) ---- */
typedef struct {
    int64_t *small, *rest;
    size_t small_len, rest_len, d, cap, small_replace_count;
} dcref_dualheap;

static void ih_up(int64_t *h, size_t pos) {
    int64_t v = h[pos];
    while (pos > 0) {
        size_t p = (pos - 1) / 2;
        if (h[p] >= v) break;
        h[pos] = h[p];
        pos = p;
    }
    h[pos] = v;
}

static void ih_down(int64_t *h, size_t len, size_t pos) {
    int64_t v = h[pos];
    for (;;) {
        size_t c = 2 * pos + 1;
        if (c >= len) break;
        if (c + 1 < len && h[c + 1] > h[c]) c++;
        if (h[c] <= v) break;
        h[pos] = h[c];
        pos = c;
    }
    h[pos] = v;
}

dcref_dualheap *dcref_dualheap_new(size_t d, size_t cap) {
    if (d < 1 || cap < d) return NULL;
    dcref_dualheap *h = (dcref_dualheap *)calloc(1, sizeof(*h));
    h->small = (int64_t *)malloc(sizeof(int64_t) * d);
    h->rest = (int64_t *)malloc(sizeof(int64_t) * (cap - d + 1));
    h->d = d;
    h->cap = cap;
    return h;
}

void dcref_dualheap_free(dcref_dualheap *h) {
    if (!h) return;
    free(h->small);
    free(h->rest);
    free(h);
}

void dcref_dualheap_push(dcref_dualheap *h, int64_t item) {
    if (h->small_len < h->d) {
        h->small[h->small_len] = item;
        ih_up(h->small, h->small_len++);
        return;
    }
    if (h->small[0] > item) {
        h->small_replace_count++;
        int64_t t = h->small[0];
        h->small[0] = item;
        ih_down(h->small, h->small_len, 0);
        item = t;
    }
    if (h->cap == h->d) return;
    if (h->rest_len < h->cap - h->d) {
        h->rest[h->rest_len] = item;
        ih_up(h->rest, h->rest_len++);
        return;
    }
    if (h->rest[0] <= item) return;
    h->rest[0] = item;
    ih_down(h->rest, h->rest_len, 0);
}

size_t dcref_dualheap_len(const dcref_dualheap *h) { return h->small_len + h->rest_len; }

/* 1 and *out set when the value exists, else 0 */
int dcref_dualheap_dth_min(const dcref_dualheap *h, int64_t *out) {
    if (dcref_dualheap_len(h) < h->d) return 0;
    *out = h->small[0];
    return 1;
}

int dcref_dualheap_kept_max(const dcref_dualheap *h, int64_t *out) {
    if (h->rest_len) { *out = h->rest[0]; return 1; }
    if (h->small_len) { *out = h->small[0]; return 1; }
    return 0;
}

static int cmp_i64(const void *a, const void *b) {
    int64_t x = *(const int64_t *)a, y = *(const int64_t *)b;
    return (x > y) - (x < y);
}

/* writes len items ascending (small then rest, each sorted); returns len */
size_t dcref_dualheap_sorted(const dcref_dualheap *h, int64_t *out) {
    memcpy(out, h->small, sizeof(int64_t) * h->small_len);
    memcpy(out + h->small_len, h->rest, sizeof(int64_t) * h->rest_len);
    qsort(out, h->small_len, sizeof(int64_t), cmp_i64);
    qsort(out + h->small_len, h->rest_len, sizeof(int64_t), cmp_i64);
    return h->small_len + h->rest_len;
}
