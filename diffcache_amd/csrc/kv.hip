// K/V store maintenance: per-token append and the prefill layout transform.
// Replaces Index::insert's row write (diffcache_cpu/src/nsw.rs:551-557) and the
// permute + host copy + Index::prefill memcpy of
// src/diffcache/kvcache/diffcache.py:142-147 / nsw.rs:503-508.
#include "dc_common.h"

namespace {

// one 16-byte chunk per thread
__global__ void append_kernel(uint16_t *__restrict__ ks, uint16_t *__restrict__ vs,
                              const uint16_t *__restrict__ nk, const uint16_t *__restrict__ nv,
                              int n_h, int hd, int64_t pos, const int32_t *__restrict__ pos_dev,
                              int64_t pos_end, int64_t sb, int64_t sh, int64_t sr, int64_t total_chunks) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total_chunks) return;
    // the row may be counted on the device (base + *pos_dev); a count that would leave the
    // caller's range writes nothing
    if (pos_dev) pos += (int64_t)*pos_dev;
    if (pos < 0 || pos >= pos_end) return;
    const int cpr = hd / 8;
    const int64_t unit = t / cpr;
    const int c = (int)(t % cpr);
    const int64_t b = unit / n_h, h = unit % n_h;
    const int64_t dst = b * sb + h * sh + pos * sr + c * 8;
    const int64_t src = unit * hd + c * 8;
    *reinterpret_cast<uint4 *>(ks + dst) = *reinterpret_cast<const uint4 *>(nk + src);
    *reinterpret_cast<uint4 *>(vs + dst) = *reinterpret_cast<const uint4 *>(nv + src);
}

// counter = min(counter + delta, limit): one thread
__global__ void step_advance_kernel(int32_t *counter, int delta, int limit) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        const int64_t c = (int64_t)*counter + delta;
        *counter = (int32_t)(c < limit ? (c < 0 ? 0 : c) : limit);
    }
}

// The step state of a sequence as four device words (dc_step_state in the header): one thread.
__global__ void step_state_advance_kernel(int32_t *s, int delta, int limit) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        int64_t n = (int64_t)s[0] + delta;
        if (n > limit) {  // the window is full: this token has no row (the caller had to roll it over)
            s[3] = 1;
            n = limit;
        }
        if (n < 0) n = 0;
        s[0] = (int32_t)n;
        s[2] = s[1] + (int32_t)n;
    }
}
__global__ void step_state_rollover_kernel(int32_t *s, int moved, int keep) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        s[1] += moved;
        s[0] = keep;
        s[2] = s[1] + keep;
    }
}

// src (n_b, seq, n_h, hd) -> store[b, h, dst_pos + s, :]; one 16-byte chunk per
// thread, threads ordered like the source so reads are fully coalesced and
// writes land as whole rows
__global__ void ingest_kernel(uint16_t *__restrict__ store, const uint16_t *__restrict__ src,
                              int seq, int n_h, int hd, int64_t dst_pos, int64_t sb, int64_t sh,
                              int64_t sr, int64_t total_chunks) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= total_chunks) return;
    const int cpr = hd / 8;
    const int c = (int)(t % cpr);
    int64_t r = t / cpr;
    const int64_t h = r % n_h;
    r /= n_h;
    const int64_t s = r % seq;
    const int64_t b = r / seq;
    const int64_t dst = b * sb + h * sh + (dst_pos + s) * sr + c * 8;
    dc_store_stream16(store + dst, dc_load_stream16(src + t * 8));
}

}  // namespace

extern "C" int dc_append_kv_bf16(void *k_store, void *v_store, const void *new_k, const void *new_v,
                                 int n_b, int n_h, int hd, int64_t pos, const int32_t *pos_dev,
                                 int64_t pos_end, int64_t sb, int64_t sh, int64_t sr, void *stream) {
    DC_REQUIRE(k_store && v_store && new_k && new_v, "dc_append_kv_bf16: null pointer");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && hd >= 8 && hd % 8 == 0 && pos >= 0, "dc_append_kv_bf16: bad sizes");
    DC_REQUIRE(pos < pos_end, "dc_append_kv_bf16: position %lld outside the store's %lld rows", (long long)pos,
               (long long)pos_end);
    DC_REQUIRE(dc_aligned16(k_store) && dc_aligned16(v_store) && dc_aligned16(new_k) && dc_aligned16(new_v),
               "dc_append_kv_bf16: pointers must be 16-byte aligned");
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0, "dc_append_kv_bf16: strides must be multiples of 8");
    const int64_t total = (int64_t)n_b * n_h * (hd / 8);
    if (total == 0) return DC_OK;
    hipLaunchKernelGGL(append_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (uint16_t *)k_store, (uint16_t *)v_store,
                       (const uint16_t *)new_k, (const uint16_t *)new_v, n_h, hd, pos, pos_dev, pos_end, sb, sh,
                       sr, total);
    DC_CHECK_LAUNCH("dc_append_kv_bf16");
    return DC_OK;
}

extern "C" int dc_step_advance(int32_t *counter, int delta, int limit, void *stream) {
    DC_REQUIRE(counter, "dc_step_advance: null pointer");
    DC_REQUIRE(limit >= 0, "dc_step_advance: negative limit");
    hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, counter, delta, limit);
    DC_CHECK_LAUNCH("dc_step_advance");
    return DC_OK;
}

extern "C" int dc_step_state_advance(int32_t *state, int delta, int limit, void *stream) {
    DC_REQUIRE(state, "dc_step_state_advance: null pointer");
    DC_REQUIRE(limit >= 0, "dc_step_state_advance: negative limit");
    hipLaunchKernelGGL(step_state_advance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, state, delta, limit);
    DC_CHECK_LAUNCH("dc_step_state_advance");
    return DC_OK;
}

extern "C" int dc_step_state_rollover(int32_t *state, int moved, int keep, void *stream) {
    DC_REQUIRE(state, "dc_step_state_rollover: null pointer");
    DC_REQUIRE(moved >= 0 && keep >= 0, "dc_step_state_rollover: negative count");
    hipLaunchKernelGGL(step_state_rollover_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, state, moved, keep);
    DC_CHECK_LAUNCH("dc_step_state_rollover");
    return DC_OK;
}

extern "C" int dc_ingest_kv_bf16(void *store, const void *src, int n_b, int seq, int n_h, int hd,
                                 int64_t dst_pos, int64_t sb, int64_t sh, int64_t sr, void *stream) {
    DC_REQUIRE(store && src, "dc_ingest_kv_bf16: null pointer");
    DC_REQUIRE(n_b >= 0 && seq >= 0 && n_h >= 1 && hd >= 8 && hd % 8 == 0 && dst_pos >= 0,
               "dc_ingest_kv_bf16: bad sizes");
    DC_REQUIRE(dc_aligned16(store) && dc_aligned16(src), "dc_ingest_kv_bf16: pointers must be 16-byte aligned");
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0, "dc_ingest_kv_bf16: strides must be multiples of 8");
    const int64_t total = (int64_t)n_b * seq * n_h * (hd / 8);
    if (total == 0) return DC_OK;
    DC_REQUIRE((total + 255) / 256 < (1ll << 31), "dc_ingest_kv_bf16: grid too large");
    hipLaunchKernelGGL(ingest_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (uint16_t *)store, (const uint16_t *)src, seq, n_h, hd,
                       dst_pos, sb, sh, sr, total);
    DC_CHECK_LAUNCH("dc_ingest_kv_bf16");
    return DC_OK;
}
