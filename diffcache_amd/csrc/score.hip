// Scoring: one query per (batch, kv-head) unit against every key row of the
// retrieval region, streamed once from HBM.  Replaces the distance loop of
// search_bruteforce (diffcache_cpu/src/nsw.rs:601-607, 129-139).
//
// Data movement.  A key row is HD bf16 = HD*2 contiguous bytes.  LPR = HD/8
// lanes cover one row with one 16-byte load each, so a wave64 load instruction
// fetches 64/LPR whole rows (four 256-byte rows at HD 128).  A wave handles 64
// consecutive rows per step: lane group g owns rows [g*LPR, (g+1)*LPR) of the
// step and issues LPR independent loads (at most 16 in flight), each followed
// by 8 FMAs and a DPP sum over the group.  The lane whose position in the group
// equals the load number keeps that row's score, so lane L ends up holding
// row L of the step and the 64 scores leave as one coalesced 256-byte store.
// The kernel is bound by HBM: 2*HD bytes read and 4 bytes written per row.
//
// The optional epilogue bins each score's ordering key into a per-block LDS
// histogram (DC_HIST_BINS buckets) and adds the non-empty bins to the unit's
// global histogram, which saves dc_topk_select one pass over the scores.
#include "dc_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DC_WAVE;
constexpr int kRowsPerWaveStep = 64;
constexpr int kRowsPerBlockStep = kWaves * kRowsPerWaveStep;  // 256

template <int HD>
__global__ __launch_bounds__(kThreads) void score_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ Q, float *__restrict__ scores,
    uint32_t *__restrict__ hist, int n_h, int n_rows, int64_t sb, int64_t sh, int64_t sr,
    int64_t scores_stride, int q_group, int mode, int steps_per_block, int blocks_per_unit) {
    constexpr int LPR = HD / 8;          // lanes per row
    constexpr int CH = LPR < 16 ? LPR : 16;  // loads in flight per lane
    __shared__ uint32_t lhist[DC_HIST_BINS];

    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int grp = lane / LPR, col = lane % LPR;

    if (hist) {
        for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;
        __syncthreads();
    }

    // this lane's 8 query values; a GQA group is averaged in fp32 and rounded to
    // bf16 first (diffcache.py:193)
    float q[8];
    dc_load_query<HD>(Q, unit, q_group, col, q);

    const uint16_t *Ku = K + b * sb + h * sh + col * 8;
    float *su = scores + (int64_t)unit * scores_stride;
    uint32_t *hu = hist ? hist + (int64_t)unit * DC_HIST_BINS : nullptr;
    const int last = n_rows - 1;

    const int64_t block_row0 = (int64_t)chunk * steps_per_block * kRowsPerBlockStep;
    for (int step = 0; step < steps_per_block; ++step) {
        const int64_t row0 = block_row0 + (int64_t)step * kRowsPerBlockStep + wave * kRowsPerWaveStep;
        if (row0 >= n_rows) break;
        float mine = 0.f;
#pragma unroll
        for (int c0 = 0; c0 < LPR; c0 += CH) {
            uint4 w[CH];
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                int64_t r = row0 + grp * LPR + c0 + j;
                r = r > last ? last : r;  // keep the load in bounds; masked below
                w[j] = dc_load_stream16(Ku + r * sr);
            }
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                float p = dc_dot8(w[j], q, 0.f);
                p = dc_group_sum<LPR>(p);
                mine = (col == c0 + j) ? p : mine;
            }
        }
        const int64_t myrow = row0 + lane;
        if (myrow < n_rows) {
            su[myrow] = mine;
            if (hu) {
                uint32_t key, bucket;
                dc_key_bucket(mine, mode, key, bucket);
                atomicAdd(&lhist[bucket], 1u);
            }
        }
    }

    if (hu) {
        __syncthreads();
        for (int i = tid; i < DC_HIST_BINS; i += kThreads) {
            uint32_t c = lhist[i];
            if (c) atomicAdd(&hu[i], c);
        }
    }
}

// scores of gathered rows: one 16-lane (LPR-lane) group per selected row
template <int HD>
__global__ __launch_bounds__(kThreads) void score_gathered_kernel(
    const uint16_t *__restrict__ K, const uint16_t *__restrict__ Q, const uint32_t *__restrict__ idx,
    float *__restrict__ scores, int n_h, int n_idx, int64_t idx_stride, int64_t row_offset,
    int64_t sb, int64_t sh, int64_t sr, int64_t scores_stride, int blocks_per_unit) {
    constexpr int LPR = HD / 8;
    constexpr int GROUPS = kThreads / LPR;
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int grp = threadIdx.x / LPR, col = threadIdx.x % LPR;
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = dc_bf16_to_f32(Q[(int64_t)unit * HD + col * 8 + i]);
    const int j = chunk * GROUPS + grp;
    const int jj = j < n_idx ? j : n_idx - 1;
    const int64_t r = row_offset + idx[(int64_t)unit * idx_stride + jj];
    uint4 w = *reinterpret_cast<const uint4 *>(K + b * sb + h * sh + r * sr + col * 8);
    float p = dc_group_sum<LPR>(dc_dot8(w, q, 0.f));
    if (j < n_idx && col == 0) scores[(int64_t)unit * scores_stride + j] = p;
}

__global__ void group_mean_kernel(const uint16_t *__restrict__ q, uint16_t *__restrict__ out,
                                  int group, int hd, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    int64_t u = i / hd;
    int d = (int)(i % hd);
    float acc = 0.f;
    for (int g = 0; g < group; ++g) acc += dc_bf16_to_f32(q[(u * group + g) * hd + d]);
    out[i] = dc_f32_to_bf16(acc / (float)group);
}

}  // namespace

extern "C" int dc_group_mean_bf16(const void *q, void *q_mean, int n_units, int group, int hd,
                                  void *stream) {
    DC_REQUIRE(q && q_mean, "dc_group_mean_bf16: null pointer");
    DC_REQUIRE(n_units >= 0 && group >= 1 && hd >= 1, "dc_group_mean_bf16: bad sizes");
    int64_t total = (int64_t)n_units * hd;
    if (total == 0) return DC_OK;
    int blocks = (int)((total + 255) / 256);
    hipLaunchKernelGGL(group_mean_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)q, (uint16_t *)q_mean, group, hd, total);
    DC_CHECK_LAUNCH("dc_group_mean_bf16");
    return DC_OK;
}

// rows a block covers; chosen so a layer of 64 units x 128K rows gives a few
// thousand blocks while the per-block histogram flush stays small
static int dc_score_steps_per_block(int n_rows) {
    int steps = 8;  // 2048 rows
    while (steps > 1 && (int64_t)steps * kRowsPerBlockStep > n_rows) steps >>= 1;
    return steps;
}

extern "C" int dc_score_bf16(const void *k, const void *q, float *scores, uint32_t *hist, int n_b,
                             int n_h, int n_rows, int hd, int64_t sb, int64_t sh, int64_t sr,
                             int64_t scores_unit_stride, int q_group, int mode, void *stream) {
    DC_REQUIRE(k && q && scores, "dc_score_bf16: null pointer");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_rows >= 0 && q_group >= 1, "dc_score_bf16: bad sizes");
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "dc_score_bf16: head_dim %d not in {64,128,256}", hd);
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "dc_score_bf16: bad mode %d", mode);
    DC_REQUIRE(dc_aligned16(k), "dc_score_bf16: k must be 16-byte aligned");
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0 && sr >= hd,
               "dc_score_bf16: strides must be multiples of 8 elements and row_stride >= hd");
    DC_REQUIRE(scores_unit_stride >= n_rows, "dc_score_bf16: scores_unit_stride < n_rows");
    const int64_t n_units = (int64_t)n_b * n_h;
    if (n_units == 0 || n_rows == 0) return DC_OK;
    const int steps = dc_score_steps_per_block(n_rows);
    const int64_t rows_per_block = (int64_t)steps * kRowsPerBlockStep;
    const int64_t bpu = (n_rows + rows_per_block - 1) / rows_per_block;
    DC_REQUIRE(n_units * bpu < (1ll << 31), "dc_score_bf16: grid too large");
    dim3 grid((unsigned)(n_units * bpu)), block(kThreads);
    hipStream_t st = (hipStream_t)stream;
#define DC_LAUNCH_SCORE(HD)                                                                        \
    hipLaunchKernelGGL(score_kernel<HD>, grid, block, 0, st, (const uint16_t *)k,                  \
                       (const uint16_t *)q, scores, hist, n_h, n_rows, sb, sh, sr,                 \
                       scores_unit_stride, q_group, mode, steps, (int)bpu)
    if (hd == 64) DC_LAUNCH_SCORE(64);
    else if (hd == 128) DC_LAUNCH_SCORE(128);
    else DC_LAUNCH_SCORE(256);
#undef DC_LAUNCH_SCORE
    DC_CHECK_LAUNCH("dc_score_bf16");
    return DC_OK;
}

extern "C" int dc_score_gathered_bf16(const void *k, const void *q, const uint32_t *idx,
                                      float *scores, int n_b, int n_h, int n_idx,
                                      int64_t idx_unit_stride, int hd, int64_t row_offset,
                                      int64_t sb, int64_t sh, int64_t sr,
                                      int64_t scores_unit_stride, void *stream) {
    DC_REQUIRE(k && q && idx && scores, "dc_score_gathered_bf16: null pointer");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_idx >= 0, "dc_score_gathered_bf16: bad sizes");
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "dc_score_gathered_bf16: head_dim %d unsupported", hd);
    DC_REQUIRE(dc_aligned16(k) && sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0,
               "dc_score_gathered_bf16: alignment");
    DC_REQUIRE(idx_unit_stride >= n_idx && scores_unit_stride >= n_idx,
               "dc_score_gathered_bf16: unit strides too small");
    const int64_t n_units = (int64_t)n_b * n_h;
    if (n_units == 0 || n_idx == 0) return DC_OK;
    const int groups = kThreads / (hd / 8);
    const int64_t bpu = (n_idx + groups - 1) / groups;
    dim3 grid((unsigned)(n_units * bpu)), block(kThreads);
    hipStream_t st = (hipStream_t)stream;
#define DC_LAUNCH_SG(HD)                                                                           \
    hipLaunchKernelGGL(score_gathered_kernel<HD>, grid, block, 0, st, (const uint16_t *)k,         \
                       (const uint16_t *)q, idx, scores, n_h, n_idx, idx_unit_stride, row_offset,  \
                       sb, sh, sr, scores_unit_stride, (int)bpu)
    if (hd == 64) DC_LAUNCH_SG(64);
    else if (hd == 128) DC_LAUNCH_SG(128);
    else DC_LAUNCH_SG(256);
#undef DC_LAUNCH_SG
    DC_CHECK_LAUNCH("dc_score_gathered_bf16");
    return DC_OK;
}
