// Product-quantisation baseline: per-query lookup tables and the asymmetric
// distance (ADC) scan.  The reference's PQ baseline directory
// (evaluation/impl/pqcache) is empty, so this follows the benchmark
// configuration only: M subspaces x 256 centroids, 8-bit codes, fp32 tables.
//
// The scan keeps the unit's tables in LDS (32 KB, laid out so that the reads of a
// wave never share a bank, see dc_pq.h) and gives each thread one key at a time:
// M code bytes, M table reads, M fp32 adds.  HBM traffic is M bytes per key.
#include "dc_common.h"
#include "dc_pq.h"

namespace {

constexpr int kThreads = 256;
constexpr int kKeysPerThread = 16;
constexpr int kKeysPerBlock = kThreads * kKeysPerThread;

__global__ __launch_bounds__(256) void pq_lut_kernel(const uint16_t *__restrict__ q,
                                                     const float *__restrict__ books,
                                                     float *__restrict__ lut, int n_h, int hd, int m) {
    const int um = blockIdx.x;  // unit * m + sub
    const int unit = um / m, sub = um % m;
    const int h = unit % n_h;
    const int ds = hd / m;
    const int c = threadIdx.x;
    const float *cb = books + (((int64_t)h * m + sub) * 256 + c) * ds;
    const uint16_t *qp = q + (int64_t)unit * hd + sub * ds;
    float acc = 0.f;
    for (int d = 0; d < ds; ++d) acc = fmaf(dc_bf16_to_f32(qp[d]), cb[d], acc);
    lut[(int64_t)um * 256 + c] = acc;
}

template <int M>
__global__ __launch_bounds__(kThreads) void pq_adc_kernel(
    const uint8_t *__restrict__ codes, const float *__restrict__ lut, float *__restrict__ scores,
    uint32_t *__restrict__ hist, int n_rows, int64_t scores_stride, int blocks_per_unit) {
    __shared__ float s_lut[kPqLutWords];
    __shared__ uint32_t lhist[DC_HIST_BINS];
    const int unit = blockIdx.x / blocks_per_unit;
    const int chunk = blockIdx.x % blocks_per_unit;
    const int tid = threadIdx.x;
    pq_stage_lut<M>(s_lut, lut + (int64_t)unit * M * 256, tid, kThreads);
    if (hist)
        for (int i = tid; i < DC_HIST_BINS; i += kThreads) lhist[i] = 0;
    PqLane<M> ln;
    ln.init(tid & 63);
    __syncthreads();
    const uint8_t *cu = codes + (int64_t)unit * n_rows * M;
    float *su = scores + (int64_t)unit * scores_stride;
    const int64_t base = (int64_t)chunk * kKeysPerBlock;  // a multiple of 64: lane = key mod 64
    for (int it = 0; it < kKeysPerThread; ++it) {
        const int64_t i = base + (int64_t)it * kThreads + tid;
        if (i >= n_rows) break;
        const uint4 *cp = reinterpret_cast<const uint4 *>(cu + i * M);
        uint32_t words[M / 4];
#pragma unroll
        for (int w = 0; w < M / 16; ++w) {
            const uint4 cw = cp[w];
            words[4 * w + 0] = cw.x;
            words[4 * w + 1] = cw.y;
            words[4 * w + 2] = cw.z;
            words[4 * w + 3] = cw.w;
        }
        const float acc = pq_adc_score<M>(words, s_lut, ln);
        su[i] = acc;
        if (hist) {
            uint32_t key, bucket;
            dc_key_bucket(acc, DC_MODE_IP, key, bucket);
            atomicAdd(&lhist[bucket], 1u);
        }
    }
    if (hist) {
        __syncthreads();
        uint32_t *hu = hist + (int64_t)unit * DC_HIST_BINS;
        for (int i = tid; i < DC_HIST_BINS; i += kThreads) {
            uint32_t c = lhist[i];
            if (c) atomicAdd(&hu[i], c);
        }
    }
}

}  // namespace

extern "C" int dc_pq_build_lut(const void *q, const float *books, float *lut, int n_b, int n_h,
                               int hd, int m, void *stream) {
    DC_REQUIRE(q && books && lut, "dc_pq_build_lut: null pointer");
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && m >= 1 && hd >= m && hd % m == 0, "dc_pq_build_lut: bad sizes");
    const int64_t blocks = (int64_t)n_b * n_h * m;
    if (blocks == 0) return DC_OK;
    hipLaunchKernelGGL(pq_lut_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)q, books, lut, n_h, hd, m);
    DC_CHECK_LAUNCH("dc_pq_build_lut");
    return DC_OK;
}

extern "C" int dc_pq_adc_scan(const uint8_t *codes, const float *lut, float *scores, uint32_t *hist,
                              int n_units, int n_rows, int m, int64_t scores_unit_stride,
                              void *stream) {
    DC_REQUIRE(codes && lut && scores, "dc_pq_adc_scan: null pointer");
    DC_REQUIRE(n_units >= 0 && n_rows >= 0, "dc_pq_adc_scan: bad sizes");
    DC_REQUIRE(m == 16 || m == 32, "dc_pq_adc_scan: m = %d subspaces unsupported (16 or 32)", m);
    DC_REQUIRE(dc_aligned16(codes) && dc_aligned16(lut), "dc_pq_adc_scan: pointers must be 16-byte aligned");
    DC_REQUIRE(scores_unit_stride >= n_rows, "dc_pq_adc_scan: scores_unit_stride < n_rows");
    if (n_units == 0 || n_rows == 0) return DC_OK;
    const int64_t bpu = ((int64_t)n_rows + kKeysPerBlock - 1) / kKeysPerBlock;
    DC_REQUIRE(n_units * bpu < (1ll << 31), "dc_pq_adc_scan: grid too large");
    dim3 grid((unsigned)(n_units * bpu));
    hipStream_t st = (hipStream_t)stream;
    if (m == 16)
        hipLaunchKernelGGL(pq_adc_kernel<16>, grid, dim3(kThreads), 0, st, codes, lut, scores, hist,
                           n_rows, scores_unit_stride, (int)bpu);
    else
        hipLaunchKernelGGL(pq_adc_kernel<32>, grid, dim3(kThreads), 0, st, codes, lut, scores, hist,
                           n_rows, scores_unit_stride, (int)bpu);
    DC_CHECK_LAUNCH("dc_pq_adc_scan");
    return DC_OK;
}
