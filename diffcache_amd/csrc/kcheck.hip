// k-check: does the top-H of a unit's result list already hold the wanted share of
// the attention mass?  Follows diffcache_cpu/src/nsw.rs:198-296: a power law is
// fitted to the logits of ranks 5..H (least squares of logit against ln(rank), sums
// in f64), the tail beyond H is modelled as v_H * H / (alpha - 1), and H is
// accepted when head / (head + tail) reaches the threshold.  The reference runs the
// check inside its graph search on the H best found so far and only reports the
// outcome (nsw.rs:367-379); here it runs on the exact, sorted result list and
// yields the number of rows worth attending to: the first H of k_check_seq (H < ef,
// in order) that passes, else ef.
#include "dc_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxSeq = 16;
constexpr int kMinRank = 5;  // nsw.rs:288
constexpr int kMaxEf = 16384;  // nsw.rs:15: sizes beyond the reference's ln(rank) table never pass (nsw.rs:207-210)

struct KSeq {
    int h[kMaxSeq];
    int n;
};

__device__ __forceinline__ double block_sum(double v, double *red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d, 64);
    __syncthreads();  // red may still be read from the previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    double s = 0.0;
#pragma unroll
    for (int w = 0; w < kThreads / 64; ++w) s += red[w];
    return s;
}

__device__ __forceinline__ float block_max(float v, double *red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
    __syncthreads();
    if (lane == 0) red[wave] = (double)v;
    __syncthreads();
    float s = (float)red[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) s = fmaxf(s, (float)red[w]);
    return s;
}

// scores: fp32 scores of the selected rows, best first.  The logit of a row is
// (65536 - dist) / sqrt(dim) with dist = f32(65536 - score) (nsw.rs:138,282-286); in
// DC_MODE_IP, where no distance exists, score / sqrt(dim).
__global__ __launch_bounds__(kThreads) void kcheck_kernel(const float *__restrict__ scores,
                                                          int64_t stride, int n_sel, int hd, int mode,
                                                          KSeq seq, float threshold,
                                                          uint32_t *__restrict__ n_eff,
                                                          float *__restrict__ alpha_out,
                                                          float *__restrict__ mass_out) {
    __shared__ double red[kThreads / 64];
    const int unit = blockIdx.x;
    const int tid = threadIdx.x;
    const float *su = scores + (int64_t)unit * stride;
    const float sqrt_dim = sqrtf((float)hd);
    auto logit = [&](int i) -> float {
        const float s = su[i];
        if (mode == DC_MODE_REF_DIST) {
            const float d = 65536.0f - s;
            return (65536.0f - d) / sqrt_dim;
        }
        return s / sqrt_dim;
    };
    const float nan = __uint_as_float(0x7fc00000u);
    uint32_t result = (uint32_t)n_sel;
    bool decided = false;
    for (int e = 0; e < seq.n; ++e) {
        const int H = seq.h[e];
        float alpha = nan, mass = nan;
        if (!decided && H < n_sel && H > kMinRank && H <= kMaxEf) {
            // least squares of logit against ln(rank) over ranks kMinRank..H
            double sx = 0.0, sy = 0.0, sxx = 0.0, sxy = 0.0;
            for (int i = kMinRank - 1 + tid; i < H; i += kThreads) {
                const double x = log((double)(i + 1));
                const double y = (double)logit(i);
                sx += x;
                sy += y;
                sxx += x * x;
                sxy += x * y;
            }
            sx = block_sum(sx, red);
            sy = block_sum(sy, red);
            sxx = block_sum(sxx, red);
            sxy = block_sum(sxy, red);
            const double n = (double)(H - kMinRank + 1);
            const double denom = n * sxx - sx * sx;
            if (n >= 2.0 && fabs(denom) >= 1e-12) {
                alpha = (float)(-((n * sxy - sx * sy) / denom));
                if (alpha > 1.0f) {
                    float mx = -INFINITY;
                    for (int i = tid; i < H; i += kThreads) mx = fmaxf(mx, logit(i));
                    mx = block_max(mx, red);
                    double hs = 0.0;
                    for (int i = tid; i < H; i += kThreads) hs += (double)expf(logit(i) - mx);
                    const float head_sum = (float)block_sum(hs, red);
                    const float v_h = expf(logit(H - 1) - mx);
                    const float tail = v_h * (float)H / (alpha - 1.0f);
                    const float den = head_sum + tail;
                    if (den > 0.f) {
                        mass = head_sum / den;
                        if (mass >= threshold) {
                            result = (uint32_t)H;
                            decided = true;
                        }
                    }
                }
            }
        }
        if (tid == 0) {
            if (alpha_out) alpha_out[(int64_t)unit * seq.n + e] = alpha;
            if (mass_out) mass_out[(int64_t)unit * seq.n + e] = mass;
        }
    }
    if (tid == 0) n_eff[unit] = result;
}

}  // namespace

extern "C" int dc_kcheck_f32(const float *scores, int64_t scores_unit_stride, int n_units, int n_sel,
                             int hd, int mode, const int *k_check_seq, int n_seq,
                             float attn_mass_threshold, uint32_t *n_eff, float *alpha_out,
                             float *mass_out, void *stream) {
    DC_REQUIRE(n_eff, "dc_kcheck_f32: null pointer");
    DC_REQUIRE(n_units >= 0 && n_sel >= 0 && hd >= 1, "dc_kcheck_f32: bad sizes");
    DC_REQUIRE(n_sel == 0 || scores, "dc_kcheck_f32: scores is null");
    DC_REQUIRE(scores_unit_stride >= n_sel, "dc_kcheck_f32: scores_unit_stride < n_sel");
    DC_REQUIRE(mode == DC_MODE_IP || mode == DC_MODE_REF_DIST, "dc_kcheck_f32: bad mode %d", mode);
    DC_REQUIRE(n_seq >= 0 && n_seq <= kMaxSeq && (n_seq == 0 || k_check_seq),
               "dc_kcheck_f32: k_check_seq must hold at most %d sizes", kMaxSeq);
    if (n_units == 0) return DC_OK;
    KSeq seq;
    seq.n = n_seq;
    for (int i = 0; i < kMaxSeq; ++i) seq.h[i] = i < n_seq ? k_check_seq[i] : 0;
    for (int i = 0; i < n_seq; ++i) DC_REQUIRE(seq.h[i] >= 0, "dc_kcheck_f32: negative size in k_check_seq");
    hipLaunchKernelGGL(kcheck_kernel, dim3(n_units), dim3(kThreads), 0, (hipStream_t)stream, scores,
                       scores_unit_stride, n_sel, hd, mode, seq, attn_mass_threshold, n_eff, alpha_out,
                       mass_out);
    DC_CHECK_LAUNCH("dc_kcheck_f32");
    return DC_OK;
}
