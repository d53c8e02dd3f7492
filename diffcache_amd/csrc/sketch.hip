// The 8-bit sketch of the key store that dc_score_select_sketch_bf16 scans.
//
// Per unit and channel d the sketch holds a scale a_d and a residual bound r_d;
// row i is stored as HD bytes u_id = c_id + 128 with c_id in [-127, 127] and
//   k_id = a_d * c_id + e_id,   |e_id| <= r_d   for every sketched row.
// r_d is measured while quantising (not assumed to be a_d / 2), so rows added
// later with values outside the range the scales were fitted to only raise r_d
// and the bound stays true.  No counterpart in the reference: the exact scan of
// diffcache_cpu/src/nsw.rs:592-630 reads every bf16 key; the sketch lets the GPU
// read half as many bytes and still return that scan's result.
#include "dc_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = 2048;

__global__ void sketch_zero_kernel(uint32_t *a, uint32_t *b, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        if (a) a[i] = 0;
        b[i] = 0;
    }
}

// largest finite bf16 magnitude (inf and NaN are clamped to it; their residual is inf)
constexpr uint32_t kMaxFiniteMag = 0x7f7fu;

// per (unit, channel) maximum |k| over the rows, as float bits (non-negative floats
// order like unsigned integers)
template <int HD>
__global__ __launch_bounds__(kThreads) void sketch_absmax_kernel(
    const uint16_t *__restrict__ K, uint32_t *__restrict__ amax_bits, int n_h, int n_rows, int64_t sb,
    int64_t sh, int64_t sr, int blocks_per_unit) {
    constexpr int LPR = HD / 8;
    constexpr int GROUPS = kThreads / LPR;
    __shared__ uint32_t smax[GROUPS][HD];
    const int unit = blockIdx.x / blocks_per_unit, blk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int grp = threadIdx.x / LPR, col = threadIdx.x % LPR;
    const uint16_t *Ku = K + b * sb + h * sh + col * 8;
    const int64_t r0 = (int64_t)blk * kRowsPerBlock;
    int64_t r1 = r0 + kRowsPerBlock;
    if (r1 > n_rows) r1 = n_rows;
    uint32_t m[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) m[i] = 0;
    for (int64_t r = r0 + grp; r < r1; r += GROUPS) {
        const uint4 w = dc_load_stream16(Ku + r * sr);
        const uint32_t x[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = x[i] & 0x7fffu, hi = (x[i] >> 16) & 0x7fffu;
            m[2 * i] = lo > m[2 * i] ? lo : m[2 * i];
            m[2 * i + 1] = hi > m[2 * i + 1] ? hi : m[2 * i + 1];
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) smax[grp][col * 8 + i] = m[i];
    __syncthreads();
    if (threadIdx.x < HD) {
        uint32_t v = 0;
        for (int g = 0; g < GROUPS; ++g) v = smax[g][threadIdx.x] > v ? smax[g][threadIdx.x] : v;
        v = v > kMaxFiniteMag ? kMaxFiniteMag : v;
        if (v) atomicMax(&amax_bits[(int64_t)unit * HD + threadIdx.x], v << 16);
    }
}

// quantise rows with a_d = amax_d / 127 (scale_is_amax) or a_d = scale_d, write the
// codes, and raise resid_d to the largest |k - a c| seen
template <int HD>
__global__ __launch_bounds__(kThreads) void sketch_quantise_kernel(
    const uint16_t *__restrict__ K, uint8_t *__restrict__ C, const float *__restrict__ scale,
    uint32_t *__restrict__ resid_bits, int n_h, int n_rows, int64_t sb, int64_t sh, int64_t sr, int64_t cb,
    int64_t ch, int64_t cr, int blocks_per_unit, int scale_is_amax) {
    constexpr int LPR = HD / 8;
    constexpr int GROUPS = kThreads / LPR;
    __shared__ uint32_t smax[GROUPS][HD];
    const int unit = blockIdx.x / blocks_per_unit, blk = blockIdx.x % blocks_per_unit;
    const int b = unit / n_h, h = unit % n_h;
    const int grp = threadIdx.x / LPR, col = threadIdx.x % LPR;
    const uint16_t *Ku = K + b * sb + h * sh + col * 8;
    uint8_t *Cu = C + b * cb + h * ch + col * 8;
    float a[8], inv[8], res[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float s = scale[(int64_t)unit * HD + col * 8 + i];
        a[i] = scale_is_amax ? s / 127.0f : s;
        inv[i] = a[i] > 0.f ? 1.0f / a[i] : 0.f;
        res[i] = 0.f;
    }
    const int64_t r0 = (int64_t)blk * kRowsPerBlock;
    int64_t r1 = r0 + kRowsPerBlock;
    if (r1 > n_rows) r1 = n_rows;
    for (int64_t r = r0 + grp; r < r1; r += GROUPS) {
        const uint4 w = dc_load_stream16(Ku + r * sr);
        const float kv[8] = {dc_bf16_lo(w.x), dc_bf16_hi(w.x), dc_bf16_lo(w.y), dc_bf16_hi(w.y),
                             dc_bf16_lo(w.z), dc_bf16_hi(w.z), dc_bf16_lo(w.w), dc_bf16_hi(w.w)};
        uint32_t code[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float c = rintf(kv[i] * inv[i]);
            c = c > 127.f ? 127.f : (c < -127.f ? -127.f : c);
            if (!(c == c)) c = 0.f;  // NaN key or 0 * inf
            const float e = fabsf(fmaf(-a[i], c, kv[i]));
            // a NaN residual must poison the bound, not vanish in the max
            if (!(e <= res[i])) res[i] = (e == e) ? e : __builtin_inff();
            code[i] = (uint32_t)((int)c + 128);
        }
        uint2 packed;
        packed.x = code[0] | (code[1] << 8) | (code[2] << 16) | (code[3] << 24);
        packed.y = code[4] | (code[5] << 8) | (code[6] << 16) | (code[7] << 24);
        dc_store_stream8(Cu + r * cr, packed);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) smax[grp][col * 8 + i] = __float_as_uint(res[i]);
    __syncthreads();
    if (threadIdx.x < HD) {
        uint32_t v = 0;
        for (int g = 0; g < GROUPS; ++g) v = smax[g][threadIdx.x] > v ? smax[g][threadIdx.x] : v;
        if (v) atomicMax(&resid_bits[(int64_t)unit * HD + threadIdx.x], v);
    }
}

__global__ void sketch_finalise_kernel(float *scale, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) scale[i] = scale[i] / 127.0f;  // the same expression the quantise kernel used
}

}  // namespace

extern "C" int dc_sketch_build_bf16(const void *k, uint8_t *codes, float *scale, float *resid, int n_b,
                                    int n_h, int n_rows, int hd, int64_t sb, int64_t sh, int64_t sr,
                                    int64_t cb, int64_t ch, int64_t cr, int keep_scale, void *stream) {
    const char *who = "dc_sketch_build_bf16";
    DC_REQUIRE(k && codes && scale && resid, "%s: null pointer", who);
    DC_REQUIRE(n_b >= 0 && n_h >= 1 && n_rows >= 0, "%s: bad sizes", who);
    DC_REQUIRE(hd == 64 || hd == 128 || hd == 256, "%s: head_dim %d not in {64,128,256}", who, hd);
    DC_REQUIRE(dc_aligned16(k) && dc_aligned16(codes), "%s: k and codes must be 16-byte aligned", who);
    DC_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && sr % 8 == 0 && sr >= hd,
               "%s: key strides must be multiples of 8 elements and row_stride >= hd", who);
    DC_REQUIRE(cb % 16 == 0 && ch % 16 == 0 && cr % 16 == 0 && cr >= hd,
               "%s: code strides must be multiples of 16 bytes and row_stride >= hd", who);
    const int64_t n_units = (int64_t)n_b * n_h;
    if (n_units == 0) return DC_OK;
    const int64_t bpu = n_rows > 0 ? ((int64_t)n_rows + kRowsPerBlock - 1) / kRowsPerBlock : 0;
    DC_REQUIRE(n_units * (bpu > 0 ? bpu : 1) < (1ll << 31), "%s: grid too large", who);
    hipStream_t st = (hipStream_t)stream;
    const int64_t n_sc = n_units * hd;
    const dim3 sgrid((unsigned)((n_sc + 255) / 256));
    if (!keep_scale) {
        hipLaunchKernelGGL(sketch_zero_kernel, sgrid, dim3(256), 0, st, (uint32_t *)scale, (uint32_t *)resid,
                           n_sc);
        DC_CHECK_LAUNCH(who);
    }
    if (bpu == 0) return DC_OK;
    const dim3 grid((unsigned)(n_units * bpu));
#define DC_LAUNCH_SKB(HD)                                                                               \
    do {                                                                                                \
        if (!keep_scale)                                                                                \
            hipLaunchKernelGGL(sketch_absmax_kernel<HD>, grid, dim3(kThreads), 0, st, (const uint16_t *)k, \
                               (uint32_t *)scale, n_h, n_rows, sb, sh, sr, (int)bpu);                   \
        hipLaunchKernelGGL(sketch_quantise_kernel<HD>, grid, dim3(kThreads), 0, st, (const uint16_t *)k, \
                           codes, scale, (uint32_t *)resid, n_h, n_rows, sb, sh, sr, cb, ch, cr, (int)bpu, \
                           keep_scale ? 0 : 1);                                                         \
    } while (0)
    if (hd == 64) DC_LAUNCH_SKB(64);
    else if (hd == 128) DC_LAUNCH_SKB(128);
    else DC_LAUNCH_SKB(256);
#undef DC_LAUNCH_SKB
    DC_CHECK_LAUNCH(who);
    if (!keep_scale) {
        hipLaunchKernelGGL(sketch_finalise_kernel, sgrid, dim3(256), 0, st, scale, n_sc);
        DC_CHECK_LAUNCH(who);
    }
    return DC_OK;
}
