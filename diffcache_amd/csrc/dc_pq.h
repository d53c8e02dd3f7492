// Device code shared by the PQ kernels: the unit's lookup tables in LDS and the
// asymmetric-distance (ADC) score of one key.
//
// A key's score is the sum of M table entries, one per code byte.  A wave reads
// 64 unrelated entries per step; if the tables sat in LDS subspace by subspace,
// the banks hit would be random and every read would take several passes.  The
// tables are therefore kept entry-major with 32 columns, word (c * 32 + col), so
// that the bank is the column, and lane l walks the subspaces starting from
// subspace l mod M: at every step the 32 lanes of a half-wave read 32 different
// columns.  With M = 16 the columns 16..31 repeat 0..15 and the upper 16 lanes of
// each half-wave use the copy.
//
// The order of the fp32 additions follows the walk: key i (i = position in the
// unit, lane = i mod 64) adds subspaces (i mod M), (i mod M) + 1, ... cyclically.
// Every PQ kernel scores keys through pq_adc_score, so all of them agree bit for bit.
#pragma once
#include "dc_common.h"

constexpr int kPqLutWords = 256 * 32;  // LDS words of a unit's tables

// tables of one unit, lut_unit[M][256] in global memory, into s_lut (kPqLutWords floats)
template <int M>
__device__ __forceinline__ void pq_stage_lut(float *__restrict__ s_lut, const float *__restrict__ lut_unit,
                                             int tid, int n_threads) {
    const float4 *src = reinterpret_cast<const float4 *>(lut_unit);
    for (int i = tid; i < M * 64; i += n_threads) {
        const int s = i % M, cg = i / M;  // subspace, group of four entries
        const float4 v = src[s * 64 + cg];
        float *dst = s_lut + (4 * cg) * 32 + s;
        dst[0] = v.x;
        dst[32] = v.y;
        dst[64] = v.z;
        dst[96] = v.w;
        if (M == 16) {
            dst[16] = v.x;
            dst[48] = v.y;
            dst[80] = v.z;
            dst[112] = v.w;
        }
    }
}

// per-lane constants of the walk
template <int M>
struct PqLane {
    uint32_t off[M];   // byte offset of the column read at step j
    uint32_t rot[3];   // all-ones where the code row is rotated by 4, 2, 1 words
    uint32_t sh;       // and by this many bytes after that
    __device__ __forceinline__ void init(int lane) {
        const uint32_t r = (uint32_t)lane % M;
        const uint32_t colbase = ((uint32_t)lane & 31u) - (M == 32 ? r : ((uint32_t)lane & 15u));
        rot[0] = (r & 16u) ? ~0u : 0u;
        rot[1] = (r & 8u) ? ~0u : 0u;
        rot[2] = (r & 4u) ? ~0u : 0u;
        sh = r & 3u;
#pragma unroll
        for (int j = 0; j < M; ++j) {
            off[j] = 4u * (colbase + ((r + j) % M));
            asm volatile("" : "+v"(off[j]));  // held in a register, not recomputed per key
        }
    }
};

// ADC score of the key whose M code bytes are w[0 .. M/4) (little-endian words)
template <int M>
__device__ __forceinline__ float pq_adc_score(const uint32_t (&w)[M / 4], const float *s_lut,
                                              const PqLane<M> &ln) {
    constexpr int NW = M / 4;
    // rotate the row left by r bytes: first by whole words, then by the odd bytes
    uint32_t a[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) a[i] = w[i];
#pragma unroll
    for (int stage = 0; stage < 3; ++stage) {
        const int bit = 4 >> stage;
        if (bit < NW) {
            const uint32_t m = ln.rot[stage];  // bitwise select keeps this a three-stage shifter
            uint32_t t[NW];
#pragma unroll
            for (int i = 0; i < NW; ++i) t[i] = (a[(i + bit) % NW] & m) | (a[i] & ~m);
#pragma unroll
            for (int i = 0; i < NW; ++i) a[i] = t[i];
        }
    }
    uint32_t rw[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) rw[i] = __builtin_amdgcn_alignbyte(a[(i + 1) % NW], a[i], ln.sh);
    const char *base = reinterpret_cast<const char *>(s_lut);
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < M; ++j) {
        const uint32_t c = (rw[j / 4] >> (8 * (j % 4))) & 0xffu;
        acc += *reinterpret_cast<const float *>(base + ((c << 7) + ln.off[j]));
    }
    return acc;
}
