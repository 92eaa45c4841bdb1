// SqueezeLLM (per-output-channel non-uniform LUT) GEMV role, batch 1:
//   out[n] += sum_c lut[n][field(n, c)] * x[c]
// with mat[K*bits/32][N] (N contiguous).  4-bit: word c/8, field at bit 4 (c % 8).  3-bit: channels
// 32u..32u+31 form a 96-bit little-endian stream over words 3u..3u+2, field at bit 3 (c % 32)
// (reference decdec_extension/sqllm.cu:28-169).
//
// A thread owns one output column, so the packed words of 64 neighbouring columns form one coalesced
// 256-byte wave load per matrix row.  The column's LUT sits in LDS as lut_s[value][thread] (fp32): a
// lookup hits bank (thread % 32) whatever the value, i.e. it is conflict-free.  The activations of
// the workgroup's K range are staged in LDS once and read as broadcasts.  fp32 accumulation; one
// atomic add per output per K range.
#pragma once
#include "common.h"

namespace decdec {

struct SqllmParams {
    const void* x;
    const uint32_t* mat;
    const void* lut;
    void* out;
    uint32_t N, K, bits;
    uint32_t kspan;            // channels per workgroup along K (multiple of 32)
    uint32_t nthreads;         // threads (= columns) that work per workgroup: multiple of 64, <= blockDim
    uint32_t n_tiles, k_tiles;
};

__host__ __device__ inline size_t sqllm_lds_bytes(uint32_t nthreads, uint32_t bits, uint32_t kspan) {
    return ((size_t)(1u << bits) * nthreads + kspan) * 4;
}

template <int DT>
__device__ __forceinline__ void sqllm_role(const SqllmParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, nthreads = p.nthreads;
    if (tid >= nthreads) return;                    // surplus waves of a wider launch leave at once
    const uint32_t nt = bid % p.n_tiles, ktile = bid / p.n_tiles;
    const uint32_t L = 1u << p.bits;
    float* lut_s = (float*)smem;                    // [L][nthreads]
    float* xs = lut_s + (size_t)L * nthreads;       // [kspan]
    const uint32_t n = nt * nthreads + tid;
    const uint32_t k0 = ktile * p.kspan;
    const uint32_t k1 = (k0 + p.kspan) < p.K ? (k0 + p.kspan) : p.K;
    const bool col_ok = n < p.N;

    if (col_ok)
        for (uint32_t v = 0; v < L; ++v) lut_s[v * nthreads + tid] = E::load(p.lut, (size_t)n * L + v);
    for (uint32_t c = k0 + tid; c < k1; c += nthreads) xs[c - k0] = E::load(p.x, c);
    __syncthreads();

    float acc = 0.f;
    const float* lt = lut_s + tid;
    if (!col_ok) {
        // nothing to accumulate; stay for the lane pairing below
    } else if (p.bits == 4) {
        const uint32_t r0 = k0 / 8u, r1 = k1 / 8u;
        constexpr int U = 8;
        for (uint32_t r = r0; r < r1; r += U) {
            uint32_t w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) w[u] = (r + u < r1) ? p.mat[(size_t)(r + u) * p.N + n] : 0u;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (r + u >= r1) break;
                const float* xv = xs + (size_t)(r + u - r0) * 8;
#pragma unroll
                for (int j = 0; j < 8; ++j) acc += lt[((w[u] >> (4 * j)) & 0xFu) * nthreads] * xv[j];
            }
        }
    } else {
        const uint32_t u0 = k0 / 32u, u1 = k1 / 32u;
        constexpr int U = 2;
        for (uint32_t g = u0; g < u1; g += U) {
            uint32_t w[U][3];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int q = 0; q < 3; ++q)
                    w[u][q] = (g + u < u1) ? p.mat[(size_t)(3 * (g + u) + q) * p.N + n] : 0u;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (g + u >= u1) break;
                const float* xv = xs + (size_t)(g + u - u0) * 32;
                const unsigned long long lo = (unsigned long long)w[u][0] | ((unsigned long long)w[u][1] << 32);
                const unsigned long long hi = (unsigned long long)(w[u][1] >> 31) | ((unsigned long long)w[u][2] << 1);
                // fields 0..20 live in bits 0..62 of lo; fields 21..31 in bits 63..95 = bits 0..32 of hi
#pragma unroll
                for (int j = 0; j < 21; ++j) acc += lt[(uint32_t)((lo >> (3 * j)) & 7ull) * nthreads] * xv[j];
#pragma unroll
                for (int j = 21; j < 32; ++j) acc += lt[(uint32_t)((hi >> (3 * j - 63)) & 7ull) * nthreads] * xv[j];
            }
        }
    }
    // Columns n and n+1 sit in neighbouring lanes (tile origins are even): the even lane merges both
    // with one packed atomic.
    const float other = __shfl_down(acc, 1, 64);
    if (col_ok && (tid & 1u) == 0u) {
        if (n + 1 < p.N) E::atomic_add2(p.out, n, acc, other);
        else E::atomic_add1(p.out, n, acc);
    }
}

}  // namespace decdec
