// LUT-GEMM (binary-coding quantisation) GEMV role, batch 1:
//   out[n] += sum_g [ q_bias[g][n] * sum_{c in g} x[c]
//                     + sum_b alpha[g][b][n] * sum_{c in g} s_b(n, c) * x[c] ],   s = +1/-1
// with s_b(n, c) = bit (c % 32) of q_weight[c / 32][b][n]  (reference
// decdec_extension/lutgemm.cu:25-150; packing llm-awq/quantize/qmodule.py:61-92).
//
// A workgroup owns KTB consecutive 32-channel tiles and a range of outputs.  It first builds, from
// the activations alone, the 256-entry signed subset-sum table of every 8-channel group of its tiles
// in LDS (fp32, so table entries carry no rounding), then every thread walks two adjacent outputs:
// one coalesced 8-byte load per (tile, bit plane), four table lookups per 32-bit word.  Partial sums
// stay in fp32 registers across all tiles of the workgroup, so an output receives K / (32 KTB) atomic
// adds instead of the reference's K / 32.
#pragma once
#include "common.h"

namespace decdec {

struct LutgemmParams {
    const void* x;
    const uint32_t* qw;        // [K/32][bits][N]
    const void* alpha;         // [K/group][bits][N]
    const void* q_bias;        // [K/group][N]
    void* out;
    uint32_t N, K, bits, group_size;
    uint32_t ktb;              // 32-channel tiles per workgroup
    uint32_t npb;              // outputs per workgroup (even)
    uint32_t n_tiles, k_tiles;
};

constexpr int kLutgemmMaxKtb = 8;

__host__ __device__ inline size_t lutgemm_lds_bytes(uint32_t ktb) {
    return (size_t)ktb * 4 * 256 * 4 + (size_t)ktb * 4;
}

template <int DT>
__device__ __forceinline__ void lutgemm_role(const LutgemmParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
    const uint32_t nt = bid % p.n_tiles, ktile = bid / p.n_tiles;
    const uint32_t kt0 = ktile * p.ktb;
    const uint32_t total_kt = p.K / 32u;
    const uint32_t nkt = (kt0 + p.ktb) <= total_kt ? p.ktb : (total_kt - kt0);
    float* tab = (float*)smem;                       // [ktb][4][256]
    float* xsum = tab + (size_t)p.ktb * 1024;        // [ktb]

    // subset-sum tables: tab[kt][y][pat] = sum_j (bit j of pat ? +1 : -1) * x[32 (kt0+kt) + 8 y + j]
    for (uint32_t idx = tid; idx < nkt * 1024u; idx += nthreads) {
        const uint32_t pat = idx & 255u, grp = idx >> 8;            // grp = kt*4 + y
        const size_t c0 = (size_t)32 * kt0 + (size_t)8 * grp;
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float xv = E::load(p.x, c0 + j);
            s += ((pat >> j) & 1u) ? xv : -xv;
        }
        tab[idx] = s;
    }
    __syncthreads();
    if (tid < nkt) xsum[tid] = tab[tid * 1024 + 255] + tab[tid * 1024 + 511] + tab[tid * 1024 + 767] + tab[tid * 1024 + 1023];
    __syncthreads();

    const uint32_t n_begin = nt * p.npb;
    const uint32_t n_end = (n_begin + p.npb) < p.N ? (n_begin + p.npb) : p.N;
    for (uint32_t n = n_begin + 2 * tid; n < n_end; n += 2 * nthreads) {
        const bool pair = (n + 1 < n_end) && ((p.N & 1u) == 0u);   // 8-byte aligned pair load
        float acc0 = 0.f, acc1 = 0.f;
        for (uint32_t kt = 0; kt < nkt; ++kt) {
            const uint32_t g = (32u * (kt0 + kt)) / p.group_size;
            const float* t = tab + (size_t)kt * 1024;
            const float xs = xsum[kt];
            acc0 += E::load(p.q_bias, (size_t)g * p.N + n) * xs;
            if (n + 1 < n_end) acc1 += E::load(p.q_bias, (size_t)g * p.N + n + 1) * xs;
            for (uint32_t b = 0; b < p.bits; ++b) {
                const size_t wo = ((size_t)(kt0 + kt) * p.bits + b) * p.N + n;
                uint32_t w0, w1 = 0u;
                if (pair) { const u32x2 w = *(const u32x2*)(p.qw + wo); w0 = w[0]; w1 = w[1]; }
                else { w0 = p.qw[wo]; if (n + 1 < n_end) w1 = p.qw[wo + 1]; }
                const size_t ao = ((size_t)g * p.bits + b) * p.N + n;
                const float t0 = t[w0 & 255u] + t[256 + ((w0 >> 8) & 255u)] + t[512 + ((w0 >> 16) & 255u)] + t[768 + (w0 >> 24)];
                acc0 += E::load(p.alpha, ao) * t0;
                if (n + 1 < n_end) {
                    const float t1 = t[w1 & 255u] + t[256 + ((w1 >> 8) & 255u)] + t[512 + ((w1 >> 16) & 255u)] + t[768 + (w1 >> 24)];
                    acc1 += E::load(p.alpha, ao + 1) * t1;
                }
            }
        }
        if ((n + 1 < n_end) && ((n & 1u) == 0u)) E::atomic_add2(p.out, n, acc0, acc1);
        else {
            E::atomic_add1(p.out, n, acc0);
            if (n + 1 < n_end) E::atomic_add1(p.out, n + 1, acc1);
        }
    }
}

}  // namespace decdec
