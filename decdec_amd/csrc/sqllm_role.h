// SqueezeLLM (per-output-channel non-uniform LUT) GEMV role, batch 1:
//   out[n] += sum_c lut[n][field(n, c)] * x[c]
// with mat[K*bits/32][N] (N contiguous).  4-bit: word c/8, field at bit 4 (c % 8).  3-bit: channels
// 32u..32u+31 form a 96-bit little-endian stream over words 3u..3u+2, field at bit 3 (c % 32)
// (reference decdec_extension/sqllm.cu:28-169).
//
// A lane owns one output column, so the packed words of 64 neighbouring columns form one coalesced
// 256-byte wave load per matrix row.  All waves of a workgroup work on the SAME 64 columns and split the
// workgroup's K range between them: the columns' LUTs are converted to fp32 once per workgroup and sit in
// LDS as lut_s[value][lane] (a lookup hits bank lane % 32 whatever the value: conflict-free), the
// activations of a wave's channels are the same for all its lanes and therefore arrive through the
// scalar cache and stay in SGPRs, the waves' partial sums are added in LDS, and an output receives one
// atomic add per workgroup (k_tiles per output in all).  fp32 accumulation.
//
// For 16-bit storage types the table holds PAIRS: entry [b][lane] is the two LUT values of the two fields
// in b (a byte of a 4-bit row, six bits of a 3-bit row) packed as one dword, so two weights cost one shift,
// one and-or, one LDS read and one dot2 against the matching activation pair (adjacent channels, one SGPR
// dword).  Building the 256 x 64 (64 x 64) table costs each of the 1024 threads 16 (4) packs.
#pragma once
#include "common.h"

namespace decdec {

#define DD_SCALAR_AS __attribute__((address_space(4)))

struct SqllmParams {
    const void* x;
    const uint32_t* mat;
    const void* lut;
    void* out;
    uint32_t N, K, bits;
    uint32_t kslice;           // channels per wave (multiple of 32)
    uint32_t n_tiles, k_tiles; // column groups of 64 x K ranges of (waves per workgroup) * kslice
};

__host__ __device__ inline size_t sqllm_lds_bytes(uint32_t bits, uint32_t waves, bool pair_table) {
    const size_t entries = pair_table ? ((size_t)1 << (2 * bits)) : ((size_t)1 << bits);
    return (entries * 64 + (size_t)waves * 64) * 4;
}

template <int DT>
__device__ __forceinline__ float sqllm_dot2(uint32_t w, uint32_t x, float acc) {
    if constexpr (DT == kFP16) return __builtin_amdgcn_fdot2(*(half2_t*)&w, *(half2_t*)&x, acc, false);
    else return __builtin_amdgcn_fdot2_f32_bf16(*(bf16x2_t*)&w, *(bf16x2_t*)&x, acc, false);
}

// Pair-table variant (fp16 / bf16); the workgroup must have exactly 16 waves.
template <int DT>
__device__ __forceinline__ void sqllm_role_pairs(const SqllmParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr uint32_t nwaves = 16;
    const uint32_t nt = bid % p.n_tiles, ktile = bid / p.n_tiles;
    const uint32_t entries = 1u << (2u * p.bits);
    uint32_t* pair_s = (uint32_t*)smem;                      // [entries][64]: (lut[b & mask] | lut[b >> bits] << 16)
    float* part = (float*)(pair_s + (size_t)entries * 64);   // [nwaves][64]
    const uint32_t n0 = nt * 64u, n = n0 + lane;
    const bool col_ok = n < p.N;
    const uint32_t nc = col_ok ? n : p.N - 1u;               // columns past the end re-read the last one
    const uint16_t* lrow = (const uint16_t*)p.lut + ((size_t)nc << p.bits);
    const DD_SCALAR_AS uint32_t* xs = (const DD_SCALAR_AS uint32_t*)p.x;
    const uint32_t k0 = (ktile * nwaves + wave) * p.kslice;
    const uint32_t k1 = (k0 + p.kslice) < p.K ? (k0 + p.kslice) : p.K;    // may be <= k0: nothing to do
    const uint32_t* col = p.mat + nc;
    float acc = 0.f;
    const unsigned char* lt = (const unsigned char*)pair_s;
    uint32_t lane4 = lane * 4u;

    if (p.bits == 4) {
        // the first words of the wave's K range are requested before the table is built (they do not depend on it),
        // and inside the loop the next words before the lookups of the current ones
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (k0 < k1) {
#pragma unroll
            for (int u = 0; u < 4; ++u) w[u] = __builtin_nontemporal_load(col + (size_t)(k0 / 8u + u) * p.N);
        }
        // build: this thread's column, high field = wave, low field 0..15
        {
            const u32x4 a = *(const u32x4*)lrow, b = *(const u32x4*)(lrow + 8);
            const uint32_t vh = (uint32_t)lrow[wave] << 16;
            uint32_t* dst = pair_s + (size_t)(wave * 16u) * 64 + lane;
#pragma unroll
            for (int lo = 0; lo < 16; ++lo) {
                const uint32_t dw = (lo < 8) ? a[(lo >> 1) & 3] : b[(lo >> 1) & 3];     // indices are constants after unrolling
                dst[lo * 64] = ((lo & 1) ? (dw >> 16) : (dw & 0xFFFFu)) | vh;
            }
        }
        __syncthreads();
        uint32_t m = 0xFF00u;
        asm volatile("" : "+v"(m), "+v"(lane4));
#pragma unroll 1
        for (uint32_t c = k0; c < k1; c += 32u) {
            uint32_t wn[4] = {w[0], w[1], w[2], w[3]};
            if (c + 32u < k1) {                                  // uniform in the wave
#pragma unroll
                for (int u = 0; u < 4; ++u) wn[u] = __builtin_nontemporal_load(col + (size_t)((c + 32u) / 8u + u) * p.N);
            }
            uint32_t xd[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) xd[i] = xs[(c >> 1) + i];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t sh = (k == 0) ? (w[u] << 8) : (k == 1) ? w[u] : (w[u] >> (8 * k - 8));
                    const uint32_t pr = *(const uint32_t*)(lt + ((sh & m) | lane4));
                    acc = sqllm_dot2<DT>(pr, xd[4 * u + k], acc);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) w[u] = wn[u];
        }
    } else {
        uint32_t w[3] = {0u, 0u, 0u};                            // requested ahead, as in the 4-bit path
        if (k0 < k1) {
#pragma unroll
            for (int u = 0; u < 3; ++u) w[u] = __builtin_nontemporal_load(col + (size_t)(3u * (k0 / 32u) + u) * p.N);
        }
        // 3-bit: 64 entries; high field = wave / 2, low fields 4 (wave & 1) .. + 3
        {
            const u32x4 a = *(const u32x4*)lrow;
            const uint32_t hi = wave >> 1, lo0 = (wave & 1u) * 4u;
            const uint32_t vh = (uint32_t)lrow[hi] << 16;
            uint32_t* dst = pair_s + (size_t)(hi * 8u + lo0) * 64 + lane;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t dw = (wave & 1u) ? a[2 + (q >> 1)] : a[q >> 1];
                dst[q * 64] = ((q & 1) ? (dw >> 16) : (dw & 0xFFFFu)) | vh;
            }
        }
        __syncthreads();
        uint32_t m = 0x3F00u;
        asm volatile("" : "+v"(m), "+v"(lane4));
#pragma unroll 1
        for (uint32_t c = k0; c < k1; c += 32u) {
            uint32_t wn[3] = {w[0], w[1], w[2]};
            if (c + 32u < k1) {                                  // uniform in the wave
#pragma unroll
                for (int u = 0; u < 3; ++u) wn[u] = __builtin_nontemporal_load(col + (size_t)(3u * ((c + 32u) / 32u) + u) * p.N);
            }
            uint32_t xd[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) xd[i] = xs[(c >> 1) + i];
            // pair k = fields 2k, 2k+1 = six bits at bit 6k of the 96-bit stream w[2]:w[1]:w[0]
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                const int bit = 6 * k, wi = bit >> 5, off = bit & 31;
                uint32_t v;                          // (six bits << 8) plus bits outside the mask
                if (off <= 26) v = (off >= 8) ? (w[wi] >> (off - 8)) : (w[wi] << (8 - off));
                else v = __builtin_amdgcn_alignbit(w[wi + 1], w[wi], off - 8);
                const uint32_t pr = *(const uint32_t*)(lt + ((v & m) | lane4));
                acc = sqllm_dot2<DT>(pr, xd[k], acc);
            }
#pragma unroll
            for (int u = 0; u < 3; ++u) w[u] = wn[u];
        }
    }
    part[wave * 64u + lane] = acc;
    __syncthreads();
    if (wave == 0 && (lane & 1u) == 0u && col_ok) {
        float v0 = 0.f, v1 = 0.f;
        for (uint32_t w2 = 0; w2 < nwaves; ++w2) { v0 += part[w2 * 64u + lane]; v1 += part[w2 * 64u + lane + 1u]; }
        if (n + 1u < p.N) E::atomic_add2(p.out, n, v0, v1);
        else E::atomic_add1(p.out, n, v0);
    }
}

// The 32 activations of channels c0 .. c0+31 as fp32 SGPR values: raw storage comes through the scalar
// cache (the address is wave-uniform), element e is converted where it is used.
template <int DT> struct SqllmX;
template <> struct SqllmX<kFP32> {
    uint32_t d[32];
    __device__ __forceinline__ void load(const void* x, uint32_t c0) {
        const DD_SCALAR_AS uint32_t* s = (const DD_SCALAR_AS uint32_t*)x + c0;
#pragma unroll
        for (int i = 0; i < 32; ++i) d[i] = s[i];
    }
    __device__ __forceinline__ float fma(int e, float w, float acc) const { return __builtin_fmaf(w, __uint_as_float(d[e]), acc); }
};
template <> struct SqllmX<kFP16> {
    uint32_t d[16];
    __device__ __forceinline__ void load(const void* x, uint32_t c0) {
        const DD_SCALAR_AS uint32_t* s = (const DD_SCALAR_AS uint32_t*)x + (c0 >> 1);
#pragma unroll
        for (int i = 0; i < 16; ++i) d[i] = s[i];
    }
    __device__ __forceinline__ float fma(int e, float w, float acc) const {
        const half2_t h = *(const half2_t*)&d[e >> 1];
        return __builtin_fmaf(w, (float)h[e & 1], acc);       // mixed-precision fma, the half comes from an SGPR
    }
};
template <> struct SqllmX<kBF16> {
    uint32_t d[16];
    __device__ __forceinline__ void load(const void* x, uint32_t c0) {
        const DD_SCALAR_AS uint32_t* s = (const DD_SCALAR_AS uint32_t*)x + (c0 >> 1);
#pragma unroll
        for (int i = 0; i < 16; ++i) d[i] = s[i];
    }
    __device__ __forceinline__ float fma(int e, float w, float acc) const {
        const uint32_t b = (e & 1) ? (d[e >> 1] & 0xFFFF0000u) : (d[e >> 1] << 16);
        return __builtin_fmaf(w, __uint_as_float(b), acc);
    }
};

template <int DT>
__device__ __forceinline__ void sqllm_role(const SqllmParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    if constexpr (DT != kFP32) {
        sqllm_role_pairs<DT>(p, bid, smem);
        return;
    }
    const uint32_t tid = threadIdx.x, lane = tid & 63u, nthreads = blockDim.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = nthreads >> 6;
    const uint32_t nt = bid % p.n_tiles, ktile = bid / p.n_tiles;
    const uint32_t L = 1u << p.bits;
    float* lut_s = (float*)smem;                    // [L][64]
    float* part = lut_s + (size_t)L * 64;           // [nwaves][64]
    const uint32_t n0 = nt * 64u, n = n0 + lane;
    const bool col_ok = n < p.N;
    const uint32_t nc = col_ok ? n : p.N - 1u;      // columns past the end re-read the last one

    // the 64 columns' LUTs: entry idx = col * L + value, coalesced in memory
    for (uint32_t idx = tid; idx < 64u * L; idx += nthreads) {
        const uint32_t col = idx >> p.bits, v = idx & (L - 1u);
        const uint32_t cn = (n0 + col < p.N) ? n0 + col : p.N - 1u;
        lut_s[v * 64u + col] = E::load(p.lut, (size_t)cn * L + v);
    }
    const uint32_t k0 = (ktile * nwaves + wave) * p.kslice;
    const uint32_t k1 = (k0 + p.kslice) < p.K ? (k0 + p.kslice) : p.K;    // may be <= k0: nothing to do
    __syncthreads();

    float acc = 0.f;
    const unsigned char* lt = (const unsigned char*)(lut_s + lane);       // + value * 256 bytes
    const uint32_t* col = p.mat + nc;
    if (p.bits == 4) {
        uint32_t m = 0xF00u;
        asm volatile("" : "+v"(m));                 // mask in a VGPR: all-VGPR operations issue at twice the rate
#pragma unroll 1
        for (uint32_t c = k0; c < k1; c += 32u) {
            uint32_t w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) w[u] = __builtin_nontemporal_load(col + (size_t)(c / 8u + u) * p.N);
            SqllmX<DT> xs;
            xs.load(p.x, c);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t sh = (4 * j >= 8) ? (w[u] >> (4 * j - 8)) : (w[u] << (8 - 4 * j));
                    const float wv = *(const float*)(lt + (sh & m));
                    acc = xs.fma(8 * u + j, wv, acc);
                }
            }
        }
    } else {
        uint32_t m = 0x700u;
        asm volatile("" : "+v"(m));
#pragma unroll 1
        for (uint32_t c = k0; c < k1; c += 32u) {
            uint32_t w[3];
#pragma unroll
            for (int u = 0; u < 3; ++u) w[u] = __builtin_nontemporal_load(col + (size_t)(3u * (c / 32u) + u) * p.N);
            SqllmX<DT> xs;
            xs.load(p.x, c);
            // field j sits at bit 3j of the 96-bit stream w[2]:w[1]:w[0]; fields 10 and 21 straddle words
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const int bit = 3 * j, wi = bit >> 5, off = bit & 31;
                uint32_t v;                          // (field << 8) plus bits outside the mask
                if (off <= 29) {
                    v = (off >= 8) ? (w[wi] >> (off - 8)) : (w[wi] << (8 - off));
                } else {
                    const uint32_t f = __builtin_amdgcn_alignbit(w[wi + 1], w[wi], off);   // stream >> bit, low 32 bits
                    v = f << 8;
                }
                const float wv = *(const float*)(lt + (v & m));
                acc = xs.fma(j, wv, acc);
            }
        }
    }
    part[wave * 64u + lane] = acc;
    __syncthreads();
    // columns n and n+1 sit in neighbouring lanes (tile origins are even): one packed atomic per pair
    if (wave == 0 && (lane & 1u) == 0u && col_ok) {
        float v0 = 0.f, v1 = 0.f;
        for (uint32_t w = 0; w < nwaves; ++w) { v0 += part[w * 64u + lane]; v1 += part[w * 64u + lane + 1u]; }
        if (n + 1u < p.N) E::atomic_add2(p.out, n, v0, v1);
        else E::atomic_add1(p.out, n, v0);
    }
}

}  // namespace decdec
