// LUT-GEMM (binary-coding quantisation) GEMV role, batch 1:
//   out[n] += sum_g [ q_bias[g][n] * sum_{c in g} x[c]
//                     + sum_b alpha[g][b][n] * sum_{c in g} s_b(n, c) * x[c] ],   s = +1/-1
// with s_b(n, c) = bit (c % 32) of q_weight[c / 32][b][n]  (reference
// decdec_extension/lutgemm.cu:25-150; packing llm-awq/quantize/qmodule.py:61-92).
//
// A lane owns one output column (the packed words of 64 neighbouring columns are one coalesced 256-byte
// wave load); the waves of a workgroup work on the same 64 columns and split the workgroup's K range.
// The signed sums depend on the activations only, so the workgroup first builds, for every group of FOUR
// channels of its K range, the 16-entry table of signed subset sums in LDS (fp32: entries carry no
// rounding); a 32-bit word of a bit plane then costs eight lookups.  Sixteen-entry tables are 16
// consecutive dwords, i.e. 16 different LDS banks: whatever nibbles the 64 lanes hold, a lookup is
// conflict-free (equal nibbles are one broadcast), which 256-entry byte tables are not.  Partial sums stay
// in fp32 registers, the waves are added in LDS, and an output receives one atomic add per workgroup
// (k_tiles per output) instead of the reference's K / 32.
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
    uint32_t slice_tiles;      // 32-channel tiles per wave
    uint32_t n_tiles, k_tiles; // column groups of 64 x K ranges of (waves per workgroup) * slice_tiles tiles
};

constexpr int kLutgemmMaxBits = 8;

__host__ __device__ inline size_t lutgemm_lds_bytes(uint32_t slice_tiles, uint32_t waves) {
    const size_t tiles = (size_t)slice_tiles * waves;
    return 512 + tiles * 8 * 16 * 4 + tiles * 4 + (size_t)waves * 64 * 4;    // 512: the tables are aligned to their size
}

#define DD_LDS_AS __attribute__((address_space(3)))

// signed sum of the 32 activations of a tile selected by the bits of w: eight conflict-free lookups.
// tb = LDS byte address of the tile's tables (a multiple of 512), m = 0x3C in a VGPR; a lookup is a
// shift, an and-or that forms the address, the read and an add.
__device__ __forceinline__ float lutgemm_word(uint32_t tb, uint32_t w, uint32_t m) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t sh = (j == 0) ? (w << 2) : (w >> (4 * j - 2));
        const uint32_t addr = (sh & m) | tb;
        s += *(const DD_LDS_AS float*)(uintptr_t)(addr + j * 64);
    }
    return s;
}

// The walk of one wave over its tiles for a compile-time number of bit planes: all requests of a tile
// (plane words, alpha, bias) are issued before its lookups.
template <int DT, int BITS>
__device__ __forceinline__ float lutgemm_tiles(const LutgemmParams& p, uint32_t t0, uint32_t lt0, uint32_t lt1,
                                               uint32_t nc, uint32_t tab_lds, const float* xsum) {
    using E = Elem<DT>;
    uint32_t m = 0x3Cu;
    asm volatile("" : "+v"(m));                      // mask in a VGPR
    float acc = 0.f;
#pragma unroll 1
    for (uint32_t lt = lt0; lt < lt1; ++lt) {
        const uint32_t gt = t0 + lt;                 // global tile
        const uint32_t g = (32u * gt) / p.group_size;
        uint32_t w[BITS], araw[BITS];
#pragma unroll
        for (int b = 0; b < BITS; ++b) {
            w[b] = __builtin_nontemporal_load(p.qw + ((size_t)gt * BITS + b) * p.N + nc);
            araw[b] = E::load_raw(p.alpha, ((size_t)g * BITS + b) * p.N + nc);
        }
        const uint32_t braw = E::load_raw(p.q_bias, (size_t)g * p.N + nc);
        const uint32_t tb = tab_lds + lt * 512u;
        acc += E::from_raw(braw) * xsum[lt];
#pragma unroll
        for (int b = 0; b < BITS; ++b) acc += E::from_raw(araw[b]) * lutgemm_word(tb, w[b], m);
    }
    return acc;
}

// The same walk with the requests of the next tile issued before the lookups of the current one, and the requests
// of the first tile issued by the caller before the tables are built (they do not depend on the tables), so that
// the first memory round trip of a wave runs behind the table build instead of after it.
template <int DT, int BITS>
struct LutgemmTile {
    uint32_t w[BITS], araw[BITS], braw;
};
template <int DT, int BITS>
__device__ __forceinline__ void lutgemm_issue(const LutgemmParams& p, uint32_t gt, uint32_t nc, LutgemmTile<DT, BITS>& r) {
    using E = Elem<DT>;
    const uint32_t g = (32u * gt) / p.group_size;
#pragma unroll
    for (int b = 0; b < BITS; ++b) {
        r.w[b] = __builtin_nontemporal_load(p.qw + ((size_t)gt * BITS + b) * p.N + nc);
        r.araw[b] = E::load_raw(p.alpha, ((size_t)g * BITS + b) * p.N + nc);
    }
    r.braw = E::load_raw(p.q_bias, (size_t)g * p.N + nc);
}
template <int DT, int BITS>
__device__ __forceinline__ float lutgemm_tiles_ahead(const LutgemmParams& p, uint32_t t0, uint32_t lt0, uint32_t lt1,
                                                     uint32_t nc, uint32_t tab_lds, const float* xsum,
                                                     LutgemmTile<DT, BITS> cur) {
    using E = Elem<DT>;
    uint32_t m = 0x3Cu;
    asm volatile("" : "+v"(m));                      // mask in a VGPR
    float acc = 0.f;
#pragma unroll 1
    for (uint32_t lt = lt0; lt < lt1; ++lt) {
        LutgemmTile<DT, BITS> nxt = cur;
        if (lt + 1u < lt1) lutgemm_issue<DT, BITS>(p, t0 + lt + 1u, nc, nxt);     // uniform in the wave
        const uint32_t tb = tab_lds + lt * 512u;
        acc += E::from_raw(cur.braw) * xsum[lt];
#pragma unroll
        for (int b = 0; b < BITS; ++b) acc += E::from_raw(cur.araw[b]) * lutgemm_word(tb, cur.w[b], m);
        cur = nxt;
    }
    return acc;
}

template <int DT>
__device__ __forceinline__ void lutgemm_role(const LutgemmParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, nthreads = blockDim.x;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = nthreads >> 6;
    const uint32_t nt = bid % p.n_tiles, ktile = bid / p.n_tiles;
    const uint32_t total_tiles = p.K / 32u;
    const uint32_t wg_tiles = p.slice_tiles * nwaves;
    const uint32_t t0 = ktile * wg_tiles;                                   // first tile of the workgroup
    const uint32_t nt_wg = (t0 + wg_tiles) <= total_tiles ? wg_tiles : (total_tiles - t0);
    // tables start at a multiple of 512 bytes of LDS, so that a table address can be formed with an OR
    const uint32_t smem_lds = (uint32_t)(uintptr_t)(DD_LDS_AS unsigned char*)smem;
    float* tab = (float*)(smem + ((512u - (smem_lds & 511u)) & 511u));   // [wg_tiles][8][16]
    float* xsum = tab + (size_t)wg_tiles * 128;      // [wg_tiles]
    float* part = xsum + wg_tiles;                   // [nwaves][64]

    const uint32_t n0 = nt * 64u, n = n0 + lane;
    const bool col_ok = n < p.N;
    const uint32_t nc = col_ok ? n : p.N - 1u;       // columns past the end re-read the last one
    const uint32_t lt0 = wave * p.slice_tiles;       // local tiles of this wave: [lt0, lt1)
    const uint32_t lt1 = (lt0 + p.slice_tiles) < nt_wg ? (lt0 + p.slice_tiles) : nt_wg;
    // three planes (the usual format): the wave's first tile is requested before the tables exist
    constexpr int kAhead = 3;
    LutgemmTile<DT, kAhead> first = {};
    const bool ahead = p.bits == (uint32_t)kAhead;
    if (ahead && lt0 < lt1) lutgemm_issue<DT, kAhead>(p, t0 + lt0, nc, first);

    // tables: tab[(tile * 8 + j) * 16 + pat] = sum_i (bit i of pat ? +1 : -1) * x[32 tile + 4 j + i]; the eight tables
    // of a tile are built by eight neighbouring lanes, which also add up the tile's plain sum (the factor of q_bias)
    for (uint32_t T = tid; T < nt_wg * 8u; T += nthreads) {
        const size_t c0 = (size_t)32 * t0 + (size_t)4 * T;
        const float x0 = E::load(p.x, c0), x1 = E::load(p.x, c0 + 1), x2 = E::load(p.x, c0 + 2), x3 = E::load(p.x, c0 + 3);
        const float lo[4] = {-x0 - x1, x0 - x1, -x0 + x1, x0 + x1};
        const float hi[4] = {-x2 - x3, x2 - x3, -x2 + x3, x2 + x3};
        float* dst = tab + (size_t)T * 16;
#pragma unroll
        for (int q = 0; q < 16; ++q) dst[q] = lo[q & 3] + hi[q >> 2];
        float sx = lo[3] + hi[3];
        sx += __shfl_xor(sx, 1, 64);
        sx += __shfl_xor(sx, 2, 64);
        sx += __shfl_xor(sx, 4, 64);
        if ((T & 7u) == 0u) xsum[T >> 3] = sx;
    }
    __syncthreads();

    const uint32_t tab_lds = (uint32_t)(uintptr_t)(DD_LDS_AS float*)tab;    // LDS byte address of the tables
    float acc;
    if (ahead) acc = lutgemm_tiles_ahead<DT, kAhead>(p, t0, lt0, lt1, nc, tab_lds, xsum, first);
    else switch (p.bits) {
        case 1: acc = lutgemm_tiles<DT, 1>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 2: acc = lutgemm_tiles<DT, 2>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 3: acc = lutgemm_tiles<DT, 3>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 4: acc = lutgemm_tiles<DT, 4>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 5: acc = lutgemm_tiles<DT, 5>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 6: acc = lutgemm_tiles<DT, 6>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        case 7: acc = lutgemm_tiles<DT, 7>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
        default: acc = lutgemm_tiles<DT, 8>(p, t0, lt0, lt1, nc, tab_lds, xsum); break;
    }
    part[wave * 64u + lane] = acc;
    __syncthreads();
    // columns n and n+1 sit in neighbouring lanes (tile origins are even): one packed atomic per pair
    if (wave == 0 && (lane & 1u) == 0u && col_ok) {
        float v0 = 0.f, v1 = 0.f;
        for (uint32_t w2 = 0; w2 < nwaves; ++w2) { v0 += part[w2 * 64u + lane]; v1 += part[w2 * 64u + lane + 1u]; }
        if (n + 1u < p.N) E::atomic_add2(p.out, n, v0, v1);
        else E::atomic_add1(p.out, n, v0);
    }
}

}  // namespace decdec
