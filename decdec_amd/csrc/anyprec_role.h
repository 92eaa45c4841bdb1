// Any-precision bitplane GEMV role (batch 1):  out[n] += sum_c lut[n][idx(n, c)] * x[c].
//
// Weight layout (reference decdec_extension/anyprec.cu:297-329 and :411-475): qweight[p][n][w],
// plane 0 = MSB of the LUT index, w = 32*i + t for 1024-channel chunk i and word t; bit
// 31 - (8j + e) of word (i, t) belongs to channel 1024 i + 8 eff j + 8 t + e, j in [0,4), e in [0,8),
// eff = 32 for full chunks and (K % 1024)/32 for a tail chunk.
//
// Mapping: a wave owns one slice of 64 consecutive words (2048 channels) of the row and keeps the
// matching 32 activations per lane in registers for every row it visits; the S slices of a row sit in
// S waves of the same workgroup and are summed in LDS, so each output receives exactly one atomic add
// (the reference's accumulate-into-output contract).  Weights stream from HBM as coalesced 256-byte
// wave loads per plane; several rows are in flight per wave.
//
// The 3-bit path keeps the row's 8-entry LUT in four VGPRs as two byte tables and looks weights up
// with v_perm_b32 (four table lookups per instruction), then multiplies with v_dot2_f32_f16 /
// v_dot2_f32_bf16 into an fp32 accumulator: no LDS traffic in the inner loop.  Other bit widths use
// a per-wave LDS copy of the row's LUT.
#pragma once
#include "common.h"

namespace decdec {

struct AnyprecParams {
    const void* x;
    const uint32_t* qweight;
    const void* lut;
    void* out;
    uint32_t N, K, W;      // W = K / 32 words per row per plane
    uint32_t S;            // slices (waves) per row handled inside one workgroup (<= 16)
    uint32_t sgroups;      // slice groups (> 1 only when ceil(W/64) > 16, i.e. K > 32768)
    uint32_t rg;           // row groups per workgroup
    uint32_t rpw;          // rows per wave: 2, 4 or 8, all in flight together
    uint32_t x_aligned;    // activation pointer is 16-byte aligned
    // tile decoder (3-bit, K a multiple of 1024): waves per tile (0 = not used), K-tiles per row group, tiles
    uint32_t tile_cs, tile_kt, tiles;
};

__host__ __device__ inline size_t anyprec_lds_bytes(uint32_t S, uint32_t rg, uint32_t rpw, int bits) {
    size_t b = (size_t)S * rg * rpw * 4;
    if (bits != 3) b += (size_t)S * rg * 256 * 4;     // per-wave LUT copy
    return b;
}

template <int DT>
__device__ __forceinline__ float dot2_acc(uint32_t w, uint32_t x, float acc) {
    if constexpr (DT == kFP16) {
        return __builtin_amdgcn_fdot2(*(half2_t*)&w, *(half2_t*)&x, acc, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(*(bf16x2_t*)&w, *(bf16x2_t*)&x, acc, false);
    }
}

// The 32 activations that belong to word `wi` of a row: issue the loads (xr[j] = the eight 16-bit values
// of group j), then arrange them for the decoders below:
// xp[e][0] = (x[j=3][e], x[j=2][e]),  xp[e][1] = (x[j=1][e], x[j=0][e])  as packed 16-bit pairs.
__device__ __forceinline__ void anyprec_issue_x(const AnyprecParams& p, uint32_t wi, uint32_t (&xr)[4][4]) {
    const uint32_t i = wi >> 5, t = wi & 31u;
    const uint32_t eff = (i == p.K / 1024u) ? (p.K % 1024u) / 32u : 32u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const size_t c0 = (size_t)1024 * i + (size_t)8 * eff * j + (size_t)8 * t;
        const uint16_t* src = (const uint16_t*)p.x + c0;
        if (p.x_aligned) {
            const u32x4 v = *(const u32x4*)src;
            xr[j][0] = v[0]; xr[j][1] = v[1]; xr[j][2] = v[2]; xr[j][3] = v[3];
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) xr[j][q] = (uint32_t)src[2 * q] | ((uint32_t)src[2 * q + 1] << 16);
        }
    }
}
__device__ __forceinline__ void anyprec_arrange_x(const uint32_t (&xr)[4][4], uint32_t (&xp)[8][2]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        xp[e][0] = __builtin_amdgcn_perm(xr[2][e >> 1], xr[3][e >> 1], sel);   // lo = j3, hi = j2
        xp[e][1] = __builtin_amdgcn_perm(xr[0][e >> 1], xr[1][e >> 1], sel);   // lo = j1, hi = j0
    }
}

// Bit masks of the 3-bit decoder, kept in VGPRs: a VALU operation whose sources are all VGPRs (or inline
// constants) issues at twice the rate of one that reads an SGPR or a 32-bit literal.
struct Anyprec3Masks {
    uint32_t m8, m4, m2, k7;
    __device__ __forceinline__ void init() {
        m8 = 0x88888888u; m4 = 0x44444444u; m2 = 0x22222222u; k7 = 0x07070707u;
        asm volatile("" : "+v"(m8), "+v"(m4), "+v"(m2), "+v"(k7));
    }
};
// bits of a where m is set, bits of b elsewhere (one three-input bit operation)
__device__ __forceinline__ uint32_t bit_select(uint32_t m, uint32_t a, uint32_t b) { return ((a ^ b) & m) ^ b; }

// One word of a 3-bit row: 32 weights looked up through byte-permutes and dotted with xp.
// lo0/lo1/hi0/hi1 are the row's byte tables: LO = low bytes of LUT entries 0..7, HI = high bytes.
template <int DT>
__device__ __forceinline__ float anyprec3_word(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t lo0, uint32_t lo1,
                                               uint32_t hi0, uint32_t hi1, const Anyprec3Masks& mk,
                                               const uint32_t (&xp)[8][2], float acc) {
    // index words: nibble n of T_o carries the 3-bit index of bit 4n+o (o = 3..0) at nibble bits 2..0; the
    // fourth nibble bit is garbage and masked below.
    const uint32_t r1 = q1 >> 1, r2 = q2 >> 2, l0 = q0 << 2, l1 = q1 << 1;
    const uint32_t t3 = bit_select(mk.m8, q0, bit_select(mk.m4, r1, r2)) >> 1;
    const uint32_t t2 = bit_select(mk.m4, q0, bit_select(mk.m2, r1, r2));
    const uint32_t t1 = bit_select(mk.m8, l0, bit_select(mk.m4, l1, q2)) >> 1;
    const uint32_t t0 = bit_select(mk.m4, l0, bit_select(mk.m2, l1, q2));
    // selector bytes 0..3 <-> j = 3..0; element e per selector as listed
    const uint32_t sel[8] = {
        (t3 >> 4) & mk.k7,   // e = 0
        (t2 >> 4) & mk.k7,   // e = 1
        (t1 >> 4) & mk.k7,   // e = 2
        (t0 >> 4) & mk.k7,   // e = 3
        t3 & mk.k7,          // e = 4
        t2 & mk.k7,          // e = 5
        t1 & mk.k7,          // e = 6
        t0 & mk.k7,          // e = 7
    };
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t L = __builtin_amdgcn_perm(lo1, lo0, sel[e]);
        const uint32_t H = __builtin_amdgcn_perm(hi1, hi0, sel[e]);
        const uint32_t w32 = __builtin_amdgcn_perm(H, L, 0x05010400u);   // weights j3, j2
        const uint32_t w10 = __builtin_amdgcn_perm(H, L, 0x07030602u);   // weights j1, j0
        acc = dot2_acc<DT>(w32, xp[e][0], acc);
        acc = dot2_acc<DT>(w10, xp[e][1], acc);
    }
    return acc;
}
// byte tables of a row's eight 16-bit LUT entries (two per dword of lut4)
__device__ __forceinline__ void anyprec3_tables(const u32x4 lut4, uint32_t& lo0, uint32_t& lo1, uint32_t& hi0, uint32_t& hi1) {
    lo0 = __builtin_amdgcn_perm(lut4[1], lut4[0], 0x06040200u);
    hi0 = __builtin_amdgcn_perm(lut4[1], lut4[0], 0x07050301u);
    lo1 = __builtin_amdgcn_perm(lut4[3], lut4[2], 0x06040200u);
    hi1 = __builtin_amdgcn_perm(lut4[3], lut4[2], 0x07050301u);
}

// One word of a 4-bit row, same scheme with 16-entry tables: the low three index bits select inside a table half
// (entries 0..7 in LO[0..1] / HI[0..1], 8..15 in LO[2..3] / HI[2..3]), the fourth picks the half bytewise.
struct Anyprec4Masks {
    uint32_t m8, m4, m2, k7, k1;
    __device__ __forceinline__ void init() {
        m8 = 0x88888888u; m4 = 0x44444444u; m2 = 0x22222222u; k7 = 0x07070707u; k1 = 0x01010101u;
        asm volatile("" : "+v"(m8), "+v"(m4), "+v"(m2), "+v"(k7), "+v"(k1));
    }
};
template <int DT>
__device__ __forceinline__ float anyprec4_word(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t q3,
                                               const uint32_t (&lo)[4], const uint32_t (&hi)[4], const Anyprec4Masks& mk,
                                               const uint32_t (&xp)[8][2], float acc) {
    // index words: nibble n of T_o carries the 4-bit index of bit 4n+o (plane 0 = most significant bit)
    const uint32_t t3 = bit_select(mk.m8, q0, bit_select(mk.m4, q1 >> 1, bit_select(mk.m2, q2 >> 2, q3 >> 3)));
    const uint32_t t2 = bit_select(mk.m8, q0 << 1, bit_select(mk.m4, q1, bit_select(mk.m2, q2 >> 1, q3 >> 2)));
    const uint32_t t1 = bit_select(mk.m8, q0 << 2, bit_select(mk.m4, q1 << 1, bit_select(mk.m2, q2, q3 >> 1)));
    const uint32_t t0 = bit_select(mk.m8, q0 << 3, bit_select(mk.m4, q1 << 2, bit_select(mk.m2, q2 << 1, q3)));
    const uint32_t tt[4] = {t3, t2, t1, t0};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        // selector bytes 0..3 <-> j = 3..0; e < 4: the upper nibbles of T_(3-e), e >= 4: the lower nibbles of T_(7-e)
        const uint32_t t = (e < 4) ? (tt[e] >> 4) : tt[e - 4];
        const uint32_t sel = t & mk.k7;
        const uint32_t half = ((t >> 3) & mk.k1) * 255u;                    // 0xFF in the bytes whose index is >= 8
        const uint32_t L = bit_select(half, __builtin_amdgcn_perm(lo[3], lo[2], sel), __builtin_amdgcn_perm(lo[1], lo[0], sel));
        const uint32_t H = bit_select(half, __builtin_amdgcn_perm(hi[3], hi[2], sel), __builtin_amdgcn_perm(hi[1], hi[0], sel));
        const uint32_t w32 = __builtin_amdgcn_perm(H, L, 0x05010400u);   // weights j3, j2
        const uint32_t w10 = __builtin_amdgcn_perm(H, L, 0x07030602u);   // weights j1, j0
        acc = dot2_acc<DT>(w32, xp[e][0], acc);
        acc = dot2_acc<DT>(w10, xp[e][1], acc);
    }
    return acc;
}
// byte tables of a row's sixteen 16-bit LUT entries (two per dword)
__device__ __forceinline__ void anyprec4_tables(const u32x4 a, const u32x4 b, uint32_t (&lo)[4], uint32_t (&hi)[4]) {
    lo[0] = __builtin_amdgcn_perm(a[1], a[0], 0x06040200u); hi[0] = __builtin_amdgcn_perm(a[1], a[0], 0x07050301u);
    lo[1] = __builtin_amdgcn_perm(a[3], a[2], 0x06040200u); hi[1] = __builtin_amdgcn_perm(a[3], a[2], 0x07050301u);
    lo[2] = __builtin_amdgcn_perm(b[1], b[0], 0x06040200u); hi[2] = __builtin_amdgcn_perm(b[1], b[0], 0x07050301u);
    lo[3] = __builtin_amdgcn_perm(b[3], b[2], 0x06040200u); hi[3] = __builtin_amdgcn_perm(b[3], b[2], 0x07050301u);
}

// Generic bit width: indices assembled bytewise, weights from a per-wave LDS copy of the LUT (fp32).
template <int DT, int BITS>
__device__ __forceinline__ float anyprec_generic_word(const uint32_t (&q)[BITS], const float* wlut,
                                                      const uint32_t (&xp)[8][2], float acc) {
#pragma unroll
    for (int o = 0; o < 8; ++o) {
        uint32_t u = 0;
#pragma unroll
        for (int pl = 0; pl < BITS; ++pl) u |= ((q[pl] >> o) & 0x01010101u) << (BITS - 1 - pl);
        const int e = 7 - o;                               // byte k of u <-> j = 3 - k
        const float w3 = wlut[u & 0xFFu], w2 = wlut[(u >> 8) & 0xFFu];
        const float w1 = wlut[(u >> 16) & 0xFFu], w0 = wlut[u >> 24];
        float x3, x2, x1, x0;
        if constexpr (DT == kFP16) {
            const half2_t a = *(const half2_t*)&xp[e][0], b = *(const half2_t*)&xp[e][1];
            x3 = (float)a[0]; x2 = (float)a[1]; x1 = (float)b[0]; x0 = (float)b[1];
        } else {
            x3 = __uint_as_float(xp[e][0] << 16); x2 = __uint_as_float(xp[e][0] & 0xFFFF0000u);
            x1 = __uint_as_float(xp[e][1] << 16); x0 = __uint_as_float(xp[e][1] & 0xFFFF0000u);
        }
        acc += w3 * x3; acc += w2 * x2; acc += w1 * x1; acc += w0 * x0;
    }
    return acc;
}

// Sum over the 64 lanes with DPP adds (no LDS traffic); the total ends up in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_read(float x) {
    // lanes outside ROW_MASK, and lanes whose source is out of range, read 0
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(x), CTRL, ROW_MASK, 0xF, true));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_read<0xB1, 0xF>(v);     // quad_perm [1,0,3,2]
    v += dpp_read<0x4E, 0xF>(v);     // quad_perm [2,3,0,1]
    v += dpp_read<0x124, 0xF>(v);    // row_ror 4
    v += dpp_read<0x128, 0xF>(v);    // row_ror 8: every lane of a 16-lane row holds the row sum
    v += dpp_read<0x142, 0xA>(v);    // row_bcast 15: rows 1 and 3 add the sum of the row before
    v += dpp_read<0x143, 0xC>(v);    // row_bcast 31: rows 2 and 3 add the sum of rows 0..1
    return v;
}

// The same reduction for G values at once, written out so that every step is ONE instruction
// (v_add_f32_dpp with destination = second source; lanes disabled by row_mask keep their value, which is
// "add zero") and so that the steps of the G values interleave: a DPP source must not be read in the two
// issue slots after the instruction that wrote it.
#define DD_DPP_STEP(ctrl) \
    "v_add_f32_dpp %0, %0, %0 " ctrl "\n v_add_f32_dpp %1, %1, %1 " ctrl "\n" \
    "v_add_f32_dpp %2, %2, %2 " ctrl "\n v_add_f32_dpp %3, %3, %3 " ctrl "\n"
__device__ __forceinline__ void wave_sum_dpp4(float& a, float& b, float& c, float& d) {
    asm volatile("s_nop 1\n"
                 DD_DPP_STEP("quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf")
                 DD_DPP_STEP("quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf")
                 DD_DPP_STEP("row_ror:4 row_mask:0xf bank_mask:0xf")
                 DD_DPP_STEP("row_ror:8 row_mask:0xf bank_mask:0xf")
                 DD_DPP_STEP("row_bcast:15 row_mask:0xa bank_mask:0xf")
                 DD_DPP_STEP("row_bcast:31 row_mask:0xc bank_mask:0xf")
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
#undef DD_DPP_STEP
template <int RB>
__device__ __forceinline__ void wave_sum_rows(float (&v)[RB]) {
    if constexpr (RB % 4 == 0) {
#pragma unroll
        for (int r = 0; r < RB; r += 4) wave_sum_dpp4(v[r], v[r + 1], v[r + 2], v[r + 3]);
    } else {
#pragma unroll
        for (int r = 0; r < RB; ++r) v[r] = wave_sum_dpp(v[r]);
    }
}

#define DD_CONST_AS __attribute__((address_space(4)))

// One wave's share of the GEMV: slice `s` of RB consecutive rows.  All weight words of the RB rows are
// requested before anything is decoded (a batch-1 GEMV is bound by the bytes it keeps in flight); the
// rows' LUTs come through the scalar cache (the address is wave-uniform), so they cost no VGPRs while
// the weights are in flight.
template <int DT, int BITS, int RB>
__device__ __forceinline__ void anyprec_rows(const AnyprecParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform by construction
    const uint32_t s = wave % p.S, g = wave / p.S;
    const uint32_t rows_per_block = p.rg * RB;
    const uint32_t sgrp = bid % p.sgroups, tile = bid / p.sgroups;
    const uint32_t block_row0 = tile * rows_per_block;
    const bool wave_active = g < p.rg;
    const uint32_t wi = (sgrp * p.S + s) * kWave + lane;    // word index inside the row
    const bool lane_ok = wi < p.W;
    const uint32_t wi_c = lane_ok ? wi : (p.W - 1u);        // out-of-range lanes re-read a valid word; their
                                                            // sums are dropped
    const bool direct = p.S * p.sgroups <= 2u;              // few slices: every wave merges its own sums
    float* part = (float*)smem;                             // [rows_per_block][S]
    float* wlut = part + (size_t)rows_per_block * p.S + (size_t)wave * 256;
    const uint32_t row0 = block_row0 + g * RB;
    if (wave_active && row0 < p.N) {
        const uint32_t nrows = (p.N - row0) < (uint32_t)RB ? (p.N - row0) : (uint32_t)RB;
        const size_t plane_stride = (size_t)p.N * p.W;
        // Activations first: they are needed before the first row can be decoded, and loads return in
        // issue order, so requesting them ahead of the weights lets row r be decoded while rows r+1..
        // are still streaming in.
        uint32_t xr[4][4];
        anyprec_issue_x(p, wi_c, xr);
        const uint32_t word_off = wi_c * 4u;        // byte offset of the lane's word inside a row
        u32x4 lut4[RB], lut4b[RB];
        if constexpr (BITS == 3) {
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const uint32_t row = ((uint32_t)r < nrows) ? row0 + r : (p.N - 1u);
                lut4[r] = *(const DD_CONST_AS u32x4*)((const uint16_t*)p.lut + (size_t)row * 8);
            }
        } else if constexpr (BITS == 4) {
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const uint32_t row = ((uint32_t)r < nrows) ? row0 + r : (p.N - 1u);
                lut4[r] = *(const DD_CONST_AS u32x4*)((const uint16_t*)p.lut + (size_t)row * 16);
                lut4b[r] = *(const DD_CONST_AS u32x4*)((const uint16_t*)p.lut + (size_t)row * 16 + 8);
            }
        }
        // unconditional loads from wave-uniform row bases (rows past the end re-read the last row)
        uint32_t q[RB][BITS];
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const uint32_t row = ((uint32_t)r < nrows) ? row0 + r : (p.N - 1u);
            const char* rp = (const char*)(p.qweight + (size_t)row * p.W);      // wave-uniform
#pragma unroll
            for (int pl = 0; pl < BITS; ++pl)
                q[r][pl] = __builtin_nontemporal_load((const uint32_t*)(rp + (size_t)pl * plane_stride * 4 + word_off));
            __builtin_amdgcn_sched_barrier(0);      // keep the requests in row order: they return in issue order
        }
        uint32_t xp[8][2];
        anyprec_arrange_x(xr, xp);
        float sums[RB];
        Anyprec3Masks mk;
        Anyprec4Masks mk4;
        if constexpr (BITS == 4) mk4.init(); else mk.init();
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            float acc;
            if constexpr (BITS == 3) {
                uint32_t lo0, lo1, hi0, hi1;
                anyprec3_tables(lut4[r], lo0, lo1, hi0, hi1);
                acc = anyprec3_word<DT>(q[r][0], q[r][1], q[r][2], lo0, lo1, hi0, hi1, mk, xp, 0.f);
            } else if constexpr (BITS == 4) {
                uint32_t lo[4], hi[4];
                anyprec4_tables(lut4[r], lut4b[r], lo, hi);
                acc = anyprec4_word<DT>(q[r][0], q[r][1], q[r][2], q[r][3], lo, hi, mk4, xp, 0.f);
            } else {
                constexpr int L = 1 << BITS;
                const uint32_t row = ((uint32_t)r < nrows) ? row0 + r : (p.N - 1u);
                __builtin_amdgcn_wave_barrier();
                for (int v = lane; v < L; v += kWave) wlut[v] = E::load(p.lut, (size_t)row * L + v);
                __builtin_amdgcn_wave_barrier();
                acc = anyprec_generic_word<DT, BITS>(q[r], wlut, xp, 0.f);
            }
            sums[r] = lane_ok ? acc : 0.f;                  // lanes past the row's end decoded a re-read word
            __builtin_amdgcn_sched_barrier(0);              // decode row by row, as the rows arrive
        }
        wave_sum_rows<RB>(sums);                            // totals in lane 63
        if (lane == 63) {
            if (direct) {
#pragma unroll
                for (int r = 0; r < RB; r += 2) {
                    if ((uint32_t)r + 1 < nrows) E::atomic_add2(p.out, row0 + r, sums[r], sums[r + 1]);
                    else if ((uint32_t)r < nrows) E::atomic_add1(p.out, row0 + r, sums[r]);
                }
            } else {
#pragma unroll
                for (int r = 0; r < RB; ++r) part[(size_t)(g * RB + r) * p.S + s] = sums[r];
            }
        }
    }
    if (direct) return;                                     // uniform for the workgroup
    __syncthreads();
    // one atomic per output pair
    for (uint32_t t = tid; t < rows_per_block / 2; t += blockDim.x) {
        const uint32_t r = 2 * t, row = block_row0 + r;
        if (row >= p.N) continue;
        float v0 = 0.f, v1 = 0.f;
        for (uint32_t ss = 0; ss < p.S; ++ss) {
            v0 += part[(size_t)r * p.S + ss];
            v1 += part[(size_t)(r + 1) * p.S + ss];
        }
        if (row + 1 < p.N) E::atomic_add2(p.out, row, v0, v1);
        else E::atomic_add1(p.out, row, v0);
    }
}

// ---- 3-bit tile decoder -----------------------------------------------------------------------------
// The decode above spends a fifth of its vector instructions on work that exists only because the 64
// lanes of a wave share a row: rearranging the activations per lane, building the row's byte tables in
// every lane, and the cross-lane sum.  Here a lane owns a ROW instead.  A tile is 64 rows x (4 CS) words;
// its 3 planes are loaded with coalesced 16-byte requests (16 CS bytes of a row per CS lanes), staged in
// LDS with a padded pitch, and read back transposed: wave `wq` of the tile reads, for its lane's row, the
// four words 4 wq .. 4 wq + 3 of every plane in three conflict-free 16-byte LDS reads.  The activations
// of those words are the same for all 64 rows, so they arrive through the scalar cache and stay in SGPRs;
// the byte tables are built once per wave; every lane ends with its row's partial sum, the CS waves of a
// tile are added in LDS and one atomic per output pair and tile goes to memory (K / (128 CS) per output).
__host__ __device__ inline size_t anyprec3_tile_lds_bytes(uint32_t cs) {
    return (size_t)3 * 64 * (cs * 16 + 16) + (size_t)cs * 64 * 4;
}

template <int DT>
__device__ __forceinline__ void anyprec3_tile(const AnyprecParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t CS = p.tile_cs;
    const uint32_t sub = wave / CS, wq = wave % CS;
    const uint32_t g = bid * ((blockDim.x >> 6) / CS) + sub;             // global tile index
    const bool tile_ok = g < p.tiles;                                    // uniform per wave
    const uint32_t gg = tile_ok ? g : 0u;
    const uint32_t rgi = gg / p.tile_kt, kt = gg % p.tile_kt;
    const uint32_t row0 = rgi * 64u, w0 = kt * 4u * CS;
    const uint32_t pitch = CS * 16u + 16u;
    unsigned char* lds = smem + (size_t)sub * anyprec3_tile_lds_bytes(CS);
    float* part = (float*)(lds + (size_t)3 * 64 * pitch);

    // -- stage the tile: thread tt of the tile loads 16 bytes of row tt / CS, column tt % CS, per plane
    {
        const uint32_t tt = wq * 64u + lane, r = tt / CS, c = tt % CS;
        const uint32_t row = (row0 + r < p.N) ? row0 + r : p.N - 1u;     // rows past the end re-read the last row
        const uint32_t* src = p.qweight + (size_t)row * p.W + w0 + 4u * c;
        const size_t plane_stride = (size_t)p.N * p.W;
        u32x4 v[3];
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) v[pl] = __builtin_nontemporal_load((const u32x4*)(src + pl * plane_stride));
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) *(u32x4*)(lds + (size_t)pl * 64 * pitch + r * pitch + 16u * c) = v[pl];
    }
    // -- this lane's row: LUT byte tables
    const uint32_t myrow = (row0 + lane < p.N) ? row0 + lane : p.N - 1u;
    const u32x4 lut4 = *(const u32x4*)((const uint16_t*)p.lut + (size_t)myrow * 8);
    uint32_t lo0, lo1, hi0, hi1;
    anyprec3_tables(lut4, lo0, lo1, hi0, hi1);
    // -- activations of the wave's four words: 16 consecutive dwords per channel group j, scalar loads
    const uint32_t wfirst = w0 + 4u * wq;                                // first word of this wave
    const uint32_t ci = wfirst >> 5, tf = wfirst & 31u;                  // chunk, word inside the chunk
    const DD_CONST_AS uint32_t* xs = (const DD_CONST_AS uint32_t*)p.x + (512u * ci + 4u * tf);
    uint32_t X[4][16];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int d = 0; d < 16; ++d) X[j][d] = xs[128 * j + d];
    Anyprec3Masks mk;
    mk.init();
    __syncthreads();
    float acc = 0.f;
    {
        u32x4 q[3];
#pragma unroll
        for (int pl = 0; pl < 3; ++pl) q[pl] = *(const u32x4*)(lds + (size_t)pl * 64 * pitch + lane * pitch + 16u * wq);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t xp[8][2];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t x3 = X[3][4 * k + (e >> 1)], x2 = X[2][4 * k + (e >> 1)];
                const uint32_t x1 = X[1][4 * k + (e >> 1)], x0 = X[0][4 * k + (e >> 1)];
                if (e & 1) {
                    xp[e][0] = (x3 >> 16) | (x2 & 0xFFFF0000u);          // lo = j3, hi = j2
                    xp[e][1] = (x1 >> 16) | (x0 & 0xFFFF0000u);          // lo = j1, hi = j0
                } else {
                    xp[e][0] = (x3 & 0xFFFFu) | (x2 << 16);
                    xp[e][1] = (x1 & 0xFFFFu) | (x0 << 16);
                }
            }
            acc = anyprec3_word<DT>(q[0][k], q[1][k], q[2][k], lo0, lo1, hi0, hi1, mk, xp, acc);
        }
    }
    part[wq * 64u + lane] = acc;
    __syncthreads();
    if (wq == 0 && lane < 32u && tile_ok) {
        const uint32_t r = 2u * lane, row = row0 + r;
        if (row < p.N) {
            float v0 = 0.f, v1 = 0.f;
            for (uint32_t w = 0; w < CS; ++w) { v0 += part[w * 64u + r]; v1 += part[w * 64u + r + 1u]; }
            if (row + 1u < p.N) E::atomic_add2(p.out, row, v0, v1);
            else E::atomic_add1(p.out, row, v0);
        }
    }
}

template <int DT, int BITS>
__device__ __forceinline__ void anyprec_role(const AnyprecParams& p, uint32_t bid, unsigned char* smem) {
    if constexpr (BITS == 3) {
        if (p.tile_cs != 0u) { anyprec3_tile<DT>(p, bid, smem); return; }
    }
    // eight rows per wave only at 3 bits: the plane words of eight rows of a wider format cost occupancy (4 bits:
    // 82 registers against 65) or do not fit the register budget at all (the launch planner never asks for it)
    if constexpr (BITS == 3) {
        if (p.rpw == 8) { anyprec_rows<DT, BITS, 8>(p, bid, smem); return; }
    }
    if (p.rpw >= 4) anyprec_rows<DT, BITS, 4>(p, bid, smem);
    else anyprec_rows<DT, BITS, 2>(p, bid, smem);
}

}  // namespace decdec
