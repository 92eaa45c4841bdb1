// DEC role: bucket top-k channel selection + zero-copy fetch of the selected 4-bit residual rows +
// residual GEMV + atomic merge into the output.  One workgroup of 1024 threads (16 wave64) plays
// this role; it is used by the standalone DEC kernels and, next to a base-GEMV role, by the fused
// single-launch kernels.
//
// Work decomposition (differs from the reference's column partition + grid barrier on purpose):
// a workgroup owns a set of 1024-channel chunks (chunk group) and a range of column segments
// (segment group).  It selects the channels of its own chunks itself -- selection needs only the
// activation vector, so no grid-wide barrier and no second launch -- and then fetches the selected
// residual rows restricted to its column segments.  A segment is 64*VEC consecutive u32 words of a
// residual row (VEC*256 bytes, one coalesced wave-wide load).  Each wave keeps several row loads in
// flight because the host link's latency, not ALU work, bounds the fetch.
//
// Reference semantics reproduced (decdec_extension/dec.cu:76-280): bucket membership
// floor[i] <= |x| < ceil[i] per bucket, buckets taken in order until k_chunk*len/1024 channels are
// found, selected_rows / selected_activations written at chunk*k_chunk + pos, residual value
// (nibble - 8) * reordered_scales[j*N/8 + m] * x[row] accumulated into output[8m + j].
// In-bucket order is ascending channel index (the reference's order is an atomicAdd race).
#pragma once
#include "common.h"

namespace decdec {

struct DecParams {
    const uint32_t* residual;   // [K][M] u32 words, host-mapped (zero-copy) or device memory
    const void* scales;         // reordered_scales[N], device memory, dtype of the activations
    const void* x;              // activations [K]
    int32_t* sel_rows;          // context scratch: selected channel indices
    void* sel_acts;             // context scratch: selected activations
    void* out;                  // output [N], accumulated atomically
    float floors[kBuckets];     // bucket floors (values exactly representable in the activation dtype)
    uint32_t K, N, M;           // M = N / 8 words per residual row
    uint32_t num_chunks, k_chunk, k_total;
    uint32_t cg, sg;            // chunk groups x segment groups = number of DEC workgroups
    uint32_t nseg;              // column segments per row
    uint32_t vec;               // u32 words per lane per load: 1, 2 or 4
    uint32_t segs_per_block;    // ceil(nseg / sg)
    uint32_t slots_per_block;   // capacity of the per-workgroup row list
    uint32_t use_lds_reduce;    // reduce across waves in LDS before the global atomics
    uint32_t fused_select;      // 1: select in-kernel; 0: row indices supplied in sel_rows
};

constexpr int kDecThreads = 1024;
constexpr int kDecWaves = kDecThreads / kWave;

__host__ __device__ inline size_t dec_lds_bytes(uint32_t slots, uint32_t segs_per_block, uint32_t vec,
                                                uint32_t use_lds_reduce) {
    size_t b = (size_t)slots * 8 + 2 * 512 * 4;
    if (use_lds_reduce) {
        uint32_t sb = segs_per_block < kDecWaves ? segs_per_block : kDecWaves;
        b += (size_t)sb * kWave * vec * 8 * 4;
    }
    return b;
}

// ---- selection of one chunk ------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void dec_select_chunk(const DecParams& p, uint32_t c, uint32_t t_local,
                                                 int32_t* lrows, float* lacts, uint32_t* cnt,
                                                 uint32_t* pre, bool write_global) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t lo = c * kChunk;
    const uint32_t len = (p.K - lo) < (uint32_t)kChunk ? (p.K - lo) : (uint32_t)kChunk;
    const uint32_t kc = p.k_chunk * len / kChunk;
    if (kc == 0) return;                                   // uniform for the workgroup

    float xv = 0.f;
    uint32_t member = 0;
    if (tid < len) {
        xv = E::load(p.x, lo + tid);
        const float a = __builtin_fabsf(xv);
#pragma unroll
        for (int i = 0; i < kBuckets; ++i) {
            const float fl = p.floors[i];
            const float ce = (i == 0) ? __builtin_inff() : p.floors[i - 1];
            member |= (uint32_t)((a >= fl) && (a < ce)) << i;
        }
    }
    // pass 1: members per (bucket, wave)
#pragma unroll
    for (int i = 0; i < kBuckets; ++i) {
        const unsigned long long m = __ballot((member >> i) & 1u);
        if (lane == 0) cnt[i * kDecWaves + wave] = (uint32_t)__popcll(m);
    }
    __syncthreads();
    // exclusive prefix over the 512 (bucket-major, wave-minor) counts, by wave 0
    if (wave == 0) {
        uint32_t v[8], s = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) { v[q] = cnt[lane * 8 + q]; s += v[q]; }
        uint32_t incl = s;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(incl, off, 64);
            if (lane >= (uint32_t)off) incl += o;
        }
        uint32_t run = incl - s;
#pragma unroll
        for (int q = 0; q < 8; ++q) { pre[lane * 8 + q] = run; run += v[q]; }
    }
    __syncthreads();
    // pass 2: position = members in earlier buckets + members of this bucket in earlier waves
    //         + rank inside the wave; ascending channel order inside a bucket by construction
#pragma unroll 1
    for (int i = 0; i < kBuckets; ++i) {
        if (pre[i * kDecWaves] >= kc) break;                // uniform: later buckets start even later
        const bool bit = (member >> i) & 1u;
        const unsigned long long m = __ballot(bit);
        if (bit) {
            const uint32_t pos = pre[i * kDecWaves + wave] + ballot_rank(m);
            if (pos < kc) {
                const uint32_t slot = t_local * p.k_chunk + pos;
                lrows[slot] = (int32_t)(lo + tid);
                lacts[slot] = xv;
                if (write_global) {
                    p.sel_rows[(size_t)c * p.k_chunk + pos] = (int32_t)(lo + tid);
                    E::store(p.sel_acts, (size_t)c * p.k_chunk + pos, xv);
                }
            }
        }
    }
}

// ---- fetch + dequantise + accumulate ------------------------------------------------------------
template <int VEC> struct WordVec;
template <> struct WordVec<1> { using type = uint32_t; };
template <> struct WordVec<2> { using type = u32x2; };
template <> struct WordVec<4> { using type = u32x4; };

__device__ __forceinline__ void dec_accumulate_word(uint32_t w, float act, float* acc) {
    const uint32_t lo = w & 0x0F0F0F0Fu;           // nibbles 0,2,4,6 as bytes
    const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;    // nibbles 1,3,5,7 as bytes
    acc[0] += (float)(lo & 0xFFu) * act;
    acc[1] += (float)(hi & 0xFFu) * act;
    acc[2] += (float)((lo >> 8) & 0xFFu) * act;
    acc[3] += (float)((hi >> 8) & 0xFFu) * act;
    acc[4] += (float)((lo >> 16) & 0xFFu) * act;
    acc[5] += (float)((hi >> 16) & 0xFFu) * act;
    acc[6] += (float)(lo >> 24) * act;
    acc[7] += (float)(hi >> 24) * act;
}

template <int DT, int VEC>
__device__ __forceinline__ void dec_fetch(const DecParams& p, uint32_t sgid, uint32_t nslots,
                                          const int32_t* lrows, const float* lacts, float* red) {
    using E = Elem<DT>;
    using V = typename WordVec<VEC>::type;
    constexpr int U = (VEC == 4) ? 8 : 8;              // residual rows in flight per wave
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t seg_lo = sgid * p.segs_per_block;
    const uint32_t seg_hi = (seg_lo + p.segs_per_block) < p.nseg ? (seg_lo + p.segs_per_block) : p.nseg;

    for (uint32_t sb0 = seg_lo; sb0 < seg_hi; sb0 += kDecWaves) {
        const uint32_t SB = (seg_hi - sb0) < (uint32_t)kDecWaves ? (seg_hi - sb0) : (uint32_t)kDecWaves;
        const uint32_t RL = kDecWaves / SB;             // waves sharing one segment
        const uint32_t ls = wave % SB, rl = wave / SB;
        const uint32_t w0 = ((sb0 + ls) * kWave + lane) * VEC;
        const bool col_ok = (rl < RL) && (w0 < p.M);

        float acc[VEC * 8];
#pragma unroll
        for (int j = 0; j < VEC * 8; ++j) acc[j] = 0.f;
        float act_sum = 0.f;

        if (col_ok) {
            const uint32_t* base = p.residual + w0;
            for (uint32_t r = rl; r < nslots; r += RL * U) {
                V data[U];
                float act[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t rr = r + (uint32_t)u * RL;
                    int32_t row = -1;
                    float a = 0.f;
                    if (rr < nslots) { row = lrows[rr]; a = lacts[rr]; }
                    row = __builtin_amdgcn_readfirstlane(row);      // wave-uniform by construction
                    if (row >= 0) {
                        data[u] = *(const V*)(base + (size_t)row * p.M);
                        act[u] = a;
                    } else {
                        data[u] = (V)(0x88888888u);                 // nibble 8 == value 0
                        act[u] = 0.f;
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    act_sum += act[u];
                    if constexpr (VEC == 1) {
                        dec_accumulate_word(data[u], act[u], acc);
                    } else {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) dec_accumulate_word(data[u][v], act[u], acc + 8 * v);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < VEC * 8; ++j) acc[j] -= 8.f * act_sum;   // stored nibble = q + 8
        }

        const bool lds_reduce = p.use_lds_reduce && (RL > 1);       // uniform
        if (lds_reduce) {
            const uint32_t n_red = SB * kWave * VEC * 8;
            for (uint32_t i = tid; i < n_red; i += kDecThreads) red[i] = 0.f;
            __syncthreads();
            if (col_ok) {
#pragma unroll
                for (int j = 0; j < VEC * 8; ++j) atomicAdd(&red[(ls * VEC * 8 + j) * kWave + lane], acc[j]);
            }
            __syncthreads();
            if (col_ok && rl == 0) {
#pragma unroll
                for (int j = 0; j < VEC * 8; ++j) acc[j] = red[(ls * VEC * 8 + j) * kWave + lane];
            }
        }
        if (col_ok && (!lds_reduce || rl == 0)) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const uint32_t m = w0 + v;
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    const float s0 = E::load(p.scales, (size_t)j * p.M + m);
                    const float s1 = E::load(p.scales, (size_t)(j + 1) * p.M + m);
                    E::atomic_add2(p.out, (size_t)8 * m + j, acc[8 * v + j] * s0, acc[8 * v + j + 1] * s1);
                }
            }
        }
        if (lds_reduce) __syncthreads();                             // red is reused by the next batch
    }
}

// ---- the role -------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void dec_role(const DecParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x;
    const uint32_t cgid = bid / p.sg, sgid = bid % p.sg;
    int32_t* lrows = (int32_t*)smem;
    float* lacts = (float*)(lrows + p.slots_per_block);
    uint32_t* cnt = (uint32_t*)(lacts + p.slots_per_block);
    uint32_t* pre = cnt + 512;
    float* red = (float*)(pre + 512);

    for (uint32_t i = tid; i < p.slots_per_block; i += kDecThreads) lrows[i] = -1;
    uint32_t nslots = 0;
    if (p.fused_select) {
        uint32_t t = 0;
        for (uint32_t c = cgid; c < p.num_chunks; c += p.cg, ++t) {
            __syncthreads();      // list initialised; cnt/pre of the previous chunk no longer read
            dec_select_chunk<DT>(p, c, t, lrows, lacts, cnt, pre, sgid == 0);
        }
        nslots = t * p.k_chunk;
    } else {
        const uint32_t per = (p.k_total + p.cg - 1) / p.cg;
        const uint32_t lo = cgid * per;
        const uint32_t hi = (lo + per) < p.k_total ? (lo + per) : p.k_total;
        __syncthreads();
        for (uint32_t i = lo + tid; i < hi; i += kDecThreads) {
            const int32_t row = p.sel_rows[i];
            const bool ok = row >= 0 && (uint32_t)row < p.K;       // out-of-range indices are ignored
            lrows[i - lo] = ok ? row : -1;
            lacts[i - lo] = ok ? E::load(p.x, (size_t)row) : 0.f;
        }
        nslots = hi > lo ? hi - lo : 0;
    }
    __syncthreads();
    if (p.vec == 4) dec_fetch<DT, 4>(p, sgid, nslots, lrows, lacts, red);
    else if (p.vec == 2) dec_fetch<DT, 2>(p, sgid, nslots, lrows, lacts, red);
    else dec_fetch<DT, 1>(p, sgid, nslots, lrows, lacts, red);
}

}  // namespace decdec
