// Host-side launch interface between the kernel translation units and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include "dec_role.h"
#include "anyprec_role.h"
#include "lutgemm_role.h"
#include "sqllm_role.h"

namespace decdec {

struct LaunchDims {
    uint32_t grid;
    uint32_t block;
    size_t lds;
    bool two_per_cu = false;   // fused launches: use the kernel instance held to 64 vector / 96 scalar registers
};

// A fused kernel runs 1024-thread workgroups.  Two of them share a compute unit (eight waves per SIMD) only
// if a wave needs at most 64 vector and 96 scalar registers; the attribute makes the compiler keep to that.
// Sharing pays when the GEMV role outlasts the DEC role (its waves then fill the whole chip); a DEC
// workgroup that shares its unit with GEMV waves takes about a microsecond longer, so launches in which
// DEC is the longer role use the unconstrained instance, one workgroup per unit.
#define DD_TWO_PER_CU(on) __attribute__((amdgpu_waves_per_eu((on) ? 8 : 4, 8)))

// Several layers that read the same activation vector in ONE launch (q | k | v, gate | up): the DEC workgroups of all
// layers come first in the grid (their host-memory reads start at once), then the GEMV workgroups, layer by layer.
// dec_end / gemv_end are running totals of workgroups over the layers (entries past n repeat the last total).
constexpr int kMaxBatch = 4;
template <typename GemvParams>
struct BatchParams {
    uint32_t n;
    uint32_t dec_end[kMaxBatch];
    uint32_t gemv_end[kMaxBatch];
    DecParams dp[kMaxBatch];
    GemvParams gp[kMaxBatch];
};
// The base GEMVs of several layers on one input, no DEC: workgroups of the GEMV's own standalone size (a batch shares
// its input width, so every layer plans the same workgroup), layer by layer in the grid.
template <typename GemvParams>
struct GemvBatchParams {
    uint32_t n;
    uint32_t gemv_end[kMaxBatch];
    GemvParams gp[kMaxBatch];
};
// the layer a workgroup of a batch belongs to, and its index inside that layer's share of the grid
__device__ __forceinline__ void batch_locate(const uint32_t (&end)[kMaxBatch], uint32_t id, uint32_t& layer, uint32_t& local) {
    layer = 0; local = id;
#pragma unroll
    for (int j = 0; j + 1 < kMaxBatch; ++j)
        if (id >= end[j]) { layer = (uint32_t)j + 1u; local = id - end[j]; }
}

// Standalone kernels.
hipError_t launch_dec(int dt, const DecParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_anyprec(int dt, int bits, const AnyprecParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_anyprec_dequant(int dt, int bits, const uint32_t* qweight, const void* lut, void* weight,
                                  uint32_t N, uint32_t K, hipStream_t s);
hipError_t launch_lutgemm(int dt, const LutgemmParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_sqllm(int dt, const SqllmParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_burner(uint32_t blocks, long long iters, hipStream_t s);
hipError_t launch_read_probe(const void* src, unsigned long long row_bytes, unsigned long long rows, uint32_t vec_words,
                             uint32_t blocks, int scramble, void* sink, hipStream_t s);

// Single-launch fused kernels: workgroups [0, dec_blocks) play the DEC role, the rest the base GEMV.
// d.grid counts the GEMV workgroups only; d.block is 1024.
hipError_t launch_dec_anyprec(int dt, int bits, const DecParams& dp, uint32_t dec_blocks,
                              const AnyprecParams& gp, const LaunchDims& d, hipStream_t s);
// A batch of up to kMaxBatch any-precision layers on one input, each with or without DEC (3 or 4 bits; d.grid and
// d.lds cover all layers; d.block is 1024).
hipError_t launch_dec_anyprec_batch(int dt, int bits, const BatchParams<AnyprecParams>& b, const LaunchDims& d, hipStream_t s);
// The same batch without DEC on any layer, in the standalone kernel's workgroups (d.block = the layers' common
// workgroup size, d.grid and d.lds cover all layers; any bit width).
hipError_t launch_anyprec_batch(int dt, int bits, const GemvBatchParams<AnyprecParams>& b, const LaunchDims& d, hipStream_t s);
// 3-bit, both roles in workgroups of `nw` (4 or 8) waves = d.block / 64; dp carries the DEC plan for that size.
hipError_t launch_dec_anyprec_small(int dt, uint32_t nw, const DecParams& dp, uint32_t dec_blocks,
                                    const AnyprecParams& gp, const LaunchDims& d, hipStream_t s);
hipError_t launch_dec_lutgemm(int dt, const DecParams& dp, uint32_t dec_blocks,
                              const LutgemmParams& gp, const LaunchDims& d, hipStream_t s);
hipError_t launch_dec_sqllm(int dt, const DecParams& dp, uint32_t dec_blocks,
                            const SqllmParams& gp, const LaunchDims& d, hipStream_t s);
// Batches of up to kMaxBatch LUT-GEMM / SqueezeLLM layers on one input (16-bit types), as launch_dec_anyprec_batch.
hipError_t launch_dec_lutgemm_batch(int dt, const BatchParams<LutgemmParams>& b, const LaunchDims& d, hipStream_t s);
hipError_t launch_dec_sqllm_batch(int dt, const BatchParams<SqllmParams>& b, const LaunchDims& d, hipStream_t s);

// Decode-step helpers (k_decode.hip).  `pos` points at the token position in device memory.
struct RopeCacheParams {
    const void* qkv;                 // [(n_head + 2 n_kv) * head_dim]: query heads, key heads, value heads
    const void* cos_table;           // [max_seq][head_dim]
    const void* sin_table;
    const long long* pos;
    void* q_out;                     // [n_head * head_dim], rotated queries
    void* k_cache;                   // [n_kv][max_seq][head_dim]
    void* v_cache;
    uint32_t n_head, n_kv, head_dim, max_seq;
};
struct AttentionParams {
    const void* q;                   // [n_head * head_dim]
    const void* k_cache;
    const void* v_cache;
    const long long* pos;            // attends cache positions 0 .. *pos
    void* out;                       // [n_head * head_dim]
    uint32_t n_head, n_kv, head_dim, max_seq;
    float scale;
    uint32_t nsplit;                 // workgroups per head (1: no workspace needed)
    float* workspace;                // [n_head][nsplit][head_dim + 2] floats
    // Rotary embedding and cache append folded in (qkv != null; q is not read then): queries and the new key are
    // rotated on the fly, the new key / value row takes the place of cache row *pos in the scan, and the first
    // query head of every key/value head writes that row to the caches.
    const void* qkv;                 // [(n_head + 2 n_kv) * head_dim]
    const void* cos_table;           // [max_seq][head_dim]
    const void* sin_table;
    // [n_head] arrival counters behind the partial results in the workspace, zero between calls (null: the ranges are
    // merged by a second kernel)
    uint32_t* counters;
    // with counters: a sequence of at most this many positions is scanned by the first workgroup of a head alone
    // (no partial results, no merge; the other workgroups of the head return at once)
    uint32_t single_below;
};
hipError_t launch_rope_cache(int dt, const RopeCacheParams& p, hipStream_t s);
hipError_t launch_decode_attention(int dt, const AttentionParams& p, hipStream_t s);
hipError_t launch_dense_gemv(int dt, const void* weight, const void* x, void* out, uint32_t N, uint32_t K, hipStream_t s);
hipError_t launch_silu_mul(int dt, const void* gate_up, void* out, uint32_t n, hipStream_t s);
size_t greedy_pick_workspace_bytes();
hipError_t launch_greedy_pick(int dt, const void* logits, uint32_t n, void* workspace, float* copy_out, long long* token,
                              long long* seq, uint32_t seq_capacity, long long* count, long long* pos, hipStream_t s);
hipError_t launch_add_rmsnorm(int dt, const void* x, const void* y, const void* weight, void* h_out, void* normed_out,
                              uint32_t rows, uint32_t dim, float eps, hipStream_t s);

}  // namespace decdec
