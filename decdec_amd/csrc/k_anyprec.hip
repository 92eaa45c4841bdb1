// Any-precision bitplane kernels: GEMV, dequantisation to a dense [N, K] matrix, and the fused
// single-launch DEC + GEMV kernel.
#include "launch.h"

namespace decdec {

template <int DT, int BITS>
__global__ __launch_bounds__(1024) void anyprec_kernel(const AnyprecParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    anyprec_role<DT, BITS>(p, blockIdx.x, smem);
}

template <int DT, int BITS, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_anyprec_kernel(const DecParams dp, const uint32_t dec_blocks,
                                                           const AnyprecParams gp) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (blockIdx.x < dec_blocks) dec_role<DT>(dp, blockIdx.x, smem);
    else anyprec_role<DT, BITS>(gp, blockIdx.x - dec_blocks, smem);
}

// Up to kMaxBatch layers on one input in one launch: a workgroup finds its layer and plays the DEC or the GEMV role
// for it, exactly as in the single-layer kernel above.
template <int DT, int BITS, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_anyprec_batch_kernel(const BatchParams<AnyprecParams> b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t ndec = b.dec_end[kMaxBatch - 1];
    uint32_t layer, local;
    if (blockIdx.x < ndec) {
        batch_locate(b.dec_end, blockIdx.x, layer, local);
        dec_role<DT>(b.dp[layer], local, smem);
    } else {
        batch_locate(b.gemv_end, blockIdx.x - ndec, layer, local);
        anyprec_role<DT, BITS>(b.gp[layer], local, smem);
    }
}

// The base GEMVs of up to kMaxBatch layers on one input in one launch, in the standalone kernel's own workgroups.
template <int DT, int BITS>
__global__ __launch_bounds__(1024) void anyprec_batch_kernel(const GemvBatchParams<AnyprecParams> b) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t layer, local;
    batch_locate(b.gemv_end, blockIdx.x, layer, local);
    anyprec_role<DT, BITS>(b.gp[layer], local, smem);
}

// The same two roles in workgroups of NW (4 or 8) waves, eight waves per SIMD: the GEMV role runs in workgroups of
// its standalone size, and a DEC workgroup holds an eighth or a quarter of a compute unit.
template <int DT, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(8, 8)))
void dec_anyprec3_small_kernel(const DecParams dp, const uint32_t dec_blocks, const AnyprecParams gp) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (blockIdx.x < dec_blocks) dec_role<DT, NW>(dp, blockIdx.x, smem);
    else anyprec_role<DT, 3>(gp, blockIdx.x - dec_blocks, smem);
}

// W[n][c] = lut[n][idx(n, c)]: one thread per (row, word); the 32 weights of a word go to four groups
// of eight consecutive channels (reference dequant_kbit_store, decdec_extension/anyprec.cu:261-331).
template <int DT, int BITS>
__global__ __launch_bounds__(256) void anyprec_dequant_kernel(const uint32_t* __restrict__ qweight,
                                                              const void* __restrict__ lut, void* __restrict__ weight,
                                                              const uint32_t N, const uint32_t K) {
    const uint32_t W = K / 32u;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (size_t)N * W) return;
    const uint32_t n = (uint32_t)(gid / W), wi = (uint32_t)(gid % W);
    const uint32_t i = wi >> 5, t = wi & 31u;
    const uint32_t eff = (i == K / 1024u) ? (K % 1024u) / 32u : 32u;
    uint32_t q[BITS];
#pragma unroll
    for (int pl = 0; pl < BITS; ++pl) q[pl] = qweight[((size_t)pl * N + n) * W + wi];
    constexpr int L = 1 << BITS;
    const uint16_t* lrow = (const uint16_t*)lut + (size_t)n * L;
    uint16_t* wrow = (uint16_t*)weight + (size_t)n * K;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint16_t vals[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int pos = 31 - (8 * j + e);
            uint32_t idx = 0;
#pragma unroll
            for (int pl = 0; pl < BITS; ++pl) idx = (idx << 1) | ((q[pl] >> pos) & 1u);
            vals[e] = lrow[idx];
        }
        uint16_t* dst = wrow + (size_t)1024 * i + (size_t)8 * eff * j + (size_t)8 * t;
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = vals[e];
    }
}

#define DD_BITS_SWITCH(BITS_EXPR, CALL)                \
    switch (BITS_EXPR) {                               \
        case 3: { constexpr int B = 3; CALL; } break;  \
        case 4: { constexpr int B = 4; CALL; } break;  \
        case 5: { constexpr int B = 5; CALL; } break;  \
        case 6: { constexpr int B = 6; CALL; } break;  \
        case 7: { constexpr int B = 7; CALL; } break;  \
        case 8: { constexpr int B = 8; CALL; } break;  \
        default: return hipErrorInvalidValue;          \
    }

hipError_t launch_anyprec(int dt, int bits, const AnyprecParams& p, const LaunchDims& d, hipStream_t s) {
    if (dt == kFP16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((anyprec_kernel<kFP16, B>), dim3(d.grid), dim3(d.block), d.lds, s, p));
    } else if (dt == kBF16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((anyprec_kernel<kBF16, B>), dim3(d.grid), dim3(d.block), d.lds, s, p));
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_anyprec(int dt, int bits, const DecParams& dp, uint32_t dec_blocks,
                              const AnyprecParams& gp, const LaunchDims& d, hipStream_t s) {
    const dim3 grid(dec_blocks + d.grid), block(d.block);
    if (d.two_per_cu && bits == 3) {       // only the 3-bit instances fit the register budget without spilling
        if (dt == kFP16) hipLaunchKernelGGL((dec_anyprec_kernel<kFP16, 3, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
        else if (dt == kBF16) hipLaunchKernelGGL((dec_anyprec_kernel<kBF16, 3, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
        else return hipErrorInvalidValue;
        return hipGetLastError();
    }
    if (dt == kFP16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((dec_anyprec_kernel<kFP16, B, false>), grid, block, d.lds, s, dp, dec_blocks, gp));
    } else if (dt == kBF16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((dec_anyprec_kernel<kBF16, B, false>), grid, block, d.lds, s, dp, dec_blocks, gp));
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_anyprec_batch(int dt, int bits, const BatchParams<AnyprecParams>& b, const LaunchDims& d, hipStream_t s) {
    const dim3 grid(d.grid), block(d.block);
    if ((dt != kFP16 && dt != kBF16) || (bits != 3 && bits != 4) || d.block != 1024u) return hipErrorInvalidValue;
    if (bits == 3 && d.two_per_cu) {
        if (dt == kFP16) hipLaunchKernelGGL((dec_anyprec_batch_kernel<kFP16, 3, true>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_anyprec_batch_kernel<kBF16, 3, true>), grid, block, d.lds, s, b);
    } else if (bits == 3) {
        if (dt == kFP16) hipLaunchKernelGGL((dec_anyprec_batch_kernel<kFP16, 3, false>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_anyprec_batch_kernel<kBF16, 3, false>), grid, block, d.lds, s, b);
    } else {
        if (dt == kFP16) hipLaunchKernelGGL((dec_anyprec_batch_kernel<kFP16, 4, false>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_anyprec_batch_kernel<kBF16, 4, false>), grid, block, d.lds, s, b);
    }
    return hipGetLastError();
}

hipError_t launch_anyprec_batch(int dt, int bits, const GemvBatchParams<AnyprecParams>& b, const LaunchDims& d, hipStream_t s) {
    if (dt == kFP16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((anyprec_batch_kernel<kFP16, B>), dim3(d.grid), dim3(d.block), d.lds, s, b));
    } else if (dt == kBF16) {
        DD_BITS_SWITCH(bits, hipLaunchKernelGGL((anyprec_batch_kernel<kBF16, B>), dim3(d.grid), dim3(d.block), d.lds, s, b));
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_anyprec_small(int dt, uint32_t nw, const DecParams& dp, uint32_t dec_blocks,
                                    const AnyprecParams& gp, const LaunchDims& d, hipStream_t s) {
    const dim3 grid(dec_blocks + d.grid), block(d.block);
    if (d.block != nw * 64u || (nw != 4u && nw != 8u) || (dt != kFP16 && dt != kBF16)) return hipErrorInvalidValue;
    if (dt == kFP16) {
        if (nw == 4u) hipLaunchKernelGGL((dec_anyprec3_small_kernel<kFP16, 4>), grid, block, d.lds, s, dp, dec_blocks, gp);
        else hipLaunchKernelGGL((dec_anyprec3_small_kernel<kFP16, 8>), grid, block, d.lds, s, dp, dec_blocks, gp);
    } else {
        if (nw == 4u) hipLaunchKernelGGL((dec_anyprec3_small_kernel<kBF16, 4>), grid, block, d.lds, s, dp, dec_blocks, gp);
        else hipLaunchKernelGGL((dec_anyprec3_small_kernel<kBF16, 8>), grid, block, d.lds, s, dp, dec_blocks, gp);
    }
    return hipGetLastError();
}

hipError_t launch_anyprec_dequant(int dt, int bits, const uint32_t* qweight, const void* lut, void* weight,
                                  uint32_t N, uint32_t K, hipStream_t s) {
    const size_t total = (size_t)N * (K / 32u);
    const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
    if (total == 0) return hipSuccess;
    // 16-bit LUT entries are copied bit for bit, so fp16 and bf16 share one instantiation
    if (dt != kFP16 && dt != kBF16) return hipErrorInvalidValue;
    DD_BITS_SWITCH(bits, hipLaunchKernelGGL((anyprec_dequant_kernel<kFP16, B>), grid, block, 0, s, qweight, lut, weight, N, K));
    return hipGetLastError();
}

}  // namespace decdec
