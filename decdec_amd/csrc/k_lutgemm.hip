// LUT-GEMM kernels: GEMV and the fused single-launch DEC + GEMV kernel.
#include "launch.h"

namespace decdec {

template <int DT>
__global__ __launch_bounds__(1024) void lutgemm_kernel(const LutgemmParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    lutgemm_role<DT>(p, blockIdx.x, smem);
}

template <int DT, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_lutgemm_kernel(const DecParams dp, const uint32_t dec_blocks,
                                                                             const LutgemmParams gp) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (blockIdx.x < dec_blocks) dec_role<DT>(dp, blockIdx.x, smem);
    else lutgemm_role<DT>(gp, blockIdx.x - dec_blocks, smem);
}

// Up to kMaxBatch layers on one input in one launch: a workgroup finds its layer and plays the DEC or the GEMV role
// for it, exactly as in the single-layer kernel above.
template <int DT, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_lutgemm_batch_kernel(const BatchParams<LutgemmParams> b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t ndec = b.dec_end[kMaxBatch - 1];
    uint32_t layer, local;
    if (blockIdx.x < ndec) {
        batch_locate(b.dec_end, blockIdx.x, layer, local);
        dec_role<DT>(b.dp[layer], local, smem);
    } else {
        batch_locate(b.gemv_end, blockIdx.x - ndec, layer, local);
        lutgemm_role<DT>(b.gp[layer], local, smem);
    }
}

hipError_t launch_lutgemm(int dt, const LutgemmParams& p, const LaunchDims& d, hipStream_t s) {
    switch (dt) {
        case kFP32: hipLaunchKernelGGL(lutgemm_kernel<kFP32>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        case kFP16: hipLaunchKernelGGL(lutgemm_kernel<kFP16>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        case kBF16: hipLaunchKernelGGL(lutgemm_kernel<kBF16>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_lutgemm(int dt, const DecParams& dp, uint32_t dec_blocks,
                              const LutgemmParams& gp, const LaunchDims& d, hipStream_t s) {
    const dim3 grid(dec_blocks + d.grid), block(d.block);
    const bool two = d.two_per_cu;
    switch (dt) {
        case kFP32:
            if (two) hipLaunchKernelGGL((dec_lutgemm_kernel<kFP32, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
            else hipLaunchKernelGGL((dec_lutgemm_kernel<kFP32, false>), grid, block, d.lds, s, dp, dec_blocks, gp);
            break;
        case kFP16:
            if (two) hipLaunchKernelGGL((dec_lutgemm_kernel<kFP16, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
            else hipLaunchKernelGGL((dec_lutgemm_kernel<kFP16, false>), grid, block, d.lds, s, dp, dec_blocks, gp);
            break;
        case kBF16:
            if (two) hipLaunchKernelGGL((dec_lutgemm_kernel<kBF16, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
            else hipLaunchKernelGGL((dec_lutgemm_kernel<kBF16, false>), grid, block, d.lds, s, dp, dec_blocks, gp);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_lutgemm_batch(int dt, const BatchParams<LutgemmParams>& b, const LaunchDims& d, hipStream_t s) {
    const dim3 grid(d.grid), block(d.block);
    if ((dt != kFP16 && dt != kBF16) || d.block != 1024u) return hipErrorInvalidValue;
    if (d.two_per_cu) {
        if (dt == kFP16) hipLaunchKernelGGL((dec_lutgemm_batch_kernel<kFP16, true>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_lutgemm_batch_kernel<kBF16, true>), grid, block, d.lds, s, b);
    } else {
        if (dt == kFP16) hipLaunchKernelGGL((dec_lutgemm_batch_kernel<kFP16, false>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_lutgemm_batch_kernel<kBF16, false>), grid, block, d.lds, s, b);
    }
    return hipGetLastError();
}

}  // namespace decdec
