// SqueezeLLM kernels: GEMV and the fused single-launch DEC + GEMV kernel.
#include "launch.h"

namespace decdec {

template <int DT>
__global__ __launch_bounds__(1024) void sqllm_kernel(const SqllmParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    sqllm_role<DT>(p, blockIdx.x, smem);
}

template <int DT, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_sqllm_kernel(const DecParams dp, const uint32_t dec_blocks,
                                                           const SqllmParams gp) {
    extern __shared__ __align__(16) unsigned char smem[];
    if (blockIdx.x < dec_blocks) dec_role<DT>(dp, blockIdx.x, smem);
    else sqllm_role<DT>(gp, blockIdx.x - dec_blocks, smem);
}

// Up to kMaxBatch layers on one input in one launch: a workgroup finds its layer and plays the DEC or the GEMV role
// for it, exactly as in the single-layer kernel above.
template <int DT, bool TWO>
__global__ __launch_bounds__(1024) DD_TWO_PER_CU(TWO) void dec_sqllm_batch_kernel(const BatchParams<SqllmParams> b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const uint32_t ndec = b.dec_end[kMaxBatch - 1];
    uint32_t layer, local;
    if (blockIdx.x < ndec) {
        batch_locate(b.dec_end, blockIdx.x, layer, local);
        dec_role<DT>(b.dp[layer], local, smem);
    } else {
        batch_locate(b.gemv_end, blockIdx.x - ndec, layer, local);
        sqllm_role<DT>(b.gp[layer], local, smem);
    }
}

// The 4-bit pair table needs more than the 64 KB of dynamic LDS a kernel gets by default.
template <typename K>
static hipError_t allow_large_lds(K kernel) {
    return hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
}
static hipError_t sqllm_prepare() {
    static hipError_t done = [] {
        hipError_t e = hipSuccess;
        auto acc = [&e](hipError_t r) { if (e == hipSuccess) e = r; };
        acc(allow_large_lds(sqllm_kernel<kFP32>)); acc(allow_large_lds(sqllm_kernel<kFP16>)); acc(allow_large_lds(sqllm_kernel<kBF16>));
        acc(allow_large_lds(dec_sqllm_kernel<kFP32, false>));
        acc(allow_large_lds(dec_sqllm_kernel<kFP16, false>)); acc(allow_large_lds(dec_sqllm_kernel<kFP16, true>));
        acc(allow_large_lds(dec_sqllm_kernel<kBF16, false>)); acc(allow_large_lds(dec_sqllm_kernel<kBF16, true>));
        acc(allow_large_lds(dec_sqllm_batch_kernel<kFP16, false>)); acc(allow_large_lds(dec_sqllm_batch_kernel<kFP16, true>));
        acc(allow_large_lds(dec_sqllm_batch_kernel<kBF16, false>)); acc(allow_large_lds(dec_sqllm_batch_kernel<kBF16, true>));
        return e;
    }();
    return done;
}

hipError_t launch_sqllm(int dt, const SqllmParams& p, const LaunchDims& d, hipStream_t s) {
    if (hipError_t e = sqllm_prepare(); e != hipSuccess) return e;
    switch (dt) {
        case kFP32: hipLaunchKernelGGL(sqllm_kernel<kFP32>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        case kFP16: hipLaunchKernelGGL(sqllm_kernel<kFP16>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        case kBF16: hipLaunchKernelGGL(sqllm_kernel<kBF16>, dim3(d.grid), dim3(d.block), d.lds, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_sqllm(int dt, const DecParams& dp, uint32_t dec_blocks,
                              const SqllmParams& gp, const LaunchDims& d, hipStream_t s) {
    if (hipError_t e = sqllm_prepare(); e != hipSuccess) return e;
    const dim3 grid(dec_blocks + d.grid), block(d.block);
    const bool two = d.two_per_cu && dt != kFP32;      // the fp32 instance would spill registers under the budget
    switch (dt) {
        case kFP32: hipLaunchKernelGGL((dec_sqllm_kernel<kFP32, false>), grid, block, d.lds, s, dp, dec_blocks, gp); break;
        case kFP16:
            if (two) hipLaunchKernelGGL((dec_sqllm_kernel<kFP16, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
            else hipLaunchKernelGGL((dec_sqllm_kernel<kFP16, false>), grid, block, d.lds, s, dp, dec_blocks, gp);
            break;
        case kBF16:
            if (two) hipLaunchKernelGGL((dec_sqllm_kernel<kBF16, true>), grid, block, d.lds, s, dp, dec_blocks, gp);
            else hipLaunchKernelGGL((dec_sqllm_kernel<kBF16, false>), grid, block, d.lds, s, dp, dec_blocks, gp);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec_sqllm_batch(int dt, const BatchParams<SqllmParams>& b, const LaunchDims& d, hipStream_t s) {
    if (hipError_t e = sqllm_prepare(); e != hipSuccess) return e;
    const dim3 grid(d.grid), block(d.block);
    if ((dt != kFP16 && dt != kBF16) || d.block != 1024u) return hipErrorInvalidValue;
    if (d.two_per_cu) {
        if (dt == kFP16) hipLaunchKernelGGL((dec_sqllm_batch_kernel<kFP16, true>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_sqllm_batch_kernel<kBF16, true>), grid, block, d.lds, s, b);
    } else {
        if (dt == kFP16) hipLaunchKernelGGL((dec_sqllm_batch_kernel<kFP16, false>), grid, block, d.lds, s, b);
        else hipLaunchKernelGGL((dec_sqllm_batch_kernel<kBF16, false>), grid, block, d.lds, s, b);
    }
    return hipGetLastError();
}

}  // namespace decdec
