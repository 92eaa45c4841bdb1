// Standalone DEC kernel (select + fetch + residual GEMV + merge) and the CU-occupying spin kernel.
#include "launch.h"

namespace decdec {

// NW = waves of the workgroup (16 by default; 4 and 8 exist for callers that want DEC workgroups which hold
// a smaller share of a compute unit).
template <int DT, int NW>
__global__ __launch_bounds__(NW * kWave) void dec_kernel(const DecParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    dec_role<DT, NW>(p, blockIdx.x, smem);
}

template <int NW>
static hipError_t launch_dec_nw(int dt, const DecParams& p, const LaunchDims& d, hipStream_t s) {
    switch (dt) {
        case kFP32: hipLaunchKernelGGL((dec_kernel<kFP32, NW>), dim3(d.grid), dim3(NW * kWave), d.lds, s, p); break;
        case kFP16: hipLaunchKernelGGL((dec_kernel<kFP16, NW>), dim3(d.grid), dim3(NW * kWave), d.lds, s, p); break;
        case kBF16: hipLaunchKernelGGL((dec_kernel<kBF16, NW>), dim3(d.grid), dim3(NW * kWave), d.lds, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dec(int dt, const DecParams& p, const LaunchDims& d, hipStream_t s) {
    switch (d.block / kWave) {
        case 4: return launch_dec_nw<4>(dt, p, d, s);
        case 8: return launch_dec_nw<8>(dt, p, d, s);
        case 16: return launch_dec_nw<16>(dt, p, d, s);
        default: return hipErrorInvalidValue;
    }
}

// Pure-ALU spin that keeps `blocks` workgroups of 1024 threads resident (the counterpart of the
// reference's sm_burner_kernel, decdec_extension/decdec.cu:790-833): used to time a base GEMV with
// part of the chip taken away.
__device__ float burner_sink[1];

__global__ __launch_bounds__(1024) void burner_kernel(long long iters) {
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = (float)(threadIdx.x + i);
    for (long long it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = acc[i] * 1.00001f + 0.0001f;
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) sum += acc[i];
    if (sum == 12345.678f) burner_sink[0] = sum;      // keeps the loop alive; practically never true
}

hipError_t launch_burner(uint32_t blocks, long long iters, hipStream_t s) {
    if (blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(burner_kernel, dim3(blocks), dim3(1024), 0, s, iters);
    return hipGetLastError();
}

}  // namespace decdec
