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
};

// Standalone kernels.
hipError_t launch_dec(int dt, const DecParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_anyprec(int dt, int bits, const AnyprecParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_anyprec_dequant(int dt, int bits, const uint32_t* qweight, const void* lut, void* weight,
                                  uint32_t N, uint32_t K, hipStream_t s);
hipError_t launch_lutgemm(int dt, const LutgemmParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_sqllm(int dt, const SqllmParams& p, const LaunchDims& d, hipStream_t s);
hipError_t launch_burner(uint32_t blocks, long long iters, hipStream_t s);

// Single-launch fused kernels: workgroups [0, dec_blocks) play the DEC role, the rest the base GEMV.
// d.grid counts the GEMV workgroups only; d.block is 1024.
hipError_t launch_dec_anyprec(int dt, int bits, const DecParams& dp, uint32_t dec_blocks,
                              const AnyprecParams& gp, const LaunchDims& d, hipStream_t s);
hipError_t launch_dec_lutgemm(int dt, const DecParams& dp, uint32_t dec_blocks,
                              const LutgemmParams& gp, const LaunchDims& d, hipStream_t s);
hipError_t launch_dec_sqllm(int dt, const DecParams& dp, uint32_t dec_blocks,
                            const SqllmParams& gp, const LaunchDims& d, hipStream_t s);

}  // namespace decdec
