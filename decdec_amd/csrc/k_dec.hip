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

// Plain read of `rows` pieces-of-rows, nothing else: the ceiling a fetch can reach on the memory it points at (pinned
// host memory read zero-copy over the host link, or device memory).  A wave reads VEC x 256 contiguous bytes per
// request (VEC dwords per lane), eight requests in flight; consecutive requests of a workgroup walk along a row,
// rows are visited in a scattered order when `scramble` is set (as the rows DEC selects are).
template <int VEC>
__global__ __launch_bounds__(1024) void read_probe_kernel(const uint32_t* __restrict__ src, const unsigned long long pieces,
                                                          const uint32_t pieces_per_row, const unsigned long long rows,
                                                          const unsigned long long row_words, const int scramble,
                                                          uint32_t* __restrict__ sink) {
    typedef uint32_t vec_t __attribute__((ext_vector_type(VEC)));
    constexpr int U = 8;
    const uint32_t lane = threadIdx.x & 63u;
    const unsigned long long wave = (unsigned long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const unsigned long long nwaves = (unsigned long long)gridDim.x * (blockDim.x >> 6);
    uint32_t acc = 0;
    for (unsigned long long g0 = wave; g0 < pieces; g0 += nwaves * U) {
        vec_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned long long g = g0 + (unsigned long long)u * nwaves;
            const unsigned long long gc = g < pieces ? g : pieces - 1;
            unsigned long long row = gc / pieces_per_row;
            const uint32_t col = (uint32_t)(gc % pieces_per_row);
            if (scramble) row = (row * 7919ull + 13ull) % rows;
            v[u] = *(const vec_t*)(src + row * row_words + (size_t)col * (64u * VEC) + (size_t)lane * VEC);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc ^= v[u][k];
        }
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;              // keeps the loads alive; practically never true
}

hipError_t launch_read_probe(const void* src, unsigned long long row_bytes, unsigned long long rows, uint32_t vec_words,
                             uint32_t blocks, int scramble, void* sink, hipStream_t s) {
    const unsigned long long row_words = row_bytes / 4u;
    const uint32_t ppr = (uint32_t)(row_words / (64u * vec_words));
    if (ppr == 0 || row_words % (64u * vec_words) != 0 || rows == 0 || blocks == 0) return hipErrorInvalidValue;
    const unsigned long long pieces = rows * ppr;
    const dim3 grid(blocks), block(1024);
    if (vec_words == 1) hipLaunchKernelGGL((read_probe_kernel<1>), grid, block, 0, s, (const uint32_t*)src, pieces, ppr, rows, row_words, scramble, (uint32_t*)sink);
    else if (vec_words == 2) hipLaunchKernelGGL((read_probe_kernel<2>), grid, block, 0, s, (const uint32_t*)src, pieces, ppr, rows, row_words, scramble, (uint32_t*)sink);
    else if (vec_words == 4) hipLaunchKernelGGL((read_probe_kernel<4>), grid, block, 0, s, (const uint32_t*)src, pieces, ppr, rows, row_words, scramble, (uint32_t*)sink);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_burner(uint32_t blocks, long long iters, hipStream_t s) {
    if (blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(burner_kernel, dim3(blocks), dim3(1024), 0, s, iters);
    return hipGetLastError();
}

}  // namespace decdec
