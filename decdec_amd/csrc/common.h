// Shared device/host helpers for the DecDEC gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace decdec {

enum : int { kFP32 = 0, kFP16 = 1, kBF16 = 2 };

constexpr int kWave = 64;            // CDNA wavefront
constexpr int kChunk = 1024;         // selector chunk (reference macros.h:8)
constexpr int kBuckets = 32;         // selector buckets (reference macros.h:18)

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef short short2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define DD_GLOBAL_AS __attribute__((address_space(1)))

// ---------------------------------------------------------------------------------------------
// Storage-type traits: activations, scales, LUTs and outputs are fp32, fp16 or bf16 arrays.  All
// arithmetic is done in fp32; values are rounded once, when they are merged into the output.
// ---------------------------------------------------------------------------------------------
template <int DT> struct Elem;

template <> struct Elem<kFP32> {
    using store_t = float;
    static constexpr int bytes = 4;
    static __device__ __forceinline__ float load(const void* p, size_t i) { return ((const float*)p)[i]; }
    // storage bits of element i, and their value (lets a caller request a value long before it converts it)
    static __device__ __forceinline__ uint32_t load_raw(const void* p, size_t i) { return ((const uint32_t*)p)[i]; }
    static __device__ __forceinline__ float from_raw(uint32_t r) { return __uint_as_float(r); }
    static __device__ __forceinline__ uint32_t to_raw(float f) { return __float_as_uint(f); }
    // storage bits of the even-aligned pair (i, i + 1) and their values
    static __device__ __forceinline__ void load_raw2(const void* p, size_t i, uint32_t& a, uint32_t& b) {
        const u32x2 v = *(const u32x2*)((const uint32_t*)p + i); a = v[0]; b = v[1];
    }
    static __device__ __forceinline__ float from_raw2_lo(uint32_t a, uint32_t) { return __uint_as_float(a); }
    static __device__ __forceinline__ float from_raw2_hi(uint32_t, uint32_t b) { return __uint_as_float(b); }
    static __device__ __forceinline__ void store(void* p, size_t i, float v) { ((float*)p)[i] = v; }
    // Atomically add (v0, v1) to out[i], out[i+1]; i is even.
    static __device__ __forceinline__ void atomic_add2(void* out, size_t i, float v0, float v1) {
        atomicAdd((float*)out + i, v0);
        atomicAdd((float*)out + i + 1, v1);
    }
    static __device__ __forceinline__ void atomic_add1(void* out, size_t i, float v) {
        atomicAdd((float*)out + i, v);
    }
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// 16-bit compare-and-swap add for an output element that has no partner (odd tail).
template <typename F>
__device__ __forceinline__ void atomic_add_u16_cas(void* out, size_t i, F add_bits) {
    uint32_t* word = (uint32_t*)((uintptr_t)((uint16_t*)out + i) & ~(uintptr_t)3);
    const bool hi = (((uintptr_t)((uint16_t*)out + i)) & 2) != 0;
    uint32_t old = *word, assumed;
    do {
        assumed = old;
        uint16_t cur = hi ? (uint16_t)(assumed >> 16) : (uint16_t)(assumed & 0xFFFFu);
        uint16_t nxt = add_bits(cur);
        uint32_t repl = hi ? ((assumed & 0x0000FFFFu) | ((uint32_t)nxt << 16))
                           : ((assumed & 0xFFFF0000u) | nxt);
        old = atomicCAS(word, assumed, repl);
    } while (old != assumed);
}

template <> struct Elem<kFP16> {
    using store_t = _Float16;
    static constexpr int bytes = 2;
    static __device__ __forceinline__ float load(const void* p, size_t i) { return (float)((const _Float16*)p)[i]; }
    static __device__ __forceinline__ uint32_t load_raw(const void* p, size_t i) { return ((const uint16_t*)p)[i]; }
    static __device__ __forceinline__ float from_raw(uint32_t r) {
        const uint16_t h = (uint16_t)r; _Float16 v; __builtin_memcpy(&v, &h, 2); return (float)v;
    }
    static __device__ __forceinline__ uint32_t to_raw(float f) {
        const _Float16 v = (_Float16)f; uint16_t h; __builtin_memcpy(&h, &v, 2); return h;
    }
    static __device__ __forceinline__ void load_raw2(const void* p, size_t i, uint32_t& a, uint32_t& b) {
        a = *(const uint32_t*)((const uint16_t*)p + i); b = 0u;
    }
    static __device__ __forceinline__ float from_raw2_lo(uint32_t a, uint32_t) { return from_raw(a & 0xFFFFu); }
    static __device__ __forceinline__ float from_raw2_hi(uint32_t a, uint32_t) { return from_raw(a >> 16); }
    static __device__ __forceinline__ void store(void* p, size_t i, float v) { ((_Float16*)p)[i] = (_Float16)v; }
    static __device__ __forceinline__ void atomic_add2(void* out, size_t i, float v0, float v1) {
        half2_t v = {(_Float16)v0, (_Float16)v1};
        __builtin_amdgcn_global_atomic_fadd_v2f16((DD_GLOBAL_AS half2_t*)((_Float16*)out + i), v);
    }
    static __device__ __forceinline__ void atomic_add1(void* out, size_t i, float v) {
        atomic_add_u16_cas(out, i, [v](uint16_t cur) {
            _Float16 c; __builtin_memcpy(&c, &cur, 2);
            _Float16 r = (_Float16)((float)c + v);
            uint16_t o; __builtin_memcpy(&o, &r, 2); return o; });
    }
};

template <> struct Elem<kBF16> {
    using store_t = uint16_t;
    static constexpr int bytes = 2;
    static __device__ __forceinline__ float load(const void* p, size_t i) { return bf16_bits_to_f32(((const uint16_t*)p)[i]); }
    static __device__ __forceinline__ uint32_t load_raw(const void* p, size_t i) { return ((const uint16_t*)p)[i]; }
    static __device__ __forceinline__ float from_raw(uint32_t r) { return bf16_bits_to_f32((uint16_t)r); }
    static __device__ __forceinline__ uint32_t to_raw(float f) { return f32_to_bf16_bits(f); }
    static __device__ __forceinline__ void load_raw2(const void* p, size_t i, uint32_t& a, uint32_t& b) {
        a = *(const uint32_t*)((const uint16_t*)p + i); b = 0u;
    }
    static __device__ __forceinline__ float from_raw2_lo(uint32_t a, uint32_t) { return __uint_as_float(a << 16); }
    static __device__ __forceinline__ float from_raw2_hi(uint32_t a, uint32_t) { return __uint_as_float(a & 0xFFFF0000u); }
    static __device__ __forceinline__ void store(void* p, size_t i, float v) { ((uint16_t*)p)[i] = f32_to_bf16_bits(v); }
    static __device__ __forceinline__ void atomic_add2(void* out, size_t i, float v0, float v1) {
        short2_t v = {(short)f32_to_bf16_bits(v0), (short)f32_to_bf16_bits(v1)};
        __builtin_amdgcn_global_atomic_fadd_v2bf16((DD_GLOBAL_AS short2_t*)((uint16_t*)out + i), v);
    }
    static __device__ __forceinline__ void atomic_add1(void* out, size_t i, float v) {
        atomic_add_u16_cas(out, i, [v](uint16_t cur) { return f32_to_bf16_bits(bf16_bits_to_f32(cur) + v); });
    }
};

__device__ __forceinline__ uint32_t lane_id() {
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}
// number of set bits of a 64-lane ballot below the calling lane
__device__ __forceinline__ uint32_t ballot_rank(unsigned long long m) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace decdec
