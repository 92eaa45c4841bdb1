// Decode-step helpers around the linear layers: rotary embedding + KV-cache append, grouped-query
// attention of one new token over the cache, and the gated activation of the feed-forward block.
// The reference leaves these to torch.compile (end-to-end/generate.py); here they are three small kernels
// so that a captured decode step is a short chain of launches.  Token position comes from device memory:
// a captured step advances it on the device and is replayed unchanged.
#include "launch.h"

namespace decdec {

// One element of a rotated pair: x c - partner s for the first element of the pair, x c + partner s for the second.
__device__ __forceinline__ float rope_rotate(float x, float partner, float c, float s, bool first) {
    const float ps = __fmul_rn(partner, s);
    return __builtin_fmaf(x, c, first ? -ps : ps);
}

template <int DT>
__global__ __launch_bounds__(256) void rope_cache_kernel(const RopeCacheParams p) {
    using E = Elem<DT>;
    const uint32_t D = p.head_dim, half = D / 2;
    const uint32_t pairs = (p.n_head + p.n_kv) * half, vals = p.n_kv * D;
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    const long long pos64 = *p.pos;
    if (pos64 < 0 || pos64 >= (long long)p.max_seq) return;            // nothing may be written outside the cache
    const uint32_t pos = (uint32_t)pos64;
    if (t < pairs) {
        const uint32_t head = t / half, i = t % half;
        const float x1 = E::load(p.qkv, (size_t)head * D + i), x2 = E::load(p.qkv, (size_t)head * D + i + half);
        const float c = E::load(p.cos_table, (size_t)pos * D + i), s = E::load(p.sin_table, (size_t)pos * D + i);
        const float y1 = rope_rotate(x1, x2, c, s, true), y2 = rope_rotate(x2, x1, c, s, false);
        if (head < p.n_head) {
            E::store(p.q_out, (size_t)head * D + i, y1);
            E::store(p.q_out, (size_t)head * D + i + half, y2);
        } else {
            const size_t base = ((size_t)(head - p.n_head) * p.max_seq + pos) * D;
            E::store(p.k_cache, base + i, y1);
            E::store(p.k_cache, base + i + half, y2);
        }
    } else if (t < pairs + vals) {
        const uint32_t j = t - pairs, kvh = j / D, d = j % D;
        const float v = E::load(p.qkv, (size_t)(p.n_head + p.n_kv) * D + j);
        E::store(p.v_cache, ((size_t)kvh * p.max_seq + pos) * D + d, v);
    }
}

// Sum over the LPP lanes that share a cache position (LPP = 8 or 16 neighbouring lanes).
template <int LPP>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_read<0xB1, 0xF>(v);                     // quad_perm [1,0,3,2]
    v += dpp_read<0x4E, 0xF>(v);                     // quad_perm [2,3,0,1]
    if constexpr (LPP == 8) {
        v += dpp_read<0x141, 0xF>(v);                // row_half_mirror: the other quad of the half row
    } else {
        v += dpp_read<0x124, 0xF>(v);                // row_ror 4
        v += dpp_read<0x128, 0xF>(v);                // row_ror 8
    }
    return v;
}

// `nsplit` workgroups per query head share the positions 0 .. pos (contiguous ranges).  In a workgroup, a group of
// D/8 lanes owns a cache position (16 bytes of K and of V per lane); a wave visits 64 / (D/8) positions per step
// and four steps per loop trip (their rows requested together), the 16 waves interleave, every lane group keeps
// its own running maximum / sum / output (online softmax), and the groups are merged through LDS.  With
// nsplit > 1 every workgroup leaves (max, sum, output) of its range in the workspace and the ranges of a head are
// merged either by the workgroup of the head that arrives last (see the end of the kernel) or by a second, small
// kernel (a merge behind device-scope fences writes back and invalidates whole L2 caches on this multi-die GPU:
// measured 110 us per launch).
template <int DT, int D>
__global__ __launch_bounds__(1024) void decode_attention_kernel(const AttentionParams p) {
    using E = Elem<DT>;
    constexpr int LPP = D / 8, PPW = 64 / LPP, NG = 16 * PPW, UN = 4;
    extern __shared__ __align__(16) unsigned char smem[];
    float* pm = (float*)smem;               // [NG] maxima
    float* pw = pm + NG;                    // [NG] merge weights
    float* pl = pw + NG;                    // [NG] sums
    float* po = pl + NG;                    // [NG][D] outputs
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t sub = lane / LPP, dl = lane % LPP;
    const uint32_t h = blockIdx.x / p.nsplit, split = blockIdx.x % p.nsplit;
    const uint32_t kvh = h / (p.n_head / p.n_kv);
    const uint16_t* kc = (const uint16_t*)p.k_cache + (size_t)kvh * p.max_seq * D + 8 * dl;
    const uint16_t* vc = (const uint16_t*)p.v_cache + (size_t)kvh * p.max_seq * D + 8 * dl;
    long long pos64 = *p.pos;
    // Short sequences: sharing a head's positions between workgroups costs more (partial results, a counter, a
    // second pass: about 3 us of memory round trips) than it saves, so the head's first workgroup takes them all.
    const bool alone = p.counters != nullptr && pos64 + 1 <= (long long)p.single_below;
    if (alone && split != 0u) return;
    const uint32_t nsplit = alone ? 1u : p.nsplit;
    const bool fused = p.qkv != nullptr;
    const bool in_cache = pos64 >= 0 && pos64 < (long long)p.max_seq;      // the new token has a cache row
    if (pos64 < 0) pos64 = 0;
    uint32_t qr[4];
    u32x4 knew = {0u, 0u, 0u, 0u}, vnew = {0u, 0u, 0u, 0u};
    const uint32_t newpos = (fused && in_cache) ? (uint32_t)pos64 : 0xFFFFFFFFu;
    if (fused) {
        // the lane's eight elements start at 8 dl; their rotation partners sit half a head away; the tables hold
        // the angle of pair i at [pos][i], i < D / 2 (a position past the tables uses their last row)
        constexpr uint32_t half = D / 2;
        const uint32_t e0 = 8u * dl, pe0 = (e0 + half) % (uint32_t)D, te0 = e0 % half;
        const bool first = e0 < half;
        const size_t trow = (size_t)((pos64 < (long long)p.max_seq) ? pos64 : (long long)p.max_seq - 1) * D;
        const u32x4 cr = *(const u32x4*)((const uint16_t*)p.cos_table + trow + te0);
        const u32x4 sr = *(const u32x4*)((const uint16_t*)p.sin_table + trow + te0);
        const uint16_t* qh = (const uint16_t*)p.qkv + (size_t)h * D;
        const uint16_t* kh = (const uint16_t*)p.qkv + (size_t)(p.n_head + kvh) * D;
        const u32x4 qs = *(const u32x4*)(qh + e0), qp = *(const u32x4*)(qh + pe0);
        const u32x4 ks = *(const u32x4*)(kh + e0), kp = *(const u32x4*)(kh + pe0);
        vnew = *(const u32x4*)((const uint16_t*)p.qkv + (size_t)(p.n_head + p.n_kv + kvh) * D + e0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t qo = 0u, ko = 0u;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int sh = 16 * hf;
                const float c = E::from_raw((cr[e] >> sh) & 0xFFFFu), sn = E::from_raw((sr[e] >> sh) & 0xFFFFu);
                const float xq = E::from_raw((qs[e] >> sh) & 0xFFFFu), pq = E::from_raw((qp[e] >> sh) & 0xFFFFu);
                const float xk = E::from_raw((ks[e] >> sh) & 0xFFFFu), pk = E::from_raw((kp[e] >> sh) & 0xFFFFu);
                // first half: x c - partner s; second half: x c + partner s, rounded to the storage type as a
                // separate rotary kernel stores them (the compiler may round a near-tie the other way here)
                const float yq = rope_rotate(xq, pq, c, sn, first), yk = rope_rotate(xk, pk, c, sn, first);
                qo |= (E::to_raw(yq) & 0xFFFFu) << sh;
                ko |= (E::to_raw(yk) & 0xFFFFu) << sh;
            }
            qr[e] = qo;
            knew[e] = ko;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) qr[e] = *(const uint32_t*)((const uint16_t*)p.q + (size_t)h * D + 8 * dl + 2 * e);
    }
    const uint32_t len = (uint32_t)((pos64 + 1 < (long long)p.max_seq) ? pos64 + 1 : (long long)p.max_seq);
    // this workgroup's positions: [lo, hi), ranges of a multiple of 16 PPW positions
    const uint32_t chunk = ((len + nsplit - 1u) / nsplit + 16u * PPW - 1u) / (16u * PPW) * (16u * PPW);
    const uint32_t lo = split * chunk < len ? split * chunk : len;
    const uint32_t hi = (lo + chunk) < len ? (lo + chunk) : len;
    float m = -__builtin_inff(), l = 0.f, o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = 0.f;
    // The scan is bound by the instruction issue of the workgroup's compute unit, so it is written to need few
    // instructions: the scores come from packed dot products of the raw registers (fp32 accumulation, scaled
    // afterwards), and the UN rows of a trip share one update of the running maximum (one rescaling of the output
    // instead of UN).
    for (uint32_t p0 = lo + wave * PPW; p0 < hi; p0 += UN * 16 * PPW) {
        u32x4 kr[UN], vr[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const uint32_t pp = p0 + (uint32_t)u * 16 * PPW + sub;
            const uint32_t ppc = pp < hi ? pp : hi - 1u;
            kr[u] = *(const u32x4*)(kc + (size_t)ppc * D);
            vr[u] = *(const u32x4*)(vc + (size_t)ppc * D);
            if (ppc == newpos) { kr[u] = knew; vr[u] = vnew; }             // the new token's row is not in the cache yet
        }
        float sc[UN];
        float mn = m;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            float t = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t ka = kr[u][e], qb = qr[e];
                if constexpr (DT == kFP16) {
                    half2_t a, b;
                    __builtin_memcpy(&a, &ka, 4); __builtin_memcpy(&b, &qb, 4);
                    t = __builtin_amdgcn_fdot2(a, b, t, false);
                } else {
                    bf16x2_t a, b;
                    __builtin_memcpy(&a, &ka, 4); __builtin_memcpy(&b, &qb, 4);
                    t = __builtin_amdgcn_fdot2_f32_bf16(a, b, t, false);
                }
            }
            t = group_sum<LPP>(t) * p.scale;
            const bool valid = p0 + (uint32_t)u * 16 * PPW + sub < hi;
            sc[u] = valid ? t : -__builtin_inff();
            mn = sc[u] > mn ? sc[u] : mn;
        }
        // a lane group without a row in the trip (mn still -inf) changes nothing: its weights are exp(-inf - 0) = 0
        const float mb = mn == -__builtin_inff() ? 0.f : mn;
        const float corr = mn == -__builtin_inff() ? 1.f : __expf(m - mn); // m = -inf, mn finite: corr = 0
        m = mn;
        l *= corr;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] *= corr;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const float pr = __expf(sc[u] - mb);                           // a row past the range: exp(-inf) = 0
            l += pr;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (DT == kFP16) {
                    half2_t v2;
                    const uint32_t vv = vr[u][e];
                    __builtin_memcpy(&v2, &vv, 4);
                    o[2 * e] = __builtin_fmaf(pr, (float)v2[0], o[2 * e]);
                    o[2 * e + 1] = __builtin_fmaf(pr, (float)v2[1], o[2 * e + 1]);
                } else {
                    o[2 * e] = __builtin_fmaf(pr, E::from_raw(vr[u][e] & 0xFFFFu), o[2 * e]);
                    o[2 * e + 1] = __builtin_fmaf(pr, E::from_raw(vr[u][e] >> 16), o[2 * e + 1]);
                }
            }
        }
    }
    // cache append: one workgroup per key/value head (its first query head, the range that holds the position)
    if (newpos != 0xFFFFFFFFu && h % (p.n_head / p.n_kv) == 0u && newpos >= lo && newpos < hi && tid < (uint32_t)LPP) {
        *(u32x4*)((uint16_t*)p.k_cache + ((size_t)kvh * p.max_seq + newpos) * D + 8 * dl) = knew;
        *(u32x4*)((uint16_t*)p.v_cache + ((size_t)kvh * p.max_seq + newpos) * D + 8 * dl) = vnew;
    }
    const uint32_t g = wave * PPW + sub;
    if (dl == 0) { pm[g] = m; pl[g] = l; }
#pragma unroll
    for (int e = 0; e < 8; ++e) po[(size_t)g * D + 8 * dl + e] = o[e];
    __syncthreads();
    // merge of the NG groups: thread i < NG turns group i's maximum into its weight exp(m_i - M) (M = overall
    // maximum, found by every such thread from the NG maxima), then thread d < D sums column d
    float M = -__builtin_inff();
    if (tid < (uint32_t)NG || tid < (uint32_t)D) {
        for (int i = 0; i < NG; ++i) M = pm[i] > M ? pm[i] : M;
    }
    if (tid < (uint32_t)NG) {
        const float mi = pm[tid];
        pw[tid] = (mi == -__builtin_inff()) ? 0.f : __expf(mi - M);
    }
    __syncthreads();
    float L = 0.f, O = 0.f;
    if (tid < (uint32_t)D) {
#pragma unroll 8
        for (int i = 0; i < NG; ++i) {
            const float w = pw[i];
            L += pl[i] * w;
            O += po[(size_t)i * D + tid] * w;
        }
    }
    if (nsplit == 1u) {
        if (tid < (uint32_t)D) E::store(p.out, (size_t)h * D + tid, O / L);
        return;
    }
    // partial result of this range: [D] outputs, then the maximum and the sum
    float* ws = p.workspace + ((size_t)h * nsplit + split) * (D + 2);
    if (p.counters == nullptr) {                     // a second kernel merges the ranges
        if (tid < (uint32_t)D) {
            ws[tid] = O;
            if (tid == 0) { ws[D] = M; ws[D + 1] = L; }
        }
        return;
    }
    // Merge by the workgroup of the head that finishes last, without fences (a device-scope fence writes back and
    // invalidates a whole L2 on this multi-die GPU): the partial results travel as relaxed device-scope atomic
    // stores and loads, which go past the L2 to memory; a workgroup counts itself in only after its stores have been
    // acknowledged, so whoever draws the last number finds every range's result in memory.
    if (tid < (uint32_t)D) {
        __hip_atomic_store(ws + tid, O, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) {
            __hip_atomic_store(ws + D, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(ws + D + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t* flag = (uint32_t*)pm;                  // the maxima are no longer read
    if (tid == 0) {
        const uint32_t drawn = __hip_atomic_fetch_add(p.counters + h, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        flag[0] = (drawn + 1u == nsplit) ? 1u : 0u;
        if (drawn + 1u == nsplit) __hip_atomic_store(p.counters + h, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
    }
    __syncthreads();
    if (flag[0] == 0u || tid >= (uint32_t)D) return;
    const float* wh = p.workspace + (size_t)h * nsplit * (D + 2);
    float ms[8], ls[8], os[8];
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) {
        const uint32_t c = (uint32_t)sp < nsplit ? (uint32_t)sp : 0u;          // all loads in flight together
        ms[sp] = __hip_atomic_load(wh + (size_t)c * (D + 2) + D, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ls[sp] = __hip_atomic_load(wh + (size_t)c * (D + 2) + D + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        os[sp] = __hip_atomic_load(wh + (size_t)c * (D + 2) + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float Mg = -__builtin_inff();
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) if ((uint32_t)sp < nsplit && ms[sp] > Mg) Mg = ms[sp];
    float Lg = 0.f, Og = 0.f;
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) {
        if ((uint32_t)sp < nsplit) {
            const float w = (ms[sp] == -__builtin_inff()) ? 0.f : __expf(ms[sp] - Mg);
            Lg += ls[sp] * w;
            Og += os[sp] * w;
        }
    }
    E::store(p.out, (size_t)h * D + tid, Og / Lg);
}

// Second step with nsplit > 1: one workgroup of D threads per head combines the ranges' partial results.
template <int DT, int D>
__global__ __launch_bounds__(D) void decode_attention_merge_kernel(const AttentionParams p) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, h = blockIdx.x, nsplit = p.nsplit;
    const float* wh = p.workspace + (size_t)h * nsplit * (D + 2);
    float ms[8], ls[8], os[8];
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) {
        const uint32_t c = (uint32_t)sp < nsplit ? (uint32_t)sp : 0u;          // all loads in flight together
        ms[sp] = wh[(size_t)c * (D + 2) + D];
        ls[sp] = wh[(size_t)c * (D + 2) + D + 1];
        os[sp] = wh[(size_t)c * (D + 2) + tid];
    }
    float Mg = -__builtin_inff();
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) if ((uint32_t)sp < nsplit && ms[sp] > Mg) Mg = ms[sp];
    float Lg = 0.f, Og = 0.f;
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) {
        if ((uint32_t)sp < nsplit) {
            const float w = (ms[sp] == -__builtin_inff()) ? 0.f : __expf(ms[sp] - Mg);
            Lg += ls[sp] * w;
            Og += os[sp] * w;
        }
    }
    E::store(p.out, (size_t)h * D + tid, Og / Lg);
}

template <int DT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const void* __restrict__ gate_up, void* __restrict__ out, uint32_t n) {
    using E = Elem<DT>;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float a = E::load(gate_up, i), b = E::load(gate_up, (size_t)n + i);
    E::store(out, i, a / (1.f + __expf(-a)) * b);
}

// ---- dense 16-bit GEMV: the unquantised output head of a decoder ------------------------------------------
// out[n] = sum_k W[n][k] x[k], W row-major.  Bound by the read of W (the head of an 8B model is a gigabyte per
// token), so the kernel is a stream: a wave owns four rows, a lane 16 bytes of each per step of 512 columns, two
// steps (eight 16-byte loads of W per lane, never reused, hence non-temporal) in flight together; x comes through
// the vector cache (every wave reads the same few KB).  Products accumulate in fp32, one rounding at the store.
typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ float dot8(const u32x4& w, const u32x4& x, float acc) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if constexpr (DT == kFP16) {
            half2_t a, b;
            const uint32_t wa = w[j], xb = x[j];
            __builtin_memcpy(&a, &wa, 4); __builtin_memcpy(&b, &xb, 4);
            acc = __builtin_amdgcn_fdot2(a, b, acc, false);
        } else {
            acc = __builtin_fmaf(__uint_as_float(w[j] << 16), __uint_as_float(x[j] << 16), acc);
            acc = __builtin_fmaf(__uint_as_float(w[j] & 0xFFFF0000u), __uint_as_float(x[j] & 0xFFFF0000u), acc);
        }
    }
    return acc;
}

constexpr int kDenseRows = 4;          // rows per wave
constexpr int kDenseWaves = 4;         // waves per workgroup

template <int DT>
__global__ __launch_bounds__(kDenseWaves * 64) void dense_gemv_kernel(const void* __restrict__ weight,
                                                                      const void* __restrict__ x, void* __restrict__ out,
                                                                      const uint32_t N, const uint32_t K) {
    using E = Elem<DT>;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t row0 = (blockIdx.x * (uint32_t)kDenseWaves + wave) * (uint32_t)kDenseRows;
    if (row0 >= N) return;
    const uint16_t* wr[kDenseRows];
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r) {
        const uint32_t rr = row0 + r < N ? row0 + r : N - 1u;      // rows past the end re-read the last one; not stored
        wr[r] = (const uint16_t*)weight + (size_t)rr * K;
    }
    float acc[kDenseRows] = {0.f, 0.f, 0.f, 0.f};
    const uint32_t steps = (K + 511u) / 512u;
    for (uint32_t s = 0; s < steps; s += 2u) {
        u32x4 wv[2][kDenseRows], xv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const uint32_t col = ((s + u) * 64u + lane) * 8u;
            const bool ok = col < K;                               // K is a multiple of 8
            const uint32_t c = ok ? col : 0u;
            xv[u] = *(const u32x4*)((const uint16_t*)x + c);
            if (!ok) xv[u] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int r = 0; r < kDenseRows; ++r) wv[u][r] = __builtin_nontemporal_load((const u32x4*)(wr[r] + c));
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < kDenseRows; ++r) acc[r] = dot8<DT>(wv[u][r], xv[u], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r) acc[r] = wave_sum(acc[r]);
    if (lane < (uint32_t)kDenseRows && row0 + lane < N) {
        const float v = lane == 0 ? acc[0] : (lane == 1 ? acc[1] : (lane == 2 ? acc[2] : acc[3]));
        E::store(out, row0 + lane, v);
    }
}

hipError_t launch_dense_gemv(int dt, const void* weight, const void* x, void* out, uint32_t N, uint32_t K, hipStream_t s) {
    const uint32_t rows_per_block = (uint32_t)(kDenseRows * kDenseWaves);
    const dim3 grid((N + rows_per_block - 1u) / rows_per_block), block(kDenseWaves * 64);
    if (dt == kFP16) hipLaunchKernelGGL((dense_gemv_kernel<kFP16>), grid, block, 0, s, weight, x, out, N, K);
    else if (dt == kBF16) hipLaunchKernelGGL((dense_gemv_kernel<kBF16>), grid, block, 0, s, weight, x, out, N, K);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// h = x + y (skipped when y is null), normed = h / rms(h) * weight: the residual add and the RMS normalisation that
// follows it in a decoder block.  One workgroup per row, four neighbouring elements per thread and pass (one 8-byte
// load each of x, y and the weight, all requested before anything is used), statistics in fp32.
template <int DT, int PASSES>
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(const void* __restrict__ x, const void* __restrict__ y,
                                                           const void* __restrict__ weight, void* __restrict__ h_out,
                                                           void* __restrict__ normed_out, uint32_t dim, float eps) {
    using E = Elem<DT>;
    __shared__ float wsum[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, nw = blockDim.x >> 6;
    const size_t row = (size_t)blockIdx.x * dim;
    const bool have_y = y != nullptr;
    u32x2 xr[PASSES], yr[PASSES], wr[PASSES];
#pragma unroll
    for (int k = 0; k < PASSES; ++k) {
        const uint32_t i = 4u * (tid + (uint32_t)k * blockDim.x);
        const uint32_t ic = (i + 4u <= dim) ? i : 0u;       // groups past the end re-read the first one; never used
        xr[k] = *(const u32x2*)((const uint16_t*)x + row + ic);
        yr[k] = have_y ? *(const u32x2*)((const uint16_t*)y + row + ic) : u32x2{0u, 0u};
        wr[k] = *(const u32x2*)((const uint16_t*)weight + ic);
    }
    float v[PASSES][4];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < PASSES; ++k) {
        const uint32_t i = 4u * (tid + (uint32_t)k * blockDim.x);
        const bool ok = i + 4u <= dim;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t sh = (e & 1) ? 16u : 0u;
            float a = E::from_raw((xr[k][e >> 1] >> sh) & 0xFFFFu);
            if (have_y) a = E::from_raw(E::to_raw(a + E::from_raw((yr[k][e >> 1] >> sh) & 0xFFFFu)));   // as stored
            v[k][e] = ok ? a : 0.f;
            ss += v[k][e] * v[k][e];
        }
        if (ok && have_y && h_out != nullptr) {
            u32x2 o;
            o[0] = E::to_raw(v[k][0]) | (E::to_raw(v[k][1]) << 16);
            o[1] = E::to_raw(v[k][2]) | (E::to_raw(v[k][3]) << 16);
            *(u32x2*)((uint16_t*)h_out + row + i) = o;
        }
    }
    ss = wave_sum_dpp(ss);                                  // total in lane 63
    if (lane == 63) wsum[wave] = ss;
    __syncthreads();
    float tot = 0.f;
    for (uint32_t w = 0; w < nw; ++w) tot += wsum[w];
    const float r = __builtin_amdgcn_rsqf(tot / (float)dim + eps);
#pragma unroll
    for (int k = 0; k < PASSES; ++k) {
        const uint32_t i = 4u * (tid + (uint32_t)k * blockDim.x);
        if (i + 4u <= dim) {
            float o4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o4[e] = v[k][e] * r * E::from_raw((wr[k][e >> 1] >> ((e & 1) ? 16u : 0u)) & 0xFFFFu);
            u32x2 o;
            o[0] = E::to_raw(o4[0]) | (E::to_raw(o4[1]) << 16);
            o[1] = E::to_raw(o4[2]) | (E::to_raw(o4[3]) << 16);
            *(u32x2*)((uint16_t*)normed_out + row + i) = o;
        }
    }
}

template <int DT>
static hipError_t launch_add_rmsnorm_dt(const void* x, const void* y, const void* weight, void* h_out, void* normed_out,
                                        uint32_t rows, uint32_t dim, float eps, hipStream_t s) {
    const uint32_t groups = dim / 4u;
    uint32_t threads = 64;
    while (threads < 1024 && threads < groups) threads *= 2;
    const dim3 grid(rows), block(threads);
    if (groups <= threads)
        hipLaunchKernelGGL((add_rmsnorm_kernel<DT, 1>), grid, block, 0, s, x, y, weight, h_out, normed_out, dim, eps);
    else if (groups <= 2 * threads)
        hipLaunchKernelGGL((add_rmsnorm_kernel<DT, 2>), grid, block, 0, s, x, y, weight, h_out, normed_out, dim, eps);
    else
        hipLaunchKernelGGL((add_rmsnorm_kernel<DT, 4>), grid, block, 0, s, x, y, weight, h_out, normed_out, dim, eps);
    return hipGetLastError();
}

hipError_t launch_add_rmsnorm(int dt, const void* x, const void* y, const void* weight, void* h_out, void* normed_out,
                              uint32_t rows, uint32_t dim, float eps, hipStream_t s) {
    if (dim % 4u != 0 || dim > 16384u) return hipErrorInvalidValue;
    if (dt == kFP16) return launch_add_rmsnorm_dt<kFP16>(x, y, weight, h_out, normed_out, rows, dim, eps, s);
    if (dt == kBF16) return launch_add_rmsnorm_dt<kBF16>(x, y, weight, h_out, normed_out, rows, dim, eps, s);
    return hipErrorInvalidValue;
}

// ---- greedy pick: argmax of the logits and the bookkeeping of a decode step ---------------------------
// Key of a logit: its value mapped to an unsigned integer that orders like the float (NaN with the sign bit
// clear above +inf, as torch.argmax treats it), then the complement of the index, so that the largest key is
// the largest logit and, among equal ones, the one with the smallest index.
__device__ __forceinline__ unsigned long long pick_key(float v, uint32_t idx) {
    const uint32_t b = __float_as_uint(v);
    const uint32_t u = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long)u << 32) | (unsigned long long)(0xFFFFFFFFu - idx);
}

__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long k) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const unsigned long long o = __shfl_xor(k, off, 64);
        k = o > k ? o : k;
    }
    return k;
}

constexpr int kPickBlocks = 128;      // partial results (and workgroups of the first kernel)

template <int DT>
__global__ __launch_bounds__(256) void greedy_partial_kernel(const void* __restrict__ logits, const uint32_t n,
                                                            unsigned long long* __restrict__ partial,
                                                            float* __restrict__ copy_out) {
    using E = Elem<DT>;
    __shared__ unsigned long long wk[4];
    unsigned long long best = 0ull;                      // below every key of a real element
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += (uint32_t)kPickBlocks * 256u) {
        const float v = E::load(logits, i);
        if (copy_out != nullptr) copy_out[i] = v;
        const unsigned long long k = pick_key(v, i);
        best = k > best ? k : best;
    }
    best = wave_max_u64(best);
    if ((threadIdx.x & 63u) == 0) wk[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long b = wk[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) b = wk[w] > b ? wk[w] : b;
        partial[blockIdx.x] = b;
    }
}

// One wave: reduces the partial keys, stores the token, appends it to the sequence, advances the position
// and the count (all in device memory, so that a captured step needs no host value).
__global__ __launch_bounds__(64) void greedy_final_kernel(const unsigned long long* __restrict__ partial,
                                                         long long* __restrict__ token, long long* __restrict__ seq,
                                                         const uint32_t seq_capacity, long long* __restrict__ count,
                                                         long long* __restrict__ pos) {
    unsigned long long best = 0ull;
    for (uint32_t i = threadIdx.x; i < (uint32_t)kPickBlocks; i += 64u) best = partial[i] > best ? partial[i] : best;
    best = wave_max_u64(best);
    if (threadIdx.x == 0) {
        const long long idx = (long long)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
        token[0] = idx;
        if (seq != nullptr && count != nullptr) {
            const long long c = count[0];
            if (c >= 0 && c < (long long)seq_capacity) seq[c] = idx;
            count[0] = c + 1;
        }
        if (pos != nullptr) pos[0] += 1;
    }
}

hipError_t launch_rope_cache(int dt, const RopeCacheParams& p, hipStream_t s) {
    const uint32_t threads = (p.n_head + p.n_kv) * (p.head_dim / 2) + p.n_kv * p.head_dim;
    const dim3 grid((threads + 255) / 256), block(256);
    if (dt == kFP16) hipLaunchKernelGGL((rope_cache_kernel<kFP16>), grid, block, 0, s, p);
    else if (dt == kBF16) hipLaunchKernelGGL((rope_cache_kernel<kBF16>), grid, block, 0, s, p);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

size_t decode_attention_lds_bytes(uint32_t head_dim) {
    const size_t ng = 16 * (64 / (head_dim / 8));
    return ng * (head_dim + 3) * sizeof(float);
}

hipError_t launch_decode_attention(int dt, const AttentionParams& p, hipStream_t s) {
    const dim3 grid(p.n_head * p.nsplit), block(1024), mgrid(p.n_head);
    const size_t lds = decode_attention_lds_bytes(p.head_dim);
    const bool merge = p.nsplit > 1 && p.counters == nullptr;
    if (dt == kFP16 && p.head_dim == 128) {
        hipLaunchKernelGGL((decode_attention_kernel<kFP16, 128>), grid, block, lds, s, p);
        if (merge) hipLaunchKernelGGL((decode_attention_merge_kernel<kFP16, 128>), mgrid, dim3(128), 0, s, p);
    } else if (dt == kFP16 && p.head_dim == 64) {
        hipLaunchKernelGGL((decode_attention_kernel<kFP16, 64>), grid, block, lds, s, p);
        if (merge) hipLaunchKernelGGL((decode_attention_merge_kernel<kFP16, 64>), mgrid, dim3(64), 0, s, p);
    } else if (dt == kBF16 && p.head_dim == 128) {
        hipLaunchKernelGGL((decode_attention_kernel<kBF16, 128>), grid, block, lds, s, p);
        if (merge) hipLaunchKernelGGL((decode_attention_merge_kernel<kBF16, 128>), mgrid, dim3(128), 0, s, p);
    } else if (dt == kBF16 && p.head_dim == 64) {
        hipLaunchKernelGGL((decode_attention_kernel<kBF16, 64>), grid, block, lds, s, p);
        if (merge) hipLaunchKernelGGL((decode_attention_merge_kernel<kBF16, 64>), mgrid, dim3(64), 0, s, p);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_silu_mul(int dt, const void* gate_up, void* out, uint32_t n, hipStream_t s) {
    const dim3 grid((n + 255) / 256), block(256);
    if (dt == kFP16) hipLaunchKernelGGL((silu_mul_kernel<kFP16>), grid, block, 0, s, gate_up, out, n);
    else if (dt == kBF16) hipLaunchKernelGGL((silu_mul_kernel<kBF16>), grid, block, 0, s, gate_up, out, n);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

size_t greedy_pick_workspace_bytes() { return (size_t)kPickBlocks * sizeof(unsigned long long); }

hipError_t launch_greedy_pick(int dt, const void* logits, uint32_t n, void* workspace, float* copy_out, long long* token,
                              long long* seq, uint32_t seq_capacity, long long* count, long long* pos, hipStream_t s) {
    unsigned long long* partial = (unsigned long long*)workspace;
    if (dt == kFP16) hipLaunchKernelGGL((greedy_partial_kernel<kFP16>), dim3(kPickBlocks), dim3(256), 0, s, logits, n, partial, copy_out);
    else if (dt == kBF16) hipLaunchKernelGGL((greedy_partial_kernel<kBF16>), dim3(kPickBlocks), dim3(256), 0, s, logits, n, partial, copy_out);
    else if (dt == kFP32) hipLaunchKernelGGL((greedy_partial_kernel<kFP32>), dim3(kPickBlocks), dim3(256), 0, s, logits, n, partial, copy_out);
    else return hipErrorInvalidValue;
    hipLaunchKernelGGL(greedy_final_kernel, dim3(1), dim3(64), 0, s, partial, token, seq, seq_capacity, count, pos);
    return hipGetLastError();
}

}  // namespace decdec
