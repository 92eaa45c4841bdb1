// DEC role: bucket top-k channel selection + zero-copy fetch of the selected 4-bit residual rows +
// residual GEMV + atomic merge into the output.  One workgroup of 16 wave64 (8 or 4 in the small forms) plays
// this role; it is used by the standalone DEC kernels and, next to a base-GEMV role, by the fused
// single-launch kernels.
//
// Work decomposition (differs from the reference's column partition + grid barrier on purpose):
// a workgroup owns a set of 1024-channel chunks (chunk group) and a range of column segments
// (segment group).  It selects the channels of its own chunks itself -- selection needs only the
// activation vector, so no grid-wide barrier and no second launch -- and then fetches the selected
// residual rows restricted to its column segments.  A segment is 64 consecutive u32 words of a
// residual row (256 bytes, one coalesced wave-wide load).  Each wave requests two, four or eight rows per round
// (the launch's choice): the host link's latency, not ALU work, bounds the fetch, and the link serves only so many
// bytes per round trip.  The code is kept small on purpose
// (rolled loops, one code path): a DEC workgroup runs its instructions once, so every instruction
// cache line it touches is a cold miss on the critical path.
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
    const void* scales;         // scale of output n at index n (the library's own copy), device memory, dtype of the activations
    const void* x;              // activations [K]
    int32_t* sel_rows;          // context scratch: selected channel indices
    void* sel_acts;             // context scratch: selected activations
    void* out;                  // output [N], accumulated atomically
    float floors[kBuckets];     // bucket floors (values exactly representable in the activation dtype)
    uint32_t monotone;          // floors are finite and non-increasing (enables the fast selection path)
    uint32_t K, N, M;           // M = N / 8 words per residual row
    uint32_t num_chunks, k_chunk, k_total;
    uint32_t cg, sg;            // chunk groups x segment groups = number of DEC workgroups
    uint32_t nseg;              // column segments (64 u32 words each) per row
    uint32_t segs_per_block;    // ceil(nseg / sg)
    uint32_t slots_per_block;   // capacity of the per-workgroup row list
    uint32_t fused_select;      // 1: select in-kernel; 0: row indices supplied in sel_rows
    uint32_t rows_in_flight;    // residual rows a wave requests at a time: 2, 4 or 8 (dec_fetch_rows)
    unsigned long long* trace;  // optional [workgroup][8] cycle stamps of the phases (diagnostics), or null
};

__device__ __forceinline__ void dec_stamp(const DecParams& p, uint32_t bid, int k) {
    if (p.trace != nullptr && threadIdx.x == 0) p.trace[(size_t)bid * 8 + k] = __builtin_readcyclecounter();
}

constexpr int kDecThreads = 1024;                            // largest DEC workgroup
constexpr int kDecWaves = kDecThreads / kWave;
constexpr int kMinDecWaves = 4;                              // smallest workgroup: two teams of two waves
constexpr int kMergeTasks = kDecWaves * 256 / kDecThreads;   // output pairs per thread and segment batch

__host__ __device__ inline size_t dec_team_lds_bytes(uint32_t nwaves);
__host__ __device__ inline size_t dec_lds_bytes(uint32_t slots, uint32_t nwaves = kDecWaves) {
    // row list (index + activation) + counters/prefix of the general selection + the buffer shared by the
    // cross-wave reduction ([nwaves][8][64] floats) and the selection teams
    const size_t red = (size_t)nwaves * 8 * kWave * 4, teams = dec_team_lds_bytes(nwaves);
    return (size_t)slots * 8 + 2 * 512 * 4 + (red > teams ? red : teams);
}

// The 32 bucket floors live in one vector register (lane i and lane i + 32 hold floor[i], read from the kernel
// argument segment once per workgroup) and are broadcast with v_readlane where they are used: as 32 scalar kernel
// arguments they would be held in scalar registers for the whole kernel.
__device__ __forceinline__ float dec_floor(float myfloor, int i) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(myfloor), i));
}

// Bucket of |x| = ca when the floors do not increase: the number of floors strictly above ca, at most 31 (the callers'
// candidates lie at or above some floor).  "Floor i is above ca" then holds for a prefix of the floors, so five
// lane-indexed reads of the floor register (ds_bpermute: a cross-lane gather, no memory) find its length; a scan
// over the floors with v_readlane is six times as many dependent steps for the single wave that ranks.
// Needs every lane of the wave active.
__device__ __forceinline__ uint32_t dec_bucket_of(float myfloor, float ca) {
    uint32_t b = 0;
#pragma unroll
    for (uint32_t step = 16u; step >= 1u; step >>= 1) {
        const float f = __uint_as_float((uint32_t)__builtin_amdgcn_ds_bpermute((int)((b + step - 1u) << 2),
                                                                              (int)__float_as_uint(myfloor)));
        b += (ca < f) ? step : 0u;
    }
    return b;
}

// ---- selection of one chunk ------------------------------------------------------------------
// General path: every wave tests its 64 channels against all 32 buckets (one ballot per bucket),
// per-(bucket, wave) counts are prefix-summed, and each member computes its position.  Exact for any
// floors (non-monotone floors can put a channel into several buckets, as in the reference kernel).
template <int DT, int NW>
__device__ __forceinline__ void dec_select_general(const DecParams& p, uint32_t c, uint32_t t_local, uint32_t kc,
                                                int32_t* lrows, float* lacts, uint32_t* cnt, uint32_t* pre,
                                                bool write_global, const float myfloor) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    constexpr uint32_t nw = NW;
    const uint32_t lo = c * kChunk;
    const uint32_t len = (p.K - lo) < (uint32_t)kChunk ? (p.K - lo) : (uint32_t)kChunk;
    // The chunk is 16 groups of 64 channels; wave w takes groups w, w + nw, ... (one group per wave in a
    // 1024-thread workgroup, four in a 256-thread one).
    // Nothing is kept between the counting and the placing step but the counts: a group's activations are
    // read again and its memberships recomputed (this path is rare; registers held here would be charged to
    // every launch of the kernels that contain it).
    const uint32_t ngroups = (uint32_t)(kChunk / kWave);
#pragma unroll 1
    for (uint32_t vw = wave; vw < ngroups; vw += nw) {
        const uint32_t ch = vw * kWave + lane;
        const bool in = ch < len;
        const float xv = in ? E::load(p.x, lo + ch) : 0.f;
        const float a = in ? __builtin_fabsf(xv) : __builtin_nanf("");   // NaN is a member of no bucket
        float ce = __builtin_inff();
#pragma unroll 1
        for (int i = 0; i < kBuckets; ++i) {
            const float fl = dec_floor(myfloor, i);
            const bool bit = (a >= fl) && (a < ce);
            ce = fl;
            const unsigned long long m = __ballot(bit);
            if (lane == 0) cnt[i * 16 + vw] = (uint32_t)__popcll(m);
        }
    }
    __syncthreads();
    if (wave == 0) {   // exclusive prefix over the 512 (bucket-major, group-minor) counts
        uint32_t v[8], sum = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) { v[q] = cnt[lane * 8 + q]; sum += v[q]; }
        uint32_t incl = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = __shfl_up(incl, off, 64);
            if (lane >= (uint32_t)off) incl += o;
        }
        uint32_t run = incl - sum;
#pragma unroll
        for (int q = 0; q < 8; ++q) { pre[lane * 8 + q] = run; run += v[q]; }
    }
    __syncthreads();
#pragma unroll 1
    for (uint32_t vw = wave; vw < ngroups; vw += nw) {
        const uint32_t ch = vw * kWave + lane;
        const bool in = ch < len;
        const float xv = in ? E::load(p.x, lo + ch) : 0.f;
        const float a = in ? __builtin_fabsf(xv) : __builtin_nanf("");
        float ce = __builtin_inff();
#pragma unroll 1
        for (int i = 0; i < kBuckets; ++i) {
            if (pre[i * 16] >= kc) break;                            // uniform: later buckets start even later
            const float fl = dec_floor(myfloor, i);
            const bool bit = (a >= fl) && (a < ce);
            ce = fl;
            const unsigned long long m = __ballot(bit);
            if (bit) {
                const uint32_t pos = pre[i * 16 + vw] + ballot_rank(m);
                if (pos < kc) {
                    const uint32_t slot = t_local * p.k_chunk + pos;
                    lrows[slot] = (int32_t)(lo + ch);
                    lacts[slot] = xv;
                    if (write_global) {
                        p.sel_rows[(size_t)c * p.k_chunk + pos] = (int32_t)(lo + ch);
                        E::store(p.sel_acts, (size_t)c * p.k_chunk + pos, xv);
                    }
                }
            }
        }
    }
}

// Inclusive prefix sum over the 64 lanes of a wave (DPP row shifts and row broadcasts, zero fill).
__device__ __forceinline__ uint32_t wave_scan(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xF, 0xF, true);   // row_shr 1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xF, 0xF, true);   // row_shr 2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xF, 0xF, true);   // row_shr 4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xF, 0xF, true);   // row_shr 8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xA, 0xF, true);   // row_bcast 15 -> rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xC, 0xF, true);   // row_bcast 31 -> rows 2, 3
    return v;
}

// Fast path (floors finite and non-increasing, checked on the host).  Then bucket(|x|) is the number of
// floors above |x|, buckets 0..T tile [floor_T, +inf), and the selection is: every channel of the buckets before
// the cut bucket b* (the first bucket at which the running count reaches kc), then the first channels of b* in
// channel order.  kAttempts cut-offs T are tried at once (a compare and a ballot each); the first whose range holds
// at least kc channels is the winning window.
//   * At most 128 channels in the window (64 in the usual case): they are compacted in channel order and one wave
//     (two beyond 64) ranks them by (bucket, channel) with ballots.
//   * More (activations weaker than the calibration set put the cut where buckets are crowded): the window spans two
//     buckets beyond the previous cut-off; one more count at the floor between them tells which of the two is b*.
//     The channels above b* -- fewer than kc, so at most 127 -- are compacted and ranked as before; the members of
//     b* need no ranking at all: their positions follow the ranked ones in channel order, so each writes its own
//     output slot from a prefix count, however many there are.
// No sequential walk over buckets, and no limit on the size of a bucket.
//
// A wave issues one instruction every four cycles whatever its kind, so a chunk is scanned by a TEAM of
// waves on different SIMDs.  The teams of a workgroup (four in a 1024-thread workgroup) take different chunks of
// the workgroup's chunk list at the same time: a workgroup that owns up to four chunks selects them in the time of
// one, which is what lets the launch plan give a workgroup several chunks (few chunk groups = few atomic adds,
// i.e. roundings, per output) at no cost in latency.  All teams run through the same workgroup barriers; what a
// team does between them depends on its own chunk only.  A chunk the fast path cannot take (non-monotone floors,
// k_chunk > 128, NaN or infinite activations that leave fewer than kc countable channels, more than 128 channels in
// the buckets down to the calibrated threshold) is afterwards selected by the whole workgroup on the general path.
constexpr int kAttempts = 9;
constexpr uint32_t kRankMax = 128;         // candidates a team of a 16-wave workgroup ranks (64 per ranking wave)
// Team geometry by workgroup size.  A 16-wave workgroup has four teams of four waves (four channels per lane);
// smaller workgroups have teams of two waves (eight channels per lane): an 8-wave workgroup then still selects
// four chunks at a time, a 4-wave one two.
template <int NW> struct DecTeam {
    static constexpr int kWaves = NW >= 16 ? 4 : 2;                 // waves of a team
    static constexpr int kThreads = kWaves * kWave;
    static constexpr int kTeams = NW / kWaves;
    static constexpr int kLaneChannels = kChunk / kThreads;         // 4 or 8
    // Windows of more than 64 channels are ranked by two waves, and crowded ones split, only in the 16-wave
    // workgroups.  The smaller ones share their kernel, and its register allocation, with a GEMV role that runs
    // eight waves per SIMD (every addition to this role made that role slower); they are chosen while DEC is the
    // shorter role, and leave the rare window of more than 64 channels to the general path.
    static constexpr bool kSplit = NW >= 16;
    // Two ranking waves (windows of up to 128 channels) also in the 8-wave form: a window of 65 .. 128 channels is
    // what a dense body two buckets below a sparse tail gives at small k_chunk, and the general path, run beside
    // seven GEMV waves per SIMD, costs such a chunk 9 us (14336 -> 4096, k_chunk 6: 22.7 us instead of 13.7).
    static constexpr uint32_t kRank = NW >= 8 ? kRankMax : 64u;     // candidates a team ranks (64 per ranking wave)
    // words of a team's area: [kAttempts][4] window counts, [4] counts at the floor inside the window,
    // [kRankMax] candidate channels, [kRankMax] candidate activations, [4] header (state, candidates, -, -)
    static constexpr int kSplitWord = 4 * kAttempts;
    static constexpr int kKeyWord = kSplitWord + 4;
    static constexpr int kHdrWord = kKeyWord + 2 * (int)kRankMax;
    static constexpr size_t kBytes = (size_t)(kHdrWord + 4) * 4;
    static_assert(kBytes % 16 == 0 && (kKeyWord * 4) % 16 == 0 && (kHdrWord * 4) % 16 == 0, "team area alignment");
};
__host__ __device__ inline size_t dec_team_lds_bytes(uint32_t nwaves) {
    return nwaves >= 16 ? (size_t)DecTeam<16>::kTeams * DecTeam<16>::kBytes
                        : (nwaves >= 8 ? (size_t)DecTeam<8>::kTeams * DecTeam<8>::kBytes
                                       : (size_t)DecTeam<4>::kTeams * DecTeam<4>::kBytes);
}
enum : uint32_t { kTeamGeneral = 0u, kTeamFast = 1u, kTeamIdle = 2u, kTeamSplit = 3u };

// The cut-offs tried: buckets 15, 17, ..., 31.  floor[15] = thresholds[k - 1]: with activations like the calibration
// set about kc channels lie above it and one bucket further down adds about kc / 2 more, so steps of two buckets keep
// the winning window at or below 64 channels (one ranking wave) there; a cut-off at every bucket cost every launch a microsecond of
// scanning.  floor[31] = 0: the last window always holds every finite channel.
__device__ __forceinline__ constexpr uint32_t dec_attempt_bucket(uint32_t u) { return 15u + 2u * u; }

// The activations a scanning lane owns: unconditional loads from clamped indices (a predicated load
// costs a branch and a full wait each).
// Storage bits only: converting at once would make the lane wait for the loads where they are issued.
template <int DT, int C>
__device__ __forceinline__ void dec_load_x(const DecParams& p, uint32_t lo, uint32_t len, uint32_t ch0, uint32_t (&xr)[C]) {
#pragma unroll
    for (int s = 0; s < C; ++s) xr[s] = Elem<DT>::load_raw(p.x, lo + ((ch0 + s < len) ? ch0 + s : len - 1u));
}

__device__ __forceinline__ uint32_t dec_chunk_len(const DecParams& p, uint32_t c) {
    const uint32_t lo = c * kChunk;
    return (p.K - lo) < (uint32_t)kChunk ? (p.K - lo) : (uint32_t)kChunk;
}

// What a team's window counts say (the same in every lane of every wave of the team).
struct DecWindow {
    uint32_t state;        // kTeamFast, kTeamSplit or kTeamGeneral
    uint32_t us;           // winning attempt
    uint32_t total;        // channels in the winning window (all buckets down to its cut-off)
    uint32_t before;       // ... of them in the team's waves before this one
    uint32_t prev_total;   // channels above the previous cut-off (0 for the first attempt): fewer than kc
    uint32_t prev_before;
};
template <int NW>
__device__ __forceinline__ DecWindow dec_read_window(const uint32_t* wc, uint32_t lane, uint32_t tw, uint32_t kc) {
    constexpr uint32_t kSelWaves = DecTeam<NW>::kWaves;
    // lane u < kAttempts looks at attempt u: total and the count of the team's waves before this one
    const u32x4 w4 = *(const u32x4*)(wc + 4u * (lane < (uint32_t)kAttempts ? lane : 0u));
    const uint32_t tot = kSelWaves == 4u ? w4[0] + w4[1] + w4[2] + w4[3] : w4[0] + w4[1];
    const uint32_t bef = (tw > 0 ? w4[0] : 0u) + (tw > 1 ? w4[1] : 0u) + (tw > 2 ? w4[2] : 0u);
    const unsigned long long okm = __ballot(lane < (uint32_t)kAttempts && tot >= kc);
    DecWindow w = {kTeamGeneral, 0u, 0u, 0u, 0u, 0u};
    if (okm == 0ull || kc > DecTeam<NW>::kRank) return w;
    w.us = (uint32_t)__builtin_ctzll(okm);                                          // first qualifying attempt
    w.total = (uint32_t)__builtin_amdgcn_readlane((int)tot, (int)w.us);
    w.before = (uint32_t)__builtin_amdgcn_readlane((int)bef, (int)w.us);
    if (w.us > 0u) {
        w.prev_total = (uint32_t)__builtin_amdgcn_readlane((int)tot, (int)w.us - 1);
        w.prev_before = (uint32_t)__builtin_amdgcn_readlane((int)bef, (int)w.us - 1);
    }
    w.state = w.total <= DecTeam<NW>::kRank ? kTeamFast : ((DecTeam<NW>::kSplit && w.us > 0u) ? kTeamSplit : kTeamGeneral);
    return w;
}

// One round of selection: team j of the workgroup takes the workgroup's local chunk t0 + j (global chunk
// cgid + (t0 + j) * cg) if there is one.  `xpre` holds the raw activations of the team's chunk when
// have_xpre (requested when the workgroup started).  Called by all threads of the workgroup.
template <int DT, int NW>
__device__ __forceinline__ void dec_select_round(const DecParams& p, uint32_t cgid, uint32_t t0, uint32_t nlocal,
                                                 int32_t* lrows, float* lacts, uint32_t* cnt,
                                                 uint32_t* pre, float* red, bool write_global,
                                                 bool have_xpre, const uint32_t (&xpre)[DecTeam<NW>::kLaneChannels],
                                                 const float myfloor) {
    using E = Elem<DT>;
    using T = DecTeam<NW>;
    constexpr uint32_t kTeams = T::kTeams, kSelWaves = T::kWaves, kTeamThreads = T::kThreads;
    constexpr int C = T::kLaneChannels;
    constexpr size_t kTeamBytes = T::kBytes;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t team = wave / kSelWaves, tw = wave % kSelWaves;
    const uint32_t ttid = tid & (kTeamThreads - 1u);
    const uint32_t t_local = t0 + team;
    const uint32_t c = cgid + t_local * p.cg;
    const bool has_chunk = t_local < nlocal;                // uniform per wave
    const uint32_t lo = has_chunk ? c * kChunk : 0u;
    const uint32_t len = has_chunk ? dec_chunk_len(p, c) : 0u;
    const uint32_t kc = p.k_chunk * len / kChunk;
    const bool active = has_chunk && kc > 0u;

    unsigned char* tbase = (unsigned char*)red + (size_t)team * kTeamBytes;
    uint32_t* wc = (uint32_t*)tbase;                       // [kAttempts][4] window counts per team wave
    uint32_t* split = wc + T::kSplitWord;                  // [4] counts at the floor inside the winning window
    uint32_t* key = wc + T::kKeyWord;                      // [kRankMax] candidate channels (chunk-relative)
    float* cx = (float*)(key + kRankMax);                  // [kRankMax] their activations
    uint32_t* hdr = wc + T::kHdrWord;                      // state, candidates to rank
    const bool scanner = active && p.monotone;             // uniform per wave

    // ---- the team scans its chunk: lane l of team wave w owns channels C (64 w + l) .. + C - 1
    // |x| of the lane's channel s as the selection sees it: NaN, inf and channels past the end are members of no
    // bucket.  Recomputed after the barriers instead of kept: registers held across them are charged to every
    // kernel that contains this role.
    float xv[C];
    const uint32_t ch0 = (uint32_t)C * ttid;
    auto mag = [&](int s) {
        const float v = __builtin_fabsf(xv[s]);
        return (ch0 + (uint32_t)s < len && v < __builtin_inff()) ? v : -__builtin_inff();
    };
    // selected channel at canonical position pos of the team's chunk
    auto emit = [&](uint32_t pos, uint32_t chl, float xs) {
        const uint32_t ch = lo + chl;
        const uint32_t slot = t_local * p.k_chunk + pos;
        lrows[slot] = (int32_t)ch;
        lacts[slot] = xs;
        if (write_global) {
            p.sel_rows[(size_t)c * p.k_chunk + pos] = (int32_t)ch;
            E::store(p.sel_acts, (size_t)c * p.k_chunk + pos, xs);
        }
    };
    // The candidates in key / cx (n of them, in channel order, n <= 128) ranked by (bucket, channel) with ballots only:
    // a candidate's position is the number of candidates in lower buckets plus the number of earlier candidates in its
    // own bucket.  A wave places the 64 candidates of half `half` (lane l holds candidate 64 half + l) and looks at
    // both halves when there are more than 64; the first min(n, kc) positions are emitted.  Called by whole waves.
    auto rank_candidates = [&](uint32_t n, uint32_t half) {
        const uint32_t nh = (T::kRank > 64u && n > 64u) ? 2u : 1u;      // halves in use (uniform)
        bool valid[2] = {false, false};
        float xs[2] = {0.f, 0.f};
        uint32_t chl[2] = {0u, 0u}, bkt[2] = {0u, 0u};
#pragma unroll
        for (uint32_t h = 0; h < 2u; ++h) {
            if (h < nh) {
                const uint32_t i = 64u * h + lane;
                valid[h] = i < n;
                xs[h] = valid[h] ? cx[i] : 0.f;
                chl[h] = valid[h] ? key[i] : 0u;
                bkt[h] = dec_bucket_of(myfloor, __builtin_fabsf(xs[h]));
            }
        }
        const uint32_t mybkt = half ? bkt[1] : bkt[0];
        uint32_t pos = 0;
#pragma unroll
        for (uint32_t h = 0; h < 2u; ++h) {
            if (h < nh) {
                unsigned long long eq = __ballot(valid[h]);             // candidates of half h in my bucket
                unsigned long long lt = 0ull;                           // ... in a lower bucket
#pragma unroll
                for (int k = 4; k >= 0; --k) {
                    const bool mybit = ((mybkt >> k) & 1u) != 0u;
                    const unsigned long long bk = __ballot(valid[h] && ((bkt[h] >> k) & 1u) != 0u);
                    lt |= mybit ? (eq & ~bk) : 0ull;
                    eq &= mybit ? bk : ~bk;
                }
                pos += (uint32_t)__popcll(lt);
                // same bucket: all of an earlier half, the earlier lanes of my own half, none of a later half
                pos += h < half ? (uint32_t)__popcll(eq) : (h == half ? ballot_rank(eq) : 0u);
            }
        }
        const bool myvalid = half ? valid[1] : valid[0];
        if (myvalid && pos < kc) emit(pos, half ? chl[1] : chl[0], half ? xs[1] : xs[0]);
    };
    // Team j ranks the first 64 candidates on its wave j and the rest on the next wave: waves w and w + 4 of a
    // workgroup share a SIMD, so the ranking waves of the four teams sit on different SIMDs (four ranking waves on one
    // SIMD took 2.2x as long).
    auto rank_on_team = [&](uint32_t n) {
        const uint32_t w0 = team & (kSelWaves - 1u), w1 = (team + 1u) & (kSelWaves - 1u);
        if (tw == w0) rank_candidates(n, 0u);
        else if (T::kRank > 64u && tw == w1 && n > 64u) rank_candidates(n, 1u);
    };
    if (scanner) {
        uint32_t xr[C];
        if (have_xpre) {                                   // uniform: requested when the workgroup started
#pragma unroll
            for (int s = 0; s < C; ++s) xr[s] = xpre[s];
        } else {
            dec_load_x<DT, C>(p, lo, len, ch0, xr);
        }
#pragma unroll
        for (int s = 0; s < C; ++s) asm volatile("" : "+v"(xr[s]));             // first use: here
#pragma unroll
        for (int s = 0; s < C; ++s) xv[s] = E::from_raw(xr[s]);
        dec_stamp(p, blockIdx.x, 5);
        uint32_t n[kAttempts];
        {
            float a[C];
#pragma unroll
            for (int s = 0; s < C; ++s) a[s] = mag(s);
#pragma unroll
            for (int u = 0; u < kAttempts; ++u) {
                const float f = dec_floor(myfloor, (int)dec_attempt_bucket(u));
                n[u] = 0;
#pragma unroll
                for (int s = 0; s < C; ++s) n[u] += (uint32_t)__popcll(__ballot(a[s] >= f));
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int u = 0; u < kAttempts; ++u) wc[u * 4 + tw] = n[u];
        }
    }
    __syncthreads();
    if (scanner) {
        const DecWindow w = dec_read_window<NW>(wc, lane, tw, kc);
        if (w.state == kTeamFast) {                        // compaction of the window in channel order
            const float f = dec_floor(myfloor, (int)dec_attempt_bucket(w.us));
            uint32_t cs[C], mine = 0;
#pragma unroll
            for (int s = 0; s < C; ++s) { cs[s] = (mag(s) >= f) ? 1u : 0u; mine += cs[s]; }
            uint32_t idx = w.before + wave_scan(mine) - mine;
#pragma unroll
            for (int s = 0; s < C; ++s) {
                if (cs[s]) { key[idx] = ch0 + s; cx[idx] = xv[s]; ++idx; }
            }
            if (ttid == 0) hdr[1] = w.total;
        } else if (w.state == kTeamSplit) {                // channels at or above the floor inside the window
            const float f = dec_floor(myfloor, (int)dec_attempt_bucket(w.us) - 1);
            uint32_t nu = 0;
#pragma unroll
            for (int s = 0; s < C; ++s) nu += (uint32_t)__popcll(__ballot(mag(s) >= f));
            if (lane == 0) split[tw] = nu;
        }
        if (ttid == 0) hdr[0] = w.state;
    } else if (ttid == 0) {
        hdr[0] = active ? kTeamGeneral : kTeamIdle;
        hdr[1] = 0u;
    }
    __syncthreads();
    // what the teams found (the same view in every thread: the branches below that hold barriers are uniform)
    bool any_split = false, any_general = false;
#pragma unroll
    for (uint32_t j = 0; j < kTeams; ++j) {
        const uint32_t st = *(const uint32_t*)((const unsigned char*)red + (size_t)j * kTeamBytes + (size_t)T::kHdrWord * 4);
        any_general = any_general || st == kTeamGeneral;
        any_split = any_split || st == kTeamSplit;
    }
    const u32x2 hd = *(const u32x2*)hdr;                    // state, candidates
    dec_stamp(p, blockIdx.x, 6);
    if (hd[0] == kTeamFast) rank_on_team(hd[1]);
    if (T::kSplit && any_split) {                          // uniform for the workgroup
        if (hd[0] == kTeamSplit) {                         // uniform per team
            const DecWindow w = dec_read_window<NW>(wc, lane, tw, kc);
            const u32x4 s4 = *(const u32x4*)split;
            const uint32_t stot = kSelWaves == 4u ? s4[0] + s4[1] + s4[2] + s4[3] : s4[0] + s4[1];
            const uint32_t sbef = (tw > 0 ? s4[0] : 0u) + (tw > 1 ? s4[1] : 0u) + (tw > 2 ? s4[2] : 0u);
            // the cut bucket is the upper one of the window's two if the count reaches kc there, else the lower one
            const bool upper = stot >= kc;
            const uint32_t bb = dec_attempt_bucket(w.us) - (upper ? 1u : 0u);                       // cut bucket
            const float fb = dec_floor(myfloor, (int)bb), fs = dec_floor(myfloor, (int)bb - 1);
            const uint32_t n_sure = upper ? w.prev_total : stot;                                   // < kc
            const uint32_t sure_before = upper ? w.prev_before : sbef;
            const uint32_t band_before = (upper ? sbef : w.before) - sure_before;
            uint32_t cs[C], cb[C], ms = 0, mb = 0;
#pragma unroll
            for (int s = 0; s < C; ++s) {
                const float a = mag(s);
                cs[s] = (a >= fs) ? 1u : 0u;
                cb[s] = (a >= fb && !(a >= fs)) ? 1u : 0u;
                ms += cs[s]; mb += cb[s];
            }
            uint32_t is = sure_before + wave_scan(ms) - ms;
            uint32_t ib = n_sure + band_before + wave_scan(mb) - mb;
#pragma unroll
            for (int s = 0; s < C; ++s) {
                if (cs[s]) { key[is] = ch0 + s; cx[is] = xv[s]; ++is; }
                if (cb[s]) { if (ib < kc) emit(ib, ch0 + s, xv[s]); ++ib; }
            }
            if (ttid == 0) hdr[1] = n_sure;
        }
        __syncthreads();
        if (hd[0] == kTeamSplit) rank_on_team(hdr[1]);
    }
    dec_stamp(p, blockIdx.x, 7);
    if (any_general) {                                     // uniform for the workgroup; rare
#pragma unroll 1
        for (uint32_t j = 0; j < kTeams; ++j) {
            const uint32_t st = *(const uint32_t*)((const unsigned char*)red + (size_t)j * kTeamBytes + (size_t)T::kHdrWord * 4);
            if (st != kTeamGeneral) continue;              // uniform
            const uint32_t tj = t0 + j, cj = cgid + tj * p.cg;
            const uint32_t kcj = p.k_chunk * dec_chunk_len(p, cj) / kChunk;
            __syncthreads();                               // cnt / pre of the previous general selection no longer read
            dec_select_general<DT, NW>(p, cj, tj, kcj, lrows, lacts, cnt, pre, write_global, myfloor);
        }
    }
}

// ---- fetch + dequantise + accumulate ------------------------------------------------------------
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

// The rows rl, rl + RL, ... of the workgroup's list for one wave's column of the residual, U requests at a time.  U is
// the launch's choice (DecParams::rows_in_flight): the host link serves about 140 KB per round trip, and a launch
// that asks for several times that makes every request wait longer (Llama-3-8B token at k_chunk 32: 2897 us with eight
// rows per wave and request round, 2801 with two, 2853 with one; at k_chunk 8, where a wave has few rows, four are best).
template <int U>
__device__ __forceinline__ void dec_fetch_rows(const uint32_t* base, uint32_t M, uint32_t rl, uint32_t RL, uint32_t nslots,
                                               const int32_t* lrows, const float* lacts, float (&acc)[8], float& act_sum) {
#pragma unroll 1
    for (uint32_t r = rl; r < nslots; r += RL * U) {
        uint32_t data[U];
        float act[U];
        int32_t row[U];
        // all list entries first (one LDS round trip), then the requests; entries are the same in
        // every lane, so they live in scalar registers
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t rr = r + (uint32_t)u * RL;
            const bool valid = rr < nslots;
            const uint32_t ri = valid ? rr : 0u;
            const int32_t rw = lrows[ri];
            const float a = lacts[ri];
            row[u] = __builtin_amdgcn_readfirstlane(valid ? rw : -1);
            act[u] = __uint_as_float((uint32_t)__builtin_amdgcn_readfirstlane((int)__float_as_uint(a)));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (row[u] >= 0) data[u] = base[(size_t)row[u] * M];
            else { data[u] = 0x88888888u; act[u] = 0.f; }                    // nibble 8 == value 0
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            act_sum += act[u];
            dec_accumulate_word(data[u], act[u], acc);
        }
    }
}

template <int DT, int NW>
__device__ __forceinline__ void dec_fetch(const DecParams& p, uint32_t bid, uint32_t sgid, uint32_t nslots,
                                          const int32_t* lrows, const float* lacts, float* red) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    constexpr uint32_t nw = NW, nt = NW * kWave;
    const uint32_t seg_lo = sgid * p.segs_per_block;
    const uint32_t seg_hi = (seg_lo + p.segs_per_block) < p.nseg ? (seg_lo + p.segs_per_block) : p.nseg;

#pragma unroll 1
    for (uint32_t sb0 = seg_lo; sb0 < seg_hi; sb0 += nw) {
        const uint32_t SB = (seg_hi - sb0) < nw ? (seg_hi - sb0) : nw;
        const uint32_t RL = nw / SB;                    // waves sharing one segment
        const uint32_t ls = wave % SB, rl = wave / SB;
        const uint32_t w0 = (sb0 + ls) * kWave + lane;  // u32 column of the residual row
        const bool col_ok = (rl < RL) && (w0 < p.M);

        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.f;
        float act_sum = 0.f;
        // the scales this thread needs in the merge step, requested before the row fetch so that their
        // latency hides behind it: merge task t -> word (t & 63) of segment t >> 8, output pair (t >> 6) & 3
        // (storage bits only: a conversion here would make the thread wait for them before the first row)
        uint32_t sc0[kMergeTasks], sc1[kMergeTasks];
#pragma unroll
        for (int q = 0; q < kMergeTasks; ++q) {
            const uint32_t t = tid + (uint32_t)q * nt;
            const uint32_t m = (sb0 + (t >> 8)) * kWave + (t & 63u), jp = (t >> 6) & 3u;
            const uint32_t mc = ((t < SB * 256u) && (m < p.M)) ? m : 0u;     // unconditional loads, clamped index
            E::load_raw2(p.scales, (size_t)8 * mc + 2 * jp, sc0[q], sc1[q]);
        }

        if (col_ok) {
            const uint32_t* base = p.residual + w0;
            if (p.rows_in_flight <= 2u) dec_fetch_rows<2>(base, p.M, rl, RL, nslots, lrows, lacts, acc, act_sum);
            else if (p.rows_in_flight <= 4u) dec_fetch_rows<4>(base, p.M, rl, RL, nslots, lrows, lacts, acc, act_sum);
            else dec_fetch_rows<8>(base, p.M, rl, RL, nslots, lrows, lacts, acc, act_sum);
        }
        dec_stamp(p, bid, 2);
        // cross-wave reduction through LDS (plain stores; LDS float atomics are slow), then one
        // atomic add per output pair for the whole workgroup
#pragma unroll
        for (int j = 0; j < 8; ++j)
            red[(wave * 8 + j) * kWave + lane] = col_ok ? (acc[j] - 8.f * act_sum) : 0.f;   // nibble = q + 8
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kMergeTasks; ++q) {
            const uint32_t t = tid + (uint32_t)q * nt;
            const uint32_t lw = t & 63u, jp = (t >> 6) & 3u, sl = t >> 8;
            const uint32_t m = (sb0 + sl) * kWave + lw;
            if (t >= SB * 256u || m >= p.M) continue;
            float v0 = 0.f, v1 = 0.f;
            for (uint32_t qq = 0; qq < RL; ++qq) {
                const uint32_t wv = qq * SB + sl;
                v0 += red[(wv * 8 + 2 * jp) * kWave + lw];
                v1 += red[(wv * 8 + 2 * jp + 1) * kWave + lw];
            }
            uint32_t r0 = sc0[q], r1 = sc1[q];
            asm volatile("" : "+v"(r0), "+v"(r1));        // first use of the scales: here, not earlier
            E::atomic_add2(p.out, (size_t)8 * m + 2 * jp, v0 * E::from_raw2_lo(r0, r1), v1 * E::from_raw2_hi(r0, r1));
        }
        dec_stamp(p, bid, 3);
        __syncthreads();                                 // red is reused by the next batch
    }
}

// ---- the role -------------------------------------------------------------------------------------
template <int DT, int NW = kDecWaves>
__device__ __forceinline__ void dec_role(const DecParams& p, uint32_t bid, unsigned char* smem) {
    using E = Elem<DT>;
    const uint32_t tid = threadIdx.x;
    const uint32_t cgid = bid / p.sg, sgid = bid % p.sg;
    int32_t* lrows = (int32_t*)smem;
    float* lacts = (float*)(lrows + p.slots_per_block);
    uint32_t* cnt = (uint32_t*)(lacts + p.slots_per_block);
    uint32_t* pre = cnt + 512;
    float* red = (float*)(pre + 512);

    dec_stamp(p, bid, 0);
    // the teams ask for the activations of their first chunks before anything else: their latency is the
    // head of the critical path
    using T = DecTeam<NW>;
    constexpr uint32_t kTeams = T::kTeams, kTeamThreads = T::kThreads;
    const uint32_t nlocal = cgid < p.num_chunks ? (p.num_chunks - cgid + p.cg - 1u) / p.cg : 0u;   // chunks cgid, cgid + cg, ...
    const float myfloor = p.floors[tid & 31u];
    uint32_t xpre[T::kLaneChannels] = {};
    const uint32_t team0 = tid / kTeamThreads;
    const bool have_xpre = p.fused_select && p.monotone;                              // uniform
    if (have_xpre && team0 < nlocal) {
        const uint32_t c = cgid + team0 * p.cg;
        dec_load_x<DT, T::kLaneChannels>(p, c * kChunk, dec_chunk_len(p, c), (uint32_t)T::kLaneChannels * (tid & (kTeamThreads - 1u)), xpre);
    }
    for (uint32_t i = tid; i < p.slots_per_block; i += (uint32_t)NW * kWave) lrows[i] = -1;
    uint32_t nslots = 0;
    if (p.fused_select) {
        for (uint32_t t0 = 0; t0 < nlocal; t0 += kTeams) {
            __syncthreads();      // list initialised; the team areas of the previous round no longer read
            dec_select_round<DT, NW>(p, cgid, t0, nlocal, lrows, lacts, cnt, pre, red, sgid == 0, have_xpre && t0 == 0, xpre, myfloor);
        }
        nslots = nlocal * p.k_chunk;
    } else {
        const uint32_t per = (p.k_total + p.cg - 1) / p.cg;
        const uint32_t lo = cgid * per;
        const uint32_t hi = (lo + per) < p.k_total ? (lo + per) : p.k_total;
        __syncthreads();
        for (uint32_t i = lo + tid; i < hi; i += (uint32_t)NW * kWave) {
            const int32_t row = p.sel_rows[i];
            const bool ok = row >= 0 && (uint32_t)row < p.K;       // out-of-range indices are ignored
            lrows[i - lo] = ok ? row : -1;
            lacts[i - lo] = ok ? E::load(p.x, (size_t)row) : 0.f;
        }
        nslots = hi > lo ? hi - lo : 0;
    }
    __syncthreads();
    dec_stamp(p, bid, 1);
    dec_fetch<DT, NW>(p, bid, sgid, nslots, lrows, lacts, red);
    dec_stamp(p, bid, 4);
}

}  // namespace decdec
