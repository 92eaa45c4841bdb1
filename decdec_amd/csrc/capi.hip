// C-ABI layer of libdecdec_hip.so: argument validation, DEC context / config objects, launch
// planning, and the two ways of running DEC next to a base GEMV (one fused launch, or the
// reference's two-stream fork/join).  Declarations and reference citations: include/decdec_hip.h.
#include <cmath>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>
#include <string>
#include <unordered_set>

#include "../../include/decdec_hip.h"
#include "launch.h"

using namespace decdec;

// Device memory that is part of the library image (see decdec_decode_attention_static): [heads] arrival counters,
// then [heads][8][head_dim + 2] floats, at the largest supported size.
constexpr uint32_t kStaticHeads = 128, kStaticHeadDim = 128, kStaticSplits = 8;
constexpr size_t kStaticScratchBytes = (size_t)kStaticHeads * 4u + (size_t)kStaticHeads * kStaticSplits * (kStaticHeadDim + 2) * 4u;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

enum { kOk = 0, kInvalid = 1, kHipError = 2, kUnsupported = 3 };

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

#define DD_HIP(expr)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess) return fail(kHipError, "HIP error in %s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

#define DD_CHECK(cond, ...)                          \
    do {                                             \
        if (!(cond)) return fail(kInvalid, __VA_ARGS__); \
    } while (0)

// ---- options -------------------------------------------------------------------------------------
struct Options {
    int fusion = 1;
    int host_noncoherent = 0;
    int anyprec_rpw = 0;
    int lutgemm_ktiles = 0;
    int sqllm_ktiles = 0;
    int dec_trace = 0;
    int anyprec_rg = 0;
    int dec_block_waves = 16;   // waves of a standalone DEC workgroup: 4, 8 or 16
    int fused_two_per_cu = -1;  // fused launches: 1 / 0 = always / never two workgroups per compute unit, -1 = by estimate
    int attention_two_step = 0; // decode attention with a workspace: 1 = merge the ranges of a head in a second kernel
    int attention_single_below = 512;  // ... and merging in the kernel: sequences up to this length are not shared at all
    int fused_small = -1;       // fused 3-bit any-precision launches with both roles in the GEMV's own smaller workgroups:
                                // -1 = when those have 5..8 waves (measured faster there), 1 = whenever they have <= 8, 0 = never
    int dec_force_cg = 0, dec_force_sg = 0;  // DEC launch plans: chunk groups / segment groups fixed by hand (tuning; 0 = planned)
    int dec_max_chunk_groups = 0;  // DEC launch plans: at most this many chunk groups (atomic adds per output); 0 = the built-in bound
    int gemv_max_k_ranges = 0;     // LUT-GEMM / SqueezeLLM launch plans: at most this many K ranges (atomic adds per output); 0 = chosen for speed
    int dec_rows_in_flight = 0;    // residual rows a DEC wave requests at a time: 2, 4 or 8; 0 = chosen per launch
    int anyprec_tile = 0;     // 3-bit tile decoder: waves per tile (2, 4, 8); 0 = off (default: the row-slice kernel is faster at decode shapes)
} g_opt;

uint32_t dec_block_threads() {
    const int w = g_opt.dec_block_waves <= 4 ? 4 : (g_opt.dec_block_waves <= 8 ? 8 : 16);
    return (uint32_t)w * kWave;
}

// Diagnostics: per-workgroup cycle stamps of the DEC phases (option "dec_trace").
constexpr int kTraceBlocks = 4096;
unsigned long long* g_trace_dev = nullptr;

int* option_slot(const char* name) {
    if (!name) return nullptr;
    if (!strcmp(name, "fusion")) return &g_opt.fusion;
    if (!strcmp(name, "host_noncoherent")) return &g_opt.host_noncoherent;
    if (!strcmp(name, "anyprec_rpw")) return &g_opt.anyprec_rpw;
    if (!strcmp(name, "lutgemm_ktiles")) return &g_opt.lutgemm_ktiles;
    if (!strcmp(name, "sqllm_ktiles")) return &g_opt.sqllm_ktiles;
    if (!strcmp(name, "dec_trace")) return &g_opt.dec_trace;
    if (!strcmp(name, "anyprec_rg")) return &g_opt.anyprec_rg;
    if (!strcmp(name, "anyprec_tile")) return &g_opt.anyprec_tile;
    if (!strcmp(name, "fused_two_per_cu")) return &g_opt.fused_two_per_cu;
    if (!strcmp(name, "fused_small")) return &g_opt.fused_small;
    if (!strcmp(name, "attention_two_step")) return &g_opt.attention_two_step;
    if (!strcmp(name, "attention_single_below")) return &g_opt.attention_single_below;
    if (!strcmp(name, "dec_block_waves")) return &g_opt.dec_block_waves;
    if (!strcmp(name, "dec_max_chunk_groups")) return &g_opt.dec_max_chunk_groups;
    if (!strcmp(name, "gemv_max_k_ranges")) return &g_opt.gemv_max_k_ranges;
    if (!strcmp(name, "dec_rows_in_flight")) return &g_opt.dec_rows_in_flight;
    if (!strcmp(name, "dec_force_cg")) return &g_opt.dec_force_cg;
    if (!strcmp(name, "dec_force_sg")) return &g_opt.dec_force_sg;
    return nullptr;
}

// ---- soft-float conversions for the host-side threshold arithmetic ---------------------------------
float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3FFu;
    if (e == 0) { const float v = (float)m * 5.9604644775390625e-08f; return sign ? -v : v; }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}
uint16_t f2h(float f) {   // round to nearest, ties to even
    const uint32_t u = f32_bits(f), sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
    if (a <= 0x33000000u) return (uint16_t)sign;
    const int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u, base = 0;
    int shift = 13;
    if (e < -14) shift += -14 - e; else { base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    return (uint16_t)(sign | (base + q));
}
float b2f(uint16_t b) { return bits_f32((uint32_t)b << 16); }
uint16_t f2b(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float round_to(float v, int dt) {
    if (dt == DECDEC_FP16) return h2f(f2h(v));
    if (dt == DECDEC_BF16) return b2f(f2b(v));
    return v;
}
float load_host(const void* p, int dt, size_t i) {
    if (dt == DECDEC_FP16) return h2f(((const uint16_t*)p)[i]);
    if (dt == DECDEC_BF16) return b2f(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}
size_t dtype_size(int dt) { return dt == DECDEC_FP32 ? 4 : 2; }
bool dtype_ok(int dt) { return dt == DECDEC_FP32 || dt == DECDEC_FP16 || dt == DECDEC_BF16; }

// The selector's 32 bucket floors (reference dec.cu:117-130): each step rounded exactly where the
// reference's typed arithmetic rounds.  volatile keeps the compiler from contracting or reassociating.
void bucket_floors(float a, float b, int dt, float* out) {
    volatile float diff = round_to(b - a, dt);
    for (int i = 0; i < kBuckets; ++i) {
        if (i < kBuckets / 2) {
            volatile float prod = diff * (float)i;
            volatile float quo = prod / (float)(kBuckets / 2 - 1);
            volatile float step = round_to(quo, dt);
            out[i] = round_to(a + step, dt);
        } else {
            volatile float prod = b * (float)(kBuckets - i - 1);
            volatile float quo = prod / (float)(kBuckets - kBuckets / 2);
            out[i] = round_to(quo, dt);
        }
    }
}

// ---- reference launch geometry (dec_config.cu:34-115), reported by read_dec_config ------------------
uint32_t cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// Compute units of the current device (256 on MI355X), asked once.
uint32_t device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cus = n;
    }
    return (uint32_t)cus;
}

int reference_geometry(uint32_t K, uint32_t N, uint32_t n_tb, uint32_t k_chunk, int dt, uint32_t max_smem,
                       decdec_config_info* o) {
    const uint32_t total = N / 8;
    uint32_t cpt = cdiv(cdiv(total, n_tb), 32) * 32, bx;
    if (cpt > 256) {
        const uint32_t times = cdiv(cpt, 256);
        bx = cdiv(total / n_tb / times, 32) * 32;
        cpt = bx * times;
    } else {
        bx = cpt;
    }
    if (bx == 0) return 1;
    const uint32_t num_blocks = cdiv(total, cpt), by = 1024 / bx, num_chunks = cdiv(K, 1024);
    const uint32_t item = (uint32_t)dtype_size(dt);
    const uint32_t rows = k_chunk * num_chunks;
    const uint32_t row_select = k_chunk * 32 * 4 + 1024 * item;
    uint32_t dec_req = rows * 4 + 8 * bx * by * item + bx * 8 * item + rows * item;
    uint32_t dyn = std::max(row_select, dec_req);
    int status = 0;
    if (dyn + 128 > max_smem) {
        dec_req = 8 * bx * by * item + bx * 8 * item;
        dyn = std::max(row_select, dec_req);
        status = (dyn + 128 > max_smem) ? -1 : 1;
    }
    o->num_chunks = (int)num_chunks; o->chunk_size = 1024; o->k_chunk = (int)k_chunk;
    o->channels_per_tb = (int)cpt; o->n_tb = (int)std::min(std::max(num_chunks, num_blocks), n_tb);
    o->block_dim_x = (int)bx; o->block_dim_y = (int)by; o->shared_memory_size = (int)dyn;
    o->reduced_shared_memory = status == 1;
    return status == -1 ? 2 : 0;
}

// ---- objects ---------------------------------------------------------------------------------------
struct Context {
    int dt;
    uint32_t num_tb;
    uint64_t buffer_numel;
    int32_t* rows;
    void* acts;
    hipStream_t sub_stream;
    hipEvent_t event;
};

struct DecPlan {
    uint32_t cg, sg, nseg, vec, segs_per_block, slots, lds_reduce;
    size_t lds;
};

struct Config {
    int dt;
    Context* ctx;
    const uint32_t* residual_dev;   // device-visible residual
    void* residual_host;            // owned pinned allocation (nullptr when borrowed from the device)
    void* scales_dev;               // owned device copy
    const void* thresholds_host;    // borrowed
    uint32_t K, N, M, k_chunk, max_smem;
    decdec_config_info info;
    DecPlan plans[3];               // for DEC workgroups of 4, 8 and 16 waves
    hipEvent_t e1, e2;
};

std::mutex g_mu;
std::unordered_set<uint64_t> g_contexts, g_configs;

Context* get_context(uint64_t h) {
    std::lock_guard<std::mutex> l(g_mu);
    return g_contexts.count(h) ? reinterpret_cast<Context*>(h) : nullptr;
}
Config* get_config(uint64_t h) {
    std::lock_guard<std::mutex> l(g_mu);
    return g_configs.count(h) ? reinterpret_cast<Config*>(h) : nullptr;
}

constexpr size_t kLdsBudget = 60 * 1024;

// Upper bound on the chunk groups of a DEC launch.  Every chunk group adds its partial sum to an output with an
// atomic add of its own, i.e. one more rounding of a 16-bit output in an order that varies from run to run; the
// reference adds once per output (dec.cu:263-276).  With 14 of them (K = 14336) an output now and then missed the
// 1e-2 bound.  A workgroup selects up to (waves / 4) chunks at a time, so few chunk groups cost little.
constexpr uint32_t kMaxChunkGroups = 4;

// Split the DEC work of one layer over at most `budget` workgroups of `nw` waves: cg chunk groups x sg
// segment groups, cg <= kMaxChunkGroups (option dec_max_chunk_groups can lower it), minimising the longest
// per-workgroup path.  The row list of a workgroup must fit in LDS: only a
// row list that fits with no allowed cg (k_chunk in the hundreds at K > 16384) lifts the bound.
int plan_dec(uint32_t K, uint32_t M, uint32_t k_chunk, uint32_t budget, uint32_t nw, DecPlan* pl) {
    const uint32_t num_chunks = cdiv(K, 1024);
    const uint32_t nseg = cdiv(M, 64);
    const uint32_t teams = nw >= 16u ? 4u : std::max(1u, nw / 2u);     // chunks a workgroup selects at a time (dec_role.h, DecTeam)
    budget = std::max(1u, budget);
    uint32_t cap = kMaxChunkGroups;
    if (g_opt.dec_max_chunk_groups >= 1) cap = std::min(cap, (uint32_t)g_opt.dec_max_chunk_groups);
    uint64_t best_cost = ~0ull;
    uint32_t best_cg = 0, best_sg = 0;
    size_t best_lds = 0;
    for (int pass = 0; pass < 2 && best_cg == 0; ++pass) {
        const uint32_t cg_max = pass == 0 ? std::min(num_chunks, cap) : num_chunks;
        for (uint32_t cg = 1; cg <= cg_max; ++cg) {
            if (g_opt.dec_force_cg > 0 && pass == 0 && cg != std::min((uint32_t)g_opt.dec_force_cg, cg_max)) continue;
            const uint32_t sg_max = std::min(nseg, std::max(1u, budget / cg));
            for (uint32_t sg = 1; sg <= sg_max; ++sg) {
                if (g_opt.dec_force_sg > 0 && pass == 0 && sg != std::min((uint32_t)g_opt.dec_force_sg, sg_max)) continue;
                const uint32_t cpb = cdiv(num_chunks, cg), spb = cdiv(nseg, sg);
                const uint32_t slots = (cpb * std::max(k_chunk, 1u) + 1u) & ~1u;   // even: keeps the LDS arrays behind the row list 16-byte aligned
                const size_t lds = dec_lds_bytes(slots, nw);
                if (lds > kLdsBudget) continue;
                // per-workgroup critical path: rounds of selection (one chunk per team of four waves), then
                // batches of eight rows per wave for each group of up to nw segments; going over the
                // workgroup budget is a last resort
                const uint32_t sb = std::min(spb, nw), rl = nw / sb;
                const uint64_t batches = (uint64_t)cdiv(spb, nw) * cdiv(slots, rl * 8);
                // Ties go to MORE chunk groups (within the bound): a workgroup then reads wider pieces of fewer rows, and
                // pieces of one row are contiguous in host memory.  Measured, DEC alone at k_chunk 32 with the same
                // number of batches: 4096 x 4096 15.3 us with 1 chunk group x 8 segment groups, 12.3 us with 4 x 2 or
                // 4 x 8; 14336 x 4096 41.6 / 32.0 / 26.3 us with 1 / 2 / 4 chunk groups; 28672 x 8192 108 / 88 / 79 us.
                // ... and, below sixteen workgroups, to more segment groups: measured on the Llama-3-8B token at k_chunk 8,
                // 1540 us with 4 / 8 / 8 workgroups for the 4096-, 14336-output and down-projection launches, 1505 us with 16
                // each (shorter merges, fewer rows per wave behind one round trip); with the residual in HBM 1539 -> 1524.
                const uint64_t cost = batches * 1000 + (uint64_t)cdiv(cpb, teams) * 600 + (uint64_t)(64u - std::min(cg, 64u)) * 10 +
                                      (uint64_t)(16u - std::min(cg * sg, 16u)) * 20 + (cg * sg > budget ? 500000ull : 0);
                if (cost < best_cost) { best_cost = cost; best_cg = cg; best_sg = sg; best_lds = lds; }
            }
        }
    }
    if (best_cg == 0) return 1;
    pl->cg = best_cg; pl->sg = best_sg; pl->nseg = nseg; pl->vec = 1;
    pl->segs_per_block = cdiv(nseg, best_sg);
    pl->slots = (cdiv(num_chunks, best_cg) * std::max(k_chunk, 1u) + 1u) & ~1u;
    pl->lds_reduce = 1; pl->lds = best_lds;
    return 0;
}

int setup_config(Config* c, uint32_t k_chunk) {
    Context* ctx = c->ctx;
    c->k_chunk = k_chunk;
    memset(&c->info, 0, sizeof(c->info));
    const int st = reference_geometry(c->K, c->N, std::max(1u, ctx->num_tb), k_chunk, c->dt, c->max_smem, &c->info);
    if (st == 1) return fail(kInvalid, "DECConfig: output size %u is too small for the DEC launch geometry", c->N);
    const uint64_t k = (uint64_t)k_chunk * c->K / 1024;
    // reference dec_config.cu:180-181
    DD_CHECK(ctx->buffer_numel >= k, "DECContext buffer size is too small for the given k_chunk.");
    DD_CHECK(k_chunk <= 1024, "k_chunk must not exceed the chunk size (1024), got %u", k_chunk);
    // num_tb counts 1024-thread workgroups; smaller workgroups get the same number of waves in total
    for (uint32_t i = 0; i < 3; ++i) {
        const uint32_t nw = 4u << i;
        if (plan_dec(c->K, c->M, k_chunk, std::max(1u, ctx->num_tb) * (16u / nw), nw, &c->plans[i]))
            return fail(kUnsupported, "DEC launch plan does not fit in LDS (k_chunk=%u, K=%u)", k_chunk, c->K);
    }
    const DecPlan& plan = c->plans[2];
    c->info.hip_dec_blocks = (int)(plan.cg * plan.sg);
    c->info.hip_chunk_groups = (int)plan.cg;
    c->info.hip_segment_groups = (int)plan.sg;
    c->info.hip_vec_words = (int)plan.vec;
    c->info.hip_lds_bytes = (int)plan.lds;
    c->info.hip_slots_per_block = (int)plan.slots;
    c->info.hip_lds_reduce = (int)plan.lds_reduce;
    c->info.hip_residual_on_host = c->residual_host != nullptr;
    return kOk;
}

// Fill the kernel parameters of one DEC call.  Returns 1 when there is nothing to do (k == 0).
const DecPlan& dec_plan(const Config* c, uint32_t nw) { return c->plans[nw <= 4 ? 0 : (nw <= 8 ? 1 : 2)]; }

// Bytes per microsecond at which a DEC role reads its residual rows: the host link's measured ceiling for a residual in
// pinned host memory; for a residual that already lives in device memory the rows cost next to nothing beside the
// role's latency floor (measured: 8.5 us at 4096 -> 4096 and 15.7 us at 14336 -> 4096, k_chunk 32, against 11.8 and 24.5).
constexpr double kHostLinkBytesPerUs = 56e3, kDeviceResidualBytesPerUs = 1e6;
double dec_residual_rate(const Config* c) { return c->residual_host ? kHostLinkBytesPerUs : kDeviceResidualBytesPerUs; }

// Residual rows a wave requests per round (dec_role.h, dec_fetch_rows): the fewest of 2, 4, 8 with which the wave's rows
// take no more rounds than fit into the time the launch's rows occupy the link anyway (a round trip under light load is
// about 2 us).  Few rows per round keep the number of requests in flight near what the link serves per round trip;
// measured on the Llama-3-8B token with one value for every launch, k_chunk 4 / 8 / 16 / 32 / 64: 1336 / 1496 / 1882 /
// 2808 / 4767 us with two, 1367 / 1459 / 1917 / 2912 / 4909 with four, 1400 / 1520 / 1935 / 2903 / 4866 with eight
// (at k_chunk 8 the down projection has eight rows per wave behind 4 us of link time and wants four per round; with the
// residual in HBM, k_chunk 64: 1874 / 1677 / 1642; Phi-3-medium decode with DEC on gate_up and down at k_chunk 8, where a
// workgroup has 18 segments for 16 waves: 320.8 / 328.5 / 328.6 tokens/s).
uint32_t dec_rows_per_round(const DecPlan& plan, uint32_t nw, double launch_link_us) {
    if (g_opt.dec_rows_in_flight > 0) return (uint32_t)g_opt.dec_rows_in_flight;
    const uint32_t sb = std::max(1u, std::min(plan.segs_per_block, nw)), waves_per_segment = std::max(1u, nw / sb);
    const uint32_t rows_per_wave = cdiv(plan.slots, waves_per_segment);
    const uint32_t passes = cdiv(plan.segs_per_block, nw);            // a workgroup with more segments than waves walks its rows again
    const uint32_t rounds = (uint32_t)std::max(1.0, launch_link_us / 2.0);
    uint32_t u = 2;
    while (u < 8u && passes * cdiv(rows_per_wave, u) > rounds) u *= 2u;
    return u;
}

int fill_dec_params(const Config* c, const void* input, void* output, bool fused_select, DecParams* p,
                    uint32_t nw = kDecWaves, const DecPlan* plan_override = nullptr, double launch_link_us = 0.0) {
    const uint64_t k = (uint64_t)c->k_chunk * c->K / 1024;       // reference decdec.cu:50
    if (k == 0) return 1;                                        // reference decdec.cu:52-54
    memset(p, 0, sizeof(*p));
    p->residual = c->residual_dev; p->scales = c->scales_dev; p->x = input;
    p->sel_rows = c->ctx->rows; p->sel_acts = c->ctx->acts; p->out = output;
    if (fused_select) {
        // thresholds[0] and thresholds[k-1] are read on the host at call time (reference decdec.cu:66-67)
        const float a = load_host(c->thresholds_host, c->dt, 0);
        const float b = load_host(c->thresholds_host, c->dt, (size_t)k - 1);
        bucket_floors(a, b, c->dt, p->floors);
        bool mono = std::isfinite(p->floors[0]) && std::isfinite(p->floors[kBuckets - 1]);
        for (int i = 1; i < kBuckets; ++i) mono = mono && (p->floors[i] <= p->floors[i - 1]);
        p->monotone = mono ? 1u : 0u;
    }
    p->K = c->K; p->N = c->N; p->M = c->M;
    p->num_chunks = cdiv(c->K, 1024); p->k_chunk = c->k_chunk; p->k_total = (uint32_t)k;
    const DecPlan& plan = plan_override ? *plan_override : dec_plan(c, nw);
    p->cg = plan.cg; p->sg = plan.sg; p->nseg = plan.nseg;
    p->segs_per_block = plan.segs_per_block; p->slots_per_block = plan.slots;
    p->fused_select = fused_select ? 1u : 0u;
    const double own_link_us = (double)k * (double)c->N * 0.5 / dec_residual_rate(c);
    p->rows_in_flight = dec_rows_per_round(plan, nw, std::max(own_link_us, launch_link_us));
    if (g_opt.dec_trace && p->cg * p->sg <= (uint32_t)kTraceBlocks) {
        if (!g_trace_dev && hipMalloc(&g_trace_dev, sizeof(unsigned long long) * 8 * kTraceBlocks) != hipSuccess)
            g_trace_dev = nullptr;
        p->trace = g_trace_dev;
    }
    return 0;
}

// DEC plan of one layer of a batched launch (1024-thread workgroups).  The layers of a batch share their contexts'
// workgroup budget by output width, with a floor of min(num_tb, 16) workgroups per layer.  Measured on the Llama-3-8B linear set at
// k_chunk 32, num_tb 32: gate | up planned with the whole budget each (2 x 28 DEC workgroups) 2951-2982 us per token,
// with 2 x 16 to 2 x 24 workgroups 2896-2904, with 2 x 12 2948-2991, with 2 x 8 2974; a layer launched alone is best with
// its full budget.
// Hence also the bound of 48 on what a batch shares out.
int plan_dec_in_batch(const Config* c, uint64_t dec_rows_in_batch, DecPlan* pl) {
    const uint64_t num_tb = std::min(48u, std::max(1u, c->ctx->num_tb)), floor_tb = std::min<uint64_t>(num_tb, 16);
    const uint32_t share = (uint32_t)std::min<uint64_t>(num_tb, std::max<uint64_t>(floor_tb, num_tb * c->N / std::max<uint64_t>(1, dec_rows_in_batch)));
    return plan_dec(c->K, c->M, c->k_chunk, share, kDecWaves, pl);
}

int check_dec_call(const Config* c, int dtype, uint32_t in_features, uint32_t out_features,
                   const void* input, const void* output) {
    DD_CHECK(c != nullptr, "invalid DECConfig handle");
    DD_CHECK(input && output, "input and output pointers must not be null");
    DD_CHECK(dtype == c->dt, "Mismatched data types between input tensor and DECConfig.");
    DD_CHECK(in_features == c->K, "input tensor size does not match with DECConfig: input size: %u, DECConfig size: %u",
             in_features, c->K);
    DD_CHECK(out_features == c->N, "output tensor size does not match with DECConfig: output size: %u, DECConfig size: %u",
             out_features, c->N);
    DD_CHECK(c->ctx != nullptr && c->ctx->dt == c->dt, "Data type mismatch between DECConfig and DECContext.");
    // 16-bit outputs are merged with packed two-element atomic adds on even element pairs
    DD_CHECK(dtype == DECDEC_FP32 || ((uintptr_t)output % 4) == 0, "output must be 4-byte aligned");
    return kOk;
}

// ---- base-GEMV launch plans ------------------------------------------------------------------------
struct AnyprecPlan { AnyprecParams p; LaunchDims d; };

int plan_anyprec(const void* input, void* output, const void* qweight, const void* lut, int bits, int dtype,
                 uint32_t K, uint32_t N, bool fused_block, AnyprecPlan* pl, uint32_t rpw_cap = 8,
                 uint64_t rows_in_launch = 0) {
    DD_CHECK(bits >= 3 && bits <= 8, "Bitwidth must be between 3 and 8.");
    if (dtype == DECDEC_FP32)
        return fail(kUnsupported, "Any-Precision GEMV does not support float data type. Please use half or bfloat16.");
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(input && output && qweight && lut, "null pointer argument");
    DD_CHECK(K >= 32 && K % 32 == 0, "input_feat must be a positive multiple of 32, got %u", K);
    DD_CHECK(N >= 1, "output_feat must be positive");
    DD_CHECK(((uintptr_t)lut % 16) == 0 || bits > 4, "lut must be 16-byte aligned");
    DD_CHECK(((uintptr_t)output % 4) == 0, "output must be 4-byte aligned");
    AnyprecParams& p = pl->p;
    memset(&p, 0, sizeof(p));
    p.x = input; p.qweight = (const uint32_t*)qweight; p.lut = lut; p.out = output;
    p.N = N; p.K = K; p.W = K / 32;
    const uint32_t s_total = cdiv(p.W, 64);
    p.sgroups = cdiv(s_total, 16);
    p.S = cdiv(s_total, p.sgroups);
    p.rg = fused_block ? std::max(1u, 16u / p.S) : std::max(1u, 4u / p.S);   // 256-thread workgroups measured best
    // Rows per wave: every wave requests all its rows at once, so more rows per wave mean more bytes
    // in flight per resident wave (large matrices), fewer rows mean more waves to share the decode
    // work (small matrices, where one wave per SIMD would issue at a quarter of the VALU rate).
    // (a layer of a batched launch is planned by the rows of the whole launch: two 14336-row layers planned alone get
    // four rows per wave and 3584 workgroups between them, whose dispatch alone outlasts the 1792 of eight rows per wave)
    const uint64_t row_slices = std::max<uint64_t>(N, rows_in_launch) * p.S * p.sgroups;
    uint32_t rpw = row_slices >= 32768 ? 8u : (row_slices >= 8192 ? 4u : 2u);
    if (row_slices >= 16384 && p.S * p.sgroups >= 4) rpw = 8u;     // long rows (K >= 8192): measured 9.0 against 10.1 us at 14336 -> 4096
    if (g_opt.anyprec_rpw == 2 || g_opt.anyprec_rpw == 4 || g_opt.anyprec_rpw == 8) rpw = (uint32_t)g_opt.anyprec_rpw;
    if (bits > 3) rpw = std::min(rpw, 4u);      // wider formats: four rows of plane words per wave fit the registers, eight do not
    if (g_opt.anyprec_rpw == 0) rpw = std::min(rpw, rpw_cap);
    p.rpw = rpw;
    if (g_opt.anyprec_rg > 0) p.rg = std::min((uint32_t)g_opt.anyprec_rg, std::max(1u, 16u / p.S));
    p.x_aligned = ((uintptr_t)input % 16) == 0;
    pl->d.grid = cdiv(N, p.rg * p.rpw) * p.sgroups;
    pl->d.block = fused_block ? 1024u : 64u * p.S * p.rg;
    pl->d.lds = anyprec_lds_bytes(p.S, p.rg, p.rpw, bits);
    // 3-bit tile decoder: needs whole 1024-channel chunks, 16-byte aligned planes and LUT rows, and a
    // dword-aligned activation vector (it is read through the scalar cache)
    const bool tile_able = bits == 3 && K % 1024 == 0 && ((uintptr_t)qweight % 16) == 0 &&
                           ((uintptr_t)input % 4) == 0 && g_opt.anyprec_tile != 0;
    // at most 8 atomic adds (roundings, in an order that varies from run to run) per 16-bit output: with 14 of them
    // (K = 14336) an output now and then missed the 1e-2 bound by a few percent of it; longer rows keep the row form
    uint32_t cs = (g_opt.anyprec_tile == 2 || g_opt.anyprec_tile == 4) ? (uint32_t)g_opt.anyprec_tile : 8u;
    while (cs < 8u && p.W / (4u * cs) > 8u) cs *= 2u;
    if (tile_able && p.W / (4u * cs) <= 8u) {
        p.tile_cs = cs;
        p.tile_kt = p.W / (4u * cs);
        p.tiles = cdiv(N, 64) * p.tile_kt;
        const uint32_t waves = fused_block ? 16u : cs;
        pl->d.block = 64u * waves;
        pl->d.grid = cdiv(p.tiles, waves / cs);
        pl->d.lds = (waves / cs) * anyprec3_tile_lds_bytes(cs);
    }
    return kOk;
}

struct LutgemmPlan { LutgemmParams p; LaunchDims d; };

int plan_lutgemm(const void* input, void* output, const void* qw, const void* alpha, const void* q_bias, int bits,
                 int group_size, int dtype, uint32_t K, uint32_t N, bool fused_block, LutgemmPlan* pl,
                 uint32_t slots_avail = 0) {
    DD_CHECK(bits >= 1 && bits <= 8, "Bitwidth must be between 1 and 8.");
    DD_CHECK(dtype_ok(dtype), "Unsupported data type.");
    DD_CHECK(input && output && qw && alpha && q_bias, "null pointer argument");
    DD_CHECK(K >= 32 && K % 32 == 0, "input_feat must be a positive multiple of 32, got %u", K);
    DD_CHECK(group_size >= 32 && group_size % 32 == 0 && K % (uint32_t)group_size == 0,
             "group_size must be a multiple of 32 that divides input_feat, got %d", group_size);
    DD_CHECK(N >= 1, "output_feat must be positive");
    DD_CHECK(((uintptr_t)output % 4) == 0, "output must be 4-byte aligned");
    LutgemmParams& p = pl->p;
    memset(&p, 0, sizeof(p));
    p.x = input; p.qw = (const uint32_t*)qw; p.alpha = alpha; p.q_bias = q_bias; p.out = output;
    p.N = N; p.K = K; p.bits = (uint32_t)bits; p.group_size = (uint32_t)group_size;
    // 16 waves per workgroup share 64 columns and split the workgroup's K range in slices of 1..7 tiles of 32
    // channels per wave (tables of 7 tiles per wave = 57 KB of LDS; two workgroups fit a compute unit).  The number
    // of K ranges (one atomic add, i.e. one rounding of a 16-bit output, each; at most 9) is the one with the
    // smallest (turns of workgroups) x (tiles per wave + start-up): a grid a little above one turn runs its rest as
    // a second, nearly empty turn.  Measured: 5120 -> 7680 with 600 workgroups 8.8 us, with 480 7.7 us;
    // 17920 -> 5120 with 720 workgroups 14.2 us, with 400 (7 tiles per wave) 12.6 us; 5120 -> 35840 with 1680
    // workgroups 26.5 us, with 1120 25.1 us.
    const uint32_t waves = 16, tiles = K / 32;
    p.n_tiles = cdiv(N, 64);
    if (g_opt.lutgemm_ktiles > 0) {
        const uint32_t kt = (uint32_t)g_opt.lutgemm_ktiles;
        p.slice_tiles = std::max(1u, std::min(4u, cdiv(tiles, kt * waves)));
        p.k_tiles = cdiv(tiles, p.slice_tiles * waves);
    } else {
        // workgroup slots this layer can count on: the whole device, or its share of it inside a batched launch
        const uint32_t slots = slots_avail ? slots_avail : 2u * device_cus();
        uint32_t best_cost = ~0u;
        // option gemv_max_k_ranges: a caller's bound on the atomic adds per output (kept while 7 tiles per wave allow it)
        const uint32_t kr_max = g_opt.gemv_max_k_ranges >= 1 ? std::min(9u, (uint32_t)g_opt.gemv_max_k_ranges) : 9u;
        for (uint32_t kr = 1; kr <= kr_max; ++kr) {
            const uint32_t slice = cdiv(tiles, kr * waves);
            if (slice > 7u) continue;
            const uint32_t k_tiles = cdiv(tiles, slice * waves);
            const uint32_t cost = cdiv(p.n_tiles * k_tiles, slots) * (2u * slice + 3u);
            if (cost < best_cost) { best_cost = cost; p.slice_tiles = slice; p.k_tiles = k_tiles; }
        }
        if (best_cost == ~0u) {                          // K beyond 9 ranges of 7 tiles per wave: more ranges
            p.slice_tiles = 7u;
            p.k_tiles = cdiv(tiles, p.slice_tiles * waves);
        }
    }
    pl->d.grid = p.n_tiles * p.k_tiles;
    pl->d.block = 64u * waves;
    pl->d.lds = lutgemm_lds_bytes(p.slice_tiles, waves);
    (void)fused_block;
    return kOk;
}

struct SqllmPlan { SqllmParams p; LaunchDims d; };

int plan_sqllm(const void* input, void* output, const void* mat, const void* lut, int bits, int dtype,
               uint32_t K, uint32_t N, bool fused_block, SqllmPlan* pl) {
    DD_CHECK(bits == 3 || bits == 4, "Bitwidth must be 3 or 4.");
    DD_CHECK(dtype_ok(dtype), "Unsupported data type.");
    DD_CHECK(input && output && mat && lut, "null pointer argument");
    DD_CHECK(K >= 32 && K % 32 == 0, "input_feat must be a positive multiple of 32, got %u", K);
    DD_CHECK(N >= 1, "output_feat must be positive");
    DD_CHECK(((uintptr_t)output % 4) == 0, "output must be 4-byte aligned");
    SqllmParams& p = pl->p;
    memset(&p, 0, sizeof(p));
    p.x = input; p.mat = (const uint32_t*)mat; p.lut = lut; p.out = output;
    p.N = N; p.K = K; p.bits = (uint32_t)bits;
    DD_CHECK(((uintptr_t)input % 4) == 0, "input must be 4-byte aligned");
    // 16 waves per workgroup share 64 columns and split the workgroup's K range; the K ranges (one atomic
    // add, i.e. one rounding of a 16-bit output, each) are few: enough for about 8 waves per SIMD, at most 8
    const uint32_t waves = 16;
    p.n_tiles = cdiv(N, 64);
    // 16-bit types: the pair table takes 68 KB of LDS, two workgroups fit a CU, so at most 512 workgroups run
    // at once; that many K ranges (measured best), fp32: enough for about 8 waves per SIMD
    uint32_t kt = dtype != DECDEC_FP32 ? 512u / std::min(512u, p.n_tiles) : cdiv(8192, p.n_tiles * waves);
    if (g_opt.gemv_max_k_ranges >= 1) kt = std::min(kt, (uint32_t)g_opt.gemv_max_k_ranges);
    if (g_opt.sqllm_ktiles > 0) kt = (uint32_t)g_opt.sqllm_ktiles;
    kt = std::max(1u, std::min(std::min(kt, 8u), std::max(1u, K / (32u * waves))));
    p.kslice = cdiv(cdiv(K, kt * waves), 32) * 32;
    p.k_tiles = cdiv(K, p.kslice * waves);
    pl->d.grid = p.n_tiles * p.k_tiles;
    pl->d.block = 64u * waves;
    pl->d.lds = sqllm_lds_bytes(p.bits, waves, dtype != DECDEC_FP32);
    DD_CHECK(dtype == DECDEC_FP32 || ((uintptr_t)lut % 16) == 0, "lut must be 16-byte aligned");
    (void)fused_block;
    return kOk;
}

// Side stream and events of the dummy_* calls (the reference creates and leaks a stream and two events
// per call, decdec.cu:851-857; one set is enough).
hipStream_t g_dummy_stream = nullptr;
hipEvent_t g_dummy_e1 = nullptr, g_dummy_e2 = nullptr;

int ensure_dummy_stream() {
    if (!g_dummy_stream) {
        DD_HIP(hipStreamCreateWithFlags(&g_dummy_stream, hipStreamNonBlocking));
        DD_HIP(hipEventCreateWithFlags(&g_dummy_e1, hipEventDisableTiming));
        DD_HIP(hipEventCreateWithFlags(&g_dummy_e2, hipEventDisableTiming));
    }
    return kOk;
}

// Two-stream form (reference decdec.cu:621-640): DEC on the caller's stream, the GEMV on the
// context's sub-stream, joined by events.
template <typename GemvLaunch>
static int two_stream(Config* c, const DecParams* dp, bool have_dec, int dtype, hipStream_t main_stream,
                      GemvLaunch gemv) {
    hipStream_t sub = c->ctx->sub_stream;
    DD_HIP(hipEventRecord(c->e1, main_stream));
    if (have_dec) {
        const DecPlan& plan = dec_plan(c, kDecWaves);
        LaunchDims d{plan.cg * plan.sg, (uint32_t)kDecThreads, plan.lds};
        DD_HIP(launch_dec(dtype, *dp, d, main_stream));
    }
    DD_HIP(hipStreamWaitEvent(sub, c->e1, 0));
    DD_HIP(gemv(sub));
    DD_HIP(hipEventRecord(c->e2, sub));
    DD_HIP(hipStreamWaitEvent(main_stream, c->e2, 0));
    return kOk;
}

template <typename GemvLaunch>
static int dummy_common(int dummy_cu, int64_t iters, hipStream_t main_stream, GemvLaunch gemv) {
    int rc = ensure_dummy_stream();
    if (rc != kOk) return rc;
    DD_HIP(hipEventRecord(g_dummy_e1, main_stream));
    if (dummy_cu > 0) DD_HIP(launch_burner((uint32_t)dummy_cu, (long long)iters, main_stream));
    DD_HIP(hipStreamWaitEvent(g_dummy_stream, g_dummy_e1, 0));
    DD_HIP(gemv(g_dummy_stream));
    DD_HIP(hipEventRecord(g_dummy_e2, g_dummy_stream));
    DD_HIP(hipStreamWaitEvent(main_stream, g_dummy_e2, 0));
    return kOk;
}

// ---- the static workspace of decdec_decode_attention_static ------------------------------------------------
// Every GPU the library runs on holds its own copy of `scratch` at its own address; host code never uses the
// array's name as a pointer, only the address hipGetSymbolAddress returns with that device current.

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out) {
    int dev = -1;
    DD_HIP(hipGetDevice(&dev));
    DD_CHECK(dev >= 0 && dev < kMaxDevices, "device index %d is outside the supported range", dev);
    std::lock_guard<std::mutex> l(g_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        DD_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        DD_CHECK(ptr != nullptr, "hipGetSymbolAddress returned a null address for the static workspace");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return kOk;
}

__global__ __launch_bounds__(128) void fill_u32_kernel(uint32_t* dst, uint32_t n, uint32_t value) {
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) dst[i] = value;
}

}  // namespace

extern "C" {

const char* decdec_last_error(void) { return g_error.c_str(); }
int decdec_version(void) { return 100; }

int decdec_set_option(const char* name, int value) {
    int* s = option_slot(name);
    DD_CHECK(s != nullptr, "unknown option '%s'", name ? name : "(null)");
    *s = value;
    return kOk;
}
int decdec_get_option(const char* name, int* value) {
    int* s = option_slot(name);
    DD_CHECK(s != nullptr && value != nullptr, "unknown option '%s'", name ? name : "(null)");
    *value = *s;
    return kOk;
}

int decdec_debug_read_trace(uint64_t* out, int workgroups) {
    DD_CHECK(out && workgroups > 0 && workgroups <= kTraceBlocks, "invalid argument");
    DD_CHECK(g_trace_dev != nullptr, "no trace has been recorded (set option dec_trace first)");
    DD_HIP(hipDeviceSynchronize());
    DD_HIP(hipMemcpy(out, g_trace_dev, sizeof(uint64_t) * 8 * (size_t)workgroups, hipMemcpyDeviceToHost));
    DD_HIP(hipMemset(g_trace_dev, 0, sizeof(uint64_t) * 8 * kTraceBlocks));
    return kOk;
}

int decdec_debug_read_probe(const void* src, uint64_t row_bytes, uint64_t rows, uint32_t vec_words, uint32_t blocks,
                            int scramble, void* sink, void* stream) {
    DD_CHECK(src && sink, "null pointer argument");
    DD_CHECK(vec_words == 1 || vec_words == 2 || vec_words == 4, "vec_words must be 1, 2 or 4");
    DD_CHECK(rows >= 1 && blocks >= 1, "rows and blocks must be positive");
    DD_CHECK(row_bytes >= 256ull * vec_words && row_bytes % (256ull * vec_words) == 0,
             "row_bytes must be a positive multiple of 256 * vec_words");
    DD_CHECK(((uintptr_t)src % 16) == 0, "src must be 16-byte aligned");
    DD_HIP(launch_read_probe(src, row_bytes, rows, vec_words, blocks, scramble, sink, (hipStream_t)stream));
    return kOk;
}

int decdec_bucket_floors(float a, float b, int dtype, float* out) {
    DD_CHECK(dtype_ok(dtype) && out, "invalid argument");
    bucket_floors(round_to(a, dtype), round_to(b, dtype), dtype, out);
    return kOk;
}

int decdec_reference_geometry(uint32_t K, uint32_t N, uint32_t n_tb, uint32_t k_chunk, int dtype,
                              uint32_t max_smem, decdec_config_info* out) {
    DD_CHECK(dtype_ok(dtype) && out && n_tb >= 1 && N >= 8, "invalid argument");
    memset(out, 0, sizeof(*out));
    const int st = reference_geometry(K, N, n_tb, k_chunk, dtype, max_smem, out);
    DD_CHECK(st != 1, "output size too small");
    return kOk;
}

int decdec_dec_launch_plan(uint32_t K, uint32_t N, uint32_t n_tb, uint32_t k_chunk, uint32_t block_waves,
                           decdec_config_info* out) {
    DD_CHECK(out && n_tb >= 1 && K >= 1 && N >= 8 && N % 8 == 0, "invalid argument");
    DD_CHECK(block_waves == 4 || block_waves == 8 || block_waves == 16, "block_waves must be 4, 8 or 16");
    DD_CHECK(k_chunk <= 1024, "k_chunk must not exceed the chunk size (1024), got %u", k_chunk);
    DecPlan pl;
    if (plan_dec(K, N / 8, k_chunk, n_tb * (16u / block_waves), block_waves, &pl))
        return fail(kUnsupported, "DEC launch plan does not fit in LDS (k_chunk=%u, K=%u)", k_chunk, K);
    memset(out, 0, sizeof(*out));
    out->num_chunks = (int)cdiv(K, 1024); out->chunk_size = 1024; out->k_chunk = (int)k_chunk;
    out->hip_dec_blocks = (int)(pl.cg * pl.sg);
    out->hip_chunk_groups = (int)pl.cg;
    out->hip_segment_groups = (int)pl.sg;
    out->hip_vec_words = (int)pl.vec;
    out->hip_lds_bytes = (int)pl.lds;
    out->hip_slots_per_block = (int)pl.slots;
    out->hip_lds_reduce = (int)pl.lds_reduce;
    return kOk;
}

// ---------------------------------------------------------------- context
int decdec_create_dec_context(uint32_t num_tb, int dtype, uint64_t buffer_numel, void* rows, void* acts,
                              uint64_t* out) {
    DD_CHECK(out != nullptr, "context_out must not be null");
    DD_CHECK(dtype_ok(dtype), "Unsupported data type.");
    DD_CHECK(rows != nullptr && acts != nullptr, "selected_rows_buffer and selected_activations_buffer must be on GPU.");
    DD_CHECK(num_tb >= 1, "num_tb must be at least 1");
    Context* c = new Context();
    c->dt = dtype; c->num_tb = num_tb; c->buffer_numel = buffer_numel;
    c->rows = (int32_t*)rows; c->acts = acts; c->sub_stream = nullptr; c->event = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&c->sub_stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->event, hipEventDisableTiming);
    if (e != hipSuccess) {
        if (c->sub_stream) (void)hipStreamDestroy(c->sub_stream);
        delete c;
        return fail(kHipError, "HIP error creating the DEC context: %s", hipGetErrorString(e));
    }
    {
        std::lock_guard<std::mutex> l(g_mu);
        g_contexts.insert(reinterpret_cast<uint64_t>(c));
    }
    *out = reinterpret_cast<uint64_t>(c);
    return kOk;
}

int decdec_destroy_dec_context(uint64_t h) {
    Context* c = get_context(h);
    DD_CHECK(c != nullptr, "invalid DECContext handle");
    {
        std::lock_guard<std::mutex> l(g_mu);
        // a config keeps a pointer to its context: destroying a context that live configs use would leave it dangling
        for (uint64_t ch : g_configs)
            if (reinterpret_cast<Config*>(ch)->ctx == c)
                return fail(kInvalid, "DECContext is still used by a DECConfig; destroy or update the config first");
        g_contexts.erase(h);
    }
    (void)hipStreamDestroy(c->sub_stream);
    (void)hipEventDestroy(c->event);
    delete c;
    return kOk;
}

// ---------------------------------------------------------------- config
int decdec_create_dec_config(uint64_t ctx_h, uint32_t k_chunk, int dtype, const void* q_residual,
                             int q_on_device, const void* scales, int scales_on_device,
                             const void* thresholds_host, uint32_t num_rows, uint32_t num_cols, uint64_t* out) {
    Context* ctx = get_context(ctx_h);
    DD_CHECK(ctx != nullptr, "invalid DECContext handle");
    DD_CHECK(out != nullptr, "config_out must not be null");
    DD_CHECK(dtype_ok(dtype), "Unsupported data type in create_dec_config.");
    DD_CHECK(dtype == ctx->dt, "Data type mismatch between DECConfig and DECContext.");
    DD_CHECK(q_residual && scales && thresholds_host, "null pointer argument");
    DD_CHECK(num_rows >= 1 && num_cols >= 8 && num_cols % 8 == 0,
             "q_residual must be [in_features, out_features / 8] with out_features a multiple of 8");
    Config* c = new Config();
    memset(c, 0, sizeof(*c));
    c->dt = dtype; c->ctx = ctx; c->K = num_rows; c->N = num_cols; c->M = num_cols / 8;
    c->thresholds_host = thresholds_host;
    int dev = 0, smem = 65536;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&smem, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
    const size_t res_bytes = (size_t)num_rows * c->M * 4, sc_bytes = (size_t)num_cols * dtype_size(dtype);
    if (e == hipSuccess) {
        c->max_smem = (uint32_t)smem;
        if (q_on_device) {
            fprintf(stderr, "DecDEC WARNING: q_residual is on the GPU; it is used in place and zero-copy host memory is NOT used.\n");
            c->residual_dev = (const uint32_t*)q_residual;
        } else {
            unsigned flags = hipHostMallocMapped | (g_opt.host_noncoherent ? hipHostMallocNonCoherent : 0u);
            e = hipHostMalloc(&c->residual_host, res_bytes, flags);
            if (e == hipSuccess) {
                memcpy(c->residual_host, q_residual, res_bytes);
                void* d = nullptr;
                e = hipHostGetDevicePointer(&d, c->residual_host, 0);
                c->residual_dev = (const uint32_t*)d;
            }
        }
    }
    // The owned copy of the scales is kept in output order (scale of output n at index n), so that the two
    // scales of an output pair arrive with one load: reordered_scales[j * N/8 + m] belongs to output 8 m + j.
    if (e == hipSuccess) e = hipMalloc(&c->scales_dev, sc_bytes);
    if (e == hipSuccess) {
        const size_t es = dtype_size(dtype);
        std::vector<unsigned char> in(sc_bytes), nat(sc_bytes);
        if (scales_on_device) e = hipMemcpy(in.data(), scales, sc_bytes, hipMemcpyDeviceToHost);
        else memcpy(in.data(), scales, sc_bytes);
        if (e == hipSuccess) {
            for (uint32_t j = 0; j < 8; ++j)
                for (uint32_t m = 0; m < c->M; ++m)
                    memcpy(&nat[((size_t)8 * m + j) * es], &in[((size_t)j * c->M + m) * es], es);
            e = hipMemcpy(c->scales_dev, nat.data(), sc_bytes, hipMemcpyHostToDevice);
        }
    }
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->e1, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->e2, hipEventDisableTiming);
    int rc = kOk;
    if (e != hipSuccess) rc = fail(kHipError, "HIP error in create_dec_config: %s", hipGetErrorString(e));
    if (rc == kOk) rc = setup_config(c, k_chunk);
    if (rc != kOk) {
        if (c->residual_host) (void)hipHostFree(c->residual_host);
        if (c->scales_dev) (void)hipFree(c->scales_dev);
        if (c->e1) (void)hipEventDestroy(c->e1);
        if (c->e2) (void)hipEventDestroy(c->e2);
        delete c;
        return rc;
    }
    {
        std::lock_guard<std::mutex> l(g_mu);
        g_configs.insert(reinterpret_cast<uint64_t>(c));
    }
    *out = reinterpret_cast<uint64_t>(c);
    return kOk;
}

int decdec_read_dec_config(uint64_t h, decdec_config_info* info) {
    Config* c = get_config(h);
    DD_CHECK(c != nullptr && info != nullptr, "invalid DECConfig handle");
    *info = c->info;
    return kOk;
}

int decdec_update_dec_config(uint64_t h, uint64_t new_ctx, uint32_t k_chunk) {
    Config* c = get_config(h);
    DD_CHECK(c != nullptr, "invalid DECConfig handle");
    Context* ctx = get_context(new_ctx);
    DD_CHECK(ctx != nullptr, "invalid DECContext handle");
    DD_CHECK(ctx->dt == c->dt, "Data type mismatch between DECConfig and DECContext.");
    Context* old = c->ctx;
    const uint32_t old_k = c->k_chunk;
    c->ctx = ctx;
    const int rc = setup_config(c, k_chunk);
    if (rc != kOk) {
        const std::string msg = g_error;
        c->ctx = old;
        (void)setup_config(c, old_k);
        g_error = msg;
        return rc;
    }
    return kOk;
}

int decdec_destroy_dec_config(uint64_t h) {
    Config* c = get_config(h);
    DD_CHECK(c != nullptr, "invalid DECConfig handle");
    {
        std::lock_guard<std::mutex> l(g_mu);
        g_configs.erase(h);
    }
    if (c->residual_host) (void)hipHostFree(c->residual_host);
    if (c->scales_dev) (void)hipFree(c->scales_dev);
    (void)hipEventDestroy(c->e1);
    (void)hipEventDestroy(c->e2);
    delete c;
    return kOk;
}

// ---------------------------------------------------------------- DEC
static int dec_common(uint64_t h, const void* input, void* output, int dtype, uint32_t K, uint32_t N,
                      void* stream, bool fused_select) {
    Config* c = get_config(h);
    int rc = check_dec_call(c, dtype, K, N, input, output);
    if (rc != kOk) return rc;
    DecParams p;
    const uint32_t nw = dec_block_threads() / kWave;
    if (fill_dec_params(c, input, output, fused_select, &p, nw)) return kOk;
    const DecPlan& plan = dec_plan(c, nw);
    LaunchDims d{plan.cg * plan.sg, nw * kWave, plan.lds};
    DD_HIP(launch_dec(dtype, p, d, (hipStream_t)stream));
    return kOk;
}

int decdec_dec(uint64_t h, const void* input, void* output, int dtype, uint32_t K, uint32_t N, void* stream) {
    return dec_common(h, input, output, dtype, K, N, stream, true);
}
int decdec_unfused_dec(uint64_t h, const void* input, void* output, int dtype, uint32_t K, uint32_t N, void* stream) {
    return dec_common(h, input, output, dtype, K, N, stream, false);
}

// ---------------------------------------------------------------- base GEMVs
int decdec_anyprec_gemv(const void* input, void* output, const void* qweight, const void* lut, int bits,
                        int dtype, uint32_t K, uint32_t N, void* stream) {
    AnyprecPlan pl;
    int rc = plan_anyprec(input, output, qweight, lut, bits, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    DD_HIP(launch_anyprec(dtype, bits, pl.p, pl.d, (hipStream_t)stream));
    return kOk;
}

int decdec_anyprec_dequant(const void* qweight, const void* lut, void* weight, int bits, int dtype,
                           uint32_t N, uint32_t K, void* stream) {
    DD_CHECK(bits >= 3 && bits <= 8, "Bitwidth must be between 3 and 8.");
    if (dtype == DECDEC_FP32)
        return fail(kUnsupported, "Any-Precision Dequantization does not support float data type. Please use half or bfloat16.");
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(qweight && lut && weight, "null pointer argument");
    DD_CHECK(K >= 32 && K % 32 == 0, "input_feat must be a positive multiple of 32, got %u", K);
    DD_HIP(launch_anyprec_dequant(dtype, bits, (const uint32_t*)qweight, lut, weight, N, K, (hipStream_t)stream));
    return kOk;
}

int decdec_lutgemm_gemv(const void* input, void* output, const void* qw, const void* alpha, const void* q_bias,
                        int bits, int group_size, int dtype, uint32_t K, uint32_t N, void* stream) {
    LutgemmPlan pl;
    int rc = plan_lutgemm(input, output, qw, alpha, q_bias, bits, group_size, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    DD_HIP(launch_lutgemm(dtype, pl.p, pl.d, (hipStream_t)stream));
    return kOk;
}

int decdec_sqllm_gemv(const void* input, void* output, const void* mat, const void* lut, int bits, int dtype,
                      uint32_t K, uint32_t N, void* stream) {
    SqllmPlan pl;
    int rc = plan_sqllm(input, output, mat, lut, bits, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    DD_HIP(launch_sqllm(dtype, pl.p, pl.d, (hipStream_t)stream));
    return kOk;
}

// ---------------------------------------------------------------- DEC + base GEMV
// Which instance of a fused kernel to launch: the one that lets two workgroups share a compute unit while the DEC
// role is not the longer one by a margin (a DEC workgroup that shares its unit takes about 1.2 us longer; the other
// instance halves the GEMV role's occupancy).  Estimates in microseconds: DEC = its latency floor (launch,
// activation load, selection, one host-link round trip, merge: about 8) plus the residual bytes at the zero-copy
// rate of the link (56 GB/s); GEMV = a start-up time plus the packed weight bytes at the rate the format's kernel
// sustains (fits of the standalone timings at the Llama-3 / Phi-3 shapes).  The ratio at which the choice flips was
// read off the cost of a launch inside a captured decode step, with either instance forced, cost over the GEMV in
// us at k_chunk 4 / 6 / 8 / 12 / 16 (shared unit | unit to itself):
//   any-precision 4096 -> 28672:  1.7 3.3 5.3 9.2 13.3 | 2.6 2.5 3.6 6.9 10.9      flips near DEC = 0.9 GEMV
//   SqueezeLLM 14336 -> 4096:     2.5 3.4 4.0 6.2 8.4  | 4.2 4.0 3.8 5.6 7.5       near 1.15
//   SqueezeLLM 4096 -> 28672:     2.4 4.1 6.2 10.0 14.1 | 6.5 6.6 6.8 8.8 9.7      near 1.1
//   LUT-GEMM 17920 -> 5120:       2.1 2.3 2.6 8.3 12.5 | 6.7 7.5 7.4 8.9 9.7       near 1.25
//   LUT-GEMM 5120 -> 35840:       1.4 1.9 3.1 3.4 7.2  | 11.0 11.5 12.3 15.5 17.6  beyond 1.27
enum GemvKind { kAnyprec = 0, kLutgemm = 1, kSqllm = 2 };

// The outputs of a batch are merged with atomic adds by different layers' workgroups at the same time: they must
// not overlap, not even partly (slices of one buffer are fine as long as their ranges are disjoint).
int check_batch_outputs(uint32_t n, void* const* outputs, const uint32_t* out_features, int dtype) {
    const size_t elem = dtype == DECDEC_FP32 ? 4 : 2;
    for (uint32_t i = 0; i < n; ++i) {
        DD_CHECK(outputs[i] != nullptr, "null pointer argument");
        const uintptr_t a0 = (uintptr_t)outputs[i], a1 = a0 + (size_t)out_features[i] * elem;
        for (uint32_t j = 0; j < i; ++j) {
            const uintptr_t b0 = (uintptr_t)outputs[j], b1 = b0 + (size_t)out_features[j] * elem;
            DD_CHECK(a1 <= b0 || b1 <= a0, "the outputs of layers %u and %u of a batch overlap", j, i);
        }
    }
    return kOk;
}

double dec_estimate_shape_us(uint32_t K, uint32_t N, uint32_t k_chunk, double bytes_per_us = kHostLinkBytesPerUs) {
    const double k = (double)((uint64_t)k_chunk * K / 1024u);              // selected rows per call
    return 8.0 + k * (double)N * 0.5 / bytes_per_us;
}
double dec_estimate_us(const Config* c) { return dec_estimate_shape_us(c->K, c->N, c->k_chunk, dec_residual_rate(c)); }
double gemv_estimate_us(GemvKind kind, double weight_bytes) {
    if (kind == kAnyprec) return 2.8 + weight_bytes / 3.7e6;
    if (kind == kSqllm) return 3.4 + weight_bytes / 4.6e6;
    return 4.2 + weight_bytes / 3.1e6;
}

bool fused_two_per_cu_at(double dec_us, GemvKind kind, double weight_bytes) {
    if (g_opt.fused_two_per_cu >= 0) return g_opt.fused_two_per_cu != 0;
    const double flip = kind == kAnyprec ? 0.9 : (kind == kSqllm ? 1.15 : 1.3);
    return dec_us < flip * gemv_estimate_us(kind, weight_bytes);
}
// Rate at which the launch-form rules price a layer's residual rows.  A device-resident residual makes the DEC role the
// short one for any-precision and LUT-GEMM launches at any k_chunk up to 32 (measured in the decode harness, residual
// in HBM: Phi-3 LUT-GEMM 284 tokens/s with the two-per-CU instance against 274 without); beside the SqueezeLLM GEMV its
// role still outlasts the GEMV at k_chunk 32 (8.5 us at 4096 -> 4096, 15.7 us at 14336 -> 4096: about 120 GB/s on top of
// the floor; Llama-3-8B SqueezeLLM, k_chunk 32 / 8: 468 / 479 tokens/s without the instance, 441 / 521 with it).
double dec_form_rate(const Config* c, GemvKind kind) {
    if (c->residual_host) return kHostLinkBytesPerUs;
    return kind == kSqllm ? 120e3 : kDeviceResidualBytesPerUs;
}
bool fused_two_per_cu(const Config* c, GemvKind kind, double weight_bytes) {
    return fused_two_per_cu_at(dec_estimate_shape_us(c->K, c->N, c->k_chunk, dec_form_rate(c, kind)), kind, weight_bytes);
}

// Whether a fused 3-bit any-precision launch runs both roles in workgroups of `nw` waves (the GEMV's standalone
// size).  Measured at 14336 -> 4096 (8 waves): 12.0 / 12.6 / 14.6 us against 13.3 / 16.4 / 15.9 us for the
// 1024-thread form at k_chunk 1 / 4 / 8, but 16.7 against 15.9 us at k_chunk 12 and 26.5 against 24.0 us at 32: a
// DEC workgroup's host-memory reads hold up the GEMV waves of its compute unit, and the small form spreads the DEC
// workgroups over four times as many units, so it only pays while the GEMV is the longer role.  Inside a decode step
// (14336 -> 4096, cost over the GEMV per launch) the small form measured 1.3 / 3.5 / 4.4 / 5.5 / 7.5 us at k_chunk
// 4 / 8 / 10 / 12 / 16 against 6.6 / 6.4 / 6.4 / 6.4 / 7.1 us: the switch sits where DEC is estimated at 1.7 x the
// GEMV (k_chunk 14 there).  With 4-wave workgroups (K <= 8192) the 1024-thread form was as fast or faster at every
// k_chunk.
bool fused_small_at(double dec_us, double gemv_bytes, uint32_t nw) {
    if (nw >= 16u || g_opt.fused_small == 0) return false;
    if (g_opt.fused_small > 0) return true;
    return nw == 8u && dec_us < 1.7 * gemv_estimate_us(kAnyprec, gemv_bytes);
}
bool fused_small(const Config* c, double gemv_bytes, uint32_t nw) { return fused_small_at(dec_estimate_us(c), gemv_bytes, nw); }

int decdec_fused_launch_form(int kind, int bits, uint32_t K, uint32_t N, uint32_t k_chunk, int* form_out) {
    DD_CHECK(form_out != nullptr, "form_out must not be null");
    DD_CHECK(kind >= 0 && kind <= 2, "kind must be 0 (any-precision), 1 (LUT-GEMM) or 2 (SqueezeLLM)");
    DD_CHECK(K >= 32 && K % 32 == 0 && N >= 1 && bits >= 1 && bits <= 8, "invalid shape");
    const double dec_us = dec_estimate_shape_us(K, N, k_chunk), bytes = (double)bits * N * K / 8.0;
    if (kind == kAnyprec && bits == 3 && g_opt.fused_small != 0) {
        // the workgroup size the standalone 3-bit kernel would use for this shape (plan_anyprec, four rows per wave)
        const uint32_t s_total = cdiv(K / 32u, 64u), sgroups = cdiv(s_total, 16u), S = cdiv(s_total, sgroups);
        const uint32_t block = 64u * S * std::max(1u, 4u / S);
        const uint32_t nw = block <= 256u ? 4u : (block <= 512u ? 8u : 16u);
        if (fused_small_at(dec_us, bytes, nw)) { *form_out = 2; return kOk; }
    }
    const bool two = (kind != kAnyprec || bits == 3) && fused_two_per_cu_at(dec_us, (GemvKind)kind, bytes);
    *form_out = two ? 1 : 0;
    return kOk;
}

int decdec_dec_anyprec(uint64_t h, const void* input, void* output, const void* qweight, const void* lut,
                       int bits, int dtype, uint32_t K, uint32_t N, void* stream) {
    Config* c = get_config(h);
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    int rc = check_dec_call(c, dtype, K, N, input, output);
    if (rc != kOk) return rc;
    DecParams dp;
    const bool have_dec = fill_dec_params(c, input, output, true, &dp) == 0;
    const bool fuse = g_opt.fusion && have_dec;
    AnyprecPlan pl;
    const bool two = fuse && bits == 3 && fused_two_per_cu(c, kAnyprec, (double)bits * N * K / 8.0);
    hipStream_t s = (hipStream_t)stream;
    if (fuse && bits == 3 && g_opt.fused_small != 0) {
        // Both roles in workgroups of the GEMV's own size (4 or 8 waves): the GEMV keeps its standalone
        // schedule and a DEC workgroup holds an eighth or a quarter of a compute unit instead of a half.
        // four rows per wave: beside DEC workgroups twice as many, shorter GEMV workgroups measured 1 us faster
        // (14336 -> 4096: 11.0 / 11.4 / 13.5 us against 12.0 / 12.6 / 14.6 us at k_chunk 1 / 4 / 8) although the
        // GEMV alone is slower that way (10.2 against 9.6 us)
        rc = plan_anyprec(input, output, qweight, lut, bits, dtype, K, N, false, &pl, 4u);
        if (rc != kOk) return rc;
        const uint32_t nw = pl.d.block <= 256u ? 4u : (pl.d.block <= 512u ? 8u : 16u);
        if (pl.p.tile_cs == 0u && fused_small(c, (double)bits * N * K / 8.0, nw)) {
            (void)fill_dec_params(c, input, output, true, &dp, nw);
            const DecPlan& plan = dec_plan(c, nw);
            LaunchDims d = pl.d;
            d.block = nw * kWave;
            d.lds = std::max(d.lds, plan.lds);
            DD_HIP(launch_dec_anyprec_small(dtype, nw, dp, plan.cg * plan.sg, pl.p, d, s));
            return kOk;
        }
    }
    rc = plan_anyprec(input, output, qweight, lut, bits, dtype, K, N, fuse, &pl);
    if (rc != kOk) return rc;
    if (fuse) {
        LaunchDims d = pl.d;
        d.lds = std::max(d.lds, c->plans[2].lds);
        d.two_per_cu = two;
        DD_HIP(launch_dec_anyprec(dtype, bits, dp, c->plans[2].cg * c->plans[2].sg, pl.p, d, s));
        return kOk;
    }
    if (!have_dec && g_opt.fusion) { DD_HIP(launch_anyprec(dtype, bits, pl.p, pl.d, s)); return kOk; }
    return two_stream(c, &dp, have_dec, dtype, s,
                      [&](hipStream_t sub) { return launch_anyprec(dtype, bits, pl.p, pl.d, sub); });
}

// Several any-precision layers that read the same input, in one launch (q | k | v, gate | up).  A layer whose config
// handle is 0, or whose config has k_chunk 0, runs its base GEMV only.
int decdec_dec_anyprec_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                             const void* const* qweights, const void* const* luts, int bits, int dtype, uint32_t K,
                             const uint32_t* out_features, void* stream) {
    DD_CHECK(n >= 1 && n <= (uint32_t)kMaxBatch, "a batch holds 1 to %d layers, got %u", kMaxBatch, n);
    DD_CHECK(outputs && qweights && luts && out_features, "null pointer argument");
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    { const int rc_out = check_batch_outputs(n, outputs, out_features, dtype); if (rc_out != kOk) return rc_out; }
    if (!g_opt.fusion || (bits != 3 && bits != 4)) {
        // no batched kernel for this case: one call per layer, same result
        for (uint32_t i = 0; i < n; ++i) {
            const int rc = (configs && configs[i])
                ? decdec_dec_anyprec(configs[i], input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], stream)
                : decdec_anyprec_gemv(input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], stream);
            if (rc != kOk) return rc;
        }
        return kOk;
    }
    // no DEC on any layer (no config, or k_chunk 0 everywhere): the GEMVs in their standalone workgroups, which run a
    // batch faster than the 1024-thread workgroups of the fused kernel (gate | up at 4096 -> 14336: 13.5 against 17.3 us)
    bool want_dec = false;
    for (uint32_t i = 0; i < n && configs; ++i) {
        if (!configs[i]) continue;
        Config* c = get_config(configs[i]);
        int rc = check_dec_call(c, dtype, K, out_features[i], input, outputs[i]);
        if (rc != kOk) return rc;
        want_dec = want_dec || (uint64_t)c->k_chunk * c->K / 1024u > 0;
    }
    if (!want_dec) {
        GemvBatchParams<AnyprecParams> gb;
        memset(&gb, 0, sizeof(gb));
        gb.n = n;
        LaunchDims gd{0, 0, 0};
        uint32_t total = 0;
        uint64_t rows = 0;
        for (uint32_t i = 0; i < n; ++i) rows += out_features[i];
        for (uint32_t i = 0; i < n; ++i) {
            AnyprecPlan pl;
            int rc = plan_anyprec(input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], false, &pl, 8, rows);
            if (rc != kOk) return rc;
            if (pl.p.tile_cs != 0u) { want_dec = true; break; }      // the tile decoder plans its own workgroups: fused form below
            DD_CHECK(gd.block == 0 || gd.block == pl.d.block, "internal: layers of a batch planned different workgroups");
            gb.gp[i] = pl.p;
            gd.block = pl.d.block;
            gd.lds = std::max(gd.lds, pl.d.lds);
            total += pl.d.grid;
            gb.gemv_end[i] = total;
        }
        if (!want_dec) {
            for (uint32_t i = n; i < (uint32_t)kMaxBatch; ++i) gb.gemv_end[i] = total;
            gd.grid = total;
            DD_HIP(launch_anyprec_batch(dtype, bits, gb, gd, (hipStream_t)stream));
            return kOk;
        }
    }
    BatchParams<AnyprecParams> b;
    memset(&b, 0, sizeof(b));
    b.n = n;
    LaunchDims d{0, 1024u, 0};
    uint32_t dec_total = 0, gemv_total = 0;
    double dec_us = 0.0, weight_bytes = 0.0;
    bool any_dec = false;
    uint64_t batch_rows = 0, dec_rows = 0;
    double batch_link_us = 0.0;
    for (uint32_t i = 0; i < n; ++i) {
        batch_rows += out_features[i];
        if (configs && configs[i]) {
            const Config* c = get_config(configs[i]);
            if (c && (uint64_t)c->k_chunk * c->K / 1024u > 0) {
                dec_rows += out_features[i];
                batch_link_us += (double)((uint64_t)c->k_chunk * c->K / 1024u) * (double)c->N * 0.5 / dec_residual_rate(c);
            }
        }
    }
    for (uint32_t i = 0; i < n; ++i) {
        Config* c = (configs && configs[i]) ? get_config(configs[i]) : nullptr;
        bool have_dec = false;
        DecPlan dplan{};
        if (configs && configs[i]) {
            int rc = check_dec_call(c, dtype, K, out_features[i], input, outputs[i]);
            if (rc != kOk) return rc;
            DD_CHECK(plan_dec_in_batch(c, dec_rows, &dplan) == 0, "internal: no DEC plan for a layer of the batch");
            have_dec = fill_dec_params(c, input, outputs[i], true, &b.dp[i], kDecWaves, &dplan, batch_link_us) == 0;
            b.dp[i].trace = nullptr;                      // the phase stamps are indexed by workgroup of a single-layer launch
        }
        AnyprecPlan pl;
        int rc = plan_anyprec(input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], true, &pl, 8, batch_rows);
        if (rc != kOk) return rc;
        b.gp[i] = pl.p;
        d.lds = std::max(d.lds, pl.d.lds);
        if (have_dec) {
            dec_total += dplan.cg * dplan.sg;
            d.lds = std::max(d.lds, dplan.lds);
            dec_us += (double)((uint64_t)c->k_chunk * c->K / 1024u) * (double)c->N * 0.5 / dec_residual_rate(c);
            any_dec = true;
        }
        gemv_total += pl.d.grid;
        weight_bytes += (double)bits * out_features[i] * K / 8.0;
        b.dec_end[i] = dec_total;
        b.gemv_end[i] = gemv_total;
    }
    for (uint32_t i = n; i < (uint32_t)kMaxBatch; ++i) { b.dec_end[i] = dec_total; b.gemv_end[i] = gemv_total; }
    d.grid = dec_total + gemv_total;
    // two workgroups per compute unit while the DEC roles together (one latency floor, the bytes of all layers) are
    // not the longer part by a margin -- the single-layer rule applied to the batch
    if (g_opt.fused_two_per_cu >= 0) d.two_per_cu = g_opt.fused_two_per_cu != 0;
    else d.two_per_cu = !any_dec || (8.0 + dec_us) < 0.9 * gemv_estimate_us(kAnyprec, weight_bytes);
    DD_HIP(launch_dec_anyprec_batch(dtype, bits, b, d, (hipStream_t)stream));
    return kOk;
}

int decdec_dec_lutgemm(uint64_t h, const void* input, void* output, const void* qw, const void* alpha,
                       const void* q_bias, int bits, int group_size, int dtype, uint32_t K, uint32_t N,
                       void* stream) {
    Config* c = get_config(h);
    int rc = check_dec_call(c, dtype, K, N, input, output);
    if (rc != kOk) return rc;
    DecParams dp;
    const bool have_dec = fill_dec_params(c, input, output, true, &dp) == 0;
    const bool fuse = g_opt.fusion && have_dec;
    LutgemmPlan pl;
    rc = plan_lutgemm(input, output, qw, alpha, q_bias, bits, group_size, dtype, K, N, fuse, &pl);
    if (rc != kOk) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (fuse) {
        LaunchDims d = pl.d;
        d.lds = std::max(d.lds, c->plans[2].lds);
        d.two_per_cu = fused_two_per_cu(c, kLutgemm, (double)bits * N * K / 8.0);
        DD_HIP(launch_dec_lutgemm(dtype, dp, c->plans[2].cg * c->plans[2].sg, pl.p, d, s));
        return kOk;
    }
    if (!have_dec && g_opt.fusion) { DD_HIP(launch_lutgemm(dtype, pl.p, pl.d, s)); return kOk; }
    return two_stream(c, &dp, have_dec, dtype, s, [&](hipStream_t sub) { return launch_lutgemm(dtype, pl.p, pl.d, sub); });
}

int decdec_dec_sqllm(uint64_t h, const void* input, void* output, const void* mat, const void* lut, int bits,
                     int dtype, uint32_t K, uint32_t N, void* stream) {
    Config* c = get_config(h);
    int rc = check_dec_call(c, dtype, K, N, input, output);
    if (rc != kOk) return rc;
    DecParams dp;
    const bool have_dec = fill_dec_params(c, input, output, true, &dp) == 0;
    const bool fuse = g_opt.fusion && have_dec;
    SqllmPlan pl;
    rc = plan_sqllm(input, output, mat, lut, bits, dtype, K, N, fuse, &pl);
    if (rc != kOk) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (fuse) {
        LaunchDims d = pl.d;
        d.lds = std::max(d.lds, c->plans[2].lds);
        d.two_per_cu = fused_two_per_cu(c, kSqllm, (double)bits * N * K / 8.0);
        DD_HIP(launch_dec_sqllm(dtype, dp, c->plans[2].cg * c->plans[2].sg, pl.p, d, s));
        return kOk;
    }
    if (!have_dec && g_opt.fusion) { DD_HIP(launch_sqllm(dtype, pl.p, pl.d, s)); return kOk; }
    return two_stream(c, &dp, have_dec, dtype, s, [&](hipStream_t sub) { return launch_sqllm(dtype, pl.p, pl.d, sub); });
}

// Batches of LUT-GEMM / SqueezeLLM layers on one input (the any-precision batch above, for the other two formats).
// `plan(i, &params, &dims)` plans layer i's GEMV role for a 1024-thread workgroup, `single(i, have_config)` runs layer i
// alone (the path without a batched kernel: fusion off, fp32).
extern "C++" {
template <typename GemvParams, typename Plan, typename Single, typename Launch>
int batch_common(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs, int dtype, uint32_t K,
                 const uint32_t* out_features, GemvKind kind, double bytes_per_weight, bool batched_kernel,
                 Plan plan, Single single, Launch launch) {
    DD_CHECK(n >= 1 && n <= (uint32_t)kMaxBatch, "a batch holds 1 to %d layers, got %u", kMaxBatch, n);
    DD_CHECK(outputs && out_features, "null pointer argument");
    DD_CHECK(dtype_ok(dtype), "Unsupported data type.");
    { const int rc_out = check_batch_outputs(n, outputs, out_features, dtype); if (rc_out != kOk) return rc_out; }
    if (!g_opt.fusion || !batched_kernel) {
        for (uint32_t i = 0; i < n; ++i) {
            const int rc = single(i, configs != nullptr && configs[i] != 0);
            if (rc != kOk) return rc;
        }
        return kOk;
    }
    BatchParams<GemvParams> b;
    memset(&b, 0, sizeof(b));
    b.n = n;
    LaunchDims d{0, 1024u, 0};
    uint32_t dec_total = 0, gemv_total = 0;
    double dec_us = 0.0, weight_bytes = 0.0;
    bool any_dec = false;
    uint64_t dec_rows = 0;
    double batch_link_us = 0.0;
    for (uint32_t i = 0; i < n; ++i) {
        if (configs && configs[i]) {
            const Config* c = get_config(configs[i]);
            if (c && (uint64_t)c->k_chunk * c->K / 1024u > 0) {
                dec_rows += out_features[i];
                batch_link_us += (double)((uint64_t)c->k_chunk * c->K / 1024u) * (double)c->N * 0.5 / dec_residual_rate(c);
            }
        }
    }
    for (uint32_t i = 0; i < n; ++i) {
        Config* c = (configs && configs[i]) ? get_config(configs[i]) : nullptr;
        bool have_dec = false;
        DecPlan dplan{};
        if (configs && configs[i]) {
            int rc = check_dec_call(c, dtype, K, out_features[i], input, outputs[i]);
            if (rc != kOk) return rc;
            DD_CHECK(plan_dec_in_batch(c, dec_rows, &dplan) == 0, "internal: no DEC plan for a layer of the batch");
            have_dec = fill_dec_params(c, input, outputs[i], true, &b.dp[i], kDecWaves, &dplan, batch_link_us) == 0;
            b.dp[i].trace = nullptr;                      // the phase stamps are indexed by workgroup of a single-layer launch
        }
        LaunchDims ld{0, 0, 0};
        int rc = plan(i, &b.gp[i], &ld);
        if (rc != kOk) return rc;
        DD_CHECK(ld.block == 1024u, "internal: batched layers need 1024-thread workgroups");
        d.lds = std::max(d.lds, ld.lds);
        if (have_dec) {
            dec_total += dplan.cg * dplan.sg;
            d.lds = std::max(d.lds, dplan.lds);
            dec_us += (double)((uint64_t)c->k_chunk * c->K / 1024u) * (double)c->N * 0.5 / dec_form_rate(c, kind);
            any_dec = true;
        }
        gemv_total += ld.grid;
        weight_bytes += bytes_per_weight * out_features[i] * K;
        b.dec_end[i] = dec_total;
        b.gemv_end[i] = gemv_total;
    }
    for (uint32_t i = n; i < (uint32_t)kMaxBatch; ++i) { b.dec_end[i] = dec_total; b.gemv_end[i] = gemv_total; }
    d.grid = dec_total + gemv_total;
    const double flip = kind == kSqllm ? 1.15 : 1.3;      // the single-layer rule (fused_two_per_cu) applied to the batch
    if (g_opt.fused_two_per_cu >= 0) d.two_per_cu = g_opt.fused_two_per_cu != 0;
    else d.two_per_cu = !any_dec || (8.0 + dec_us) < flip * gemv_estimate_us(kind, weight_bytes);
    DD_HIP(launch(b, d));
    return kOk;
}
}  // extern "C++"

int decdec_dec_lutgemm_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                             const void* const* q_weights, const void* const* alphas, const void* const* q_biases,
                             int bits, int group_size, int dtype, uint32_t K, const uint32_t* out_features, void* stream) {
    DD_CHECK(q_weights && alphas && q_biases, "null pointer argument");
    hipStream_t s = (hipStream_t)stream;
    return batch_common<LutgemmParams>(
        n, configs, input, outputs, dtype, K, out_features, kLutgemm, bits / 8.0, dtype != DECDEC_FP32,
        [&](uint32_t i, LutgemmParams* gp, LaunchDims* ld) {
            LutgemmPlan pl;
            // the layers of a batch share the device in proportion to their widths
            uint64_t total = 0;
            for (uint32_t j = 0; j < n; ++j) total += out_features[j];
            const uint32_t share = (uint32_t)std::max<uint64_t>(32u, (uint64_t)2u * device_cus() * out_features[i] / std::max<uint64_t>(total, 1));
            const int rc = plan_lutgemm(input, outputs[i], q_weights[i], alphas[i], q_biases[i], bits, group_size, dtype, K,
                                        out_features[i], true, &pl, share);
            *gp = pl.p; *ld = pl.d;
            return rc;
        },
        [&](uint32_t i, bool have_config) {
            return have_config ? decdec_dec_lutgemm(configs[i], input, outputs[i], q_weights[i], alphas[i], q_biases[i], bits,
                                                    group_size, dtype, K, out_features[i], stream)
                               : decdec_lutgemm_gemv(input, outputs[i], q_weights[i], alphas[i], q_biases[i], bits, group_size,
                                                     dtype, K, out_features[i], stream);
        },
        [&](const BatchParams<LutgemmParams>& b, const LaunchDims& d) { return launch_dec_lutgemm_batch(dtype, b, d, s); });
}

int decdec_dec_sqllm_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                           const void* const* qweights, const void* const* luts, int bits, int dtype, uint32_t K,
                           const uint32_t* out_features, void* stream) {
    DD_CHECK(qweights && luts, "null pointer argument");
    hipStream_t s = (hipStream_t)stream;
    return batch_common<SqllmParams>(
        n, configs, input, outputs, dtype, K, out_features, kSqllm, bits / 8.0, dtype != DECDEC_FP32,
        [&](uint32_t i, SqllmParams* gp, LaunchDims* ld) {
            SqllmPlan pl;
            const int rc = plan_sqllm(input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], true, &pl);
            *gp = pl.p; *ld = pl.d;
            return rc;
        },
        [&](uint32_t i, bool have_config) {
            return have_config ? decdec_dec_sqllm(configs[i], input, outputs[i], qweights[i], luts[i], bits, dtype, K,
                                                  out_features[i], stream)
                               : decdec_sqllm_gemv(input, outputs[i], qweights[i], luts[i], bits, dtype, K, out_features[i], stream);
        },
        [&](const BatchParams<SqllmParams>& b, const LaunchDims& d) { return launch_dec_sqllm_batch(dtype, b, d, s); });
}

// ---------------------------------------------------------------- dummies
int decdec_dummy_anyprec(const void* input, void* output, const void* qweight, const void* lut, int bits,
                         int dtype, uint32_t K, uint32_t N, int dummy_cu, int64_t iters, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "dummy_anyprec supports FP16/BF16 only.");
    AnyprecPlan pl;
    int rc = plan_anyprec(input, output, qweight, lut, bits, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    return dummy_common(dummy_cu, iters, (hipStream_t)stream,
                        [&](hipStream_t sub) { return launch_anyprec(dtype, bits, pl.p, pl.d, sub); });
}

int decdec_dummy_lutgemm(const void* input, void* output, const void* qw, const void* alpha, const void* q_bias,
                         int bits, int group_size, int dtype, uint32_t K, uint32_t N, int dummy_cu,
                         int64_t iters, void* stream) {
    LutgemmPlan pl;
    int rc = plan_lutgemm(input, output, qw, alpha, q_bias, bits, group_size, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    return dummy_common(dummy_cu, iters, (hipStream_t)stream,
                        [&](hipStream_t sub) { return launch_lutgemm(dtype, pl.p, pl.d, sub); });
}

int decdec_dummy_sqllm(const void* input, void* output, const void* mat, const void* lut, int bits, int dtype,
                       uint32_t K, uint32_t N, int dummy_cu, int64_t iters, void* stream) {
    DD_CHECK(bits == 3 || bits == 4, "SQLLM bitwidth must be 3 or 4.");
    SqllmPlan pl;
    int rc = plan_sqllm(input, output, mat, lut, bits, dtype, K, N, false, &pl);
    if (rc != kOk) return rc;
    return dummy_common(dummy_cu, iters, (hipStream_t)stream,
                        [&](hipStream_t sub) { return launch_sqllm(dtype, pl.p, pl.d, sub); });
}

// ---------------------------------------------------------------- decode-step helpers
// Workspace layout: [n_head] arrival counters (u32, zero between calls), then [n_head][nsplit][head_dim + 2] floats.
uint64_t decdec_decode_attention_workspace_bytes(uint32_t n_head, uint32_t head_dim, uint32_t nsplit) {
    return (uint64_t)n_head * 4u + (uint64_t)n_head * nsplit * (head_dim + 2) * 4u;
}

// Workgroups per query head of the decode attention: as many as the workspace allows, up to 8, without asking for
// more workgroups than the device has compute units (40 heads x 8 would run in two turns: 6 each).
static uint32_t attention_splits(uint32_t n_head, uint32_t head_dim, uint64_t workspace_bytes) {
    const uint32_t cus = device_cus();
    for (uint32_t n = 8; n > 1; --n) {
        if (n_head * n > cus && n > 2) continue;
        if (decdec_decode_attention_workspace_bytes(n_head, head_dim, n) <= workspace_bytes) return n;
    }
    return 1;
}

int decdec_rope_cache_update(const void* qkv, const void* cos_table, const void* sin_table, const int64_t* pos_device,
                             void* q_out, void* k_cache, void* v_cache, int dtype, uint32_t n_head,
                             uint32_t n_kv_head, uint32_t head_dim, uint32_t max_seq, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(qkv && cos_table && sin_table && pos_device && q_out && k_cache && v_cache, "null pointer argument");
    DD_CHECK(n_head >= 1 && n_kv_head >= 1 && n_head % n_kv_head == 0, "n_head must be a multiple of n_kv_head");
    DD_CHECK(head_dim >= 2 && head_dim % 2 == 0 && max_seq >= 1, "head_dim must be even and max_seq positive");
    RopeCacheParams p{qkv, cos_table, sin_table, (const long long*)pos_device, q_out, k_cache, v_cache,
                      n_head, n_kv_head, head_dim, max_seq};
    DD_HIP(launch_rope_cache(dtype, p, (hipStream_t)stream));
    return kOk;
}

// Argument checks of the decode attention entry points, and the number of workgroups that share a head (1: no
// workspace in use).  Nothing is enqueued here.
static int decode_attention_check(const void* q, const void* k_cache, const void* v_cache, const int64_t* pos_device,
                                  void* out, int dtype, uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim,
                                  uint32_t max_seq, void* workspace, uint64_t workspace_bytes, uint32_t* nsplit_out) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(q && k_cache && v_cache && pos_device && out, "null pointer argument");
    DD_CHECK(n_head >= 1 && n_kv_head >= 1 && n_head % n_kv_head == 0, "n_head must be a multiple of n_kv_head");
    DD_CHECK(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128, got %u", head_dim);
    DD_CHECK(max_seq >= 1, "max_seq must be positive");
    DD_CHECK(((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0, "caches must be 16-byte aligned");
    DD_CHECK(((uintptr_t)q % 4) == 0, "q must be 4-byte aligned");
    // as many workgroups per head as the workspace allows, up to 8 (256 workgroups at 32 heads)
    uint32_t nsplit = 1;
    if (workspace != nullptr && max_seq > 256) {
        DD_CHECK(((uintptr_t)workspace % 4) == 0, "workspace must be 4-byte aligned");
        nsplit = attention_splits(n_head, head_dim, workspace_bytes);
    }
    *nsplit_out = nsplit;
    return kOk;
}

static int decode_attention_launch(const void* q, const void* k_cache, const void* v_cache, const int64_t* pos_device,
                                   void* out, int dtype, uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim,
                                   uint32_t max_seq, void* workspace, uint32_t nsplit, void* stream) {
    AttentionParams p{q, k_cache, v_cache, (const long long*)pos_device, out, n_head, n_kv_head, head_dim, max_seq,
                      1.0f / std::sqrt((float)head_dim), nsplit, nsplit > 1 ? (float*)workspace + n_head : nullptr,
                      nullptr, nullptr, nullptr,
                      (nsplit > 1 && g_opt.attention_two_step == 0) ? (uint32_t*)workspace : nullptr,
                      (uint32_t)std::max(0, g_opt.attention_single_below)};
    DD_HIP(launch_decode_attention(dtype, p, (hipStream_t)stream));
    return kOk;
}

int decdec_decode_attention(const void* q, const void* k_cache, const void* v_cache, const int64_t* pos_device,
                            void* out, int dtype, uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim,
                            uint32_t max_seq, void* workspace, uint64_t workspace_bytes, void* stream) {
    uint32_t nsplit = 1;
    int rc = decode_attention_check(q, k_cache, v_cache, pos_device, out, dtype, n_head, n_kv_head, head_dim, max_seq,
                                    workspace, workspace_bytes, &nsplit);
    if (rc != kOk) return rc;
    return decode_attention_launch(q, k_cache, v_cache, pos_device, out, dtype, n_head, n_kv_head, head_dim, max_seq,
                                   workspace, nsplit, stream);
}

int decdec_decode_attention_static(const void* q, const void* k_cache, const void* v_cache, const int64_t* pos_device,
                                   void* out, int dtype, uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim,
                                   uint32_t max_seq, void* stream) {
    DD_CHECK(n_head <= kStaticHeads, "decdec_decode_attention_static: n_head %u exceeds the limit of %u heads", n_head,
             kStaticHeads);
    DD_CHECK(head_dim <= kStaticHeadDim, "decdec_decode_attention_static: head_dim %u exceeds the limit of %u", head_dim,
             kStaticHeadDim);
    void* ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc != kOk) return rc;
    // every argument is checked before anything is enqueued (the caller's stream may be under capture)
    uint32_t nsplit = 1;
    rc = decode_attention_check(q, k_cache, v_cache, pos_device, out, dtype, n_head, n_kv_head, head_dim, max_seq, ws,
                                kStaticScratchBytes, &nsplit);
    if (rc != kOk) return rc;
    // The array keeps what the last call left.  Every call leaves the arrival counters at zero; clearing the ones
    // this call uses makes that independent of what ran before (a fill kernel, not a memset node: safe under
    // capture).  They are used only when the heads are shared and merged in the kernel.
    if (nsplit > 1 && g_opt.attention_two_step == 0) {
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(128), 0, (hipStream_t)stream, (uint32_t*)ws, n_head, 0u);
        DD_HIP(hipGetLastError());
    }
    return decode_attention_launch(q, k_cache, v_cache, pos_device, out, dtype, n_head, n_kv_head, head_dim, max_seq, ws,
                                   nsplit, stream);
}

int decdec_rope_attention(const void* qkv, const void* cos_table, const void* sin_table, const int64_t* pos_device,
                          void* out, void* k_cache, void* v_cache, int dtype, uint32_t n_head, uint32_t n_kv_head,
                          uint32_t head_dim, uint32_t max_seq, void* workspace, uint64_t workspace_bytes, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(qkv && cos_table && sin_table && k_cache && v_cache && pos_device && out, "null pointer argument");
    DD_CHECK(n_head >= 1 && n_kv_head >= 1 && n_head % n_kv_head == 0, "n_head must be a multiple of n_kv_head");
    DD_CHECK(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128, got %u", head_dim);
    DD_CHECK(max_seq >= 1, "max_seq must be positive");
    DD_CHECK(((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0 && ((uintptr_t)qkv % 16) == 0 &&
             ((uintptr_t)cos_table % 16) == 0 && ((uintptr_t)sin_table % 16) == 0,
             "qkv, the tables and the caches must be 16-byte aligned");
    uint32_t nsplit = 1;
    if (workspace != nullptr && max_seq > 256) {
        DD_CHECK(((uintptr_t)workspace % 4) == 0, "workspace must be 4-byte aligned");
        nsplit = attention_splits(n_head, head_dim, workspace_bytes);
    }
    AttentionParams p{nullptr, k_cache, v_cache, (const long long*)pos_device, out, n_head, n_kv_head, head_dim, max_seq,
                      1.0f / std::sqrt((float)head_dim), nsplit, nsplit > 1 ? (float*)workspace + n_head : nullptr,
                      qkv, cos_table, sin_table,
                      (nsplit > 1 && g_opt.attention_two_step == 0) ? (uint32_t*)workspace : nullptr,
                      (uint32_t)std::max(0, g_opt.attention_single_below)};
    DD_HIP(launch_decode_attention(dtype, p, (hipStream_t)stream));
    return kOk;
}

int decdec_dense_gemv(const void* weight, const void* x, void* out, int dtype, uint32_t N, uint32_t K, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(weight && x && out, "null pointer argument");
    DD_CHECK(K >= 8 && K % 8 == 0, "in_features must be a positive multiple of 8, got %u", K);
    DD_CHECK(((uintptr_t)weight % 16) == 0 && ((uintptr_t)x % 16) == 0, "weight and x must be 16-byte aligned");
    if (N == 0) return kOk;
    DD_HIP(launch_dense_gemv(dtype, weight, x, out, N, K, (hipStream_t)stream));
    return kOk;
}

int decdec_silu_mul(const void* gate_up, void* out, int dtype, uint32_t n, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(gate_up && out, "null pointer argument");
    if (n == 0) return kOk;
    DD_HIP(launch_silu_mul(dtype, gate_up, out, n, (hipStream_t)stream));
    return kOk;
}

uint64_t decdec_greedy_pick_workspace_bytes(void) { return (uint64_t)greedy_pick_workspace_bytes(); }

int decdec_greedy_pick(const void* logits, uint32_t n, int dtype, void* workspace, float* logits_f32_out,
                       int64_t* token, int64_t* seq, uint32_t seq_capacity, int64_t* count, int64_t* pos, void* stream) {
    DD_CHECK(dtype_ok(dtype), "Unsupported data type.");
    DD_CHECK(logits && workspace && token, "null pointer argument");
    DD_CHECK(n >= 1, "there must be at least one logit");
    DD_CHECK((seq == nullptr) == (count == nullptr), "seq and count go together");
    DD_CHECK(((uintptr_t)workspace % 8) == 0, "workspace must be 8-byte aligned");
    DD_HIP(launch_greedy_pick(dtype, logits, n, workspace, logits_f32_out, (long long*)token, (long long*)seq,
                              seq_capacity, (long long*)count, (long long*)pos, (hipStream_t)stream));
    return kOk;
}

int decdec_add_rmsnorm(const void* x, const void* y, const void* weight, void* h_out, void* normed_out, int dtype,
                       uint32_t rows, uint32_t dim, float eps, void* stream) {
    DD_CHECK(dtype == DECDEC_FP16 || dtype == DECDEC_BF16, "Unsupported data type.");
    DD_CHECK(x && weight && normed_out, "null pointer argument");
    DD_CHECK(dim >= 4 && dim % 4 == 0 && dim <= 16384, "dim must be a multiple of 4 up to 16384, got %u", dim);
    DD_CHECK(((uintptr_t)x % 8) == 0 && ((uintptr_t)weight % 8) == 0 && ((uintptr_t)normed_out % 8) == 0 &&
             ((uintptr_t)y % 8) == 0 && ((uintptr_t)h_out % 8) == 0, "tensors must be 8-byte aligned");
    if (rows == 0) return kOk;
    DD_HIP(launch_add_rmsnorm(dtype, x, y, weight, h_out, normed_out, rows, dim, eps, (hipStream_t)stream));
    return kOk;
}

}  // extern "C"
