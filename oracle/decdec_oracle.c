/*
 * CPU oracle for DecDEC's decode-time linear-layer path -- plain C restatement.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/_build/libdecdec_oracle.so and loaded by
 * tests, the smoke check and the cpu_baseline leg of the benchmark.  The product library
 * never links or loads it.
 *
 * Written independently of the NumPy oracle (own soft-float conversions, scalar loops that
 * follow the kernels' loop structure) so that the two can be compared bit for bit on the
 * integer / fp16-threshold part and to 1e-12 on the float64 sums.
 *
 * Reference text followed (paths relative to the reference checkout):
 *   dd_bucket_floors   decdec_extension/dec.cu:117-137
 *   dd_select          decdec_extension/dec.cu:78-182, decdec.cu:48-67
 *   dd_dec_apply       decdec_extension/dec.cu:186-279
 *   dd_anyprec_gemv    decdec_extension/anyprec.cu:344-514 (load addresses :427, :467)
 *   dd_lutgemm_gemv    decdec_extension/lutgemm.cu:25-150
 *   dd_sqllm_gemv      decdec_extension/sqllm.cu:28-169
 *
 * dtype codes: 0 = fp32 (values passed as float bit patterns in uint32), 1 = fp16,
 * 2 = bf16 (both passed as uint16 bit patterns).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CHUNK 1024
#define NBUCKET 32

/* ---------------------------------------------------------------- soft float */
static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float half_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1F;
    uint32_t man = h & 0x3FF;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112) << 23) | (man << 13));
}

/* round-to-nearest-even float32 -> fp16 */
static uint16_t f32_to_half(float f) {
    uint32_t u = f32_to_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7FFFFFFFu;
    if (absu >= 0x7F800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absu > 0x7F800000u) ? 0x200u : 0));
    }
    if (absu >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);   /* >= 65520 rounds to inf */
    if (absu < 0x33000001u) return (uint16_t)sign;   /* <= 2^-25 rounds to zero (tie -> even 0) */
    int32_t e = (int32_t)(absu >> 23) - 127;
    uint32_t m = (absu & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
    int shift;
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }            /* subnormal half */
    else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));            /* carry into the exponent is correct */
}

static float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }
static uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

/* value of element i of a typed array as float */
static float load_f(const void *p, int dtype, size_t i) {
    if (dtype == 0) return ((const float *)p)[i];
    if (dtype == 1) return half_to_f32(((const uint16_t *)p)[i]);
    return bf16_to_f32(((const uint16_t *)p)[i]);
}
/* round a float to the dtype and return it as float */
static float round_t(float v, int dtype) {
    if (dtype == 0) return v;
    if (dtype == 1) return half_to_f32(f32_to_half(v));
    return bf16_to_f32(f32_to_bf16(v));
}

uint16_t dd_f32_to_half(float f) { return f32_to_half(f); }
float dd_half_to_f32(uint16_t h) { return half_to_f32(h); }
uint16_t dd_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* ---------------------------------------------------------------- A1 floors */
/* dec.cu:117-130.  a, b already hold values of the dtype.  floors_out[32] as float. */
void dd_bucket_floors(float a, float b, int dtype, float *floors_out) {
    volatile float diff = round_t(b - a, dtype);            /* T(b - a): one rounding */
    for (int idx = 0; idx < NBUCKET; idx++) {
        if (idx < NBUCKET / 2) {
            volatile float prod = diff * (float)idx;        /* float * uint -> float */
            volatile float quo = prod / (float)(NBUCKET / 2 - 1);
            volatile float step = round_t(quo, dtype);      /* TO_DTYPE(...) */
            floors_out[idx] = round_t(a + step, dtype);     /* typed add */
        } else {
            volatile float prod = b * (float)(NBUCKET - idx - 1);
            volatile float quo = prod / (float)(NBUCKET - NBUCKET / 2);
            floors_out[idx] = round_t(quo, dtype);
        }
    }
}

/* ---------------------------------------------------------------- A1 select */
/*
 * rows_out / acts_out have num_chunks * k_chunk slots; untouched slots keep their input
 * contents (the kernel does not write them either).  acts_out receives bit copies of x.
 * Returns the number of slots written.  Order inside a bucket: ascending channel.
 */
int dd_select(const void *x, int dtype, uint32_t K, float thr_a, float thr_b,
              uint32_t k_chunk, int32_t *rows_out, void *acts_out) {
    uint32_t k = (uint32_t)(((uint64_t)k_chunk * K) / CHUNK);
    if (k == 0) return 0;
    float fl[NBUCKET];
    dd_bucket_floors(thr_a, thr_b, dtype, fl);
    uint32_t num_chunks = (K + CHUNK - 1) / CHUNK;
    int written = 0;
    for (uint32_t c = 0; c < num_chunks; c++) {
        uint32_t lo = c * CHUNK, hi = lo + CHUNK < K ? lo + CHUNK : K;
        uint32_t kc = k_chunk * (hi - lo) / CHUNK;
        uint32_t count = 0;
        for (int i = 0; i < NBUCKET && count < kc; i++) {
            float floor_i = fl[i];
            float ceil_i = (i == 0) ? INFINITY : fl[i - 1];
            for (uint32_t ch = lo; ch < hi && count < kc; ch++) {
                float v = fabsf(load_f(x, dtype, ch));
                if (v >= floor_i && v < ceil_i) {
                    size_t slot = (size_t)c * k_chunk + count;
                    rows_out[slot] = (int32_t)ch;
                    if (dtype == 0) ((float *)acts_out)[slot] = ((const float *)x)[ch];
                    else ((uint16_t *)acts_out)[slot] = ((const uint16_t *)x)[ch];
                    count++; written++;
                }
            }
        }
    }
    return written;
}

/* ---------------------------------------------------------------- A2 DEC */
/* out[n] += sum over the listed rows of (nib - 8) * scale[n] * x[row]  in double.
 * rows < 0 or >= K are skipped. */
void dd_dec_apply(const void *x, int dtype, const uint32_t *cheatsheet, const void *reordered_scales,
                  const int32_t *rows, uint32_t nrows, uint32_t K, uint32_t N, double *out) {
    uint32_t M = N / 8;
    double *acc = (double *)calloc(N, sizeof(double));
    for (uint32_t i = 0; i < nrows; i++) {
        int32_t r = rows[i];
        if (r < 0 || (uint32_t)r >= K) continue;
        double act = (double)load_f(x, dtype, (size_t)r);
        const uint32_t *row = cheatsheet + (size_t)r * M;
        for (uint32_t m = 0; m < M; m++) {
            uint32_t w = row[m];
            for (int j = 0; j < 8; j++) {
                int nib = (int)((w >> (4 * j)) & 0xF) - 8;
                acc[8 * m + j] += (double)nib * act;
            }
        }
    }
    for (uint32_t m = 0; m < M; m++)
        for (int j = 0; j < 8; j++)
            out[8 * m + j] += acc[8 * m + j] * (double)load_f(reordered_scales, dtype, (size_t)j * M + m);
    free(acc);
}

/* ---------------------------------------------------------------- B1 any-precision */
/* out[n] += sum_c lut[n][idx(n,c)] * x[c]; loop structure of matmul_kbit_32 (chunk i, lane t,
 * group j, element e; x address 8*(eff*j + 128 i + t) + e; bit 31-(8j+e)); double accumulate. */
void dd_anyprec_gemv(const void *x, int dtype, const uint32_t *qweight, const void *lut,
                     int bits, uint32_t N, uint32_t K, double *out) {
    uint32_t W = K / 32;
    uint32_t nchunk = (K + 1023) / 1024;
    int L = 1 << bits;
    double *xd = (double *)malloc(sizeof(double) * K);
    for (uint32_t c = 0; c < K; c++) xd[c] = (double)load_f(x, dtype, c);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < (int64_t)N; n++) {
        double lutd[256];
        for (int v = 0; v < L; v++) lutd[v] = (double)load_f(lut, dtype, (size_t)n * L + v);
        double sum = 0.0;
        for (uint32_t i = 0; i < nchunk; i++) {
            uint32_t eff = (i == K / 1024) ? (K % 1024) / 32 : 32;
            for (uint32_t t = 0; t < eff; t++) {
                uint32_t q[8];
                for (int p = 0; p < bits; p++)
                    q[p] = qweight[((size_t)p * N + (size_t)n) * W + 32 * i + t];
                for (int j = 0; j < 4; j++) {
                    size_t base = 8 * ((size_t)eff * j + 128 * (size_t)i + t);
                    for (int e = 0; e < 8; e++) {
                        int pos = 31 - (8 * j + e);
                        int idx = 0;
                        for (int p = 0; p < bits; p++) idx = (idx << 1) | (int)((q[p] >> pos) & 1u);
                        sum += lutd[idx] * xd[base + e];
                    }
                }
            }
        }
        out[n] += sum;
    }
    free(xd);
}

/* ---------------------------------------------------------------- B2 LUT-GEMM */
/* W[K/32][bits][N], alpha[K/g][bits][N], q_bias[K/g][N]; tile loop of nqmv_bias. */
void dd_lutgemm_gemv(const void *x, int dtype, const uint32_t *qw, const void *alpha,
                     const void *q_bias, int bits, int group_size, uint32_t N, uint32_t K, double *out) {
    uint32_t KT = K / 32;
    double *xd = (double *)malloc(sizeof(double) * K);
    for (uint32_t c = 0; c < K; c++) xd[c] = (double)load_f(x, dtype, c);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < (int64_t)N; n++) {
        double sum = 0.0;
        for (uint32_t kt = 0; kt < KT; kt++) {
            uint32_t g = (kt * 32) / (uint32_t)group_size;
            double xs = 0.0;
            for (int j = 0; j < 32; j++) xs += xd[32 * kt + j];                  /* lut[..][255] */
            sum += (double)load_f(q_bias, dtype, (size_t)g * N + n) * xs;
            for (int b = 0; b < bits; b++) {
                uint32_t w = qw[((size_t)kt * bits + b) * N + n];
                double t = 0.0;
                for (int j = 0; j < 32; j++) t += ((w >> j) & 1u) ? xd[32 * kt + j] : -xd[32 * kt + j];
                sum += (double)load_f(alpha, dtype, ((size_t)g * bits + b) * N + n) * t;
            }
        }
        out[n] += sum;
    }
    free(xd);
}

/* ---------------------------------------------------------------- B3 SqueezeLLM */
void dd_sqllm_gemv(const void *x, int dtype, const uint32_t *mat, const void *lut,
                   int bits, uint32_t N, uint32_t K, double *out) {
    int L = 1 << bits;
    double *xd = (double *)malloc(sizeof(double) * K);
    for (uint32_t c = 0; c < K; c++) xd[c] = (double)load_f(x, dtype, c);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < (int64_t)N; n++) {
        double lutd[16];
        for (int v = 0; v < L; v++) lutd[v] = (double)load_f(lut, dtype, (size_t)n * L + v);
        double sum = 0.0;
        if (bits == 4) {
            for (uint32_t r = 0; r < K / 8; r++) {
                uint32_t w = mat[(size_t)r * N + n];
                for (int j = 0; j < 8; j++) sum += lutd[(w >> (4 * j)) & 0xF] * xd[8 * r + j];
            }
        } else {
            for (uint32_t u = 0; u < K / 32; u++) {
                uint32_t w0 = mat[(size_t)(3 * u) * N + n];
                uint32_t w1 = mat[(size_t)(3 * u + 1) * N + n];
                uint32_t w2 = mat[(size_t)(3 * u + 2) * N + n];
                /* sqllm.cu:64-112: ten fields, a straddling field, ten, a straddling field, ten */
                const double *xv = xd + 32 * (size_t)u;
                int k = 0;
                for (int f = 0; f < 10; f++) sum += lutd[(w0 >> (3 * f)) & 7] * xv[k++];
                sum += lutd[((w0 >> 30) | ((w1 << 2) & 4)) & 7] * xv[k++];
                uint32_t t1 = w1 >> 1;
                for (int f = 0; f < 10; f++) sum += lutd[(t1 >> (3 * f)) & 7] * xv[k++];
                sum += lutd[((t1 >> 30) | ((w2 << 1) & 6)) & 7] * xv[k++];
                uint32_t t2 = w2 >> 2;
                for (int f = 0; f < 10; f++) sum += lutd[(t2 >> (3 * f)) & 7] * xv[k++];
            }
        }
        out[n] += sum;
    }
    free(xd);
}

/* ---------------------------------------------------------------- whole layer (CPU baseline) */
/*
 * y = deq(Wq) x + R_hat[:, sel] x[sel] for one any-precision layer with DEC, the operation
 * the GPU path performs per linear layer: select, residual rows, base GEMV.  out is
 * overwritten.  scratch_rows needs ceil(K/1024)*k_chunk entries.
 */
void dd_layer_anyprec_dec(const void *x, int dtype, const uint32_t *qweight, const void *lut, int bits,
                          const uint32_t *cheatsheet, const void *reordered_scales,
                          float thr_a, float thr_b, uint32_t k_chunk,
                          uint32_t N, uint32_t K, int32_t *scratch_rows, double *out) {
    uint32_t num_chunks = (K + CHUNK - 1) / CHUNK;
    size_t slots = (size_t)num_chunks * (k_chunk ? k_chunk : 1);
    for (size_t i = 0; i < slots; i++) scratch_rows[i] = -1;
    for (uint32_t n = 0; n < N; n++) out[n] = 0.0;
    if (k_chunk) {
        void *acts = malloc(slots * 4);
        dd_select(x, dtype, K, thr_a, thr_b, k_chunk, scratch_rows, acts);
        free(acts);
        dd_dec_apply(x, dtype, cheatsheet, reordered_scales, scratch_rows, (uint32_t)slots, K, N, out);
    }
    dd_anyprec_gemv(x, dtype, qweight, lut, bits, N, K, out);
}
