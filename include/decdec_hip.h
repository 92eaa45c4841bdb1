/*
 * C ABI of libdecdec_hip.so -- the MI355X (gfx950) implementation of DecDEC's decode-time
 * linear-layer path.  Plain pointers and sizes only; no torch types.
 *
 * Every entry point replaces one function of the reference's pybind module `decdec_ext`
 * (reference decdec_extension/bindings.cpp:19-40); the reference function and the file:line of
 * its C++ implementation are cited at each declaration.  Tensor arguments of the reference become
 * (pointer, dtype, sizes); the "current CUDA stream" of the reference (decdec.cu:144, :331)
 * becomes the explicit `stream` argument (a hipStream_t; NULL = default stream).
 *
 * Conventions
 *   - return value 0 = success; non-zero = failure, decdec_last_error() then returns a message
 *     (thread-local).  1 = invalid argument, 2 = HIP runtime error, 3 = unsupported.
 *   - all device pointers must be valid on the current HIP device; kernels are enqueued on
 *     `stream` and the calls do not synchronise.
 *   - every GEMV / DEC entry point ACCUMULATES into `output` with atomic adds, as the reference
 *     kernels do (anyprec.cu:508-510, lutgemm.cu:143-148, sqllm.cu:115, dec.cu:275): callers
 *     zero `output` first (reference end-to-end/APLinear.py:51).
 *   - handles are opaque 64-bit integers (the reference returns uintptr_t object addresses,
 *     dec_config.cu:243, dec_context.cu:59).
 *   - not thread-safe per handle; callers are single-threaded like the reference's.
 */
#ifndef DECDEC_HIP_H
#define DECDEC_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of activations / scales / LUTs / outputs (reference datatype.h:8-12) */
enum { DECDEC_FP32 = 0, DECDEC_FP16 = 1, DECDEC_BF16 = 2 };

typedef struct decdec_config_info {
    /* keys of the reference's read_dec_config (dec_config.cu:343-351), computed with the
     * reference's own integer formulas (dec_config.cu:34-115) so tools that read them see the
     * same values */
    int32_t num_chunks, chunk_size, k_chunk, channels_per_tb, n_tb;
    int32_t block_dim_x, block_dim_y, shared_memory_size, reduced_shared_memory;
    /* launch plan actually used by the gfx950 DEC kernel */
    int32_t hip_dec_blocks;        /* workgroups of 1024 threads given to DEC (<= num_tb) */
    int32_t hip_chunk_groups;      /* = atomic adds each output receives from DEC */
    int32_t hip_segment_groups;
    int32_t hip_vec_words;         /* u32 words per lane per residual load (always 1: 256-byte wave loads) */
    int32_t hip_lds_bytes;
    int32_t hip_slots_per_block;
    int32_t hip_lds_reduce;
    int32_t hip_residual_on_host;  /* 1: zero-copy from pinned host memory */
} decdec_config_info;

const char* decdec_last_error(void);
int decdec_version(void);

/* Library options (process-wide integers).  No counterpart in the reference.
 *
 * Options a caller is meant to set:
 *   "fusion"                1 = DEC and the base GEMV in one kernel launch [default]; 0 = the reference's two-stream
 *                           fork/join (decdec.cu:621-640).
 *   "dec_max_chunk_groups"  DEC launch plans made from now on use at most this many chunk groups, i.e. atomic adds
 *                           (roundings of a 16-bit output in varying order) per output: 1 to 4; 1 = the reference's
 *                           single add (dec.cu:263-276); 0 = the built-in bound of 4 [default].
 *   "gemv_max_k_ranges"     LUT-GEMM and SqueezeLLM launch plans use at most this many K ranges, each of which adds
 *                           to an output with one atomic add (the reference adds once per 32 or 128 channels,
 *                           lutgemm.cu:143-148, sqllm.cu:115); 0 = as many as run fastest, up to 9 / 8 [default].
 *                           LUT-GEMM rows longer than 3584 x the bound still get as many ranges as they need.
 *   "host_noncoherent"      1 = allocate the pinned residual with hipHostMallocNonCoherent; 0 [default].
 *
 * Experimental: launch-shape overrides and measurement aids used to tune and profile the library.  Their defaults are
 * what the library ships with; their meaning may change with the kernels, and nothing outside a tuning session
 * should depend on them.
 *   "fused_two_per_cu"      fused launches: 1 / 0 = always / never the kernel instance that lets two workgroups share
 *                           a compute unit; -1 = chosen per launch [default].
 *   "fused_small"           fused 3-bit any-precision launches with both roles in the GEMV's own 4- or 8-wave
 *                           workgroups: -1 = when those have 5 to 8 waves and DEC is the shorter role [default],
 *                           1 = whenever they have at most 8 waves, 0 = never.
 *   "dec_block_waves"       waves of a standalone DEC workgroup: 4, 8 or 16 [default]; the launch plan follows.
 *   "dec_force_cg", "dec_force_sg"   DEC launch plans made from now on use this many chunk groups / segment groups
 *                           where the shape allows; 0 = planned [default].
 *   "dec_rows_in_flight"    residual rows a DEC wave requests per round: 2, 4 or 8; 0 = chosen per launch from the rows
 *                           per wave and the time the launch occupies the link [default].
 *   "anyprec_rpw", "anyprec_rg", "lutgemm_ktiles", "sqllm_ktiles"   rows per wave / row groups per workgroup / K ranges
 *                           of the base GEMVs; 0 = automatic [default].  (sqllm_ktiles = 1 and lutgemm_ktiles = 1 give
 *                           every output a single atomic add from the GEMV.)
 *   "anyprec_tile"          3-bit LDS-transposed tile decoder for K <= 8192, waves per tile 2 / 4 / 8; 0 = off [default].
 *   "attention_two_step"    decode attention with a workspace: 1 = merge in a second kernel, 0 = in the kernel [default].
 *   "attention_single_below"  ... merging in the kernel: sequences of at most this many positions are scanned by one
 *                           workgroup per head; default 512, 0 = always share.
 *   "dec_trace"             see decdec_debug_read_trace. */
int decdec_set_option(const char* name, int value);
int decdec_get_option(const char* name, int* value);

/* create_dec_context (dec_context.cu:62-103).  Borrows the two scratch buffers (device memory,
 * `buffer_numel` elements each: int32 rows, `dtype` activations); creates the sub-stream and event
 * used by the two-stream mode.  The reference has no destroy; decdec_destroy_dec_context is an
 * addition. */
int decdec_create_dec_context(uint32_t num_tb, int dtype, uint64_t buffer_numel,
                              void* selected_rows_buffer, void* selected_activations_buffer,
                              uint64_t* context_out);
int decdec_destroy_dec_context(uint64_t context);

/* create_dec_config (dec_config.cu:186-292).  q_residual: int32 [num_rows, num_cols/8]; when it is
 * host memory it is copied into pinned, device-mapped memory owned by the config (zero-copy fetch);
 * when it is device memory it is used in place (borrowed).  reordered_scales: `dtype`[num_cols],
 * copied into device memory owned by the config.  thresholds: host memory, `dtype`[num_rows],
 * BORROWED -- read again at every decdec_dec* call (decdec.cu:66-67), so it must outlive the config. */
int decdec_create_dec_config(uint64_t context, uint32_t k_chunk, int dtype,
                             const void* q_residual, int q_residual_on_device,
                             const void* reordered_scales, int reordered_scales_on_device,
                             const void* thresholds_host,
                             uint32_t num_rows, uint32_t num_cols, uint64_t* config_out);
/* read_dec_config (dec_config.cu:337-354) */
int decdec_read_dec_config(uint64_t config, decdec_config_info* info_out);
/* update_dec_config (dec_config.cu:295-326): new context and k_chunk, residual not re-copied */
int decdec_update_dec_config(uint64_t config, uint64_t new_context, uint32_t k_chunk);
/* destroy_dec_config (dec_config.cu:329-334) */
int decdec_destroy_dec_config(uint64_t config);

/* dec (decdec.cu:139-146 -> dec_templated :40-91 -> fused_dec_kernel dec.cu:26-280): select
 * k_chunk channels per 1024-channel chunk, fetch their residual rows, accumulate into output.
 * Writes the selection into the context's scratch buffers at [chunk*k_chunk + pos]. */
int decdec_dec(uint64_t config, const void* input, void* output, int dtype,
               uint32_t in_features, uint32_t out_features, void* stream);
/* unfused_dec (decdec.cu:238-245 -> dec_kernel dec.cu:284-426): as dec, but the first
 * k_chunk*in_features/1024 entries of the context's row buffer are supplied by the caller. */
int decdec_unfused_dec(uint64_t config, const void* input, void* output, int dtype,
                       uint32_t in_features, uint32_t out_features, void* stream);

/* anyprec_gemv (decdec.cu:324-333 -> matmul_kbit_32 anyprec.cu:344-514). qweight int32
 * [>=bitwidth, out, in/32] (only the first `bitwidth` planes are read; plane p starts at word
 * p*out*in/32), lut `dtype`[out, 2^bitwidth]; fp16 / bf16 only; bitwidth 3..8. */
int decdec_anyprec_gemv(const void* input, void* output, const void* qweight, const void* lut,
                        int bitwidth, int dtype, uint32_t in_features, uint32_t out_features,
                        void* stream);
/* anyprec_dequant (decdec.cu:386-393 -> dequant_kbit_store anyprec.cu:261-331): weight_out
 * `dtype`[out, in], allocated by the caller. */
int decdec_anyprec_dequant(const void* qweight, const void* lut, void* weight_out, int bitwidth,
                           int dtype, uint32_t out_features, uint32_t in_features, void* stream);
/* lutgemm_gemv (decdec.cu:485-496 -> nqmv_bias lutgemm.cu:25-150). q_weight int32
 * [in/32, bitwidth, out], alpha [in/group, bitwidth, out], q_bias [in/group, out]. */
int decdec_lutgemm_gemv(const void* input, void* output, const void* q_weight, const void* alpha,
                        const void* q_bias, int bitwidth, int group_size, int dtype,
                        uint32_t in_features, uint32_t out_features, void* stream);
/* sqllm_gemv (decdec.cu:594-603 -> VecQuant{3,4}MatMulKernelNUQPerChannel sqllm.cu:28-169).
 * qweight int32 [in*bitwidth/32, out], lut [out, 2^bitwidth]; bitwidth 3 or 4.  `input` must be 4-byte
 * aligned (it is read through the scalar cache). */
int decdec_sqllm_gemv(const void* input, void* output, const void* qweight, const void* lut,
                      int bitwidth, int dtype, uint32_t in_features, uint32_t out_features,
                      void* stream);

/* dec_anyprec / dec_lutgemm / dec_sqllm (decdec.cu:643-659, :701-721, :761-779): DEC and the base
 * GEMV run concurrently on the pre-zeroed output; on return the work is ordered on `stream`. */
int decdec_dec_anyprec(uint64_t config, const void* input, void* output, const void* qweight,
                       const void* lut, int bitwidth, int dtype, uint32_t in_features,
                       uint32_t out_features, void* stream);
int decdec_dec_lutgemm(uint64_t config, const void* input, void* output, const void* q_weight,
                       const void* alpha, const void* q_bias, int bitwidth, int group_size,
                       int dtype, uint32_t in_features, uint32_t out_features, void* stream);
int decdec_dec_sqllm(uint64_t config, const void* input, void* output, const void* qweight,
                     const void* lut, int bitwidth, int dtype, uint32_t in_features,
                     uint32_t out_features, void* stream);

/* dummy_anyprec / dummy_lutgemm / dummy_sqllm (decdec.cu:874-1013): the base GEMV on a side stream
 * while `dummy_cu` workgroups of 1024 threads spin for `dummy_iters` iterations on `stream`. */
int decdec_dummy_anyprec(const void* input, void* output, const void* qweight, const void* lut,
                         int bitwidth, int dtype, uint32_t in_features, uint32_t out_features,
                         int dummy_cu, int64_t dummy_iters, void* stream);
int decdec_dummy_lutgemm(const void* input, void* output, const void* q_weight, const void* alpha,
                         const void* q_bias, int bitwidth, int group_size, int dtype,
                         uint32_t in_features, uint32_t out_features,
                         int dummy_cu, int64_t dummy_iters, void* stream);
int decdec_dummy_sqllm(const void* input, void* output, const void* qweight, const void* lut,
                       int bitwidth, int dtype, uint32_t in_features, uint32_t out_features,
                       int dummy_cu, int64_t dummy_iters, void* stream);

/* Several any-precision layers that read the SAME input vector, in one launch: q | k | v and gate | up of a decoder
 * layer are independent given their input, and one launch pays the launch and selection latencies once instead of once
 * per layer.  Layer i: config configs[i] (0, or a config with k_chunk 0: base GEMV only; configs may be NULL when no
 * layer has DEC), output outputs[i] (out_features[i] elements; the ranges of different layers must not overlap, not
 * even partly; zeroed by the caller as for the single-layer ops), qweights[i], luts[i].  1 to 4 layers, the same bitwidth and dtype; results are those of n
 * decdec_dec_anyprec / decdec_anyprec_gemv calls.  Configs of one batch that belong to the same context write their
 * selections into the same scratch buffers at the same time: give each layer of a batch a context of its own if the
 * selection is read back.  The layers with DEC share the workgroup budget: layer i is planned against its context's
 * num_tb (48 if num_tb is larger) times its share of the batch's DEC output features, but against at least
 * min(num_tb, 16) workgroups: a batch occupies about num_tb workgroups with DEC when num_tb is 32 or more, and up to
 * n x num_tb when num_tb is 16 or less.
 * No counterpart in the reference, which fuses such projections by concatenating their weights (end-to-end/model.py
 * wqkv, w1w3). */
int decdec_dec_anyprec_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                             const void* const* qweights, const void* const* luts, int bitwidth, int dtype,
                             uint32_t in_features, const uint32_t* out_features, void* stream);

/* The same for LUT-GEMM and SqueezeLLM layers (argument meaning as in decdec_dec_lutgemm / decdec_dec_sqllm, one
 * pointer per layer; fp16 and bf16 run in one launch, fp32 as one call per layer with the same result).  No
 * counterpart in the reference. */
int decdec_dec_lutgemm_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                             const void* const* q_weights, const void* const* alphas, const void* const* q_biases,
                             int bitwidth, int group_size, int dtype, uint32_t in_features,
                             const uint32_t* out_features, void* stream);
int decdec_dec_sqllm_batch(uint32_t n, const uint64_t* configs, const void* input, void* const* outputs,
                           const void* const* qweights, const void* const* luts, int bitwidth, int dtype,
                           uint32_t in_features, const uint32_t* out_features, void* stream);

/* Decode-step helpers for a caller that drives the linear layers from a captured decode step (the
 * reference leaves these operations to torch.compile, end-to-end/generate.py; they have no counterpart in
 * its extension).  All tensors are fp16 or bf16 in device memory; `pos_device` points at the token position
 * (int64) in DEVICE memory, so a captured step can advance it on the device.
 *   decdec_rope_cache_update: qkv = [query heads | key heads | value heads] of one token; rotates pair
 *     (i, i + head_dim/2) of every query and key head by cos/sin_table[pos][i] (tables [max_seq][head_dim]),
 *     writes the rotated queries to q_out and the rotated keys and the values into row `pos` of the caches
 *     ([n_kv_head][max_seq][head_dim]).  A position outside [0, max_seq) writes nothing.
 *   decdec_decode_attention: out[h] = softmax(q[h] . K[kv(h)][0..pos] / sqrt(head_dim)) V[kv(h)][0..pos],
 *     head_dim 64 or 128, grouped-query heads (kv(h) = h / (n_head / n_kv_head)).  With a workspace of
 *     decdec_decode_attention_workspace_bytes(n_head, head_dim, 8) bytes (caller-owned device memory, ZERO when
 *     first used: it starts with one arrival counter per head, which every call leaves at zero; one workspace serves
 *     any number of calls that do not overlap in time) the positions of a head are shared by up to 8 workgroups (no
 *     more workgroups than the device has compute units) and the workgroup of a head that finishes last merges
 *     them (option "attention_two_step" = 1: a second small kernel does); workspace NULL = one workgroup per head.
 *   decdec_rope_attention: the two calls above in one launch (plus the merge kernel when a workspace is given): takes
 *     the un-rotated qkv, rotates the queries and the new key on the fly (rounded to the storage type; a value
 *     within rounding error of a tie may differ by one unit in the last place from what decdec_rope_cache_update
 *     stores), attends cache rows 0 .. pos - 1 and the new row, and appends the new
 *     key / value row to the caches (position outside [0, max_seq): nothing is appended, rows 0 .. max_seq - 1 are
 *     attended).  qkv, the tables and the caches 16-byte aligned.
 *   decdec_dense_gemv: out[n] = sum_k weight[n][k] * x[k] for an unquantised row-major fp16 / bf16 weight [N][K]
 *     (a decoder's output head), fp32 accumulation, `out` is overwritten (not accumulated).  K a multiple of 8,
 *     weight and x 16-byte aligned.
 *   decdec_silu_mul: out[i] = silu(gate_up[i]) * gate_up[n + i], i < n.
 *   decdec_add_rmsnorm: per row of `dim` elements (a multiple of 4, <= 16384; 8-byte aligned tensors), h = x + y rounded to the storage type and written to
 *     h_out (y and h_out may be NULL: then h = x), normed_out = h / sqrt(mean(h^2) + eps) * weight.
 *   decdec_greedy_pick: the end of a greedy decode step in two small launches.  token[0] = index of the largest of
 *     the `n` logits (fp16, bf16 or fp32; the smallest index among equal ones; a NaN with the sign bit clear counts
 *     as the largest, as in torch.argmax); if seq and count are given, seq[count[0]] = that index (when count[0] <
 *     seq_capacity) and count[0] += 1; if pos is given, pos[0] += 1; if logits_f32_out is given it receives the
 *     logits as fp32.  token, seq, count and pos are int64 in device memory; workspace is
 *     decdec_greedy_pick_workspace_bytes() bytes of 8-byte aligned device memory (contents irrelevant). */
int decdec_rope_cache_update(const void* qkv, const void* cos_table, const void* sin_table,
                             const int64_t* pos_device, void* q_out, void* k_cache, void* v_cache,
                             int dtype, uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim,
                             uint32_t max_seq, void* stream);
uint64_t decdec_decode_attention_workspace_bytes(uint32_t n_head, uint32_t head_dim, uint32_t nsplit);
int decdec_decode_attention(const void* q, const void* k_cache, const void* v_cache,
                            const int64_t* pos_device, void* out, int dtype, uint32_t n_head,
                            uint32_t n_kv_head, uint32_t head_dim, uint32_t max_seq,
                            void* workspace, uint64_t workspace_bytes, void* stream);
int decdec_rope_attention(const void* qkv, const void* cos_table, const void* sin_table,
                          const int64_t* pos_device, void* out, void* k_cache, void* v_cache, int dtype,
                          uint32_t n_head, uint32_t n_kv_head, uint32_t head_dim, uint32_t max_seq,
                          void* workspace, uint64_t workspace_bytes, void* stream);
/* decdec_decode_attention for callers that cannot allocate or own a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same kernels and the same result, with the workspace (arrival
 * counters and partial results of the shared heads) held in a device array that is part of the library image --
 * 532,992 bytes on every GPU the library runs on, until the process ends.  Limits: n_head <= 128, head_dim 64 or 128;
 * anything larger is refused with an error.  The call allocates nothing; it clears the counters it uses with a small
 * fill kernel and then launches the attention kernel on `stream`.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race.  The first call on a device looks the
 * array's address up and must not run under stream capture.  No counterpart in the reference. */
int decdec_decode_attention_static(const void* q, const void* k_cache, const void* v_cache,
                                   const int64_t* pos_device, void* out, int dtype, uint32_t n_head,
                                   uint32_t n_kv_head, uint32_t head_dim, uint32_t max_seq, void* stream);
int decdec_dense_gemv(const void* weight, const void* x, void* out, int dtype, uint32_t N, uint32_t K,
                      void* stream);
int decdec_silu_mul(const void* gate_up, void* out, int dtype, uint32_t n, void* stream);
int decdec_add_rmsnorm(const void* x, const void* y, const void* weight, void* h_out, void* normed_out,
                       int dtype, uint32_t rows, uint32_t dim, float eps, void* stream);
uint64_t decdec_greedy_pick_workspace_bytes(void);
int decdec_greedy_pick(const void* logits, uint32_t n, int dtype, void* workspace, float* logits_f32_out,
                       int64_t* token, int64_t* seq, uint32_t seq_capacity, int64_t* count, int64_t* pos,
                       void* stream);

/* Diagnostics: with option "dec_trace" = 1 every DEC workgroup stores shader-clock stamps of its
 * phases (0 start, 5 the scanning teams' activations in registers, 6 winning window compacted, 7 selected
 * channels ranked, 1 selection done, 2 residual rows accumulated, 3 merged, 4 end) into a
 * library-owned device buffer (at most 4096 workgroups); this copies the first `workgroups` x 8 stamps to the host (it
 * synchronises the device).  No counterpart in the reference. */
int decdec_debug_read_trace(uint64_t* stamps_out, int workgroups);
/* Diagnostics: a plain read kernel, nothing but loads -- the rate a fetch can reach on the memory `src` points at
 * (pinned host memory through its device address: the ceiling of the zero-copy residual fetch over the host link;
 * device memory: the ceiling of a streaming read).  Reads `rows` rows of `row_bytes` bytes (a multiple of
 * 256 * vec_words) laid out back to back, with `blocks` workgroups of 1024 threads, vec_words (1, 2, 4) dwords per lane
 * and request, eight requests in flight per wave; `scramble` != 0 visits the rows in a scattered order, as DEC's
 * selected rows are.  `sink`: 4 bytes of device memory.  No counterpart in the reference. */
int decdec_debug_read_probe(const void* src, uint64_t row_bytes, uint64_t rows, uint32_t vec_words,
                            uint32_t blocks, int scramble, void* sink, void* stream);

/* Host-only helpers (no GPU needed).  decdec_bucket_floors evaluates the selector's 32 bucket
 * floors exactly as dec.cu:117-130 does, in `dtype` arithmetic; decdec_reference_geometry evaluates
 * dec_config.cu:34-115 for a shape.  No counterpart in the reference's API. */
int decdec_bucket_floors(float threshold_a, float threshold_b, int dtype, float* floors32_out);
int decdec_reference_geometry(uint32_t num_rows, uint32_t num_cols, uint32_t num_tb,
                              uint32_t k_chunk, int dtype, uint32_t max_shared_memory,
                              decdec_config_info* info_out);
/* The library's own DEC launch plan for a shape (the hip_* fields of decdec_config_info, plus num_chunks,
 * chunk_size, k_chunk) for DEC workgroups of `block_waves` (4, 8 or 16) waves: num_tb counts 1024-thread
 * workgroups, smaller ones get the same number of waves in total.  Host-only; takes the place of the launch
 * geometry of dec_config.cu:34-115, which it does not follow (one workgroup per chunk group x column-segment
 * group, no grid barrier). */
int decdec_dec_launch_plan(uint32_t num_rows, uint32_t num_cols, uint32_t num_tb, uint32_t k_chunk,
                           uint32_t block_waves, decdec_config_info* info_out);
/* Which instance of the fused DEC + GEMV kernel a single-layer call launches for a shape under the current options:
 * 0 = 1024-thread workgroups, one per compute unit; 1 = 1024-thread workgroups, two per compute unit; 2 = both roles
 * in the GEMV's own 4- or 8-wave workgroups (3-bit any-precision only).  kind: 0 any-precision, 1 LUT-GEMM,
 * 2 SqueezeLLM.  Host-only; the choice rests on time estimates of the two roles, not on data.  No counterpart in
 * the reference. */
int decdec_fused_launch_form(int kind, int bitwidth, uint32_t in_features, uint32_t out_features, uint32_t k_chunk,
                             int* form_out);

#ifdef __cplusplus
}
#endif
#endif /* DECDEC_HIP_H */
