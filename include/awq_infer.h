/*
 * awq_infer.h -- C ABI of the MI355X AWQ int4 decode engine.
 *
 * Plain pointers and sizes only.  Every function that can fail returns 0 on
 * success and a non-zero code otherwise; awq_last_error() then describes the
 * failure for the calling thread.  (The reference prints to stderr and calls
 * exit(1), Inference.cu:52-71; the C++ wrapper class QWen3AWQInfer restores
 * that behaviour on top of these codes.)
 *
 * Device pointers are HIP device addresses; `stream` is a hipStream_t passed
 * as void* (NULL = the default stream).  Kernel entry points only enqueue
 * work; they do not synchronise.  FP16 data is IEEE binary16 stored as
 * uint16_t.
 */
#ifndef AWQ_INFER_H
#define AWQ_INFER_H

#include <stdint.h>
#include "awq_synth.h" /* enum awq_tensor_kind / awq_tensor_part */

#ifdef __cplusplus
extern "C" {
#endif

#define AWQ_OK 0
#define AWQ_ERR_ARG 1     /* bad argument or unsupported shape */
#define AWQ_ERR_IO 2      /* missing or short weight file */
#define AWQ_ERR_HIP 3     /* a HIP runtime call failed */
#define AWQ_ERR_STATE 4   /* call order violated (e.g. generate before finalize) */

/* Model shape.  awq_default_config gives the constants of Inference.cu:33-47. */
typedef struct awq_config {
  int32_t n_layers;   /* NUM_HIDDEN_LAYERS 36    Inference.cu:37 */
  int32_t hidden;     /* HIDDEN_SIZE 4096        Inference.cu:33, multiple of 256 */
  int32_t inter;      /* INTERMEDIATE_SIZE 12288 Inference.cu:34, multiple of 128 */
  int32_t vocab;      /* VOCAB_SIZE 151936       Inference.cu:38, multiple of 128 */
  int32_t max_pos;    /* MAX_POS_EMBEDDINGS 40960 Inference.cu:39, KV cache rows per head */
  int32_t split_idx;  /* SPLIT_IDX 18            Inference.cu:47: layers below it attend one
                         position fewer during generation (Inference.cu:1118 with 1364) */
  float eps;          /* RMS_NORM_EPS 1e-6       Inference.cu:41 */
} awq_config;

typedef struct awq_engine awq_engine;

const char* awq_last_error(void);
void awq_default_config(awq_config* cfg);

/* ----------------------------------------------------------------------------
 * Engine: replaces class QWen3AWQInfer (Inference.cu:356-415).
 * ------------------------------------------------------------------------- */

/* Host-only check that `dir` holds every file of Inference.cu:780-899 with at
 * least the expected byte count.  Touches no GPU. */
int awq_validate_weight_dir(const char* dir, const awq_config* cfg);

/* Constructor, Inference.cu:422-470: loads the weight directory onto the
 * current device, repacks, builds rotary tables, zeroes the KV cache.
 * cfg == NULL means the reference constants.
 * Loader (readBinaryFileToDevice, Inference.cu:297-311, called from :766-903):
 * a reader thread fills two pinned staging buffers in turn while the previous
 * file's host-to-device copy and the previous tensor's reordering run on the
 * engine's stream, so file reads, copies and reordering overlap.  A missing or
 * short file fails with AWQ_ERR_IO as the reference does (:299-308); bytes
 * beyond the expected count are ignored (:304). */
int awq_create(const char* weight_dir, const awq_config* cfg, awq_engine** out);
/* Seconds the last successful awq_create on this thread spent between opening
 * the first file and the last tensor being reordered on the device (0 when
 * none ran).  No counterpart in the reference. */
double awq_last_load_seconds(void);

/* Same engine without a directory: allocate, then awq_upload every array, then
 * awq_finalize.  Used with in-memory synthetic weights. */
int awq_create_empty(const awq_config* cfg, awq_engine** out);
int awq_upload(awq_engine* e, int layer, int kind, int part, const void* host_src, int64_t bytes);
int awq_finalize(awq_engine* e);

/* generateResponse, Inference.cu:1297-1408.  Writes max_new_tokens ids to
 * out_ids.  Restarts from an empty sequence on every call.  Fails (instead of
 * the reference's assert / cache overrun) when n_prompt + max_new_tokens >
 * max_pos. */
int awq_generate(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt, int32_t max_new_tokens,
                 int32_t* out_ids);

/* The same loop in pieces, for timing: reset, the prompt loop
 * (Inference.cu:1304-1343), then n_steps generation steps
 * (Inference.cu:1352-1405).  awq_decode returns after the device finished. */
int awq_reset(awq_engine* e);
int awq_prefill(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt);
int awq_decode(awq_engine* e, int32_t n_steps, int32_t* out_ids);

/* The prompt loop (Inference.cu:1304-1343) for all prompt positions together:
 * per layer one W4A16 matrix product over the prompt instead of one
 * matrix-vector product per token (the reference streams every weight once per
 * prompt token, Inference.cu:1326-1332).  Each token attends exactly the
 * positions the sequential loop gives it.  Leaves the same state as awq_prefill
 * up to rounding: the products are summed in a different order, so K/V and the
 * hidden state agree to binary16 rounding noise, not bit for bit.
 * awq_set_prefill_mode(e, 1) makes awq_generate use it; the default (0) is the
 * token-by-token loop. */
int awq_prefill_batched(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt);
int awq_set_prefill_mode(awq_engine* e, int batched);
/* Test hook, no counterpart in the reference: some of the batched pass's
 * products hand partial sums from workgroup to workgroup through a bounded
 * wait (see awq_gemm).  With `on` non-zero every such wait of the next
 * awq_prefill_batched call gives up before its first poll: all kernels end
 * normally, the call returns AWQ_ERR_HIP, and the engine is usable again
 * after awq_reset.  The fused launches of the token-by-token steps (see
 * awq_set_fused_mode) take the same path; with `on` == 2 their condition is
 * set again by the next awq_reset, once, so that a whole awq_generate call
 * (which starts with a reset) meets it. */
int awq_debug_force_handover_giveup(awq_engine* e, int on);

/* No counterpart in the reference: pairs of a layer's launches as ONE launch,
 * with bit-identical results.  `enabled` is a sum of
 *   1  the attention output product (Inference.cu:1128-1155) and RMSNorm + W1 +
 *      GeLU (:1163-1198): 256 workgroups hand the hidden state to each other
 *      through memory, W1's weights requested while that hand-over is under way
 *      (hidden 4096 / intermediate 12288);
 *   2  RMSNorm + Wqkv + rotary + KV append (:1040-1103) and the attention
 *      (:1110) up to 4096 attended positions: the eight workgroups of a head sit
 *      on one die and hand partial scores to each other through its L2 (hidden
 *      4096, 32 heads; longer sequences keep the two launches).  The launch
 *      reads the caches from a second copy that the engine keeps for it, the
 *      first min(max_pos, 4096) positions as [head][8][position][16] (2 x 33.5 MB
 *      per layer at 4096 positions).
 * The first is off by default: on MI355X it measures 2 % slower than the two
 * launches it replaces (a hand-over between all workgroups costs what a kernel
 * boundary costs).  The second is on by default where the device can run it
 * (1049 against 987 tok/s at 137..392 positions, 764 against 625 at 2104..2144,
 * 676 against 594 at 3004..3044, 606 against 574 at 3504..3544).  A fused launch
 * needs all its 256 workgroups resident at once, i.e. a device of at least 256
 * compute units to itself, and the second one workgroups whose indices agree
 * modulo 8 on one die (probed with a launch of the same grid when it is
 * switched on).  A wait that cannot end gives up after a bounded number of
 * polls and the call (awq_prefill, awq_decode) returns AWQ_ERR_HIP, never a
 * wrong token; awq_reset leaves the engine usable.  awq_generate (the drop-in
 * call) then switches the fused launches off and runs the whole request again
 * with every launch on its own; they stay off until this is called again.  Asking
 * for a launch where it is not supported leaves it off; awq_fused_mode tells
 * which are in use. */
int awq_set_fused_mode(awq_engine* e, int enabled);
int awq_fused_mode(const awq_engine* e);
/* Diagnostics, no counterpart in the reference: runs the fused launch of every
 * layer back to back with one layer's launch instrumented and returns, per
 * workgroup, the device time (10 ns units) at which its first thread passed
 * each of *n_stamps points (request, staged, multiplied, stored, hidden state
 * seen, ...; listed where bench.py prints them).  host_out holds at least
 * 256 * 16 values.  Leaves the engine reset. */
int awq_debug_fused_timeline(awq_engine* e, int32_t layer, uint64_t* host_out, int32_t* n_workgroups,
                             int32_t* n_stamps);
/* The same for the fused Wqkv + attention launch, at position `pos` attending
 * pos + 1 positions (pos < min(max_pos, 4096)). */
int awq_debug_qkv_attention_timeline(awq_engine* e, int32_t layer, int32_t pos, uint64_t* host_out,
                                     int32_t* n_workgroups, int32_t* n_stamps);

/* Copies of internal state for tests: hidden state [hidden] and the logits of
 * the last sampled position [vocab], both FP16, to host memory. */
int awq_read_hidden(awq_engine* e, uint16_t* host_dst);
int awq_read_logits(awq_engine* e, uint16_t* host_dst);
/* 0: every op is its own launch; 1 (default): one captured graph per step */
int awq_set_graph_mode(awq_engine* e, int enabled);

/* Measurement aid with no counterpart in the reference: runs the engine's own
 * fused-linear launch of `kind` (AWQ_T_WQKV/WO/W1/W2/UNEMBED) over every
 * layer's resident matrix, n_rounds times, between two HIP events on the
 * engine's stream (a round is captured once and replayed as a graph, the way
 * the decode step issues these launches).  Returns the mean launch duration and the algorithmic bytes
 * of one launch (packed weights + scales + zero-points + input + output).
 * AWQ_T_UNEMBED is timed as the decode step issues it: final norm, logits,
 * argmax and the small launch that ends the step, counted as one launch.
 * Overwrites the activations and resets the sequence. */
int awq_time_linear(awq_engine* e, int kind, int32_t n_rounds, float* avg_us_per_launch, int64_t* bytes_per_launch);

/* Destructor, Inference.cu:475-558 */
void awq_destroy(awq_engine* e);

/* Writes a weight directory in the layout of Inference.cu:780-899 filled from
 * awq_synth.h under `seed` (the reference ships no producer of its format). */
int awq_write_weight_dir(const char* dir, const awq_config* cfg, uint64_t seed);
/* the same with the value distributions chosen: AWQ_SYNTH_SPEC (what awq_write_weight_dir draws) or
 * AWQ_SYNTH_BALANCED (awq_synth.h) */
int awq_write_weight_dir_profile(const char* dir, const awq_config* cfg, uint64_t seed, int profile);

/* Host-side synthetic data (awq_synth.h).  `count` is in elements of the
 * array: bytes for AWQ_P_PACKED, halves otherwise. */
int awq_synth_fill(uint64_t seed, int layer, int kind, int part, void* host_dst, int64_t count);
/* profile: AWQ_SYNTH_SPEC (what awq_synth_fill draws) or AWQ_SYNTH_BALANCED (awq_synth.h) */
int awq_synth_fill_profile(int profile, uint64_t seed, int layer, int kind, int part, void* host_dst, int64_t count);
int awq_synth_normal_f16(uint64_t seed, uint64_t stream, uint16_t* host_dst, int64_t count, float mean, float std);
int awq_synth_tokens(uint64_t seed, uint64_t stream, int32_t* host_dst, int64_t count, int32_t vocab);

/* Rotary tables, Inference.cu:443-454, computed on the host with libm as the
 * reference does; cos_t / sin_t are host arrays of max_pos*64 halves. */
int awq_rope_tables_host(uint16_t* cos_t, uint16_t* sin_t, int64_t max_pos);

/* ----------------------------------------------------------------------------
 * Kernels (device pointers).
 * ------------------------------------------------------------------------- */

/* dequantAwqKernel and its launches, Inference.cu:76-106, 908-1008.
 * packed [rows][cols/2] bytes, scale/zp [n_groups] FP16, out [rows][cols] FP16.
 * group = (col/128) % n_groups.  cols must be even. */
int awq_dequant(const void* packed, const void* scale, const void* zp, void* out, int64_t rows, int64_t cols,
                int64_t n_groups, void* stream);

/* Load-time reordering of the packed int4 stream of an [m outputs x k inputs]
 * matrix (file layout: nibble p = j*m + i, Inference.cu:1059 read of :105)
 * into the order the product kernels stream it in.  Same byte count. */
int awq_linear_repack(const void* packed_in, void* repacked_out, int64_t m, int64_t k, void* stream);

/* cublasGemmEx with n = 1, Inference.cu:1052-1065, 1128-1141, 1176-1189,
 * 1201-1214, 1260-1273, fused with the dequantisation:
 *     y[i] = h( sum over blocks of 32 inputs of s * c * (sum q*I - z * sum I) ),
 *     the blocked arithmetic of awq_canon_math.h: the inputs of a block as 16-bit
 *     integers I under the block's power of two c (x = I*c up to a rounding of
 *     2^-16 of the block's largest input), exact integer sums over the raw
 *     nibbles q, scale and zero-point applied to a block's sums in FP32, block
 *     values added in a fixed tree; a block that holds an infinity or a NaN
 *     makes every output a NaN.  Within 1e-2 (in practice a few 1e-4) of the
 *     FP32-accumulated product of the FP16-dequantised weights.
 * repacked from awq_linear_repack; scale/zp [m/128]; x [k], y [m] FP16.
 * k <= 16384 (the workgroup keeps x in LDS).
 * workspace: awq_gemv_workspace_bytes(m,k) bytes, zero-filled once before its
 * first use (launches leave it zeroed); must not be shared by launches that
 * may overlap. */
int64_t awq_gemv_workspace_bytes(int64_t m, int64_t k);
int awq_gemv(const void* repacked, const void* scale, const void* zp, int64_t m, int64_t k, const void* x, void* y,
             void* workspace, void* stream);

/* The same kernel with the neighbouring operators of runOneLayer /
 * sampleNextToken fused in, as the engine launches it:
 *   prologue AWQ_PRO_RMSNORM   x is the un-normalised hidden state; rmsNormKernel
 *                              (Inference.cu:111-145) with gamma/eps runs first (k % 256 == 0)
 *   epilogue AWQ_EPI_RESIDUAL  y = h(residual + h(acc))          Inference.cu:1149-1155
 *            AWQ_EPI_GELU      y = h(gelu(h(acc)))               Inference.cu:271-279
 *            AWQ_EPI_QKV_ROPE  m == 3*hidden: rows [0,hidden) rotated to y (Q), rows
 *                              [hidden,2*hidden) rotated into k_cache at pos, the rest
 *                              into v_cache at pos                Inference.cu:1070-1103
 *            AWQ_EPI_ARGMAX    y = h(acc) and *out_token = greedy token  Inference.cu:1278-1290
 * Unused pointers may be NULL. */
#define AWQ_PRO_NONE 0
#define AWQ_PRO_RMSNORM 1
#define AWQ_EPI_STORE 0
#define AWQ_EPI_RESIDUAL 1
#define AWQ_EPI_GELU 2
#define AWQ_EPI_QKV_ROPE 3
#define AWQ_EPI_ARGMAX 4
typedef struct awq_linear_args {
  const void* repacked;
  const void* scale;
  const void* zp;
  int64_t m, k;
  const void* x;
  void* y;
  int32_t reserved0;     /* 0 */
  int32_t prologue;
  int32_t epilogue;
  float eps;
  const void* gamma;     /* [k] FP16 */
  const void* residual;  /* [m] FP16, may alias y */
  const void* cos_t;     /* [max_pos][64] FP16 */
  const void* sin_t;
  void* k_cache;         /* [hidden/128][max_pos][128] FP16 */
  void* v_cache;
  int32_t hidden;
  int32_t reserved;
  int64_t max_pos;
  int64_t pos;
  void* out_token;       /* device int32 */
  void* workspace;       /* awq_gemv_workspace_bytes(m,k), zero-filled once */
} awq_linear_args;
int awq_gemv_fused(const awq_linear_args* args, void* stream);

/* The same product for M tokens at once (prefill, batched decode): the
 * reference's cublasGemmEx with n = M, ldb = k, ldc = m (it only ever calls it
 * with n = 1, Inference.cu:1056).  x [M][k], y [M][m] row-major FP16, x and the
 * weights 16-byte aligned (AWQ_ERR_ARG otherwise).  Weights
 * are dequantised on load and contracted on the matrix cores with FP32
 * accumulation: within rounding noise of awq_gemv applied to each token, not
 * bit-identical to it.  Matrices whose scale group depends on the input index
 * (the 151936 x 4096 unembedding) are not supported.  workspace: NULL, or
 * awq_gemm_workspace_bytes(m, k, M) bytes of device memory whose first 4096
 * bytes are zero before the first call (every call leaves them zero); with it,
 * products with few output tiles also cut k over several workgroups (FP32
 * partial sums, added in a fixed order whatever the timing, by a second launch
 * or by the workgroup that holds a tile's last part of k).  That workgroup
 * waits for the others; they have lower indices and never wait themselves, so
 * the wait ends while the device dispatches workgroups in index order.  It is
 * bounded all the same: should it expire, the first int32 of the workspace
 * becomes 1 (read it after synchronising; the workgroup that gave up leaves
 * its tile of y unwritten, and the header must be zeroed again).  The second
 * int32 is a "give up now" word: non-zero makes every such wait give up
 * before its first poll, so that a test can drive this path with every kernel
 * ending normally.  Calls that share a workspace must not overlap.
 * zp_integral: 1 selects a shorter conversion for zero-points that are
 * integers in [0,1024] (true of AWQ checkpoints), 0 takes arbitrary
 * zero-points and -1 has the call inspect them (synchronises). */
int64_t awq_gemm_workspace_bytes(int64_t m, int64_t k, int64_t M);
/* Which workgroup shape awq_gemm takes for a product (host arithmetic only; no counterpart in the
 * reference, for diagnostics and tests): 0 the few-token kernel (M <= 4), 1 k split over the
 * wavefronts of a 64-row workgroup, 2 rows split with a 256 x 128 tile per workgroup, 3 rows split
 * with 64 tokens per workgroup, 4 rows split with the work cut evenly and FP32 sums handed over
 * (needs the workspace), 5 two to sixteen tokens on a k that is a multiple of 4096 (up to 16384):
 * 16 wavefronts share up to three 16-row groups and split k, 6 17..64 and 129..192 tokens on 4096 rows and a k of
 * 2048 or 4096: one 16-row group per workgroup, all weights requested at the start, the tokens
 * streamed through LDS, 7 17 to 256 tokens on 10240 to 16384 rows the same way: 64 rows per
 * workgroup on the 32 x 32 x 16 matrix instruction, 64 tokens after the other against weights
 * that stay in registers, 8 the same with k cut over four workgroups and a second launch that adds
 * their FP32 sums (4096 x 12288 at 128 to 320 tokens; needs the workspace). */
int awq_gemm_plan(int64_t m, int64_t k, int64_t M, int has_workspace);
int awq_gemm(const void* repacked, const void* scale, const void* zp, int64_t m, int64_t k, const void* x, void* y,
             int64_t M, int32_t zp_integral, void* workspace, void* stream);

/* rmsNormKernel, Inference.cu:111-145.  n multiple of 256. */
int awq_rmsnorm(const void* x, const void* gamma, void* out, int64_t n, float eps, void* stream);

/* QKV split (Inference.cu:1070-1077), applyRotaryKernel on Q and K
 * (:1082-1091) and the KV-cache append (:1094-1103) in one launch.
 * qkv [3*n_heads*128]; q_out [n_heads*128]; caches [n_heads][max_pos][128]. */
int awq_rope_kv_append(const void* qkv, const void* cos_t, const void* sin_t, void* q_out, void* k_cache,
                       void* v_cache, int32_t n_heads, int64_t max_pos, int64_t pos, void* stream);

/* attentionKernel, Inference.cu:182-266, for one query over L cached
 * positions.  Up to 704 positions one launch, four workgroups per head (each
 * with all keys and a quarter of the head's dimensions); beyond, the sequence
 * is cut into 32 parts per head over two to four launches with the same summation
 * orders (bit-identical results).  workspace:
 * awq_attention_workspace_bytes(n_heads, max_pos), contents irrelevant. */
int64_t awq_attention_workspace_bytes(int32_t n_heads, int64_t max_pos);
int awq_decode_attention(const void* q, const void* k_cache, const void* v_cache, void* ctx, int32_t n_heads,
                         int64_t max_pos, int64_t L, void* workspace, void* stream);

/* awq_decode_attention without a workspace argument and without any allocation.
 * No counterpart in the reference: it is for callers that cannot allocate device
 * memory (code under HIP stream capture, tight serving loops, harnesses that
 * forbid hipMalloc).  The scores and partial sums live in a 3,166,208-byte device
 * array inside the library, one copy per GPU, held until the process ends.
 * Limits: n_heads <= 32 and L <= 8192 (max_pos, the cache's row capacity, may be
 * larger); anything beyond is refused with AWQ_ERR_ARG.  Same kernels and same
 * bits as awq_decode_attention.  All calls on one GPU share the array: calls
 * that may overlap there (different streams, different threads) race.  The
 * first call on a GPU looks the array's address up; make it outside stream
 * capture. */
int awq_decode_attention_static(const void* q, const void* k_cache, const void* v_cache, void* ctx, int32_t n_heads,
                                int64_t max_pos, int64_t L, void* stream);

/* No counterpart in the reference: awq_gemv_fused(RMSNorm, Wqkv, rotary + KV
 * append) and awq_decode_attention as ONE launch for hidden 4096 and 32 heads
 * (wqkv_repacked is the 12288 x 4096 matrix from awq_linear_repack; caches
 * [head][max_pos][128]; x, gamma [4096]; q_out, ctx [4096]), position `pos`
 * attending the first L positions, L <= pos + 1 and L <= 4096.  Same bits as the
 * two calls.  Every head is given to eight workgroups that the device places on
 * one die (awq_qkv_attention_supported probes that and that all 256 workgroups
 * are resident at once: 1 = yes); they hand partial scores to each other through
 * that die's L2, in words that carry a tag derived from call_tag: any value in
 * [1, 2^30) that differs from the previous call's on the same workspace.
 * Each workgroup reads 16 of a cached row's 128 dimensions, so the launch reads
 * the caches from a second copy in its own order, k_parts and v_parts,
 * [head][8][parts_pos][16] FP16 (awq_kv_parts_bytes(n_heads, parts_pos) bytes
 * each, L <= parts_pos): it appends the new position to the caches AND to
 * these; rows that got into the caches another way are copied with
 * awq_kv_cache_to_parts (positions pos0 .. pos0 + n - 1).
 * workspace: awq_qkv_attention_workspace_bytes(n_heads) bytes, zero-filled once;
 * calls on one workspace must not overlap.  A wait that cannot end gives up
 * after a bounded number of polls and leaves ctx unwritten:
 * awq_qkv_attention_status (synchronises the stream) then returns AWQ_ERR_HIP
 * once and clears the condition. */
int64_t awq_qkv_attention_workspace_bytes(int32_t n_heads);
int awq_qkv_attention_supported(int64_t hidden, int32_t n_heads, void* stream);
int64_t awq_kv_parts_bytes(int32_t n_heads, int64_t parts_pos);
int awq_kv_cache_to_parts(const void* k_cache, const void* v_cache, int64_t max_pos, int32_t n_heads, void* k_parts,
                          void* v_parts, int64_t parts_pos, int64_t pos0, int64_t n, void* stream);
int awq_qkv_attention(const void* wqkv_repacked, const void* scale, const void* zp, const void* x, const void* gamma,
                      float eps, const void* cos_t, const void* sin_t, void* k_cache, void* v_cache, int64_t max_pos,
                      void* k_parts, void* v_parts, int64_t parts_pos, int32_t n_heads, int64_t pos, int64_t L,
                      void* q_out, void* ctx, void* workspace, int32_t call_tag, void* stream);
int awq_qkv_attention_status(void* workspace, void* stream);

/* The same attention for n_tokens consecutive prompt positions pos0 ..
 * pos0 + n_tokens - 1 at once (their keys and values already appended): q and
 * ctx are [n_tokens][n_heads*128].  The token at position p attends p + 1
 * positions, or, with first_layer != 0, max(p, 1): layer 0 of the prompt loop
 * reads current_seq_len_ before it is updated (Inference.cu:1118 vs :1331).
 * Keys and values go through LDS once per 128 queries and the products run on
 * the matrix cores (streaming softmax, probabilities rounded to binary16), so
 * the result agrees with awq_decode_attention to rounding noise, not bit for
 * bit. */
int awq_prefill_attention(const void* q, const void* k_cache, const void* v_cache, void* ctx, int32_t n_heads,
                          int64_t max_pos, int64_t pos0, int64_t n_tokens, int32_t first_layer, void* stream);

/* residual add lambda, Inference.cu:1149-1155: out = h(a + b); out may be a */
int awq_residual_add(const void* a, const void* b, void* out, int64_t n, void* stream);

/* geluKernel, Inference.cu:271-279, in place */
int awq_gelu(void* x, int64_t n, void* stream);

/* finalSoftmaxKernel + D2H + host argmax, Inference.cu:1278-1290, on device:
 * *out_token (device int32) = lowest index of the largest FP16 logit.
 * workspace: awq_argmax_workspace_bytes(n) bytes, zero-filled once. */
int64_t awq_argmax_workspace_bytes(int64_t n);
int awq_logits_argmax(const void* logits, int64_t n, void* out_token, void* workspace, void* stream);

/* gather lambda, Inference.cu:1310-1324: out[idx] = dequantised
 * word_embedding[idx][tok], read from the packed [hidden][vocab] file layout. */
int awq_embed_gather(const void* packed, const void* scale, const void* zp, int64_t hidden, int64_t vocab,
                     int32_t tok, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AWQ_INFER_H */
