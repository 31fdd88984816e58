// Shared declarations of the HIP side: FP16 vector types, error plumbing and
// the launcher prototypes that the C ABI (api.cpp) and the engine call.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "../../include/awq_canon_math.h"
#include "../../include/awq_infer.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// binary32 -> binary16, round to nearest even, as its own instruction.  Without
// the barrier the compiler folds a preceding multiply into v_fma_mixlo_f16 with
// a +0 addend, which turns a product of -0 into +0.
__device__ __forceinline__ half_t to_half_rn(float v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#endif
  return (half_t)v;
}

// error string of the calling thread (awq_last_error)
void awq_set_error(const std::string& msg);

#define AWQ_HIP_TRY(expr)                                                                                 \
  do {                                                                                                    \
    hipError_t err__ = (expr);                                                                            \
    if (err__ != hipSuccess) {                                                                            \
      awq_set_error(std::string("HIP error at ") + __FILE__ + ":" + std::to_string(__LINE__) + " code=" + \
                    std::to_string((int)err__) + " \"" + hipGetErrorString(err__) + "\" in " #expr);       \
      return AWQ_ERR_HIP;                                                                                 \
    }                                                                                                     \
  } while (0)

#define AWQ_REQUIRE(cond, msg)                                       \
  do {                                                               \
    if (!(cond)) {                                                   \
      awq_set_error(std::string(__func__) + ": " + (msg));           \
      return AWQ_ERR_ARG;                                            \
    }                                                                \
  } while (0)

// Where row (head, position) of a key or value cache starts, in binary16 elements:
//   head * head_stride + (position >> shift) * block_stride + (position % 2^shift) * 128.
//   head major: [head][max_pos][128], the reference's arrangement (Inference.cu:676)
//     and that of the kernel-level entry points;
//   blocked: [position / 64][head][position % 64][128], the engine's own.  The rows
//     a step touches are then a prefix of the layer's cache whatever max_pos is, and
//     a head's 64 consecutive positions are still 16 KB in one piece.  Head major
//     they are n_heads islands max_pos * 256 bytes apart.
struct KvLayout {
  int32_t head_stride;
  int32_t block_stride;
  int32_t shift;
};
inline KvLayout kv_head_major(int64_t max_pos) { return KvLayout{(int32_t)(max_pos * 128), 0, 30}; }
inline KvLayout kv_blocked(int n_heads) { return KvLayout{64 * 128, n_heads * 64 * 128, 6}; }
__host__ __device__ inline int64_t kv_row(const KvLayout& kv, int head, int pos) {
  return (int64_t)head * kv.head_stride + (int64_t)(pos >> kv.shift) * kv.block_stride +
         (int64_t)(pos & ((1 << kv.shift) - 1)) * 128;
}

// Values that change from step to step live in device memory so that a
// captured graph can be replayed unchanged: kernels read them from here.
struct StepState {
  int32_t pos;        // position written to the KV cache this step
  int32_t len_lo;     // attended length for layers <  split
  int32_t len_hi;     // attended length for layers >= split
  int32_t token;      // prompt token to embed at the start of the step, -1 = keep the hidden state
  int32_t out_index;  // where the sampled token goes in the output array
  int32_t sample;     // 1 = run the sampler at the end of the step
  int32_t epoch;      // grows by the number of layers every step and never repeats within 2^16 launches: epoch +
                      // layer tags the vectors that a fused launch hands from workgroup to workgroup
};

// what the fused linear kernel does to its input and its output
enum LinearPrologue {
  PRO_NONE = 0,     // x is used as is
  PRO_RMSNORM = 1,  // x is the un-normalised hidden state: rmsNormKernel (Inference.cu:111-145) first
};
enum LinearEpilogue {
  EPI_STORE = 0,     // y = h(acc)
  EPI_RESIDUAL = 1,  // y = h(res + h(acc))                              Inference.cu:1149-1155
  EPI_GELU = 2,      // y = h(gelu(h(acc)))                              Inference.cu:271-279
  EPI_QKV_ROPE = 3,  // split, rotary on Q and K, K/V appended to the cache  Inference.cu:1070-1103
  EPI_ARGMAX = 4,    // y = h(acc) and the greedy token                  Inference.cu:1278-1290
};

struct LinearArgs {
  const void* wq = nullptr;       // repacked int4
  const half_t* scale = nullptr;  // [m/128]
  const half_t* zp = nullptr;     // [m/128]
  const half_t* x = nullptr;      // [k]
  half_t* y = nullptr;            // [m] ([hidden] rotated Q for EPI_QKV_ROPE)
  const half_t* res = nullptr;    // EPI_RESIDUAL: [m], may alias y
  int64_t m = 0, k = 0;
  int prologue = PRO_NONE;
  int epilogue = EPI_STORE;
  const half_t* gamma = nullptr;  // PRO_RMSNORM: [k]
  float eps = 0.0f;
  const half_t* cos_t = nullptr;  // EPI_QKV_ROPE
  const half_t* sin_t = nullptr;
  half_t* k_cache = nullptr;
  half_t* v_cache = nullptr;
  int32_t hidden = 0;
  int32_t pos = 0;
  int64_t max_pos = 0;
  KvLayout kv = {0, 0, 0};
  const StepState* dyn = nullptr;     // pos / out_index come from here when set
  unsigned long long* best = nullptr;  // EPI_ARGMAX: zero between launches
  int32_t* out_token = nullptr;
  int32_t* out_array = nullptr;
  // EPI_ARGMAX in the engine's decode step: the small launch that turns the best candidate into the token also
  // ends the step (keeps a copy of the hidden state, gathers the sampled token's embedding into it for the
  // next step, advances the step state)
  half_t* fin_hidden = nullptr;        // [fin_n], null = the launch only samples
  half_t* fin_hidden_last = nullptr;
  const uint8_t* fin_emb = nullptr;    // the embedding's token rows (launch_embed_rows), fin_n/2 bytes each
  const half_t* fin_emb_scale = nullptr;
  const half_t* fin_emb_zp = nullptr;
  int32_t fin_n = 0;
  StepState* fin_state = nullptr;
  int32_t fin_epoch_step = 0;          // what the step adds to the state's epoch (the number of layers)
};

// Greedy sampling key: an order-preserving integer image of a binary16 logit
// with NaN lowest, so that the reference's scan "strict > from index 0"
// (Inference.cu:1282-1289) becomes a maximum over (key, -index).
__host__ __device__ inline int32_t awq_logit_key(uint16_t bits) {
  if ((bits & 0x7fffu) > 0x7c00u) return INT32_MIN;  // NaN never wins
  if ((bits & 0x7fffu) == 0) return 0;               // -0 == +0 in a float compare
  return (bits & 0x8000u) ? -(int32_t)(bits & 0x7fffu) : (int32_t)bits;
}
__host__ __device__ inline unsigned long long awq_pack_candidate(int32_t key, uint32_t idx) {
  return ((unsigned long long)((uint32_t)key ^ 0x80000000u) << 32) | (uint32_t)(0xffffffffu - idx);
}

int launch_dequant(const uint8_t* packed, const half_t* scale, const half_t* zp, half_t* out, int64_t rows,
                   int64_t cols, int64_t n_groups, hipStream_t st);
int launch_repack(const uint8_t* in, void* out, int64_t m, int64_t k, hipStream_t st);
int64_t gemv_workspace_bytes(int64_t m, int64_t k);
int launch_gemv(const LinearArgs& a, hipStream_t st);
int64_t gemm_workspace_bytes(int64_t m, int64_t k, int64_t M);
int gemm_plan(int64_t m, int64_t k, int64_t M, int has_workspace);
int launch_gemm(const void* wq, const half_t* scale, const half_t* zp, int64_t m, int64_t k, const half_t* x,
                half_t* y, int64_t M, int zp_integral, int epilogue, const half_t* res, void* workspace,
                int64_t workspace_bytes, hipStream_t st);
int launch_rmsnorm(const half_t* x, const half_t* gamma, half_t* out, int64_t n, float eps, hipStream_t st);
int launch_rope_kv_append(const half_t* qkv, const half_t* cos_t, const half_t* sin_t, half_t* q_out, half_t* kc,
                          half_t* vc, int n_heads, int64_t max_pos, KvLayout kv, int64_t pos, const StepState* dyn,
                          hipStream_t st);
// How the decode attention is launched, by an upper bound of the attended length
// (measured in the decode loop of the 36-layer model, where every layer's cache
// comes from HBM, and with the attention sweep of bench.py):
//   <= kAttnShortMax         as the next form;
//   <= kAttnOneWorkgroupMax  four workgroups per head, each with all of the head's keys and a
//        quarter of every value row, do everything: a handful of memory round trips on 128
//        compute units.  Above kAttnShortMax with the length in device memory the keys and values
//        of the first kAttnShortMax positions are requested before the length has arrived (one
//        memory round trip less: -0.15 us per launch, 794.3 -> 797.6 tok/s); a shorter sequence
//        would pay for rows it does not use, hence the bound of its own;
//   <= kAttnTwoLaunchMax     the keys are streamed by all compute units (scores and part
//        maxima to memory), a second launch with four workgroups per head does the rest,
//        one 64-position chunk per wavefront;
//   <= kAttnMergedMax        three launches: scores; exponentials, chunk sums and chunk
//        vectors per part (the exponentials are recomputed by every workgroup of a
//        head); ordered sum (17.7 us at 1536, 20.1 us at 2048 positions);
//   beyond                   four launches (26.5 us at 4096; three would take 29.1 us).
// Tokens per second over 128 decode steps, one launch against two: 691 / 685 at 568..696
// positions, 668 / 673 at 708..836 with the switch at 768 -- the two forms meet near 700.
// (With one workgroup per head they met near 576: 716 against 683 tok/s at 448..576 positions
// and 669 against 649 at 708..836 is what the four workgroups per head brought.)
constexpr int64_t kAttnShortMax = 128;
constexpr int64_t kAttnOneWorkgroupMax = 704;
constexpr int64_t kAttnTwoLaunchMax = 1024;
constexpr int64_t kAttnMergedMax = 2048;
// the fused Wqkv + attention launch (qkv_attn.hip) covers attended lengths up to here: four 64-position chunks per
// wavefront of its workgroups (606 against 574 tok/s at 3500 positions, 564 against 558 at 4050: every workgroup
// reads all eight partial scores of every position, as many bytes as its share of the cache rows, so the gain
// ends here)
constexpr int64_t kFusedQkvAttnMax = 4096;
int64_t attention_workspace_bytes(int n_heads, int64_t max_pos);
int launch_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads, int64_t max_pos,
                     KvLayout kv, int64_t L, const StepState* dyn, int use_len_hi, int64_t len_bound, void* ws,
                     hipStream_t st);
int launch_attention_static(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                            int64_t max_pos, int64_t L, hipStream_t st);
int launch_prefill_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                             int64_t max_pos, KvLayout kv, int64_t pos0, int64_t M, int use_len_hi, hipStream_t st);
int launch_embed_batch(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                       const int32_t* tokens_dev, int64_t M, half_t* out, hipStream_t st);
int launch_rmsnorm_batch(const half_t* x, const half_t* gamma, half_t* out, int64_t n, int64_t M, float eps,
                         hipStream_t st);
int launch_rope_kv_append_batch(const half_t* qkv, const half_t* cos_t, const half_t* sin_t, half_t* q_out,
                                half_t* kc, half_t* vc, int n_heads, int64_t max_pos, KvLayout kv, int64_t pos0,
                                int64_t M, hipStream_t st, half_t* k_parts = nullptr, half_t* v_parts = nullptr,
                                int parts_pos = 0);
int launch_residual(const half_t* a, const half_t* b, half_t* out, int64_t n, hipStream_t st);
int launch_gelu(half_t* x, int64_t n, hipStream_t st);
int64_t argmax_workspace_bytes(int64_t n);
int launch_argmax(const half_t* logits, int64_t n, int32_t* out_token, void* ws, const StepState* dyn,
                  int32_t* out_array, hipStream_t st);
// token rows of the packed embedding: rows[tok][hidden/2], low nibble = even hidden element
int launch_embed_rows(const uint8_t* packed, uint8_t* rows, int64_t hidden, int64_t vocab, hipStream_t st);
int launch_embed(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                 int32_t tok, const StepState* dyn, half_t* out, hipStream_t st);
int launch_set_state(StepState* dst, StepState v, hipStream_t st);
// Wo + residual and RMSNorm + W1 + GeLU of one layer in one launch (fused.hip)
int fused_wo_w1_supported(int64_t hidden, int64_t inter);
int launch_fused_wo_w1(const void* wo, const half_t* wo_scale, const half_t* wo_zp, const void* w1,
                       const half_t* w1_scale, const half_t* w1_zp, const half_t* gamma, float eps, const half_t* ctx,
                       half_t* hidden, half_t* mid, uint32_t* hid_tag, int32_t* status, const StepState* dyn, int layer,
                       int64_t hidden_size, int64_t inter, unsigned long long* stamps, hipStream_t st);
constexpr int kFusedStamps = 13;  // time stamps per workgroup of the instrumented fused launch
// RMSNorm + Wqkv + rotary + KV append and the attention of one layer in one launch (qkv_attn.hip), for attended
// lengths up to kAttnOneWorkgroupMax
int fused_qkv_attn_supported(int64_t hidden, int n_heads, hipStream_t st);
int64_t fused_qkv_attn_exchange_bytes(int n_heads);
int launch_fused_qkv_attn(const void* wq, const half_t* scale, const half_t* zp, int64_t m, const half_t* x,
                          const half_t* gamma, float eps, const half_t* cos_t, const half_t* sin_t, half_t* k_cache,
                          half_t* v_cache, KvLayout kv, half_t* k_parts, half_t* v_parts, int parts_pos, half_t* q_out,
                          half_t* ctx, uint32_t* score_tag, int32_t* status, const StepState* dyn, int layer,
                          int use_len_hi, int64_t len_bound, int n_heads, unsigned long long* stamps, hipStream_t st);
// the caches a second time in the order the fused launch reads them: [head][8][parts_pos][16]
int64_t fused_qkv_attn_parts_bytes(int n_heads, int64_t parts_pos);
int launch_kv_to_parts(const half_t* k_cache, const half_t* v_cache, KvLayout kv, half_t* k_parts, half_t* v_parts,
                       int n_heads, int parts_pos, int64_t pos0, int64_t n, hipStream_t st);
constexpr int kQkvStamps = 11;  // time stamps per workgroup of the instrumented launch
int launch_fill_zero(void* p, int64_t bytes, hipStream_t st);
int launch_copy(const void* src, void* dst, int64_t bytes, hipStream_t st);
