// The small per-token operators of the decode step, each restating one kernel
// of the reference with the same rounding points.
#include "common.hpp"

namespace {

// rmsNormKernel (Inference.cu:111-145): 256 strided partial sums (fma), the
// stride-halving tree of :130-135, then two binary16 multiplies per element.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const half_t* __restrict__ x, const half_t* __restrict__ gamma,
                                                      half_t* __restrict__ out, int n, float eps) {
  __shared__ float buf[256];
  const int tid = threadIdx.x;
  float acc = 0.0f;
  for (int i = tid; i < n; i += 256) {
    float v = (float)x[i];
    acc = __builtin_fmaf(v, v, acc);
  }
  buf[tid] = acc;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) buf[tid] += buf[tid + stride];
    __syncthreads();
  }
  float mean_sq = buf[0] / (float)n;
  half_t sc = (half_t)awq_rsqrtf(mean_sq + eps);
  for (int i = tid; i < n; i += 256) {
    half_t t = x[i] * sc;
    out[i] = t * gamma[i];
  }
}

// QKV split + applyRotaryKernel on Q and K + KV append
// (Inference.cu:1070-1103, 150-177).  One workgroup per head, one thread per
// rotary pair.
__global__ __launch_bounds__(64) void rope_kv_kernel(const half_t* __restrict__ qkv, const half_t* __restrict__ cos_t,
                                                     const half_t* __restrict__ sin_t, half_t* __restrict__ q_out,
                                                     half_t* __restrict__ kc, half_t* __restrict__ vc, int n_heads,
                                                     KvLayout kv, int pos_arg, const StepState* dyn) {
  const int pos = dyn ? dyn->pos : pos_arg;
  const int hd = blockIdx.x, i = threadIdx.x;
  const int H = n_heads * AWQ_HEAD_DIM;
  const half_t c = cos_t[(int64_t)pos * 64 + i], s = sin_t[(int64_t)pos * 64 + i];
  const int e = hd * AWQ_HEAD_DIM + 2 * i;
  const int64_t dst = kv_row(kv, hd, pos) + 2 * i;
  {
    half_t a = qkv[e], b = qkv[e + 1];
    half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    q_out[e] = ac - bs;
    q_out[e + 1] = as + bc;
  }
  {
    half_t a = qkv[H + e], b = qkv[H + e + 1];
    half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    kc[dst] = ac - bs;
    kc[dst + 1] = as + bc;
  }
  vc[dst] = qkv[2 * H + e];
  vc[dst + 1] = qkv[2 * H + e + 1];
}

// residual add lambda (Inference.cu:1149-1155)
__global__ __launch_bounds__(256) void residual_kernel(const half_t* a, const half_t* b, half_t* out, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = a[i] + b[i];
}

// geluKernel (Inference.cu:271-279)
__global__ __launch_bounds__(256) void gelu_kernel(half_t* x, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = to_half_rn(awq_gelu_f32((float)x[i]));
}

// gather lambda (Inference.cu:1310-1324) straight from the packed [hidden][vocab]
// embedding: element (idx, tok) is nibble tok&1 of byte idx*(vocab/2) + tok/2.
__global__ __launch_bounds__(256) void embed_kernel(const uint8_t* __restrict__ packed,
                                                    const half_t* __restrict__ scale, const half_t* __restrict__ zp,
                                                    int hidden, int64_t vocab, int tok_arg, const StepState* dyn,
                                                    half_t* __restrict__ out) {
  int tok = tok_arg;
  if (dyn) {
    tok = dyn->token;
    if (tok < 0) return;  // keep the hidden state (Inference.cu:1357)
  }
  int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= hidden) return;
  int g = (tok / AWQ_GROUP_SIZE) % (hidden / AWQ_GROUP_SIZE);
  uint32_t byte = packed[(int64_t)idx * (vocab >> 1) + (tok >> 1)];
  uint32_t q = (tok & 1) ? (byte >> 4) : (byte & 15u);
  half_t d = (half_t)(float)q - zp[g];
  out[idx] = d * scale[g];
}

// One-time transposition of the packed [hidden][vocab] embedding into token rows: byte j of row tok holds
// the weights of hidden elements 2j (low nibble) and 2j+1 (high nibble) of token tok, so that the gather
// lambda's column (Inference.cu:1310-1324) is hidden/2 contiguous bytes.  A workgroup turns a tile of 128
// hidden elements by 128 tokens through LDS; both sides move 64-byte runs.
__global__ __launch_bounds__(256) void embed_rows_kernel(const uint8_t* __restrict__ packed, uint8_t* __restrict__ rows,
                                                         int hidden, int64_t vocab) {
  __shared__ uint32_t tile[128][17];  // [hidden element][16 words = 128 tokens], one word of skew
  const int tid = threadIdx.x;
  const int64_t tok0 = (int64_t)blockIdx.x * 128;
  const int idx0 = blockIdx.y * 128;
  const int c = tid & 15, r0 = tid >> 4;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = r0 + 16 * i;
    tile[r][c] = *reinterpret_cast<const uint32_t*>(packed + (int64_t)(idx0 + r) * (vocab >> 1) + (tok0 >> 1) + 4 * c);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int t = r0 + 16 * i;  // token of the tile; this thread writes bytes 4c..4c+3 of its row
    uint32_t out = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int e = 8 * c + 2 * b;
      const uint32_t lo = (tile[e][t >> 3] >> (4 * (t & 7))) & 15u;
      const uint32_t hi = (tile[e + 1][t >> 3] >> (4 * (t & 7))) & 15u;
      out |= (lo | (hi << 4)) << (8 * b);
    }
    *reinterpret_cast<uint32_t*>(rows + (tok0 + t) * (hidden >> 1) + (idx0 >> 1) + 4 * c) = out;
  }
}

// Greedy sampling (Inference.cu:1278-1290) without leaving the device.
__global__ __launch_bounds__(256) void argmax_kernel(const uint16_t* __restrict__ logits, int64_t n,
                                                     unsigned long long* cand, int32_t* counter, int32_t* out_token,
                                                     const StepState* dyn, int32_t* out_array) {
  __shared__ unsigned long long sh[256];
  const int tid = threadIdx.x;
  unsigned long long best = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + tid; i < n; i += (int64_t)gridDim.x * 256) {
    unsigned long long c = awq_pack_candidate(awq_logit_key(logits[i]), (uint32_t)i);
    best = c > best ? c : best;
  }
  sh[tid] = best;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) sh[tid] = sh[tid] > sh[tid + stride] ? sh[tid] : sh[tid + stride];
    __syncthreads();
  }
  __shared__ int is_last;
  if (tid == 0) {
    __hip_atomic_store(&cand[blockIdx.x], sh[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();
    int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (old == (int)gridDim.x - 1);
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();
  best = 0;
  for (int b = tid; b < (int)gridDim.x; b += 256) {
    unsigned long long c = __hip_atomic_load(&cand[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    best = c > best ? c : best;
  }
  sh[tid] = best;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) sh[tid] = sh[tid] > sh[tid + stride] ? sh[tid] : sh[tid + stride];
    __syncthreads();
  }
  if (tid == 0) {
    int32_t tok = (int32_t)(0xffffffffu - (uint32_t)(sh[0] & 0xffffffffull));
    // a NaN at index 0 beats everything in the reference's scan (every '>' is false)
    if ((logits[0] & 0x7fffu) > 0x7c00u) tok = 0;
    *out_token = tok;
    if (out_array && dyn) out_array[dyn->out_index] = tok;
    __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

__global__ void set_state_kernel(StepState* dst, StepState v) {
  if (threadIdx.x == 0) *dst = v;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, int64_t n_words) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * 256) p[i] = 0;
}

__global__ __launch_bounds__(256) void copy_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                   int64_t n_words) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_words; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}

}  // namespace

int launch_copy(const void* src, void* dst, int64_t bytes, hipStream_t st) {
  AWQ_REQUIRE(bytes % 4 == 0 && bytes >= 0, "byte count must be a multiple of 4");
  if (bytes == 0) return AWQ_OK;
  int64_t words = bytes / 4, blocks = (words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)src, (uint32_t*)dst, words);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rmsnorm(const half_t* x, const half_t* gamma, half_t* out, int64_t n, float eps, hipStream_t st) {
  AWQ_REQUIRE(n > 0 && n % 256 == 0 && n < (1 << 30), "n must be a positive multiple of 256");
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(256), 0, st, x, gamma, out, (int)n, eps);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rope_kv_append(const half_t* qkv, const half_t* cos_t, const half_t* sin_t, half_t* q_out, half_t* kc,
                          half_t* vc, int n_heads, int64_t max_pos, KvLayout kv, int64_t pos, const StepState* dyn,
                          hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0, "n_heads and max_pos must be positive");
  AWQ_REQUIRE(dyn || (pos >= 0 && pos < max_pos), "pos out of range");
  hipLaunchKernelGGL(rope_kv_kernel, dim3(n_heads), dim3(64), 0, st, qkv, cos_t, sin_t, q_out, kc, vc, n_heads,
                     kv, (int)pos, dyn);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_residual(const half_t* a, const half_t* b, half_t* out, int64_t n, hipStream_t st) {
  AWQ_REQUIRE(n > 0, "n must be positive");
  hipLaunchKernelGGL(residual_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, b, out, n);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_gelu(half_t* x, int64_t n, hipStream_t st) {
  AWQ_REQUIRE(n > 0, "n must be positive");
  hipLaunchKernelGGL(gelu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, n);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_embed(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                 int32_t tok, const StepState* dyn, half_t* out, hipStream_t st) {
  AWQ_REQUIRE(hidden > 0 && hidden % 128 == 0 && vocab > 0 && vocab % 2 == 0, "bad embedding shape");
  AWQ_REQUIRE(dyn || (tok >= 0 && tok < vocab), "token id out of range");
  hipLaunchKernelGGL(embed_kernel, dim3((unsigned)((hidden + 255) / 256)), dim3(256), 0, st, packed, scale, zp,
                     (int)hidden, vocab, tok, dyn, out);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_embed_rows(const uint8_t* packed, uint8_t* rows, int64_t hidden, int64_t vocab, hipStream_t st) {
  AWQ_REQUIRE(hidden > 0 && hidden % 128 == 0 && vocab > 0 && vocab % 128 == 0, "bad embedding shape");
  hipLaunchKernelGGL(embed_rows_kernel, dim3((unsigned)(vocab / 128), (unsigned)(hidden / 128)), dim3(256), 0, st,
                     packed, rows, (int)hidden, vocab);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

static int argmax_blocks(int64_t n) {
  int64_t b = (n + 2047) / 2048;
  if (b < 1) b = 1;
  if (b > 256) b = 256;
  return (int)b;
}

int64_t argmax_workspace_bytes(int64_t n) { return (int64_t)argmax_blocks(n) * 8 + 64; }

int launch_argmax(const half_t* logits, int64_t n, int32_t* out_token, void* ws, const StepState* dyn,
                  int32_t* out_array, hipStream_t st) {
  AWQ_REQUIRE(n > 0 && n < (1ll << 32), "n out of range");
  AWQ_REQUIRE(ws != nullptr, "workspace required");
  int blocks = argmax_blocks(n);
  int32_t* counter = (int32_t*)ws;
  unsigned long long* cand = (unsigned long long*)((char*)ws + 64);
  hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(256), 0, st, (const uint16_t*)logits, n, cand, counter,
                     out_token, dyn, out_array);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_set_state(StepState* dst, StepState v, hipStream_t st) {
  hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, st, dst, v);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_fill_zero(void* p, int64_t bytes, hipStream_t st) {
  AWQ_REQUIRE(bytes % 4 == 0, "byte count must be a multiple of 4");
  if (bytes == 0) return AWQ_OK;
  int64_t words = bytes / 4;
  int64_t blocks = (words + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (uint32_t*)p, words);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
