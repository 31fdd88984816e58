// The per-token operators of the prompt loop (Inference.cu:1304-1343) for M
// prompt positions at once.  Each token goes through exactly the arithmetic of
// the one-token kernels (same rounding points, same summation orders); only
// the matrix products between them change, from M matrix-vector products to
// one product on the matrix cores.
//
// Activations are [M][n] row-major: token t's vector is contiguous, which is
// what the reference's column-per-token cublasGemmEx operands (ldb = k,
// ldc = m) look like in memory.
#include "common.hpp"

namespace {

// gather lambda, Inference.cu:1310-1324, for M token ids
__global__ __launch_bounds__(256) void embed_batch_kernel(const uint8_t* __restrict__ packed,
                                                          const half_t* __restrict__ scale,
                                                          const half_t* __restrict__ zp, int hidden, int64_t vocab,
                                                          const int32_t* __restrict__ tokens,
                                                          half_t* __restrict__ out) {
  const int tok = tokens[blockIdx.y];
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= hidden) return;
  const int g = (tok / AWQ_GROUP_SIZE) % (hidden / AWQ_GROUP_SIZE);
  const uint32_t byte = packed[(int64_t)idx * (vocab >> 1) + (tok >> 1)];
  const uint32_t q = (tok & 1) ? (byte >> 4) : (byte & 15u);
  const half_t d = (half_t)(float)q - zp[g];
  out[(int64_t)blockIdx.y * hidden + idx] = d * scale[g];
}

// rmsNormKernel, Inference.cu:111-145, one workgroup per token
__global__ __launch_bounds__(256) void rmsnorm_batch_kernel(const half_t* __restrict__ x,
                                                            const half_t* __restrict__ gamma,
                                                            half_t* __restrict__ out, int n, float eps) {
  __shared__ float buf[256];
  const int tid = threadIdx.x;
  x += (int64_t)blockIdx.x * n;
  out += (int64_t)blockIdx.x * n;
  float acc = 0.0f;
  for (int i = tid; i < n; i += 256) {
    const float v = (float)x[i];
    acc = __builtin_fmaf(v, v, acc);
  }
  buf[tid] = acc;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) buf[tid] += buf[tid + stride];
    __syncthreads();
  }
  const half_t sc = (half_t)awq_rsqrtf(buf[0] / (float)n + eps);
  for (int i = tid; i < n; i += 256) {
    const half_t t = x[i] * sc;
    out[i] = t * gamma[i];
  }
}

// QKV split, rotary on Q and K, KV append (Inference.cu:1070-1103, 150-177) for
// token blockIdx.y at position pos0 + blockIdx.y; one workgroup per head.
__global__ __launch_bounds__(64) void rope_kv_batch_kernel(const half_t* __restrict__ qkv,
                                                           const half_t* __restrict__ cos_t,
                                                           const half_t* __restrict__ sin_t,
                                                           half_t* __restrict__ q_out, half_t* __restrict__ kc,
                                                           half_t* __restrict__ vc, int n_heads, int64_t max_pos,
                                                           int pos0) {
  const int tok = blockIdx.y, pos = pos0 + tok;
  const int hd = blockIdx.x, i = threadIdx.x;
  const int H = n_heads * AWQ_HEAD_DIM;
  qkv += (int64_t)tok * 3 * H;
  q_out += (int64_t)tok * H;
  const half_t c = cos_t[(int64_t)pos * 64 + i], s = sin_t[(int64_t)pos * 64 + i];
  const int e = hd * AWQ_HEAD_DIM + 2 * i;
  const int64_t dst = ((int64_t)hd * max_pos + pos) * AWQ_HEAD_DIM + 2 * i;
  {
    const half_t a = qkv[e], b = qkv[e + 1];
    const half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    q_out[e] = ac - bs;
    q_out[e + 1] = as + bc;
  }
  {
    const half_t a = qkv[H + e], b = qkv[H + e + 1];
    const half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    kc[dst] = ac - bs;
    kc[dst + 1] = as + bc;
  }
  vc[dst] = qkv[2 * H + e];
  vc[dst + 1] = qkv[2 * H + e + 1];
}

}  // namespace

int launch_embed_batch(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                       const int32_t* tokens_dev, int64_t M, half_t* out, hipStream_t st) {
  AWQ_REQUIRE(hidden > 0 && hidden % 128 == 0 && vocab > 0 && vocab % 2 == 0, "bad embedding shape");
  AWQ_REQUIRE(M >= 1 && M <= 65535 && tokens_dev, "token count out of range");
  hipLaunchKernelGGL(embed_batch_kernel, dim3((unsigned)((hidden + 255) / 256), (unsigned)M), dim3(256), 0, st, packed,
                     scale, zp, (int)hidden, vocab, tokens_dev, out);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rmsnorm_batch(const half_t* x, const half_t* gamma, half_t* out, int64_t n, int64_t M, float eps,
                         hipStream_t st) {
  AWQ_REQUIRE(n > 0 && n % 256 == 0 && n < (1 << 30), "n must be a positive multiple of 256");
  AWQ_REQUIRE(M >= 1 && M < (1ll << 31), "token count out of range");
  hipLaunchKernelGGL(rmsnorm_batch_kernel, dim3((unsigned)M), dim3(256), 0, st, x, gamma, out, (int)n, eps);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rope_kv_append_batch(const half_t* qkv, const half_t* cos_t, const half_t* sin_t, half_t* q_out,
                                half_t* kc, half_t* vc, int n_heads, int64_t max_pos, int64_t pos0, int64_t M,
                                hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0, "n_heads and max_pos must be positive");
  AWQ_REQUIRE(M >= 1 && M <= 65535 && pos0 >= 0 && pos0 + M <= max_pos, "positions out of range");
  hipLaunchKernelGGL(rope_kv_batch_kernel, dim3((unsigned)n_heads, (unsigned)M), dim3(64), 0, st, qkv, cos_t, sin_t,
                     q_out, kc, vc, n_heads, max_pos, (int)pos0);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
