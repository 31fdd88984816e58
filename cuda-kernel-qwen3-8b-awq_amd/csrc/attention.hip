// Single-query attention over the KV cache for decode: the math that the
// comments of attentionKernel (Inference.cu:201, 228, 258) describe, with the
// summation orders fixed so that a CPU evaluation can reproduce the bits:
//   dot product   16 lanes x 8 consecutive d as fma chains, adjacent-pair tree
//   sum of exps   chunks of 64 positions, adjacent-pair tree inside a chunk,
//                 chunks added in order
//   context       per chunk four interleaved fma chains (position mod 4),
//                 combined (0+1)+(2+3); chunk vectors added in order
// Cache layout [head][max_pos][128] FP16 (Inference.cu:1097): a position is one
// 256-byte row, so a wavefront load of 16 bytes per lane covers 4 positions.
#include "common.hpp"

namespace {

constexpr int kMaxChunks = 1024;  // 65536 positions

__device__ __forceinline__ float xor_add(float v, int mask) { return v + __shfl_xor(v, mask, 64); }

__global__ __launch_bounds__(256) void attention_kernel(const half_t* __restrict__ q, const half_t* __restrict__ kc,
                                                        const half_t* __restrict__ vc, half_t* __restrict__ ctx,
                                                        int64_t max_pos, int L_arg, const StepState* dyn,
                                                        int use_len_hi, float* __restrict__ ws_scores,
                                                        float* __restrict__ ws_cv, int max_chunks) {
  __shared__ float cs[kMaxChunks];
  __shared__ float wmax[4];
  const int L = dyn ? (use_len_hi ? dyn->len_hi : dyn->len_lo) : L_arg;
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* kh = kc + (int64_t)head * max_pos * AWQ_HEAD_DIM;
  const half_t* vh = vc + (int64_t)head * max_pos * AWQ_HEAD_DIM;
  float* s = ws_scores + (int64_t)head * max_pos;
  float* cv = ws_cv + (int64_t)head * max_chunks * AWQ_HEAD_DIM;
  const int nchunks = (L + 63) >> 6;
  const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);  // Inference.cu:218

  float qf[8];
  {
    half8_t qv = *reinterpret_cast<const half8_t*>(q + head * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
  }

  // scores (Inference.cu:202-226) and their maximum (:229-233)
  float lmax = -1e9f;
  for (int chunk = wave; chunk < nchunks; chunk += 4) {
    const int base = chunk << 6;
#pragma unroll 4
    for (int nl = 0; nl < 16; ++nl) {
      const int t = base + 4 * nl + tq;
      float part = 0.0f;
      if (t < L) {
        half8_t kv = *reinterpret_cast<const half8_t*>(kh + (int64_t)t * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
        for (int i = 0; i < 8; ++i) part = __builtin_fmaf(qf[i], (float)kv[i], part);
      }
      part = xor_add(part, 1);
      part = xor_add(part, 2);
      part = xor_add(part, 4);
      part = xor_add(part, 8);
      const float sc = part * scale;
      if (t < L) {
        if (dl == 0) s[t] = sc;
        lmax = fmaxf(lmax, sc);
      }
    }
  }
#pragma unroll
  for (int mask = 1; mask < 64; mask <<= 1) lmax = fmaxf(lmax, __shfl_xor(lmax, mask, 64));
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  const float mx = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));

  // exponentials and their sum (Inference.cu:239-249)
  for (int chunk = wave; chunk < nchunks; chunk += 4) {
    const int t = (chunk << 6) + lane;
    float e = 0.0f;
    if (t < L) {
      e = awq_expf(s[t] - mx);
      s[t] = e;
    }
#pragma unroll
    for (int mask = 1; mask < 64; mask <<= 1) e = xor_add(e, mask);
    if (lane == 0) cs[chunk] = e;
  }
  __syncthreads();
  float Z = cs[0];
  for (int c = 1; c < nchunks; ++c) Z += cs[c];

  // weighted sum of V (Inference.cu:251-265)
  for (int chunk = wave; chunk < nchunks; chunk += 4) {
    const int base = chunk << 6;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll 4
    for (int nl = 0; nl < 16; ++nl) {
      const int t = base + 4 * nl + tq;
      if (t < L) {
        const float p = s[t] / Z;
        half8_t vv = *reinterpret_cast<const half8_t*>(vh + (int64_t)t * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, (float)vv[i], acc[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[i] = xor_add(acc[i], 16);
      acc[i] = xor_add(acc[i], 32);
    }
    if (tq == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) cv[chunk * AWQ_HEAD_DIM + 8 * dl + i] = acc[i];
    }
  }
  __syncthreads();
  if (tid < AWQ_HEAD_DIM) {
    float out = cv[tid];
    for (int c = 1; c < nchunks; ++c) out += cv[c * AWQ_HEAD_DIM + tid];
    ctx[head * AWQ_HEAD_DIM + tid] = (half_t)out;
  }
}

}  // namespace

static int64_t chunks_for(int64_t max_pos) { return (max_pos + 63) / 64; }

int64_t attention_workspace_bytes(int n_heads, int64_t max_pos) {
  return (int64_t)n_heads * (max_pos + chunks_for(max_pos) * AWQ_HEAD_DIM) * 4;
}

int launch_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads, int64_t max_pos,
                     int64_t L, const StepState* dyn, int use_len_hi, void* ws, hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0 && max_pos <= (int64_t)kMaxChunks * 64, "max_pos must be in 1..65536");
  AWQ_REQUIRE(dyn || (L >= 1 && L <= max_pos), "attended length out of range");
  AWQ_REQUIRE(ws != nullptr, "workspace required");
  float* scores = (float*)ws;
  float* cv = scores + (int64_t)n_heads * max_pos;
  hipLaunchKernelGGL(attention_kernel, dim3(n_heads), dim3(256), 0, st, q, kc, vc, ctx, max_pos, (int)L, dyn,
                     use_len_hi, scores, cv, (int)chunks_for(max_pos));
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
