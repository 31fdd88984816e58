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
//
// One workgroup of NW wavefronts per head (16 for decode).  Scores: the
// positions go round the wavefronts in groups of 4, so all wavefronts stream
// keys even for short sequences.  Context: one wavefront per chunk.
#include "common.hpp"

namespace {

constexpr int kMaxChunks = 1024;    // 65536 positions
constexpr int kLdsPositions = 8192; // scores kept in LDS up to this length
constexpr int kLdsChunks = 32;      // chunk vectors kept in LDS up to this many chunks
constexpr int kWaves = 16;   // wavefronts per workgroup of the decode variants
constexpr int kThreads = kWaves * 64;

// v + (value of lane ^ mask) inside a row of 16 lanes.  After the xor-1 and
// xor-2 steps all four lanes of a quad hold the same sum, so mirroring inside
// 8 (resp. 16) lanes fetches exactly what an xor with 4 (resp. 8) would.
__device__ __forceinline__ float dpp_add_xor1(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_add_xor2(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_add_half_mirror(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_add_mirror(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));
}
__device__ __forceinline__ float xor_add(float v, int mask) { return v + __shfl_xor(v, mask, 64); }

// sum over the 16 lanes of a row, adjacent pairs first
__device__ __forceinline__ float row16_tree_sum(float v) {
  v = dpp_add_xor1(v);
  v = dpp_add_xor2(v);
  v = dpp_add_half_mirror(v);
  v = dpp_add_mirror(v);
  return v;
}
// sum over the 64 lanes of a wavefront, adjacent pairs first
__device__ __forceinline__ float wave_tree_sum(float v) {
  v = row16_tree_sum(v);
  v = xor_add(v, 16);
  v = xor_add(v, 32);
  return v;
}

// BATCH: blockIdx.y is a prompt token at position L_arg + blockIdx.y with its
// own query and output rows ([token][head][128]); it attends the positions the
// prompt loop gives it (Inference.cu:1118 read before or after :1331):
// max(pos, 1) when use_len_hi is 0, pos + 1 otherwise.
// NW wavefronts; SCAP positions of scores and CCAP chunks (sums, and vectors
// when LDS_CV) fit the LDS arrays.
template <bool LDS_SCORES, bool LDS_CV, bool BATCH, int NW, int SCAP, int CCAP>
__global__ __launch_bounds__(NW * 64) void attention_kernel(const half_t* __restrict__ q,
                                                             const half_t* __restrict__ kc,
                                                             const half_t* __restrict__ vc, half_t* __restrict__ ctx,
                                                             int64_t max_pos, int L_arg, const StepState* dyn,
                                                             int use_len_hi, float* __restrict__ ws_scores,
                                                             float* __restrict__ ws_cv, int max_chunks) {
  __shared__ float cs[CCAP];
  __shared__ float wmax[NW];
  __shared__ float s_lds[LDS_SCORES ? SCAP : 1];
  __shared__ float cv_lds[LDS_CV ? CCAP * AWQ_HEAD_DIM : 1];
  int L;
  if (BATCH) {
    const int pos = L_arg + blockIdx.y;
    L = use_len_hi ? pos + 1 : (pos > 1 ? pos : 1);
    q += (int64_t)blockIdx.y * gridDim.x * AWQ_HEAD_DIM;
    ctx += (int64_t)blockIdx.y * gridDim.x * AWQ_HEAD_DIM;
  } else {
    L = dyn ? (use_len_hi ? dyn->len_hi : dyn->len_lo) : L_arg;
  }
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* kh = kc + (int64_t)head * max_pos * AWQ_HEAD_DIM;
  const half_t* vh = vc + (int64_t)head * max_pos * AWQ_HEAD_DIM;
  float* s = LDS_SCORES ? s_lds : ws_scores + (int64_t)head * max_pos;
  float* cv = LDS_CV ? cv_lds : ws_cv + (int64_t)head * max_chunks * AWQ_HEAD_DIM;
  const int nchunks = (L + 63) >> 6;
  const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);  // Inference.cu:218

  float qf[8];
  {
    half8_t qv = *reinterpret_cast<const half8_t*>(q + head * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
  }

  // scores (Inference.cu:202-226) and their maximum (:229-233): groups of four
  // positions go round the wavefronts, six groups' loads in flight.  The values
  // of this wavefront's first chunk are requested right behind the first keys,
  // so that both arrive in one memory round trip.
  half8_t vv[16];
  float lmax = -1e9f;
  const int nquads = (L + 3) >> 2;
  for (int q0 = wave; q0 < nquads; q0 += 6 * NW) {
    half8_t kv[6];
#pragma unroll
    for (int u = 0; u < 6; ++u) {
      const int t = 4 * (q0 + u * NW) + tq;
      if (t < L) kv[u] = *reinterpret_cast<const half8_t*>(kh + (int64_t)t * AWQ_HEAD_DIM + 8 * dl);
    }
    if (q0 == wave && wave < nchunks) {
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) {
        const int t = (wave << 6) + 4 * nl + tq;
        if (t < L) vv[nl] = *reinterpret_cast<const half8_t*>(vh + (int64_t)t * AWQ_HEAD_DIM + 8 * dl);
      }
    }
#pragma unroll
    for (int u = 0; u < 6; ++u) {
      const int t = 4 * (q0 + u * NW) + tq;
      float part = 0.0f;
      if (t < L) {
#pragma unroll
        for (int i = 0; i < 8; ++i) part = __builtin_fmaf(qf[i], (float)kv[u][i], part);
      }
      part = row16_tree_sum(part);
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
  float mx = wmax[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) mx = fmaxf(mx, wmax[w]);

  // exponentials and their sum (Inference.cu:239-249), one wavefront per chunk
  for (int chunk = wave; chunk < nchunks; chunk += NW) {
    const int t = (chunk << 6) + lane;
    float e = 0.0f;
    if (t < L) {
      e = awq_expf(s[t] - mx);
      s[t] = e;
    }
    e = wave_tree_sum(e);
    if (lane == 0) cs[chunk] = e;
  }
  __syncthreads();
  float Z = cs[0];
  for (int c = 1; c < nchunks; ++c) Z += cs[c];

  // weighted sum of V (Inference.cu:251-265), one wavefront per chunk; the 16
  // loads of a chunk are issued together
  for (int chunk = wave; chunk < nchunks; chunk += NW) {
    const int base = chunk << 6;
    if (chunk != wave) {  // the first chunk's values were requested at the start
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) {
        const int t = base + 4 * nl + tq;
        if (t < L) vv[nl] = *reinterpret_cast<const half8_t*>(vh + (int64_t)t * AWQ_HEAD_DIM + 8 * dl);
      }
    }
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) {
      const int t = base + 4 * nl + tq;
      if (t < L) {
        const float p = s[t] / Z;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, (float)vv[nl][i], acc[i]);
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
                     int64_t L, const StepState* dyn, int use_len_hi, int64_t len_bound, void* ws, hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0 && max_pos <= (int64_t)kMaxChunks * 64, "max_pos must be in 1..65536");
  AWQ_REQUIRE(dyn || (L >= 1 && L <= max_pos), "attended length out of range");
  AWQ_REQUIRE(ws != nullptr, "workspace required");
  float* scores = (float*)ws;
  float* cv = scores + (int64_t)n_heads * max_pos;
  // With a device-side length the caller states an upper bound for it (it
  // decides where the scores live); with a length known here, the length itself.
  const int64_t bound = dyn ? (len_bound > 0 ? len_bound : max_pos) : L;
  const int mc = (int)chunks_for(max_pos);
  if (bound <= kLdsChunks * 64) {
    hipLaunchKernelGGL((attention_kernel<true, true, false, kWaves, kLdsChunks * 64, kLdsChunks>), dim3(n_heads),
                       dim3(kThreads), 0, st, q, kc, vc, ctx, max_pos,
                       (int)L, dyn, use_len_hi, scores, cv, mc);
  } else if (bound <= kLdsPositions) {
    hipLaunchKernelGGL((attention_kernel<true, false, false, kWaves, kLdsPositions, kMaxChunks>), dim3(n_heads),
                       dim3(kThreads), 0, st, q, kc, vc, ctx, max_pos,
                       (int)L, dyn, use_len_hi, scores, cv, mc);
  } else {
    hipLaunchKernelGGL((attention_kernel<false, false, false, kWaves, 1, kMaxChunks>), dim3(n_heads),
                       dim3(kThreads), 0, st, q, kc, vc, ctx,
                       max_pos, (int)L, dyn, use_len_hi, scores, cv, mc);
  }
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

// Attention of M consecutive prompt positions pos0 .. pos0+M-1, whose keys and
// values are already in the cache.  While the longest attended length fits the
// LDS variant all tokens go in one launch; beyond that, one launch per token.
int launch_attention_batch(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                           int64_t max_pos, int64_t pos0, int64_t M, int use_len_hi, void* ws, hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0 && max_pos <= (int64_t)kMaxChunks * 64, "max_pos must be in 1..65536");
  AWQ_REQUIRE(M >= 1 && M <= 65535 && pos0 >= 0 && pos0 + M <= max_pos, "positions out of range");
  AWQ_REQUIRE(ws != nullptr, "workspace required");
  // short prompts: small workgroups (4 wavefronts, 3 KiB of LDS), many of them per compute unit
  if (pos0 + M <= 256) {
    hipLaunchKernelGGL((attention_kernel<true, true, true, 4, 256, 4>), dim3(n_heads, (unsigned)M), dim3(256), 0, st,
                       q, kc, vc, ctx, max_pos, (int)pos0, nullptr, use_len_hi, nullptr, nullptr, 0);
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  if (pos0 + M <= kLdsChunks * 64) {
    hipLaunchKernelGGL((attention_kernel<true, true, true, kWaves, kLdsChunks * 64, kLdsChunks>),
                       dim3(n_heads, (unsigned)M), dim3(kThreads), 0, st, q, kc, vc, ctx, max_pos, (int)pos0, nullptr,
                       use_len_hi, nullptr, nullptr, 0);
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  const int64_t H = (int64_t)n_heads * AWQ_HEAD_DIM;
  for (int64_t t = 0; t < M; ++t) {
    const int64_t pos = pos0 + t;
    const int64_t L = use_len_hi ? pos + 1 : (pos > 1 ? pos : 1);
    if (int rc = launch_attention(q + t * H, kc, vc, ctx + t * H, n_heads, max_pos, L, nullptr, 0, 0, ws, st))
      return rc;
  }
  return AWQ_OK;
}
