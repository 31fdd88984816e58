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
// Workgroups of NW wavefronts (16 for decode), kHeadParts per head.  Scores: the
// positions go round the wavefronts in groups of 4, so all wavefronts stream
// keys even for short sequences.  Context: one wavefront per chunk.
#include "common.hpp"

#include <mutex>

namespace {

constexpr int kMaxChunks = 1024;    // 65536 positions
constexpr int kLdsChunks = 32;      // chunk vectors kept in LDS up to this many chunks
constexpr int kWaves = 16;   // wavefronts per workgroup of the decode variants
constexpr int kThreads = kWaves * 64;
constexpr int kSplit = 32;   // parts per head when the sequence is cut over several workgroups
constexpr int kHeadParts = 4;  // workgroups per head in attention_kernel, a quarter of the head's dimensions each
                               // (decode at 448..576 positions: 683 tok/s with one, 706 with two, 716 with four)

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
// v + (value of lane ^ 16), v + (value of lane ^ 32): gfx950's lane-swap instructions exchange rows of 16 lanes
// (halves of the wavefront) between two registers, a register operation where a general shuffle is an LDS
// round trip.  After the swap a holds rows (0,0,2,2) and b rows (1,1,3,3) of v (resp. the low and the high
// half), so a + b is the sum in every lane; a + b and b + a are the same number.  The waits around the
// instruction are the data-hazard slots the compiler would insert if it saw it.
__device__ __forceinline__ void swap16(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap32(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float add_xor16(float v) {
  float a = v, b = v;
  swap16(a, b);
  return a + b;
}
__device__ __forceinline__ float add_xor32(float v) {
  float a = v, b = v;
  swap32(a, b);
  return a + b;
}
// maximum over the 64 lanes of a wavefront, in every lane (the maximum does not depend on the order)
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true)));
  float a = v, b = v;
  swap16(a, b);
  v = fmaxf(a, b);
  a = v, b = v;
  swap32(a, b);
  return fmaxf(a, b);
}

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
  v = add_xor16(v);
  v = add_xor32(v);
  return v;
}

// NW wavefronts; SCAP positions of scores and CCAP chunks (sums and vectors)
// fit the LDS arrays.  Longer sequences take the split kernels further down.
// FROM_SCORES: the scores and the maxima of their kSplit parts were left in memory
// by attn_scores_kernel (all compute units stream the keys); this launch does the
// rest of the head.
// DS: workgroups per head (blockIdx.y).  Every one of them computes the head's scores, exponentials and
// sums (the same instructions on the same data: the same bits) and then the context of its 128/DS of the
// head's dimensions, i.e. it reads all keys but only 1/DS of every value row.  One compute unit keeps only
// about 37 KB of requests in flight, so the bytes a unit has to pull set the time beyond about 128 positions.
template <int NW, int SCAP, int CCAP, bool FROM_SCORES = false, int DS = 1, int EAGER = 0>
__global__ __launch_bounds__(NW * 64) void attention_kernel(const half_t* __restrict__ q,
                                                             const half_t* __restrict__ kc,
                                                             const half_t* __restrict__ vc, half_t* __restrict__ ctx,
                                                             KvLayout lay, int L_arg, const StepState* dyn,
                                                             int use_len_hi, int64_t max_pos,
                                                             const float* __restrict__ scores_g,
                                                             const float* __restrict__ pmax_g) {
  __shared__ float cs[CCAP];
  __shared__ float wmax[NW];
  __shared__ float s[SCAP];
  constexpr int DP = AWQ_HEAD_DIM / DS;  // dimensions of this workgroup
  constexpr int DL = 8 / DS;             // dimensions per lane in the context phase
  typedef _Float16 vrow_t __attribute__((ext_vector_type(DL)));
  __shared__ float cv[CCAP * DP];
  const int L = dyn ? (use_len_hi ? dyn->len_hi : dyn->len_lo) : L_arg;
  const int head = blockIdx.x;
  const int d0 = blockIdx.y * DP;  // first dimension of this workgroup
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* kh = kc;
  const half_t* vh = vc;
  // Row addresses.  Rows 64 positions apart are a constant apart in both cache arrangements (whole blocks of 64
  // positions, or one run per head), and with 16 wavefronts the groups of a round are 64 positions apart, so a
  // wavefront's requests are one row address plus multiples of a constant instead of a 64-bit row computation
  // per request (18 of them before the first request left: 0.3 us of the launch).
  static_assert(4 * NW == 64, "groups of a round are one block of 64 positions apart");
  const int64_t step64 = kv_row(lay, 0, 64) - kv_row(lay, 0, 0);
  const int64_t head0 = kv_row(lay, head, 0);
  auto key_row = [&](int t) -> const half_t* {  // this lane's 8 elements of row t
    return kh + head0 + (int64_t)(t >> 6) * step64 + (t & 63) * AWQ_HEAD_DIM + 8 * dl;
  };
  auto value_row = [&](int chunk) -> const half_t* {  // this lane's elements of row 64 chunk + tq
    return vh + head0 + (int64_t)chunk * step64 + tq * AWQ_HEAD_DIM + d0 + DL * dl;
  };
  const int nchunks = (L + 63) >> 6;
  const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);  // Inference.cu:218

  vrow_t vv[16];
  float mx;
  if constexpr (FROM_SCORES) {
    // the values of this wavefront's first chunk travel while the scores arrive
    if (wave < nchunks) {
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) {
        const int t = (wave << 6) + 4 * nl + tq;
        if (t < L) vv[nl] = *reinterpret_cast<const vrow_t*>(value_row(wave) + nl * (4 * AWQ_HEAD_DIM));
      }
    }
    for (int t = tid; t < L; t += NW * 64) s[t] = scores_g[(int64_t)head * max_pos + t];
    mx = pmax_g[head * kSplit];
#pragma unroll
    for (int i = 1; i < kSplit; ++i) mx = fmaxf(mx, pmax_g[head * kSplit + i]);
    __syncthreads();
  } else {
  float qf[8];
  {
    half8_t qv = *reinterpret_cast<const half8_t*>(q + head * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
  }

  // scores (Inference.cu:202-226) and their maximum (:229-233): groups of four
  // positions go round the wavefronts, six groups' loads in flight.  The values
  // of this wavefront's first chunk are requested right behind the first keys,
  // so that both arrive in one memory round trip.  The keys and values of the
  // first EAGER positions are requested before the attended length is known
  // (it sits in memory, a round trip of its own); rows past the length are valid
  // cache memory and are never used.
  constexpr int kEagerGroups = EAGER / (4 * NW);
  static_assert(kEagerGroups <= 6 && EAGER % 64 == 0 && EAGER % (4 * NW) == 0, "eager part of the first trip");
  // (an eager launch is only made for caches of at least EAGER positions, so its rows need no clamp)
  half8_t kv[6];
  const half_t* const k_wave = key_row(4 * wave + tq);
#pragma unroll
  for (int u = 0; u < kEagerGroups; ++u) kv[u] = *reinterpret_cast<const half8_t*>(k_wave + u * step64);
  if (wave < EAGER / 64) {
    const half_t* const v_wave = value_row(wave);
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) vv[nl] = *reinterpret_cast<const vrow_t*>(v_wave + nl * (4 * AWQ_HEAD_DIM));
  }
  float lmax = -1e9f;
  const int nquads = (L + 3) >> 2;
  for (int q0 = wave; q0 < nquads; q0 += 6 * NW) {
    const bool first = q0 == wave;
    const half_t* const k_round = key_row(4 * q0 + tq);
#pragma unroll
    for (int u = 0; u < 6; ++u) {
      const int t = 4 * (q0 + u * NW) + tq;
      if (t < L && !(first && u < kEagerGroups)) kv[u] = *reinterpret_cast<const half8_t*>(k_round + u * step64);
    }
    if (first && wave >= EAGER / 64 && wave < nchunks) {
      const half_t* const v_wave = value_row(wave);
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) {
        const int t = (wave << 6) + 4 * nl + tq;
        if (t < L) vv[nl] = *reinterpret_cast<const vrow_t*>(v_wave + nl * (4 * AWQ_HEAD_DIM));
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
  lmax = wave_max(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  mx = wmax[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) mx = fmaxf(mx, wmax[w]);
  }

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
  // A wavefront without a chunk among the first NW leaves zeros in its places: the sums below then add the
  // first NW entries unconditionally (x + 0 is x for the non-negative sums and for the chunk vectors, which
  // are never -0: every chain starts at +0)
  constexpr int kBatch = CCAP < NW ? CCAP : NW;
  if (wave >= nchunks && wave < kBatch) {
    if (lane == 0) cs[wave] = 0.0f;
    if (lane < DP) cv[wave * DP + lane] = 0.0f;
  }
  __syncthreads();
  // the chunk sums, added in chunk order; the first reads are issued together (a read per term is an LDS
  // round trip per chunk, serialised by the additions)
  float Z;
  {
    float zc[kBatch];
#pragma unroll
    for (int c = 0; c < kBatch; ++c) zc[c] = cs[c];
    Z = zc[0];
#pragma unroll
    for (int c = 1; c < kBatch; ++c) Z += zc[c];
    for (int c = kBatch; c < nchunks; ++c) Z += cs[c];
  }

  // weighted sum of V (Inference.cu:251-265), one wavefront per chunk; the 16
  // loads of a chunk are issued together
  for (int chunk = wave; chunk < nchunks; chunk += NW) {
    const int base = chunk << 6;
    if (chunk != wave) {  // the first chunk's values were requested at the start
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) {
        const int t = base + 4 * nl + tq;
        if (t < L) vv[nl] = *reinterpret_cast<const vrow_t*>(value_row(chunk) + nl * (4 * AWQ_HEAD_DIM));
      }
    }
    // one division per position (lane = position in the chunk), handed to the 16 lanes that
    // multiply that position's values
    const float p_lane = base + lane < L ? s[base + lane] / Z : 0.0f;
    float acc[DL];
#pragma unroll
    for (int i = 0; i < DL; ++i) acc[i] = 0.0f;
    // all 16 exchanges are issued before the first product, and a position past the length keeps the sum
    // by a select, not a branch: with a branch per position the compiler waits for every exchange (an LDS
    // round trip) before it issues the next, 16 round trips in a row
    float pp[16];
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) pp[nl] = __shfl(p_lane, 4 * nl + tq, 64);
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) {
      const bool in = base + 4 * nl + tq < L;
#pragma unroll
      for (int i = 0; i < DL; ++i) {
        const float r = __builtin_fmaf(pp[nl], (float)vv[nl][i], acc[i]);
        acc[i] = in ? r : acc[i];
      }
    }
#pragma unroll
    for (int i = 0; i < DL; ++i) {
      acc[i] = add_xor16(acc[i]);
      acc[i] = add_xor32(acc[i]);
    }
    if (tq == 0) {
#pragma unroll
      for (int i = 0; i < DL; ++i) cv[chunk * DP + DL * dl + i] = acc[i];
    }
  }
  __syncthreads();
  if (tid < DP) {
    float oc[kBatch];
#pragma unroll
    for (int c = 0; c < kBatch; ++c) oc[c] = cv[c * DP + tid];
    float out = oc[0];
#pragma unroll
    for (int c = 1; c < kBatch; ++c) out += oc[c];
    for (int c = kBatch; c < nchunks; ++c) out += cv[c * DP + tid];
    ctx[head * AWQ_HEAD_DIM + d0 + tid] = (half_t)out;
  }
}

// ---------------------------------------------------------------------------
// Long sequences: the same computation cut along the sequence, kSplit parts
// (contiguous ranges of 64-position chunks) per head, so that a few hundred
// workgroups stream the cache instead of one per head.  The summation orders
// are unchanged -- every chunk is still summed by one wavefront, chunk results
// are added in chunk order -- so the result is bit-identical to the one-kernel
// path.  Four launches: scores and part maxima; exponentials and chunk sums;
// chunk context vectors; their ordered sum.  Scores, chunk sums, chunk vectors
// and part maxima live in the workspace.
// ---------------------------------------------------------------------------
constexpr int kSplitWaves = 4;     // wavefronts per workgroup of the split kernels

struct SplitArgs {
  const half_t* q;
  const half_t* kc;
  const half_t* vc;
  half_t* ctx;
  int64_t max_pos;
  KvLayout kv;
  int L_arg;
  const StepState* dyn;
  int use_len_hi;
  float* scores;  // [head][max_pos]
  float* cv;      // [head][max_chunks][128]
  float* cs;      // [head][max_chunks]
  float* pmax;    // [head][kSplit]
  int max_chunks;
};

__device__ __forceinline__ int split_len(const SplitArgs& a) {
  return a.dyn ? (a.use_len_hi ? a.dyn->len_hi : a.dyn->len_lo) : a.L_arg;
}
// chunk range [lo, hi) of part blockIdx.y
__device__ __forceinline__ void split_range(int nchunks, int* lo, int* hi) {
  const int per = (nchunks + kSplit - 1) / kSplit;
  *lo = min((int)blockIdx.y * per, nchunks);
  *hi = min(*lo + per, nchunks);
}

// scores (Inference.cu:202-226) of this part and their maximum (:229-233)
__global__ __launch_bounds__(kSplitWaves * 64) void attn_scores_kernel(SplitArgs a) {
  __shared__ float wmax[kSplitWaves];
  const int L = split_len(a);
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* kh = a.kc;
  const KvLayout lay = a.kv;
  float* s = a.scores + (int64_t)head * a.max_pos;
  int c_lo, c_hi;
  split_range((L + 63) >> 6, &c_lo, &c_hi);
  const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);  // Inference.cu:218
  float qf[8];
  {
    half8_t qv = *reinterpret_cast<const half8_t*>(a.q + head * AWQ_HEAD_DIM + 8 * dl);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
  }
  float lmax = -1e9f;
  const int q_hi = min(c_hi * 16, (L + 3) >> 2);
  // eight groups of four positions per trip; the next trip's keys are in flight
  // while this one's are multiplied
  half8_t kv[8], kn[8];
  auto load_keys = [&](int q0, half8_t (&dst)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = 4 * (q0 + u * kSplitWaves) + tq;
      if (q0 + u * kSplitWaves < q_hi && t < L)
        dst[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(kh + kv_row(lay, head, t) + 8 * dl));
    }
  };
  load_keys(c_lo * 16 + wave, kn);
  for (int q0 = c_lo * 16 + wave; q0 < q_hi; q0 += 8 * kSplitWaves) {
#pragma unroll
    for (int u = 0; u < 8; ++u) kv[u] = kn[u];
    load_keys(q0 + 8 * kSplitWaves, kn);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = 4 * (q0 + u * kSplitWaves) + tq;
      const bool ok = q0 + u * kSplitWaves < q_hi && t < L;
      float part = 0.0f;
      if (ok) {
#pragma unroll
        for (int i = 0; i < 8; ++i) part = __builtin_fmaf(qf[i], (float)kv[u][i], part);
      }
      part = row16_tree_sum(part);
      const float sc = part * scale;
      if (ok) {
        if (dl == 0) s[t] = sc;
        lmax = fmaxf(lmax, sc);
      }
    }
  }
  lmax = wave_max(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  if (tid == 0) {
    float mx = wmax[0];
#pragma unroll
    for (int w = 1; w < kSplitWaves; ++w) mx = fmaxf(mx, wmax[w]);
    a.pmax[head * kSplit + blockIdx.y] = mx;
  }
}

// exponentials and chunk sums (Inference.cu:239-249), one wavefront per chunk
__global__ __launch_bounds__(kSplitWaves * 64) void attn_exp_kernel(SplitArgs a) {
  const int L = split_len(a);
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* s = a.scores + (int64_t)head * a.max_pos;
  int c_lo, c_hi;
  split_range((L + 63) >> 6, &c_lo, &c_hi);
  float mx = a.pmax[head * kSplit];
#pragma unroll
  for (int i = 1; i < kSplit; ++i) mx = fmaxf(mx, a.pmax[head * kSplit + i]);
  for (int chunk = c_lo + wave; chunk < c_hi; chunk += kSplitWaves) {
    const int t = (chunk << 6) + lane;
    float e = 0.0f;
    if (t < L) {
      e = awq_expf(s[t] - mx);
      s[t] = e;
    }
    e = wave_tree_sum(e);
    if (lane == 0) a.cs[(int64_t)head * a.max_chunks + chunk] = e;
  }
}

// weighted sums of V per chunk (Inference.cu:251-265), one wavefront per chunk.
// The normaliser Z is the ordered sum of all chunk sums: they go through LDS
// once per workgroup (every thread then adds them in order from broadcast reads;
// read straight from memory the same loop cost tens of microseconds per
// wavefront).  A lane divides one probability of the chunk and the lanes exchange
// them; the values stream in two halves so that loads stay in flight while the
// other half is multiplied.
__global__ __launch_bounds__(kSplitWaves * 64) void attn_pv_kernel(SplitArgs a) {
  extern __shared__ float zs[];  // the chunk sums of this head
  const int L = split_len(a);
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* vh = a.vc;
  const KvLayout lay = a.kv;
  const float* s = a.scores + (int64_t)head * a.max_pos;
  const float* cs = a.cs + (int64_t)head * a.max_chunks;
  float* cv = a.cv + (int64_t)head * a.max_chunks * AWQ_HEAD_DIM;
  const int nchunks = (L + 63) >> 6;
  int c_lo, c_hi;
  split_range(nchunks, &c_lo, &c_hi);
  if (c_lo >= c_hi) return;
  half8_t va[8], vb[8];
  auto load_half = [&](int chunk, int half, half8_t (&dst)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = (chunk << 6) + 4 * (8 * half + u) + tq;
      if (chunk < c_hi && t < L)
        dst[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + kv_row(lay, head, t) + 8 * dl));
    }
  };
  int chunk = c_lo + wave;
  // this wavefront's first exponentials and values are requested before the sum of the chunk sums
  float e_lane = (chunk < c_hi && (chunk << 6) + lane < L) ? s[(chunk << 6) + lane] : 0.0f;
  load_half(chunk, 0, va);
  load_half(chunk, 1, vb);
  for (int c = tid; c < nchunks; c += kSplitWaves * 64) zs[c] = cs[c];
  __syncthreads();
  float Z = zs[0];
  for (int c = 1; c < nchunks; ++c) Z += zs[c];
  for (; chunk < c_hi; chunk += kSplitWaves) {
    const int base = chunk << 6;
    const float p_lane = e_lane / Z;  // probability of position base + lane
    const int nxt = chunk + kSplitWaves;
    e_lane = (nxt < c_hi && (nxt << 6) + lane < L) ? s[(nxt << 6) + lane] : 0.0f;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    // (this loop streams: exchange and product per position under a branch measured 7 % faster here than all
    // exchanges first with selects, the form of the one-workgroup kernel, which holds 16 more registers)
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = base + 4 * u + tq;
      const float pr = __shfl(p_lane, 4 * u + tq, 64);
      if (t < L) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(pr, (float)va[u][i], acc[i]);
      }
    }
    load_half(nxt, 0, va);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = base + 4 * (8 + u) + tq;
      const float pr = __shfl(p_lane, 4 * (8 + u) + tq, 64);
      if (t < L) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(pr, (float)vb[u][i], acc[i]);
      }
    }
    load_half(nxt, 1, vb);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[i] = add_xor16(acc[i]);
      acc[i] = add_xor32(acc[i]);
    }
    if (tq == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) cv[chunk * AWQ_HEAD_DIM + 8 * dl + i] = acc[i];
    }
  }
}

// The two kernels above as one launch, for sequences of at most kMergedMax
// positions: every workgroup computes the head's exponentials and chunk sums
// for itself (at most 8 exponentials per thread: cheaper than a launch), keeps
// those of its own chunks in LDS and goes on to their weighted sums.  A chunk is
// still summed by one wavefront with position = lane and the chunk sums are
// added in order, so the bits are those of the separate launches.
constexpr int kMergedMax = 2048;
constexpr int kMergedChunks = kMergedMax / 64;
constexpr int kMergedOwn = (kMergedChunks + kSplit - 1) / kSplit;  // chunks per part
__global__ __launch_bounds__(kSplitWaves * 64) void attn_exp_pv_kernel(SplitArgs a) {
  __shared__ float zs[kMergedChunks];
  __shared__ float es[kMergedOwn * 64];
  const int L = split_len(a);
  const int head = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tq = lane >> 4, dl = lane & 15;
  const half_t* vh = a.vc;
  const KvLayout lay = a.kv;
  const float* s = a.scores + (int64_t)head * a.max_pos;
  float* cv = a.cv + (int64_t)head * a.max_chunks * AWQ_HEAD_DIM;
  const int nchunks = (L + 63) >> 6;
  int c_lo, c_hi;
  split_range(nchunks, &c_lo, &c_hi);
  if (c_lo >= c_hi) return;  // the whole workgroup
  // the values of this wavefront's chunk travel while the exponentials are computed
  half8_t vv[16];
  const int chunk = c_lo + wave;  // at most one chunk per wavefront: kMergedOwn <= kSplitWaves
  if (chunk < c_hi) {
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) {
      const int t = (chunk << 6) + 4 * nl + tq;
      if (t < L) vv[nl] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(vh + kv_row(lay, head, t) + 8 * dl));
    }
  }
  float mx = a.pmax[head * kSplit];
#pragma unroll
  for (int i = 1; i < kSplit; ++i) mx = fmaxf(mx, a.pmax[head * kSplit + i]);
  for (int c = wave; c < nchunks; c += kSplitWaves) {
    const int t = (c << 6) + lane;
    float e = 0.0f;
    if (t < L) e = awq_expf(s[t] - mx);
    if (c >= c_lo && c < c_hi) es[(c - c_lo) * 64 + lane] = e;
    e = wave_tree_sum(e);
    if (lane == 0) zs[c] = e;
  }
  __syncthreads();
  if (chunk >= c_hi) return;
  float Z = zs[0];
  for (int c = 1; c < nchunks; ++c) Z += zs[c];
  const int base = chunk << 6;
  const float p_lane = base + lane < L ? es[(chunk - c_lo) * 64 + lane] / Z : 0.0f;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
  float pp[16];  // all exchanges before the first product; selects, not branches (see attention_kernel)
#pragma unroll
  for (int nl = 0; nl < 16; ++nl) pp[nl] = __shfl(p_lane, 4 * nl + tq, 64);
#pragma unroll
  for (int nl = 0; nl < 16; ++nl) {
    const bool in = base + 4 * nl + tq < L;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float r = __builtin_fmaf(pp[nl], (float)vv[nl][i], acc[i]);
      acc[i] = in ? r : acc[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    acc[i] = add_xor16(acc[i]);
    acc[i] = add_xor32(acc[i]);
  }
  if (tq == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) cv[chunk * AWQ_HEAD_DIM + 8 * dl + i] = acc[i];
  }
}

// chunk vectors added in chunk order (Inference.cu:259-265 runs over t in order).
// The additions of one output element are a sequential chain, but the loads
// need not be: 16 wavefronts per head (8 stages x 2 halves of the 128 elements)
// each request up to 80 consecutive chunks of their half at once, then stage
// after stage continues the running sums, which pass through LDS.
constexpr int kSumStages = 8;
constexpr int kSumRows = 80;  // chunks per stage and round
__global__ __launch_bounds__(kSumStages * 2 * 64) void attn_sum_kernel(SplitArgs a) {
  __shared__ float run[AWQ_HEAD_DIM];
  const int L = split_len(a);
  const int head = blockIdx.x, tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int stage = wave >> 1, col = (wave & 1) * 64 + lane;
  const float* cv = a.cv + (int64_t)head * a.max_chunks * AWQ_HEAD_DIM;
  const int nchunks = (L + 63) >> 6;
  for (int c0 = 0; c0 < nchunks; c0 += kSumStages * kSumRows) {
    const int first = c0 + stage * kSumRows;
    const int count = min(kSumRows, nchunks - first);  // <= 0: nothing for this stage
    float v[kSumRows];
#pragma unroll
    for (int i = 0; i < kSumRows; ++i)
      if (i < count) v[i] = cv[(int64_t)(first + i) * AWQ_HEAD_DIM + col];
    for (int s = 0; s < kSumStages; ++s) {
      if (s == stage && count > 0) {
        // chunk 0 starts the sum (0 + x would turn a -0 into +0)
        float out = first == 0 ? v[0] : run[col];
#pragma unroll
        for (int i = 0; i < kSumRows; ++i)
          if (i < count && first + i > 0) out += v[i];
        run[col] = out;
      }
      __syncthreads();
    }
  }
  if (stage == 0) a.ctx[head * AWQ_HEAD_DIM + col] = (half_t)run[col];
}

}  // namespace

static int64_t chunks_for(int64_t max_pos) { return (max_pos + 63) / 64; }

// scores, chunk vectors, chunk sums, part maxima
int64_t attention_workspace_bytes(int n_heads, int64_t max_pos) {
  return (int64_t)n_heads * (max_pos + chunks_for(max_pos) * (AWQ_HEAD_DIM + 1) + kSplit) * 4;
}

// ws_pos: the number of positions the workspace is laid out for (the cache's own
// max_pos for a workspace of attention_workspace_bytes(n_heads, max_pos))
static int launch_attention_ws(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                               int64_t max_pos, KvLayout kv, int64_t L, const StepState* dyn, int use_len_hi,
                               int64_t len_bound, void* ws, int64_t ws_pos, hipStream_t st);

int launch_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads, int64_t max_pos,
                     KvLayout kv, int64_t L, const StepState* dyn, int use_len_hi, int64_t len_bound, void* ws,
                     hipStream_t st) {
  return launch_attention_ws(q, kc, vc, ctx, n_heads, max_pos, kv, L, dyn, use_len_hi, len_bound, ws, max_pos, st);
}

static int launch_attention_ws(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                               int64_t cache_pos, KvLayout kv, int64_t L, const StepState* dyn, int use_len_hi,
                               int64_t len_bound, void* ws, int64_t max_pos, hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0 && max_pos <= (int64_t)kMaxChunks * 64, "max_pos must be in 1..65536");
  AWQ_REQUIRE(dyn || (L >= 1 && L <= max_pos && L <= cache_pos), "attended length out of range");
  AWQ_REQUIRE(ws != nullptr, "workspace required");
  AWQ_REQUIRE(kv.shift == 6 || kv.block_stride == 0, "cache rows 64 positions apart must be a constant apart");
  float* scores = (float*)ws;
  float* cv = scores + (int64_t)n_heads * max_pos;
  // With a device-side length the caller states an upper bound for it (it
  // decides where the scores live); with a length known here, the length itself.
  const int64_t bound = dyn ? (len_bound > 0 ? len_bound : max_pos) : L;
  const int mc = (int)chunks_for(max_pos);
  static_assert(kAttnOneWorkgroupMax <= kLdsChunks * 64, "the one-workgroup kernel keeps its scores in LDS");
  static_assert(kAttnMergedMax == kMergedMax && kMergedOwn <= kSplitWaves, "one chunk per wavefront in the merged launch");
  static_assert(kAttnTwoLaunchMax <= kWaves * 64 && kAttnTwoLaunchMax <= kLdsChunks * 64, "one chunk per wavefront after the scores launch");
  if (bound > kAttnOneWorkgroupMax) {
    // long sequences: cut along the sequence
    SplitArgs a;
    a.q = q;
    a.kc = kc;
    a.vc = vc;
    a.ctx = ctx;
    a.max_pos = max_pos;
    a.kv = kv;
    a.L_arg = (int)L;
    a.dyn = dyn;
    a.use_len_hi = use_len_hi;
    a.scores = scores;
    a.cv = cv;
    a.cs = cv + (int64_t)n_heads * mc * AWQ_HEAD_DIM;
    a.pmax = a.cs + (int64_t)n_heads * mc;
    a.max_chunks = mc;
    AWQ_REQUIRE((int64_t)mc * 4 <= 65536, "sequence too long for the chunk-sum buffer in LDS");
    const dim3 grid(n_heads, kSplit), block(kSplitWaves * 64);
    hipLaunchKernelGGL(attn_scores_kernel, grid, block, 0, st, a);
    if (bound <= kAttnTwoLaunchMax) {
      // the rest of the head in one workgroup: at most one chunk per wavefront
      hipLaunchKernelGGL((attention_kernel<kWaves, kLdsChunks * 64, kLdsChunks, true, kHeadParts>),
                         dim3(n_heads, kHeadParts), dim3(kThreads), 0, st, q, kc, vc, ctx, kv, (int)L, dyn, use_len_hi,
                         max_pos, a.scores, a.pmax);
      AWQ_HIP_TRY(hipGetLastError());
      return AWQ_OK;
    }
    if (bound <= kMergedMax) {
      hipLaunchKernelGGL(attn_exp_pv_kernel, grid, block, 0, st, a);
    } else {
      hipLaunchKernelGGL(attn_exp_kernel, grid, block, 0, st, a);
      hipLaunchKernelGGL(attn_pv_kernel, grid, block, (size_t)a.max_chunks * 4, st, a);
    }
    hipLaunchKernelGGL(attn_sum_kernel, dim3(n_heads), dim3(kSumStages * 2 * 64), 0, st, a);
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  // A length that sits in device memory and is known to exceed kAttnShortMax: the first rows are
  // requested before it arrives.
  if (dyn && bound > kAttnShortMax && max_pos >= kAttnShortMax)
    hipLaunchKernelGGL((attention_kernel<kWaves, kLdsChunks * 64, kLdsChunks, false, kHeadParts, (int)kAttnShortMax>),
                       dim3(n_heads, kHeadParts), dim3(kThreads), 0, st, q, kc, vc, ctx, kv, (int)L, dyn, use_len_hi,
                       max_pos, (const float*)nullptr, (const float*)nullptr);
  else
    hipLaunchKernelGGL((attention_kernel<kWaves, kLdsChunks * 64, kLdsChunks, false, kHeadParts>),
                       dim3(n_heads, kHeadParts), dim3(kThreads), 0, st, q, kc, vc, ctx, kv, (int)L, dyn, use_len_hi,
                       max_pos, (const float*)nullptr, (const float*)nullptr);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

// ---------------------------------------------------------------------------
// The same attention for callers that cannot allocate (code under stream
// capture, serving loops, harnesses that forbid hipMalloc): scores, part
// maxima, chunk sums and chunk vectors live in a file-scope device array of
// fixed size instead of a caller-provided workspace.  Each device holds its own
// copy of the array at its own address, looked up once per device with
// hipGetSymbolAddress; every call on a device shares it, so calls that may
// overlap on one device race.  The kernels write every word before they read
// it, so nothing needs clearing between calls.
// ---------------------------------------------------------------------------
constexpr int kStaticHeads = 32;
constexpr int64_t kStaticPos = 8192;
constexpr int64_t kStaticBytes =
    (int64_t)kStaticHeads * (kStaticPos + (kStaticPos / 64) * (AWQ_HEAD_DIM + 1) + kSplit) * 4;  // 3,166,208 B
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[64];  // per device; null until its first call

int launch_attention_static(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                            int64_t max_pos, int64_t L, hipStream_t st) {
  AWQ_REQUIRE(n_heads >= 1 && n_heads <= kStaticHeads, "at most 32 heads fit the built-in scratch array");
  AWQ_REQUIRE(L >= 1 && L <= kStaticPos, "at most 8192 attended positions fit the built-in scratch array");
  AWQ_REQUIRE(max_pos >= L, "attended length exceeds the cache");
  int dev = 0;
  AWQ_HIP_TRY(hipGetDevice(&dev));
  AWQ_REQUIRE(dev >= 0 && dev < 64, "device index out of range");
  void* ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
      void* p = nullptr;
      AWQ_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
      g_scratch_ptr[dev] = p;
    }
    ws = g_scratch_ptr[dev];
  }
  static_assert(kStaticBytes == (int64_t)kStaticHeads * (kStaticPos + ((kStaticPos + 63) / 64) * (AWQ_HEAD_DIM + 1) + kSplit) * 4,
                "the array is attention_workspace_bytes(32, 8192)");
  // the workspace is laid out for n_heads x kStaticPos positions whatever the cache's capacity
  return launch_attention_ws(q, kc, vc, ctx, n_heads, max_pos, kv_head_major(max_pos), L, nullptr, 0, 0, ws, kStaticPos, st);
}
