// Int4 weight kernels for gfx950: the bit-exact standalone dequantisation, the
// load-time reordering of the packed stream, and the fused dequant + matrix-
// vector product used for decode.
//
// Weight stream after reordering.  The [m outputs x k inputs] matrix is cut
// into groups of 16 output rows; the k inputs of a row into blocks of 32 in
// the order of awq_block_elem (awq_canon_math.h).  One 16-byte load hands a
// lane one whole block of its row:
//     byte offset = ((rg * (k/32) + blk) * 16 + r) * 16,   rg = row/16, r = row%16
// A workgroup owns one row group and all of k, so no partial sums ever leave
// the workgroup: lane (wavefront w, quarter q = lane/16, r = lane%16) takes the
// G consecutive blocks starting at (4w+q)*G of row 16*rg + r; a wavefront load
// is four contiguous 256-byte pieces, and the G loads of a lane walk 256*G
// contiguous bytes per quarter.  Inside the 16 bytes, dword c holds elements
// 8c..8c+7 with nibble positions {0,16,4,20,8,24,12,28}[t & 7]: masking with
// 0x000f000f / 0x00f000f0 (and the same after one shift by 8) yields two
// weights as the low mantissa bits of a packed pair of binary16 numbers 1024+q
// or 1024+16q.
#include "common.hpp"
#include <stdlib.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// ---------------------------------------------------------------------------
// dequantAwqKernel (Inference.cu:76-106): one thread per packed byte, two
// outputs.  __hsub / __hmul there are separate binary16 operations, so no
// contraction here either.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ packed,
                                                      const half_t* __restrict__ scale,
                                                      const half_t* __restrict__ zp, half_t* __restrict__ out,
                                                      int64_t rows, int64_t cols, int64_t n_groups) {
  int64_t pc = cols >> 1;
  int64_t total = rows * pc;
  for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < total; b += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = b / pc, cb = b - r * pc;
    int64_t c = cb * 2;
    int64_t g = (c / AWQ_GROUP_SIZE) % n_groups;
    uint32_t byte = packed[b];
    half_t s = scale[g], z = zp[g];
    half_t q0 = (half_t)(float)(byte & 15u), q1 = (half_t)(float)(byte >> 4);
    half_t d0 = q0 - z, d1 = q1 - z;
    half2_t w;
    w.x = d0 * s;
    w.y = d1 * s;
    *reinterpret_cast<half2_t*>(out + r * cols + c) = w;
  }
}

// ---------------------------------------------------------------------------
// reorder: one thread builds one 16-byte lane block
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void repack_kernel(const uint8_t* __restrict__ in, uint4* __restrict__ out,
                                                     int64_t m, int64_t k, int C) {
  const int64_t nblk = k / AWQ_BLOCK_K;
  const int64_t total = (m / 16) * nblk * 16;
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  int r = (int)(id & 15);
  int64_t blk = (id >> 4) % nblk;
  int64_t rg = (id >> 4) / nblk;
  int64_t row = rg * 16 + r;
  uint32_t d[4] = {0, 0, 0, 0};
  for (int t = 0; t < AWQ_BLOCK_K; ++t) {
    int64_t j = awq_block_elem(k, C, blk, t);
    int64_t p = j * m + row;
    uint32_t q = (in[p >> 1] >> ((p & 1) * 4)) & 15u;
    int tt = t & 7;
    int pos = (tt >> 1) * 4 + (tt & 1) * 16;
    d[t >> 3] |= q << pos;
  }
  out[id] = make_uint4(d[0], d[1], d[2], d[3]);
}

// ---------------------------------------------------------------------------
// fused dequant + matrix-vector product
// ---------------------------------------------------------------------------
struct GroupConst {
  half2_t s2;  // (s, s)
  half2_t a2;  // integral zp: -(1024+z) twice; otherwise -z twice
  half2_t b2;  // integral zp: -(64+z) twice; unused otherwise
};

template <bool ZINT>
__device__ __forceinline__ GroupConst make_group(half_t s, half_t z) {
  GroupConst g;
  g.s2 = half2_t{s, s};
  if (ZINT) {
    half_t a = -((half_t)1024.0f + z);  // exact: z is an integer in [0,1024]
    half_t b = -((half_t)64.0f + z);
    g.a2 = half2_t{a, a};
    g.b2 = half2_t{b, b};
  } else {
    g.a2 = half2_t{-z, -z};
    g.b2 = g.a2;
  }
  return g;
}

// (x & mask) | 0x64006400 in one instruction.  gfx950's three-operand encoding
// takes no literal, so the mask travels in a scalar register and the exponent
// pattern in a vector register.
__device__ __forceinline__ uint32_t and_or_magic(uint32_t x, uint32_t mask) {
  uint32_t r;
  const uint32_t magic = 0x64006400u;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
  return r;
}

// two weights from the pair 1024+q (LOW) or 1024+16q (!LOW):
//   h( h(q - z) * s )  exactly as Inference.cu:102-104 rounds it
template <bool ZINT, bool LOW>
__device__ __forceinline__ half2_t dq_pair(uint32_t word, const GroupConst& g) {
  half2_t v = as_half2(and_or_magic(word, LOW ? 0x000f000fu : 0x00f000f0u));
  const half2_t k16 = half2_t{(half_t)0.0625f, (half_t)0.0625f};
  half2_t u;
  if (ZINT) {
    // (1024+q) - (1024+z) and (1024+16q)/16 - (64+z) are both q - z with no rounding
    u = LOW ? (v + g.a2) : __builtin_elementwise_fma(v, k16, g.b2);
  } else {
    const half2_t m1024 = half2_t{(half_t)-1024.0f, (half_t)-1024.0f};
    const half2_t m64 = half2_t{(half_t)-64.0f, (half_t)-64.0f};
    half2_t q = LOW ? (v + m1024) : __builtin_elementwise_fma(v, k16, m64);  // q exactly
    u = q + g.a2;                                                            // h(q - z)
  }
  return u * g.s2;
}

// one block: 32 weights of this lane's row against 32 inputs in LDS, a
// sequential fma chain that starts from 0
template <bool ZINT>
__device__ __forceinline__ float block_dot(const u32x4& w, const half_t* xs, const GroupConst& g) {
  const uint32_t d[4] = {w.x, w.y, w.z, w.w};
  float acc = 0.0f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint4 xv = *reinterpret_cast<const uint4*>(xs + 8 * c);
    const half2_t x0 = as_half2(xv.x), x1 = as_half2(xv.y), x2 = as_half2(xv.z), x3 = as_half2(xv.w);
    const uint32_t v = d[c], v8 = v >> 8;
    const half2_t wa = dq_pair<ZINT, true>(v, g);
    const half2_t wb = dq_pair<ZINT, false>(v, g);
    const half2_t wc = dq_pair<ZINT, true>(v8, g);
    const half2_t wd = dq_pair<ZINT, false>(v8, g);
    acc = __builtin_fmaf((float)wa.x, (float)x0.x, acc);
    acc = __builtin_fmaf((float)wa.y, (float)x0.y, acc);
    acc = __builtin_fmaf((float)wb.x, (float)x1.x, acc);
    acc = __builtin_fmaf((float)wb.y, (float)x1.y, acc);
    acc = __builtin_fmaf((float)wc.x, (float)x2.x, acc);
    acc = __builtin_fmaf((float)wc.y, (float)x2.y, acc);
    acc = __builtin_fmaf((float)wd.x, (float)x3.x, acc);
    acc = __builtin_fmaf((float)wd.y, (float)x3.y, acc);
  }
  return acc;
}

struct GemvParams {
  const u32x4* wq;
  const half_t* scale;
  const half_t* zp;
  const half_t* x;
  half_t* y;
  const half_t* res;
  int32_t m, k;
  int32_t nblk;      // k/32
  int32_t C;         // group period
  int32_t n_waves;   // wavefronts per workgroup = k/32/G/4
  int32_t mg, kg;    // m/128, k/128
  int32_t prologue, epilogue;
  // PRO_RMSNORM
  const half_t* gamma;
  float eps;
  // EPI_QKV_ROPE
  const half_t* cos_t;
  const half_t* sin_t;
  half_t* k_cache;
  half_t* v_cache;
  int32_t hidden;
  int32_t pos;
  KvLayout kv;
  const StepState* dyn;
  // EPI_ARGMAX
  unsigned long long* best;
};

// the 16 finished rows of a workgroup; r = lane = row % 16, lanes 0..15 of wavefront 0
__device__ __forceinline__ void epilogue(const GemvParams& p, int row, int r, float acc, half_t res) {
  half_t v = (half_t)acc;
  switch (p.epilogue) {
    case EPI_RESIDUAL:  // Inference.cu:1149-1155
      p.y[row] = res + v;
      return;
    case EPI_GELU:  // Inference.cu:271-279
      p.y[row] = to_half_rn(awq_gelu_f32((float)v));
      return;
    case EPI_QKV_ROPE: {
      // Inference.cu:1070-1103: rows [0,H) are Q, [H,2H) K, [2H,3H) V.  Q and K
      // are rotated pairwise (Inference.cu:158-176); K and V go to the cache
      // row of this position, Q to y.
      const int pos = p.dyn ? p.dyn->pos : p.pos;
      const int H = p.hidden;
      const int sec = row / H;  // same for the whole workgroup
      const int rr = row - sec * H;
      const int d = rr & (AWQ_HEAD_DIM - 1);
      half_t other = __builtin_bit_cast(half_t, (unsigned short)__shfl_xor((int)__builtin_bit_cast(unsigned short, v), 1, 64));
      half_t out = v;
      if (sec < 2) {
        const half_t c = p.cos_t[(int64_t)pos * 64 + (d >> 1)], s = p.sin_t[(int64_t)pos * 64 + (d >> 1)];
        const half_t a = (r & 1) ? other : v, b = (r & 1) ? v : other;
        if (r & 1) {
          half_t as = a * s, bc = b * c;
          out = as + bc;
        } else {
          half_t ac = a * c, bs = b * s;
          out = ac - bs;
        }
      }
      if (sec == 0) {
        p.y[rr] = out;
      } else {
        half_t* cache = sec == 1 ? p.k_cache : p.v_cache;
        cache[kv_row(p.kv, rr >> 7, pos) + d] = out;
      }
      return;
    }
    case EPI_ARGMAX: {
      // Inference.cu:1278-1290 on the device: the best (value, lowest index)
      // pair of the vocabulary is kept with a 64-bit atomic max, which does
      // not depend on arrival order.  Most workgroups find a better candidate
      // already there and skip the atomic.
      p.y[row] = v;
      const unsigned short bits = __builtin_bit_cast(unsigned short, v);
      int32_t key = awq_logit_key(bits);
      if (row == 0 && (bits & 0x7fffu) > 0x7c00u) key = INT32_MAX;  // a NaN at index 0 is never displaced
      unsigned long long cand = awq_pack_candidate(key, (uint32_t)row);
#pragma unroll
      for (int mask = 1; mask < 16; mask <<= 1) {
        unsigned long long o = __shfl_xor(cand, mask, 64);
        cand = o > cand ? o : cand;
      }
      if (r == 0 && cand > __hip_atomic_load(p.best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        __hip_atomic_fetch_max(p.best, cand, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    default:
      p.y[row] = v;
  }
}

// LDS position (in halves) of block-order element e of x.  The four quarters of
// a wavefront read four different lane groups at the same time; 16 bytes of
// skew per lane group keep those reads in different banks.
template <int G>
__device__ __forceinline__ int xs_index(int e) {
  return e + (e / (G * AWQ_BLOCK_K)) * 8;
}

// A workgroup takes row groups blockIdx.x, blockIdx.x + gridDim.x, ... (16
// output rows x all of k each).  n_waves wavefronts; lane (w, q, r) owns blocks
// (4w+q)*G .. +G-1 of row 16*rg + r.  x is staged (and normalised) once per
// workgroup; the weights of the next row group are in flight while the current
// one is multiplied.
// The arguments every wavefront needs before its first load come first and
// one by one: the first 16 dwords of the argument block are preloaded into
// scalar registers at wavefront launch (see the build flags), which takes one
// memory round trip off the start of the kernel.
// UFAST (periodic matrices only): the class length k/32/C when it is known at
// compile time and divides G, so that a lane's G blocks are G/UFAST whole classes
// whose constants it reads once per row group; 0 = look the class up per block.
template <int G, bool ZINT, bool PERIODIC, int UFAST = 0>
__global__ __launch_bounds__(1024) void gemv_kernel(const u32x4* __restrict__ wq, const half_t* __restrict__ x,
                                                    const half_t* __restrict__ gamma, const half_t* __restrict__ scale,
                                                    const half_t* __restrict__ zp, int32_t k, int32_t nblk,
                                                    int32_t n_waves, int32_t m, int32_t prologue, int32_t C,
                                                    GemvParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  half_t* xs = reinterpret_cast<half_t*>(smem);  // x in block order, k halves
  __shared__ float red[2][16][16];  // double-buffered: one barrier per row group
  __shared__ float nbuf[256];
  __shared__ GroupConst gtab[2][PERIODIC ? 64 : 1];
  constexpr int MAXU = 8;  // 8-byte units of x a thread may hold in registers

  const int tid = threadIdx.x;
  const int nthreads = n_waves * 64;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int n_rg = m >> 4;
  const int blk0 = (4 * wave + q) * G;
  const int U = nblk / C;  // blocks per class (PERIODIC)

  int rg = blockIdx.x;
  const u32x4* wp = wq + ((int64_t)rg * nblk + blk0) * 16 + r;
  u32x4 w[G], wn[G];

  // ---- x into LDS in block order ------------------------------------------
  // Unit u of a thread is the 4 consecutive block-order elements 4*(tid + u*nthreads)..+3;
  // in natural order they are 4 consecutive indices too unless the matrix is
  // periodic (then they are C apart and are gathered one by one).
  const int total_units = k >> 2;  // at most MAXU * nthreads (checked by the launcher)
  const bool norm = prologue == PRO_RMSNORM;
  uint2 xu[MAXU], gu[MAXU];
#pragma unroll
  for (int u = 0; u < MAXU; ++u) {
    if (tid + u * nthreads < total_units) {
      const int e = 4 * (tid + u * nthreads);
      if (PERIODIC) {
        half_t hx[4], hg[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = (int)awq_block_elem(k, C, (e + i) >> 5, (e + i) & 31);
          hx[i] = x[j];
          hg[i] = norm ? gamma[j] : (half_t)0.0f;
        }
        xu[u] = __builtin_bit_cast(uint2, *reinterpret_cast<uint64_t*>(hx));
        gu[u] = __builtin_bit_cast(uint2, *reinterpret_cast<uint64_t*>(hg));
      } else {
        xu[u] = reinterpret_cast<const uint2*>(x)[tid + u * nthreads];
        if (norm) gu[u] = reinterpret_cast<const uint2*>(gamma)[tid + u * nthreads];
      }
    }
  }
  // x first, and almost alone: once every wavefront of the device has its 8 KiB of
  // weight loads in flight, a small load of x (an L2 hit) waits microseconds in
  // the same queues.  So only the first weight block is requested along with x
  // (it brings the stream's first round trip forward: +2.8 % tokens/s over none;
  // two blocks +2.4 %, four +0.6 %) and the rest starts when x has arrived.
  w[0] = __builtin_nontemporal_load(wp);
  asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
#pragma unroll
  for (int b = 1; b < G; ++b) w[b] = __builtin_nontemporal_load(wp + b * 16);
  if (norm) {
    // rmsNormKernel, Inference.cu:111-145: 256 strided fma partial sums over the
    // natural order, the stride-halving tree, then two binary16 multiplies.
    // The raw values go through LDS in natural order (unskewed, in the same
    // buffer; it is overwritten afterwards) for the partial sums.
    half_t* xn = xs;
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      if (tid + u * nthreads < total_units) {
        const int e = 4 * (tid + u * nthreads);
        if (PERIODIC) {
          half_t hx[4];
          *reinterpret_cast<uint64_t*>(hx) = __builtin_bit_cast(uint64_t, xu[u]);
#pragma unroll
          for (int i = 0; i < 4; ++i) xn[awq_block_elem(k, C, (e + i) >> 5, (e + i) & 31)] = hx[i];
        } else {
          reinterpret_cast<uint2*>(xn)[tid + u * nthreads] = xu[u];
        }
      }
    }
    __syncthreads();
    if (tid < 256) {
      float acc = 0.0f;
      for (int i = tid; i < k; i += 256) {
        float v = (float)xn[i];
        acc = __builtin_fmaf(v, v, acc);
      }
      nbuf[tid] = acc;
    }
    __syncthreads();
    if (tid < 128) nbuf[tid] += nbuf[tid + 128];
    __syncthreads();
    if (tid < 64) {
      float v = nbuf[tid] + nbuf[tid + 64];
#pragma unroll
      for (int stride = 32; stride > 0; stride >>= 1) v += __shfl_down(v, stride, 64);
      if (tid == 0) nbuf[0] = v;
    }
    __syncthreads();
    const half_t sc = (half_t)awq_rsqrtf(nbuf[0] / (float)k + p.eps);
    const half2_t sc2 = half2_t{sc, sc};
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      if (tid + u * nthreads < total_units) {
        half2_t t0 = as_half2(xu[u].x) * sc2, t1 = as_half2(xu[u].y) * sc2;
        t0 = t0 * as_half2(gu[u].x);
        t1 = t1 * as_half2(gu[u].y);
        xu[u].x = __builtin_bit_cast(uint32_t, t0);
        xu[u].y = __builtin_bit_cast(uint32_t, t1);
      }
    }
  }
  if (norm) __syncthreads();  // everyone is done with the natural-order copy
#pragma unroll
  for (int u = 0; u < MAXU; ++u)
    if (tid + u * nthreads < total_units)
      *reinterpret_cast<uint2*>(xs + xs_index<G>(4 * (tid + u * nthreads))) = xu[u];

  // Group constants.  When the scale group depends on the input index it is
  // constant within a class of blocks; the (at most 64) classes of a row group
  // go through a table in LDS, filled one row group ahead.
  if (PERIODIC && tid < C && rg < n_rg) {
    int gi = (int)((((int64_t)tid * p.mg + (rg >> 3)) % p.kg) % p.mg);
    gtab[0][tid] = make_group<ZINT>(scale[gi], zp[gi]);
  }
  __syncthreads();  // xs and the first table
  for (int it = 0; rg < n_rg; rg += gridDim.x, ++it) {
    const int rg_next = rg + gridDim.x;
    if (rg_next < n_rg) {
      const u32x4* wpn = wq + ((int64_t)rg_next * nblk + blk0) * 16 + r;
#pragma unroll
      for (int b = 0; b < G; ++b) wn[b] = __builtin_nontemporal_load(wpn + b * 16);
    }
    // the residual row is requested before the pass multiplies: the end of the
    // launch then does not wait for one more round trip to memory
    half_t res = (half_t)0.0f;
    if (tid < 16 && p.epilogue == EPI_RESIDUAL) res = p.res[rg * 16 + r];
    // scale group of these 16 rows: row/128, then Inference.cu:90 with the index
    // wrapped to the m/128 stored entries
    const int a = rg >> 3;
    GroupConst g;
    if (!PERIODIC) {
      int gi = (a % p.kg) % p.mg;
      g = make_group<ZINT>(scale[gi], zp[gi]);
    } else if (tid < C && rg_next < n_rg) {
      // the next row group's table; its buffer was last read two barriers ago
      int gi = (int)((((int64_t)tid * p.mg + (rg_next >> 3)) % p.kg) % p.mg);
      gtab[(it + 1) & 1][tid] = make_group<ZINT>(scale[gi], zp[gi]);
    }
    int cls = 0, cls_left = 0;  // class of the next block and blocks left in it
    if (PERIODIC) {
      cls = blk0 / U;
      cls_left = U - (blk0 - cls * U);
    }
    float bs[G];
    if (PERIODIC && UFAST > 0) {
      constexpr int NC = UFAST > 0 ? G / UFAST : 1;
      GroupConst gc[NC];
#pragma unroll
      for (int c = 0; c < NC; ++c) gc[c] = gtab[it & 1][blk0 / UFAST + c];
#pragma unroll
      for (int b = 0; b < G; ++b)
        bs[b] = block_dot<ZINT>(w[b], xs + xs_index<G>((blk0 + b) * AWQ_BLOCK_K), gc[UFAST > 0 ? b / UFAST : 0]);
    } else {
#pragma unroll
      for (int b = 0; b < G; ++b) {
        if (PERIODIC) {
          g = gtab[it & 1][cls];
          if (--cls_left == 0) {
            ++cls;
            cls_left = U;
          }
        }
        bs[b] = block_dot<ZINT>(w[b], xs + xs_index<G>((blk0 + b) * AWQ_BLOCK_K), g);
      }
    }
    // adjacent-pair tree: this lane's G blocks, then the four quarters of the
    // wavefront (consecutive block ranges), then the wavefronts
#pragma unroll
    for (int n = G; n > 1; n >>= 1) {
#pragma unroll
      for (int i = 0; i < n / 2; ++i) bs[i] = bs[2 * i] + bs[2 * i + 1];
    }
    float v = bs[0];
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    // The only barrier of the pass.  The 16 finishing lanes read this pass's
    // buffer while the other wavefronts already multiply the next row group; the
    // buffer is written again two passes on, after a barrier those lanes are part of.
    float(*rd)[16] = red[it & 1];
    if (q == 0) rd[wave][r] = v;
    __syncthreads();
    if (tid < 16) {
      int n = n_waves;
      while (n > 1 && (n & 1) == 0) {
        n >>= 1;
        for (int i = 0; i < n; ++i) rd[i][r] = rd[2 * i][r] + rd[2 * i + 1][r];
      }
      float tot = rd[0][r];
      for (int i = 1; i < n; ++i) tot += rd[i][r];
      epilogue(p, rg * 16 + r, r, tot, res);
    }
#pragma unroll
    for (int b = 0; b < G; ++b) w[b] = wn[b];
  }
}

// Inference.cu:1282-1290, last step: turn the best candidate into the token id
__global__ void sample_finish_kernel(unsigned long long* best, int32_t* out_token, const StepState* dyn,
                                     int32_t* out_array) {
  if (threadIdx.x != 0) return;
  unsigned long long b = *best;
  int32_t tok = (int32_t)(0xffffffffu - (uint32_t)(b & 0xffffffffull));
  *out_token = tok;
  if (out_array && dyn) out_array[dyn->out_index] = tok;
  *best = 0;
}

struct GemvPlan {
  int g;        // blocks per lane: 1, 2, 4 or 8
  int n_waves;  // wavefronts per workgroup
};

// Lane groups per workgroup = (k/32)/G must be a multiple of 4 and at most 64.
// Prefer long per-lane runs (G = 8) unless that leaves the device with few
// wavefronts.
bool plan_gemv(int64_t m, int64_t k, GemvPlan* out) {
  const int64_t nblk = k / AWQ_BLOCK_K;
  bool found = false;
  for (int g = 8; g >= 1; g >>= 1) {
    if (nblk % g) continue;
    int64_t groups = nblk / g;
    if (groups % 4 || groups > 64) continue;
    *out = GemvPlan{g, (int)(groups / 4)};
    found = true;
    // at least 4 wavefronts: the fused norm sums with 256 threads
    if (groups / 4 >= 4 && (m / 16) * (groups / 4) >= 2048) break;
  }
  return found;
}

#define GEMV_HOT_ARGS p.wq, p.x, p.gamma, p.scale, p.zp, p.k, p.nblk, p.n_waves, p.m, p.prologue, p.C
template <int G>
void launch_g(const GemvParams& p, bool zint, bool periodic, dim3 grid, dim3 block, size_t lds, hipStream_t st) {
  if (G == 8 && periodic && p.nblk / p.C == 4) {  // the unembedding: classes of 4 blocks
    if (zint) hipLaunchKernelGGL((gemv_kernel<G, true, true, G == 8 ? 4 : 0>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else hipLaunchKernelGGL((gemv_kernel<G, false, true, G == 8 ? 4 : 0>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    return;
  }
  if (zint) {
    if (periodic) hipLaunchKernelGGL((gemv_kernel<G, true, true>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else hipLaunchKernelGGL((gemv_kernel<G, true, false>), grid, block, lds, st, GEMV_HOT_ARGS, p);
  } else {
    if (periodic) hipLaunchKernelGGL((gemv_kernel<G, false, true>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else hipLaunchKernelGGL((gemv_kernel<G, false, false>), grid, block, lds, st, GEMV_HOT_ARGS, p);
  }
}

}  // namespace

int launch_dequant(const uint8_t* packed, const half_t* scale, const half_t* zp, half_t* out, int64_t rows,
                   int64_t cols, int64_t n_groups, hipStream_t st) {
  AWQ_REQUIRE(rows > 0 && cols > 0 && (cols & 1) == 0, "rows, cols must be positive and cols even");
  AWQ_REQUIRE(n_groups > 0, "n_groups must be positive");
  int64_t total = rows * (cols / 2);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1048576) blocks = 1048576;
  hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, st, packed, scale, zp, out, rows, cols,
                     n_groups);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

static int check_linear_shape(int64_t m, int64_t k) {
  AWQ_REQUIRE(m > 0 && k > 0 && m % 128 == 0, "m must be a positive multiple of 128");
  AWQ_REQUIRE(k % 512 == 0, "k must be a positive multiple of 512");
  AWQ_REQUIRE(m < (1ll << 31) && k <= 24576, "shape too large (k is limited to 24576 by the LDS copy of x)");
  int C = awq_group_period(m, k);
  AWQ_REQUIRE((k / AWQ_BLOCK_K) % C == 0, "k/32 must be a multiple of the scale-group period");
  AWQ_REQUIRE(C <= 64, "scale-group period above 64 is not supported");
  GemvPlan plan;
  AWQ_REQUIRE(plan_gemv(m, k, &plan), "k/32 has no supported split into lane groups");
  return AWQ_OK;
}

int launch_repack(const uint8_t* in, void* out, int64_t m, int64_t k, hipStream_t st) {
  if (int rc = check_linear_shape(m, k)) return rc;
  int64_t total = m * (k / AWQ_BLOCK_K);
  hipLaunchKernelGGL(repack_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, in, (uint4*)out, m, k,
                     awq_group_period(m, k));
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int64_t gemv_workspace_bytes(int64_t m, int64_t k) {
  // the sampler's 64-bit best candidate; the product itself needs no scratch
  (void)m;
  (void)k;
  return 256;
}

int launch_gemv(const LinearArgs& a, hipStream_t st) {
  if (int rc = check_linear_shape(a.m, a.k)) return rc;
  GemvPlan plan;
  plan_gemv(a.m, a.k, &plan);
  AWQ_REQUIRE(a.prologue != PRO_RMSNORM || (a.gamma && a.k % 256 == 0), "fused RMSNorm needs gamma and k % 256 == 0");
  AWQ_REQUIRE(a.epilogue != EPI_RESIDUAL || a.res, "residual epilogue needs res");
  if (a.epilogue == EPI_QKV_ROPE) {
    AWQ_REQUIRE(a.cos_t && a.sin_t && a.k_cache && a.v_cache && a.hidden > 0 && a.m == 3 * (int64_t)a.hidden &&
                    a.hidden % AWQ_HEAD_DIM == 0 && a.max_pos > 0 && a.kv.head_stride > 0,
                "QKV epilogue needs rotary tables, caches and m == 3*hidden");
    AWQ_REQUIRE(a.dyn || (a.pos >= 0 && a.pos < a.max_pos), "pos out of range");
  }
  if (a.epilogue == EPI_ARGMAX) AWQ_REQUIRE(a.best && a.out_token, "argmax epilogue needs its workspace");
  GemvParams p;
  p.wq = (const u32x4*)a.wq;
  p.scale = a.scale;
  p.zp = a.zp;
  p.x = a.x;
  p.y = a.y;
  p.res = a.res;
  p.m = (int32_t)a.m;
  p.k = (int32_t)a.k;
  p.nblk = (int32_t)(a.k / AWQ_BLOCK_K);
  p.C = awq_group_period(a.m, a.k);
  p.n_waves = plan.n_waves;
  p.mg = (int32_t)(a.m / 128);
  p.kg = (int32_t)(a.k / 128);
  p.prologue = a.prologue;
  p.epilogue = a.epilogue;
  p.gamma = a.gamma;
  p.eps = a.eps;
  p.cos_t = a.cos_t;
  p.sin_t = a.sin_t;
  p.k_cache = a.k_cache;
  p.v_cache = a.v_cache;
  p.hidden = a.hidden;
  p.pos = a.pos;
  p.kv = a.kv;
  p.dyn = a.dyn;
  p.best = a.best;
  const bool periodic = p.C > 1;
  AWQ_REQUIRE(a.k / 4 <= 8 * plan.n_waves * 64, "k too large for this workgroup size");
  // one workgroup per row group while that fits the device a few times over;
  // beyond that a workgroup walks several row groups and stages x once
  int64_t n_rg = a.m / 16, n_wg = n_rg;
  if (n_rg > 1024) n_wg = 1024;
  dim3 grid((unsigned)n_wg), block((unsigned)(plan.n_waves * 64));
  size_t lds = (size_t)a.k * 2 + (size_t)(a.k / AWQ_BLOCK_K / plan.g) * 16;  // x plus 16 bytes of skew per lane group
  switch (plan.g) {
    case 1: launch_g<1>(p, a.zp_integral, periodic, grid, block, lds, st); break;
    case 2: launch_g<2>(p, a.zp_integral, periodic, grid, block, lds, st); break;
    case 4: launch_g<4>(p, a.zp_integral, periodic, grid, block, lds, st); break;
    default: launch_g<8>(p, a.zp_integral, periodic, grid, block, lds, st); break;
  }
  AWQ_HIP_TRY(hipGetLastError());
  if (a.epilogue == EPI_ARGMAX) {
    hipLaunchKernelGGL(sample_finish_kernel, dim3(1), dim3(64), 0, st, a.best, a.out_token, a.dyn, a.out_array);
    AWQ_HIP_TRY(hipGetLastError());
  }
  return AWQ_OK;
}
