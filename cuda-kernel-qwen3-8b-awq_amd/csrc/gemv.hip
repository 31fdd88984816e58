// Int4 weight kernels for gfx950: the bit-exact standalone dequantisation, the
// load-time reordering of the packed stream, and the fused dequant + matrix-
// vector product used for decode.
//
// Weight stream after reordering.  The [m outputs x k inputs] matrix is cut
// into groups of 64 output rows; the k inputs of a row into blocks of 32 in
// the order of awq_block_elem (awq_canon_math.h).  Lane l of a wavefront owns
// row 64*rg + l, and one 16-byte load hands it one whole block:
//     byte offset = ((rg * (k/32) + blk) * 64 + l) * 16
// so a wavefront load is 1 KiB contiguous and successive blocks follow each
// other.  Inside the 16 bytes, dword c holds elements 8c..8c+7 with nibble
// positions {0,16,4,20,8,24,12,28}[t & 7]: masking with 0x000f000f / 0x00f000f0
// (and the same after one shift by 8) yields two weights as the low mantissa
// bits of a packed pair of binary16 numbers 1024+q or 1024+16q.
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
  const int64_t total = (m / 64) * nblk * 64;
  int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  int lane = (int)(id & 63);
  int64_t blk = (id >> 6) % nblk;
  int64_t rg = (id >> 6) / nblk;
  int64_t row = rg * 64 + lane;
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
  float* partials;
  int32_t* counters;
  int32_t m, k;
  int32_t nblk;      // k/32
  int32_t C;         // group period
  int32_t n_slabs;   // workgroups along k
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
  int64_t max_pos;
  const StepState* dyn;
  // EPI_ARGMAX
  unsigned long long* best;
  int32_t* done;
  int32_t* out_token;
  int32_t* out_array;
};

__device__ __forceinline__ void epilogue(const GemvParams& p, int row, int lane, float acc) {
  half_t v = (half_t)acc;
  switch (p.epilogue) {
    case EPI_RESIDUAL:  // Inference.cu:1149-1155
      p.y[row] = p.res[row] + v;
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
      const int sec = row / H;  // same for the whole wavefront
      const int r = row - sec * H;
      const int d = r & (AWQ_HEAD_DIM - 1);
      half_t other = __builtin_bit_cast(half_t, (unsigned short)__shfl_xor((int)__builtin_bit_cast(unsigned short, v), 1, 64));
      half_t out = v;
      if (sec < 2) {
        const half_t c = p.cos_t[(int64_t)pos * 64 + (d >> 1)], s = p.sin_t[(int64_t)pos * 64 + (d >> 1)];
        const half_t a = (lane & 1) ? other : v, b = (lane & 1) ? v : other;
        if (lane & 1) {
          half_t as = a * s, bc = b * c;
          out = as + bc;
        } else {
          half_t ac = a * c, bs = b * s;
          out = ac - bs;
        }
      }
      if (sec == 0) {
        p.y[r] = out;
      } else {
        half_t* cache = sec == 1 ? p.k_cache : p.v_cache;
        cache[((int64_t)(r >> 7) * p.max_pos + pos) * AWQ_HEAD_DIM + d] = out;
      }
      return;
    }
    case EPI_ARGMAX: {
      // Inference.cu:1278-1290 on the device: the best (value, lowest index)
      // pair of the vocabulary is kept with a 64-bit atomic max, which does
      // not depend on arrival order.
      p.y[row] = v;
      const unsigned short bits = __builtin_bit_cast(unsigned short, v);
      int32_t key = awq_logit_key(bits);
      if (row == 0 && (bits & 0x7fffu) > 0x7c00u) key = INT32_MAX;  // a NaN at index 0 is never displaced
      unsigned long long cand = awq_pack_candidate(key, (uint32_t)row);
#pragma unroll
      for (int mask = 1; mask < 64; mask <<= 1) {
        unsigned long long o = __shfl_xor(cand, mask, 64);
        cand = o > cand ? o : cand;
      }
      if (lane == 0) {
        __hip_atomic_fetch_max(p.best, cand, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0);
        int old = __hip_atomic_fetch_add(p.done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == p.m / 64 - 1) {
          unsigned long long b = __hip_atomic_load(p.best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          int32_t tok = (int32_t)(0xffffffffu - (uint32_t)(b & 0xffffffffull));
          *p.out_token = tok;
          if (p.out_array && p.dyn) p.out_array[p.dyn->out_index] = tok;
          __hip_atomic_store(p.best, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(p.done, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      return;
    }
    default:
      p.y[row] = v;
  }
}

// NI groups of four blocks per wavefront; 4 wavefronts per workgroup cover
// 16*NI consecutive blocks of one 64-row group.
template <int NI, bool ZINT, bool PERIODIC>
__global__ __launch_bounds__(256) void gemv_kernel(GemvParams p) {
  constexpr int NB = 4 * NI;
  __shared__ __attribute__((aligned(16))) half_t xs[4 * NB * AWQ_BLOCK_K];
  __shared__ float red[4][64];
  __shared__ float fin[16][64];  // slab partials of the finishing wavefront
  __shared__ GroupConst gtab[PERIODIC ? 64 : 1];
  __shared__ float nbuf[256];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rg = blockIdx.x;
  const int slab = blockIdx.y;
  const int blk_wg = slab * 4 * NB;
  const int blk_wave = blk_wg + wave * NB;

  const u32x4* wp = p.wq + ((int64_t)rg * p.nblk + blk_wave) * 64 + lane;
  u32x4 wreg[2][4];
#pragma unroll
  for (int n = 0; n < 4; ++n) wreg[0][n] = __builtin_nontemporal_load(wp + n * 64);

  // stage this workgroup's slice of x in block order, normalising it on the
  // way when the RMSNorm is fused in (Inference.cu:111-145: 256 strided fma
  // partial sums, stride-halving tree, then two binary16 multiplies)
  half_t sc = (half_t)1.0f;
  if (p.prologue == PRO_RMSNORM) {
    float acc = 0.0f;
    for (int i = tid; i < p.k; i += 256) {
      float v = (float)p.x[i];
      acc = __builtin_fmaf(v, v, acc);
    }
    nbuf[tid] = acc;
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
    sc = (half_t)awq_rsqrtf(nbuf[0] / (float)p.k + p.eps);
  }
  if (PERIODIC || p.prologue == PRO_RMSNORM) {
    for (int e = tid; e < 4 * NB * AWQ_BLOCK_K; e += 256) {
      int64_t j = PERIODIC ? awq_block_elem(p.k, p.C, blk_wg + (e >> 5), e & 31) : (int64_t)blk_wg * AWQ_BLOCK_K + e;
      half_t v = p.x[j];
      if (p.prologue == PRO_RMSNORM) {
        half_t t = v * sc;
        v = t * p.gamma[j];
      }
      xs[e] = v;
    }
  } else {
    const uint2* src = reinterpret_cast<const uint2*>(p.x + (int64_t)blk_wg * AWQ_BLOCK_K);
    for (int e = tid; e < NB * AWQ_BLOCK_K; e += 256) reinterpret_cast<uint2*>(xs)[e] = src[e];
  }

  // scale group of this wavefront's 64 rows: row/128, then Inference.cu:90 with
  // the index wrapped to the m/128 stored entries.  When the group depends on
  // the input index it is constant within a class of blocks; the (at most 64)
  // classes go through a table in LDS.
  const int a = rg >> 1;
  GroupConst g;
  if (!PERIODIC) {
    int gi = (a % p.kg) % p.mg;
    g = make_group<ZINT>(p.scale[gi], p.zp[gi]);
  } else if (tid < p.C) {
    int gi = (int)((((int64_t)tid * p.mg + a) % p.kg) % p.mg);
    gtab[tid] = make_group<ZINT>(p.scale[gi], p.zp[gi]);
  }
  const int U = p.nblk / p.C;  // blocks per class (PERIODIC)
  int cls = 0, cls_left = 0;   // class of the next block and blocks left in it
  if (PERIODIC) {
    cls = blk_wave / U;
    cls_left = U - (blk_wave - cls * U);
  }
  __syncthreads();

  float g4[NI];
#pragma unroll
  for (int it = 0; it < NI; ++it) {
    if (it + 1 < NI) {
#pragma unroll
      for (int n = 0; n < 4; ++n) wreg[(it + 1) & 1][n] = __builtin_nontemporal_load(wp + ((it + 1) * 4 + n) * 64);
    }
    float bs[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int bl = it * 4 + n;
      if (PERIODIC) {
        g = gtab[cls];
        if (--cls_left == 0) {
          ++cls;
          cls_left = U;
        }
      }
      bs[n] = block_dot<ZINT>(wreg[it & 1][n], xs + (wave * NB + bl) * AWQ_BLOCK_K, g);
    }
    g4[it] = (bs[0] + bs[1]) + (bs[2] + bs[3]);
  }
  // adjacent-pair tree over this lane's groups
#pragma unroll
  for (int n = NI; n > 1; n >>= 1) {
#pragma unroll
    for (int q = 0; q < n / 2; ++q) g4[q] = g4[2 * q] + g4[2 * q + 1];
  }
  red[wave][lane] = g4[0];
  __syncthreads();
  if (wave != 0) return;
  float v = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
  const int row = rg * 64 + lane;
  if (p.n_slabs == 1) {
    epilogue(p, row, lane, v);
    return;
  }
  // Split along k: publish, and let the last workgroup of this row group
  // finish the tree in slab order.  The partial sums travel as device-scope
  // atomic stores and loads (they go to the level of the memory system that
  // all compute dies share), so no cache write-back or invalidate is needed:
  // wait until this wavefront's stores have been acknowledged, then count.
  __hip_atomic_store(&p.partials[(int64_t)slab * p.m + row], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0);
  int old = 0;
  if (lane == 0) old = __hip_atomic_fetch_add(&p.counters[rg], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  if (old != p.n_slabs - 1) return;
  int n = p.n_slabs;
  for (int s = 0; s < n; ++s)
    fin[s][lane] = __hip_atomic_load(&p.partials[(int64_t)s * p.m + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (n > 1 && (n & 1) == 0) {
    n >>= 1;
    for (int q = 0; q < n; ++q) fin[q][lane] = fin[2 * q][lane] + fin[2 * q + 1][lane];
  }
  float tot = fin[0][lane];
  for (int q = 1; q < n; ++q) tot += fin[q][lane];
  if (lane == 0) __hip_atomic_store(&p.counters[rg], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  epilogue(p, row, lane, tot);
}

struct GemvPlan {
  int ni;       // 1, 2, 4 or 8
  int n_slabs;  // workgroups along k
};

// 16*NI blocks per workgroup; pick the split so that the launch has at least
// ~2 workgroups per compute unit when the shape allows it
GemvPlan plan_gemv(int64_t m, int64_t k) {
  int64_t units = k / AWQ_BLOCK_K / 16;  // NI * n_slabs
  int64_t rgs = m / 64;
  GemvPlan best{1, (int)units};
  if (const char* f = getenv("AWQ_DEV_NI")) {
    int ni = atoi(f);
    if (ni >= 1 && units % ni == 0 && units / ni <= 16) return GemvPlan{ni, (int)(units / ni)};
  }
  for (int ni = 8; ni >= 1; ni >>= 1) {
    if (units % ni) continue;
    int64_t slabs = units / ni;
    if (slabs > 16) continue;
    best = GemvPlan{ni, (int)slabs};
    if (rgs * slabs >= 512) break;
  }
  return best;
}

template <int NI>
void launch_ni(const GemvParams& p, bool zint, bool periodic, dim3 grid, hipStream_t st) {
  if (zint) {
    if (periodic) hipLaunchKernelGGL((gemv_kernel<NI, true, true>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gemv_kernel<NI, true, false>), grid, dim3(256), 0, st, p);
  } else {
    if (periodic) hipLaunchKernelGGL((gemv_kernel<NI, false, true>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gemv_kernel<NI, false, false>), grid, dim3(256), 0, st, p);
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
  AWQ_REQUIRE(m < (1ll << 31) && k < (1ll << 31) && m / 64 < 2147483647ll, "shape too large");
  int C = awq_group_period(m, k);
  AWQ_REQUIRE((k / AWQ_BLOCK_K) % C == 0, "k/32 must be a multiple of the scale-group period");
  AWQ_REQUIRE(C <= 64, "scale-group period above 64 is not supported");
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
  // 64 bytes for the sampler, one counter per 64-row group, up to 16 slabs of FP32 partials
  (void)k;
  return 64 + 16 * m * 4 + ((m / 64) * 4 + 255) / 256 * 256;
}

int launch_gemv(const LinearArgs& a, hipStream_t st) {
  if (int rc = check_linear_shape(a.m, a.k)) return rc;
  GemvPlan plan = plan_gemv(a.m, a.k);
  AWQ_REQUIRE(plan.n_slabs <= 16, "k too large for the split workspace");
  AWQ_REQUIRE(plan.n_slabs == 1 || (a.partials && a.counters), "split-k launch needs a workspace");
  AWQ_REQUIRE(a.prologue != PRO_RMSNORM || (a.gamma && a.k % 256 == 0), "fused RMSNorm needs gamma and k % 256 == 0");
  AWQ_REQUIRE(a.epilogue != EPI_RESIDUAL || a.res, "residual epilogue needs res");
  if (a.epilogue == EPI_QKV_ROPE) {
    AWQ_REQUIRE(a.cos_t && a.sin_t && a.k_cache && a.v_cache && a.hidden > 0 && a.m == 3 * (int64_t)a.hidden &&
                    a.hidden % AWQ_HEAD_DIM == 0 && a.max_pos > 0,
                "QKV epilogue needs rotary tables, caches and m == 3*hidden");
    AWQ_REQUIRE(a.dyn || (a.pos >= 0 && a.pos < a.max_pos), "pos out of range");
  }
  if (a.epilogue == EPI_ARGMAX) AWQ_REQUIRE(a.best && a.done && a.out_token, "argmax epilogue needs its workspace");
  GemvParams p;
  p.wq = (const u32x4*)a.wq;
  p.scale = a.scale;
  p.zp = a.zp;
  p.x = a.x;
  p.y = a.y;
  p.res = a.res;
  p.partials = a.partials;
  p.counters = a.counters;
  p.m = (int32_t)a.m;
  p.k = (int32_t)a.k;
  p.nblk = (int32_t)(a.k / AWQ_BLOCK_K);
  p.C = awq_group_period(a.m, a.k);
  p.n_slabs = plan.n_slabs;
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
  p.max_pos = a.max_pos;
  p.dyn = a.dyn;
  p.best = a.best;
  p.done = a.done;
  p.out_token = a.out_token;
  p.out_array = a.out_array;
  bool periodic = p.C > 1;
  dim3 grid((unsigned)(a.m / 64), (unsigned)plan.n_slabs);
  switch (plan.ni) {
    case 1: launch_ni<1>(p, a.zp_integral, periodic, grid, st); break;
    case 2: launch_ni<2>(p, a.zp_integral, periodic, grid, st); break;
    case 4: launch_ni<4>(p, a.zp_integral, periodic, grid, st); break;
    default: launch_ni<8>(p, a.zp_integral, periodic, grid, st); break;
  }
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
