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
};

template <int EPI>
__device__ __forceinline__ void epilogue(const GemvParams& p, int row, float acc) {
  half_t v = (half_t)acc;
  if (EPI == EPI_RESIDUAL) {
    v = p.res[row] + v;
  } else if (EPI == EPI_GELU) {
    v = to_half_rn(awq_gelu_f32((float)v));
  }
  p.y[row] = v;
}

// NI groups of four blocks per wavefront; 4 wavefronts per workgroup cover
// 16*NI consecutive blocks of one 64-row group.
template <int NI, bool ZINT, bool PERIODIC, int EPI>
__global__ __launch_bounds__(256) void gemv_kernel(GemvParams p) {
  constexpr int NB = 4 * NI;
  __shared__ __attribute__((aligned(16))) half_t xs[4 * NB * AWQ_BLOCK_K];
  __shared__ float red[4][64];
  __shared__ float fin[16][64];  // slab partials of the finishing wavefront

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

  // stage this workgroup's slice of x in block order
  if (PERIODIC) {
    for (int e = tid; e < 4 * NB * AWQ_BLOCK_K; e += 256) {
      int64_t j = awq_block_elem(p.k, p.C, blk_wg + (e >> 5), e & 31);
      xs[e] = p.x[j];
    }
  } else {
    const uint2* src = reinterpret_cast<const uint2*>(p.x + (int64_t)blk_wg * AWQ_BLOCK_K);
    for (int e = tid; e < NB * AWQ_BLOCK_K; e += 256) reinterpret_cast<uint2*>(xs)[e] = src[e];
  }

  // scale group of this wavefront's 64 rows: row/128, then Inference.cu:90 with
  // the index wrapped to the m/128 stored entries
  const int a = rg >> 1;
  GroupConst g;
  if (!PERIODIC) {
    int gi = (a % p.kg) % p.mg;
    g = make_group<ZINT>(p.scale[gi], p.zp[gi]);
  }
  const int U = p.nblk / p.C;  // blocks per class (PERIODIC)
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
        int c = (blk_wave + bl) / U;
        int gi = (int)((((int64_t)c * p.mg + a) % p.kg) % p.mg);
        g = make_group<ZINT>(p.scale[gi], p.zp[gi]);
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
    epilogue<EPI>(p, row, v);
    return;
  }
  // split along k: publish, and let the last workgroup of this row group
  // finish the tree in slab order
  p.partials[(int64_t)slab * p.m + row] = v;
  __threadfence();
  int old = 0;
  if (lane == 0) old = __hip_atomic_fetch_add(&p.counters[rg], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  if (old != p.n_slabs - 1) return;
  __threadfence();
  int n = p.n_slabs;
  for (int s = 0; s < n; ++s)
    fin[s][lane] = __hip_atomic_load(&p.partials[(int64_t)s * p.m + row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (n > 1 && (n & 1) == 0) {
    n >>= 1;
    for (int q = 0; q < n; ++q) fin[q][lane] = fin[2 * q][lane] + fin[2 * q + 1][lane];
  }
  float tot = fin[0][lane];
  for (int q = 1; q < n; ++q) tot += fin[q][lane];
  epilogue<EPI>(p, row, tot);
  if (lane == 0) __hip_atomic_store(&p.counters[rg], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
  for (int ni = 8; ni >= 1; ni >>= 1) {
    if (units % ni) continue;
    int64_t slabs = units / ni;
    if (slabs > 16) continue;
    best = GemvPlan{ni, (int)slabs};
    if (rgs * slabs >= 512) break;
  }
  return best;
}

template <int NI, bool ZINT, bool PERIODIC>
void launch_epi(const GemvParams& p, int epi, dim3 grid, hipStream_t st) {
  switch (epi) {
    case EPI_RESIDUAL: hipLaunchKernelGGL((gemv_kernel<NI, ZINT, PERIODIC, EPI_RESIDUAL>), grid, dim3(256), 0, st, p); break;
    case EPI_GELU: hipLaunchKernelGGL((gemv_kernel<NI, ZINT, PERIODIC, EPI_GELU>), grid, dim3(256), 0, st, p); break;
    default: hipLaunchKernelGGL((gemv_kernel<NI, ZINT, PERIODIC, EPI_STORE>), grid, dim3(256), 0, st, p); break;
  }
}

template <int NI>
void launch_ni(const GemvParams& p, bool zint, bool periodic, int epi, dim3 grid, hipStream_t st) {
  if (zint) {
    if (periodic) launch_epi<NI, true, true>(p, epi, grid, st);
    else launch_epi<NI, true, false>(p, epi, grid, st);
  } else {
    if (periodic) launch_epi<NI, false, true>(p, epi, grid, st);
    else launch_epi<NI, false, false>(p, epi, grid, st);
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
  // up to 16 slabs of FP32 partials plus one counter per 64-row group
  (void)k;
  return 16 * m * 4 + ((m / 64) * 4 + 255) / 256 * 256;
}

int launch_gemv(const LinearArgs& a, hipStream_t st) {
  if (int rc = check_linear_shape(a.m, a.k)) return rc;
  GemvPlan plan = plan_gemv(a.m, a.k);
  AWQ_REQUIRE(plan.n_slabs <= 16, "k too large for the split workspace");
  AWQ_REQUIRE(plan.n_slabs == 1 || (a.partials && a.counters), "split-k launch needs a workspace");
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
  bool periodic = p.C > 1;
  dim3 grid((unsigned)(a.m / 64), (unsigned)plan.n_slabs);
  switch (plan.ni) {
    case 1: launch_ni<1>(p, a.zp_integral, periodic, a.epilogue, grid, st); break;
    case 2: launch_ni<2>(p, a.zp_integral, periodic, a.epilogue, grid, st); break;
    case 4: launch_ni<4>(p, a.zp_integral, periodic, a.epilogue, grid, st); break;
    default: launch_ni<8>(p, a.zp_integral, periodic, a.epilogue, grid, st); break;
  }
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
