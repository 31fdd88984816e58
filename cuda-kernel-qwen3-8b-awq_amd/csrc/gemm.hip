// W4A16 matrix product for several tokens at once (prefill and batched decode):
//     Y[t][i] = h( sum_j w(i,j) * X[t][j] ),  X [M][k], Y [M][m] row-major
// which is the reference's cublasGemmEx with n = M (ldb = k, ldc = m;
// Inference.cu:1052-1065) applied to the same column-major reading of the
// dequantised weights.  The weights stay packed int4 in memory and are turned
// into binary16 in registers, bit-exactly as Inference.cu:102-104 rounds them;
// the contraction runs on the matrix cores (v_mfma_f32_16x16x32_f16) with FP32
// accumulation, so results agree with a sequential FP32 sum to rounding noise,
// not bit for bit.
//
// Same weight stream as the decode kernel: [16-row group][32-wide block][row][16 B].
// Lane l of a wavefront takes dword l/16 of row l%16 of a block: its 8 nibbles are
// elements 8*(l/16)..+7 of that row, which is exactly the per-lane operand shape
// of the 16x16x32 instruction (index l%16, 8 consecutive k at 8*(l/16)).  The
// tokens ride in the other operand, read from an LDS tile [token][32 k].
//
// Workgroup tile: 128 weight rows x TN tokens, 4 wavefronts x 2 row groups each;
// a wavefront reuses every token operand for its two row groups.
#include "common.hpp"

namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

struct GemmParams {
  const uint32_t* wq;   // reordered int4 stream, as dwords
  const half_t* scale;
  const half_t* zp;
  const half_t* x;      // [M][k]
  half_t* y;            // [M][m]
  int32_t m, k, M;
  int32_t nblk;
  int32_t mg, kg;
};

// 8 nibbles of one dword -> 8 binary16 weights in element order, h(h(q-z)*s)
template <bool ZINT>
__device__ __forceinline__ half8_t dequant8(uint32_t v, half_t s, half_t z) {
  const half2_t s2 = half2_t{s, s};
  const half2_t k16 = half2_t{(half_t)0.0625f, (half_t)0.0625f};
  const uint32_t v8 = v >> 8;
  const half2_t lo0 = as_half2((v & 0x000f000fu) | 0x64006400u), hi0 = as_half2((v & 0x00f000f0u) | 0x64006400u);
  const half2_t lo1 = as_half2((v8 & 0x000f000fu) | 0x64006400u), hi1 = as_half2((v8 & 0x00f000f0u) | 0x64006400u);
  half2_t u0, u1, u2, u3;
  if (ZINT) {
    const half_t a = -((half_t)1024.0f + z), b = -((half_t)64.0f + z);
    const half2_t a2 = half2_t{a, a}, b2 = half2_t{b, b};
    u0 = lo0 + a2;
    u1 = __builtin_elementwise_fma(hi0, k16, b2);
    u2 = lo1 + a2;
    u3 = __builtin_elementwise_fma(hi1, k16, b2);
  } else {
    const half2_t m1024 = half2_t{(half_t)-1024.0f, (half_t)-1024.0f}, m64 = half2_t{(half_t)-64.0f, (half_t)-64.0f};
    const half2_t nz = half2_t{-z, -z};
    u0 = (lo0 + m1024) + nz;
    u1 = __builtin_elementwise_fma(hi0, k16, m64) + nz;
    u2 = (lo1 + m1024) + nz;
    u3 = __builtin_elementwise_fma(hi1, k16, m64) + nz;
  }
  const half2_t w0 = u0 * s2, w1 = u1 * s2, w2 = u2 * s2, w3 = u3 * s2;
  return half8_t{w0.x, w0.y, w1.x, w1.y, w2.x, w2.y, w3.x, w3.y};
}

constexpr int kXStride = 40;  // halves per token row of the LDS tile: 32 + 8 of padding

template <int TT, bool ZINT>  // TT 16-token tiles per workgroup
__global__ __launch_bounds__(256) void gemm_kernel(GemmParams p) {
  constexpr int TN = 16 * TT;
  __shared__ __attribute__((aligned(16))) half_t xs[2][TN * kXStride];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, kq = lane >> 4;
  const int rg0 = blockIdx.x * 8 + wave * 2;  // this wavefront's two 16-row groups
  const int t0 = blockIdx.y * TN;

  // scale group of a row group: (row/128) folded as in Inference.cu:90 (see the decode kernel)
  half_t sc[2], zz[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int gi = (((rg0 + a) >> 3) % p.kg) % p.mg;
    sc[a] = p.scale[gi];
    zz[a] = p.zp[gi];
  }

  // staging of the token tile: thread -> (token, 16-byte piece) pairs
  constexpr int PIECES = TN * 4;  // 16-byte pieces per k-block
  constexpr int PPT = (PIECES + 255) / 256;
  uint4 xr[PPT];
  auto load_x = [&](int kb) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int pc = tid + i * 256;
      const int tok = pc >> 2, part = pc & 3;
      xr[i] = make_uint4(0, 0, 0, 0);
      if (pc < PIECES && t0 + tok < p.M)
        xr[i] = *reinterpret_cast<const uint4*>(p.x + (int64_t)(t0 + tok) * p.k + kb * 32 + part * 8);
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int pc = tid + i * 256;
      if (pc < PIECES) *reinterpret_cast<uint4*>(&xs[buf][(pc >> 2) * kXStride + (pc & 3) * 8]) = xr[i];
    }
  };

  const uint32_t* wp[2];
#pragma unroll
  for (int a = 0; a < 2; ++a) wp[a] = p.wq + ((int64_t)(rg0 + a) * p.nblk * 16 + r) * 4 + kq;
  constexpr int PF = 4;  // weight dwords in flight per row group
  uint32_t wd[2][PF];
#pragma unroll
  for (int f = 0; f < PF; ++f)
#pragma unroll
    for (int a = 0; a < 2; ++a) wd[a][f] = f < p.nblk ? wp[a][(int64_t)f * 64] : 0u;

  float4_t acc[2][TT];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int t = 0; t < TT; ++t) acc[a][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

  load_x(0);
  store_x(0);
  for (int kb0 = 0; kb0 < p.nblk; kb0 += PF) {
#pragma unroll
    for (int f = 0; f < PF; ++f) {
      const int kb = kb0 + f;
      if (kb >= p.nblk) break;
      if (kb + 1 < p.nblk) load_x(kb + 1);
      __syncthreads();  // tile kb is in xs[kb & 1]; tile kb-1's readers are done
      half8_t wop[2];
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        wop[a] = dequant8<ZINT>(wd[a][f], sc[a], zz[a]);
        wd[a][f] = kb + PF < p.nblk ? wp[a][(int64_t)(kb + PF) * 64] : 0u;
      }
      const half_t* xb = &xs[kb & 1][0];
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const half8_t xop = *reinterpret_cast<const half8_t*>(xb + (t * 16 + r) * kXStride + kq * 8);
#pragma unroll
        for (int a = 0; a < 2; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xop, wop[a], acc[a][t], 0, 0, 0);
      }
      if (kb + 1 < p.nblk) store_x((kb + 1) & 1);
    }
  }
  // D[token 4*(lane/16)+i][row lane%16]
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int row = (rg0 + a) * 16 + r;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tok = t0 + t * 16 + kq * 4 + i;
        if (tok < p.M) p.y[(int64_t)tok * p.m + row] = (half_t)acc[a][t][i];
      }
    }
  }
}

// Few tokens (batched decode): the work is streaming the weights once, so the
// decode kernel's decomposition is kept -- one workgroup per 16-row group, all
// of k split over its wavefronts, lane (w, q, r) holding G whole blocks of row r
// -- and only the dot products move to the matrix cores.  For a fixed b and
// dword c the four quarters' blocks form one 32-wide contraction: lane (q, r)
// supplies dword c of block (4w+q)*G+b, lane (q, n) of the token operand
// supplies X[token n][that block, elements 8c..8c+7].
template <int G, int TT, bool ZINT>
__global__ __launch_bounds__(1024) void gemm_small_kernel(GemmParams p, int n_waves) {
  __shared__ float red[16][TT][64][4];
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int rg = blockIdx.x;
  const int t0 = blockIdx.y * (16 * TT);
  const int blk0 = (4 * wave + q) * G;
  const int gi = ((rg >> 3) % p.kg) % p.mg;
  const half_t sc = p.scale[gi], zz = p.zp[gi];
  const u32x4* wp = reinterpret_cast<const u32x4*>(p.wq) + ((int64_t)rg * p.nblk + blk0) * 16 + r;
  u32x4 w[G];
#pragma unroll
  for (int b = 0; b < G; ++b) w[b] = __builtin_nontemporal_load(wp + b * 16);
  float4_t acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int b = 0; b < G; ++b) {
    const uint32_t d[4] = {w[b].x, w[b].y, w[b].z, w[b].w};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const half8_t wop = dequant8<ZINT>(d[c], sc, zz);
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const int tok = t0 + t * 16 + r;
        half8_t xop = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (tok < p.M) xop = *reinterpret_cast<const half8_t*>(p.x + (int64_t)tok * p.k + (blk0 + b) * 32 + c * 8);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xop, wop, acc[t], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][lane][i] = acc[t][i];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < TT; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = red[0][t][lane][i];
      for (int wv = 1; wv < n_waves; ++wv) v += red[wv][t][lane][i];
      const int tok = t0 + t * 16 + q * 4 + i;  // D[token 4*(lane/16)+i][row lane%16]
      if (tok < p.M) p.y[(int64_t)tok * p.m + rg * 16 + r] = (half_t)v;
    }
  }
}

template <int G, int TT>
void launch_small(const GemmParams& p, bool zint, int n_waves, dim3 grid, hipStream_t st) {
  if (zint) hipLaunchKernelGGL((gemm_small_kernel<G, TT, true>), grid, dim3(n_waves * 64), 0, st, p, n_waves);
  else hipLaunchKernelGGL((gemm_small_kernel<G, TT, false>), grid, dim3(n_waves * 64), 0, st, p, n_waves);
}

template <int TT>
void launch_tt(const GemmParams& p, bool zint, dim3 grid, hipStream_t st) {
  if (zint) hipLaunchKernelGGL((gemm_kernel<TT, true>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((gemm_kernel<TT, false>), grid, dim3(256), 0, st, p);
}

}  // namespace

int launch_gemm(const void* wq, const half_t* scale, const half_t* zp, int64_t m, int64_t k, const half_t* x,
                half_t* y, int64_t M, int zp_integral, hipStream_t st) {
  AWQ_REQUIRE(m > 0 && m % 128 == 0 && k > 0 && k % 128 == 0, "m and k must be positive multiples of 128");
  AWQ_REQUIRE(M >= 1 && M <= (1 << 20), "M out of range");
  AWQ_REQUIRE(awq_group_period(m, k) == 1, "matrices whose scale group depends on the input index are not supported here");
  AWQ_REQUIRE(m < (1ll << 31) && k < (1ll << 31), "shape too large");
  GemmParams p;
  p.wq = (const uint32_t*)wq;
  p.scale = scale;
  p.zp = zp;
  p.x = x;
  p.y = y;
  p.m = (int32_t)m;
  p.k = (int32_t)k;
  p.M = (int32_t)M;
  p.nblk = (int32_t)(k / AWQ_BLOCK_K);
  p.mg = (int32_t)(m / 128);
  p.kg = (int32_t)(k / 128);
  if (M <= 64) {
    // lane groups of G blocks: (k/32)/G of them, a multiple of 4 and at most 64
    const int64_t nblk = k / AWQ_BLOCK_K;
    int g = 0;
    for (int c : {8, 4, 2, 1})
      if (nblk % c == 0 && (nblk / c) % 4 == 0 && nblk / c <= 64) {
        g = c;
        break;
      }
    // 17..64 tokens on a matrix with many rows: the tiled kernel reads X less often
    if (M > 16 && m >= 8192) g = 0;
    if (g) {
      const int n_waves = (int)(nblk / g / 4);
      const bool one = M <= 16;
      dim3 grid((unsigned)(m / 16), (unsigned)((M + (one ? 15 : 63)) / (one ? 16 : 64)));
      switch (g) {
        case 8: one ? launch_small<8, 1>(p, zp_integral, n_waves, grid, st) : launch_small<8, 4>(p, zp_integral, n_waves, grid, st); break;
        case 4: one ? launch_small<4, 1>(p, zp_integral, n_waves, grid, st) : launch_small<4, 4>(p, zp_integral, n_waves, grid, st); break;
        case 2: one ? launch_small<2, 1>(p, zp_integral, n_waves, grid, st) : launch_small<2, 4>(p, zp_integral, n_waves, grid, st); break;
        default: one ? launch_small<1, 1>(p, zp_integral, n_waves, grid, st) : launch_small<1, 4>(p, zp_integral, n_waves, grid, st); break;
      }
    } else {
      launch_tt<4>(p, zp_integral, dim3((unsigned)(m / 128), (unsigned)((M + 63) / 64)), st);
    }
  } else {
    launch_tt<8>(p, zp_integral, dim3((unsigned)(m / 128), (unsigned)((M + 127) / 128)), st);
  }
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
