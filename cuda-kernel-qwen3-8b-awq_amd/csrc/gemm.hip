// W4A16 matrix product for several tokens at once (prefill and batched decode):
//     Y[t][i] = h( sum_j w(i,j) * X[t][j] ),  X [M][k], Y [M][m] row-major
// which is the reference's cublasGemmEx with n = M (ldb = k, ldc = m;
// Inference.cu:1052-1065) applied to the same column-major reading of the
// dequantised weights.  The weights stay packed int4 in memory and are turned
// into binary16 in registers; the contraction runs on the matrix cores with
// FP32 accumulation, so results agree with a sequential FP32 sum to rounding
// noise, not bit for bit.  The few-token kernel rounds every weight as
// Inference.cu:102-104 does, h(h(q-z)*s); the many-token kernel multiplies
// h(q-z), which is exact, and applies the row's scale to the FP32 sum (one
// rounding fewer per weight than the reference).
//
// Same weight stream as the decode kernel: [16-row group][32-wide block][row][16 B],
// dword c of a row holding elements 8c..8c+7 of the block.  The kernels:
//   up to 4 tokens   the decode kernel's decomposition, products on v_mfma_f32_16x16x32_f16
//   up to 16 tokens, k a multiple of 4096 (taken first)
//                    the same operand shapes, 16 wavefronts sharing up to three row groups
//   17..64 tokens on 4096 rows, 17..256 on 10240..16384 rows (k of 2048 or 4096), 128..320 on 4096 x 12288
//                    16 or 64 rows per workgroup, all its weights requested at the start into registers, the
//                    tokens shared by eight wavefronts through rotating LDS tiles
//   more tokens      64 rows x 32..128 tokens per wavefront on v_mfma_f32_32x32x16_f16,
//                    tokens staged through LDS
#include "common.hpp"

#include <atomic>
#include <type_traits>
#include <utility>

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
  int32_t epilogue;     // EPI_STORE, EPI_RESIDUAL or EPI_GELU
  const half_t* res;    // EPI_RESIDUAL: [M][m], may be y itself
  int32_t kz;           // k is cut into kz chunks over blockIdx.z (k-split workgroups only)
  float* part;          // kz > 1: FP32 partial sums [kz][M][m], finished by reduce_parts_kernel
  int32_t nr, n_tiles;  // rows split: 256-row blocks, tiles = row blocks x 128-token blocks (row block fastest)
  int32_t* sk_head;     // rows split with handed-over sums: status word at [0], "give up now" at [1], counters at [16 + workgroup]
  float* sk_part;       // and one tile of FP32 sums per workgroup
};

// exact-erf GeLU (Inference.cu:274-277) for the many-token kernels, whose sums are not bit-identical
// to the decode path's anyway: erfc by Abramowitz & Stegun 7.1.26 (absolute error <= 1.5e-7, far
// below the binary16 rounding of the result) on the hardware reciprocal and exponential, about a
// fifth of the instructions of the bit-exact awq_gelu_f32 and free of branches.
__device__ __forceinline__ float gelu_approx(float v) {
  const float x = __builtin_fabsf(v) * 0.70710678f;
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, x, 1.0f));
  float q = __builtin_fmaf(t, 1.061405429f, -1.453152027f);
  q = __builtin_fmaf(q, t, 1.421413741f);
  q = __builtin_fmaf(q, t, -0.284496736f);
  q = __builtin_fmaf(q, t, 0.254829592f);
  const float erfc_abs = (q * t) * __builtin_amdgcn_exp2f((x * x) * -1.44269504f);  // 1 - erf(|v| / sqrt 2)
  return (0.5f * v) * (v >= 0.0f ? 2.0f - erfc_abs : erfc_abs);                     // 1 + erf(v / sqrt 2)
}

// one finished output: the same epilogues as the decode kernel's.  The kind is
// a template argument so that the fully unrolled output loops stay free of
// branches (a branch inside them makes the accumulators an indexed array in
// scratch memory).
template <int EPI, bool WIDE = false>
__device__ __forceinline__ void store_out(const GemmParams& p, int tok, int row, float acc) {
  const int64_t at = (int64_t)tok * p.m + row;
  const half_t v = (half_t)acc;
  if (EPI == EPI_RESIDUAL) p.y[at] = p.res[at] + v;                          // Inference.cu:1149-1155
  else if (EPI == EPI_GELU) p.y[at] = to_half_rn(WIDE ? gelu_approx((float)v) : awq_gelu_f32((float)v));  // Inference.cu:271-279
  else p.y[at] = v;
}
// f(integral_constant<int, kind>) for the kind in p.epilogue
template <class F>
__device__ __forceinline__ void with_epilogue(const GemmParams& p, F&& f) {
  if (p.epilogue == EPI_RESIDUAL) f(std::integral_constant<int, EPI_RESIDUAL>{});
  else if (p.epilogue == EPI_GELU) f(std::integral_constant<int, EPI_GELU>{});
  else f(std::integral_constant<int, EPI_STORE>{});
}

// (x & mask) | 0x64006400 in one instruction; the three-operand encoding takes no
// literal, so the mask travels in a scalar register and the exponent pattern in
// a vector register
__device__ __forceinline__ uint32_t and_or_magic(uint32_t x, uint32_t mask) {
  uint32_t r;
  const uint32_t magic = 0x64006400u;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(magic));
  return r;
}

// 8 nibbles of one dword -> 8 binary16 weights in element order, h(h(q-z)*s);
// SCALED = false stops at h(q-z) for a caller that multiplies its sums by s
template <bool ZINT, bool SCALED = true>
__device__ __forceinline__ half8_t dequant8(uint32_t v, half_t s, half_t z) {
  const half2_t s2 = half2_t{s, s};
  const half2_t k16 = half2_t{(half_t)0.0625f, (half_t)0.0625f};
  const uint32_t v8 = v >> 8;
  const half2_t lo0 = as_half2(and_or_magic(v, 0x000f000fu)), hi0 = as_half2(and_or_magic(v, 0x00f000f0u));
  const half2_t lo1 = as_half2(and_or_magic(v8, 0x000f000fu)), hi1 = as_half2(and_or_magic(v8, 0x00f000f0u));
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
  if (!SCALED) return half8_t{u0.x, u0.y, u1.x, u1.y, u2.x, u2.y, u3.x, u3.y};
  const half2_t w0 = u0 * s2, w1 = u1 * s2, w2 = u2 * s2, w3 = u3 * s2;
  return half8_t{w0.x, w0.y, w1.x, w1.y, w2.x, w2.y, w3.x, w3.y};
}

// Very few tokens (batched decode): the work is streaming the weights once, so the
// decode kernel's decomposition is kept -- one workgroup per 16-row group, all
// of k split over its wavefronts, lane (w, q, r) holding G whole blocks of row r
// -- and only the dot products move to the matrix cores.  For a fixed b and
// dword c the four quarters' blocks form one 32-wide contraction: lane (q, r)
// supplies dword c of block (4w+q)*G+b, lane (q, n) of the token operand
// supplies X[token n][that block, elements 8c..8c+7].
template <int G, int TT, bool ZINT, int XR>
__global__ __launch_bounds__(1024) void gemm_small_kernel(GemmParams p, int n_waves) {
  __shared__ float red[16][TT][64][4];
  // the tokens of this workgroup, [token][k] with 16 bytes of skew per lane group of G blocks (the four
  // quarters of a wavefront read four lane groups at once) and 16 bytes between token rows
  extern __shared__ __attribute__((aligned(16))) unsigned char small_lds[];
  half_t* xs = reinterpret_cast<half_t*>(small_lds);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int rg = blockIdx.x;
  const int t0 = blockIdx.y * (16 * TT);
  const int blk0 = (4 * wave + q) * G;
  // Loads return in the order of their requests. Scale and zero-point go first (small, needed by the first
  // product), then XR 16-byte pieces of the tokens per thread (the host picks the smallest
  // of 2, 4 and 8 that covers them: every request costs its slot in the memory pipeline, needed or not), then the weights: the tokens come out of
  // L2 and are in LDS while the weights are still arriving, so that the products start with the first weights
  // instead of after the last. Pieces beyond XR per thread (more tokens) follow the weights.
  const int gi = ((rg >> 3) % p.kg) % p.mg;
  const half_t sc = p.scale[gi], zz = p.zp[gi];
  // piece e8 of token row j lies at j * stride + e8 * 8 + (e8 / (4 G)) * 8 halves
  const int n_tok = min(16 * TT, p.M - t0);
  const int k8 = p.k >> 3;
  const int stride = p.k + (p.nblk / G) * 8 + 8;
  const int n_pc = n_tok * k8, n_thr = n_waves * 64;
  u32x4 xv[XR];
  int xo[XR];
#pragma unroll
  for (int i = 0; i < XR; ++i) {
    const int pc = min(tid + i * n_thr, n_pc - 1);
    const int j = pc / k8, e8 = pc - j * k8;
    xv[i] = *reinterpret_cast<const u32x4*>(p.x + (int64_t)(t0 + j) * p.k + e8 * 8);
    xo[i] = j * stride + e8 * 8 + (e8 / (4 * G)) * 8;
  }
  const u32x4* wp = reinterpret_cast<const u32x4*>(p.wq) + ((int64_t)rg * p.nblk + blk0) * 16 + r;
  u32x4 w[G];
#pragma unroll
  for (int b = 0; b < G; ++b) w[b] = __builtin_nontemporal_load(wp + b * 16);
#pragma unroll
  for (int i = 0; i < XR; ++i)
    if (tid + i * n_thr < n_pc) *reinterpret_cast<u32x4*>(xs + xo[i]) = xv[i];
  for (int pc = tid + XR * n_thr; pc < n_pc; pc += n_thr) {
    const int j = pc / k8, e8 = pc - j * k8;
    const u32x4 v = *reinterpret_cast<const u32x4*>(p.x + (int64_t)(t0 + j) * p.k + e8 * 8);
    *reinterpret_cast<u32x4*>(xs + j * stride + e8 * 8 + (e8 / (4 * G)) * 8) = v;
  }
  __syncthreads();
  float4_t acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  // this lane's token row (r) and lane group in LDS; lanes beyond the last token read the last token's row
  // (their accumulator columns are never stored)
  const half_t* xl = xs + (blk0 * 32) + (blk0 / G) * 8;
  // The token operands are read from LDS in batches of up to 16, each batch ahead of its products: a read per
  // product would put an LDS round trip between every two matrix instructions.
  constexpr int NB = G * 4 < 16 ? G * 4 : 16;
  const half_t* row[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) row[t] = xl + min(t * 16 + r, n_tok - 1) * stride;
#pragma unroll
  for (int b0 = 0; b0 < G * 4; b0 += NB) {
    half8_t xr[TT][NB];
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int i = 0; i < NB; ++i) xr[t][i] = *reinterpret_cast<const half8_t*>(row[t] + (b0 + i) * 8);
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int bc = b0 + i;
      const half8_t wop = dequant8<ZINT>(w[bc >> 2][bc & 3], sc, zz);
#pragma unroll
      for (int t = 0; t < TT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xr[t][i], wop, acc[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][lane][i] = acc[t][i];
  __syncthreads();
  if (wave != 0) return;
  with_epilogue(p, [&](auto E) {
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      // the wavefronts' sums in wavefront order; all 16-byte reads are issued together (a read per term is an
      // LDS round trip each, serialised by the additions)
      float4_t part[16];
#pragma unroll
      for (int wv = 0; wv < 16; ++wv)
        if (wv < n_waves) part[wv] = *reinterpret_cast<const float4_t*>(&red[wv][t][lane][0]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = part[0][i];
#pragma unroll
        for (int wv = 1; wv < 16; ++wv)
          if (wv < n_waves) v += part[wv][i];
        const int tok = t0 + t * 16 + q * 4 + i;  // D[token 4*(lane/16)+i][row lane%16]
        if (tok < p.M) store_out<decltype(E)::value>(p, tok, rg * 16 + r, v);
      }
    }
  });
}

// Two to sixteen tokens, k a multiple of 4096: still a weight stream, but every workgroup of the kernel above
// needs all tokens' inputs (2 k bytes each) for its 8 k bytes of weights.  Here a workgroup of 16 wavefronts
// takes RG row groups and all of k: wavefront w, quarter q holds blocks (4w+q)G.. of each of its rows -- the
// operand shapes of the kernel above -- so per pair of blocks (a "slice": b = 2h, 2h+1) the wavefront needs
// four 128-byte pieces of every token, once for the RG row groups.  It reads them 16 bytes per lane, two
// tokens per instruction (a lane reading its own operand straight from memory touches 64 cache lines per
// instruction, and the compute unit looks up one line per clock: 14 us at 16 tokens), and turns them into
// operand order through a piece of LDS of its own -- no workgroup barrier: the LDS instructions of one
// wavefront execute in order.  Requests go out in the order of need: scales, the first two slices of tokens,
// all RG G blocks of weights per lane (96 KB per workgroup for the model's shapes, as in the decode kernel);
// a further slice of tokens is requested as soon as a register set is free, long before the weights ahead
// of it have arrived.  The 16 wavefronts' sums meet in LDS, in the place of the token pieces.
constexpr int kMidRow = 4 * 144 + 16;  // bytes per token in a wavefront's piece: quarters 144 bytes apart (conflict-free operand reads)
template <int G, int RG, bool ZINT>
__global__ __launch_bounds__(1024) void gemm_mid_kernel(GemmParams p, int n_rg) {
  constexpr int NW = 16, NS = G / 2, S = NS < 2 ? NS : 2;
  static_assert(G % 2 == 0 && RG * G <= 8, "slices of two blocks; register budget of 1024 threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char mid_lds[];
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int rg0 = blockIdx.x * RG;
  const int blk0 = (4 * wave + q) * G;
  half_t sc[RG], zz[RG];
#pragma unroll
  for (int i = 0; i < RG; ++i) {
    const int rg = min(rg0 + i, n_rg - 1);  // a workgroup past the last row group repeats it and stores nothing
    const int gi = ((rg >> 3) % p.kg) % p.mg;
    sc[i] = p.scale[gi];
    zz[i] = p.zp[gi];
  }
  // instruction i of a slice brings tokens 2i and 2i+1: lane = (token parity, quarter, 16-byte piece); tokens
  // beyond the last repeat the last (their accumulator columns are never stored)
  const int n_tok = min(16, p.M);
  const int tpar = lane >> 5, tq = (lane >> 3) & 3, tp = lane & 7;
  const half_t* xg = p.x + ((4 * wave + tq) * G) * 32 + tp * 8;
  u32x4 xs[S][8];
  auto request = [&](int h, u32x4* dst) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      dst[i] = *reinterpret_cast<const u32x4*>(xg + (int64_t)min(2 * i + tpar, n_tok - 1) * p.k + h * 64);
  };
#pragma unroll
  for (int h = 0; h < S; ++h) request(h, xs[h]);
  u32x4 w[RG][G];
#pragma unroll
  for (int i = 0; i < RG; ++i) {
    const int rg = min(rg0 + i, n_rg - 1);
    const u32x4* wp = reinterpret_cast<const u32x4*>(p.wq) + ((int64_t)rg * p.nblk + blk0) * 16 + r;
#pragma unroll
    for (int b = 0; b < G; ++b) w[i][b] = __builtin_nontemporal_load(wp + b * 16);
  }
  unsigned char* mine = mid_lds + wave * (16 * kMidRow);
  unsigned char* put = mine + tpar * kMidRow + tq * 144 + tp * 16;
  const unsigned char* get = mine + r * kMidRow + q * 144;
  float4_t acc[RG];
#pragma unroll
  for (int i = 0; i < RG; ++i) acc[i] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int h = 0; h < NS; ++h) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(put + 2 * i * kMidRow) = xs[h % S][i];
    if (h + S < NS) request(h + S, xs[h % S]);
    half8_t xr[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xr[i] = *reinterpret_cast<const half8_t*>(get + i * 16);
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
      for (int bc = 0; bc < 8; ++bc) {
        const half8_t wop = dequant8<ZINT>(w[i][2 * h + (bc >> 2)][bc & 3], sc[i], zz[i]);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xr[bc], wop, acc[i], 0, 0, 0);
      }
  }
  __syncthreads();  // every wavefront has read its operands: the token pieces make room for the sums
  float* red = reinterpret_cast<float*>(mid_lds);  // [NW][RG][64][4]
#pragma unroll
  for (int i = 0; i < RG; ++i) *reinterpret_cast<float4_t*>(red + ((wave * RG + i) * 64 + lane) * 4) = acc[i];
  __syncthreads();
  // D[token 4 (lane / 16) + e][row lane % 16] sits in element e of the lane: thread (i, token, row), rows fastest
  if (tid >= RG * 256) return;
  const int i = tid >> 8, tok = (tid >> 4) & 15, row = tid & 15;
  if (tok >= p.M || rg0 + i >= n_rg) return;
  const float* first = red + (i * 64 + (tok >> 2) * 16 + row) * 4 + (tok & 3);
  float part[NW];
#pragma unroll
  for (int wv = 0; wv < NW; ++wv) part[wv] = first[wv * (RG * 256)];
  float v = part[0];
#pragma unroll
  for (int wv = 1; wv < NW; ++wv) v += part[wv];
  with_epilogue(p, [&](auto E) { store_out<decltype(E)::value>(p, tok, (rg0 + i) * 16 + row, v); });
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <class F, int... I>
__device__ __forceinline__ void static_for_seq(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_seq(f, std::make_integer_sequence<int, N>{});
}

// s_waitcnt vmcnt(n) lgkmcnt(0), no wait for exports, as the immediate of the instruction (the builtin, not inline
// assembly: the compiler then knows that the LDS reads before it are complete)
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | (7 << 4) | ((n >> 4) << 14); }

// 17..64 (and 129..192) tokens, 4096 rows, k of 2048 or 4096 (the model's attention output matrix): one workgroup of eight
// wavefronts per compute unit takes one 16-row group, all of k and ALL tokens.  Whichever way the rows are cut,
// every compute unit has to read every token (512 KB at 64 tokens), and what a compute unit has requested comes
// back in the order of the requests: a token piece out of L2 queued behind weights out of memory arrives with
// the weights' latency.  So the two are not mixed: a wavefront requests ALL its weights at the start, NS dwords
// per lane (lane (q, r): dword q of row r of block 8 s + v, the decode kernel's stream read 4 bytes at a time),
// and the tokens stream through LDS behind them: a step is 256 inputs, its token tile [16 TT tokens][256] comes
// straight into LDS (global_load_lds_dwordx4, four tiles rotating, the 16-byte pieces of a row at positions
// piece ^ (row & 15) so that the operand reads of sixteen rows hit all banks), wavefront v multiplies block v
// of the step against the TT token tiles, v_mfma_f32_16x16x32_f16 with the tokens as the first operand.  The
// eight wavefronts' sums meet in LDS, in the place of the tiles.  No hand-over between workgroups, no second
// launch.  (RG row groups per workgroup: written for up to three, which the 12288-row matrices would take;
// there it took 15.7 us at 64 tokens, as long as the k-split workgroups -- 12 of these half-rate matrix
// instructions per wavefront and step are 0.32 us of a 0.39 us step -- so only RG = 1 is launched, and those
// matrices go to gemm_shared32_kernel.)
template <int TT, int RG, int NS, bool ZINT>
__global__ __launch_bounds__(512) void gemm_shared_kernel(GemmParams p, int n_rg) {
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  constexpr int kTile = 16 * TT * 256;  // halves per tile
  static_assert(NS * RG + TT < 64, "the request counter has six bits");
  extern __shared__ __attribute__((aligned(16))) unsigned char shared_lds[];
  half_t* const tiles = reinterpret_cast<half_t*>(shared_lds);  // four of them
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int rg0 = blockIdx.x * RG;
  // The workgroups of a die (those whose indices agree mod 8) take the steps in different rotations: in step
  // with each other they would all ask the same few channels of the die's L2 for the same 512-byte columns of
  // the tokens.
  const int first_step = ((blockIdx.x >> 3) & 31) * NS >> 5;
  auto step_at = [&](int s) __attribute__((always_inline)) { return (s + first_step) & (NS - 1); };
  static_assert((NS & (NS - 1)) == 0, "the rotation wraps with a mask");
  // Requests return in the order they are made: the scales, three tiles out of L2, then the weights.  Those into
  // registers are issued by hand and waited for by the counts at the barriers: the compiler, which counts them
  // together with the requests into LDS, would wait for everything in flight at the first use of any of them.
  uint32_t sc_raw[RG], zz_raw[RG];
  uint32_t w[NS][RG];
#pragma unroll
  for (int i = 0; i < RG; ++i) {
    const int rg = min(rg0 + i, n_rg - 1);  // a workgroup past the last row group repeats it and stores nothing
    const int gi = ((rg >> 3) % p.kg) % p.mg;
    asm volatile("global_load_ushort %0, %1, off" : "=v"(sc_raw[i]) : "v"(p.scale + gi) : "memory");
    asm volatile("global_load_ushort %0, %1, off" : "=v"(zz_raw[i]) : "v"(p.zp + gi) : "memory");
  }
  half_t sc[RG], zz[RG];
  // the operand of token tile t: row 16 t + r, piece 4 wave + q of the step
  const int xoff = r * 256 + (((4 * wave + q) ^ r) << 3);
  // More than 16 TT tokens: one slab of 16 TT tokens after the other against the same weights, which stay in
  // their registers.  Only the first slab has weights in flight next to its tiles.
  auto slab = [&](auto FIRST, int t0) __attribute__((always_inline)) {
    constexpr bool first = decltype(FIRST)::value;
    // token tile requests: instruction i of this wavefront brings token rows 2 (wave TT + i) and + 1, 1 KB
    const half_t* src[TT];
#pragma unroll
    for (int i = 0; i < TT; ++i) {
      const int row = 2 * (wave * TT + i) + (lane >> 5);
      const int piece = (lane & 31) ^ (row & 15);
      src[i] = p.x + (int64_t)min(t0 + row, p.M - 1) * p.k + piece * 8;
    }
    auto request = [&](int s) __attribute__((always_inline)) {
      half_t* const tile = tiles + (s & 3) * kTile + wave * TT * 512;
#pragma unroll
      for (int i = 0; i < TT; ++i)
        __builtin_amdgcn_global_load_lds((gptr_t)(src[i] + step_at(s) * 256), (lptr_t)(tile + i * 512), 16, 0, 0);
    };
    request(0);
    request(1);
    request(2);
    asm volatile("" ::: "memory");
    if constexpr (first) {
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int i = 0; i < RG; ++i) {
          const int rg = min(rg0 + i, n_rg - 1);
          const uint32_t* at = p.wq + (((int64_t)rg * p.nblk + wave + 8 * step_at(s)) * 16 + r) * 4 + q;
          asm volatile("global_load_dword %0, %1, off nt" : "=v"(w[s][i]) : "v"(at) : "memory");
        }
    }
    float4_t acc[RG][TT];
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
      for (int t = 0; t < TT; ++t) acc[i][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    half8_t xr[2][TT], wop[2][RG];
    // Bare barriers: __syncthreads() would wait for every request in flight.  The counts say how many of this
    // wavefront's requests may still be out: a tile complete here is complete for everybody behind the barrier.
    // The scales, tiles 0 to 2 and the first weights; a later slab: tile 0.
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(first ? (NS - 1) * RG : 2 * TT));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < RG; ++i) {
      asm volatile("" : "+v"(w[0][i]));  // not read before the wait above
      if constexpr (first) {
        asm volatile("" : "+v"(sc_raw[i]), "+v"(zz_raw[i]));
        sc[i] = __builtin_bit_cast(half_t, (unsigned short)sc_raw[i]);
        zz[i] = __builtin_bit_cast(half_t, (unsigned short)zz_raw[i]);
      }
    }
#pragma unroll
    for (int t = 0; t < TT; ++t) xr[0][t] = *reinterpret_cast<const half8_t*>(tiles + t * 16 * 256 + xoff);
#pragma unroll
    for (int i = 0; i < RG; ++i) wop[0][i] = dequant8<ZINT, false>(w[0][i], sc[i], zz[i]);
    // A step reads the operands of the next one out of LDS and dequantises the next one's weights while the
    // matrix cores work on its own.
    static_for<NS>([&](auto S) __attribute__((always_inline)) {
      constexpr int s = decltype(S)::value, c = s & 1, n = c ^ 1;
      // the weights of step s + 1 and tile s + 1 (in the first slab tiles 1 and 2 were requested ahead of the
      // weights, tile 3 and later behind all of them: tile s + 2, if there is one, may be out), and this
      // wavefront's operand reads of tile s are done: tile s - 1 can be replaced
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(first && s < 2 ? (NS - 2 - s) * RG + s * TT : (s + 2 < NS ? TT : 0)));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if constexpr (s + 1 < NS) {
#pragma unroll
        for (int i = 0; i < RG; ++i) asm volatile("" : "+v"(w[s + 1][i]));  // not read before the wait above
      }
      // (what this step multiplies is not touched before the barrier: its products would wait for the reads there)
#pragma unroll
      for (int t = 0; t < TT; ++t) asm volatile("" : "+v"(xr[c][t]));
#pragma unroll
      for (int i = 0; i < RG; ++i) asm volatile("" : "+v"(wop[c][i]));
      if constexpr (s + 3 < NS) request(s + 3);
      if constexpr (s + 1 < NS) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
          xr[n][t] = *reinterpret_cast<const half8_t*>(tiles + ((s + 1) & 3) * kTile + t * 16 * 256 + xoff);
      }
#pragma unroll
      for (int i = 0; i < RG; ++i) {
        if constexpr (s + 1 < NS) wop[n][i] = dequant8<ZINT, false>(w[s + 1][i], sc[i], zz[i]);
#pragma unroll
        for (int t = 0; t < TT; ++t) acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xr[c][t], wop[c][i], acc[i][t], 0, 0, 0);
      }
    });
    __syncthreads();  // every wavefront has read its operands: the tiles make room for the sums
    float* red = reinterpret_cast<float*>(shared_lds);  // [8 wavefronts][RG][TT][64 lanes][4]
#pragma unroll
    for (int i = 0; i < RG; ++i)
#pragma unroll
      for (int t = 0; t < TT; ++t) *reinterpret_cast<float4_t*>(red + (((wave * RG + i) * TT + t) * 64 + lane) * 4) = acc[i][t];
    __syncthreads();
    // D[token 4 (lane / 16) + e][row lane % 16] sits in element e of the lane; thread (i, t, token, row), rows fastest
    with_epilogue(p, [&](auto E) {
#pragma unroll
      for (int i = 0; i < RG; ++i) {
        if (rg0 + i >= n_rg) continue;
        const float scf = (float)sc[i];
#pragma unroll
        for (int idx = tid; idx < TT * 256; idx += 512) {
          const int t = idx >> 8, row = idx & 15, e = (idx >> 4) & 3, q4 = (idx >> 6) & 3;
          const int tok = t0 + 16 * t + 4 * q4 + e;
          const float* part = red + ((i * TT + t) * 64 + q4 * 16 + row) * 4 + e;
          float v = part[0];
#pragma unroll
          for (int wv = 1; wv < 8; ++wv) v += part[wv * (RG * TT * 256)];
          if (tok < p.M) store_out<decltype(E)::value, true>(p, tok, (rg0 + i) * 16 + row, v * scf);
        }
      }
    });
  };
  slab(std::true_type{}, 0);
  for (int t0 = 16 * TT; t0 < p.M; t0 += 16 * TT) {
    __syncthreads();  // the sums of the slab before have been read: its place takes tiles again
    slab(std::false_type{}, t0);
  }
}

// Many tokens: a wavefront owns 64 weight rows x 128 tokens as 2 x 4 accumulator
// tiles of v_mfma_f32_32x32x16_f16 (twice the rate of the 16x16x32 shape on this
// device).  Every token operand read from LDS feeds two products and every
// dequantised weight operand four.  Operand shapes: lane (n, kh) = (lane % 32,
// lane / 32) supplies 8 consecutive k of token / weight row n; a 32-wide block
// of k goes through two instructions, slice j taking dwords j (kh = 0) and
// j + 2 (kh = 1) of each row's 16 bytes, so that a lane's two weight dwords
// (2kh, 2kh + 1) are adjacent in the weight stream.
// Two workgroup shapes:
//   rows split: 4 wavefronts x 64 rows = 256 rows, one shared
//     token tile per step; for products with many tiles.
//   k split: the 4 wavefronts share 64 rows and take a quarter
//     of k each (a token tile of their own per step), partial sums meet in LDS;
//     four times as many workgroups for products with few tiles.
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t xvec_t __attribute__((ext_vector_type(4)));  // 16 bytes of tokens in flight
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kWideRP = 2;                              // 32-row pairs of row groups per wavefront
constexpr int kWideTT = 4;                              // 32-token tiles per wavefront (1 or 2 for few tokens, k split)
constexpr int kWideTokens = 32 * kWideTT;               // 128
constexpr int kWideNH = 2;                              // 32-wide blocks of k per step
constexpr int kWideStride = 32 * kWideNH + 8;           // halves per token row of a tile in LDS (16 bytes of padding)
constexpr int wide_lds_bytes(bool ksplit, int tt) {
  if (!ksplit) return 0;  // rows split: three static tiles
  const int tiles = 4 * 2 * (32 * tt) * kWideStride * 2;  // slots x double buffer x tile
  const int sums = 4 * kWideRP * tt * 64 * 16 * 4;        // the partial sums
  return sums > tiles ? sums : tiles;
}

// Rows split, work cut evenly: the steps of all tiles, in tile order, form one
// sequence that is cut into gridDim.x equal ranges, one per workgroup, in units
// of two steps.  A range covers the tail of one tile, whole tiles and the head
// of another.  A workgroup whose piece of a tile does not reach the tile's last
// step leaves its FP32 sums in its own slot of the workspace and counts itself
// in at the workgroup that holds the last step; that one waits for the count,
// adds the slots in workgroup order (a fixed order whatever the timing) and
// writes the outputs.  Pieces are taken last tile first, so sums are handed
// over early and collected late.  The collector has the highest index among a
// tile's workgroups: with workgroups dispatched in index order, the ones it
// waits for never wait themselves and are running or done.  The wait is
// bounded all the same and reports through the status word.
constexpr int kSkHeaderBytes = 4096;               // status word, then one counter per workgroup
constexpr int kSkWgs = 256;                        // workgroups of a product whose work is cut evenly: one per compute unit
constexpr int kSkTileFloats = 256 * kWideTokens;   // FP32 sums of one tile
constexpr int kSkSpinLimit = 1 << 22;
constexpr int kRowsSplitMinTiles = 80;             // fewer 256 x 128 tiles than this: k-split workgroups

// the workgroup whose range holds step pair q, ranges being [b W / G, (b + 1) W / G)
__device__ __forceinline__ int sk_wg_of(int64_t q, int64_t W, int G) {
  int b = (int)(q * G / W);
  while ((int64_t)(b + 1) * W / G <= q) ++b;
  while ((int64_t)b * W / G > q) --b;
  return b;
}

enum WideMode { WIDE_ROWS = 0, WIDE_K = 1, WIDE_ROWS_CUT = 2 };  // rows split (a tile per workgroup), k split, rows split with work cut evenly

template <bool ZINT, int MODE, int EPI, int TT>
__global__ __launch_bounds__(256, (MODE == WIDE_K && TT == 4) ? 1 : ((MODE == WIDE_ROWS && TT == 2) ? 3 : 2)) void gemm_wide_kernel(GemmParams p) {
  constexpr bool KSPLIT = MODE == WIDE_K;
  constexpr bool CUT = MODE == WIDE_ROWS_CUT;
  constexpr int kTokens = 32 * TT;                   // tokens per workgroup
  constexpr int kSlot = kTokens * kWideStride;       // halves per token tile in LDS
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  half_t* xs = reinterpret_cast<half_t*>(smem_raw);  // [2][NKB][32 TT tokens][kWideStride]
  constexpr int NKB = KSPLIT ? 4 : 1;
  constexpr int NH = kWideNH;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, kh = lane >> 5;
  // a step is NH blocks of k; a tile (k split: this wavefront's quarter of this workgroup's chunk) has
  // an even number of them (checked by the launcher)
  const int tile_steps = (KSPLIT ? p.nblk / (4 * p.kz) : p.nblk) / NH;
  const int slot = KSPLIT ? wave : 0;

  // work cut evenly: this workgroup's range [lo, hi) of step pairs; otherwise one tile, whole
  const int S2 = tile_steps / 2;
  const int64_t W2 = (int64_t)p.n_tiles * S2;
  const int64_t lo = CUT ? (int64_t)blockIdx.x * W2 / gridDim.x : 0;
  const int64_t hi = CUT ? (int64_t)(blockIdx.x + 1) * W2 / gridDim.x : 1;
  const int tile_first = CUT ? (int)(lo / S2) : 0;
  int tile = CUT ? (int)((hi - 1) / S2) : (int)blockIdx.x;

  do {
    // this piece: steps [s_lo, s_lo + steps) of the tile
    int s_lo = 0, steps = tile_steps;
    if (CUT) {
      const int64_t q0 = (int64_t)tile * S2;
      const int pb = (int)((lo > q0 ? lo : q0) - q0), pe = (int)((hi < q0 + S2 ? hi : q0 + S2) - q0);
      s_lo = 2 * pb;
      steps = 2 * (pe - pb);
    }
    const int rb = KSPLIT ? (int)blockIdx.x : tile % p.nr;
    const int tb = KSPLIT ? (int)blockIdx.y : tile / p.nr;
    const int rg0 = KSPLIT ? rb * 4 : (rb * 4 + wave) * 4;  // first of this wavefront's 4 row groups
    const bool rows_ok = rg0 * 16 < p.m;                    // rows split: the last tile may hang over the edge
    const int t0 = tb * kTokens;
    // first block of this workgroup's part of k, then of this wavefront's
    const int kb_wg = KSPLIT ? (int)blockIdx.z * 4 * tile_steps * NH : s_lo * NH;
    const int kb_base = kb_wg + (KSPLIT ? wave * tile_steps * NH : 0);

    // the 64 rows share one scale group (rg0 is a multiple of 4, a group is 8 row groups)
    const int gi = rows_ok ? ((rg0 >> 3) % p.kg) % p.mg : 0;
    const half_t sc = p.scale[gi], zz = p.zp[gi];

    // Token tile staging: piece = (slot, token, 16 bytes).  Two tiles are on their
    // way in registers while a third is multiplied: a tile is requested two steps
    // before its use and written to LDS one step before.  The main loop has no
    // conditionals: loads past the end repeat the last tile (never used), tokens
    // past M repeat token M-1 (never stored).
    constexpr int PCS = kTokens * 4 * NH;  // pieces per slot
    constexpr int PPT = NKB * PCS / 256;
    const half_t* xsrc[PPT];
    int xdst[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      // k split: every wavefront stages its own slot (nobody else reads it: no workgroup barrier in the main loop)
      const int pc = KSPLIT ? wave * PCS + lane + i * 64 : tid + i * 256;
      const int j = pc / PCS, tok = (pc % PCS) / (4 * NH), part = pc % (4 * NH);
      const int tg = t0 + tok < p.M ? t0 + tok : p.M - 1;
      xsrc[i] = p.x + (int64_t)tg * p.k + (kb_wg + (KSPLIT ? j * tile_steps * NH : 0)) * 32 + part * 8;
      xdst[i] = j * kSlot + tok * kWideStride + part * 8;
    }
    xvec_t xr0[PPT], xr1[PPT];  // two named register sets (an indexed array would live in scratch memory)
    auto load_x = [&](int s, xvec_t (&dst)[PPT]) __attribute__((always_inline)) {
      const int sc_ = s < steps ? s : steps - 1;
#pragma unroll
      for (int i = 0; i < PPT; ++i) dst[i] = *reinterpret_cast<const xvec_t*>(xsrc[i] + sc_ * (32 * NH));
    };
    auto store_x = [&](int buf, const xvec_t (&src)[PPT]) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < PPT; ++i) *reinterpret_cast<xvec_t*>(xs + buf * NKB * kSlot + xdst[i]) = src[i];
    };

    // weights: row n of pair rp is row n % 16 of row group rg0 + 2 rp + n / 16; dwords 2kh, 2kh + 1 of its block
    const u32x2_t* wp[kWideRP];
#pragma unroll
    for (int a = 0; a < kWideRP; ++a) {
      const int rg = rows_ok ? rg0 + 2 * a + (n >> 4) : 0;
      wp[a] = reinterpret_cast<const u32x2_t*>(p.wq + (((int64_t)rg * p.nblk + kb_base) * 16 + (n & 15)) * 4 + 2 * kh);
    }
    // steps of weight dwords in registers.  Rows split: three sets, so that the set a step frees is
    // requested again at the very start of the next step, ahead of the token tile's requests: the wait
    // for the tile at the end of a step then covers no younger load.
    constexpr int PF = KSPLIT ? 2 : 3;
    u32x2_t wd[kWideRP][PF][NH];
#pragma unroll
    for (int f = 0; f < PF; ++f)
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wd[a][f][h] = KSPLIT ? __builtin_nontemporal_load(wp[a] + (int64_t)(f * NH + h) * 32) : wp[a][(int64_t)(f * NH + h) * 32];

    f32x16_t acc[kWideRP][TT];
#pragma unroll
    for (int a = 0; a < kWideRP; ++a)
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[a][t][i] = 0.0f;

    if constexpr (!KSPLIT) {
      // Rows split: the token tile of a step goes from memory straight into LDS
      // (global_load_lds_dwordx4: lane l of a wavefront instruction lands at base + 16 l), no
      // staging registers and no LDS writes.  A tile is [32 TT tokens][64 k] halves, 128 bytes per
      // token and unpadded; the eight 16-byte pieces of token row r sit at positions c ^ (r & 7), so
      // that the eight lanes that read the same piece of eight consecutive rows hit all 32 banks.
      // Three tiles rotate: during step s the requests for tile s + 2 are in flight (issued behind
      // the step's barrier, which the readers of tile s - 1 have passed), tile s is multiplied and
      // the last slice reads the first operands of tile s + 1.  The three tiles are three arrays so
      // that the compiler can tell which LDS reads a pending request may alias: it waits for the
      // requests only at the next barrier.  Same software pipeline over quarter steps as below.
      typedef __attribute__((address_space(1))) const void* gptr_t;
      typedef __attribute__((address_space(3))) void* lptr_t;
      constexpr int kTile = kTokens * 64;  // halves
      __shared__ __attribute__((aligned(16))) half_t tile_a[kTile];
      __shared__ __attribute__((aligned(16))) half_t tile_b[kTile];
      __shared__ __attribute__((aligned(16))) half_t tile_c[kTile];
      // requests: instruction i of this wavefront covers token rows (wave TT + i) 8 .. + 7
      const int piece = (lane & 7) ^ ((lane >> 3) & 7);  // piece of k this lane fetches for its row
      const half_t* src[TT];
#pragma unroll
      for (int i = 0; i < TT; ++i) {
        const int tok = t0 + (wave * TT + i) * 8 + (lane >> 3);
        src[i] = p.x + (int64_t)(tok < p.M ? tok : p.M - 1) * p.k + kb_wg * 32 + piece * 8;
      }
      auto request = [&](half_t* tile, int s) __attribute__((always_inline)) {
        const int sc_ = s < steps ? s : steps - 1;  // past the end: the last tile again, never used
#pragma unroll
        for (int i = 0; i < TT; ++i)
          __builtin_amdgcn_global_load_lds((gptr_t)(src[i] + sc_ * (32 * NH)), (lptr_t)(tile + (wave * TT + i) * 8 * 64), 16, 0, 0);
      };
      // operands: lane (n, kh) reads piece 4 h + 2 kh + j of token row 32 t + n
      const int swz = (2 * kh) ^ (n & 7);
      auto read_x = [&](const half_t* tile, int h, int j, half8_t (&dst)[TT]) __attribute__((always_inline)) {
        const half_t* at = tile + n * 64 + (((4 * h + j) ^ swz) << 3);
#pragma unroll
        for (int t = 0; t < TT; ++t) dst[t] = *reinterpret_cast<const half8_t*>(at + t * 32 * 64);
      };
      auto mma = [&](const half8_t (&xo)[TT], const half8_t (&wo)[kWideRP]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int a = 0; a < kWideRP; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xo[t], wo[a], acc[a][t], 0, 0, 0);
      };
      auto interleave = [&]() __attribute__((always_inline)) {
#define AWQ_SLOT(valu, lds)                                        \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); /* matrix */  \
  __builtin_amdgcn_sched_group_barrier(0x002, valu, 0);            \
  __builtin_amdgcn_sched_group_barrier(0x100, lds, 0);
        static_assert(TT == 4 || TT == 2, "slot patterns of the rows-split shapes");
        if constexpr (TT == 4) {
          AWQ_SLOT(3, 1) AWQ_SLOT(3, 1) AWQ_SLOT(2, 1) AWQ_SLOT(2, 1)
          AWQ_SLOT(2, 0) AWQ_SLOT(2, 0) AWQ_SLOT(2, 0) AWQ_SLOT(2, 0)
        } else {
          AWQ_SLOT(5, 1) AWQ_SLOT(5, 1) AWQ_SLOT(4, 0) AWQ_SLOT(4, 0)
        }
#undef AWQ_SLOT
      };
      half8_t xa[TT], xb_[TT], wa[kWideRP], wb[kWideRP];
      if (CUT) __syncthreads();  // the previous piece's readers are done
      request(tile_a, 0);
      request(tile_b, 1);
      __syncthreads();
      read_x(tile_a, 0, 0, xa);
#pragma unroll
      for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][0][0].x, sc, zz);
      // one step; B = s % 3 picks the tile and the weight register set
      auto step = [&](int s, auto B) __attribute__((always_inline)) {
        constexpr int bi = decltype(B)::value, b1 = (bi + 1) % 3, b2 = (bi + 2) % 3;
        half_t* const cur = bi == 0 ? tile_a : (bi == 1 ? tile_b : tile_c);
        half_t* const nxt = bi == 0 ? tile_b : (bi == 1 ? tile_c : tile_a);
        half_t* const tgt = bi == 0 ? tile_c : (bi == 1 ? tile_a : tile_b);
        // everything this wavefront requested a step ago has arrived (said here, so that no wait for a
        // register lands behind the new requests below)
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        __syncthreads();  // tile s + 1 has landed and is visible; the readers of tile s - 1 are done
        const int sn = s + 2 < steps ? s + 2 : steps - 1;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
          for (int a = 0; a < kWideRP; ++a) wd[a][b2][h] = wp[a][(int64_t)(sn * NH + h) * 32];
        request(tgt, s + 2);
        __builtin_amdgcn_sched_barrier(0);  // the requests stay here, a whole step ahead of the wait for them
        // slice (h 0, j 0): prepare (0, 1)
        read_x(cur, 0, 1, xb_);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wb[a] = dequant8<ZINT, false>(wd[a][bi][0].y, sc, zz);
        mma(xa, wa);
        interleave();
        // slice (0, 1): prepare (1, 0)
        read_x(cur, 1, 0, xa);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][bi][1].x, sc, zz);
        mma(xb_, wb);
        interleave();
        // slice (1, 0): prepare (1, 1)
        read_x(cur, 1, 1, xb_);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wb[a] = dequant8<ZINT, false>(wd[a][bi][1].y, sc, zz);
        mma(xa, wa);
        interleave();
        // slice (1, 1): prepare (0, 0) of the next step
        read_x(nxt, 0, 0, xa);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][b1][0].x, sc, zz);
        mma(xb_, wb);
        interleave();
      };
      using I0 = std::integral_constant<int, 0>;
      using I1 = std::integral_constant<int, 1>;
      using I2 = std::integral_constant<int, 2>;
      for (int s0 = 0; s0 < steps; s0 += 3) {
        step(s0, I0{});
        if (s0 + 1 < steps) step(s0 + 1, I1{});
        if (s0 + 2 < steps) step(s0 + 2, I2{});
      }
    } else {
      // k split: the same software pipeline over quarter steps.  A wavefront stages its own slot
      // (through registers: two tiles in flight) and nobody else reads it, so there is no workgroup
      // barrier; its LDS instructions execute in order, which lets two tiles do: tile s + 1 is written
      // before the last slice of step s reads it.
      auto publish = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the writes have left the queue
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      };
      auto wload = [&](int a, int64_t blk) __attribute__((always_inline)) {
        return __builtin_nontemporal_load(wp[a] + blk * 32);
      };
      load_x(0, xr0);
      store_x(0, xr0);
      load_x(1, xr1);
      half8_t xa[TT], xb_[TT], wa[kWideRP], wb[kWideRP];
      const half_t* xlane = xs + slot * kSlot + n * kWideStride + 16 * kh;
      auto read_x = [&](const half_t* tile, int h, int j, half8_t (&dst)[TT]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t) dst[t] = *reinterpret_cast<const half8_t*>(tile + t * 32 * kWideStride + h * 32 + 8 * j);
      };
      auto mma = [&](const half8_t (&xo)[TT], const half8_t (&wo)[kWideRP]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int a = 0; a < kWideRP; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xo[t], wo[a], acc[a][t], 0, 0, 0);
      };
      // the order the scheduler is asked for inside a slice: one matrix-core instruction, then a few
      // of the next slice's dequantisation instructions and one of its LDS reads
      auto interleave = [&]() __attribute__((always_inline)) {
#define AWQ_SLOT(valu, lds)                                        \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); /* matrix */  \
  __builtin_amdgcn_sched_group_barrier(0x002, valu, 0);            \
  __builtin_amdgcn_sched_group_barrier(0x100, lds, 0);
        if constexpr (TT == 4) {
          AWQ_SLOT(3, 1) AWQ_SLOT(3, 1) AWQ_SLOT(2, 1) AWQ_SLOT(2, 1)
          AWQ_SLOT(2, 0) AWQ_SLOT(2, 0) AWQ_SLOT(2, 0) AWQ_SLOT(2, 0)
        } else if constexpr (TT == 2) {
          AWQ_SLOT(5, 1) AWQ_SLOT(5, 1) AWQ_SLOT(4, 0) AWQ_SLOT(4, 0)
        } else {
          AWQ_SLOT(9, 1) AWQ_SLOT(9, 0)
        }
#undef AWQ_SLOT
      };
      publish();
      read_x(xlane, 0, 0, xa);
#pragma unroll
      for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][0][0].x, sc, zz);
      // one step; F is its index inside the unrolled pair (a compile-time constant): tile s is in
      // buffer F, tile s + 1 goes to the other one
      auto step = [&](int s0, auto F) __attribute__((always_inline)) {
        constexpr int f = decltype(F)::value;
        const int s = s0 + f;
        // the tile that left these registers one step ago
        if constexpr (f & 1) load_x(s + 2, xr1);
        else load_x(s + 2, xr0);
        const half_t* cur = xlane + f * NKB * kSlot;
        const half_t* nxt = xlane + (f ^ 1) * NKB * kSlot;
        const int sn = s + PF < steps ? s + PF : steps - 1;
        // slice (h 0, j 0): prepare (0, 1)
        read_x(cur, 0, 1, xb_);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) {
          wb[a] = dequant8<ZINT, false>(wd[a][f][0].y, sc, zz);
          wd[a][f][0] = wload(a, (int64_t)(sn * NH + 0));
        }
        mma(xa, wa);
        interleave();
        // slice (0, 1): prepare (1, 0)
        read_x(cur, 1, 0, xa);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][f][1].x, sc, zz);
        mma(xb_, wb);
        interleave();
        // slice (1, 0): prepare (1, 1)
        read_x(cur, 1, 1, xb_);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) {
          wb[a] = dequant8<ZINT, false>(wd[a][f][1].y, sc, zz);
          wd[a][f][1] = wload(a, (int64_t)(sn * NH + 1));
        }
        mma(xa, wa);
        interleave();
        // tile s + 1 goes to the other buffer now, ahead of the read below
        if constexpr (f & 1) store_x(0, xr0);
        else store_x(1, xr1);
        publish();
        // slice (1, 1): prepare (0, 0) of the next step
        read_x(nxt, 0, 0, xa);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) wa[a] = dequant8<ZINT, false>(wd[a][f ^ 1][0].x, sc, zz);
        mma(xb_, wb);
        interleave();
      };
      for (int s0 = 0; s0 < steps; s0 += 2) {
        step(s0, std::integral_constant<int, 0>{});
        step(s0, std::integral_constant<int, 1>{});
      }
    }

    const float scf = (float)sc;  // the wavefront's rows share one scale: it multiplies the sums, not every weight
    // acc[a][t][i] is D[token 32 t + 8 (i / 4) + 4 kh + i % 4][row 32 a + n]
    if constexpr (!KSPLIT) {
      typedef unsigned long long u64;
      const int b = blockIdx.x;
      // opaque to the compiler: the 64 slot addresses below are formed here, after the main loop, and
      // not once before the tile loop (where they would sit in scratch memory across the main loop)
      int tl = tid;
      asm volatile("" : "+v"(tl));
      if (CUT && s_lo + steps != tile_steps) {
        // the tile's last step is elsewhere: hand the sums over, element (a, t, i) pairs [thread]
        u64* mine = reinterpret_cast<u64*>(p.sk_part) + (int64_t)b * (kSkTileFloats / 2);
#pragma unroll
        for (int a = 0; a < kWideRP; ++a)
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const float2 v = float2{acc[a][t][2 * i], acc[a][t][2 * i + 1]};
              __hip_atomic_store(mine + ((a * TT + t) * 8 + i) * 256 + tl, __builtin_bit_cast(u64, v), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
            }
        // every wavefront's sums have reached the device-coherent level before the barrier; the count is a
        // release at agent scope, paired with the acquire after the owner's wait below
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
          const int owner = sk_wg_of((int64_t)(tile + 1) * S2 - 1, W2, gridDim.x);
          __hip_atomic_fetch_add(p.sk_head + 16 + owner, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
        continue;
      }
      if (CUT && s_lo != 0) {
        // the tile's first steps were taken by workgroups first .. b - 1, one slot each
        const int first = sk_wg_of((int64_t)tile * S2, W2, gridDim.x);
        // A wait that gives up (too many polls, or the host's "give up now" word at [1], looked at before the
        // first poll: the tests set it so that this path runs without any wait ever timing out) reports
        // through the status word, and the workgroup leaves its tile unwritten rather than storing sums
        // it does not have.
        __shared__ int gave_up;
        if (tid == 0) {
          int spins = 0;
          int lost = __hip_atomic_load(p.sk_head + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
          while (!lost && __hip_atomic_load(p.sk_head + 16 + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < b - first) {
            if (++spins > kSkSpinLimit) lost = 1;
            else __builtin_amdgcn_s_sleep(4);
          }
          if (lost) __hip_atomic_store(p.sk_head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // the counted workgroups' sums are visible from here
          // for the next launch.  (After giving up, the counted workgroups may still add to it: the host
          // clears the whole header when it sees the status word.)
          __hip_atomic_store(p.sk_head + 16 + b, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          gave_up = lost;
        }
        __syncthreads();
        if (gave_up) {
          __syncthreads();  // every thread has read the flag before the next tile's wait may write it
          continue;
        }
        for (int c = first; c < b; ++c) {
          const u64* theirs = reinterpret_cast<const u64*>(p.sk_part) + (int64_t)c * (kSkTileFloats / 2);
#pragma unroll
          for (int a = 0; a < kWideRP; ++a)
#pragma unroll
            for (int t = 0; t < TT; ++t) {
#pragma unroll
              for (int i = 0; i < 8; ++i) {
                const float2 v = __builtin_bit_cast(
                    float2, __hip_atomic_load(theirs + ((a * TT + t) * 8 + i) * 256 + tl, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT));
                acc[a][t][2 * i] += v.x;
                acc[a][t][2 * i + 1] += v.y;
              }
              __builtin_amdgcn_sched_barrier(0);  // 8 loads in flight, not all 64 (registers)
            }
        }
      }
      if (!rows_ok) continue;
#pragma unroll
      for (int a = 0; a < kWideRP; ++a) {
        const int row = rg0 * 16 + a * 32 + n;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int tok = t0 + t * 32 + (i >> 2) * 8 + kh * 4 + (i & 3);
            if (tok < p.M) store_out<EPI, true>(p, tok, row, acc[a][t][i] * scf);
          }
        }
      }
    } else {
      // k split: the four partial sums of every output meet in LDS (the token tiles
      // are dead by now); wavefront w finishes quarter w of every accumulator tile
      float4_t* red = reinterpret_cast<float4_t*>(smem_raw);  // [wave][pair][tile][quarter][lane]
      __syncthreads();
#pragma unroll
      for (int a = 0; a < kWideRP; ++a)
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4)
            red[(((wave * kWideRP + a) * TT + t) * 4 + i4) * 64 + lane] =
                float4_t{acc[a][t][4 * i4], acc[a][t][4 * i4 + 1], acc[a][t][4 * i4 + 2], acc[a][t][4 * i4 + 3]};
      __syncthreads();
      auto finish = [&](auto E) {
        constexpr int epi = decltype(E)::value;  // -1: this workgroup's chunk of k only, as FP32 partial sums
#pragma unroll
        for (int a = 0; a < kWideRP; ++a) {
          const int row = rg0 * 16 + a * 32 + n;
          const int i4 = wave;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            float4_t v = red[(((0 * kWideRP + a) * TT + t) * 4 + i4) * 64 + lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) v += red[(((w * kWideRP + a) * TT + t) * 4 + i4) * 64 + lane];
            v *= scf;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int tok = t0 + t * 32 + i4 * 8 + kh * 4 + i;
              if (tok < p.M) {
                if (epi < 0) p.part[((int64_t)blockIdx.z * p.M + tok) * p.m + row] = v[i];
                else store_out<(epi < 0 ? 0 : epi), true>(p, tok, row, v[i]);
              }
            }
          }
        }
      };
      if (p.kz > 1) finish(std::integral_constant<int, -1>{});
      else finish(std::integral_constant<int, EPI>{});
    }
  } while (CUT && --tile >= tile_first);
}

// 17..256 tokens on the 12288 x 4096 matrices: gemm_shared_kernel's scheme -- all weights requested at the start,
// the tokens through four rotating LDS tiles behind them, k split over eight wavefronts by 32-input block -- on
// RP pairs of 16-row groups per workgroup (64 rows: 192 workgroups) and v_mfma_f32_32x32x16_f16, twice the rate
// of the 16x16x32 shape, which holds gemm_shared_kernel at 0.39 us per step with three row groups.  A block is
// two matrix instructions of 16 inputs: lane (h, n) holds dwords 2 h and 2 h + 1 of weight row n of the pair
// (one 8-byte request) and reads the token pieces 2 h and 2 h + 1 of the block.  The 64 rows share one scale.
// On 4096 x 12288 k is cut over four workgroups as well (256 workgroups of 12 steps): their FP32 sums go to the
// workspace and a second launch adds them in slice order.
template <int TT32, int RP, int NS, int A, bool ZINT>
__global__ __launch_bounds__(512) void gemm_shared32_kernel(GemmParams p) {
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  constexpr int TD = 2 * TT32;             // tile requests per wavefront: 1 KB, two token rows each
  constexpr int kTile = 32 * TT32 * 256;   // halves per tile
  constexpr int NSLOT = 4;                 // tiles in LDS; A <= NSLOT of them requested ahead: step s reads tile s + 1, tile s was read a step ago
  static_assert((NS - 2) * RP + A * TD < 64, "the request counter has six bits");
  static_assert(A >= 2 && A <= NSLOT && A < NS, "at least two tiles ahead, each in a slot of its own");
  extern __shared__ __attribute__((aligned(16))) unsigned char shared32_lds[];
  half_t* const tiles = reinterpret_cast<half_t*>(shared32_lds);  // NSLOT of them
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5, n = lane & 31;
  const int rg0 = blockIdx.x * (2 * RP);
  const int step0 = blockIdx.y * NS;  // k cut over p.kz workgroups: NS steps each, their FP32 sums to p.part
  // the request order and the counts at the barriers are gemm_shared_kernel's
  uint32_t sc_raw, zz_raw;
  u32x2_t w[NS][RP];
  {
    const int gi = ((rg0 >> 3) % p.kg) % p.mg;
    asm volatile("global_load_ushort %0, %1, off" : "=v"(sc_raw) : "v"(p.scale + gi) : "memory");
    asm volatile("global_load_ushort %0, %1, off" : "=v"(zz_raw) : "v"(p.zp + gi) : "memory");
  }
  half_t sc, zz;
  // the operands of token tile t: row 32 t + n, pieces 4 wave + 2 h and + 1 of the step
  const int xoff0 = n * 256 + (((4 * wave + 2 * h) ^ n) << 3), xoff1 = n * 256 + (((4 * wave + 2 * h + 1) ^ n) << 3);
  // More than 32 TT32 tokens: one slab of 32 TT32 tokens after the other against the same weights, which stay in
  // their registers.  Only the first slab has weights in flight next to its tiles.
  auto slab = [&](auto FIRST, int t0) __attribute__((always_inline)) {
    constexpr bool first = decltype(FIRST)::value;
    const half_t* src[TD];
#pragma unroll
    for (int i = 0; i < TD; ++i) {
      const int row = 2 * (wave * TD + i) + (lane >> 5);
      const int piece = (lane & 31) ^ (row & 31);
      src[i] = p.x + (int64_t)min(t0 + row, p.M - 1) * p.k + piece * 8 + step0 * 256;
    }
    auto request = [&](int s) __attribute__((always_inline)) {
      half_t* const tile = tiles + (s % NSLOT) * kTile + wave * TD * 512;
#pragma unroll
      for (int i = 0; i < TD; ++i) __builtin_amdgcn_global_load_lds((gptr_t)(src[i] + s * 256), (lptr_t)(tile + i * 512), 16, 0, 0);
    };
#pragma unroll
    for (int s = 0; s < A; ++s) request(s);
    asm volatile("" ::: "memory");
    if constexpr (first) {
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int a = 0; a < RP; ++a) {
          const int rg = rg0 + 2 * a + (n >> 4);
          const uint32_t* at = p.wq + (((int64_t)rg * p.nblk + wave + 8 * (step0 + s)) * 16 + (n & 15)) * 4 + 2 * h;
          asm volatile("global_load_dwordx2 %0, %1, off nt" : "=v"(w[s][a]) : "v"(at) : "memory");
        }
    }
    f32x16_t acc[RP][TT32];
#pragma unroll
    for (int a = 0; a < RP; ++a)
#pragma unroll
      for (int t = 0; t < TT32; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[a][t][e] = 0.0f;
    // the scales, the tiles ahead and the first weights; a later slab: tile 0
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(first ? (NS - 1) * RP : (A - 1) * TD));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (first) {
      asm volatile("" : "+v"(sc_raw), "+v"(zz_raw));
      sc = __builtin_bit_cast(half_t, (unsigned short)sc_raw);
      zz = __builtin_bit_cast(half_t, (unsigned short)zz_raw);
    }
    half8_t xr[2][TT32][2], wop[2][RP][2];
#pragma unroll
    for (int t = 0; t < TT32; ++t) {
      xr[0][t][0] = *reinterpret_cast<const half8_t*>(tiles + t * 32 * 256 + xoff0);
      xr[0][t][1] = *reinterpret_cast<const half8_t*>(tiles + t * 32 * 256 + xoff1);
    }
#pragma unroll
    for (int a = 0; a < RP; ++a) {
      asm volatile("" : "+v"(w[0][a]));
      wop[0][a][0] = dequant8<ZINT, false>(w[0][a].x, sc, zz);
      wop[0][a][1] = dequant8<ZINT, false>(w[0][a].y, sc, zz);
    }
    static_for<NS>([&](auto S) __attribute__((always_inline)) {
      constexpr int s = decltype(S)::value, c = s & 1, nx = c ^ 1;
      // Tile s + 1 and the weights of step s + 1.  A tile requested before the loop of the first slab is ahead
      // of the weights: the later steps' weights and the tiles requested by the steps so far may be out.  A tile
      // requested by a step is behind all the weights, and a later slab has none in flight: the tiles requested
      // since may be out.
      constexpr int since = A - 2 < NS - 2 - s ? A - 2 : (NS - 2 - s > 0 ? NS - 2 - s : 0);
      constexpr int so_far = s < NS - A ? s : NS - A;
      __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(first && s + 1 < A ? (NS - 2 - s) * RP + so_far * TD : since * TD));
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if constexpr (s + 1 < NS) {
#pragma unroll
        for (int a = 0; a < RP; ++a) asm volatile("" : "+v"(w[s + 1][a]));  // not read before the wait above
      }
      // (what this step multiplies is not touched before the barrier: its products would wait for the reads there)
#pragma unroll
      for (int t = 0; t < TT32; ++t) asm volatile("" : "+v"(xr[c][t][0]), "+v"(xr[c][t][1]));
#pragma unroll
      for (int a = 0; a < RP; ++a) asm volatile("" : "+v"(wop[c][a][0]), "+v"(wop[c][a][1]));
      if constexpr (s + A < NS) request(s + A);
      if constexpr (s + 1 < NS) {
#pragma unroll
        for (int t = 0; t < TT32; ++t) {
          xr[nx][t][0] = *reinterpret_cast<const half8_t*>(tiles + ((s + 1) % NSLOT) * kTile + t * 32 * 256 + xoff0);
          xr[nx][t][1] = *reinterpret_cast<const half8_t*>(tiles + ((s + 1) % NSLOT) * kTile + t * 32 * 256 + xoff1);
        }
      }
#pragma unroll
      for (int a = 0; a < RP; ++a) {
        if constexpr (s + 1 < NS) {
          wop[nx][a][0] = dequant8<ZINT, false>(w[s + 1][a].x, sc, zz);
          wop[nx][a][1] = dequant8<ZINT, false>(w[s + 1][a].y, sc, zz);
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int t = 0; t < TT32; ++t)
            acc[a][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xr[c][t][kk], wop[c][a][kk], acc[a][t], 0, 0, 0);
      }
    });
    __syncthreads();  // every wavefront has read its operands: the tiles make room for the sums
    float4_t* red = reinterpret_cast<float4_t*>(shared32_lds);  // [wavefront][pair][token tile][quarter][lane]
#pragma unroll
    for (int a = 0; a < RP; ++a)
#pragma unroll
      for (int t = 0; t < TT32; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          red[(((wave * RP + a) * TT32 + t) * 4 + g) * 64 + lane] =
              float4_t{acc[a][t][4 * g], acc[a][t][4 * g + 1], acc[a][t][4 * g + 2], acc[a][t][4 * g + 3]};
    __syncthreads();
    // D[token 8 g + 4 (lane / 32) + e][row lane % 32] sits in element 4 g + e of the lane
    const float scf = (float)sc;
    with_epilogue(p, [&](auto E) {
#pragma unroll
      for (int idx = tid; idx < RP * TT32 * 256; idx += 512) {
        const int a = idx / (TT32 * 256), t = (idx >> 8) % TT32, g = (idx >> 6) & 3;
        float4_t v = red[idx];
#pragma unroll
        for (int wv = 1; wv < 8; ++wv) v += red[wv * (RP * TT32 * 256) + idx];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int tok = t0 + 32 * t + 8 * g + 4 * h + e, row = (rg0 + 2 * a) * 16 + n;
          if (tok >= p.M) continue;
          if (p.kz > 1) p.part[((int64_t)blockIdx.y * p.M + tok) * p.m + row] = v[e] * scf;  // finished by reduce_parts_kernel
          else store_out<decltype(E)::value, true>(p, tok, row, v[e] * scf);
        }
      }
    });
  };
  slab(std::true_type{}, 0);
  for (int t0 = 32 * TT32; t0 < p.M; t0 += 32 * TT32) {
    __syncthreads();  // the sums of the slab before have been read: its place takes tiles again
    slab(std::false_type{}, t0);
  }
}

// k cut over several workgroups: the chunks' FP32 partial sums are added in
// chunk order (whatever order the workgroups ran in), then the epilogue
__global__ __launch_bounds__(256) void reduce_parts_kernel(GemmParams p) {
  const int64_t total = (int64_t)p.M * p.m;
  const int64_t at = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (at >= total) return;
  float v = p.part[at];
  for (int z = 1; z < p.kz; ++z) v += p.part[(int64_t)z * total + at];
  with_epilogue(p, [&](auto E) { store_out<decltype(E)::value, true>(p, (int)(at / p.m), (int)(at % p.m), v); });
}

// tokens per workgroup of the k-split shape: 32, 64 or 128
// tokens per workgroup of the k-split shape, in units of 32: 32, 64 or 128 by the token count; fewer
// when a matrix with few rows and short k would otherwise get under 128 workgroups (4096 x 4096 at
// 128 tokens: 18.4 -> 14.5 us; with long k the cut over workgroups does better)
int wide_tt(int64_t m, int64_t k, int64_t M) {
  int tt = M <= 32 ? 1 : (M <= 64 ? 2 : 4);
  if (k <= 4096)
    while (tt > 1 && (m / 64) * ((M + 32 * tt - 1) / (32 * tt)) < 128) tt >>= 1;
  return tt;
}

template <int MODE, int TT>
int launch_wide(const GemmParams& p, bool zint, int n_wgs, hipStream_t st) {
  constexpr bool KSPLIT = MODE == WIDE_K;
  // the main loop takes two steps of two 32-wide blocks per trip (per quarter of k when k is split)
  AWQ_REQUIRE(p.nblk % (KSPLIT ? 16 * p.kz : 4) == 0, KSPLIT ? "k must be a multiple of 512" : "k must be a multiple of 128");
  constexpr int lds = wide_lds_bytes(KSPLIT, TT);
  static_assert(lds <= 160 * 1024, "LDS of one compute unit");
  dim3 grid((unsigned)(p.m / 64), (unsigned)((p.M + 32 * TT - 1) / (32 * TT)), (unsigned)p.kz);
  if (!KSPLIT) grid = dim3((unsigned)n_wgs);
  void (*kern)(GemmParams);
  int variant;
  if (p.epilogue == EPI_RESIDUAL) {
    kern = zint ? gemm_wide_kernel<true, MODE, EPI_RESIDUAL, TT> : gemm_wide_kernel<false, MODE, EPI_RESIDUAL, TT>;
    variant = zint ? 0 : 1;
  } else if (p.epilogue == EPI_GELU) {
    kern = zint ? gemm_wide_kernel<true, MODE, EPI_GELU, TT> : gemm_wide_kernel<false, MODE, EPI_GELU, TT>;
    variant = zint ? 2 : 3;
  } else {
    kern = zint ? gemm_wide_kernel<true, MODE, EPI_STORE, TT> : gemm_wide_kernel<false, MODE, EPI_STORE, TT>;
    variant = zint ? 4 : 5;
  }
  if (lds > 65536) {
    // more LDS than a launch gets by default: raise this kernel's limit, once per device
    static std::atomic<uint64_t> raised[6];
    int dev = 0;
    AWQ_HIP_TRY(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (!(raised[variant].load(std::memory_order_relaxed) & bit)) {
      AWQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
      raised[variant].fetch_or(bit, std::memory_order_relaxed);
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, p);
  if (KSPLIT && p.kz > 1) {
    const int64_t total = (int64_t)p.M * p.m;
    hipLaunchKernelGGL(reduce_parts_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p);
  }
  return AWQ_OK;
}

template <int G, int TT>
int launch_small(const GemmParams& p, bool zint, int n_waves, dim3 grid, hipStream_t st) {
  // the tokens of a workgroup in LDS: rows of k halves plus the skew and 16 bytes between rows
  const size_t lds = (size_t)std::min<int64_t>(16 * TT, p.M) * (p.k + (p.nblk / G) * 8 + 8) * 2;
  // token pieces per thread that are requested ahead of the weights
  const int64_t pieces = (std::min<int64_t>(16 * TT, p.M) * (p.k / 8) + n_waves * 64 - 1) / (n_waves * 64);
  auto kern = pieces <= 2 ? (zint ? gemm_small_kernel<G, TT, true, 2> : gemm_small_kernel<G, TT, false, 2>)
            : pieces <= 4 ? (zint ? gemm_small_kernel<G, TT, true, 4> : gemm_small_kernel<G, TT, false, 4>)
                          : (zint ? gemm_small_kernel<G, TT, true, 8> : gemm_small_kernel<G, TT, false, 8>);
  if (lds > 65536 - sizeof(float) * 16 * TT * 64 * 4) {
    // more LDS than a launch gets by default: raise this kernel's limit (cheap, so done per call)
    AWQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  hipLaunchKernelGGL(kern, grid, dim3(n_waves * 64), lds, st, p, n_waves);
  return AWQ_OK;
}

}  // namespace

constexpr int kMidLdsBytes = 16 * 16 * kMidRow;  // 16 wavefronts x 16 tokens (the sums need less)
template <int G, int RG>
int launch_mid(const GemmParams& p, bool zint, int n_rg, hipStream_t st) {
  auto kern = zint ? gemm_mid_kernel<G, RG, true> : gemm_mid_kernel<G, RG, false>;
  // more LDS than a launch gets by default: raise this kernel's limit (cheap, so done per call)
  AWQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kMidLdsBytes));
  hipLaunchKernelGGL(kern, dim3((unsigned)((n_rg + RG - 1) / RG)), dim3(1024), kMidLdsBytes, st, p, n_rg);
  return AWQ_OK;
}
// 2..16 tokens and k of 128, 256, 384 or 512 blocks: the row groups per workgroup (0: this kernel does not
// take the product).  As many as the registers hold (at most three) while at least 256 workgroups remain.
int mid_row_groups(int64_t m, int64_t k, int64_t M) {
  if (M < 2 || M > 16 || k % 4096 != 0 || k > 16384 || m % 16 != 0) return 0;
  int rg = (int)(4 / (k / 4096));
  if (rg > 3) rg = 3;
  if (rg < 1) rg = 1;
  while (rg > 1 && (m / 16 + rg - 1) / rg < 256) --rg;
  return rg;
}

// 17..64 and 129..192 tokens on 4096 rows and k of 2048 or 4096: gemm_shared_kernel, one 16-row group per compute
// unit (4096 x 4096: 6.4-6.8 us at 17..32 tokens, 8.6-9.4 us at 48..64, against 9.1-9.2 and 10.3-10.5 us of the
// k-split workgroups; in slabs of 64 tokens 19.2 against 22.1 us at 192, level with them at 65..128 -- 13.4-14.2 --
// and behind at 256, 24.3 against 22.7)
bool shared_takes(int64_t m, int64_t k, int64_t M) {
  return ((M >= 17 && M <= 64) || (M >= 129 && M <= 192)) && (k == 2048 || k == 4096) && m == 4096;
}
template <int TT, int NS>
int launch_shared(const GemmParams& p, bool zint, hipStream_t st) {
  auto kern = zint ? gemm_shared_kernel<TT, 1, NS, true> : gemm_shared_kernel<TT, 1, NS, false>;
  constexpr int lds = 4 * 16 * TT * 256 * 2;  // four token tiles (the sums need no more)
  static_assert(lds >= 8 * TT * 1024, "the sums take the place of the tiles");
  if (lds > 65536) {
    // more LDS than a launch gets by default: raise this kernel's limit, once per device
    static std::atomic<uint64_t> raised[2];
    int dev = 0;
    AWQ_HIP_TRY(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (!(raised[zint].load(std::memory_order_relaxed) & bit)) {
      AWQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
      raised[zint].fetch_or(bit, std::memory_order_relaxed);
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.m / 16)), dim3(512), lds, st, p, p.m / 16);
  return AWQ_OK;
}

// 17..256 tokens on 10240..16384 rows and k of 2048 or 4096 (the model's 12288 x 4096): gemm_shared32_kernel, 64
// rows per workgroup, slabs of 64 tokens (12288 x 4096: 22.9 us at 128 tokens, 31.5 at 192, 39.5 at 256 against
// 24.6 / 45.0 / 44.8 of the k-split and rows-split workgroups; 48.1 against 44.9 at 320)
bool shared32_takes(int64_t m, int64_t k, int64_t M) {
  return M >= 17 && M <= 256 && (k == 2048 || k == 4096) && m % 128 == 0 && m >= 10240 && m <= 16384;
}
// ... and 128..320 tokens on 4096 x 12288 with k cut over four workgroups (needs the workspace for their sums):
// 25.9 us at 128 tokens, 35.2 at 192, 43.3 at 256, 52.1 at 320 against 26.8 / 45.0 / 47.2 / 57.9 of the k-split
// and rows-split workgroups (slower than those below 128 and from 384 on, and on 4096 x 4096 throughout)
bool shared32_kcut_takes(int64_t m, int64_t k, int64_t M) { return M >= 128 && M <= 320 && k == 12288 && m == 4096; }
template <int TT32, int NS>
int launch_shared32(const GemmParams& p, bool zint, hipStream_t st) {
  // tiles requested ahead of the weights (and kept ahead of the steps): 64 tokens 13.8 us with three, 14.2 with
  // four, 14.3 with five slots and five ahead; up to 32 tokens 10.4 / 10.2 / 10.7 (eight)
  constexpr int A = TT32 == 2 ? 3 : 4;
  auto kern = zint ? gemm_shared32_kernel<TT32, 2, NS, A, true> : gemm_shared32_kernel<TT32, 2, NS, A, false>;
  constexpr int lds = 4 * 32 * TT32 * 256 * 2;  // four token tiles; the eight wavefronts' sums need as much
  static_assert(lds >= 8 * 2 * TT32 * 4096, "the sums take the place of the tiles");
  if (lds > 65536) {
    // more LDS than a launch gets by default: raise this kernel's limit, once per device
    static std::atomic<uint64_t> raised[2];
    int dev = 0;
    AWQ_HIP_TRY(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (!(raised[zint].load(std::memory_order_relaxed) & bit)) {
      AWQ_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
      raised[zint].fetch_or(bit, std::memory_order_relaxed);
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.m / 64), (unsigned)p.kz), dim3(512), lds, st, p);
  if (p.kz > 1) {
    const int64_t total = (int64_t)p.M * p.m;
    hipLaunchKernelGGL(reduce_parts_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p);
  }
  return AWQ_OK;
}

// Which workgroup shape a many-token product takes (measured on the three matrix shapes of the
// model, 128 to 4096 tokens):
//   fewer than 80 tiles of 256 rows x 128 tokens          k split
//   tiles would leave a third of the compute units idle:
//     k <= 4096 and at least 128 tiles of 64 tokens       rows split, 64 tokens per workgroup (no hand-over;
//                                                         the attention output matrix at 640..1024 tokens: -25 %)
//     otherwise, with a workspace                          rows split, work cut evenly: two aligned pieces per
//                                                         tile up to 128 tiles, 256 equal ranges above
//   257..384 tiles, k <= 4096                              rows split, 64 tokens per workgroup, three workgroups per
//                                                         compute unit in one round instead of two uneven rounds
//   otherwise                                              rows split, a tile per workgroup
enum WidePlan { PLAN_K, PLAN_ROWS, PLAN_ROWS_64, PLAN_ROWS_CUT };
// k split: k also cut over 2-4 workgroups (second launch adds the chunks) when the 64-row workgroups
// are few; with 65..128 of them only for long k (4096 x 4096 at 256 tokens: 29 us with, 23 us without;
// 4096 x 12288: 48 us with, 58 us without)
static bool k_cut_pays(int64_t wgs, int64_t k) { return wgs <= 64 || (wgs <= 128 && k >= 8192); }
static WidePlan plan_wide(int64_t m, int64_t k, int64_t M, bool has_workspace) {
  const int64_t nr = (m + 255) / 256;
  const int64_t tiles = nr * ((M + kWideTokens - 1) / kWideTokens), tiles64 = nr * ((M + 63) / 64);
  if (tiles < kRowsSplitMinTiles) return PLAN_K;
  // 257..384 tiles would run as two uneven rounds of two workgroups per compute unit; as 64-token tiles
  // they are one round of three (12288 x 4096 at 704..1024 tokens: -5 to -11 %)
  if (k <= 4096 && tiles > kSkWgs && tiles64 <= 3 * kSkWgs) return PLAN_ROWS_64;
  if (tiles * 3 > kSkWgs * 2) return PLAN_ROWS;
  if (k <= 4096 && tiles64 >= 128) return PLAN_ROWS_64;
  const int64_t pairs = tiles * (k / AWQ_BLOCK_K / kWideNH / 2);
  return has_workspace && pairs / 4 >= kSkWgs ? PLAN_ROWS_CUT : PLAN_ROWS;
}

// room for a header and the partial sums of a product whose work is cut over workgroups (0: never cut)
// the shape awq_gemm takes for a product (diagnostics and tests): 0 few tokens, 1 k split, 2 rows split
// with a tile per workgroup, 3 rows split with 64 tokens per workgroup, 4 rows split with the work cut evenly,
// 5 up to 16 tokens with several row groups per workgroup, 6 17..64 and 129..192 tokens on 4096 rows with the tokens shared
// through LDS, 7 17..256 tokens on 10240..16384 rows the same way with 64 rows per workgroup, 8 the same with k
// cut over four workgroups (4096 x 12288 at 128..320 tokens)
int gemm_plan(int64_t m, int64_t k, int64_t M, int has_workspace) {
  if (M >= 2 && mid_row_groups(m, k, M)) return 5;
  if (shared_takes(m, k, M)) return 6;
  if (shared32_takes(m, k, M)) return 7;
  if (has_workspace && shared32_kcut_takes(m, k, M)) return 8;
  if (M <= 4) return 0;
  switch (plan_wide(m, k, M, has_workspace != 0)) {
    case PLAN_K: return 1;
    case PLAN_ROWS: return 2;
    case PLAN_ROWS_64: return 3;
    default: return 4;
  }
}

int64_t gemm_workspace_bytes(int64_t m, int64_t k, int64_t M) {
  if (shared32_kcut_takes(m, k, M)) return kSkHeaderBytes + 4 * M * m * 4;
  if (M <= 4 || mid_row_groups(m, k, M) || shared_takes(m, k, M) || shared32_takes(m, k, M)) return 0;
  switch (plan_wide(m, k, M, true)) {
    case PLAN_ROWS_CUT: return kSkHeaderBytes + (int64_t)kSkWgs * kSkTileFloats * 4;
    case PLAN_K: {
      const int tokens = 32 * wide_tt(m, k, M);
      const int64_t wgs = (m / 64) * ((M + tokens - 1) / tokens);
      return k_cut_pays(wgs, k) ? kSkHeaderBytes + 4 * M * m * 4 : 0;
    }
    default: return 0;
  }
}

int launch_gemm(const void* wq, const half_t* scale, const half_t* zp, int64_t m, int64_t k, const half_t* x,
                half_t* y, int64_t M, int zp_integral, int epilogue, const half_t* res, void* workspace,
                int64_t workspace_bytes, hipStream_t st) {
  AWQ_REQUIRE(epilogue == EPI_STORE || epilogue == EPI_GELU || (epilogue == EPI_RESIDUAL && res),
              "epilogue must be store, GeLU or residual (with res)");
  AWQ_REQUIRE(m > 0 && m % 128 == 0 && k > 0 && k % 128 == 0, "m and k must be positive multiples of 128");
  AWQ_REQUIRE(M >= 1 && M <= (1 << 20), "M out of range");
  AWQ_REQUIRE(awq_group_period(m, k) == 1, "matrices whose scale group depends on the input index are not supported here");
  AWQ_REQUIRE(m < (1ll << 31) && k < (1ll << 31), "shape too large");
  // the kernels read the weights and the tokens 16 bytes at a time (the tokens also straight into LDS)
  AWQ_REQUIRE(((uintptr_t)wq & 15) == 0 && ((uintptr_t)x & 15) == 0, "the weights and x must be 16-byte aligned");
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
  p.epilogue = epilogue;
  p.res = res;
  p.kz = 1;
  p.part = nullptr;
  p.nr = p.n_tiles = 0;
  p.sk_head = nullptr;
  p.sk_part = nullptr;
  if (shared32_kcut_takes(m, k, M) && workspace && kSkHeaderBytes + 4 * M * m * 4 <= workspace_bytes) {
    p.kz = 4;
    p.part = (float*)((char*)workspace + kSkHeaderBytes);
    if (int rc = launch_shared32<2, 12>(p, zp_integral, st)) return rc;
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  if (shared32_takes(m, k, M)) {
    int rc;
    if (k == 4096) rc = M <= 32 ? launch_shared32<1, 16>(p, zp_integral, st) : launch_shared32<2, 16>(p, zp_integral, st);
    else rc = M <= 32 ? launch_shared32<1, 8>(p, zp_integral, st) : launch_shared32<2, 8>(p, zp_integral, st);
    if (rc) return rc;
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  if (shared_takes(m, k, M)) {
    int rc;
    if (k == 4096) rc = M <= 32 ? launch_shared<2, 16>(p, zp_integral, st) : launch_shared<4, 16>(p, zp_integral, st);
    else rc = M <= 32 ? launch_shared<2, 8>(p, zp_integral, st) : launch_shared<4, 8>(p, zp_integral, st);
    if (rc) return rc;
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  if (const int rgs = mid_row_groups(m, k, M)) {
    const int n_rg = (int)(m / 16);
    int rc;
    switch ((int)(k / 4096) * 4 + rgs) {
      case 1 * 4 + 3: rc = launch_mid<2, 3>(p, zp_integral, n_rg, st); break;
      case 1 * 4 + 2: rc = launch_mid<2, 2>(p, zp_integral, n_rg, st); break;
      case 1 * 4 + 1: rc = launch_mid<2, 1>(p, zp_integral, n_rg, st); break;
      case 2 * 4 + 2: rc = launch_mid<4, 2>(p, zp_integral, n_rg, st); break;
      case 2 * 4 + 1: rc = launch_mid<4, 1>(p, zp_integral, n_rg, st); break;
      case 3 * 4 + 1: rc = launch_mid<6, 1>(p, zp_integral, n_rg, st); break;
      default: rc = launch_mid<8, 1>(p, zp_integral, n_rg, st); break;
    }
    if (rc) return rc;
    AWQ_HIP_TRY(hipGetLastError());
    return AWQ_OK;
  }
  // up to 4 tokens: the decode kernel's decomposition (one 16-token operand tile, mostly padding)
  int g = 0;
  if (M <= 4) {
    // lane groups of G blocks: (k/32)/G of them, a multiple of 4 and at most 64
    const int64_t nblk = k / AWQ_BLOCK_K;
    // the longest run per lane that still gives the workgroup eight wavefronts (as in the decode kernel)
    for (int c : {8, 4, 2, 1})
      if (nblk % c == 0 && (nblk / c) % 4 == 0 && nblk / c <= 64) {
        g = c;
        if (nblk / c / 4 >= 8) break;
      }
  }
  if (g) {
    const int n_waves = (int)(k / AWQ_BLOCK_K / g / 4);
    dim3 grid((unsigned)(m / 16), 1);
    int rc;
    switch (g) {
      case 8: rc = launch_small<8, 1>(p, zp_integral, n_waves, grid, st); break;
      case 4: rc = launch_small<4, 1>(p, zp_integral, n_waves, grid, st); break;
      case 2: rc = launch_small<2, 1>(p, zp_integral, n_waves, grid, st); break;
      default: rc = launch_small<1, 1>(p, zp_integral, n_waves, grid, st); break;
    }
    if (rc) return rc;
  } else {
    const int64_t nr = (m + 255) / 256;
    const int64_t tiles = nr * ((M + kWideTokens - 1) / kWideTokens);
    // the partial sums start behind the header, whichever kernel writes them
    char* ws_part = workspace ? (char*)workspace + kSkHeaderBytes : nullptr;
    const int64_t part_bytes = workspace_bytes - kSkHeaderBytes;
    const bool room = workspace && kSkWgs * (int64_t)kSkTileFloats * 4 <= part_bytes;
    const WidePlan plan = plan_wide(m, k, M, room);
    if (plan != PLAN_K) {
      AWQ_REQUIRE(tiles < (1ll << 30), "too many output tiles");
      p.nr = (int32_t)nr;
      p.n_tiles = (int32_t)tiles;
      int rc;
      if (plan == PLAN_ROWS_64) {
        p.n_tiles = (int32_t)(nr * ((M + 63) / 64));
        rc = launch_wide<WIDE_ROWS, 2>(p, zp_integral, p.n_tiles, st);
      } else if (plan == PLAN_ROWS_CUT) {
        p.sk_head = (int32_t*)workspace;
        p.sk_part = (float*)ws_part;
        rc = launch_wide<WIDE_ROWS_CUT, 4>(p, zp_integral, (int)(2 * tiles <= kSkWgs ? 2 * tiles : kSkWgs), st);
      } else {
        rc = launch_wide<WIDE_ROWS, 4>(p, zp_integral, (int)tiles, st);
      }
      if (rc) return rc;
    } else {
      // few 64-row workgroups too (a matrix with few rows): cut k over 4 or 2 workgroups as well,
      // when the caller brought room for the partial sums
      const int tt = wide_tt(m, k, M);
      const int64_t wgs = (m / 64) * ((M + 32 * tt - 1) / (32 * tt));
      if (k_cut_pays(wgs, k) && workspace) {
        for (int kz : {4, 2})
          if (p.nblk % (16 * kz) == 0 && (int64_t)kz * M * m * 4 <= part_bytes) {
            p.kz = kz;
            p.part = (float*)ws_part;
            break;
          }
      }
      if (int rc = tt == 1 ? launch_wide<WIDE_K, 1>(p, zp_integral, 0, st)
                           : tt == 2 ? launch_wide<WIDE_K, 2>(p, zp_integral, 0, st)
                                     : launch_wide<WIDE_K, 4>(p, zp_integral, 0, st))
        return rc;
    }
  }
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
