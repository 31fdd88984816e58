// Int4 weight kernels for gfx950: the bit-exact standalone dequantisation, the
// load-time reordering of the packed stream, and the fused dequant + matrix-
// vector product used for decode.
//
// Weight stream after reordering.  The [m outputs x k inputs] matrix is cut
// into groups of 16 output rows; the k inputs of a row into blocks of 32 in
// the order of awq_block_elem (awq_canon_math.h).  One 16-byte load hands a
// lane one whole block of its row:
//     byte offset = ((rg * (k/32) + blk) * 16 + r) * 16,   rg = row/16, r = row%16
// A workgroup owns one row group (or half of one) and all of k, so no partial
// sums ever leave the workgroup: lane (wavefront w, quarter q = lane/16,
// r = lane%16) takes the G consecutive blocks starting at (4w+q)*G of row
// 16*rg + r; a wavefront load is four contiguous 256-byte pieces, and the G
// loads of a lane walk 256*G contiguous bytes per quarter.  Inside the 16
// bytes, dword c holds elements 8c..8c+7 with nibble positions
// {0,16,4,20,8,24,12,28}[t & 7].  The decode kernel hands a lane's 16 bytes to
// v_mfma_i32_16x16x64_i8 as they stand but for two masks (low nibbles, high
// nibbles) against byte planes of the inputs, or, for half row groups and eight
// blocks per lane, multiplies a dword as it is in v_dot8_u32_u4 (eight 4-bit
// weights against eight 4-bit digits of the inputs laid out the same way); the
// many-token kernels mask with 0x000f000f / 0x00f000f0 (and the same after one
// shift by 8) to get two weights at a time as a packed pair of binary16 values.
#include "common.hpp"
#include "gemv_device.hpp"

#include <stdlib.h>

#include <algorithm>

namespace {

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

// arguments of the sampling step's last launch
struct SampleFinish {
  unsigned long long* best;
  int32_t* out_token;
  int32_t* out_array;
  const StepState* dyn;
  half_t* hidden;  // null = only the token id is produced
  half_t* hidden_last;
  const uint8_t* emb_rows;
  const half_t* emb_scale;
  const half_t* emb_zp;
  int32_t n;
  StepState* state;
  int32_t epoch_step;
};

// the 16 finished rows of a workgroup; r = lane = row % 16, lanes 0..15 of wavefront 0
// (Requesting the position, cosine and sine of the rotary epilogue at the start of the launch instead of after
// the reduction was tried in three forms -- position before the weight requests, after them, as a vector load
// with x -- and made the launch 0.4 to 1.0 us slower each time.)
__device__ __forceinline__ void epilogue(const GemvParams& p, int epi, int row, int r, float acc, half_t res,
                                         unsigned long long& best_here) {
  half_t v = (half_t)acc;
  switch (epi) {
    case EPI_RESIDUAL:  // Inference.cu:1149-1155
      store_through(p.y + row, res + v);
      return;
    case EPI_GELU:  // Inference.cu:271-279
      store_through(p.y + row, to_half_rn(awq_gelu_f32((float)v)));
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
      // Inference.cu:1278-1290 on the device: the best (value, lowest index) pair is a maximum over
      // 64-bit candidates, which does not depend on the order; each lane keeps the best of its rows
      // and the workgroup publishes one candidate when it has walked all its row groups
      p.y[row] = v;
      const unsigned short bits = __builtin_bit_cast(unsigned short, v);
      int32_t key = awq_logit_key(bits);
      if (row == 0 && (bits & 0x7fffu) > 0x7c00u) key = INT32_MAX;  // a NaN at index 0 is never displaced
      const unsigned long long cand = awq_pack_candidate(key, (uint32_t)row);
      best_here = cand > best_here ? cand : best_here;
      return;
    }
    default:
      p.y[row] = v;
  }
}

// Last launch of the sampling step (Inference.cu:1282-1290, then :1384-1398): turns the best candidate into
// the token id and, in the engine's decode step, prepares the next step: a copy of the hidden state for
// readers, the sampled token's embedding (gather lambda, Inference.cu:1310-1324) as the new hidden state,
// and the step state advanced by one position.  One workgroup; the embedding comes from the table's
// token rows, fin_n/2 contiguous bytes.  (Counting the GEMV's workgroups so that its last one does this
// work was measured: the agent-scope release every workgroup then needs costs far more than this launch.)
__global__ __launch_bounds__(256) void sample_finish_kernel(SampleFinish f) {
  const int tid = threadIdx.x;
  const unsigned long long b = *f.best;
  const int32_t tok = (int32_t)(0xffffffffu - (uint32_t)(b & 0xffffffffull));
  if (f.hidden) {
    const int g = (tok / AWQ_GROUP_SIZE) % (f.n / AWQ_GROUP_SIZE);
    const half_t es = f.emb_scale[g], ez = f.emb_zp[g];
    const uint8_t* row = f.emb_rows + (int64_t)tok * (f.n >> 1);
    for (int i = tid; i < f.n / 8; i += 256) {  // 8 hidden elements = one dword of the row
      const uint32_t w = *reinterpret_cast<const uint32_t*>(row + 4 * i);
      const u32x4 keep = *reinterpret_cast<const u32x4*>(f.hidden + 8 * i);
      union {
        u32x4 v;
        half_t h[8];
      } o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const half_t d = (half_t)(float)((w >> (4 * e)) & 15u) - ez;
        o.h[e] = d * es;
      }
      *reinterpret_cast<u32x4*>(f.hidden_last + 8 * i) = keep;
      *reinterpret_cast<u32x4*>(f.hidden + 8 * i) = o.v;
    }
  }
  if (tid == 0) {
    *f.out_token = tok;
    if (f.out_array && f.dyn) f.out_array[f.dyn->out_index] = tok;
    if (f.state) {
      StepState s = *f.state;
      s.pos += 1;
      s.len_lo = s.pos;  // layers below the split still see the previous length (Inference.cu:1118, 1364)
      s.len_hi = s.pos + 1;
      s.token = -1;
      s.out_index += 1;
      s.epoch += f.epoch_step;
      *f.state = s;
    }
    *f.best = 0ull;
  }
}
// (row / 128 % (k / 128)) % (m / 128), the group of a row (Inference.cu:90 with the index wrapped to the m / 128
// stored entries), without a division where there is nothing to divide: row / 128 < m / 128, so with
// k / 128 >= m / 128 both remainders change nothing, and otherwise the second one does not.  (The divisions stood
// between the requests for x and the first request for weights.)  A row group past the matrix gets a valid index.
__device__ __forceinline__ unsigned group_index(int row_over_128, int kg, int mg) {
  const unsigned g = min((unsigned)row_over_128, (unsigned)mg - 1u);
  if (kg >= mg) return g;
  return (kg & (kg - 1)) == 0 ? g & (unsigned)(kg - 1) : g % (unsigned)kg;
}


// A workgroup takes row groups blockIdx.x, blockIdx.x + gridDim.x, ... (16
// output rows x all of k each).  n_waves wavefronts; lane (w, q, r) owns blocks
// (4w+q)*G .. +G-1 of row 16*rg + r.  x is staged (normalised, with the input
// sum of every block beside it) once per workgroup; the weights of the next row
// group are in flight while the current one is multiplied.
// The arguments a wavefront needs early (pointers, the norm's and the scale
// group's scalars, the epilogue selector) come first and one by one: the first
// 16 dwords of the argument block are preloaded into scalar registers at
// wavefront launch (see the build flags); the rest of the argument block is a
// memory round trip away.
// k = n_waves * 64/RH * 32 * G, so a thread stages G * (64/RH) / 16 units of eight inputs
// (with G * 64/RH = 8 every second thread stages one).
// UFAST (periodic matrices only): the class length k/32/C when it is known at
// compile time and divides G, so that a lane's G blocks are G/UFAST whole classes
// whose constants it reads once per row group; 0 = look the class up per block.
//
// Dynamic LDS: x in block order, 2 bytes per input, as byte planes for the matrix cores (64 bytes per block)
// or as nibble planes for the dot products (skewed 16 bytes per lane group) | the
// blocks' powers of two, k/32 floats | the blocks' integer sums, k/32 floats | periodic matrices: group
// constants per (pass, class) | several row groups per workgroup: the finished sums, RH floats per pass |
// with the fused norm, x in natural order (k halves).
// NWC: the number of wavefronts when it is known at compile time (the model's
// own shapes: k, the staging loops and the reduction are then constants), 0 = take
// it from the launch.  MULTI: the grid is smaller than the number of row groups
// and a workgroup walks several of them.
// RH: output rows per workgroup, 16 or 8.  With 8 a wavefront's lanes are (eighth q = lane/8, r = lane%8): a
// workgroup takes half a 16-row group (its wavefront loads are eight 128-byte pieces) and covers the same
// number of blocks per wavefront with half the blocks per lane, so a matrix with few rows and long k
// (4096 x 12288: 256 row groups, 12 wavefronts each) runs as twice the workgroups -- two per compute unit.
// PRO, EPI: the prologue and the epilogue when they are known at compile time (the model's own launches), -1 =
// taken from the arguments.
template <int G, bool PERIODIC, int UFAST = 0, int NWC = 0, bool MULTI = true, int RH = 16, int PRO = -1, int EPI = -1>
__global__ __launch_bounds__(NWC ? NWC * 64 : 1024) void gemv_kernel(
    const u32x4* __restrict__ wq, const half_t* __restrict__ x, const half_t* __restrict__ gamma,
    const half_t* __restrict__ scale, const half_t* __restrict__ zp, int32_t mg, int32_t kg, float eps,
    int32_t pro_epi, GemvParams p) {
  // (14 dwords up to here: what is preloaded.  The norm's epsilon among them: read from the argument block it was
  // a memory round trip between the norm's statistic and its reciprocal square root.)
  const int prologue = PRO >= 0 ? PRO : (pro_epi & 0xff);
  const int epi = EPI >= 0 ? EPI : (pro_epi >> 8);
  const int m = mg * 128;
  const int n_waves = NWC ? NWC : p.n_waves;
  constexpr int Q = 64 / RH;  // lanes that share a row = consecutive block ranges of a wavefront
  // The block products on the matrix cores.  16 rows per wavefront: the lanes (q, r) are the matrix
  // instruction's (k-group, column) as they stand.  Not with eight blocks per lane (the input operands of a
  // lane's blocks stay in registers, 8 per block: that spills), nor for half row groups (a k-group then holds
  // two lanes' blocks; with rows for both and the sum of q from a second product or from dot products it
  // measured 6.6 against 6.4 us at 4096 x 12288).
  constexpr bool MM = RH == 16 && G <= 4;
  static_assert(RH == 16 || (RH == 8 && !PERIODIC), "half row groups are for one scale group per 16 rows");
  const int k = NWC ? NWC * Q * 32 * G : p.k;
  const int nblk = NWC ? NWC * Q * G : p.nblk;
  const int C = PERIODIC ? p.C : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* xs = smem;                                                      // 2k bytes of nibble planes + skew
  float* xc = reinterpret_cast<float*>(smem + (size_t)(k + (nblk / G) * 8) * 2);  // nblk powers of two
  float* xS = xc + nblk;                                                         // nblk integer sums
  // PERIODIC: the group constants of every (pass, class) of this workgroup, filled once
  GroupConst* gt = reinterpret_cast<GroupConst*>(xS + nblk);
  const int n_pass = MULTI ? (m / RH + (int)gridDim.x - 1) / (int)gridDim.x : 1;  // passes of the longest-running workgroup
  float* ysum = reinterpret_cast<float*>(gt + (PERIODIC ? (n_pass * C + 1 & ~1) : 0));  // MULTI: a pass's finished sums, RH per pass
  half_t* xn = reinterpret_cast<half_t*>(ysum + (MULTI ? n_pass * RH : 0));      // k halves (fused norm only)
  __shared__ float red[2][16][16];  // double-buffered: one barrier per row group
  __shared__ __attribute__((aligned(16))) float part[256];
  // A thread stages units of 8 consecutive block-order inputs (the inputs of one weight dword): k/8 units over
  // n_waves * 64 = k/(G*Q/2) threads, i.e. G*Q/16 units per thread, or one unit in every second thread
  constexpr int MAXU = G * Q >= 16 ? G * Q / 16 : 1;
  static_assert(G * Q >= 8, "a thread stages whole units");
  const int tid = threadIdx.x;
  const int nthreads = n_waves * 64;
  const bool stager = G * Q >= 16 || tid < nthreads / 2;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane / RH, r = lane % RH;
  const int n_rg = m / RH;
  const int blk0 = (Q * wave + q) * G;
  const int U = nblk / C;  // blocks per class (PERIODIC)

  int rg = blockIdx.x;
  // row group of 16 in the weight stream and the row inside it
  const u32x4* wp = wq + ((int64_t)(rg * RH >> 4) * nblk + blk0) * 16 + ((rg * RH) & 15) + r;
  u32x4 w[G], wn[G];

  // ---- x: unit u of a thread is the 8 consecutive block-order elements 8*(tid + u*nthreads)..+7; in natural
  // order they are 8 consecutive indices too unless the matrix is periodic (then they are C apart and are
  // gathered one by one)
  const bool norm = prologue == PRO_RMSNORM;
  uint4 xu[MAXU], gu[MAXU];
#pragma unroll
  for (int u = 0; u < MAXU; ++u) {
    const int unit = tid + u * nthreads;
    if (!stager) {
      xu[u] = gu[u] = uint4{0, 0, 0, 0};
    } else if (PERIODIC) {
      half_t hx[8], hg[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = (int)awq_block_elem(k, C, unit >> 2, (8 * unit + i) & 31);
        hx[i] = x[j];
        hg[i] = norm ? gamma[j] : (half_t)0.0f;
      }
      xu[u] = *reinterpret_cast<uint4*>(hx);
      gu[u] = *reinterpret_cast<uint4*>(hg);
    } else {
      xu[u] = reinterpret_cast<const uint4*>(x)[unit];
      if (norm) gu[u] = reinterpret_cast<const uint4*>(gamma)[unit];
    }
  }
  // scale and zero-point of the first row group (row/128, then Inference.cu:90 with the index wrapped to
  // the m/128 stored entries): requested with x, so that they are there when the first block is done
  half_t gs = (half_t)0.0f, gz = (half_t)0.0f;
  if (!PERIODIC) {
    const unsigned gi = group_index(rg * RH >> 7, kg, mg);
    gs = scale[gi];
    gz = zp[gi];
  }
  // Every request for x of this workgroup goes out before any of its requests
  // for weights: the memory pipeline of a compute unit serves requests in order,
  // and a small load of x that queues behind kilobytes of weight loads arrives
  // microseconds late (measured: 7.9 -> 7.45 us per launch at 12288 x 4096).
  __syncthreads();
  // With the fused norm (the model's own launches: three workgroups per compute unit) only the first block of a
  // lane is requested here and the others behind the barrier that ends the staging of x.  A wavefront passes a
  // barrier only once the memory pipeline has accepted all its requests, and a compute unit accepts about 37 KB
  // before it makes the next wavefront wait: with all 96 KB of its three workgroups asked for up front, the norm
  // of the second and third workgroup stood at its barriers until most of the stream was through.  12288 x 4096,
  // launches of this shape back to back: 6.67 us with all four blocks here, 6.37 with three of them behind the
  // norm's second barrier, 6.20 behind the staging barrier (921 / 935 / 938 tok/s); two blocks here and two
  // behind the staging barrier 7.0 us, nothing here 6.95 us (the stream then starts late).
  constexpr int kEarly = (PRO == PRO_RMSNORM && NWC > 0 && !MULTI && G > 1) ? 1 : G;
#pragma unroll
  for (int b = 0; b < kEarly; ++b) w[b] = __builtin_nontemporal_load(wp + b * 16);
  if (norm) {
    // rmsNormKernel, Inference.cu:111-145: 256 strided fma partial sums over the
    // natural order, the stride-halving tree, then two binary16 multiplies
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      const int unit = tid + u * nthreads;
      if (!stager) continue;
      if (PERIODIC) {
        half_t hx[8];
        *reinterpret_cast<uint4*>(hx) = xu[u];
#pragma unroll
        for (int i = 0; i < 8; ++i) xn[awq_block_elem(k, C, unit >> 2, (8 * unit + i) & 31)] = hx[i];
      } else {
        reinterpret_cast<uint4*>(xn)[unit] = xu[u];
      }
    }
    __syncthreads();
    for (int pi = tid; pi < 256; pi += nthreads) {
      // 16 reads in flight per round: an LDS round trip per term would serialise the chain
      float acc = 0.0f;
      for (int i0 = pi; i0 < k; i0 += 16 * 256) {
        half_t hv[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) hv[j] = i0 + 256 * j < k ? xn[i0 + 256 * j] : (half_t)0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j)
          if (i0 + 256 * j < k) {
            const float v = (float)hv[j];
            acc = __builtin_fmaf(v, v, acc);
          }
      }
      part[pi] = acc;
    }
    __syncthreads();
    // the tree of Inference.cu:130-135, by every wavefront for itself: lane t of a
    // row of 16 takes part[t + 16 j]; strides 128..16 are then additions in its own
    // registers and strides 8..1 exchanges within the row (a + b == b + a, so
    // the butterfly leaves in lane 0 what the one-sided tree leaves in part[0])
    float pv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) pv[j] = part[(lane & 15) + 16 * j];
#pragma unroll
    for (int n = 8; n >= 1; n >>= 1) {
#pragma unroll
      for (int j = 0; j < n; ++j) pv[j] += pv[j + n];
    }
    float tot = pv[0];
    tot += dpp_f<kDppRor8>(tot);
    tot += dpp_f<kDppRor4>(tot);
    tot += dpp_f<kDppXor2>(tot);
    tot += dpp_f<kDppXor1>(tot);
    tot = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, tot)));
    const half_t sc = rsqrt_half(tot / (float)k + eps);
    const half2_t sc2 = half2_t{sc, sc};
#pragma unroll
    for (int u = 0; u < MAXU; ++u) {
      uint32_t* d = reinterpret_cast<uint32_t*>(&xu[u]);
      const uint32_t* g = reinterpret_cast<const uint32_t*>(&gu[u]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        half2_t t = as_half2(d[i]) * sc2;
        t = t * as_half2(g[i]);
        d[i] = __builtin_bit_cast(uint32_t, t);
      }
    }
  }
  // x in block fixed point: nibble planes, the power of two and the integer sum of every block
  // (four threads share a block)
#pragma unroll
  for (int u = 0; u < MAXU; ++u) {
    const int unit = tid + u * nthreads;
    if (!stager) continue;
    const uint32_t h[4] = {xu[u].x, xu[u].y, xu[u].z, xu[u].w};
    float c, S;
    if (MM) {
      uint32_t lo0, lo1, hi0, hi1;
      stage_unit8_bytes(h, lo0, lo1, hi0, hi1, c, S);
      uint32_t* blk = reinterpret_cast<uint32_t*>(xs + (size_t)(unit >> 2) * 64) + (unit & 3);
      blk[0] = lo0, blk[4] = lo1, blk[8] = hi0, blk[12] = hi1;
    } else {
      u32x4 planes;
      stage_unit8(h, planes, c, S);
      *reinterpret_cast<u32x4*>(xs + (size_t)(unit + (unit / (4 * G))) * 16) = planes;
    }
    if ((tid & 3) == 0) {
      xc[unit >> 2] = c;
      xS[unit >> 2] = S;
    }
  }

  // Group constants.  When the scale group depends on the input index it is constant within a class of
  // blocks; the (at most 64) classes of every row group this workgroup will walk go into a table in LDS
  // here, so that the loop issues no loads but the weights'.  (A value requested and used inside the loop
  // makes its wavefront wait for every load issued before it, the weights just requested for the next pass
  // among them, and the whole workgroup with it at the pass's barrier.)
  if (PERIODIC) {
    for (int e = tid; e < n_pass * C; e += nthreads) {
      const int pass = e / C, cls = e - pass * C;
      const int row_group = blockIdx.x + pass * (int)gridDim.x;
      if (row_group < n_rg) {
        // 32-bit arithmetic: class * m/128 stays far below 2^31
        const unsigned gi = (((unsigned)cls * (unsigned)mg + (unsigned)(row_group >> 3)) % (unsigned)kg) % (unsigned)mg;
        gt[e] = make_group(scale[gi], zp[gi]);
      }
    }
  }
  __syncthreads();  // the planes, the blocks' constants and the table
#pragma unroll
  for (int b = kEarly; b < G; ++b) w[b] = __builtin_nontemporal_load(wp + b * 16);
  float xcb[G], xSb[G];
  if (G >= 4) {
#pragma unroll
    for (int b = 0; b < G; b += 4) {
      const float4 t = *reinterpret_cast<const float4*>(xc + blk0 + b);
      const float4 v = *reinterpret_cast<const float4*>(xS + blk0 + b);
      xcb[b] = t.x, xcb[b + 1] = t.y, xcb[b + 2] = t.z, xcb[b + 3] = t.w;
      xSb[b] = v.x, xSb[b + 1] = v.y, xSb[b + 2] = v.z, xSb[b + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int b = 0; b < G; ++b) xcb[b] = xc[blk0 + b], xSb[b] = xS[blk0 + b];
  }
  // the G blocks of this lane in LDS: 64 bytes each, the lane group's skew included
  const unsigned char* xl = xs + (size_t)(blk0 * 4 + blk0 / G) * 16;
  // on the matrix cores: this lane's share of the input operand of its wavefront's G block columns, kept in
  // registers for all row groups of the workgroup
  u32x4 a_lo[MM ? G : 1], a_hi[MM ? G : 1];
  if (MM) {
#pragma unroll
    for (int b = 0; b < G; ++b) load_planes(xs + (size_t)(blk0 + b) * 64, lane, a_lo[b], a_hi[b]);
  }
  auto dot = [&](const u32x4& wv, int b) -> float {
    if (MM) return block_dot_mfma(wv, a_lo[b], a_hi[b]);
    return block_dot(wv, xl + 64 * b);
  };
  unsigned long long best_here = 0;  // EPI_ARGMAX: best candidate among this lane's rows

  // the weights of one row group, and (one scale group per 16 rows) its scale and zero-point
  auto request = [&](u32x4(&dst)[G], half_t& s_out, half_t& z_out, int row_group) {
    const u32x4* src = wq + ((int64_t)(row_group * RH >> 4) * nblk + blk0) * 16 + ((row_group * RH) & 15) + r;
#pragma unroll
    for (int b = 0; b < G; ++b) dst[b] = __builtin_nontemporal_load(src + b * 16);
    if (!PERIODIC) {
      const unsigned gi = group_index(row_group * RH >> 7, kg, mg);
      s_out = scale[gi];
      z_out = zp[gi];
    }
  };

  // One pass: row group row_group from the weights in wc.  With MULTI the finished sums stay in LDS until
  // the workgroup has walked all its row groups: a store inside the loop would share the counter of
  // outstanding memory operations with the loads requested for the next pass, and since loads and stores
  // complete in no fixed order relative to each other every wait for weights would have to wait for
  // everything outstanding -- the next pass's weights included (151936 x 4096: 59 -> 5x us).
  auto pass = [&](const u32x4(&wc)[G], half_t s_cur, half_t z_cur, int row_group, int it) {
    // the residual row is requested before the pass multiplies: the end of the
    // launch then does not wait for one more round trip to memory
    half_t res = (half_t)0.0f;
    if (!MULTI && tid < RH && epi == EPI_RESIDUAL) res = p.res[row_group * RH + r];
    GroupConst g = make_group(s_cur, z_cur);
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
      for (int c = 0; c < NC; ++c) gc[c] = gt[it * C + blk0 / UFAST + c];
#pragma unroll
      for (int b = 0; b < G; ++b) {
        const GroupConst& gb = gc[UFAST > 0 ? b / UFAST : 0];
        bs[b] = __builtin_fmaf(gb.zn, xSb[b], dot(wc[b], b)) * (gb.s * xcb[b]);
      }
    } else {
#pragma unroll
      for (int b = 0; b < G; ++b) {
        if (PERIODIC) {
          g = gt[it * C + cls];
          if (--cls_left == 0) {
            ++cls;
            cls_left = U;
          }
        }
        bs[b] = __builtin_fmaf(g.zn, xSb[b], dot(wc[b], b)) * (g.s * xcb[b]);
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
    if (RH == 8) v += dpp_f<kDppRor8>(v);  // lane i + lane i ^ 8
    v = sum_rows_of_16(v);
    // The only barrier of the pass.  The 16 finishing lanes read this pass's
    // buffer while the other wavefronts already multiply the next row group; the
    // buffer is written again two passes on, after a barrier those lanes are part of.
    float(*rd)[16] = red[it & 1];
    if (q == 0) rd[wave][r] = v;
    __syncthreads();
    if (tid < RH) {
      // awq_tree_sum over the wavefronts' sums, in registers (all reads in flight at once)
      float t[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) t[i] = i < n_waves ? rd[i][r] : 0.0f;
      int n = n_waves;
#pragma unroll
      for (int lvl = 0; lvl < 4; ++lvl)
        if (n > 1 && (n & 1) == 0) {
          n >>= 1;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (i < n) t[i] = t[2 * i] + t[2 * i + 1];
        }
      float tot = t[0];
#pragma unroll
      for (int i = 1; i < 16; ++i)
        if (i < n) tot += t[i];
      if (MULTI) ysum[it * RH + r] = tot;
      else epilogue(p, epi, row_group * RH + r, r, tot, res, best_here);
    }
  };

  if (!MULTI) {
    pass(w, gs, gz, rg, 0);
  } else if (rg < n_rg) {
    // Two register sets take turns, so that no pass copies weights, and the last pass is written out
    // on its own, so that every request inside the loop is unconditional: the compiler then knows how
    // many younger loads are outstanding when it waits for a pass's weights and lets them stay in flight.
    // (Requesting two passes ahead with three register sets measured the same, 151936 x 4096 in 57 us
    // either way: a compute unit keeps about 37 KB of requests in flight whatever its wavefronts have
    // asked for, which at the memory's latency under load is about 6 TB/s for the device.)
    const int step = (int)gridDim.x;
    half_t gsn = (half_t)0.0f, gzn = (half_t)0.0f;
    int it = 0;
    while (true) {
      if (rg + step >= n_rg) {
        pass(w, gs, gz, rg, it);
        break;
      }
      request(wn, gsn, gzn, rg + step);
      pass(w, gs, gz, rg, it);
      rg += step, ++it;
      if (rg + step >= n_rg) {
        pass(wn, gsn, gzn, rg, it);
        break;
      }
      request(w, gs, gz, rg + step);
      pass(wn, gsn, gzn, rg, it);
      rg += step, ++it;
    }
    // the epilogues of all passes: each finishing lane reads back what it wrote
    if (tid < RH) {
      int row_group = blockIdx.x;
      for (int i = 0; row_group < n_rg; row_group += step, ++i) {
        const half_t res = epi == EPI_RESIDUAL ? p.res[row_group * RH + r] : (half_t)0.0f;
        epilogue(p, epi, row_group * RH + r, r, ysum[i * RH + r], res, best_here);
      }
    }
  }
  if (epi == EPI_ARGMAX && tid < RH) {
    // one 64-bit atomic max per workgroup at most: a workgroup that finds a better candidate already
    // there skips it (additions to one address are served one after the other)
#pragma unroll
    for (int mask = 1; mask < RH; mask <<= 1) {
      const unsigned long long o = __shfl_xor(best_here, mask, 64);
      best_here = o > best_here ? o : best_here;
    }
    if (r == 0 && best_here > __hip_atomic_load(p.best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      __hip_atomic_fetch_max(p.best, best_here, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

struct GemvPlan {
  int g;        // blocks per lane: 1, 2, 4 or 8
  int n_waves;  // wavefronts per workgroup
  int rh;       // output rows per workgroup: 16, or 8 (half a row group)
};

// Lane groups per workgroup = (k/32)/G must be a multiple of 4 and at most 64.
// The longest per-lane run (G = 8, 4, 2) that still gives a workgroup eight wavefronts: with k = 4096
// eight wavefronts of four blocks per lane beat four wavefronts of eight (12288 x 4096: 6.85 against
// 7.15 us).  G >= 2: the staging works in units of eight inputs.
bool plan_gemv(int64_t m, int64_t k, GemvPlan* out) {
  const int64_t nblk = k / AWQ_BLOCK_K;
  bool found = false;
  for (int g = 8; g >= 2; g >>= 1) {
    if (nblk % g) continue;
    int64_t groups = nblk / g;
    if (groups % 4 || groups > 64) continue;
    *out = GemvPlan{g, (int)(groups / 4), 16};
    found = true;
    if (groups / 4 >= 8) break;
  }
  // few rows and long k (4096 x 12288: one 16-row workgroup of 12 wavefronts per compute unit): half the rows
  // and half the blocks per lane, twice the workgroups (8.2 -> 7.55 us with the first arithmetic; 4096 x 4096
  // the same way measured no different, 3.94 against 3.95 us, so only where a lane has eight blocks)
  if (found && m / 16 <= 256 && out->g == 8 && out->n_waves >= 8) {
    out->g = 4;
    out->rh = 8;
  }
  return found;
}

#define GEMV_HOT_ARGS p.wq, p.x, p.gamma, p.scale, p.zp, p.mg, p.kg, p.eps, (p.prologue | (p.epilogue << 8))
template <int G>
void launch_g(const GemvParams& p, bool periodic, bool multi, int rh, dim3 grid, dim3 block, size_t lds, hipStream_t st) {
  if (rh == 8) {  // plan_gemv: four blocks per lane, not periodic, one row group per workgroup
    if (p.n_waves == 12 && p.prologue == PRO_NONE && p.epilogue == EPI_RESIDUAL)
      hipLaunchKernelGGL((gemv_kernel<4, false, 0, 12, false, 8, PRO_NONE, EPI_RESIDUAL>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else if (p.n_waves == 12) hipLaunchKernelGGL((gemv_kernel<4, false, 0, 12, false, 8>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else hipLaunchKernelGGL((gemv_kernel<4, false, 0, 0, true, 8>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    return;
  }
  if (G == 4 && periodic && p.nblk / p.C == 4 && p.n_waves == 8) {  // the unembedding: one class of 4 blocks per lane
    hipLaunchKernelGGL((gemv_kernel<G, true, G == 4 ? 4 : 0, 8, true>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    return;
  }
  if (G == 8 && periodic && p.nblk / p.C == 4) {  // classes of 4 blocks, long k
    hipLaunchKernelGGL((gemv_kernel<G, true, G == 8 ? 4 : 0>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    return;
  }
  if (periodic) {
    hipLaunchKernelGGL((gemv_kernel<G, true>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    return;
  }
  // the per-layer matrices of the model: 4096 inputs as 4 wavefronts x 8 blocks or 8 x 4, 12288 as 12 x 8
  if (!multi && G == 8 && p.n_waves == 12) hipLaunchKernelGGL((gemv_kernel<G, false, 0, 12, false>), grid, block, lds, st, GEMV_HOT_ARGS, p);
  else if (!multi && G == 4 && p.n_waves == 8) {
    // the model's own launches with 4096 inputs: prologue and epilogue are compile-time constants too
    if (p.prologue == PRO_RMSNORM && p.epilogue == EPI_QKV_ROPE)
      hipLaunchKernelGGL((gemv_kernel<G, false, 0, 8, false, 16, PRO_RMSNORM, EPI_QKV_ROPE>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else if (p.prologue == PRO_RMSNORM && p.epilogue == EPI_GELU)
      hipLaunchKernelGGL((gemv_kernel<G, false, 0, 8, false, 16, PRO_RMSNORM, EPI_GELU>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else if (p.prologue == PRO_NONE && p.epilogue == EPI_RESIDUAL)
      hipLaunchKernelGGL((gemv_kernel<G, false, 0, 8, false, 16, PRO_NONE, EPI_RESIDUAL>), grid, block, lds, st, GEMV_HOT_ARGS, p);
    else
      hipLaunchKernelGGL((gemv_kernel<G, false, 0, 8, false>), grid, block, lds, st, GEMV_HOT_ARGS, p);
  } else hipLaunchKernelGGL((gemv_kernel<G, false>), grid, block, lds, st, GEMV_HOT_ARGS, p);
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
  AWQ_REQUIRE(m < (1ll << 31) && k <= 16384, "shape too large (k is limited to 16384: 64 lane groups of 8 blocks per workgroup)");
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
  if (periodic && plan.rh == 8) {  // half row groups only with one scale group per 16 rows
    plan.g *= 2;
    plan.rh = 16;
  }
  // one workgroup per row group while that fits the device a few times over;
  // beyond that a workgroup walks several row groups and stages x once
  int64_t n_rg = a.m / plan.rh, n_wg = n_rg;
  // Four wavefronts per SIMD (measured: 151936 x 4096 with argmax as 512 workgroups of 8 wavefronts 60 us, as
  // 1024 of 4 wavefronts 64 us, 576 of 8: 80 us), and at most 32 passes: the table of group constants is per pass.
  if (n_rg > 1024) n_wg = std::max<int64_t>(4096 / plan.n_waves, (n_rg + 31) / 32);
  dim3 grid((unsigned)n_wg), block((unsigned)(plan.n_waves * 64));
  // x as nibble planes plus 16 bytes of skew per lane group, two floats per block, the table of group
  // constants of a periodic matrix (passes x classes), and with the fused norm x in natural order
  const int64_t n_pass = (n_rg + n_wg - 1) / n_wg;
  size_t lds = (size_t)a.k * 2 + (size_t)(a.k / AWQ_BLOCK_K / plan.g) * 16 + (size_t)(a.k / AWQ_BLOCK_K) * 8 +
               (periodic ? (size_t)(n_pass * p.C + 1 & ~1) * sizeof(GroupConst) : 0) + (size_t)n_pass * plan.rh * 4 +
               (a.prologue == PRO_RMSNORM ? (size_t)a.k * 2 : 0);
  // the kernel's static arrays (the wavefronts' sums, double-buffered, and the norm's partial sums) come on top
  constexpr size_t kStaticLds = 2 * 16 * 16 * sizeof(float) + 256 * sizeof(float);
  AWQ_REQUIRE(lds + kStaticLds <= 65536, "k too large for the fused norm (x is kept twice in LDS)");
  switch (plan.g) {
    case 2: launch_g<2>(p, periodic, n_wg < n_rg, plan.rh, grid, block, lds, st); break;
    case 4: launch_g<4>(p, periodic, n_wg < n_rg, plan.rh, grid, block, lds, st); break;
    default: launch_g<8>(p, periodic, n_wg < n_rg, plan.rh, grid, block, lds, st); break;
  }
  AWQ_HIP_TRY(hipGetLastError());
  if (a.epilogue == EPI_ARGMAX) {
    SampleFinish f{a.best,      a.out_token, a.out_array,     a.dyn,        a.fin_hidden, a.fin_hidden_last,
                   a.fin_emb,   a.fin_emb_scale, a.fin_emb_zp, a.fin_n,      a.fin_state, a.fin_epoch_step};
    hipLaunchKernelGGL(sample_finish_kernel, dim3(1), dim3(256), 0, st, f);
    AWQ_HIP_TRY(hipGetLastError());
  }
  return AWQ_OK;
}
