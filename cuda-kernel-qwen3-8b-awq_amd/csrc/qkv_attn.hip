// The first two launches of a decoder layer as ONE: RMSNorm + Wqkv + rotary + KV append (Inference.cu:1040-1103)
// and the attention over the cache (Inference.cu:1110, attentionKernel :182-267), for attended lengths that the
// attention covers in at most three launches of its own, and half as far again (kFusedQkvAttnMax = 3072).
//
// Of all the boundaries between a layer's launches this is the one across which the data dependence is local:
// the attention of head h needs rows 128 h .. 128 h + 127 of Q and of K and nothing else of the product.  A
// head is given to eight workgroups ON ONE DIE -- workgroups are handed to the eight dies in turn, so those
// whose indices agree modulo 8 share a die and its L2 -- and what they owe each other travels through that L2:
// nontemporal stores and loads go past the compute unit's own cache and meet in the L2, a quarter of a
// microsecond from store to load where a kernel boundary costs 1.6 us and the first loads behind it a memory
// round trip more.  One hand-over per launch:
//   every workgroup computes 16 of the head's 128 dimensions of Q, K and V (three 16-row groups of the product,
//   x normalised and staged once for all three), rotates its Q and K and appends K and V to the cache.  With its
//   16 dimensions of Q it forms, for every attended position, the sum over its 16 dimensions of the score's dot
//   product -- two chains of eight and their sum, which is exactly one node of the dot product's adjacent-pair
//   tree -- and publishes these partial scores as tagged words (the halves of the binary32 pattern next to a
//   16-bit tag: only a 4-byte word is seen whole by a load that races with the store -- an 8-byte (score, tag)
//   pair was observed with the new tag next to the old score).  All eight workgroups read all eight partial
//   scores of every position, finish the tree, and normalise for themselves (the same instructions on the same
//   data: the same bits); each forms the context of its own 16 dimensions, for which it needs only its own V.
//   (A first version handed Q and K round first and the finished scores of an eighth of the positions second:
//   two hand-overs, 0.5 and 0.75 us.)
// The keys and values a workgroup needs from the cache are its 16 dimensions of every attended position: 32
// bytes of every 256-byte row, for which the L2 hands over whole lines.  They are therefore kept a second time
// in the order of this launch, [head][workgroup of the head][position][16 dimensions] (the "parts" arrays, for
// positions below their capacity), where a chunk of 64 positions is 2 KB in a row: the launch appends to both
// forms and reads the second, requested right behind its weights.  The new position's key and value come from
// the workgroup's own product, not from the rows just written.
//
// Every wait is bounded and looks at the status word the other fused launch uses: a workgroup that gives up
// sets it and stores no context, the others follow, the launch ends, and the host finds the word after the
// step.  A tag that never arrives (a stale line in another die's L2, were workgroups ever placed otherwise)
// therefore ends in an error, never in a wrong token.
//
// Arithmetic: the product is gemv_kernel's (awq_canon_math.h: block fixed point, canonical tree -- the same
// tree for 16 wavefronts of two blocks per lane as for 8 of four), the attention is attention_kernel's (dot
// products as 16 lanes x 8 fma chains and an adjacent-pair tree, chunks of 64 positions, four interleaved
// chains per chunk and dimension, chunk results added in order), so the bits are those of the two launches.
#include "common.hpp"
#include "gemv_device.hpp"

namespace {

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kK = 4096;            // inputs of the product
constexpr int kBlocks = kK / 32;    // 128 blocks of 32 inputs
constexpr int kG = 2;               // blocks per lane and row group
constexpr int kParts = 8;           // workgroups per head
constexpr int kDP = AWQ_HEAD_DIM / kParts;  // dimensions per workgroup: one 16-row group each of Q, K and V
constexpr int kMaxLen = (int)kFusedQkvAttnMax;
constexpr int kMaxCPW = 4;          // chunks of 64 positions per wavefront: 1 up to 1024 attended positions, 2 up to 2048, 3 beyond
constexpr int kChunkCap = kMaxCPW * kWaves;
constexpr int kScoreStride = kChunkCap * 64;  // (score, tag) pairs per head in the exchange buffer
static_assert(kDP == 16 && kMaxLen <= kChunkCap * 64 && kMaxLen <= kScoreStride, "shape of the fused launch");
// Wavefront 0 finishes the product (rotary, stores): what queues behind bulk requests in the compute unit's
// memory pipeline waits for them, so chunk c of the cache goes to wavefront 1 + c % 16 for c % 16 < 15 and
// wavefront 0 streams one only beyond 960 attended positions.  (Handing the chunks out from the last wavefront
// down instead measured 981 against 987 tok/s.)
static_assert((kMaxLen + 63) / 64 <= kChunkCap, "kMaxCPW chunks of keys and values per wavefront");
static_assert(kChunkCap * 64 * sizeof(float) >= kK * sizeof(half_t), "the scores take the place of x in natural order");

struct QkvAttnArgs {
  const u32x4* wq;
  const half_t* scale;
  const half_t* zp;
  const half_t* x;        // [4096] hidden state
  const half_t* gamma;
  const half_t* cos_t;
  const half_t* sin_t;
  half_t* k_cache;
  half_t* v_cache;
  half_t* k_parts;        // [heads][8][parts_pos][16]: the same rows in the order this launch reads them
  half_t* v_parts;
  half_t* q_out;          // [4096] rotated Q, as the separate launch leaves it
  half_t* ctx;            // [4096] attention output
  uint32_t* score_tag;    // [heads][8 workgroups][kScoreStride][2] the halves of a partial score as (half | tag << 16)
  int32_t* status;        // [0] != 0: a wait gave up (or the host asks every wait to)
  const StepState* dyn;
  KvLayout kv;
  int32_t spin_limit;
  int32_t parts_pos;      // positions the parts arrays hold
  float eps;
  unsigned long long* stamps;  // STAMPS: [workgroup][kQkvStamps] times of thread 0, 10 ns units
};

typedef _Float16 half8v_t __attribute__((ext_vector_type(8)));

// 16 bytes past the compute unit's cache, complete on return (the wait also covers every load the wavefront
// issued before: they return in order)
__device__ __forceinline__ u32x4 load_l2_16(const void* p) {
  u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}

// eight 8-byte pieces `stride` bytes apart the same way
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void load_l2_8x8(const char* p, u32x2 (&v)[8]) {
  constexpr int kPiece = kScoreStride * 8;  // bytes between the workgroups' pieces of one position
  const char* p2 = p + 4 * kPiece;
  asm volatile(
      "global_load_dwordx2 %0, %8, off nt\n\tglobal_load_dwordx2 %1, %9, off nt\n\t"
      "global_load_dwordx2 %2, %10, off nt\n\tglobal_load_dwordx2 %3, %11, off nt\n\t"
      "global_load_dwordx2 %4, %12, off nt\n\tglobal_load_dwordx2 %5, %13, off nt\n\t"
      "global_load_dwordx2 %6, %14, off nt\n\tglobal_load_dwordx2 %7, %15, off nt\n\ts_waitcnt vmcnt(0)"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
      : "v"(p), "v"(p + kPiece), "v"(p + 2 * kPiece), "v"(p + 3 * kPiece), "v"(p2), "v"(p2 + kPiece), "v"(p2 + 2 * kPiece), "v"(p2 + 3 * kPiece)
      : "memory");
}

template <int CTRL>
__device__ __forceinline__ float add_dpp(float v) {
  return v + dpp_f<CTRL>(v);
}
constexpr int kDppMirror = 0x140;  // lane i <-> 15 - i within 16
// sum over the 16 lanes of a row, adjacent pairs first (attention_kernel's row16_tree_sum)
__device__ __forceinline__ float row16_sum(float v) {
  v = add_dpp<kDppXor1>(v);
  v = add_dpp<kDppXor2>(v);
  v = add_dpp<kDppHalfMirror>(v);
  v = add_dpp<kDppMirror>(v);
  return v;
}
__device__ __forceinline__ float add_swap16(float v) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
__device__ __forceinline__ float add_swap32(float v) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
__device__ __forceinline__ float wave_sum(float v) { return add_swap32(add_swap16(row16_sum(v))); }
__device__ __forceinline__ float wave_maxf(float v) {
  v = fmaxf(v, dpp_f<kDppXor1>(v));
  v = fmaxf(v, dpp_f<kDppXor2>(v));
  v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_f<kDppMirror>(v));
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  v = fmaxf(a, b);
  a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}

// the canonical tree over the 16 wavefronts' sums of one row
__device__ __forceinline__ float sum_16_waves(const float (*rd)[16], int r) {
  float t[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) t[i] = rd[i][r];
#pragma unroll
  for (int n = 8; n >= 1; n >>= 1) {
#pragma unroll
    for (int i = 0; i < n; ++i) t[i] = t[2 * i] + t[2 * i + 1];
  }
  return t[0];
}

// workgroup -> (head, part): the eight parts of a head are the workgroups idx = 8 g .. 8 g + 7 of one residue
// class w % 8 (one die); head = 8 g + class
__device__ __forceinline__ void head_of(int w, int& head, int& part) {
  const int cls = w & 7, idx = w >> 3;
  head = (idx >> 3) * 8 + cls;
  part = idx & 7;
}

__global__ __launch_bounds__(64) void die_probe_kernel(int32_t* die_of) {
  if (threadIdx.x == 0) die_of[blockIdx.x] = __builtin_amdgcn_s_getreg((20) | (0 << 6) | ((4 - 1) << 11)) & 15;  // XCC_ID
}

// rows [pos0, pos0 + n) of both caches into the parts arrays: a thread moves 16 bytes
__global__ __launch_bounds__(256) void kv_to_parts_kernel(const half_t* __restrict__ kc, const half_t* __restrict__ vc,
                                                          KvLayout lay, half_t* __restrict__ kp, half_t* __restrict__ vp,
                                                          int n_heads, int parts_pos, int pos0, int n) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // (head, position, piece of 8 dimensions)
  if (idx >= (int64_t)n_heads * n * 16) return;
  const int piece = (int)(idx & 15);
  const int pos = pos0 + (int)((idx >> 4) % n);
  const int head = (int)((idx >> 4) / n);
  const int64_t src = kv_row(lay, head, pos) + 8 * piece;
  const int64_t dst = (((int64_t)head * kParts + (piece >> 1)) * parts_pos + pos) * kDP + 8 * (piece & 1);
  *reinterpret_cast<uint4*>(kp + dst) = *reinterpret_cast<const uint4*>(kc + src);
  *reinterpret_cast<uint4*>(vp + dst) = *reinterpret_cast<const uint4*>(vc + src);
}

// kCPW: chunks per wavefront (the launcher's bound on the attended length is 1024 kCPW).  The pointers a workgroup
// needs first are arguments of their own ahead of the struct: the first 14 dwords of the arguments are in scalar
// registers when a wavefront starts (kernarg preload), the rest takes a memory round trip.
template <bool STAMPS, int kCPW>
__global__ __launch_bounds__(kThreads) void qkv_attn_kernel(const half_t* __restrict__ hot_x, const half_t* __restrict__ hot_gamma,
                                                            const StepState* __restrict__ hot_dyn,
                                                            const u32x4* __restrict__ hot_wq, const half_t* __restrict__ hot_scale,
                                                            const half_t* __restrict__ hot_zp, int hot_use_len_hi, int hot_layer, QkvAttnArgs a) {
  constexpr int kChunks = kCPW * kWaves;  // of this instance; the LDS arrays and the exchange buffer are laid out for kChunkCap
  __shared__ __attribute__((aligned(16))) unsigned char xs[kBlocks * 64];  // byte planes, 64 bytes per block
  __shared__ __attribute__((aligned(16))) float xc[kBlocks];
  __shared__ __attribute__((aligned(16))) float xS[kBlocks];
  __shared__ __attribute__((aligned(16))) float s[kChunkCap * 64];  // the scores; before them, x in natural order
  half_t* const xn = reinterpret_cast<half_t*>(s);
  __shared__ float red[3][16][16];
  __shared__ __attribute__((aligned(16))) float part_sum[256];
  __shared__ __attribute__((aligned(16))) half_t own[3 * kDP];  // this workgroup's 16 dimensions of the rotated Q, of the new key and of the new value
  __shared__ __attribute__((aligned(16))) half_t vt[kWaves][64 * kDP];  // a wavefront's chunk of values, [position][dimension]
  __shared__ float cs[kChunkCap];
  __shared__ float wmax[kWaves];
  float* const cv = reinterpret_cast<float*>(xs);  // [kChunkCap][kDP] chunk vectors, once the products have read the planes
  static_assert(sizeof(xs) >= kChunkCap * kDP * sizeof(float), "the chunk vectors take the place of the byte planes");
  __shared__ int lost;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int tq = q, dl = r;  // the attention's names: position within a group of four, lane of a row
  const int blk0 = (4 * wave + q) * kG;
  const bool stager = tid < kThreads / 2;  // 512 units of eight inputs
  int head, part;
  head_of((int)blockIdx.x, head, part);
  if (tid == 0) lost = 0;
  int n_stamp = 0;
  auto stamp = [&]() {
    if (STAMPS && tid == 0) a.stamps[(size_t)blockIdx.x * kQkvStamps + n_stamp++] = wall_clock64();
  };
  stamp();  // 0 start

  // ---- requests, in the order the compute unit's memory pipeline should serve them
  uint4 xu = uint4{0, 0, 0, 0}, gu = uint4{0, 0, 0, 0};
  if (stager) {
    xu = reinterpret_cast<const uint4*>(hot_x)[tid];
    gu = reinterpret_cast<const uint4*>(hot_gamma)[tid];
  }
  const int32_t pos = hot_dyn->pos;
  // (the launcher's bound is kMaxLen; the clamp keeps every index inside the arrays whatever the state says)
  const int32_t L = min(hot_use_len_hi ? hot_dyn->len_hi : hot_dyn->len_lo, kChunks * 64);
  const int32_t epoch = hot_dyn->epoch;
  // the three row groups of this workgroup: dimensions 16 part .. + 15 of the head's Q, K and V
  int rg[3];
  half_t gs[3], gz[3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    rg[i] = i * (kK / 16) + head * kParts + part;
    const unsigned gi = (unsigned)(rg[i] * 16 >> 7) % (unsigned)(kK / 128);  // (... % (m / 128) of Inference.cu:90 changes nothing: m / 128 = 96 > 31)
    gs[i] = hot_scale[gi];
    gz[i] = hot_zp[gi];
  }
  __syncthreads();  // every request for x is out before any request for weights
  u32x4 wr[3][kG];
  auto request_w = [&](int i) {
    const u32x4* wp = hot_wq + ((int64_t)rg[i] * kBlocks + blk0) * 16 + r;
#pragma unroll
    for (int b = 0; b < kG; ++b) wr[i][b] = __builtin_nontemporal_load(wp + b * 16);
  };
  // the first row group now (32 KB: what a compute unit accepts at once), the others behind the staging:
  // a wavefront passes a barrier only once the memory pipeline has accepted all its requests
  request_w(0);
  stamp();  // 1 first requests issued
  // 1 .. 65535: never the 0 of a cleared buffer.  Q and K words are all rewritten by every launch, so a word
  // holds the previous launch's tag until then; score words beyond the attended length are not, which is why
  // the buffer is cleared when a sequence starts (a sequence stays below 65535 launches of this kind)
  const uint32_t tag16 = 1u + (uint32_t)(epoch + hot_layer) % 65535u;

  // ---- rmsNormKernel, Inference.cu:111-145: x in natural order for the 256 strided partial sums
  if (stager) reinterpret_cast<uint4*>(xn)[tid] = xu;
  __syncthreads();
  if (tid < 256) {
    half_t hv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) hv[j] = xn[tid + 256 * j];
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float v = (float)hv[j];
      acc = __builtin_fmaf(v, v, acc);
    }
    part_sum[tid] = acc;
  }
  __syncthreads();
  {
    // the tree of Inference.cu:130-135, by every wavefront for itself (see gemv_kernel)
    float pv[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) pv[j] = part_sum[(lane & 15) + 16 * j];
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
    const half_t sc = rsqrt_half(tot / (float)kK + a.eps);
    const half2_t sc2 = half2_t{sc, sc};
    uint32_t* d = reinterpret_cast<uint32_t*>(&xu);
    const uint32_t* g = reinterpret_cast<const uint32_t*>(&gu);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t t = as_half2(d[i]) * sc2;
      t = t * as_half2(g[i]);
      d[i] = __builtin_bit_cast(uint32_t, t);
    }
  }
  // x in block fixed point: byte planes, the power of two and the integer sum of every block
  if (stager) {
    const uint32_t h[4] = {xu.x, xu.y, xu.z, xu.w};
    uint32_t lo0, lo1, hi0, hi1;
    float cc, S;
    stage_unit8_bytes(h, lo0, lo1, hi0, hi1, cc, S);
    uint32_t* blk = reinterpret_cast<uint32_t*>(xs + (size_t)(tid >> 2) * 64) + (tid & 3);
    blk[0] = lo0, blk[4] = lo1, blk[8] = hi0, blk[12] = hi1;
    if ((tid & 3) == 0) {
      xc[tid >> 2] = cc;
      xS[tid >> 2] = S;
    }
  }
  stamp();  // 2 x normalised and staged (this wavefront)
  __syncthreads();
  stamp();  // 3 ... by all wavefronts
  request_w(1);
  request_w(2);
  // ---- what the attention needs from the cache, requested right behind the weights so that it arrives right
  // behind them: one chunk of 64 positions per wavefront, this workgroup's 16 dimensions of every key and
  // value row as two 16-byte pieces (lane = (position % 32, piece))
  const int nchunks = (L + 63) >> 6;
  const int aw = wave == 0 ? kWaves - 1 : wave - 1;  // this wavefront's chunks are aw, aw + 16
  // (the values of a third chunk are requested once the keys' registers are free)
  constexpr int kVEarly = kCPW < 2 ? kCPW : 2;
  half8v_t kraw[kCPW][2], vraw[kCPW][2];
  const int64_t parts_base = ((int64_t)head * kParts + part) * a.parts_pos * kDP + 8 * (lane & 1);
#pragma unroll
  for (int i = 0; i < kCPW; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = ((aw + kWaves * i) << 6) + 32 * j + (lane >> 1);
      if (t < L) kraw[i][j] = *reinterpret_cast<const half8v_t*>(a.k_parts + parts_base + (int64_t)t * kDP);
    }
  // (the keys first: the partial scores wait for them alone)
#pragma unroll
  for (int i = 0; i < kVEarly; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = ((aw + kWaves * i) << 6) + 32 * j + (lane >> 1);
      if (t < L) vraw[i][j] = *reinterpret_cast<const half8v_t*>(a.v_parts + parts_base + (int64_t)t * kDP);
    }

  // a wait that gave up in an earlier launch: this one does not wait at all (asked for behind the bulk requests,
  // needed long after them)
  const int32_t gave_up_before = __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- the three products (Inference.cu:1052)
  {
    u32x4 a_lo[kG], a_hi[kG];
    float cb[kG], Sb[kG];
#pragma unroll
    for (int b = 0; b < kG; ++b) {
      load_planes(xs + (size_t)(blk0 + b) * 64, lane, a_lo[b], a_hi[b]);
      cb[b] = xc[blk0 + b];
      Sb[b] = xS[blk0 + b];
    }
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const GroupConst g = make_group(gs[i], gz[i]);
      float bs[kG];
#pragma unroll
      for (int b = 0; b < kG; ++b)
        bs[b] = __builtin_fmaf(g.zn, Sb[b], block_dot_mfma(wr[i][b], a_lo[b], a_hi[b])) * (g.s * cb[b]);
      const float v = sum_rows_of_16(bs[0] + bs[1]);
      if (q == 0) red[i][wave][r] = v;
    }
  }

  // the wavefront that finishes the product asks for its rotary constants now
  half_t rc = (half_t)0.0f, rs = (half_t)0.0f;
  if (tid < 2 * kDP) {
    const int d = kDP * part + r;
    rc = a.cos_t[(int64_t)pos * 64 + (d >> 1)];
    rs = a.sin_t[(int64_t)pos * 64 + (d >> 1)];
  }
  // the sums below add all kChunkCap entries unconditionally: zeros where there is no chunk (x + 0 is x for the
  // non-negative sums and for the chunk vectors, which are never -0: every chain starts at +0)
  if (tid >= nchunks && tid < kChunks) cs[tid] = 0.0f;
  stamp();  // 4 products multiplied (this wavefront: its weights have arrived)
  __syncthreads();
  stamp();  // 5 ... by all wavefronts
  if (tid < kChunks * kDP && (tid >> 4) >= nchunks) cv[tid] = 0.0f;  // (every wavefront is done with the planes)

  // ---- split, rotary, KV append (Inference.cu:1070-1103) and the first hand-over
  half_t fin_out = (half_t)0.0f;
  if (tid < 3 * kDP) {
    const int sec = tid >> 4;  // 0 Q, 1 K, 2 V
    const half_t v = (half_t)sum_16_waves(red[sec], r);
    const int d = kDP * part + r;
    const half_t other = __builtin_bit_cast(half_t, (unsigned short)__builtin_bit_cast(uint32_t, dpp_f<kDppXor1>(__builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(unsigned short, v)))));
    half_t out = v;
    if (sec < 2) {  // pairs (2i, 2i + 1) are rotated (Inference.cu:158-176)
      const half_t av = (r & 1) ? other : v, bv = (r & 1) ? v : other;
      if (r & 1) {
        half_t as = av * rs, bc = bv * rc;
        out = as + bc;
      } else {
        half_t ac = av * rc, bs = bv * rs;
        out = ac - bs;
      }
    }
    own[tid] = out;
    fin_out = out;
  }
  stamp();  // 6 this workgroup's Q, K, V rotated
  __syncthreads();
  stamp();  // 7 ... and in LDS for all wavefronts
  if (tid < 3 * kDP) {  // the stores, off the path of the scores
    const int sec = tid >> 4, d = kDP * part + r;
    const int64_t prow = (((int64_t)head * kParts + part) * a.parts_pos + pos) * kDP + r;
    if (sec == 0) {
      a.q_out[head * AWQ_HEAD_DIM + d] = fin_out;
    } else if (sec == 1) {
      a.k_cache[kv_row(a.kv, head, pos) + d] = fin_out;
      if (pos < a.parts_pos) a.k_parts[prow] = fin_out;
    } else {
      a.v_cache[kv_row(a.kv, head, pos) + d] = fin_out;
      if (pos < a.parts_pos) a.v_parts[prow] = fin_out;
    }
  }

  // ---- this workgroup's share of every score (Inference.cu:202-226): lane (position, piece) runs the chain of
  // eight dimensions of its piece, the two pieces of a position are added (the first level of the dot
  // product's adjacent-pair tree), and the sum is published
  if (aw < nchunks) {
    float qf[8];
    const half8v_t qv = *reinterpret_cast<const half8v_t*>(own + 8 * (lane & 1));
    const half8v_t knew = *reinterpret_cast<const half8v_t*>(own + kDP + 8 * (lane & 1));
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
#pragma unroll
    for (int i = 0; i < kCPW; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int t = ((aw + kWaves * i) << 6) + 32 * j + (lane >> 1);
        const half8v_t kv = t == pos ? knew : kraw[i][j];  // not from the row just written
        float pt = 0.0f;
        if (t < L) {
#pragma unroll
          for (int d = 0; d < 8; ++d) pt = __builtin_fmaf(qf[d], (float)kv[d], pt);
        }
        pt = add_dpp<kDppXor1>(pt);
        if (t < L && (lane & 1) == 0) {
          const uint32_t bits = __builtin_bit_cast(uint32_t, pt);
          uint32_t* dst = a.score_tag + (((size_t)head * kParts + part) * kScoreStride + t) * 2;
          __builtin_nontemporal_store((bits & 0xffffu) | (tag16 << 16), dst);
          __builtin_nontemporal_store((bits >> 16) | (tag16 << 16), dst + 1);
        }
      }
  }
  // this wavefront's first chunk of values into the order of the sums, [position][dimension], while the other
  // workgroups' partial scores are on their way; the new position's row comes from this workgroup's own product,
  // not from the row just written
  const half8v_t vnew = *reinterpret_cast<const half8v_t*>(own + 2 * kDP + 8 * (lane & 1));
  auto values_to_lds = [&](int i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = ((aw + kWaves * i) << 6) + 32 * j + (lane >> 1);
      if (t < L) *reinterpret_cast<half8v_t*>(&vt[wave][(32 * j + (lane >> 1)) * kDP + 8 * (lane & 1)]) = t == pos ? vnew : vraw[i][j];
    }
  };
#pragma unroll
  for (int i = kVEarly; i < kCPW; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int t = ((aw + kWaves * i) << 6) + 32 * j + (lane >> 1);
      if (t < L) vraw[i][j] = *reinterpret_cast<const half8v_t*>(a.v_parts + parts_base + (int64_t)t * kDP);
    }
  if (aw < nchunks) values_to_lds(0);
  stamp();  // 8 partial scores published (this wavefront)
  if ((wave << 6) < L) {
    // the eight partial scores of positions tid and tid + 1024: the rest of the tree (Inference.cu:218 scales the sum)
    const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);
    bool dead = gave_up_before != 0;
    float my_max = -1e9f;
#pragma unroll
    for (int i = 0; i < kCPW; ++i) {
      const int t = tid + kThreads * i;
      if ((wave << 6) + kThreads * i >= L) break;  // the same for the whole wavefront
      const bool mine = t < L;
      const char* src = reinterpret_cast<const char*>(a.score_tag + ((size_t)head * kParts * kScoreStride + t) * 2);
      int spins = 0;
      while (!dead) {
        int32_t st = 0;
        const bool look = (spins & 7) == 7;  // every eighth poll also reads the status word
        if (look) st = __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        u32x2 w[8];
        bool ok = true;
        if (mine) {
          load_l2_8x8(src, w);
#pragma unroll
          for (int j = 0; j < 8; ++j) ok = ok && (w[j].x >> 16) == tag16 && (w[j].y >> 16) == tag16;
        }
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
          if (mine) {
            float p8[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) p8[j] = __builtin_bit_cast(float, (w[j].x & 0xffffu) | (w[j].y << 16));
            const float tot = ((p8[0] + p8[1]) + (p8[2] + p8[3])) + ((p8[4] + p8[5]) + (p8[6] + p8[7]));
            const float sc = tot * scale;
            s[t] = sc;
            my_max = fmaxf(my_max, sc);
          }
          break;
        }
        if (++spins > a.spin_limit) {
          if (lane == 0) __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          dead = true;
        }
        if (look && st != 0) dead = true;
      }
    }
    if (dead && lane == 0) lost = 1;
    // maximum (Inference.cu:229-233; it does not depend on the order): this wavefront's positions
    my_max = wave_maxf(my_max);
    if (lane == 0) wmax[wave] = my_max;
  } else if (lane == 0) {
    wmax[wave] = -1e9f;
  }
  __syncthreads();
  stamp();  // 9 all scores of the head seen
  float mx = lane < kWaves ? wmax[lane] : -1e9f;  // (read together with the flag: one LDS round trip, not two)
  const int gave_up = lost;
  if (gave_up) return;
  // The partial scores (and the rows appended to the caches) sit dirty in this die's L2, and the launch cannot end
  // before they are written back.  One wavefront of a head's first workgroup starts that write-back now, when the
  // head's scores have all been written, instead of leaving all of it to the end of the kernel; it does not wait
  // for it.  1040 -> 1049 tok/s (one workgroup per die, or two per head: the same; every workgroup: 1019).
  if (wave == kWaves - 1 && part == 0) asm volatile("buffer_wbl2 sc1" ::: "memory");
  mx = wave_maxf(mx);

  // ---- exponentials and their sum (Inference.cu:239-249), a chunk at a time; the exponential of position
  // 64 chunk + lane stays in its register
  float e_lane[kCPW];
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const int c = aw + kWaves * i;
    e_lane[i] = 0.0f;
    if (c < nchunks) {
      const int t = (c << 6) + lane;
      if (t < L) e_lane[i] = awq_expf(s[t] - mx);
      const float e = wave_sum(e_lane[i]);
      if (lane == 0) cs[c] = e;
    }
  }
  // this lane's part of the first chunk's values back, ahead of the barrier: it does not depend on the normaliser
  auto values_of = [&](half_t (&vv)[16]) {
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) vv[nl] = vt[wave][(4 * nl + tq) * kDP + dl];
  };
  half_t vv0[16];
  if (aw < nchunks) values_of(vv0);
  __syncthreads();
  float Z;
  {
    float zc[kChunks];
#pragma unroll
    for (int c = 0; c < kChunks; ++c) zc[c] = cs[c];
    Z = zc[0];
#pragma unroll
    for (int c = 1; c < kChunks; ++c) Z += zc[c];
  }

  // ---- weighted sum of V (Inference.cu:251-265), a chunk at a time: lane (tq, dl) runs the chain of positions
  // 4 nl + tq for dimension dl
#pragma unroll
  for (int i = 0; i < kCPW; ++i) {
    const int c = aw + kWaves * i;
    if (c >= nchunks) break;  // the same for the whole wavefront
    const int base = c << 6;
    half_t vv[16];
    if (i == 0) {
#pragma unroll
      for (int nl = 0; nl < 16; ++nl) vv[nl] = vv0[nl];
    } else {
      values_to_lds(i);  // the wavefront's LDS accesses execute in order: the slot is free again
      values_of(vv);
    }
    const float p_lane = base + lane < L ? e_lane[i] / Z : 0.0f;
    float acc = 0.0f;
    float pp[16];
    // through the chunk's own slots of the scores (this wavefront alone reads them, and has): position 4 nl + tq at 16 tq + nl
    s[base + 16 * (lane & 3) + (lane >> 2)] = p_lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float4 v = *reinterpret_cast<const float4*>(&s[base + 16 * tq + 4 * j]);
      pp[4 * j] = v.x, pp[4 * j + 1] = v.y, pp[4 * j + 2] = v.z, pp[4 * j + 3] = v.w;
    }
#pragma unroll
    for (int nl = 0; nl < 16; ++nl) {
      const int t = base + 4 * nl + tq;
      const float rr = __builtin_fmaf(pp[nl], (float)vv[nl], acc);
      acc = t < L ? rr : acc;
    }
    acc = add_swap16(acc);
    acc = add_swap32(acc);
    if (tq == 0) cv[c * kDP + dl] = acc;
  }
  __syncthreads();
  if (tid < kDP) {
    float oc[kChunks];
#pragma unroll
    for (int c = 0; c < kChunks; ++c) oc[c] = cv[c * kDP + tid];
    float out = oc[0];
#pragma unroll
    for (int c = 1; c < kChunks; ++c) out += oc[c];
    store_through(a.ctx + head * AWQ_HEAD_DIM + kDP * part + tid, (half_t)out);
  }
  stamp();  // 10 end
}

}  // namespace

// hidden 4096 with 32 heads of 128, every workgroup resident at once, and workgroups whose indices agree
// modulo 8 on one die (checked with a probe launch of the same grid: 0 = not so, or not known)
int fused_qkv_attn_supported(int64_t hidden, int n_heads, hipStream_t st) {
  if (hidden != kK || n_heads != kK / AWQ_HEAD_DIM) return 0;
  int dev = 0, cus = 0, occ = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, qkv_attn_kernel<false, kMaxCPW>, kThreads, 0) != hipSuccess) return 0;
  const int n_wg = n_heads * kParts;
  if (occ < 1 || (int64_t)cus * occ < n_wg) return 0;
  int32_t* d = nullptr;
  if (hipMalloc((void**)&d, n_wg * sizeof(int32_t)) != hipSuccess) return 0;
  int32_t h[kK / AWQ_HEAD_DIM * kParts];
  bool ok = true;
  for (int round = 0; round < 2 && ok; ++round) {
    hipLaunchKernelGGL(die_probe_kernel, dim3((unsigned)n_wg), dim3(64), 0, st, d);
    ok = hipGetLastError() == hipSuccess && hipStreamSynchronize(st) == hipSuccess &&
         hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess;
    for (int w = 8; w < n_wg && ok; ++w) ok = h[w] == h[w & 7];
  }
  (void)hipFree(d);
  return ok ? 1 : 0;
}

int launch_fused_qkv_attn(const void* wq, const half_t* scale, const half_t* zp, int64_t m, const half_t* x,
                          const half_t* gamma, float eps, const half_t* cos_t, const half_t* sin_t, half_t* k_cache,
                          half_t* v_cache, KvLayout kv, half_t* k_parts, half_t* v_parts, int parts_pos, half_t* q_out,
                          half_t* ctx, uint32_t* score_tag, int32_t* status, const StepState* dyn, int layer,
                          int use_len_hi, int64_t len_bound, int n_heads, unsigned long long* stamps, hipStream_t st) {
  AWQ_REQUIRE(m == 3 * kK && n_heads == kK / AWQ_HEAD_DIM, "the fused launch is built for hidden 4096 and 32 heads");
  AWQ_REQUIRE(wq && x && gamma && cos_t && sin_t && k_cache && v_cache && k_parts && v_parts && q_out && ctx && score_tag &&
                  status && dyn,
              "NULL pointer");
  AWQ_REQUIRE(parts_pos > 0 && len_bound <= parts_pos, "the parts arrays do not hold the attended positions");
  QkvAttnArgs a;
  a.wq = (const u32x4*)wq;
  a.scale = scale;
  a.zp = zp;
  a.x = x;
  a.gamma = gamma;
  a.cos_t = cos_t;
  a.sin_t = sin_t;
  a.k_cache = k_cache;
  a.v_cache = v_cache;
  a.k_parts = k_parts;
  a.v_parts = v_parts;
  a.parts_pos = parts_pos;
  a.q_out = q_out;
  a.ctx = ctx;
  a.score_tag = score_tag;
  a.status = status;
  a.dyn = dyn;
  a.kv = kv;
  a.spin_limit = 1 << 20;
  a.eps = eps;
  a.stamps = stamps;
  AWQ_REQUIRE(len_bound > 0 && len_bound <= kMaxLen, "attended length beyond what the fused launch covers");
#define QKV_HOT_ARGS a.x, a.gamma, a.dyn, a.wq, a.scale, a.zp, use_len_hi, layer
  const dim3 grid((unsigned)(n_heads * kParts)), block(kThreads);
  if (len_bound <= 64 * kWaves) {
    if (stamps) hipLaunchKernelGGL((qkv_attn_kernel<true, 1>), grid, block, 0, st, QKV_HOT_ARGS, a);
    else hipLaunchKernelGGL((qkv_attn_kernel<false, 1>), grid, block, 0, st, QKV_HOT_ARGS, a);
  } else if (len_bound <= 2 * 64 * kWaves) {
    if (stamps) hipLaunchKernelGGL((qkv_attn_kernel<true, 2>), grid, block, 0, st, QKV_HOT_ARGS, a);
    else hipLaunchKernelGGL((qkv_attn_kernel<false, 2>), grid, block, 0, st, QKV_HOT_ARGS, a);
  } else if (len_bound <= 3 * 64 * kWaves) {
    if (stamps) hipLaunchKernelGGL((qkv_attn_kernel<true, 3>), grid, block, 0, st, QKV_HOT_ARGS, a);
    else hipLaunchKernelGGL((qkv_attn_kernel<false, 3>), grid, block, 0, st, QKV_HOT_ARGS, a);
  } else {
    if (stamps) hipLaunchKernelGGL((qkv_attn_kernel<true, 4>), grid, block, 0, st, QKV_HOT_ARGS, a);
    else hipLaunchKernelGGL((qkv_attn_kernel<false, 4>), grid, block, 0, st, QKV_HOT_ARGS, a);
  }
#undef QKV_HOT_ARGS
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int64_t fused_qkv_attn_exchange_bytes(int n_heads) {
  return (int64_t)n_heads * kScoreStride * kParts * 8;
}

int64_t fused_qkv_attn_parts_bytes(int n_heads, int64_t parts_pos) { return (int64_t)n_heads * AWQ_HEAD_DIM * parts_pos * 2; }

int launch_kv_to_parts(const half_t* k_cache, const half_t* v_cache, KvLayout kv, half_t* k_parts, half_t* v_parts,
                       int n_heads, int parts_pos, int64_t pos0, int64_t n, hipStream_t st) {
  AWQ_REQUIRE(k_cache && v_cache && k_parts && v_parts, "NULL pointer");
  AWQ_REQUIRE(n_heads > 0 && parts_pos > 0 && pos0 >= 0 && n >= 0 && pos0 + n <= parts_pos, "positions beyond the parts arrays");
  if (n == 0) return AWQ_OK;
  const int64_t threads = (int64_t)n_heads * n * 16;
  hipLaunchKernelGGL(kv_to_parts_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, k_cache, v_cache, kv,
                     k_parts, v_parts, n_heads, parts_pos, (int)pos0, (int)n);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
