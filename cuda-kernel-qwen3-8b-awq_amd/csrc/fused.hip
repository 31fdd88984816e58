// Two dependent products of a decoder layer in ONE launch: the attention output product with its residual
// add (Inference.cu:1128-1155) and, on its result, RMSNorm + W1 + GeLU (Inference.cu:1163-1198).
//
// One workgroup of 16 wavefronts per compute unit, all of them resident at once.  Every workgroup requests
// its share of BOTH matrices when it starts -- one 16-row group of Wo and three of W1, 128 KB, straight into
// registers -- so W1 streams from memory while the Wo product, which a launch of its own would spend mostly
// waiting (a kernel boundary, then one round trip for 8 MB), is still on its way.  The hidden state goes from
// the first product to the second through memory, from every workgroup to every workgroup: each 4-byte word
// carries a binary16 value and a 16-bit tag that is different in every launch, the producers store the words
// with device-scope stores (they bypass the L2 caches of the eight dies, which are not coherent with each
// other), and the consumers poll the vector itself with device-scope loads until every word carries the tag:
// one memory round trip after the last producer's store, no counter, no flag, no fence.
//
// Every wait is bounded.  A workgroup that gives up sets the status word and leaves its outputs unwritten;
// every poll also looks at the status word, so the others follow within a few polls and the launch (and
// every later launch that finds the word set) runs to its end.  The host reads the word after the step.
//
// The arithmetic is that of gemv_kernel (awq_canon_math.h): lane (wavefront w, quarter q, row r) takes blocks
// (4w + q) * 2, + 1 of its row, a lane adds its two blocks, the quarters by lane swaps, the 16 wavefronts
// through LDS in the canonical tree -- the same tree whatever the number of wavefronts, so the bits are those
// of the separate launches.
#include "common.hpp"
#include "gemv_device.hpp"

namespace {

constexpr int kWaves = 16;
constexpr int kThreads = kWaves * 64;
constexpr int kK = 4096;            // inputs of both products
constexpr int kBlocks = kK / 32;    // 128 blocks of 32 inputs
constexpr int kG = 2;               // blocks per lane and row group
constexpr int kW1Groups = 3;        // W1 row groups per workgroup

struct FusedArgs {
  const u32x4* wo;
  const half_t* wo_scale;
  const half_t* wo_zp;
  const u32x4* w1;
  const half_t* w1_scale;
  const half_t* w1_zp;
  const half_t* gamma;
  const half_t* ctx;      // [4096] attention output
  half_t* hidden;         // [4096] residual in, new hidden state out
  half_t* mid;            // [12288] GeLU(W1 ...) out
  uint32_t* hid_tag;      // [4096] the new hidden state as (binary16 | tag << 16)
  int32_t* status;        // [0] != 0: a wait gave up (or the host asks every wait to)
  const StepState* dyn;   // epoch of the step
  int32_t layer;
  int32_t spin_limit;
  float eps;
  int32_t mg_o, mg_1;     // m / 128 of the two matrices
  unsigned long long* stamps;  // STAMPS: [workgroup][kFusedStamps] times of thread 0, 10 ns units
};

// 32 bytes with device-scope loads (sc1: served from beyond the L2 of this die), complete on return; the wait
// also covers every load the wavefront issued before (they return in order)
__device__ __forceinline__ void load_dev_2x4(const void* p, u32x4& lo, u32x4& hi) {
  asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(lo), "=&v"(hi)
               : "v"(p)
               : "memory");
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

// STAMPS: thread 0 of every workgroup notes the time (s_memrealtime, 100 MHz) at the points listed in
// kFusedStampNames -- the instrumented build behind awq_debug_fused_timeline
template <bool STAMPS>
__global__ __launch_bounds__(kThreads) void wo_w1_kernel(FusedArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned char xs[(kK / 8 + kBlocks / kG) * 16];  // planes + skew
  __shared__ __attribute__((aligned(16))) float xc[kBlocks];
  __shared__ __attribute__((aligned(16))) float xS[kBlocks];
  __shared__ __attribute__((aligned(16))) half_t xn[kK];
  __shared__ float red[kW1Groups][16][16];
  __shared__ __attribute__((aligned(16))) float part[256];
  __shared__ int lost;
  const int tid = threadIdx.x, c = blockIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int q = lane >> 4, r = lane & 15;
  const int blk0 = (4 * wave + q) * kG;
  const bool stager = tid < kThreads / 2;  // 512 units of eight inputs
  if (tid == 0) lost = 0;
  int n_stamp = 0;
  auto stamp = [&]() {
    if (STAMPS && tid == 0) a.stamps[(size_t)c * kFusedStamps + n_stamp++] = wall_clock64();
  };
  stamp();  // 0 start

  // ---- requests, in the order the compute unit's memory pipeline should serve them: the small vectors the
  // first product needs, then its weights, then everything of the second product
  uint4 xu = uint4{0, 0, 0, 0}, gu = uint4{0, 0, 0, 0};
  if (stager) {
    xu = reinterpret_cast<const uint4*>(a.ctx)[tid];
    gu = reinterpret_cast<const uint4*>(a.gamma)[tid];
  }
  const int32_t epoch = a.dyn->epoch;
  const int32_t gave_up_before = __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  half_t gs_o, gz_o, gs_1[kW1Groups], gz_1[kW1Groups];
  {
    const unsigned gi = ((unsigned)(c * 16 >> 7) % (unsigned)(kK / 128)) % (unsigned)a.mg_o;
    gs_o = a.wo_scale[gi];
    gz_o = a.wo_zp[gi];
#pragma unroll
    for (int i = 0; i < kW1Groups; ++i) {
      const unsigned g1 = ((unsigned)((kW1Groups * c + i) * 16 >> 7) % (unsigned)(kK / 128)) % (unsigned)a.mg_1;
      gs_1[i] = a.w1_scale[g1];
      gz_1[i] = a.w1_zp[g1];
    }
  }
  half_t res = (half_t)0.0f;
  if (tid < 16) res = a.hidden[c * 16 + tid];
  __syncthreads();
  u32x4 wo_r[kG], w1_r[kW1Groups][kG];
  {
    const u32x4* wp = a.wo + ((int64_t)c * kBlocks + blk0) * 16 + r;
#pragma unroll
    for (int b = 0; b < kG; ++b) wo_r[b] = __builtin_nontemporal_load(wp + b * 16);
  }
  // The second product's weights are requested once the first product's sums are on their way to LDS: a
  // wavefront cannot pass a barrier before the memory pipeline has accepted all its requests, and 128 KB per
  // compute unit take microseconds to be accepted -- requested at the start, they held the first product's
  // barriers back until the whole stream was nearly through.
  auto request_w1 = [&]() {
    const u32x4* w1p = a.w1 + ((int64_t)(kW1Groups * c) * kBlocks + blk0) * 16 + r;
#pragma unroll
    for (int i = 0; i < kW1Groups; ++i)
#pragma unroll
      for (int b = 0; b < kG; ++b) w1_r[i][b] = __builtin_nontemporal_load(w1p + ((int64_t)i * kBlocks + b) * 16);
  };
  const uint32_t tag = (uint32_t)(epoch + a.layer) & 0xffffu;
  stamp();  // 1 all requests issued

  // x in block fixed point: nibble planes, the power of two and the integer sum of every block
  auto stage = [&](const uint4& v) {
    if (stager) {
      const uint32_t h[4] = {v.x, v.y, v.z, v.w};
      u32x4 planes;
      float cc, S;
      stage_unit8(h, planes, cc, S);
      *reinterpret_cast<u32x4*>(xs + (size_t)(tid + (tid / (4 * kG))) * 16) = planes;
      if ((tid & 3) == 0) {
        xc[tid >> 2] = cc;
        xS[tid >> 2] = S;
      }
    }
  };
  const unsigned char* xl = xs + (size_t)(blk0 * 4 + blk0 / kG) * 16;

  // ================= attention output product + residual (Inference.cu:1128-1155) =================
  stage(xu);
  stamp();  // 2 attention output arrived and staged (this wavefront)
  __syncthreads();
  stamp();  // 3 ... by all wavefronts
  {
    const GroupConst g = make_group(gs_o, gz_o);
    float bs[kG];
#pragma unroll
    for (int b = 0; b < kG; ++b)
      bs[b] = __builtin_fmaf(g.zn, xS[blk0 + b], block_dot(wo_r[b], xl + 64 * b)) * (g.s * xc[blk0 + b]);
    const float v = sum_rows_of_16(bs[0] + bs[1]);
    if (q == 0) red[0][wave][r] = v;
  }
  stamp();  // 4 first product multiplied (this wavefront: its Wo weights have arrived)
  __syncthreads();
  stamp();  // 5 ... by all wavefronts
  if (tid < 16 && !gave_up_before) {
    const half_t v = (half_t)sum_16_waves(red[0], r);
    const half_t out = res + v;
    a.hidden[c * 16 + tid] = out;
    __hip_atomic_store(a.hid_tag + c * 16 + tid, (uint32_t)__builtin_bit_cast(unsigned short, out) | (tag << 16),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  stamp();  // 6 new hidden rows stored
  // (a compute unit serves its requests in order: the stores leave before any of the 96 KB requested next)
  __syncthreads();
  request_w1();
  // ================= RMSNorm + W1 + GeLU (Inference.cu:1163-1198) =================
  // the new hidden state from all workgroups: this thread's eight values are eight tagged words
  if (stager) {
    const uint32_t* src = a.hid_tag + 8 * tid;
    int spins = 0;
    bool dead = gave_up_before != 0;
    while (!dead) {
      int32_t st = 0;
      const bool look = (spins & 7) == 7;  // every eighth poll also reads the status word
      if (look) st = __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      u32x4 lo, hi;
      load_dev_2x4(src, lo, hi);
      const bool ok = (lo.x >> 16) == tag && (lo.y >> 16) == tag && (lo.z >> 16) == tag && (lo.w >> 16) == tag &&
                      (hi.x >> 16) == tag && (hi.y >> 16) == tag && (hi.z >> 16) == tag && (hi.w >> 16) == tag;
      if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
        xu.x = (lo.x & 0xffffu) | (lo.y << 16);
        xu.y = (lo.z & 0xffffu) | (lo.w << 16);
        xu.z = (hi.x & 0xffffu) | (hi.y << 16);
        xu.w = (hi.z & 0xffffu) | (hi.w << 16);
        break;
      }
      if (++spins > a.spin_limit) {
        if (lane == 0) __hip_atomic_store(a.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        dead = true;
      }
      if (look && st != 0) dead = true;
    }
    if (dead && lane == 0) lost = 1;
    // rmsNormKernel, Inference.cu:111-145: x in natural order for the 256 strided partial sums
    reinterpret_cast<uint4*>(xn)[tid] = xu;
  }
  stamp();  // 7 the whole new hidden state seen (this wavefront's share)
  __syncthreads();
  stamp();  // 8 ... by all wavefronts
  if (lost) return;  // the same for every thread of the workgroup; nothing of the second product is stored
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
    part[tid] = acc;
  }
  __syncthreads();
  {
    // the tree of Inference.cu:130-135, by every wavefront for itself (see gemv_kernel)
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
  stage(xu);  // the planes of the first product were last read before the barrier that ended it
  stamp();  // 9 normalised and staged
  __syncthreads();
  {
    float bs[kW1Groups][kG];
#pragma unroll
    for (int b = 0; b < kG; ++b) {
      uint4 xv[4];
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) xv[cc] = *reinterpret_cast<const uint4*>(xl + 64 * b + 16 * cc);
      const float S = xS[blk0 + b], cb = xc[blk0 + b];
#pragma unroll
      for (int i = 0; i < kW1Groups; ++i) {
        const GroupConst g = make_group(gs_1[i], gz_1[i]);
        bs[i][b] = __builtin_fmaf(g.zn, S, block_dot_regs(w1_r[i][b], xv)) * (g.s * cb);
      }
    }
#pragma unroll
    for (int i = 0; i < kW1Groups; ++i) {
      const float v = sum_rows_of_16(bs[i][0] + bs[i][1]);
      if (q == 0) red[i][wave][r] = v;
    }
  }
  stamp();  // 10 second product multiplied (this wavefront)
  __syncthreads();
  stamp();  // 11 ... by all wavefronts
  if (tid < 16 * kW1Groups) {
    const half_t v = (half_t)sum_16_waves(red[tid >> 4], r);
    a.mid[kW1Groups * 16 * c + tid] = to_half_rn(awq_gelu_f32((float)v));  // Inference.cu:271-279
  }
  stamp();  // 12 end
}

}  // namespace

int fused_wo_w1_supported(int64_t hidden, int64_t inter) {
  if (hidden != kK || inter != 3 * kK) return 0;
  int dev = 0, cus = 0, occ = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, wo_w1_kernel<false>, kThreads, 0) != hipSuccess) return 0;
  // every workgroup waits for every other one: all hidden/16 of them must be resident at once
  return occ >= 1 && (int64_t)cus * occ >= hidden / 16;
}

int launch_fused_wo_w1(const void* wo, const half_t* wo_scale, const half_t* wo_zp, const void* w1,
                       const half_t* w1_scale, const half_t* w1_zp, const half_t* gamma, float eps, const half_t* ctx,
                       half_t* hidden, half_t* mid, uint32_t* hid_tag, int32_t* status, const StepState* dyn, int layer,
                       int64_t hidden_size, int64_t inter, unsigned long long* stamps, hipStream_t st) {
  AWQ_REQUIRE(hidden_size == kK && inter == 3 * kK, "the fused launch is built for hidden 4096 and intermediate 12288");
  AWQ_REQUIRE(wo && w1 && ctx && hidden && mid && hid_tag && status && dyn, "NULL pointer");
  FusedArgs a;
  a.wo = (const u32x4*)wo;
  a.wo_scale = wo_scale;
  a.wo_zp = wo_zp;
  a.w1 = (const u32x4*)w1;
  a.w1_scale = w1_scale;
  a.w1_zp = w1_zp;
  a.gamma = gamma;
  a.ctx = ctx;
  a.hidden = hidden;
  a.mid = mid;
  a.hid_tag = hid_tag;
  a.status = status;
  a.dyn = dyn;
  a.layer = layer;
  a.spin_limit = 1 << 20;
  a.eps = eps;
  a.mg_o = (int32_t)(hidden_size / 128);
  a.mg_1 = (int32_t)(inter / 128);
  a.stamps = stamps;
  if (stamps) hipLaunchKernelGGL(wo_w1_kernel<true>, dim3((unsigned)(hidden_size / 16)), dim3(kThreads), 0, st, a);
  else hipLaunchKernelGGL(wo_w1_kernel<false>, dim3((unsigned)(hidden_size / 16)), dim3(kThreads), 0, st, a);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
