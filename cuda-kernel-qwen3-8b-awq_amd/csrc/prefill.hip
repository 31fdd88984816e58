// The per-token operators of the prompt loop (Inference.cu:1304-1343) for M
// prompt positions at once.  Each token goes through exactly the arithmetic of
// the one-token kernels (same rounding points, same summation orders); only
// the matrix products between them change, from M matrix-vector products to
// one product on the matrix cores.
//
// Activations are [M][n] row-major: token t's vector is contiguous, which is
// what the reference's column-per-token cublasGemmEx operands (ldb = k,
// ldc = m) look like in memory.
#include "common.hpp"

namespace {

// gather lambda, Inference.cu:1310-1324, for M token ids
__global__ __launch_bounds__(256) void embed_batch_kernel(const uint8_t* __restrict__ packed,
                                                          const half_t* __restrict__ scale,
                                                          const half_t* __restrict__ zp, int hidden, int64_t vocab,
                                                          const int32_t* __restrict__ tokens,
                                                          half_t* __restrict__ out) {
  const int tok = tokens[blockIdx.y];
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= hidden) return;
  const int g = (tok / AWQ_GROUP_SIZE) % (hidden / AWQ_GROUP_SIZE);
  const uint32_t byte = packed[(int64_t)idx * (vocab >> 1) + (tok >> 1)];
  const uint32_t q = (tok & 1) ? (byte >> 4) : (byte & 15u);
  const half_t d = (half_t)(float)q - zp[g];
  out[(int64_t)blockIdx.y * hidden + idx] = d * scale[g];
}

// rmsNormKernel, Inference.cu:111-145, one workgroup per token: 16-byte loads, the
// sum of squares through wavefront shuffles and one LDS exchange
__global__ __launch_bounds__(256) void rmsnorm_batch_kernel(const half_t* __restrict__ x,
                                                            const half_t* __restrict__ gamma,
                                                            half_t* __restrict__ out, int n, float eps) {
  __shared__ float wsum[4];
  const int tid = threadIdx.x;
  const half8_t* xv = reinterpret_cast<const half8_t*>(x + (int64_t)blockIdx.x * n);
  const half8_t* gv = reinterpret_cast<const half8_t*>(gamma);
  half8_t* ov = reinterpret_cast<half8_t*>(out + (int64_t)blockIdx.x * n);
  const int chunks = n >> 3;
  constexpr int kKeep = 4;  // chunks a thread keeps in registers (n <= 8192: all of them)
  half8_t held[kKeep];
  float acc = 0.0f;
#pragma unroll
  for (int c = 0; c < kKeep; ++c) {
    const int at = tid + c * 256;
    if (at < chunks) {
      held[c] = xv[at];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = __builtin_fmaf((float)held[c][e], (float)held[c][e], acc);
    }
  }
  for (int at = tid + kKeep * 256; at < chunks; at += 256) {
    const half8_t v = xv[at];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = __builtin_fmaf((float)v[e], (float)v[e], acc);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if ((tid & 63) == 0) wsum[tid >> 6] = acc;
  __syncthreads();
  const float total = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
  const half_t sc = (half_t)awq_rsqrtf(total / (float)n + eps);
  const half8_t sc8 = half8_t{sc, sc, sc, sc, sc, sc, sc, sc};
#pragma unroll
  for (int c = 0; c < kKeep; ++c) {
    const int at = tid + c * 256;
    if (at < chunks) ov[at] = (held[c] * sc8) * gv[at];
  }
  for (int at = tid + kKeep * 256; at < chunks; at += 256) ov[at] = (xv[at] * sc8) * gv[at];
}

// QKV split, rotary on Q and K, KV append (Inference.cu:1070-1103, 150-177) for
// token blockIdx.y at position pos0 + blockIdx.y; one wavefront per head, four heads per workgroup.
__global__ __launch_bounds__(256) void rope_kv_batch_kernel(const half_t* __restrict__ qkv,
                                                           const half_t* __restrict__ cos_t,
                                                           const half_t* __restrict__ sin_t,
                                                           half_t* __restrict__ q_out, half_t* __restrict__ kc,
                                                           half_t* __restrict__ vc, int n_heads, KvLayout kv,
                                                           int pos0, half_t* __restrict__ kp,
                                                           half_t* __restrict__ vp, int parts_pos) {
  const int tok = blockIdx.y, pos = pos0 + tok;
  const int hd = blockIdx.x * 4 + (threadIdx.x >> 6), i = threadIdx.x & 63;
  if (hd >= n_heads) return;
  const int H = n_heads * AWQ_HEAD_DIM;
  qkv += (int64_t)tok * 3 * H;
  q_out += (int64_t)tok * H;
  const half_t c = cos_t[(int64_t)pos * 64 + i], s = sin_t[(int64_t)pos * 64 + i];
  const int e = hd * AWQ_HEAD_DIM + 2 * i;
  const int64_t dst = kv_row(kv, hd, pos) + 2 * i;
  {
    const half_t a = qkv[e], b = qkv[e + 1];
    const half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    q_out[e] = ac - bs;
    q_out[e + 1] = as + bc;
  }
  // the same rows a second time in the order the fused Wqkv + attention launch of the decode steps reads them,
  // [head][dimension / 16][position][dimension % 16], for the positions that copy holds
  const bool parts = kp != nullptr && pos < parts_pos;
  const int64_t dst_p = (((int64_t)hd * 8 + (i >> 3)) * parts_pos + pos) * 16 + 2 * (i & 7);
  {
    const half_t a = qkv[H + e], b = qkv[H + e + 1];
    const half_t ac = a * c, bs = b * s, as = a * s, bc = b * c;
    const half_t k0 = ac - bs, k1 = as + bc;
    kc[dst] = k0;
    kc[dst + 1] = k1;
    if (parts) kp[dst_p] = k0, kp[dst_p + 1] = k1;
  }
  const half_t v0 = qkv[2 * H + e], v1 = qkv[2 * H + e + 1];
  vc[dst] = v0;
  vc[dst + 1] = v1;
  if (parts) vp[dst_p] = v0, vp[dst_p + 1] = v1;
}


// ---------------------------------------------------------------------------
// Attention of a tile of 128 prompt positions of one head against the cache,
// on the matrix cores: keys and values of 32 positions at a time go through
// LDS once per workgroup instead of once per query.  Same mathematics as
// attentionKernel's comments (Inference.cu:201-265) -- scores scaled by
// 1/sqrt(128) after the dot product, softmax over the attended positions,
// weighted sum of V -- in the usual streaming form (running maximum and sum,
// context rescaled when the maximum moves; probabilities rounded to binary16
// for the second product), so it agrees with the one-query kernel to rounding
// noise, not bit for bit.  Every query is a column of the accumulators:
//   S^T[key][query] = K[key][:] . Q[query][:]      v_mfma_f32_32x32x16_f16 x 8
//   O^T[d][query]  += V^T[d][key] * P^T[key][query]  x 8 (4 tiles of d, 2 of keys)
// so that a query's maximum, sum and rescaling stay inside one lane (plus its
// partner lane + 32), and the probabilities a lane computed are exactly the
// operand elements it has to supply to the second product.
// ---------------------------------------------------------------------------
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

constexpr int kFaQueries = 128;   // per workgroup, 32 per wavefront
constexpr int kFaKeys = 32;       // per step
constexpr int kFaKStride = 136;   // halves per key row of the K tile (128 + 8 of padding)
constexpr int kFaVStride = 144;   // halves per key row of the V tile (128 + 16: four consecutive rows start 8 banks apart)
typedef short short4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256, 2) void prefill_attention_kernel(const half_t* __restrict__ q,
                                                                const half_t* __restrict__ kc,
                                                                const half_t* __restrict__ vc,
                                                                half_t* __restrict__ ctx, KvLayout kv, int pos0,
                                                                int M, int use_len_hi) {
  __shared__ __attribute__((aligned(16))) half_t ks2[2 * kFaKeys * kFaKStride];
  __shared__ __attribute__((aligned(16))) half_t vs2[2 * kFaKeys * kFaVStride];
  const int head = blockIdx.x, n_heads = gridDim.x;
  const int H = n_heads * AWQ_HEAD_DIM;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, kh = lane >> 5;
  const half_t* kh_ptr = kc;
  const half_t* vh_ptr = vc;
  // attended length of the query at position p (Inference.cu:1118 read before or after :1331)
  auto len_of = [&](int p) { return use_len_hi ? p + 1 : (p > 1 ? p : 1); };
  const int q_first = blockIdx.y * kFaQueries;
  const int qi = q_first + wave * 32 + n;                 // this lane's query (a column)
  const int qc = qi < M ? qi : M - 1;
  const int Lq = len_of(pos0 + qc);
  const int L_wg = len_of(pos0 + min(q_first + kFaQueries - 1, M - 1));      // lengths grow with the position
  const int L_wave = len_of(pos0 + min(q_first + wave * 32 + 31, M - 1));
  const int L_wave_min = len_of(pos0 + min(q_first + wave * 32, M - 1));  // the shortest range among its queries

  // the query's 128 components as the second operand of the 8 slices of the first product
  half8_t qop[8];
#pragma unroll
  for (int s = 0; s < 8; ++s)
    qop[s] = *reinterpret_cast<const half8_t*>(q + (int64_t)qc * H + head * AWQ_HEAD_DIM + 16 * s + 8 * kh);

  f32x16_t o[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
  float m_run = -1e30f, l_run = 0.0f;
  // exp(x) = 2^(x log2 e); the scale of Inference.cu:218 folded into the same factor
  const float scale2 = (1.0f / sqrtf((float)AWQ_HEAD_DIM)) * 1.44269504088896340736f;

  // this thread's two 16-byte pieces of the key tile and of the value tile: (key, part of its row).
  // Two tiles are on their way at any time (register sets A and B): with one, a step lasted as long
  // as a trip to memory, which is longer than its arithmetic.
  struct TileRegs {
    u32x4_t k[2];
    half8_t v[2];
  };
  TileRegs ra, rb;
  auto load_tile = [&](int k0, TileRegs& r) __attribute__((always_inline)) {
    if (k0 >= L_wg) return;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int pc = tid + i * 256;
      const int key = pc >> 4, part = pc & 15;
      const int kg = k0 + key < L_wg ? k0 + key : L_wg - 1;  // rows past the end are masked below
      r.k[i] = *reinterpret_cast<const u32x4_t*>(kh_ptr + kv_row(kv, head, kg) + part * 8);
      r.v[i] = *reinterpret_cast<const half8_t*>(vh_ptr + kv_row(kv, head, kg) + part * 8);
    }
  };
  // both register sets go to LDS between one pair of barriers (two tiles of 32 keys per step)
  auto stage = [&](int k0) __attribute__((always_inline)) {
    __syncthreads();  // the previous tiles' readers are done
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int pc = tid + i * 256;
      const int key = pc >> 4, part = pc & 15;
      *reinterpret_cast<u32x4_t*>(ks2 + key * kFaKStride + part * 8) = ra.k[i];
      *reinterpret_cast<half8_t*>(vs2 + key * kFaVStride + part * 8) = ra.v[i];
      if (k0 + kFaKeys < L_wg) {
        *reinterpret_cast<u32x4_t*>(ks2 + (kFaKeys + key) * kFaKStride + part * 8) = rb.k[i];
        *reinterpret_cast<half8_t*>(vs2 + (kFaKeys + key) * kFaVStride + part * 8) = rb.v[i];
      }
    }
    __syncthreads();
    // the next two tiles travel while these are multiplied
    load_tile(k0 + 2 * kFaKeys, ra);
    load_tile(k0 + 3 * kFaKeys, rb);
  };
  auto step = [&](int k0, int half) __attribute__((always_inline)) {
    if (k0 >= L_wave) return;  // nothing of this tile is attended by this wavefront's queries
    const half_t* ks = ks2 + half * kFaKeys * kFaKStride;
    const half_t* vs = vs2 + half * kFaKeys * kFaVStride;

    f32x16_t sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const half8_t kop = *reinterpret_cast<const half8_t*>(ks + n * kFaKStride + 16 * s + 8 * kh);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kop, qop[s], sacc, 0, 0, 0);
    }
    // sacc[i] is the score of key k0 + 8 (i / 4) + 4 kh + i % 4 for this lane's query.  A tile that
    // lies wholly inside the attended range of every query of the wavefront (nearly all tiles of a
    // long prompt) needs no masks; the scale goes into the exponent's multiply-add.
    const bool masked = k0 + kFaKeys > L_wave_min;  // same for the whole wavefront
    float mx = -1e30f;
    if (masked) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = k0 + 8 * (i >> 2) + 4 * kh + (i & 3);
        sacc[i] = key < Lq ? sacc[i] : -1e30f;  // 2^(scale * -1e30 - m) is 0
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sacc[i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // (a tile in which none of this query's keys is attended leaves the maximum where it was)
    const float m_new = fmaxf(m_run, mx > -1e29f ? mx * scale2 : -1e30f);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float rs = 0.0f;
    half8_t pop[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[i], scale2, -m_new));
      rs += pe;
      pop[i >> 3][i & 7] = (half_t)pe;
    }
    rs += __shfl_xor(rs, 32, 64);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    // once the running maxima have settled (most tiles), alpha is 1 in every lane
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
    }
    // second product: slice j takes keys 16 j + 8 (e / 4) + 4 kh + e % 4, e = 0..7, which are this
    // lane's probabilities 8 j .. 8 j + 7.  Its first operand is V transposed: component 32 dt + n of
    // four consecutive keys per 8-byte half.  The transposing LDS read delivers exactly that from the
    // tile as it came from memory: within 16 lanes, lane i receives element i % 4 of the 8-byte pieces
    // that lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12 point at -- so lane L points at the row of key
    // L / 4 of the four, components 4 (L % 4) .. + 3 of the group's sixteen.
    const int L16 = lane & 15;
    const half_t* vlane = vs + (4 * kh + (L16 >> 2)) * kFaVStride + 16 * ((lane >> 4) & 1) + 4 * (L16 & 3);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const half_t* vp = vlane + 16 * j * kFaVStride + dt * 32;
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3)))*)vp);
        const short4_t hi =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3)))*)(vp + 8 * kFaVStride));
        const half4_t lh = __builtin_bit_cast(half4_t, lo), hh = __builtin_bit_cast(half4_t, hi);
        const half8_t vop = half8_t{lh[0], lh[1], lh[2], lh[3], hh[0], hh[1], hh[2], hh[3]};
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vop, pop[j], o[dt], 0, 0, 0);
      }
    }
  };
  load_tile(0, ra);
  load_tile(kFaKeys, rb);
  for (int k0 = 0; k0 < L_wg; k0 += 2 * kFaKeys) {
    stage(k0);
    step(k0, 0);
    if (k0 + kFaKeys < L_wg) step(k0 + kFaKeys, 1);
  }
  // o[dt][i] is component 32 dt + 8 (i / 4) + 4 kh + i % 4 of this lane's query
  if (qi < M) {
    const float inv = 1.0f / l_run;
    half_t* out = ctx + (int64_t)qi * H + head * AWQ_HEAD_DIM;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const half4_t v = half4_t{(half_t)(o[dt][4 * g] * inv), (half_t)(o[dt][4 * g + 1] * inv),
                                  (half_t)(o[dt][4 * g + 2] * inv), (half_t)(o[dt][4 * g + 3] * inv)};
        *reinterpret_cast<half4_t*>(out + dt * 32 + 8 * g + 4 * kh) = v;
      }
  }
}

}  // namespace

int launch_embed_batch(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                       const int32_t* tokens_dev, int64_t M, half_t* out, hipStream_t st) {
  AWQ_REQUIRE(hidden > 0 && hidden % 128 == 0 && vocab > 0 && vocab % 2 == 0, "bad embedding shape");
  AWQ_REQUIRE(M >= 1 && M <= 65535 && tokens_dev, "token count out of range");
  hipLaunchKernelGGL(embed_batch_kernel, dim3((unsigned)((hidden + 255) / 256), (unsigned)M), dim3(256), 0, st, packed,
                     scale, zp, (int)hidden, vocab, tokens_dev, out);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rmsnorm_batch(const half_t* x, const half_t* gamma, half_t* out, int64_t n, int64_t M, float eps,
                         hipStream_t st) {
  AWQ_REQUIRE(n > 0 && n % 256 == 0 && n < (1 << 30), "n must be a positive multiple of 256");
  AWQ_REQUIRE(M >= 1 && M < (1ll << 31), "token count out of range");
  hipLaunchKernelGGL(rmsnorm_batch_kernel, dim3((unsigned)M), dim3(256), 0, st, x, gamma, out, (int)n, eps);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_rope_kv_append_batch(const half_t* qkv, const half_t* cos_t, const half_t* sin_t, half_t* q_out,
                                half_t* kc, half_t* vc, int n_heads, int64_t max_pos, KvLayout kv, int64_t pos0,
                                int64_t M, hipStream_t st, half_t* k_parts, half_t* v_parts, int parts_pos) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0, "n_heads and max_pos must be positive");
  AWQ_REQUIRE((k_parts == nullptr) == (v_parts == nullptr) && (k_parts == nullptr || parts_pos > 0), "parts arrays: both or none");
  AWQ_REQUIRE(M >= 1 && M <= 65535 && pos0 >= 0 && pos0 + M <= max_pos, "positions out of range");
  hipLaunchKernelGGL(rope_kv_batch_kernel, dim3((unsigned)((n_heads + 3) / 4), (unsigned)M), dim3(256), 0, st, qkv, cos_t, sin_t,
                     q_out, kc, vc, n_heads, kv, (int)pos0, k_parts, v_parts, parts_pos);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}

int launch_prefill_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                             int64_t max_pos, KvLayout kv, int64_t pos0, int64_t M, int use_len_hi, hipStream_t st) {
  AWQ_REQUIRE(n_heads > 0 && max_pos > 0, "n_heads and max_pos must be positive");
  AWQ_REQUIRE(M >= 1 && M <= 65535 * kFaQueries && pos0 >= 0 && pos0 + M <= max_pos, "positions out of range");
  hipLaunchKernelGGL(prefill_attention_kernel, dim3((unsigned)n_heads, (unsigned)((M + kFaQueries - 1) / kFaQueries)),
                     dim3(256), 0, st, q, kc, vc, ctx, kv, (int)pos0, (int)M, use_len_hi);
  AWQ_HIP_TRY(hipGetLastError());
  return AWQ_OK;
}
