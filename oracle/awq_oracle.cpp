// awq_oracle.cpp -- CPU restatement of the reference engine's arithmetic.
//
// TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
// calls this file; it is the checker that the HIP kernels are compared with
// (tests/, the smoke check and the cpu_baseline leg of bench.py).
//
// The reference is /root/reference/Inference.cu ("I:" below).  It is CUDA +
// cuBLAS, has no tests or golden vectors, and does not compile as written, so
// each function here restates the reference lines it cites and is pinned by
// closed forms, invariants and brute force in tests/test_oracle_*.py:
//
//   function            follows            pinned by
//   awqo_dequant        I:76-106           exhaustive nibble x (scale,zp) grid vs an
//                                          integer-only soft-float; byte 0xA3 known answer
//   awqo_linear*        I:1052-1065 (+4)   FP64 brute force over the unrounded weights, a second
//                                          (numpy) statement of the block order, one-hot weight
//                                          probe of the column-major reading, 1e-2 against the
//                                          sequential FP32 sum over the reference's rounded
//                                          weights, M>1 == M single products
//   awqo_rmsnorm        I:111-145          constant-vector closed form, FP64 comparison
//   awqo_rope_tables    I:443-454          pos 0 == (1,0), FP64 comparison
//   awqo_rotary         I:150-177          pos 0 identity, pair structure, norm preservation
//   awqo_attention      I:182-266 intended L=1 -> V[0], equal keys -> mean of V, FP64 softmax
//   awqo_gelu           I:271-279          gelu(0)=0, tails, FP64 erf
//   awqo_residual       I:1149-1155        FP16 add closed form
//   awqo_argmax         I:1282-1290        ties -> lowest index, NaN rule
//   awqo_embed          I:1310-1324        equals dequant of the [H][V] matrix, column tok
//   awqo_generate       I:1297-1408        position/length schedule table, L bookkeeping
//   awqo_kv_append      I:1094-1103        numpy [head][pos][128] indexing
//   awqo_model_layer    I:1029-1230        one decoder layer composed in Python from the
//                                          primitives above in the order of I:1035-1228, bit
//                                          for bit (which gamma, what is rotated, where the
//                                          cache rows go, which buffer the residual takes)
//   awqo_model_sample   I:1235-1292        RMSNorm with the last layer's gamma + linear +
//                                          argmax composed in Python, bit for bit
//
// Parity unpinned (no executable reference exists for them, see the notes in
// each function): the accumulation order inside cuBLAS (I:1052), the bits of
// CUDA's expf/erff/rsqrtf, and the three undefined behaviours of the reference
// that are given a definition here (scale index wrap, attention for L > 1,
// aliasing of the Wo product).
//
// Rounding: h(.) is float -> binary16 round-to-nearest-even, f(.) the exact
// widening.  A single +,-,* of two halves evaluated in binary32 and rounded
// with h(.) equals the IEEE binary16 operation, which is what __hadd, __hsub
// and __hmul compute.

#include <immintrin.h>
#include <omp.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#include <algorithm>
#include <chrono>
#include <string>
#include <vector>

#include "../include/awq_canon_math.h"

#define AWQO_API extern "C" __attribute__((visibility("default")))

typedef uint16_t half_t;

static inline float h2f(half_t h) { return _cvtsh_ss(h); }
static inline half_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

// ---------------------------------------------------------------------------
// Integer-only binary16 conversions, used by the tests to cross-check the
// F16C instructions above (two independent implementations of h and f).
// ---------------------------------------------------------------------------
AWQO_API float awqo_soft_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t out;
  if (exp == 0) {
    if (man == 0) {
      out = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while ((man & 0x400u) == 0);
      out = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
    }
  } else if (exp == 31) {
    out = sign | 0x7f800000u | man << 13;
  } else {
    out = sign | (exp + 112) << 23 | man << 13;
  }
  return awq_bits_to_f32(out);
}

AWQO_API uint16_t awqo_soft_f2h(float f) {
  uint32_t x = awq_f32_to_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u | ((ax >> 13) & 0x3ffu) : 0));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to >= 65520 -> inf
  int e = (int)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  int shift;  // bits dropped from the 24-bit significand
  uint32_t base;
  if (e >= -14) {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
  } else {
    shift = 13 + (-14 - e);
    base = 0;
    if (shift > 25) return (uint16_t)sign;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (e >= -14) q &= 0x3ffu;
  uint32_t r = base + q;
  if (rem > halfway || (rem == halfway && (r & 1u))) ++r;  // carry into the exponent is correct
  return (uint16_t)(sign | r);
}

AWQO_API float awqo_h2f(uint16_t h) { return h2f(h); }
AWQO_API uint16_t awqo_f2h(float f) { return f2h(f); }
AWQO_API float awqo_expf(float x) { return awq_expf(x); }
AWQO_API float awqo_erff(float x) { return awq_erff(x); }
AWQO_API int awqo_group_index(int64_t m, int64_t k, int64_t i, int64_t j) { return awq_group_index(m, k, i, j); }
AWQO_API int awqo_group_period(int64_t m, int64_t k) { return awq_group_period(m, k); }
AWQO_API int awqo_num_threads(void) { return omp_get_max_threads(); }

// ---------------------------------------------------------------------------
// dequant, I:76-106.   w[r*cols + c] = h( f(h(float(q) - f(z[g]))) * f(s[g]) )
// with q the low nibble of byte r*((cols+1)/2) + c/2 for even c, the high
// nibble for odd c, and g = c/128 wrapped to the rows/128 entries the scale
// array holds (the wrap is this build's definition of an index the reference
// reads out of bounds, I:90 with I:661).  n_groups is that entry count.
// ---------------------------------------------------------------------------
static inline half_t dequant_one(int q, half_t s, half_t z) {
  half_t sub = f2h((float)q - h2f(z));
  return f2h(h2f(sub) * h2f(s));
}

AWQO_API void awqo_dequant(const uint8_t* packed, const half_t* scale, const half_t* zp, half_t* out, int64_t rows,
                           int64_t cols, int64_t n_groups) {
  int64_t pc = (cols + 1) / 2;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t c = 0; c < cols; ++c) {
      uint8_t b = packed[r * pc + (c >> 1)];
      int q = (c & 1) ? (b >> 4) & 15 : b & 15;
      int64_t g = (c / AWQ_GROUP_SIZE) % n_groups;
      out[r * cols + c] = dequant_one(q, scale[g], zp[g]);
    }
  }
}

// value of flat nibble p of a matrix whose flat stream has even row length
static inline int nibble_at(const uint8_t* packed, int64_t p) {
  uint8_t b = packed[p >> 1];
  return (p & 1) ? (b >> 4) & 15 : b & 15;
}

// ---------------------------------------------------------------------------
// linear layers, I:1052-1065 / 1128-1141 / 1176-1189 / 1201-1214 / 1260-1273.
// cuBLAS reads the dequantised buffer column-major with lda = m:
//     y[i] = h( sum_j f(w[i + j*m]) * f(x[j]) )        (binary32 accumulation)
// Batched: row t of x ([M][k]) gives row t of y ([M][m]) (ldb = k, ldc = m).
//
// Three evaluations:
//   awqo_linear_f64   double accumulation of the dequantised weights h(h(q-z)*s), no final
//                     rounding (brute-force pin)
//   awqo_linear_seq   binary32, j ascending, multiply then add, the same dequantised weights:
//                     the plain FP32-accumulate reference the GPU product is held to (1e-2)
//   awqo_linear       the blocked arithmetic of awq_canon_math.h (per block of 32 inputs: the inputs in
//                     block fixed point, exact integer sums over the raw nibbles, the scale and
//                     zero-point applied to the block's sums in binary32), which the GPU kernels also
//                     follow: results agree bit for bit
// ---------------------------------------------------------------------------
static void build_lut(const half_t* scale, const half_t* zp, int64_t n_groups, std::vector<float>& lut) {
  lut.resize((size_t)n_groups * 16);
  for (int64_t g = 0; g < n_groups; ++g)
    for (int q = 0; q < 16; ++q) lut[g * 16 + q] = h2f(dequant_one(q, scale[g], zp[g]));
}

AWQO_API void awqo_linear_f64(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t m, int64_t k,
                              const half_t* x, double* y, int64_t M) {
  std::vector<float> lut;
  build_lut(scale, zp, m / AWQ_GROUP_SIZE, lut);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    for (int64_t t = 0; t < M; ++t) {
      double acc = 0.0;
      for (int64_t j = 0; j < k; ++j) {
        int g = awq_group_index(m, k, i, j);
        acc += (double)lut[g * 16 + nibble_at(packed, j * m + i)] * (double)h2f(x[t * k + j]);
      }
      y[t * m + i] = acc;
    }
  }
}

AWQO_API void awqo_linear_seq(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t m, int64_t k,
                              const half_t* x, half_t* y, int64_t M) {
  std::vector<float> lut;
  build_lut(scale, zp, m / AWQ_GROUP_SIZE, lut);
  // Every row keeps its own accumulator and sees j = 0, 1, 2, ... in that order (multiply, then add, both
  // rounded to binary32), so the loops may run with j outside and the rows of a 128-row block inside: the
  // nibbles of consecutive rows are consecutive in memory, and a block of 128 aligned rows shares one scale
  // group for a given j (j*m and k are multiples of 128).
  std::vector<float> xf((size_t)k);
  for (int64_t t = 0; t < M; ++t) {
    for (int64_t j = 0; j < k; ++j) xf[j] = h2f(x[t * k + j]);
#pragma omp parallel for schedule(static)
    for (int64_t i0 = 0; i0 < m; i0 += AWQ_GROUP_SIZE) {
      float acc[AWQ_GROUP_SIZE];
      for (int r = 0; r < AWQ_GROUP_SIZE; ++r) acc[r] = 0.0f;
      for (int64_t j = 0; j < k; ++j) {
        const float* lg = &lut[(size_t)awq_group_index(m, k, i0, j) * 16];
        const uint8_t* src = packed + ((j * m + i0) >> 1);  // j*m + i0 is even
        const float xj = xf[j];
        for (int r = 0; r < AWQ_GROUP_SIZE; r += 2) {
          const uint8_t b = src[r >> 1];
          const float p0 = lg[b & 15] * xj, p1 = lg[b >> 4] * xj;
          acc[r] = acc[r] + p0;
          acc[r + 1] = acc[r + 1] + p1;
        }
      }
      for (int r = 0; r < AWQ_GROUP_SIZE; ++r) y[t * m + i0 + r] = f2h(acc[r]);
    }
  }
}

// scalar statement of the blocked arithmetic (the definition)
AWQO_API void awqo_linear_scalar(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t m, int64_t k,
                                 const half_t* x, half_t* y, int64_t M) {
  const int C = awq_group_period(m, k);
  const int64_t nblk = k / AWQ_BLOCK_K;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    std::vector<float> part((size_t)nblk);
    for (int64_t t = 0; t < M; ++t) {
      for (int64_t blk = 0; blk < nblk; ++blk) {
        int q[AWQ_BLOCK_K];
        float xf[AWQ_BLOCK_K];
        int32_t I[AWQ_BLOCK_K], S;
        int g = 0;
        for (int e = 0; e < AWQ_BLOCK_K; ++e) {
          int64_t j = awq_block_elem(k, C, blk, e);
          g = awq_group_index(m, k, i, j);  // the same for the whole block
          q[e] = nibble_at(packed, j * m + i);
          xf[e] = h2f(x[t * k + j]);
        }
        const float c = awq_block_fixed(xf, I, &S);
        part[blk] = awq_block_value(awq_block_idot(q, I), S, c, h2f(scale[g]), h2f(zp[g]));
      }
      y[t * m + i] = f2h(awq_tree_sum(part.data(), nblk));
    }
  }
}

// AVX2 evaluation of the same arithmetic: 8 outputs per vector, integer sums per lane (exact, so the
// bits equal awqo_linear_scalar; tests compare the two).
// Returns the FP32 sums before rounding when y32 != NULL.
static void linear_blocked(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t m, int64_t k,
                           const half_t* x, half_t* y, float* y32) {
  const int C = awq_group_period(m, k);
  const int64_t nblk = k / AWQ_BLOCK_K;
  const int64_t RC = 64;  // rows per task
  // block fixed point of x, once per input vector
  std::vector<int32_t> xi((size_t)k), xS((size_t)nblk);
  std::vector<float> xc((size_t)nblk);
  for (int64_t blk = 0; blk < nblk; ++blk) {
    float t[AWQ_BLOCK_K];
    for (int e = 0; e < AWQ_BLOCK_K; ++e) t[e] = h2f(x[awq_block_elem(k, C, blk, e)]);
    xc[blk] = awq_block_fixed(t, &xi[blk * AWQ_BLOCK_K], &xS[blk]);
  }
  const __m256i shifts = _mm256_setr_epi32(0, 4, 8, 12, 16, 20, 24, 28);
  const __m256i nib = _mm256_set1_epi32(15);
#pragma omp parallel
  {
    std::vector<float> part((size_t)nblk * RC);
#pragma omp for schedule(dynamic, 4)
    for (int64_t i0 = 0; i0 < m; i0 += RC) {
      for (int64_t blk = 0; blk < nblk; ++blk) {
        __m256i acc[8];
        for (int v = 0; v < 8; ++v) acc[v] = _mm256_setzero_si256();
        int g = 0;
        for (int e = 0; e < AWQ_BLOCK_K; ++e) {
          int64_t j = awq_block_elem(k, C, blk, e);
          g = awq_group_index(m, k, i0, j);  // 64 rows starting at a multiple of 64 share a group, a block too
          const uint8_t* src = packed + ((j * m + i0) >> 1);
          // q (0..15) times I (16 bits) as one 16-bit multiply-add per 32-bit lane: the upper halves are zero
          const __m256i iv = _mm256_set1_epi32(xi[blk * AWQ_BLOCK_K + e] & 0xffff);
          for (int v = 0; v < 8; ++v) {
            uint32_t w32;
            memcpy(&w32, src + 4 * v, 4);
            __m256i q = _mm256_and_si256(_mm256_srlv_epi32(_mm256_set1_epi32((int)w32), shifts), nib);
            acc[v] = _mm256_add_epi32(acc[v], _mm256_madd_epi16(q, iv));
          }
        }
        const __m256 zn = _mm256_set1_ps(-h2f(zp[g])), sc = _mm256_set1_ps(h2f(scale[g]) * xc[blk]),
                     S = _mm256_set1_ps((float)xS[blk]);
        for (int v = 0; v < 8; ++v)
          _mm256_storeu_ps(&part[blk * RC + 8 * v], _mm256_mul_ps(_mm256_fmadd_ps(zn, S, _mm256_cvtepi32_ps(acc[v])), sc));
      }
      // awq_tree_sum over blocks, 64 rows at a time
      int64_t n = nblk;
      while (n > 1 && (n & 1) == 0) {
        n >>= 1;
        for (int64_t a = 0; a < n; ++a)
          for (int r = 0; r < RC; r += 8)
            _mm256_storeu_ps(&part[a * RC + r], _mm256_add_ps(_mm256_loadu_ps(&part[2 * a * RC + r]),
                                                              _mm256_loadu_ps(&part[(2 * a + 1) * RC + r])));
      }
      for (int r = 0; r < RC; r += 8) {
        __m256 s = _mm256_loadu_ps(&part[r]);
        for (int64_t a = 1; a < n; ++a) s = _mm256_add_ps(s, _mm256_loadu_ps(&part[a * RC + r]));
        float tmp[8];
        _mm256_storeu_ps(tmp, s);
        for (int q = 0; q < 8; ++q) {
          if (y) y[i0 + r + q] = f2h(tmp[q]);
          if (y32) y32[i0 + r + q] = tmp[q];
        }
      }
    }
  }
}

AWQO_API void awqo_linear(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t m, int64_t k,
                          const half_t* x, half_t* y, int64_t M) {
  for (int64_t t = 0; t < M; ++t) linear_blocked(packed, scale, zp, m, k, x + t * k, y + t * m, nullptr);
}

// ---------------------------------------------------------------------------
// RMSNorm, I:111-145.  256 strided partial sums of squares (I:123-127; nvcc
// contracts acc += v*v to an fma by default, so fmaf here), the stride-halving
// tree of I:130-135, scale = h(1/sqrt(mean + eps)), out = h(h(x*scale)*gamma).
// rsqrtf (I:137) is replaced by awq_rsqrtf; its CUDA bits are unpinned.
// ---------------------------------------------------------------------------
AWQO_API void awqo_rmsnorm(const half_t* x, const half_t* gamma, half_t* out, int64_t n, float eps) {
  float part[256];
  for (int t = 0; t < 256; ++t) {
    float acc = 0.0f;
    for (int64_t i = t; i < n; i += 256) {
      float v = h2f(x[i]);
      acc = fmaf(v, v, acc);
    }
    part[t] = acc;
  }
  for (int stride = 128; stride > 0; stride >>= 1)
    for (int t = 0; t < stride; ++t) part[t] += part[t + stride];
  float mean_sq = part[0] / (float)n;
  half_t sc = f2h(awq_rsqrtf(mean_sq + eps));
  for (int64_t i = 0; i < n; ++i) {
    half_t tmp = f2h(h2f(x[i]) * h2f(sc));
    out[i] = f2h(h2f(tmp) * h2f(gamma[i]));
  }
}

// ---------------------------------------------------------------------------
// rotary tables (I:443-454) and rotation (I:150-177).  The tables come from
// the host libm in the reference too (powf/cosf/sinf in the constructor).
// ---------------------------------------------------------------------------
AWQO_API void awqo_rope_tables(half_t* cos_t, half_t* sin_t, int64_t max_pos) {
  const int hp = AWQ_HEAD_DIM / 2;
#pragma omp parallel for schedule(static)
  for (int64_t pos = 0; pos < max_pos; ++pos) {
    for (int i = 0; i < hp; ++i) {
      float inv_freq = 1.0f / powf(10000.0f, (float)(2 * i) / (float)AWQ_HEAD_DIM);
      float angle = (float)pos * inv_freq;
      cos_t[pos * hp + i] = f2h(cosf(angle));
      sin_t[pos * hp + i] = f2h(sinf(angle));
    }
  }
}

AWQO_API void awqo_rotary(half_t* x, const half_t* cos_t, const half_t* sin_t, int n_heads, int64_t pos) {
  const int hp = AWQ_HEAD_DIM / 2;
  for (int hd = 0; hd < n_heads; ++hd) {
    for (int i = 0; i < hp; ++i) {
      half_t a = x[hd * AWQ_HEAD_DIM + 2 * i], b = x[hd * AWQ_HEAD_DIM + 2 * i + 1];
      half_t c = cos_t[pos * hp + i], s = sin_t[pos * hp + i];
      half_t ac = f2h(h2f(a) * h2f(c)), bs = f2h(h2f(b) * h2f(s));
      half_t as = f2h(h2f(a) * h2f(s)), bc = f2h(h2f(b) * h2f(c));
      x[hd * AWQ_HEAD_DIM + 2 * i] = f2h(h2f(ac) - h2f(bs));
      x[hd * AWQ_HEAD_DIM + 2 * i + 1] = f2h(h2f(as) + h2f(bc));
    }
  }
}

// KV append, I:1094-1103: cache[h][pos][:] <- cur[h][:], head stride max_pos*128
AWQO_API void awqo_kv_append(half_t* cache, const half_t* cur, int n_heads, int64_t max_pos, int64_t pos) {
  for (int hd = 0; hd < n_heads; ++hd)
    memcpy(cache + ((int64_t)hd * max_pos + pos) * AWQ_HEAD_DIM, cur + hd * AWQ_HEAD_DIM, AWQ_HEAD_DIM * sizeof(half_t));
}

// ---------------------------------------------------------------------------
// attention, the math the comments of I:201, 228, 258 describe (the kernel as
// written overwrites its own scores for L > 1, so those lines are followed for
// intent; for L == 1 this equals what the kernel computes, V[0]).
//   s_t = (sum_d q_d k_td) * (1/sqrt(128))           I:203-219
//   mx  = max(-1e9, max_t s_t)                        I:229-233
//   e_t = exp(s_t - mx), Z = sum_t e_t, p_t = e_t/Z   I:241-254
//   ctx_d = h( sum_t p_t v_td )                       I:259-265
// Summation orders (this build's definition, shared with the GPU kernel):
//   dot: 16 partials over 8 consecutive d (fma chains), adjacent-pair tree
//   Z:   positions in chunks of 64, adjacent-pair tree inside a chunk (zero
//        padded), chunks added in order
//   ctx: per chunk of 64 positions four interleaved fma chains (t mod 4),
//        combined (0+1)+(2+3); chunk vectors added in order
// ---------------------------------------------------------------------------
AWQO_API void awqo_attention(const half_t* q, const half_t* kc, const half_t* vc, half_t* ctx, int n_heads,
                             int64_t max_pos, int64_t L, float* scores_out) {
  const float scale = 1.0f / sqrtf((float)AWQ_HEAD_DIM);
#pragma omp parallel for schedule(dynamic, 1)
  for (int hd = 0; hd < n_heads; ++hd) {
    const half_t* qh = q + hd * AWQ_HEAD_DIM;
    const half_t* kh = kc + (int64_t)hd * max_pos * AWQ_HEAD_DIM;
    const half_t* vh = vc + (int64_t)hd * max_pos * AWQ_HEAD_DIM;
    std::vector<float> s((size_t)L), e((size_t)L);
    float qf[AWQ_HEAD_DIM];
    for (int d = 0; d < AWQ_HEAD_DIM; ++d) qf[d] = h2f(qh[d]);
    float mx = -1e9f;
    for (int64_t t = 0; t < L; ++t) {
      float part[16];
      for (int l = 0; l < 16; ++l) {
        float acc = 0.0f;
        for (int d = 8 * l; d < 8 * l + 8; ++d) acc = fmaf(qf[d], h2f(kh[t * AWQ_HEAD_DIM + d]), acc);
        part[l] = acc;
      }
      s[t] = awq_tree_sum(part, 16) * scale;
      mx = fmaxf(mx, s[t]);
    }
    if (scores_out) memcpy(scores_out + (int64_t)hd * L, s.data(), L * sizeof(float));
    float Z = 0.0f;
    for (int64_t base = 0; base < L; base += 64) {
      float c[64];
      for (int u = 0; u < 64; ++u) {
        int64_t t = base + u;
        c[u] = 0.0f;
        if (t < L) c[u] = e[t] = awq_expf(s[t] - mx);
      }
      float cs = awq_tree_sum(c, 64);
      Z = (base == 0) ? cs : Z + cs;
    }
    float out[AWQ_HEAD_DIM];
    for (int64_t base = 0; base < L; base += 64) {
      float acc[4][AWQ_HEAD_DIM];
      memset(acc, 0, sizeof(acc));
      for (int u = 0; u < 64; ++u) {
        int64_t t = base + u;
        if (t >= L) break;
        float p = e[t] / Z;
        for (int d = 0; d < AWQ_HEAD_DIM; ++d) acc[u & 3][d] = fmaf(p, h2f(vh[t * AWQ_HEAD_DIM + d]), acc[u & 3][d]);
      }
      for (int d = 0; d < AWQ_HEAD_DIM; ++d) {
        float cv = (acc[0][d] + acc[1][d]) + (acc[2][d] + acc[3][d]);
        out[d] = (base == 0) ? cv : out[d] + cv;
      }
    }
    for (int d = 0; d < AWQ_HEAD_DIM; ++d) ctx[hd * AWQ_HEAD_DIM + d] = f2h(out[d]);
  }
}

// residual add, I:1149-1155:  out = h(f(a) + f(b))
AWQO_API void awqo_residual(const half_t* a, const half_t* b, half_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = f2h(h2f(a[i]) + h2f(b[i]));
}

// GeLU, I:271-279, erff replaced by awq_erff (CUDA's bits are unpinned)
AWQO_API void awqo_gelu(half_t* x, int64_t n) {
  for (int64_t i = 0; i < n; ++i) x[i] = f2h(awq_gelu_f32(h2f(x[i])));
}

// greedy argmax over FP16 logits widened to float, I:1278-1290: strict '>'
// scanning from index 0, so the lowest index wins ties and a NaN never wins
// unless it sits at index 0.
AWQO_API int awqo_argmax(const half_t* logits, int64_t n) {
  int best = 0;
  float best_score = h2f(logits[0]);
  for (int64_t i = 1; i < n; ++i) {
    float v = h2f(logits[i]);
    if (v > best_score) {
      best_score = v;
      best = (int)i;
    }
  }
  return best;
}

// embedding gather, I:1310-1324: hidden[idx] = dq[idx*V + tok] where dq is the
// dequantised [rows=H][cols=V] word embedding, i.e. column tok of every row.
AWQO_API void awqo_embed(const uint8_t* packed, const half_t* scale, const half_t* zp, int64_t hidden, int64_t vocab,
                         int64_t tok, half_t* out) {
  int64_t n_groups = hidden / AWQ_GROUP_SIZE;
  int64_t g = (tok / AWQ_GROUP_SIZE) % n_groups;
  int64_t pc = (vocab + 1) / 2;
  for (int64_t idx = 0; idx < hidden; ++idx) {
    uint8_t b = packed[idx * pc + (tok >> 1)];
    int q = (tok & 1) ? (b >> 4) & 15 : b & 15;
    out[idx] = dequant_one(q, scale[g], zp[g]);
  }
}

// ---------------------------------------------------------------------------
// model: weights in host memory, literal transcription of runOneLayer
// (I:1029-1230), sampleNextToken (I:1235-1292) and generateResponse
// (I:1297-1408).
// ---------------------------------------------------------------------------
struct awqo_config {
  int n_layers;   // I:37
  int hidden;     // I:33
  int inter;      // I:34
  int vocab;      // I:38
  int max_pos;    // I:39
  int split_idx;  // I:47, kept because it decides the attended length (I:1331, 1364)
  float eps;      // I:41
};

enum { T_WQKV = 0, T_WO = 1, T_W1 = 2, T_W2 = 3, T_GAMMA = 4, T_EMBED = 5, T_UNEMBED = 6 };
enum { P_PACKED = 0, P_SCALE = 1, P_ZP = 2 };

struct Tensor {
  std::vector<uint8_t> packed;
  std::vector<half_t> scale, zp;
  int64_t out_dim = 0, in_dim = 0;
  void alloc(int64_t o, int64_t i) {
    out_dim = o;
    in_dim = i;
    packed.assign((size_t)(o * ((i + 1) / 2)), 0);
    scale.assign((size_t)(o / AWQ_GROUP_SIZE), 0);
    zp.assign((size_t)(o / AWQ_GROUP_SIZE), 0);
  }
};

struct awqo_model {
  awqo_config cfg;
  int n_heads;
  std::vector<Tensor> wqkv, wo, w1, w2;
  std::vector<std::vector<half_t>> gamma;
  Tensor embed, unembed;
  std::vector<std::vector<half_t>> kcache, vcache;
  std::vector<half_t> cos_t, sin_t;
  std::vector<half_t> hidden, normed, qkv, ctx, attn_out, mid, mlp_out, logits;
  std::vector<half_t> last_layer_out;  // hidden state after the last layer of the latest position
  int current_seq_len = 0;
  // statistics of the last generate call
  std::vector<float> margins;
  double seconds_linear = 0;
  // 0: the blocked arithmetic the GPU kernels follow (awqo_linear); 1: the reference's own -- weights rounded to
  // binary16 as dequantAwqKernel leaves them (I:102-104), binary32 accumulation in input order (awqo_linear_seq).
  // Mode 1 exists so that the distance between the two can be measured on a whole model.
  int linear_mode = 0;
};

static Tensor* model_tensor(awqo_model* m, int layer, int kind) {
  switch (kind) {
    case T_WQKV: return &m->wqkv[layer];
    case T_WO: return &m->wo[layer];
    case T_W1: return &m->w1[layer];
    case T_W2: return &m->w2[layer];
    case T_EMBED: return &m->embed;
    case T_UNEMBED: return &m->unembed;
  }
  return nullptr;
}

AWQO_API awqo_model* awqo_model_create(const awqo_config* cfg) {
  awqo_model* m = new awqo_model();
  m->cfg = *cfg;
  const int H = cfg->hidden, I = cfg->inter, V = cfg->vocab, NL = cfg->n_layers;
  m->n_heads = H / AWQ_HEAD_DIM;
  m->wqkv.resize(NL);
  m->wo.resize(NL);
  m->w1.resize(NL);
  m->w2.resize(NL);
  m->gamma.resize(NL);
  m->kcache.resize(NL);
  m->vcache.resize(NL);
  for (int l = 0; l < NL; ++l) {
    m->wqkv[l].alloc(3 * H, H);  // I:616
    m->wo[l].alloc(H, H);        // I:630
    m->w1[l].alloc(I, H);        // I:644
    m->w2[l].alloc(H, I);        // I:658
    m->gamma[l].assign(H, 0);
    size_t kv = (size_t)m->n_heads * cfg->max_pos * AWQ_HEAD_DIM;  // I:676
    m->kcache[l].assign(kv, 0);
    m->vcache[l].assign(kv, 0);
  }
  m->embed.alloc(H, V);    // I:693
  m->unembed.alloc(V, H);  // I:708
  m->cos_t.resize((size_t)cfg->max_pos * (AWQ_HEAD_DIM / 2));
  m->sin_t.resize(m->cos_t.size());
  awqo_rope_tables(m->cos_t.data(), m->sin_t.data(), cfg->max_pos);
  m->hidden.assign(H, 0);
  m->normed.assign(H, 0);
  m->qkv.assign(3 * H, 0);
  m->ctx.assign(H, 0);
  m->attn_out.assign(H, 0);
  m->mid.assign(I, 0);
  m->mlp_out.assign(H, 0);
  m->logits.assign(V, 0);
  return m;
}

AWQO_API void awqo_model_destroy(awqo_model* m) { delete m; }

// pointer to (and byte size of) one stored array so a caller can fill it
AWQO_API void* awqo_model_tensor(awqo_model* m, int layer, int kind, int part, int64_t* bytes) {
  if (kind == T_GAMMA) {
    *bytes = (int64_t)m->gamma[layer].size() * 2;
    return m->gamma[layer].data();
  }
  Tensor* t = model_tensor(m, layer, kind);
  if (!t) return nullptr;
  if (part == P_PACKED) {
    *bytes = (int64_t)t->packed.size();
    return t->packed.data();
  }
  std::vector<half_t>& v = (part == P_SCALE) ? t->scale : t->zp;
  *bytes = (int64_t)v.size() * 2;
  return v.data();
}

static int read_file(const std::string& path, void* dst, size_t bytes) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) {
    fprintf(stderr, "ERROR: could not open %s\n", path.c_str());  // I:299-302
    return 1;
  }
  size_t got = fread(dst, 1, bytes, f);
  fclose(f);
  if (got != bytes) {
    fprintf(stderr, "ERROR: read failed for %s\n", path.c_str());  // I:305-308
    return 1;
  }
  return 0;
}

// weight directory, file names of I:780-899
AWQO_API int awqo_model_load_dir(awqo_model* m, const char* dir) {
  std::string d(dir);
  int rc = 0;
  auto rd = [&](const std::string& name, void* p, size_t n) { rc |= read_file(d + "/" + name, p, n); };
  for (int l = 0; l < m->cfg.n_layers && !rc; ++l) {
    std::string p = "layer_" + std::to_string(l);
    struct {
      Tensor* t;
      const char *w, *s, *z;
    } parts[4] = {{&m->wqkv[l], "_wqkv.bin", "_bqkv_scale.bin", "_bqkv_zp.bin"},
                  {&m->wo[l], "_wo.bin", "_wo_scale.bin", "_wo_zp.bin"},
                  {&m->w1[l], "_w1.bin", "_w1_scale.bin", "_w1_zp.bin"},
                  {&m->w2[l], "_w2.bin", "_w2_scale.bin", "_w2_zp.bin"}};
    for (auto& q : parts) {
      rd(p + q.w, q.t->packed.data(), q.t->packed.size());
      rd(p + q.s, q.t->scale.data(), q.t->scale.size() * 2);
      rd(p + q.z, q.t->zp.data(), q.t->zp.size() * 2);
    }
    rd("rms_norm_gamma_" + std::to_string(l) + ".bin", m->gamma[l].data(), m->gamma[l].size() * 2);
  }
  if (!rc) {
    rd("word_embedding.bin", m->embed.packed.data(), m->embed.packed.size());
    rd("word_embed_scale.bin", m->embed.scale.data(), m->embed.scale.size() * 2);
    rd("word_embed_zp.bin", m->embed.zp.data(), m->embed.zp.size() * 2);
    rd("unembed.bin", m->unembed.packed.data(), m->unembed.packed.size());
    rd("unembed_scale.bin", m->unembed.scale.data(), m->unembed.scale.size() * 2);
    rd("unembed_zp.bin", m->unembed.zp.data(), m->unembed.zp.size() * 2);
  }
  return rc;
}

static void model_linear(awqo_model* m, Tensor& t, const half_t* x, half_t* y) {
  auto t0 = std::chrono::steady_clock::now();
  if (m->linear_mode == 1) awqo_linear_seq(t.packed.data(), t.scale.data(), t.zp.data(), t.out_dim, t.in_dim, x, y, 1);
  else linear_blocked(t.packed.data(), t.scale.data(), t.zp.data(), t.out_dim, t.in_dim, x, y, nullptr);
  m->seconds_linear += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

// runOneLayer, I:1029-1230.  L is the attended length current_seq_len_+1 of I:1118.
AWQO_API void awqo_model_layer(awqo_model* m, int l, int64_t pos, int64_t L) {
  const int H = m->cfg.hidden, I = m->cfg.inter, NH = m->n_heads;
  awqo_rmsnorm(m->hidden.data(), m->gamma[l].data(), m->normed.data(), H, m->cfg.eps);  // I:1040
  model_linear(m, m->wqkv[l], m->normed.data(), m->qkv.data());                          // I:1052
  half_t* Q = m->qkv.data();                                                             // I:1070-1072
  half_t* K = Q + H;
  half_t* V = Q + 2 * H;
  awqo_rotary(Q, m->cos_t.data(), m->sin_t.data(), NH, pos);  // I:1082
  awqo_rotary(K, m->cos_t.data(), m->sin_t.data(), NH, pos);  // I:1087
  awqo_kv_append(m->kcache[l].data(), K, NH, m->cfg.max_pos, pos);  // I:1096-1103
  awqo_kv_append(m->vcache[l].data(), V, NH, m->cfg.max_pos, pos);
  awqo_attention(Q, m->kcache[l].data(), m->vcache[l].data(), m->ctx.data(), NH, m->cfg.max_pos, L, nullptr);  // I:1110
  // I:1125-1141; input and output are separate buffers here (they alias in the reference)
  model_linear(m, m->wo[l], m->ctx.data(), m->attn_out.data());
  awqo_residual(m->hidden.data(), m->attn_out.data(), m->hidden.data(), H);              // I:1155
  awqo_rmsnorm(m->hidden.data(), m->gamma[l].data(), m->normed.data(), H, m->cfg.eps);  // I:1163, same gamma
  model_linear(m, m->w1[l], m->normed.data(), m->mid.data());                            // I:1176
  awqo_gelu(m->mid.data(), I);                                                           // I:1196
  model_linear(m, m->w2[l], m->mid.data(), m->mlp_out.data());                           // I:1201
  awqo_residual(m->hidden.data(), m->mlp_out.data(), m->hidden.data(), H);               // I:1227
}

// sampleNextToken, I:1235-1292
AWQO_API int awqo_model_sample(awqo_model* m) {
  const int H = m->cfg.hidden;
  awqo_rmsnorm(m->hidden.data(), m->gamma[m->cfg.n_layers - 1].data(), m->normed.data(), H, m->cfg.eps);  // I:1247
  model_linear(m, m->unembed, m->normed.data(), m->logits.data());                                       // I:1260
  int best = awqo_argmax(m->logits.data(), m->cfg.vocab);
  // top-1 / top-2 margin, for diagnostics only
  float b1 = -INFINITY, b2 = -INFINITY;
  for (int i = 0; i < m->cfg.vocab; ++i) {
    float v = h2f(m->logits[i]);
    if (v > b1) {
      b2 = b1;
      b1 = v;
    } else if (v > b2) {
      b2 = v;
    }
  }
  m->margins.push_back(b1 - b2);
  return best;
}

static void model_embed(awqo_model* m, int tok) {
  awqo_embed(m->embed.packed.data(), m->embed.scale.data(), m->embed.zp.data(), m->cfg.hidden, m->cfg.vocab, tok,
             m->hidden.data());
}

AWQO_API void awqo_model_reset(awqo_model* m) {
  m->current_seq_len = 0;  // the reference sets this in the constructor only (I:430); reset per call here
  std::fill(m->hidden.begin(), m->hidden.end(), 0);
  m->margins.clear();
  m->seconds_linear = 0;
}

// generateResponse, I:1297-1408.  Returns the number of generated ids, or -1
// when prompt + new tokens do not fit max_pos (the reference asserts on the
// prompt alone, I:1301, and would run off the cache).
AWQO_API int awqo_model_generate(awqo_model* m, const int* prompt, int n_prompt, int max_new, int* out) {
  if (n_prompt < 0 || max_new < 0 || (int64_t)n_prompt + max_new > m->cfg.max_pos) return -1;
  awqo_model_reset(m);
  const int NL = m->cfg.n_layers, SP = m->cfg.split_idx;
  for (int t = 0; t < n_prompt; ++t) {  // I:1304
    model_embed(m, prompt[t]);           // I:1313
    for (int l = 0; l < NL; ++l) {       // I:1329-1342
      awqo_model_layer(m, l, t, m->current_seq_len + 1);
      m->current_seq_len = t;  // I:1331, 1341: updated after every layer
    }
    m->last_layer_out = m->hidden;
  }
  for (int step = 0; step < max_new; ++step) {  // I:1352
    int pos = n_prompt + step;
    // I:1357: the hidden state left by the last layer is the input of this
    // position; for step > 0 that buffer holds the embedding of the sampled
    // token (I:1392-1403).
    for (int l = 0; l < SP; ++l) awqo_model_layer(m, l, pos, m->current_seq_len + 1);  // I:1361-1363
    m->current_seq_len = pos;                                                           // I:1364
    for (int l = SP; l < NL; ++l) awqo_model_layer(m, l, pos, m->current_seq_len + 1);  // I:1371-1373
    m->current_seq_len = pos;                                                           // I:1374
    int tok = awqo_model_sample(m);                                                     // I:1377
    out[step] = tok;
    m->last_layer_out = m->hidden;
    model_embed(m, tok);  // I:1392
  }
  return max_new;
}

AWQO_API const uint16_t* awqo_model_hidden(awqo_model* m) { return m->hidden.data(); }
AWQO_API const uint16_t* awqo_model_logits(awqo_model* m) { return m->logits.data(); }
AWQO_API const uint16_t* awqo_model_last_layer_out(awqo_model* m) {
  if (m->last_layer_out.empty()) m->last_layer_out = m->hidden;
  return m->last_layer_out.data();
}
AWQO_API uint16_t* awqo_model_hidden_mut(awqo_model* m) { return m->hidden.data(); }
AWQO_API uint16_t* awqo_model_kcache(awqo_model* m, int l) { return m->kcache[l].data(); }
AWQO_API uint16_t* awqo_model_vcache(awqo_model* m, int l) { return m->vcache[l].data(); }
AWQO_API int awqo_model_margins(awqo_model* m, float* out, int cap) {
  int n = (int)std::min<size_t>(m->margins.size(), (size_t)cap);
  memcpy(out, m->margins.data(), n * sizeof(float));
  return n;
}
AWQO_API double awqo_model_seconds_linear(awqo_model* m) { return m->seconds_linear; }
AWQO_API void awqo_model_set_linear_mode(awqo_model* m, int mode) { m->linear_mode = mode; }
