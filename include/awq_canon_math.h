/*
 * awq_canon_math.h -- the arithmetic that must come out bit-identical on the
 * host and on the GPU.
 *
 * The reference engine calls expf (Inference.cu:242), erff (Inference.cu:276)
 * and rsqrtf (Inference.cu:137) from the CUDA math library.  Those routines are
 * not bit-reproducible on other platforms, so greedy token identity between a
 * GPU run and a CPU run is only possible when both sides evaluate the same
 * sequence of IEEE-754 binary32 operations.  This header fixes that sequence.
 * Every function below uses only +, -, *, /, sqrt and fma on binary32 plus
 * integer bit manipulation, all of which are correctly rounded on x86-64 and
 * on gfx950 (compile without fast-math and with FP contraction off).
 *
 * Accuracy (measured by tests/test_oracle_ops.py::test_canonical_exp_erf_accuracy against libm in double):
 *   awq_expf   <= 1 ulp on [-104, 88.7]
 *   awq_erff   <= 2 ulp for |x| < 1, absolute error <= 1 ulp(1.0) elsewhere
 *   awq_rsqrtf <= 1 ulp (a correctly rounded sqrt followed by a correctly
 *              rounded divide)
 *
 * Also here: the scale/zero-point group index (Inference.cu:90) with the
 * out-of-bounds cases given a defined value, and its period along the input
 * dimension, which fixes the summation order of the linear layers.
 */
#ifndef AWQ_CANON_MATH_H
#define AWQ_CANON_MATH_H

#include <stdint.h>
#include <math.h>
#include <string.h>

#if defined(__HIPCC__)
#define AWQ_HD __host__ __device__ inline
#else
#define AWQ_HD static inline
#endif

#define AWQ_GROUP_SIZE 128      /* Inference.cu:40 */
#define AWQ_HEAD_DIM 128        /* Inference.cu:36 */
#define AWQ_BLOCK_K 32          /* inputs per block of a linear layer (one power of two per block) */

AWQ_HD float awq_bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
AWQ_HD uint32_t awq_f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* exp(x) in binary32.  x = n*ln2 + r, |r| <= ln2/2, exp(r) by a degree-7
 * polynomial, then two exact power-of-two scalings so that results in the
 * subnormal range are rounded once. */
AWQ_HD float awq_expf(float x) {
  if (x != x) return x;
  if (x > 88.72283f) return awq_bits_to_f32(0x7f800000u);
  if (x < -103.98f) return 0.0f;
  const float magic = 12582912.0f; /* 1.5 * 2^23: adding it rounds to nearest integer */
  float t = fmaf(x, 1.44269504f, magic);
  float n = t - magic;
  int ni = (int)(awq_f32_to_bits(t) - awq_f32_to_bits(magic));
  float r = fmaf(n, -0.693145752f, x);       /* ln2 high part, 12 trailing zero bits */
  r = fmaf(n, -1.42860677e-06f, r);          /* ln2 low part */
  float p = 0.00019899285689461976f;
  p = fmaf(p, r, 0.0013933650916442275f);
  p = fmaf(p, r, 0.0083332983776927f);
  p = fmaf(p, r, 0.04166646674275398f);
  p = fmaf(p, r, 0.1666666716337204f);
  p = fmaf(p, r, 0.5f);
  float r2 = r * r;
  float e = fmaf(p, r2, r) + 1.0f;
  int n1 = ni / 2;
  int n2 = ni - n1;
  float s1 = awq_bits_to_f32((uint32_t)(n1 + 127) << 23);
  float s2 = awq_bits_to_f32((uint32_t)(n2 + 127) << 23);
  return (e * s1) * s2;
}

/* erf(x) in binary32.  |x| < 1: x*P(x^2).  1 <= |x| < 4: 1 - exp(-|x|*Q(|x|)).
 * Beyond 4 the result is +-1 in binary32. */
AWQ_HD float awq_erff(float x) {
  if (x != x) return x;
  float a = fabsf(x);
  if (a < 1.0f) {
    float s = x * x;
    float p = 7.882497448008507e-05f;
    p = fmaf(p, s, -0.0008018855005502701f);
    p = fmaf(p, s, 0.005189312156289816f);
    p = fmaf(p, s, -0.02685432881116867f);
    p = fmaf(p, s, 0.11283597350120544f);
    p = fmaf(p, s, -0.3761262595653534f);
    p = fmaf(p, s, 1.1283791065216064f);
    return x * p;
  }
  float y;
  if (a >= 4.0f) {
    y = 1.0f;
  } else {
    float q = -2.37608659858779e-07f;
    q = fmaf(q, a, 3.659137064460083e-06f);
    q = fmaf(q, a, -5.208507445786381e-06f);
    q = fmaf(q, a, -0.00031440466409549117f);
    q = fmaf(q, a, 0.0037855366244912148f);
    q = fmaf(q, a, -0.024242741987109184f);
    q = fmaf(q, a, 0.10692556202411652f);
    q = fmaf(q, a, 0.634675145149231f);
    q = fmaf(q, a, 1.1287782192230225f);
    y = 1.0f - awq_expf(-(a * q));
  }
  return x < 0.0f ? -y : y;
}

/* 1/sqrt(x): stands in for rsqrtf at Inference.cu:137. */
AWQ_HD float awq_rsqrtf(float x) { return 1.0f / sqrtf(x); }

/* exact-erf GeLU in binary32, Inference.cu:274-277 */
AWQ_HD float awq_gelu_f32(float v) {
  float e = awq_erff(v * 0.70710678f);
  return (0.5f * v) * (1.0f + e);
}

/*
 * Scale / zero-point group of element (out index i, in index j) of a linear
 * layer with m outputs and k inputs (both multiples of 128).
 *
 * The reference dequantises a [rows=m][cols=k] row-major buffer with
 * group = (flat % cols) / 128 (Inference.cu:88-90) and then hands that buffer
 * to a column-major GEMM with lda = m (Inference.cu:1059), so the weight that
 * multiplies x[j] for output i is flat element p = j*m + i.  The scale arrays
 * hold m/128 entries (Inference.cu:619); an index past that is undefined in
 * the reference and is wrapped here.
 */
AWQ_HD int awq_group_index(int64_t m, int64_t k, int64_t i, int64_t j) {
  int64_t p = j * m + i;
  int64_t g = (p % k) / AWQ_GROUP_SIZE;
  return (int)(g % (m / AWQ_GROUP_SIZE));
}

/*
 * Smallest C such that awq_group_index(m,k,i,j) == awq_group_index(m,k,i,j+C)
 * for all i, j.  It is 1 for every per-layer matrix and 32 for the
 * 151936 x 4096 unembedding.
 */
AWQ_HD int awq_group_period(int64_t m, int64_t k) {
  int64_t mg = m / AWQ_GROUP_SIZE, kg = k / AWQ_GROUP_SIZE;
  if (mg % kg == 0 || kg % mg == 0) return 1;
  int64_t a = mg, b = kg;
  while (b) {
    int64_t t = a % b;
    a = b;
    b = t;
  }
  return (int)(kg / a);
}

/*
 * Arithmetic of a linear layer, y[i] = sum_j w(i,j) * x[j] with w = (q - z) * s.
 *
 * The k inputs of one output are cut into k/32 blocks; block number blk holds,
 * for t = 0..31, input index
 *     j = c + C*(32*u + t),   C = awq_group_period(m,k), blk = c*(k/(32*C)) + u
 * so that all 32 share one scale group (s, z).  C must divide k/32.
 *
 * The inputs of a block are first put into block fixed point (once per input
 * vector, the same for every output row):
 *     e    = the largest binary16 exponent field among the 32 inputs (0..31)
 *     c    = 2^(max(e,1) - 29)                  (a NaN when e == 31: the block holds an infinity or a NaN)
 *     I[t] = x[t] / c rounded to the nearest integer, ties to even;  |I[t]| <= 32752
 *     S    = sum I[t]
 * i.e. a 16-bit integer per input under the block's common power of two: the block's largest inputs keep
 * all 11 significand bits, an input 2^-n below the largest exponent loses its last n - 5 bits.  Per row
 *     D = sum q[t] * I[t]                       exact in integers, |D| < 2^24, q the raw nibble
 *     v = fma(-z, S, D) * (s * c)               binary32; S and D convert exactly, s * c is exact
 * and the k/32 block values v are combined by awq_tree_sum; the result is rounded to binary16 once.
 * The scale and the zero-point are applied to a block's sums rather than to every weight, so the binary16
 * rounding of each dequantised weight (Inference.cu:102-104) does not appear here; it stays in the
 * standalone dequantisation and in the plain sequential FP32 reference that the tests hold this arithmetic
 * to (1e-2 relative).  Against the exact product of the unrounded weights the only errors are the
 * rounding of I (at most c/2 per input, 2^-16 of the block's largest magnitude), one rounding per block
 * value and the tree.
 *
 * Why integers: on the GPU v_dot8_u32_u4 multiplies eight weight nibbles by eight 4-bit digits of the
 * inputs and adds them up exactly in one instruction, straight from the packed weight dword; a CPU adds
 * the same integers.  Nothing depends on an order of summation inside a block.
 */
AWQ_HD int64_t awq_block_elem(int64_t k, int C, int64_t blk, int t) {
  int64_t U = k / ((int64_t)AWQ_BLOCK_K * C);
  int64_t c = blk / U, u = blk % U;
  return c + (int64_t)C * (AWQ_BLOCK_K * u + t);
}

/* Block fixed point of one block: x[t] the block's 32 inputs widened to binary32 (binary16 values).
 * Writes I[0..31] and *S, returns c. */
AWQ_HD float awq_block_fixed(const float* x, int32_t* I, int32_t* S) {
  uint32_t emax = 0;
  for (int t = 0; t < AWQ_BLOCK_K; ++t) {
    uint32_t e = (awq_f32_to_bits(x[t]) & 0x7fffffffu) >> 23; /* binary16 field + 112 for a normal half */
    if (e > emax) emax = e;
  }
  const uint32_t e16 = emax == 255u ? 31u : (emax > 113u ? emax - 112u : 1u); /* max(e,1), 31 = not finite */
  const uint32_t cbits = (e16 + 98u) << 23;
  const float inv = awq_bits_to_f32(0x7f000000u - cbits); /* 1/c */
  int32_t sum = 0;
  for (int t = 0; t < AWQ_BLOCK_K; ++t) {
    /* adding 1.5 * 2^23 + 32768 rounds x/c to an integer; its low 16 bits are I + 32768 */
    const uint32_t u = awq_f32_to_bits(fmaf(x[t], inv, 12615680.0f)) & 0xffffu;
    I[t] = (int32_t)u - 32768;
    sum += I[t];
  }
  *S = sum;
  return awq_bits_to_f32(e16 == 31u ? 0x7fc00000u : cbits);
}

/* D of one block: q[t] in 0..15 */
AWQ_HD int32_t awq_block_idot(const int* q, const int32_t* I) {
  int32_t d = 0;
  for (int t = 0; t < AWQ_BLOCK_K; ++t) d += q[t] * I[t];
  return d;
}

/* v of one block from its D, the block's S and c, and the group's scale and zero-point */
AWQ_HD float awq_block_value(int32_t D, int32_t S, float c, float s, float z) {
  return fmaf(-z, (float)S, (float)D) * (s * c);
}

/* Combine n partial sums in place: adjacent pairs while the count is even,
 * then left to right.  Returns the total. */
AWQ_HD float awq_tree_sum(float* v, int64_t n) {
  while (n > 1 && (n & 1) == 0) {
    n >>= 1;
    for (int64_t a = 0; a < n; ++a) v[a] = v[2 * a] + v[2 * a + 1];
  }
  float s = v[0];
  for (int64_t a = 1; a < n; ++a) s += v[a];
  return s;
}

#endif /* AWQ_CANON_MATH_H */
