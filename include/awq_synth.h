/*
 * awq_synth.h -- seeded synthetic weights and inputs.
 *
 * The reference ships no weights and no tool that writes its .bin layout, so
 * tests and benchmarks fill tensors from a counter-based generator: element
 * number idx of stream sid under seed s is a pure function of (s, sid, idx).
 * The same numbers therefore reach the GPU engine and the CPU checker, in any
 * order and from any number of threads.
 *
 *   packed int4 bytes   uniform 0..255 (both nibbles uniform 0..15)
 *   scale               h(0.002 + 0.018*u), u uniform [0,1) with 24 bits
 *   zero-point          h(r mod 16), an integer 0..15
 *   gamma               h(1 + 0.02*n), n ~ N(0,1)
 *   activations / KV    h(n)
 *   token ids           r mod vocab
 *
 * Normals use Box-Muller in double precision and are rounded to binary16 once.
 *
 * Those are the distributions of the benchmark definition.  A 36-layer model
 * drawn from them overflows binary16 within four layers (the zero-points give
 * every weight row a large mean), after which every logit is NaN and greedy
 * decoding returns token 0 whatever the arithmetic does.  AWQ_SYNTH_BALANCED
 * keeps the same format and generator but draws
 *   scale               h(0.0025 + 0.0015*u)
 *   zero-point          h(7 + (r mod 2)), i.e. 7 or 8
 * so that activations stay finite and token identity is a real test.
 */
#ifndef AWQ_SYNTH_H
#define AWQ_SYNTH_H

#include <math.h>
#include <stdint.h>

/* tensor kinds and parts, shared with awq_infer.h */
enum awq_tensor_kind {
  AWQ_T_WQKV = 0,    /* layer_{l}_wqkv.bin, [3H x H]          Inference.cu:780 */
  AWQ_T_WO = 1,      /* layer_{l}_wo.bin, [H x H]             Inference.cu:802 */
  AWQ_T_W1 = 2,      /* layer_{l}_w1.bin, [I x H]             Inference.cu:822 */
  AWQ_T_W2 = 3,      /* layer_{l}_w2.bin, [H x I]             Inference.cu:842 */
  AWQ_T_GAMMA = 4,   /* rms_norm_gamma_{l}.bin, [H] FP16      Inference.cu:856 */
  AWQ_T_EMBED = 5,   /* word_embedding.bin, [H x V]           Inference.cu:870 */
  AWQ_T_UNEMBED = 6  /* unembed.bin, [V x H]                  Inference.cu:891 */
};
enum awq_tensor_part { AWQ_P_PACKED = 0, AWQ_P_SCALE = 1, AWQ_P_ZP = 2 };
enum awq_synth_profile { AWQ_SYNTH_SPEC = 0, AWQ_SYNTH_BALANCED = 1 };

static inline uint64_t awq_synth_hash(uint64_t seed, uint64_t sid, uint64_t idx) {
  uint64_t z = seed * 0x9E3779B97F4A7C15ull + (sid + 1) * 0xD1B54A32D192ED03ull + idx * 0xA0761D6478BD642Full;
  z ^= z >> 30;
  z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27;
  z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

/* stream id of one stored array; layer is ignored for the two global tensors */
static inline uint64_t awq_synth_stream(int layer, int kind, int part) {
  uint64_t l = (kind == AWQ_T_EMBED || kind == AWQ_T_UNEMBED) ? 0u : (uint64_t)(layer + 1);
  return l * 64u + (uint64_t)kind * 4u + (uint64_t)part;
}

/* streams for things that are not stored tensors */
#define AWQ_SYNTH_STREAM_INPUT 0x100000ull  /* + any caller-chosen offset */

static inline float awq_synth_uniform(uint64_t h) { return (float)(h >> 40) * (1.0f / 16777216.0f); }

static inline double awq_synth_normal(uint64_t seed, uint64_t sid, uint64_t idx) {
  uint64_t a = awq_synth_hash(seed, sid, 2 * idx), b = awq_synth_hash(seed, sid, 2 * idx + 1);
  double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0,1] */
  double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);         /* [0,1) */
  return sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2);
}

#endif /* AWQ_SYNTH_H */
