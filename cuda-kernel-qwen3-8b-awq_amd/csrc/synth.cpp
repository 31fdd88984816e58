// Host-side synthetic data and the weight-directory writer (awq_synth.h).
#include <stdio.h>
#include <string.h>

#include <string>
#include <vector>

#include "common.hpp"
#include "engine.hpp"

static uint16_t to_half_bits(float f) {
  half_t h = (half_t)f;  // round to nearest even
  uint16_t u;
  memcpy(&u, &h, 2);
  return u;
}

extern "C" int awq_synth_fill(uint64_t seed, int layer, int kind, int part, void* host_dst, int64_t count) {
  return awq_synth_fill_profile(AWQ_SYNTH_SPEC, seed, layer, kind, part, host_dst, count);
}

extern "C" int awq_synth_fill_profile(int profile, uint64_t seed, int layer, int kind, int part, void* host_dst,
                                      int64_t count) {
  AWQ_REQUIRE(host_dst && count >= 0, "bad destination");
  AWQ_REQUIRE(profile == AWQ_SYNTH_SPEC || profile == AWQ_SYNTH_BALANCED, "bad profile");
  AWQ_REQUIRE(kind >= AWQ_T_WQKV && kind <= AWQ_T_UNEMBED, "bad tensor kind");
  const uint64_t sid = awq_synth_stream(layer, kind, part);
  if (kind == AWQ_T_GAMMA) {
    uint16_t* d = (uint16_t*)host_dst;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; ++i) d[i] = to_half_bits((float)(1.0 + 0.02 * awq_synth_normal(seed, sid, (uint64_t)i)));
    return AWQ_OK;
  }
  if (part == AWQ_P_PACKED) {
    uint8_t* d = (uint8_t*)host_dst;
    int64_t words = count / 8;
#pragma omp parallel for schedule(static)
    for (int64_t w = 0; w < words; ++w) {
      uint64_t h = awq_synth_hash(seed, sid, (uint64_t)w);
      memcpy(d + 8 * w, &h, 8);  // little endian: byte b of the word is bits 8b..8b+7
    }
    if (count % 8) {
      uint64_t h = awq_synth_hash(seed, sid, (uint64_t)words);
      memcpy(d + 8 * words, &h, (size_t)(count % 8));
    }
    return AWQ_OK;
  }
  uint16_t* d = (uint16_t*)host_dst;
  for (int64_t i = 0; i < count; ++i) {
    uint64_t h = awq_synth_hash(seed, sid, (uint64_t)i);
    if (part == AWQ_P_SCALE) {
      float u = awq_synth_uniform(h);
      float v = (profile == AWQ_SYNTH_BALANCED ? 0.0015f : 0.018f) * u;
      d[i] = to_half_bits((profile == AWQ_SYNTH_BALANCED ? 0.0025f : 0.002f) + v);
    } else {
      d[i] = to_half_bits(profile == AWQ_SYNTH_BALANCED ? (float)(7u + (unsigned)(h & 1u)) : (float)(h & 15u));
    }
  }
  return AWQ_OK;
}

extern "C" int awq_synth_normal_f16(uint64_t seed, uint64_t stream, uint16_t* host_dst, int64_t count, float mean,
                                    float std) {
  AWQ_REQUIRE(host_dst && count >= 0, "bad destination");
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < count; ++i)
    host_dst[i] = to_half_bits((float)((double)mean + (double)std * awq_synth_normal(seed, stream, (uint64_t)i)));
  return AWQ_OK;
}

extern "C" int awq_synth_tokens(uint64_t seed, uint64_t stream, int32_t* host_dst, int64_t count, int32_t vocab) {
  AWQ_REQUIRE(host_dst && count >= 0 && vocab > 0, "bad arguments");
  for (int64_t i = 0; i < count; ++i) host_dst[i] = (int32_t)(awq_synth_hash(seed, stream, (uint64_t)i) % (uint64_t)vocab);
  return AWQ_OK;
}

extern "C" int awq_rope_tables_host(uint16_t* cos_t, uint16_t* sin_t, int64_t max_pos) {
  AWQ_REQUIRE(cos_t && sin_t && max_pos > 0, "bad arguments");
  // Inference.cu:447-452, binary32 libm on the host as in the reference
#pragma omp parallel for schedule(static)
  for (int64_t pos = 0; pos < max_pos; ++pos) {
    for (int i = 0; i < AWQ_HEAD_DIM / 2; ++i) {
      float inv_freq = 1.0f / powf(10000.0f, (float)(2 * i) / (float)AWQ_HEAD_DIM);
      float angle = (float)pos * inv_freq;
      cos_t[pos * (AWQ_HEAD_DIM / 2) + i] = to_half_bits(cosf(angle));
      sin_t[pos * (AWQ_HEAD_DIM / 2) + i] = to_half_bits(sinf(angle));
    }
  }
  return AWQ_OK;
}

static int write_file(const std::string& path, const void* src, size_t bytes) {
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) {
    awq_set_error("could not create " + path);
    return AWQ_ERR_IO;
  }
  size_t put = fwrite(src, 1, bytes, f);
  fclose(f);
  if (put != bytes) {
    awq_set_error("short write to " + path);
    return AWQ_ERR_IO;
  }
  return AWQ_OK;
}

extern "C" int awq_write_weight_dir_profile(const char* dir, const awq_config* cfg_in, uint64_t seed, int profile) {
  AWQ_REQUIRE(dir != nullptr, "dir is NULL");
  awq_config cfg;
  if (cfg_in) cfg = *cfg_in;
  else awq_default_config(&cfg);
  if (int rc = awq_check_config(&cfg)) return rc;
  std::vector<uint8_t> buf;
  for (const WeightFile& wf : awq_weight_files(cfg)) {
    buf.resize((size_t)wf.bytes);
    int64_t count = (wf.part == AWQ_P_PACKED && wf.kind != AWQ_T_GAMMA) ? wf.bytes : wf.bytes / 2;
    if (int rc = awq_synth_fill_profile(profile, seed, wf.layer, wf.kind, wf.part, buf.data(), count)) return rc;
    if (int rc = write_file(std::string(dir) + "/" + wf.name, buf.data(), buf.size())) return rc;
  }
  return AWQ_OK;
}

extern "C" int awq_write_weight_dir(const char* dir, const awq_config* cfg_in, uint64_t seed) {
  return awq_write_weight_dir_profile(dir, cfg_in, seed, AWQ_SYNTH_SPEC);
}
