// Host side of the engine: the C ABI of include/awq_infer.h.
//
// Replaces class QWen3AWQInfer of the reference (Inference.cu:356-415):
// constructor (:422-470), loader (:766-903), runOneLayer (:1029-1230),
// sampleNextToken (:1235-1292) and generateResponse (:1297-1408), with all
// layers, the embedding and the unembedding on the current device, weights kept
// as packed int4, and no host round trip inside a step.
#include "engine.hpp"

#include <stdio.h>
#include <string.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <memory>
#include <mutex>
#include <thread>

static thread_local std::string g_last_error;
void awq_set_error(const std::string& msg) { g_last_error = msg; }
extern "C" const char* awq_last_error(void) { return g_last_error.c_str(); }

extern "C" void awq_default_config(awq_config* cfg) {
  cfg->n_layers = 36;      // Inference.cu:37
  cfg->hidden = 4096;      // :33
  cfg->inter = 12288;      // :34
  cfg->vocab = 151936;     // :38
  cfg->max_pos = 40960;    // :39
  cfg->split_idx = 18;     // :47
  cfg->eps = 1e-6f;        // :41
}

int awq_check_config(const awq_config* c) {
  AWQ_REQUIRE(c != nullptr, "config is NULL");
  AWQ_REQUIRE(c->n_layers >= 1 && c->n_layers <= 4096, "n_layers out of range");
  AWQ_REQUIRE(c->hidden >= 512 && c->hidden % 512 == 0, "hidden must be a positive multiple of 512");
  AWQ_REQUIRE(c->inter >= 512 && c->inter % 512 == 0, "inter must be a positive multiple of 512");
  AWQ_REQUIRE(c->vocab >= 128 && c->vocab % 128 == 0, "vocab must be a positive multiple of 128");
  AWQ_REQUIRE(c->max_pos >= 1 && c->max_pos <= 65536, "max_pos must be in 1..65536");
  AWQ_REQUIRE(c->split_idx >= 0 && c->split_idx <= c->n_layers, "split_idx out of range");
  AWQ_REQUIRE(c->eps > 0.0f, "eps must be positive");
  int C = awq_group_period(c->vocab, c->hidden);
  AWQ_REQUIRE((c->hidden / AWQ_BLOCK_K) % C == 0, "hidden/32 must be a multiple of the unembedding's scale-group period");
  return AWQ_OK;
}

void awq_tensor_dims(const awq_config& cfg, int kind, int64_t* out_dim, int64_t* in_dim) {
  const int64_t H = cfg.hidden, I = cfg.inter, V = cfg.vocab;
  switch (kind) {
    case AWQ_T_WQKV: *out_dim = 3 * H; *in_dim = H; break;  // Inference.cu:616
    case AWQ_T_WO: *out_dim = H; *in_dim = H; break;        // :630
    case AWQ_T_W1: *out_dim = I; *in_dim = H; break;        // :644
    case AWQ_T_W2: *out_dim = H; *in_dim = I; break;        // :658
    case AWQ_T_EMBED: *out_dim = H; *in_dim = V; break;     // :693
    case AWQ_T_UNEMBED: *out_dim = V; *in_dim = H; break;   // :708
    default: *out_dim = 0; *in_dim = 0;
  }
}

static int64_t part_bytes(const awq_config& cfg, int kind, int part) {
  if (kind == AWQ_T_GAMMA) return (int64_t)cfg.hidden * 2;
  int64_t o, i;
  awq_tensor_dims(cfg, kind, &o, &i);
  if (part == AWQ_P_PACKED) return o * ((i + 1) / 2);  // Inference.cu:775
  return (o / AWQ_GROUP_SIZE) * 2;                      // :776: out_dim/128 entries
}

std::vector<WeightFile> awq_weight_files(const awq_config& cfg) {
  std::vector<WeightFile> v;
  static const struct {
    int kind;
    const char *w, *s, *z;
  } per_layer[4] = {{AWQ_T_WQKV, "_wqkv.bin", "_bqkv_scale.bin", "_bqkv_zp.bin"},  // Inference.cu:780-790
                    {AWQ_T_WO, "_wo.bin", "_wo_scale.bin", "_wo_zp.bin"},            // :802-810
                    {AWQ_T_W1, "_w1.bin", "_w1_scale.bin", "_w1_zp.bin"},            // :822-830
                    {AWQ_T_W2, "_w2.bin", "_w2_scale.bin", "_w2_zp.bin"}};           // :842-850
  for (int l = 0; l < cfg.n_layers; ++l) {
    std::string p = "layer_" + std::to_string(l);
    for (const auto& t : per_layer) {
      v.push_back({p + t.w, l, t.kind, AWQ_P_PACKED, part_bytes(cfg, t.kind, AWQ_P_PACKED)});
      v.push_back({p + t.s, l, t.kind, AWQ_P_SCALE, part_bytes(cfg, t.kind, AWQ_P_SCALE)});
      v.push_back({p + t.z, l, t.kind, AWQ_P_ZP, part_bytes(cfg, t.kind, AWQ_P_ZP)});
    }
    v.push_back({"rms_norm_gamma_" + std::to_string(l) + ".bin", l, AWQ_T_GAMMA, 0, part_bytes(cfg, AWQ_T_GAMMA, 0)});  // :856
  }
  v.push_back({"word_embedding.bin", 0, AWQ_T_EMBED, AWQ_P_PACKED, part_bytes(cfg, AWQ_T_EMBED, AWQ_P_PACKED)});  // :870
  v.push_back({"word_embed_scale.bin", 0, AWQ_T_EMBED, AWQ_P_SCALE, part_bytes(cfg, AWQ_T_EMBED, AWQ_P_SCALE)});
  v.push_back({"word_embed_zp.bin", 0, AWQ_T_EMBED, AWQ_P_ZP, part_bytes(cfg, AWQ_T_EMBED, AWQ_P_ZP)});
  v.push_back({"unembed.bin", 0, AWQ_T_UNEMBED, AWQ_P_PACKED, part_bytes(cfg, AWQ_T_UNEMBED, AWQ_P_PACKED)});     // :891
  v.push_back({"unembed_scale.bin", 0, AWQ_T_UNEMBED, AWQ_P_SCALE, part_bytes(cfg, AWQ_T_UNEMBED, AWQ_P_SCALE)});
  v.push_back({"unembed_zp.bin", 0, AWQ_T_UNEMBED, AWQ_P_ZP, part_bytes(cfg, AWQ_T_UNEMBED, AWQ_P_ZP)});
  return v;
}

extern "C" int awq_validate_weight_dir(const char* dir, const awq_config* cfg_in) {
  AWQ_REQUIRE(dir != nullptr, "dir is NULL");
  awq_config cfg;
  if (cfg_in) cfg = *cfg_in;
  else awq_default_config(&cfg);
  if (int rc = awq_check_config(&cfg)) return rc;
  for (const WeightFile& wf : awq_weight_files(cfg)) {
    std::string path = std::string(dir) + "/" + wf.name;
    struct stat st;
    if (stat(path.c_str(), &st) != 0 || !S_ISREG(st.st_mode)) {
      awq_set_error("could not open " + path);  // Inference.cu:299-302
      return AWQ_ERR_IO;
    }
    if ((int64_t)st.st_size < wf.bytes) {
      awq_set_error("read failed for " + path + ": " + std::to_string((long long)st.st_size) + " bytes, need " +
                    std::to_string((long long)wf.bytes));  // :305-308
      return AWQ_ERR_IO;
    }
  }
  return AWQ_OK;
}

// ---------------------------------------------------------------------------

namespace {

struct DevLinear {
  uint8_t* packed = nullptr;  // file order; freed after reordering except for the embedding
  void* stream_order = nullptr;
  half_t* scale = nullptr;
  half_t* zp = nullptr;
  int64_t m = 0, k = 0;
  int zp_integral = 0;
  bool have[3] = {false, false, false};
  bool reordered = false;  // stream_order already holds the reordered copy (the directory loader does it on the fly)
};

struct LayerDev {
  DevLinear wqkv, wo, w1, w2;
  half_t* gamma = nullptr;
  bool have_gamma = false;
  half_t* kcache = nullptr;
  half_t* vcache = nullptr;
  // the first parts_pos positions of both a second time, in the order the fused Wqkv + attention launch reads them
  half_t* kparts = nullptr;
  half_t* vparts = nullptr;
};

}  // namespace

struct awq_engine {
  awq_config cfg;
  int n_heads = 0;
  int device = 0;
  hipStream_t stream = nullptr;
  std::vector<LayerDev> layers;
  DevLinear embed, unembed;
  half_t *cos_t = nullptr, *sin_t = nullptr;
  // activations (Inference.cu:334-348)
  half_t *hidden = nullptr, *q = nullptr, *ctx = nullptr, *mid = nullptr, *logits = nullptr;
  half_t* hidden_last = nullptr;  // the last layer's output of the latest generation step (hidden then holds the next input)
  // workspaces
  void* attn_ws = nullptr;
  void* sample_ws = nullptr;  // best candidate and workgroup counts of the sampling launch
  uint8_t* embed_rows = nullptr;  // the embedding transposed into token rows, for the sampling launch's gather
  StepState* d_state = nullptr;
  int32_t* d_token = nullptr;
  int32_t* d_out = nullptr;
  // sequence state
  int current_seq_len = 0;  // current_seq_len_ of Inference.cu:408
  int n_positions = 0;      // forward passes since reset
  int n_generated = 0;
  bool finalized = false;
  bool graph_mode = true;
  hipGraphExec_t graphs[3][7] = {};  // [prompt | generation step | kStepsPerGraph generation steps][length bound]
  // activations of the batched prompt pass, [chunk][n] each; allocated at first use
  struct {
    half_t *hidden = nullptr, *norm = nullptr, *qkv = nullptr, *q = nullptr, *ctx = nullptr, *mid = nullptr;
    int32_t* tokens = nullptr;
    void* gemm_ws = nullptr;  // partial sums of products whose k is cut over workgroups
    int64_t chunk = 0;
  } pb;
  bool batched_prefill = false;
  // Wo and W1 of a layer as one launch (fused.hip): the hidden state between them as tagged words, and the word
  // through which a wait that gave up reports
  bool fused = false;
  uint32_t* hid_tag = nullptr;
  // Wqkv and the attention of a layer as one launch (qkv_attn.hip): the partial scores as tagged words, handed
  // between the eight workgroups of a head
  bool fused_qkv = false;
  bool handover_gave_up = false;  // a fused launch's wait gave up since awq_generate last cleared this
  bool giveup_after_reset = false;  // test hook: the next awq_reset leaves the status word set
  uint32_t* score_tag = nullptr;
  int parts_pos = 0;  // positions the layers' parts arrays hold (0: none allocated, the launch is not available)
  int32_t* handover_status = nullptr;
  int32_t epoch_next = 0;  // the epoch of the next step (mirrors what the device adds per step)
  std::vector<void*> allocations;
  // the reordered weight streams of all layers and the unembedding share one allocation, in the order the
  // decode step reads them
  char* stream_slab = nullptr;
  int64_t slab_used = 0, slab_size = 0;
};

namespace {

int dev_alloc(awq_engine* e, void** p, int64_t bytes) {
  AWQ_HIP_TRY(hipMalloc(p, (size_t)(bytes > 0 ? bytes : 4)));
  e->allocations.push_back(*p);
  return AWQ_OK;
}

// Room for one reordered weight stream.  One allocation for all of them (3.3 GB for the reference model) instead
// of one per matrix: measured 0.5 % on the decode rate (fewer, larger pages for the address translation to hold).
int stream_alloc(awq_engine* e, void** p, int64_t bytes) {
  const auto pad = [](int64_t b) { return (b + 4095) & ~4095ll; };
  if (!e->stream_slab) {
    const int64_t H = e->cfg.hidden, I = e->cfg.inter, V = e->cfg.vocab;
    const int64_t total = e->cfg.n_layers * (pad(3 * H * H / 2) + pad(H * H / 2) + 2 * pad(I * H / 2)) + pad(V * H / 2);
    if (int rc = dev_alloc(e, (void**)&e->stream_slab, total)) return rc;
    e->slab_size = total;
  }
  if (e->slab_used + pad(bytes) > e->slab_size) return dev_alloc(e, p, bytes);  // not one of the model's own matrices
  *p = e->stream_slab + e->slab_used;
  e->slab_used += pad(bytes);
  return AWQ_OK;
}

int dev_free(awq_engine* e, void* p) {
  for (auto& a : e->allocations)
    if (a == p) {
      a = nullptr;
      AWQ_HIP_TRY(hipFree(p));
      return AWQ_OK;
    }
  return AWQ_OK;
}

DevLinear* find_linear(awq_engine* e, int layer, int kind) {
  if (kind == AWQ_T_EMBED) return &e->embed;
  if (kind == AWQ_T_UNEMBED) return &e->unembed;
  if (layer < 0 || layer >= e->cfg.n_layers) return nullptr;
  switch (kind) {
    case AWQ_T_WQKV: return &e->layers[layer].wqkv;
    case AWQ_T_WO: return &e->layers[layer].wo;
    case AWQ_T_W1: return &e->layers[layer].w1;
    case AWQ_T_W2: return &e->layers[layer].w2;
  }
  return nullptr;
}

// with_packed false: the file-order bytes of this tensor never rest on the device (the directory loader reorders
// them out of a staging buffer)
int alloc_linear(awq_engine* e, DevLinear& t, int kind, bool with_packed = true) {
  awq_tensor_dims(e->cfg, kind, &t.m, &t.k);
  if (with_packed)
    if (int rc = dev_alloc(e, (void**)&t.packed, part_bytes(e->cfg, kind, AWQ_P_PACKED))) return rc;
  if (int rc = dev_alloc(e, (void**)&t.scale, part_bytes(e->cfg, kind, AWQ_P_SCALE))) return rc;
  if (int rc = dev_alloc(e, (void**)&t.zp, part_bytes(e->cfg, kind, AWQ_P_ZP))) return rc;
  return AWQ_OK;
}

bool zp_all_integral(const uint16_t* zp, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    half_t h;
    memcpy(&h, &zp[i], 2);
    float f = (float)h;
    if (!(f >= 0.0f && f <= 1024.0f) || f != (float)(int)f) return false;
  }
  return true;
}

// one fused-linear launch on the engine's stream
LinearArgs linear_args(awq_engine* e, const DevLinear& t, const half_t* x, half_t* y) {
  LinearArgs a;
  a.wq = t.stream_order;
  a.scale = t.scale;
  a.zp = t.zp;
  a.x = x;
  a.y = y;
  a.m = t.m;
  a.k = t.k;
  a.eps = e->cfg.eps;
  a.dyn = e->d_state;
  return a;
}

// runOneLayer, Inference.cu:1029-1230, as five launches.  The position and the
// attended length come from the device-side step state.
// :1040 RMSNorm, :1052 Wqkv, :1070-1103 split + rotary + KV append of layer l
int enqueue_wqkv(awq_engine* e, int l) {
  LayerDev& L = e->layers[l];
  LinearArgs a = linear_args(e, L.wqkv, e->hidden, e->q);
  a.prologue = PRO_RMSNORM;
  a.gamma = L.gamma;
  a.epilogue = EPI_QKV_ROPE;
  a.cos_t = e->cos_t;
  a.sin_t = e->sin_t;
  a.k_cache = L.kcache;
  a.v_cache = L.vcache;
  a.hidden = e->cfg.hidden;
  a.max_pos = e->cfg.max_pos;
  a.kv = kv_blocked(e->n_heads);
  return launch_gemv(a, e->stream);
}

int enqueue_layer(awq_engine* e, int l, int use_len_hi, int64_t len_bound) {
  LayerDev& L = e->layers[l];
  hipStream_t st = e->stream;
  if (e->fused_qkv && len_bound <= e->parts_pos) {  // :1040-1110 in one launch
    if (int rc = launch_fused_qkv_attn(L.wqkv.stream_order, L.wqkv.scale, L.wqkv.zp, L.wqkv.m, e->hidden, L.gamma,
                                       e->cfg.eps, e->cos_t, e->sin_t, L.kcache, L.vcache, kv_blocked(e->n_heads),
                                       L.kparts, L.vparts, e->parts_pos, e->q, e->ctx, e->score_tag,
                                       e->handover_status, e->d_state, l,
                                       use_len_hi, len_bound, e->n_heads, nullptr, st))
      return rc;
  } else {
    if (int rc = enqueue_wqkv(e, l)) return rc;
    if (int rc = launch_attention(e->q, L.kcache, L.vcache, e->ctx, e->n_heads, e->cfg.max_pos,
                                  kv_blocked(e->n_heads), 0, e->d_state,
                                  use_len_hi, len_bound, e->attn_ws, st))
      return rc;  // :1110
  }
  if (e->fused) {  // :1128-1198 in one launch
    if (int rc = launch_fused_wo_w1(L.wo.stream_order, L.wo.scale, L.wo.zp, L.w1.stream_order, L.w1.scale, L.w1.zp,
                                    L.gamma, e->cfg.eps, e->ctx, e->hidden, e->mid, e->hid_tag, e->handover_status,
                                    e->d_state, l, e->cfg.hidden, e->cfg.inter, nullptr, st))
      return rc;
  } else {
    {  // :1128-1155 Wo product and residual add; input and output are distinct
       // buffers (they alias in the reference)
      LinearArgs a = linear_args(e, L.wo, e->ctx, e->hidden);
      a.epilogue = EPI_RESIDUAL;
      a.res = e->hidden;
      if (int rc = launch_gemv(a, st)) return rc;
    }
    {  // :1163 RMSNorm with the same gamma, :1176 W1, :1196 GeLU
      LinearArgs a = linear_args(e, L.w1, e->hidden, e->mid);
      a.prologue = PRO_RMSNORM;
      a.gamma = L.gamma;
      a.epilogue = EPI_GELU;
      if (int rc = launch_gemv(a, st)) return rc;
    }
  }
  {  // :1201 W2, :1227 residual add
    LinearArgs a = linear_args(e, L.w2, e->mid, e->hidden);
    a.epilogue = EPI_RESIDUAL;
    a.res = e->hidden;
    if (int rc = launch_gemv(a, st)) return rc;
  }
  return AWQ_OK;
}

// sampleNextToken, Inference.cu:1235-1292: final RMSNorm (gamma of the last
// layer), unembedding and greedy argmax in one launch
LinearArgs sample_args(awq_engine* e) {
  const int NL = e->cfg.n_layers;
  LinearArgs a = linear_args(e, e->unembed, e->hidden, e->logits);
  a.prologue = PRO_RMSNORM;
  a.gamma = e->layers[NL - 1].gamma;
  a.epilogue = EPI_ARGMAX;
  a.best = (unsigned long long*)e->sample_ws;
  a.out_token = e->d_token;
  a.out_array = e->d_out;
  // the launch also ends the step: the sampled token's embedding becomes the next input (:1384-1398)
  a.fin_hidden = e->hidden;
  a.fin_hidden_last = e->hidden_last;
  a.fin_emb = e->embed_rows;
  a.fin_emb_scale = e->embed.scale;
  a.fin_emb_zp = e->embed.zp;
  a.fin_n = e->cfg.hidden;
  a.fin_state = e->d_state;
  a.fin_epoch_step = e->cfg.n_layers;
  return a;
}

int enqueue_sample(awq_engine* e) { return launch_gemv(sample_args(e), e->stream); }

// everything of one position after the step state has been written
int enqueue_step_body(awq_engine* e, bool gen, int64_t len_bound) {
  // Prompt positions gather their token's embedding (Inference.cu:1310-1324).  A generation step starts
  // from the hidden state as it stands: the last layer's output after the prompt (:1357), afterwards the
  // embedding that the previous step's sampling launch gathered (:1384-1398).
  if (!gen)
    if (int rc = launch_embed(e->embed.packed, e->embed.scale, e->embed.zp, e->cfg.hidden, e->cfg.vocab, 0,
                              e->d_state, e->hidden, e->stream))
      return rc;
  const int split = gen ? e->cfg.split_idx : 1;
  for (int l = 0; l < e->cfg.n_layers; ++l)
    if (int rc = enqueue_layer(e, l, l >= split, len_bound)) return rc;
  if (gen) return enqueue_sample(e);
  return AWQ_OK;
}

// the attention launches are specialised by an upper bound of the attended length (one workgroup per head, or two
// to four launches cut along the sequence; the fused launch's chunks per wavefront); one captured graph per bound
constexpr int64_t kLengthBounds[7] = {kAttnShortMax, kAttnOneWorkgroupMax, kAttnTwoLaunchMax, kAttnMergedMax, 3072, kFusedQkvAttnMax, 1 << 30};
static_assert(kFusedQkvAttnMax == 4096, "the fused launch's instances: three chunks of 64 positions per wavefront up to 3072 positions, four beyond");
int length_bucket(int64_t len) {
  int bucket = 0;
  while (len > kLengthBounds[bucket]) ++bucket;
  return bucket;
}
constexpr int kStepsPerGraph = 4;

int build_graph(awq_engine* e, bool gen, int64_t len_bound, hipGraphExec_t* out, int n_steps = 1) {
  hipGraph_t graph = nullptr;
  AWQ_HIP_TRY(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
  int rc = 0;
  for (int i = 0; i < n_steps && !rc; ++i) rc = enqueue_step_body(e, gen, len_bound);
  hipError_t err = hipStreamEndCapture(e->stream, &graph);
  if (rc) {
    if (graph) hipGraphDestroy(graph);
    return rc;
  }
  AWQ_HIP_TRY(err);
  AWQ_HIP_TRY(hipGraphInstantiate(out, graph, nullptr, nullptr, 0));
  AWQ_HIP_TRY(hipGraphDestroy(graph));
  return AWQ_OK;
}

// `write_state` false: the device already holds `s` (the previous generation step advanced it)
int run_step(awq_engine* e, bool gen, StepState s, bool write_state = true, int n_steps = 1) {
  s.epoch = e->epoch_next;
  for (int i = 0; i < n_steps; ++i)
    e->epoch_next = (e->epoch_next + e->cfg.n_layers) & 0x3fffffff;  // what the step's last launch adds on the device
  if (write_state)
    if (int rc = launch_set_state(e->d_state, s, e->stream)) return rc;
  const int bucket = length_bucket(s.len_hi);
  const int64_t len_bound = kLengthBounds[bucket] < e->cfg.max_pos ? kLengthBounds[bucket] : e->cfg.max_pos;
  if (e->graph_mode) {
    hipGraphExec_t* g = &e->graphs[n_steps > 1 ? 2 : (gen ? 1 : 0)][bucket];
    if (!*g)
      if (int rc = build_graph(e, gen, len_bound, g, n_steps)) return rc;
    AWQ_HIP_TRY(hipGraphLaunch(*g, e->stream));
    return AWQ_OK;
  }
  return enqueue_step_body(e, gen, len_bound);
}

// readBinaryFileToDevice's host half (Inference.cu:297-308): exactly `bytes` bytes of the file (more are
// ignored, fewer are an error).  A large file is read by four threads, a quarter each: one thread copies
// out of the page cache at 8-10 GB/s, well below what the copy to the device takes.
int read_file(const std::string& path, int64_t bytes, void* dst, std::string* err) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) {
    *err = "could not open " + path;  // Inference.cu:299-302
    return AWQ_ERR_IO;
  }
  auto read_range = [fd, dst](int64_t from, int64_t to) {
    while (from < to) {
      const ssize_t got = pread(fd, (char*)dst + from, (size_t)(to - from), (off_t)from);
      if (got <= 0) return false;  // end of file or an error: the file is short
      from += got;
    }
    return true;
  };
  // from a cold disk: have the whole range scheduled as one sequential read before four threads ask for
  // quarters of it (no effect on cached files)
  (void)posix_fadvise(fd, 0, (off_t)bytes, POSIX_FADV_WILLNEED);
  bool ok = true;
  constexpr int64_t kParallelFrom = 8ll << 20;
  constexpr int kReaders = 4;
  if (bytes >= kParallelFrom) {
    bool part_ok[kReaders];
    std::thread helper[kReaders - 1];
    const int64_t piece = ((bytes / kReaders) + 4095) & ~4095ll;
    for (int i = 1; i < kReaders; ++i)
      helper[i - 1] = std::thread([&, i] { part_ok[i] = read_range(std::min(bytes, i * piece), std::min(bytes, (i + 1) * piece)); });
    part_ok[0] = read_range(0, std::min(bytes, piece));
    for (auto& h : helper) h.join();
    for (bool p_ok : part_ok) ok = ok && p_ok;
  } else {
    ok = read_range(0, bytes);
  }
  close(fd);
  if (!ok) {
    *err = "read failed for " + path;  // :305-308
    return AWQ_ERR_IO;
  }
  return AWQ_OK;
}

// Reorders one linear layer on the engine's stream right after its packed bytes were copied.
int reorder_now(awq_engine* e, DevLinear* t) {
  if (int rc = stream_alloc(e, &t->stream_order, t->m * (t->k / 2))) return rc;
  if (int rc = launch_repack(t->packed, t->stream_order, t->m, t->k, e->stream)) return rc;
  t->reordered = true;
  return AWQ_OK;
}

thread_local double g_last_load_seconds = 0.0;

}  // namespace

namespace {
int create_engine(const awq_config* cfg_in, awq_engine** out, bool packed_on_device);
}
extern "C" int awq_create_empty(const awq_config* cfg_in, awq_engine** out) {
  return create_engine(cfg_in, out, true);
}
namespace {
// packed_on_device: every linear layer gets a device buffer for its file-order bytes (awq_upload fills it,
// awq_finalize reorders it and frees it); without, only the embedding does (it is gathered from in file order)
int create_engine(const awq_config* cfg_in, awq_engine** out, bool packed_on_device) {
  AWQ_REQUIRE(out != nullptr, "out is NULL");
  *out = nullptr;
  awq_config cfg;
  if (cfg_in) cfg = *cfg_in;
  else awq_default_config(&cfg);
  if (int rc = awq_check_config(&cfg)) return rc;
  int ndev = 0;
  AWQ_HIP_TRY(hipGetDeviceCount(&ndev));
  if (ndev < 1) {
    awq_set_error("no HIP device found");
    return AWQ_ERR_HIP;
  }
  std::unique_ptr<awq_engine> e(new awq_engine());
  e->cfg = cfg;
  e->n_heads = cfg.hidden / AWQ_HEAD_DIM;
  AWQ_HIP_TRY(hipGetDevice(&e->device));
  AWQ_HIP_TRY(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
  e->layers.resize(cfg.n_layers);
  awq_engine* ep = e.get();
  auto fail = [&](int rc) {
    awq_destroy(e.release());
    return rc;
  };
  const int64_t H = cfg.hidden, I = cfg.inter, V = cfg.vocab;
  // Inference.cu:676; the rows are kept in blocks of 64 positions here (see KvLayout), so whole blocks
  // are allocated
  const int64_t kv_bytes = (int64_t)e->n_heads * ((cfg.max_pos + 63) / 64 * 64) * AWQ_HEAD_DIM * 2;
  for (int l = 0; l < cfg.n_layers; ++l) {
    LayerDev& L = e->layers[l];
    if (int rc = alloc_linear(ep, L.wqkv, AWQ_T_WQKV, packed_on_device)) return fail(rc);
    if (int rc = alloc_linear(ep, L.wo, AWQ_T_WO, packed_on_device)) return fail(rc);
    if (int rc = alloc_linear(ep, L.w1, AWQ_T_W1, packed_on_device)) return fail(rc);
    if (int rc = alloc_linear(ep, L.w2, AWQ_T_W2, packed_on_device)) return fail(rc);
    if (int rc = dev_alloc(ep, (void**)&L.gamma, H * 2)) return fail(rc);
    if (int rc = dev_alloc(ep, (void**)&L.kcache, kv_bytes)) return fail(rc);
    if (int rc = dev_alloc(ep, (void**)&L.vcache, kv_bytes)) return fail(rc);
  }
  if (int rc = alloc_linear(ep, e->embed, AWQ_T_EMBED)) return fail(rc);
  if (int rc = alloc_linear(ep, e->unembed, AWQ_T_UNEMBED, packed_on_device)) return fail(rc);
  const int64_t table_bytes = (int64_t)cfg.max_pos * (AWQ_HEAD_DIM / 2) * 2;
  if (int rc = dev_alloc(ep, (void**)&e->cos_t, table_bytes)) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->sin_t, table_bytes)) return fail(rc);
  struct {
    half_t** p;
    int64_t n;
  } acts[] = {{&e->hidden, H}, {&e->hidden_last, H}, {&e->q, H}, {&e->ctx, H}, {&e->mid, I}, {&e->logits, V}};
  for (auto& a : acts)
    if (int rc = dev_alloc(ep, (void**)a.p, a.n * 2)) return fail(rc);
  if (int rc = dev_alloc(ep, &e->attn_ws, attention_workspace_bytes(e->n_heads, cfg.max_pos))) return fail(rc);
  if (int rc = dev_alloc(ep, &e->sample_ws, gemv_workspace_bytes(V, H))) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->embed_rows, V * (H / 2))) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->d_state, sizeof(StepState))) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->d_token, 4)) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->d_out, (int64_t)cfg.max_pos * 4)) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->hid_tag, H * 4)) return fail(rc);
  if (int rc = dev_alloc(ep, (void**)&e->handover_status, 256)) return fail(rc);
  const int64_t xch_bytes = fused_qkv_attn_exchange_bytes(e->n_heads);
  if (int rc = dev_alloc(ep, (void**)&e->score_tag, xch_bytes)) return fail(rc);
  // tags start at 0 (Wo + W1) resp. never are 0 (Wqkv + attention): the vectors must not hold a launch's tag
  // before the launch wrote it
  if (hipMemset(e->hid_tag, 0xff, (size_t)H * 4) != hipSuccess || hipMemset(e->handover_status, 0, 256) != hipSuccess ||
      hipMemset(e->score_tag, 0, (size_t)xch_bytes) != hipSuccess) {
    awq_set_error("hipMemset of the hand-over buffers failed");
    return fail(AWQ_ERR_HIP);
  }
  e->fused = false;  // measured slower than two launches (904 against 924 tok/s): awq_set_fused_mode switches it on
  // Wqkv + attention as one launch where the device can run it (992 against 966 tok/s); awq_set_fused_mode(e, 0)
  // switches it off.  The launch reads the caches from a second copy in its own order.
  e->fused_qkv = cfg.hidden / AWQ_HEAD_DIM == e->n_heads && fused_qkv_attn_supported(cfg.hidden, e->n_heads, e->stream) != 0;
  if (e->fused_qkv) {
    e->parts_pos = (int)std::min<int64_t>((cfg.max_pos + 63) / 64 * 64, kFusedQkvAttnMax);
    const int64_t parts_bytes = fused_qkv_attn_parts_bytes(e->n_heads, e->parts_pos);
    for (auto& L : e->layers) {
      if (int rc = dev_alloc(ep, (void**)&L.kparts, parts_bytes)) return fail(rc);
      if (int rc = dev_alloc(ep, (void**)&L.vparts, parts_bytes)) return fail(rc);
    }
  }
  *out = e.release();
  return AWQ_OK;
}
}  // namespace

extern "C" int awq_upload(awq_engine* e, int layer, int kind, int part, const void* host_src, int64_t bytes) {
  AWQ_REQUIRE(e && host_src, "NULL argument");
  if (e->finalized) {
    awq_set_error("awq_upload after awq_finalize");
    return AWQ_ERR_STATE;
  }
  AWQ_REQUIRE(kind >= AWQ_T_WQKV && kind <= AWQ_T_UNEMBED, "bad tensor kind");
  int64_t need = part_bytes(e->cfg, kind, part);
  AWQ_REQUIRE(bytes == need, "byte count " + std::to_string((long long)bytes) + " != expected " +
                                 std::to_string((long long)need));
  if (kind == AWQ_T_GAMMA) {
    AWQ_REQUIRE(layer >= 0 && layer < e->cfg.n_layers, "layer out of range");
    AWQ_HIP_TRY(hipMemcpy(e->layers[layer].gamma, host_src, (size_t)bytes, hipMemcpyHostToDevice));  // :309
    e->layers[layer].have_gamma = true;
    return AWQ_OK;
  }
  AWQ_REQUIRE(part >= AWQ_P_PACKED && part <= AWQ_P_ZP, "bad tensor part");
  DevLinear* t = find_linear(e, layer, kind);
  AWQ_REQUIRE(t != nullptr, "layer out of range");
  void* dst = part == AWQ_P_PACKED ? (void*)t->packed : part == AWQ_P_SCALE ? (void*)t->scale : (void*)t->zp;
  AWQ_HIP_TRY(hipMemcpy(dst, host_src, (size_t)bytes, hipMemcpyHostToDevice));
  if (part == AWQ_P_ZP) t->zp_integral = zp_all_integral((const uint16_t*)host_src, bytes / 2);
  t->have[part] = true;
  return AWQ_OK;
}

extern "C" int awq_finalize(awq_engine* e) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  if (e->finalized) return AWQ_OK;
  // everything uploaded?
  for (int l = 0; l < e->cfg.n_layers; ++l) {
    LayerDev& L = e->layers[l];
    DevLinear* ts[4] = {&L.wqkv, &L.wo, &L.w1, &L.w2};
    for (DevLinear* t : ts)
      if (!(t->have[0] && t->have[1] && t->have[2])) {
        awq_set_error("layer " + std::to_string(l) + " has tensors that were never uploaded");
        return AWQ_ERR_STATE;
      }
    if (!L.have_gamma) {
      awq_set_error("gamma of layer " + std::to_string(l) + " was never uploaded");
      return AWQ_ERR_STATE;
    }
  }
  for (DevLinear* t : {&e->embed, &e->unembed})
    if (!(t->have[0] && t->have[1] && t->have[2])) {
      awq_set_error("embedding or unembedding was never uploaded");
      return AWQ_ERR_STATE;
    }
  hipStream_t st = e->stream;
  // reorder every linear layer's stream; the file-order copy is then dropped.
  // The embedding is only ever gathered from, so it stays in file order.
  std::vector<DevLinear*> all;
  for (auto& L : e->layers) {
    all.push_back(&L.wqkv);
    all.push_back(&L.wo);
    all.push_back(&L.w1);
    all.push_back(&L.w2);
  }
  all.push_back(&e->unembed);
  for (DevLinear* t : all)
    if (!t->reordered) {
      if (int rc = stream_alloc(e, &t->stream_order, t->m * (t->k / 2))) return rc;
      if (int rc = launch_repack(t->packed, t->stream_order, t->m, t->k, st)) return rc;
      t->reordered = true;
    }
  AWQ_HIP_TRY(hipStreamSynchronize(st));
  for (DevLinear* t : all)
    if (t->packed) {
      if (int rc = dev_free(e, t->packed)) return rc;
      t->packed = nullptr;
    }
  // rotary tables, Inference.cu:443-464
  {
    std::vector<uint16_t> c((size_t)e->cfg.max_pos * 64), s(c.size());
    if (int rc = awq_rope_tables_host(c.data(), s.data(), e->cfg.max_pos)) return rc;
    AWQ_HIP_TRY(hipMemcpy(e->cos_t, c.data(), c.size() * 2, hipMemcpyHostToDevice));
    AWQ_HIP_TRY(hipMemcpy(e->sin_t, s.data(), s.size() * 2, hipMemcpyHostToDevice));
  }
  // zero the KV caches (Inference.cu:431-437) and the self-resetting workspaces
  const int64_t kv_bytes = (int64_t)e->n_heads * ((e->cfg.max_pos + 63) / 64 * 64) * AWQ_HEAD_DIM * 2;
  for (auto& L : e->layers) {
    if (int rc = launch_fill_zero(L.kcache, kv_bytes, st)) return rc;
    if (int rc = launch_fill_zero(L.vcache, kv_bytes, st)) return rc;
    if (L.kparts) {
      const int64_t parts_bytes = fused_qkv_attn_parts_bytes(e->n_heads, e->parts_pos);
      if (int rc = launch_fill_zero(L.kparts, parts_bytes, st)) return rc;
      if (int rc = launch_fill_zero(L.vparts, parts_bytes, st)) return rc;
    }
  }
  if (int rc = launch_fill_zero(e->sample_ws, gemv_workspace_bytes(e->cfg.vocab, e->cfg.hidden), st)) return rc;
  if (int rc = launch_embed_rows((const uint8_t*)e->embed.packed, e->embed_rows, e->cfg.hidden, e->cfg.vocab, st)) return rc;
  if (int rc = launch_fill_zero(e->d_token, 4, st)) return rc;
  if (int rc = launch_fill_zero(e->hidden, (int64_t)e->cfg.hidden * 2, st)) return rc;
  AWQ_HIP_TRY(hipStreamSynchronize(st));
  e->finalized = true;
  return awq_reset(e);
}

extern "C" double awq_last_load_seconds(void) { return g_last_load_seconds; }

// Constructor with the loader of Inference.cu:766-903.  Three stages overlap: a reader thread fills
// two pinned buffers in turn (four threads on a large file), this thread sends a full buffer to the device (hipMemcpyAsync
// on the engine's stream) and, for the packed bytes of a linear layer, queues its reordering behind
// the copy; a buffer goes back to the reader once its copy has completed.
extern "C" int awq_create(const char* weight_dir, const awq_config* cfg_in, awq_engine** out) {
  AWQ_REQUIRE(weight_dir != nullptr && out != nullptr, "NULL argument");
  *out = nullptr;
  // look at the directory before touching the GPU
  if (int rc = awq_validate_weight_dir(weight_dir, cfg_in)) return rc;
  awq_engine* e = nullptr;
  if (int rc = create_engine(cfg_in, &e, false)) return rc;
  const std::vector<WeightFile> files = awq_weight_files(e->cfg);
  int64_t largest = 0, largest_reordered = 0;
  for (const WeightFile& wf : files) {
    largest = std::max(largest, wf.bytes);
    if (wf.part == AWQ_P_PACKED && wf.kind != AWQ_T_EMBED && wf.kind != AWQ_T_GAMMA)
      largest_reordered = std::max(largest_reordered, wf.bytes);
  }
  // The file-order bytes of a linear layer pass through one of two device buffers on their way into the
  // reordered stream: the engine's stream runs copy, reorder, copy, reorder, ... in order, so a buffer is free
  // again when its turn comes two matrices later.  (One device buffer per matrix, freed after the last
  // reordering, held a second copy of all weights until the end of the load.)
  void* dstage[2] = {nullptr, nullptr};
  int n_staged = 0;
  const auto t_begin = std::chrono::steady_clock::now();

  struct Slot {
    void* host = nullptr;      // pinned
    hipEvent_t copied = nullptr;
    int file = -1;             // index of the file it holds
    int state = 0;             // 0 free for the reader, 1 full, 2 copy in flight
    int rc = AWQ_OK;
    std::string err;
  } slot[2];
  std::mutex mu;
  std::condition_variable cv;
  bool stop = false;
  int rc = AWQ_OK;
  for (void*& d : dstage)
    if (rc == AWQ_OK && hipMalloc(&d, (size_t)std::max<int64_t>(largest_reordered, 4)) != hipSuccess) {
      awq_set_error("hipMalloc of a device staging buffer failed");
      rc = AWQ_ERR_HIP;
    }
  for (Slot& s : slot) {
    if (rc == AWQ_OK && hipHostMalloc(&s.host, (size_t)largest, hipHostMallocDefault) != hipSuccess) {
      awq_set_error("hipHostMalloc of a staging buffer failed");
      rc = AWQ_ERR_HIP;
    }
    if (rc == AWQ_OK && hipEventCreateWithFlags(&s.copied, hipEventDisableTiming) != hipSuccess) {
      awq_set_error("hipEventCreate failed");
      rc = AWQ_ERR_HIP;
    }
  }
  std::thread reader;
  if (rc == AWQ_OK) {
    reader = std::thread([&]() {
      for (size_t i = 0; i < files.size(); ++i) {
        Slot& s = slot[i & 1];
        {
          std::unique_lock<std::mutex> lock(mu);
          cv.wait(lock, [&] { return s.state == 0 || stop; });
          if (stop) return;
        }
        std::string err;
        int frc = read_file(std::string(weight_dir) + "/" + files[i].name, files[i].bytes, s.host, &err);
        {
          std::lock_guard<std::mutex> lock(mu);
          s.file = (int)i;
          s.rc = frc;
          s.err = err;
          s.state = 1;
        }
        cv.notify_all();
        if (frc) return;
      }
    });
    for (size_t i = 0; i < files.size() && rc == AWQ_OK; ++i) {
      Slot& s = slot[i & 1];
      {
        std::unique_lock<std::mutex> lock(mu);
        cv.wait(lock, [&] { return s.state == 1; });
      }
      if (s.rc) {
        awq_set_error(s.err);
        rc = s.rc;
        break;
      }
      const WeightFile& wf = files[i];
      void* dst = nullptr;
      DevLinear* t = nullptr;
      if (wf.kind == AWQ_T_GAMMA) {
        dst = e->layers[wf.layer].gamma;
        e->layers[wf.layer].have_gamma = true;
      } else {
        t = find_linear(e, wf.layer, wf.kind);
        if (wf.part == AWQ_P_PACKED && wf.kind != AWQ_T_EMBED) t->packed = (uint8_t*)dstage[n_staged++ & 1];
        dst = wf.part == AWQ_P_PACKED ? (void*)t->packed : wf.part == AWQ_P_SCALE ? (void*)t->scale : (void*)t->zp;
        if (wf.part == AWQ_P_ZP) t->zp_integral = zp_all_integral((const uint16_t*)s.host, wf.bytes / 2);
        t->have[wf.part] = true;
      }
      if (hipMemcpyAsync(dst, s.host, (size_t)wf.bytes, hipMemcpyHostToDevice, e->stream) != hipSuccess ||
          hipEventRecord(s.copied, e->stream) != hipSuccess) {
        awq_set_error("host-to-device copy of " + wf.name + " failed");
        rc = AWQ_ERR_HIP;
        break;
      }
      // the embedding is only ever gathered from, so it stays in file order
      if (t && wf.part == AWQ_P_PACKED && wf.kind != AWQ_T_EMBED) {
        rc = reorder_now(e, t);
        t->packed = nullptr;  // the staging buffer is not the tensor's
      }
      {
        std::lock_guard<std::mutex> lock(mu);
        s.state = 2;
      }
      // the other buffer's copy was queued one file ago: once it has completed the reader may refill it
      Slot& o = slot[(i + 1) & 1];
      bool in_flight;
      {
        std::lock_guard<std::mutex> lock(mu);
        in_flight = o.state == 2;
      }
      if (in_flight) {
        if (hipEventSynchronize(o.copied) != hipSuccess) {
          awq_set_error("waiting for a host-to-device copy failed");
          rc = AWQ_ERR_HIP;
          break;
        }
        {
          std::lock_guard<std::mutex> lock(mu);
          o.state = 0;
        }
        cv.notify_all();
      }
    }
    {
      std::lock_guard<std::mutex> lock(mu);
      stop = true;
    }
    cv.notify_all();
    reader.join();
  }
  if (rc == AWQ_OK && hipStreamSynchronize(e->stream) != hipSuccess) {
    awq_set_error("the weight upload did not complete");
    rc = AWQ_ERR_HIP;
  } else if (rc != AWQ_OK) {
    (void)hipStreamSynchronize(e->stream);  // nothing may still read the staging buffers
  }
  for (Slot& s : slot) {
    if (s.copied) (void)hipEventDestroy(s.copied);
    if (s.host) (void)hipHostFree(s.host);
  }
  for (void* d : dstage)
    if (d) (void)hipFree(d);
  if (rc == AWQ_OK) g_last_load_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_begin).count();
  if (rc == AWQ_OK) rc = awq_finalize(e);
  if (rc) {
    awq_destroy(e);
    return rc;
  }
  *out = e;
  return AWQ_OK;
}

extern "C" void awq_destroy(awq_engine* e) {
  if (!e) return;
  if (e->stream) (void)hipStreamSynchronize(e->stream);
  for (auto& row : e->graphs)
    for (hipGraphExec_t g : row)
      if (g) (void)hipGraphExecDestroy(g);
  for (void* p : e->allocations)
    if (p) (void)hipFree(p);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  delete e;
}

extern "C" int awq_set_graph_mode(awq_engine* e, int enabled) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  e->graph_mode = enabled != 0;
  return AWQ_OK;
}

extern "C" int awq_reset(awq_engine* e) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  if (!e->finalized) {
    awq_set_error("awq_reset before awq_finalize");
    return AWQ_ERR_STATE;
  }
  // The reference initialises current_seq_len_ in the constructor only
  // (Inference.cu:430); a second generateResponse would attend stale positions.
  // Each sequence starts clean here, with a zero hidden state.
  e->current_seq_len = 0;
  e->n_positions = 0;
  e->n_generated = 0;
  if (int rc = launch_fill_zero(e->hidden, (int64_t)e->cfg.hidden * 2, e->stream)) return rc;
  // the words through which waits report (and the tests ask them to give up) start clean
  if (int rc = launch_fill_zero(e->handover_status, 4, e->stream)) return rc;
  // scores of an earlier sequence must not meet their tag again
  if (e->fused_qkv)
    if (int rc = launch_fill_zero(e->score_tag, fused_qkv_attn_exchange_bytes(e->n_heads), e->stream)) return rc;
  if (e->pb.gemm_ws)
    if (int rc = launch_fill_zero(e->pb.gemm_ws, 8, e->stream)) return rc;
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  if (e->giveup_after_reset) {  // awq_debug_force_handover_giveup(e, 2): the sequence that starts here meets the condition
    e->giveup_after_reset = false;
    const int32_t word = 1;
    AWQ_HIP_TRY(hipMemcpy(e->handover_status, &word, 4, hipMemcpyHostToDevice));
  }
  return AWQ_OK;
}

namespace {
// After the stream has drained: did a wait inside a fused launch give up?  The word is cleared, so the engine
// works again after awq_reset.
int check_handover(awq_engine* e) {
  if (!e->fused && !e->fused_qkv) return AWQ_OK;
  int32_t word = 0;
  AWQ_HIP_TRY(hipMemcpy(&word, e->handover_status, 4, hipMemcpyDeviceToHost));
  if (word == 0) return AWQ_OK;
  AWQ_HIP_TRY(hipMemset(e->handover_status, 0, 4));
  e->handover_gave_up = true;
  awq_set_error("a fused launch gave up waiting for what other workgroups hand over");
  return AWQ_ERR_HIP;
}
}  // namespace

extern "C" int awq_set_fused_mode(awq_engine* e, int enabled) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  // bit 0: Wo + W1 as one launch; bit 1: Wqkv + attention as one launch; each only where the device can run it
  const bool want = (enabled & 1) != 0 && fused_wo_w1_supported(e->cfg.hidden, e->cfg.inter) != 0;
  // (the parts arrays exist if the launch was available when the engine was created)
  const bool want_qkv = (enabled & 2) != 0 && e->parts_pos > 0 &&
                        fused_qkv_attn_supported(e->cfg.hidden, e->n_heads, e->stream) != 0;
  if (want != e->fused || want_qkv != e->fused_qkv) {
    // the captured steps hold the other launches
    AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
    for (auto& row : e->graphs)
      for (hipGraphExec_t& g : row)
        if (g) {
          (void)hipGraphExecDestroy(g);
          g = nullptr;
        }
    if (want_qkv && !e->fused_qkv && e->n_positions > 0) {
      // the rows appended while the launch was off
      const int64_t n = std::min<int64_t>(e->n_positions, e->parts_pos);
      for (auto& L : e->layers)
        if (int rc = launch_kv_to_parts(L.kcache, L.vcache, kv_blocked(e->n_heads), L.kparts, L.vparts, e->n_heads,
                                        e->parts_pos, 0, n, e->stream))
          return rc;
      AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
    }
    e->fused = want;
    e->fused_qkv = want_qkv;
  }
  return AWQ_OK;
}

extern "C" int awq_fused_mode(const awq_engine* e) { return e ? (e->fused ? 1 : 0) | (e->fused_qkv ? 2 : 0) : 0; }

// The fused launch of every layer, back to back, with layer `layer`'s launch instrumented: thread 0 of each of its
// hidden/16 workgroups notes the time at kFusedStamps points (10 ns units, one clock for the whole device).
extern "C" int awq_debug_fused_timeline(awq_engine* e, int32_t layer, uint64_t* host_out, int32_t* n_workgroups,
                                        int32_t* n_stamps) {
  AWQ_REQUIRE(e && host_out && n_workgroups && n_stamps, "NULL argument");
  AWQ_REQUIRE(e->finalized, "awq_debug_fused_timeline before awq_finalize");
  AWQ_REQUIRE(fused_wo_w1_supported(e->cfg.hidden, e->cfg.inter) != 0,
              "the fused launch needs hidden 4096, intermediate 12288 and 256 compute units");
  AWQ_REQUIRE(layer >= 0 && layer < e->cfg.n_layers, "layer out of range");
  const int wgs = e->cfg.hidden / 16;
  unsigned long long* d_stamps = nullptr;
  AWQ_HIP_TRY(hipMalloc((void**)&d_stamps, (size_t)wgs * kFusedStamps * 8));
  StepState s{0, 1, 1, -1, 0, 0, 0};
  s.epoch = e->epoch_next;
  e->epoch_next = (e->epoch_next + e->cfg.n_layers) & 0x3fffffff;
  int rc = launch_set_state(e->d_state, s, e->stream);
  for (int rep = 0; rep < 3 && rc == AWQ_OK; ++rep) {  // the last round is the one that counts (warm clocks)
    if (rep) {
      s.epoch = e->epoch_next;
      e->epoch_next = (e->epoch_next + e->cfg.n_layers) & 0x3fffffff;
      rc = launch_set_state(e->d_state, s, e->stream);
    }
    for (int l = 0; l < e->cfg.n_layers && rc == AWQ_OK; ++l) {
      LayerDev& L = e->layers[l];
      rc = launch_fused_wo_w1(L.wo.stream_order, L.wo.scale, L.wo.zp, L.w1.stream_order, L.w1.scale, L.w1.zp, L.gamma,
                              e->cfg.eps, e->ctx, e->hidden, e->mid, e->hid_tag, e->handover_status, e->d_state, l,
                              e->cfg.hidden, e->cfg.inter, l == layer ? d_stamps : nullptr, e->stream);
    }
  }
  if (rc == AWQ_OK && hipStreamSynchronize(e->stream) != hipSuccess) rc = AWQ_ERR_HIP;
  if (rc == AWQ_OK && hipMemcpy(host_out, d_stamps, (size_t)wgs * kFusedStamps * 8, hipMemcpyDeviceToHost) != hipSuccess)
    rc = AWQ_ERR_HIP;
  (void)hipFree(d_stamps);
  if (rc) return rc;
  *n_workgroups = wgs;
  *n_stamps = kFusedStamps;
  {
    int32_t word = 0;
    AWQ_HIP_TRY(hipMemcpy(&word, e->handover_status, 4, hipMemcpyDeviceToHost));
    if (word != 0) {
      AWQ_HIP_TRY(hipMemset(e->handover_status, 0, 4));
      awq_set_error("a fused launch gave up waiting for the hidden state of other workgroups");
      return AWQ_ERR_HIP;
    }
  }
  return awq_reset(e);
}

// prompt loop, Inference.cu:1304-1343
extern "C" int awq_prefill(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt) {
  AWQ_REQUIRE(e != nullptr && n_prompt >= 0 && (n_prompt == 0 || prompt_ids), "bad arguments");
  if (!e->finalized) {
    awq_set_error("awq_prefill before awq_finalize");
    return AWQ_ERR_STATE;
  }
  AWQ_REQUIRE(e->n_generated == 0, "prompt tokens cannot follow generated ones; call awq_reset");
  AWQ_REQUIRE((int64_t)e->n_positions + n_prompt <= e->cfg.max_pos, "prompt does not fit max_pos");
  for (int32_t i = 0; i < n_prompt; ++i) {
    AWQ_REQUIRE(prompt_ids[i] >= 0 && prompt_ids[i] < e->cfg.vocab, "token id out of range");
    const int t = e->n_positions;
    StepState s;
    s.pos = t;
    s.len_lo = e->current_seq_len + 1;  // layer 0 still sees the previous value (:1118 before :1331)
    s.len_hi = t + 1;                   // later layers see current_seq_len_ = t
    s.token = prompt_ids[i];
    s.out_index = 0;
    s.sample = 0;
    if (int rc = run_step(e, false, s)) return rc;
    e->current_seq_len = t;
    e->n_positions = t + 1;
  }
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  return check_handover(e);
}

namespace {

constexpr int64_t kPrefillChunk = 1280;      // prompt positions per batched pass
constexpr int64_t kPrefillLongChunk = 1024;  // ... of a sequence longer than kPrefillLongFrom
constexpr int64_t kPrefillLongFrom = 4096;
constexpr int64_t kGemmWsBytes = (64ll << 20) + 4096;  // header + partial sums (256 tiles, or 4 chunks of k for few rows)

int ensure_prefill_buffers(awq_engine* e) {
  if (e->pb.chunk) return AWQ_OK;
  const int64_t C = std::min<int64_t>(kPrefillChunk, e->cfg.max_pos), H = e->cfg.hidden, I = e->cfg.inter;
  if (int rc = dev_alloc(e, (void**)&e->pb.hidden, C * H * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.norm, C * H * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.qkv, C * 3 * H * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.q, C * H * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.ctx, C * H * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.mid, C * I * 2)) return rc;
  if (int rc = dev_alloc(e, (void**)&e->pb.tokens, C * 4)) return rc;
  if (int rc = dev_alloc(e, &e->pb.gemm_ws, kGemmWsBytes)) return rc;
  AWQ_HIP_TRY(hipMemset(e->pb.gemm_ws, 0, 4096));  // status word and hand-over counters start at zero
  e->pb.chunk = C;
  return AWQ_OK;
}

int gemm_of(awq_engine* e, const DevLinear& t, const half_t* x, half_t* y, int64_t M, int epilogue = EPI_STORE,
            const half_t* res = nullptr) {
  return launch_gemm(t.stream_order, t.scale, t.zp, t.m, t.k, x, y, M, t.zp_integral, epilogue, res, e->pb.gemm_ws,
                     kGemmWsBytes, e->stream);
}

// runOneLayer, Inference.cu:1029-1230, for M prompt positions pos0.. at once.
// Layer 0 reads current_seq_len_ before the prompt loop updates it (:1118, :1331).
int enqueue_layer_batch(awq_engine* e, int l, int64_t pos0, int64_t M) {
  LayerDev& L = e->layers[l];
  hipStream_t st = e->stream;
  const int64_t H = e->cfg.hidden;
  auto& b = e->pb;
  if (int rc = launch_rmsnorm_batch(b.hidden, L.gamma, b.norm, H, M, e->cfg.eps, st)) return rc;  // :1040
  if (int rc = gemm_of(e, L.wqkv, b.norm, b.qkv, M)) return rc;                                    // :1052
  // (with the fused launch on, the appended rows also go into its second copy of the caches)
  if (int rc = launch_rope_kv_append_batch(b.qkv, e->cos_t, e->sin_t, b.q, L.kcache, L.vcache, e->n_heads,
                                           e->cfg.max_pos, kv_blocked(e->n_heads), pos0, M, st,
                                           e->fused_qkv ? L.kparts : nullptr, e->fused_qkv ? L.vparts : nullptr,
                                           e->parts_pos))
    return rc;  // :1070-1103
  if (int rc = launch_prefill_attention(b.q, L.kcache, L.vcache, b.ctx, e->n_heads, e->cfg.max_pos,
                                        kv_blocked(e->n_heads), pos0, M, l >= 1,
                                        st))
    return rc;  // :1110
  // :1128 Wo product, :1149 residual add in its epilogue
  if (int rc = gemm_of(e, L.wo, b.ctx, b.hidden, M, EPI_RESIDUAL, b.hidden)) return rc;
  if (int rc = launch_rmsnorm_batch(b.hidden, L.gamma, b.norm, H, M, e->cfg.eps, st)) return rc;  // :1163
  if (int rc = gemm_of(e, L.w1, b.norm, b.mid, M, EPI_GELU)) return rc;  // :1176, :1196
  return gemm_of(e, L.w2, b.mid, b.hidden, M, EPI_RESIDUAL, b.hidden);   // :1201, :1221
}

}  // namespace

// The prompt loop (Inference.cu:1304-1343) with all prompt positions of a chunk
// going through each layer together: the weights are read once per chunk and
// the products run on the matrix cores.  Every token still sees exactly the
// positions the sequential loop shows it.  The products are summed in another
// order than the one-token kernel's, so the cache it leaves agrees with
// awq_prefill's to binary16 rounding noise, not bit for bit.
extern "C" int awq_prefill_batched(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt) {
  AWQ_REQUIRE(e != nullptr && n_prompt >= 0 && (n_prompt == 0 || prompt_ids), "bad arguments");
  if (!e->finalized) {
    awq_set_error("awq_prefill_batched before awq_finalize");
    return AWQ_ERR_STATE;
  }
  AWQ_REQUIRE(e->n_generated == 0, "prompt tokens cannot follow generated ones; call awq_reset");
  AWQ_REQUIRE((int64_t)e->n_positions + n_prompt <= e->cfg.max_pos, "prompt does not fit max_pos");
  for (int32_t i = 0; i < n_prompt; ++i)
    AWQ_REQUIRE(prompt_ids[i] >= 0 && prompt_ids[i] < e->cfg.vocab, "token id out of range");
  if (n_prompt == 0) return AWQ_OK;
  if (int rc = ensure_prefill_buffers(e)) return rc;
  const int64_t H = e->cfg.hidden;
  for (int64_t off = 0, M = 0; off < n_prompt; off += M) {
    // equal passes rather than full ones and a small rest (whole 128-token tiles each): 4096 positions
    // go as 4 x 1024, not 3 x 1280 + 256.  Sequences beyond kPrefillLongFrom positions take at most
    // 1024 per pass: deep in a long prompt the attention dominates, and 1024 positions x 32 heads
    // are 256 of its workgroups (one per compute unit) where 1280 are 320, which outweighs the
    // products' better tile count at 1280 (8192 tokens: 159 -> 146 ms, 30,000: 0.93 -> 0.89 s;
    // 2560 tokens stay at 2 x 1280).
    const int64_t rest = n_prompt - off;
    const int64_t chunk = e->n_positions + rest > kPrefillLongFrom ? std::min<int64_t>(e->pb.chunk, kPrefillLongChunk)
                                                                  : e->pb.chunk;
    const int64_t passes = (rest + chunk - 1) / chunk;
    M = std::min<int64_t>(rest, std::min<int64_t>(chunk, ((rest + passes - 1) / passes + 127) / 128 * 128));
    const int64_t pos0 = e->n_positions;
    AWQ_HIP_TRY(hipMemcpyAsync(e->pb.tokens, prompt_ids + off, (size_t)M * 4, hipMemcpyHostToDevice, e->stream));
    if (int rc = launch_embed_batch(e->embed.packed, e->embed.scale, e->embed.zp, H, e->cfg.vocab, e->pb.tokens, M,
                                    e->pb.hidden, e->stream))
      return rc;
    for (int l = 0; l < e->cfg.n_layers; ++l)
      if (int rc = enqueue_layer_batch(e, l, pos0, M)) return rc;
    // the state the generation loop starts from (:1357): the last position's output
    AWQ_HIP_TRY(hipMemcpyAsync(e->hidden, e->pb.hidden + (M - 1) * H, (size_t)H * 2, hipMemcpyDeviceToDevice,
                               e->stream));
    AWQ_HIP_TRY(hipStreamSynchronize(e->stream));  // the token ids were read from the caller's buffer
    int32_t gemm_status = 0;
    AWQ_HIP_TRY(hipMemcpy(&gemm_status, e->pb.gemm_ws, 4, hipMemcpyDeviceToHost));
    if (gemm_status != 0) {
      AWQ_HIP_TRY(hipMemset(e->pb.gemm_ws, 0, 4096));
      awq_set_error("a matrix product gave up waiting for partial sums of another workgroup");
      return AWQ_ERR_HIP;
    }
    e->current_seq_len = (int)(pos0 + M - 1);
    e->n_positions = (int)(pos0 + M);
  }
  return AWQ_OK;
}

// The same for the fused Wqkv + attention launch (kQkvStamps points), position `pos` attending pos + 1 positions.
extern "C" int awq_debug_qkv_attention_timeline(awq_engine* e, int32_t layer, int32_t pos, uint64_t* host_out,
                                                int32_t* n_workgroups, int32_t* n_stamps) {
  AWQ_REQUIRE(e && host_out && n_workgroups && n_stamps, "NULL argument");
  AWQ_REQUIRE(e->finalized, "awq_debug_qkv_attention_timeline before awq_finalize");
  AWQ_REQUIRE(e->parts_pos > 0 && fused_qkv_attn_supported(e->cfg.hidden, e->n_heads, e->stream) != 0,
              "the fused launch needs hidden 4096, 32 heads and 256 compute units");
  AWQ_REQUIRE(layer >= 0 && layer < e->cfg.n_layers, "layer out of range");
  AWQ_REQUIRE(pos >= 0 && pos < e->cfg.max_pos && pos + 1 <= e->parts_pos, "pos out of range");
  const int wgs = e->n_heads * 8;
  unsigned long long* d_stamps = nullptr;
  AWQ_HIP_TRY(hipMalloc((void**)&d_stamps, (size_t)wgs * kQkvStamps * 8));
  StepState s{pos, pos + 1, pos + 1, -1, 0, 0, 0};
  int rc = launch_fill_zero(e->score_tag, fused_qkv_attn_exchange_bytes(e->n_heads), e->stream);
  for (int rep = 0; rep < 3 && rc == AWQ_OK; ++rep) {  // the last round is the one that counts (warm clocks)
    s.epoch = e->epoch_next;
    e->epoch_next = (e->epoch_next + e->cfg.n_layers) & 0x3fffffff;
    rc = launch_set_state(e->d_state, s, e->stream);
    for (int l = 0; l < e->cfg.n_layers && rc == AWQ_OK; ++l) {
      LayerDev& L = e->layers[l];
      rc = launch_fused_qkv_attn(L.wqkv.stream_order, L.wqkv.scale, L.wqkv.zp, L.wqkv.m, e->hidden, L.gamma, e->cfg.eps,
                                 e->cos_t, e->sin_t, L.kcache, L.vcache, kv_blocked(e->n_heads), L.kparts, L.vparts,
                                 e->parts_pos, e->q, e->ctx, e->score_tag, e->handover_status, e->d_state, l, 1, pos + 1, e->n_heads,
                                 l == layer ? d_stamps : nullptr, e->stream);
    }
  }
  if (rc == AWQ_OK && hipStreamSynchronize(e->stream) != hipSuccess) rc = AWQ_ERR_HIP;
  if (rc == AWQ_OK && hipMemcpy(host_out, d_stamps, (size_t)wgs * kQkvStamps * 8, hipMemcpyDeviceToHost) != hipSuccess)
    rc = AWQ_ERR_HIP;
  (void)hipFree(d_stamps);
  if (rc) return rc;
  *n_workgroups = wgs;
  *n_stamps = kQkvStamps;
  {
    int32_t word = 0;
    AWQ_HIP_TRY(hipMemcpy(&word, e->handover_status, 4, hipMemcpyDeviceToHost));
    if (word != 0) {
      AWQ_HIP_TRY(hipMemset(e->handover_status, 0, 4));
      awq_set_error("a fused launch gave up waiting for what other workgroups hand over");
      return AWQ_ERR_HIP;
    }
  }
  return awq_reset(e);
}

extern "C" int awq_debug_force_handover_giveup(awq_engine* e, int on) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  if (int rc = ensure_prefill_buffers(e)) return rc;
  const int32_t word = on ? 1 : 0;
  e->giveup_after_reset = on == 2;
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  AWQ_HIP_TRY(hipMemcpy((int32_t*)e->pb.gemm_ws + 1, &word, 4, hipMemcpyHostToDevice));
  // the fused launches of the token-by-token steps look at their status word before they wait
  AWQ_HIP_TRY(hipMemcpy(e->handover_status, &word, 4, hipMemcpyHostToDevice));
  return AWQ_OK;
}

extern "C" int awq_set_prefill_mode(awq_engine* e, int batched) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  e->batched_prefill = batched != 0;
  return AWQ_OK;
}

// generation loop, Inference.cu:1352-1405
extern "C" int awq_decode(awq_engine* e, int32_t n_steps, int32_t* out_ids) {
  AWQ_REQUIRE(e != nullptr && n_steps >= 0 && (n_steps == 0 || out_ids), "bad arguments");
  if (!e->finalized) {
    awq_set_error("awq_decode before awq_finalize");
    return AWQ_ERR_STATE;
  }
  AWQ_REQUIRE((int64_t)e->n_positions + n_steps <= e->cfg.max_pos, "sequence does not fit max_pos");
  const int first = e->n_generated;
  for (int32_t i = 0; i < n_steps; ++i) {
    const int pos = e->n_positions;
    // kStepsPerGraph steps as one graph launch where the call has that many left and they share a length bound
    // (the steps advance their own state on the device, so the nodes of one step are those of the next): a
    // graph launch costs about 8 us beyond its kernels, 1031 -> 1037 tok/s with four steps per launch, the
    // same with 8, 16 or 32
    if (e->graph_mode && i > 0 && i + kStepsPerGraph <= n_steps && length_bucket(pos + 1) == length_bucket(pos + kStepsPerGraph)) {
      StepState s;
      s.pos = pos;
      s.len_lo = e->current_seq_len + 1;
      s.len_hi = pos + 1;
      s.token = -1;
      s.out_index = e->n_generated;
      s.sample = 1;
      if (int rc = run_step(e, true, s, false, kStepsPerGraph)) return rc;
      e->current_seq_len = pos + kStepsPerGraph - 1;
      e->n_positions = pos + kStepsPerGraph;
      e->n_generated += kStepsPerGraph;
      i += kStepsPerGraph - 1;
      continue;
    }
    StepState s;
    s.pos = pos;
    s.len_lo = e->current_seq_len + 1;  // layers below split_idx run before :1364
    s.len_hi = pos + 1;                 // the others after it
    s.token = -1;
    s.out_index = e->n_generated;
    s.sample = 1;
    // the state is written for the first step of the call; every step leaves the next one's on the device
    if (int rc = run_step(e, true, s, i == 0)) return rc;
    e->current_seq_len = pos;
    e->n_positions = pos + 1;
    e->n_generated += 1;
  }
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  if (int rc = check_handover(e)) return rc;
  if (n_steps > 0)
    AWQ_HIP_TRY(hipMemcpy(out_ids, e->d_out + first, (size_t)n_steps * 4, hipMemcpyDeviceToHost));
  return AWQ_OK;
}

extern "C" int awq_generate(awq_engine* e, const int32_t* prompt_ids, int32_t n_prompt, int32_t max_new_tokens,
                            int32_t* out_ids) {
  AWQ_REQUIRE(e != nullptr, "engine is NULL");
  AWQ_REQUIRE(n_prompt >= 0 && max_new_tokens >= 0, "negative count");
  AWQ_REQUIRE((int64_t)n_prompt + max_new_tokens <= e->cfg.max_pos, "prompt + new tokens exceed max_pos");
  auto once = [&]() -> int {
    if (int rc = awq_reset(e)) return rc;
    if (int rc = e->batched_prefill ? awq_prefill_batched(e, prompt_ids, n_prompt) : awq_prefill(e, prompt_ids, n_prompt))
      return rc;
    return awq_decode(e, max_new_tokens, out_ids);
  };
  e->handover_gave_up = false;
  int rc = once();
  if (rc == AWQ_ERR_HIP && e->handover_gave_up && (e->fused || e->fused_qkv)) {
    // A fused launch needs all its workgroups resident at once.  Where that does not hold (the device shared
    // with other work) its bounded waits give up; the whole request is then run again with every launch on its
    // own, as the reference has them, and the engine stays that way until awq_set_fused_mode is called again.
    if (int rc2 = awq_set_fused_mode(e, 0)) return rc2;
    rc = once();
  }
  return rc;
}

extern "C" int awq_read_hidden(awq_engine* e, uint16_t* host_dst) {
  AWQ_REQUIRE(e && host_dst, "NULL argument");
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  const half_t* src = e->n_generated > 0 ? e->hidden_last : e->hidden;
  AWQ_HIP_TRY(hipMemcpy(host_dst, src, (size_t)e->cfg.hidden * 2, hipMemcpyDeviceToHost));
  return AWQ_OK;
}

extern "C" int awq_read_logits(awq_engine* e, uint16_t* host_dst) {
  AWQ_REQUIRE(e && host_dst, "NULL argument");
  AWQ_HIP_TRY(hipStreamSynchronize(e->stream));
  AWQ_HIP_TRY(hipMemcpy(host_dst, e->logits, (size_t)e->cfg.vocab * 2, hipMemcpyDeviceToHost));
  return AWQ_OK;
}

// Times the engine's own fused-linear launches of one tensor kind over all
// layers' resident weights (a different matrix every launch, so the working
// set is n_layers matrices), with HIP events on the engine's stream.
extern "C" int awq_time_linear(awq_engine* e, int kind, int32_t n_rounds, float* avg_us_per_launch,
                               int64_t* bytes_per_launch) {
  AWQ_REQUIRE(e && avg_us_per_launch && n_rounds > 0, "bad arguments");
  if (!e->finalized) {
    awq_set_error("awq_time_linear before awq_finalize");
    return AWQ_ERR_STATE;
  }
  AWQ_REQUIRE(kind == AWQ_T_WQKV || kind == AWQ_T_WO || kind == AWQ_T_W1 || kind == AWQ_T_W2 || kind == AWQ_T_UNEMBED,
              "kind must be a linear layer");
  // events and the graph are released on every way out
  struct Held {
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    ~Held() {
      if (exec) (void)hipGraphExecDestroy(exec);
      if (graph) (void)hipGraphDestroy(graph);
      if (ev0) (void)hipEventDestroy(ev0);
      if (ev1) (void)hipEventDestroy(ev1);
    }
  } held;
  hipEvent_t& ev0 = held.ev0;
  hipEvent_t& ev1 = held.ev1;
  AWQ_HIP_TRY(hipEventCreate(&ev0));
  AWQ_HIP_TRY(hipEventCreate(&ev1));
  const int n_mats = kind == AWQ_T_UNEMBED ? 1 : e->cfg.n_layers;
  auto one_round = [&]() -> int {
    for (int l = 0; l < n_mats; ++l) {
      const DevLinear& t = *find_linear(e, l, kind);
      int rc = AWQ_OK;
      LinearArgs a;
      switch (kind) {
        case AWQ_T_WQKV:
          a = linear_args(e, t, e->hidden, e->q);
          a.prologue = PRO_RMSNORM;
          a.gamma = e->layers[l].gamma;
          a.epilogue = EPI_QKV_ROPE;
          a.cos_t = e->cos_t;
          a.sin_t = e->sin_t;
          a.k_cache = e->layers[l].kcache;
          a.v_cache = e->layers[l].vcache;
          a.hidden = e->cfg.hidden;
          a.max_pos = e->cfg.max_pos;
          a.kv = kv_blocked(e->n_heads);
          break;
        case AWQ_T_WO:
          a = linear_args(e, t, e->ctx, e->hidden);
          a.epilogue = EPI_RESIDUAL;
          a.res = e->hidden;
          break;
        case AWQ_T_W1:
          a = linear_args(e, t, e->hidden, e->mid);
          a.prologue = PRO_RMSNORM;
          a.gamma = e->layers[l].gamma;
          a.epilogue = EPI_GELU;
          break;
        case AWQ_T_W2:
          a = linear_args(e, t, e->mid, e->hidden);
          a.epilogue = EPI_RESIDUAL;
          a.res = e->hidden;
          break;
        default:
          // the sampling launch as the decode step issues it (norm, logits, argmax, then the small
          // launch that ends the step); both launches count as one in the average
          a = sample_args(e);
          a.out_array = nullptr;  // nothing is appended to the output and the step state stays as set below
          a.fin_state = nullptr;
          break;
      }
      rc = launch_gemv(a, e->stream);
      if (rc) return rc;
    }
    return AWQ_OK;
  };
  StepState s0{0, 1, 1, -1, 0, 0};
  if (int rc = launch_set_state(e->d_state, s0, e->stream)) return rc;
  if (int rc = one_round()) return rc;  // warm-up
  // A round is replayed as a captured graph, which is how the decode step issues
  // these launches: the host's launch rate stays out of the figure.
  hipGraph_t& graph = held.graph;
  hipGraphExec_t& exec = held.exec;
  // (with few matrices several rounds go into one graph, so that a replay is long
  // against the cost of starting one)
  const int per_graph = std::min<int>(n_rounds, std::max(1, 32 / n_mats));
  const int replays = (n_rounds + per_graph - 1) / per_graph;
  AWQ_HIP_TRY(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
  int crc = AWQ_OK;
  for (int r = 0; r < per_graph && crc == AWQ_OK; ++r) crc = one_round();
  hipError_t cerr = hipStreamEndCapture(e->stream, &graph);
  if (crc) return crc;
  AWQ_HIP_TRY(cerr);
  AWQ_HIP_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  // warm-up: as many replays as are timed (at most 16): the first rounds after other work (another
  // shape's launches, an idle stretch) read up to 5 % long
  for (int r = 0; r < std::min(replays, 16); ++r) AWQ_HIP_TRY(hipGraphLaunch(exec, e->stream));
  AWQ_HIP_TRY(hipEventRecord(ev0, e->stream));
  for (int r = 0; r < replays; ++r) AWQ_HIP_TRY(hipGraphLaunch(exec, e->stream));
  AWQ_HIP_TRY(hipEventRecord(ev1, e->stream));
  AWQ_HIP_TRY(hipEventSynchronize(ev1));
  float ms = 0.0f;
  AWQ_HIP_TRY(hipEventElapsedTime(&ms, ev0, ev1));
  *avg_us_per_launch = ms * 1000.0f / (float)((int64_t)replays * per_graph * n_mats);
  if (bytes_per_launch) {
    const DevLinear& t = *find_linear(e, 0, kind);
    // packed weights + scales + zero-points + input vector + output vector
    *bytes_per_launch = t.m * (t.k / 2) + 2 * (t.m / 128) * 2 + t.k * 2 + t.m * 2;
  }
  return awq_reset(e);
}

// ---------------------------------------------------------------------------
// kernel-level entry points
// ---------------------------------------------------------------------------
extern "C" int awq_dequant(const void* packed, const void* scale, const void* zp, void* out, int64_t rows, int64_t cols,
                           int64_t n_groups, void* stream) {
  AWQ_REQUIRE(packed && scale && zp && out, "NULL pointer");
  return launch_dequant((const uint8_t*)packed, (const half_t*)scale, (const half_t*)zp, (half_t*)out, rows, cols,
                        n_groups, (hipStream_t)stream);
}

extern "C" int awq_linear_repack(const void* packed_in, void* repacked_out, int64_t m, int64_t k, void* stream) {
  AWQ_REQUIRE(packed_in && repacked_out && packed_in != repacked_out, "NULL or aliased pointers");
  return launch_repack((const uint8_t*)packed_in, repacked_out, m, k, (hipStream_t)stream);
}

extern "C" int64_t awq_gemv_workspace_bytes(int64_t m, int64_t k) { return gemv_workspace_bytes(m, k); }

extern "C" int awq_gemv_fused(const awq_linear_args* u, void* stream) {
  AWQ_REQUIRE(u != nullptr, "args is NULL");
  AWQ_REQUIRE(u->repacked && u->scale && u->zp && u->x && u->y && u->workspace, "NULL pointer");
  AWQ_REQUIRE(u->m > 0 && u->m % 128 == 0, "m must be a positive multiple of 128");
  AWQ_REQUIRE(u->prologue == AWQ_PRO_NONE || u->prologue == AWQ_PRO_RMSNORM, "bad prologue");
  AWQ_REQUIRE(u->epilogue >= AWQ_EPI_STORE && u->epilogue <= AWQ_EPI_ARGMAX, "bad epilogue");
  LinearArgs a;
  a.wq = u->repacked;
  a.scale = (const half_t*)u->scale;
  a.zp = (const half_t*)u->zp;
  a.x = (const half_t*)u->x;
  a.y = (half_t*)u->y;
  a.res = (const half_t*)u->residual;
  a.best = (unsigned long long*)u->workspace;  // the sampler's best candidate
  a.m = u->m;
  a.k = u->k;
  a.prologue = u->prologue;
  a.epilogue = u->epilogue;
  a.gamma = (const half_t*)u->gamma;
  a.eps = u->eps;
  a.cos_t = (const half_t*)u->cos_t;
  a.sin_t = (const half_t*)u->sin_t;
  a.k_cache = (half_t*)u->k_cache;
  a.v_cache = (half_t*)u->v_cache;
  a.hidden = u->hidden;
  a.pos = (int32_t)u->pos;
  a.max_pos = u->max_pos;
  a.kv = kv_head_major(u->max_pos);
  a.out_token = (int32_t*)u->out_token;
  return launch_gemv(a, (hipStream_t)stream);
}

// workspace of awq_qkv_attention: the step state the launch reads, the status word, then the exchange buffers
namespace {
constexpr int64_t kQkvWsHeader = 256;  // StepState at 0, status word at 128
}
extern "C" int64_t awq_qkv_attention_workspace_bytes(int32_t n_heads) {
  if (n_heads <= 0) return -1;
  return kQkvWsHeader + fused_qkv_attn_exchange_bytes(n_heads);
}

extern "C" int awq_qkv_attention_supported(int64_t hidden, int32_t n_heads, void* stream) {
  return fused_qkv_attn_supported(hidden, n_heads, (hipStream_t)stream);
}

extern "C" int64_t awq_kv_parts_bytes(int32_t n_heads, int64_t parts_pos) {
  if (n_heads <= 0 || parts_pos <= 0) return -1;
  return fused_qkv_attn_parts_bytes(n_heads, parts_pos);
}

extern "C" int awq_kv_cache_to_parts(const void* k_cache, const void* v_cache, int64_t max_pos, int32_t n_heads,
                                     void* k_parts, void* v_parts, int64_t parts_pos, int64_t pos0, int64_t n,
                                     void* stream) {
  AWQ_REQUIRE(max_pos > 0 && pos0 >= 0 && n >= 0 && pos0 + n <= max_pos && parts_pos > 0 && parts_pos < (1ll << 30),
              "positions out of range");
  return launch_kv_to_parts((const half_t*)k_cache, (const half_t*)v_cache, kv_head_major(max_pos), (half_t*)k_parts,
                            (half_t*)v_parts, n_heads, (int)parts_pos, pos0, n, (hipStream_t)stream);
}

extern "C" int awq_qkv_attention(const void* wqkv_repacked, const void* scale, const void* zp, const void* x,
                                 const void* gamma, float eps, const void* cos_t, const void* sin_t, void* k_cache,
                                 void* v_cache, int64_t max_pos, void* k_parts, void* v_parts, int64_t parts_pos,
                                 int32_t n_heads, int64_t pos, int64_t L, void* q_out, void* ctx, void* workspace,
                                 int32_t call_tag, void* stream) {
  AWQ_REQUIRE(workspace != nullptr, "workspace is NULL");
  AWQ_REQUIRE(n_heads == 32, "the fused launch is built for 32 heads of 128");
  AWQ_REQUIRE(max_pos > 0 && pos >= 0 && pos < max_pos, "pos out of range");
  AWQ_REQUIRE(L >= 0 && L <= pos + 1 && L <= kFusedQkvAttnMax, "attended length out of range for the fused launch");
  AWQ_REQUIRE(parts_pos > 0 && parts_pos < (1ll << 30) && L <= parts_pos, "the parts arrays do not hold the attended positions");
  AWQ_REQUIRE(call_tag >= 1 && call_tag < (1 << 30), "call_tag must be in [1, 2^30)");
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  StepState s{};
  s.pos = (int32_t)pos;
  s.len_lo = s.len_hi = (int32_t)L;
  s.token = -1;
  s.epoch = call_tag;
  if (int rc = launch_set_state((StepState*)ws, s, st)) return rc;
  const int64_t hidden = (int64_t)n_heads * AWQ_HEAD_DIM;
  uint32_t* score_tag = (uint32_t*)(ws + kQkvWsHeader);
  // the words of an earlier call must not meet their tag again
  if (int rc = launch_fill_zero(score_tag, fused_qkv_attn_exchange_bytes(n_heads), st)) return rc;
  return launch_fused_qkv_attn(wqkv_repacked, (const half_t*)scale, (const half_t*)zp, 3 * hidden, (const half_t*)x,
                               (const half_t*)gamma, eps, (const half_t*)cos_t, (const half_t*)sin_t, (half_t*)k_cache,
                               (half_t*)v_cache, kv_head_major(max_pos), (half_t*)k_parts, (half_t*)v_parts, (int)parts_pos,
                               (half_t*)q_out, (half_t*)ctx, score_tag,
                               (int32_t*)(ws + 128), (const StepState*)ws, 0, 0, L > 0 ? L : 1, n_heads, nullptr, st);
}

// after the stream has drained: 0, or AWQ_ERR_HIP when a wait of the last launches gave up (the word is cleared)
extern "C" int awq_qkv_attention_status(void* workspace, void* stream) {
  AWQ_REQUIRE(workspace != nullptr, "workspace is NULL");
  AWQ_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  int32_t word = 0;
  AWQ_HIP_TRY(hipMemcpy(&word, (char*)workspace + 128, 4, hipMemcpyDeviceToHost));
  if (word == 0) return AWQ_OK;
  AWQ_HIP_TRY(hipMemset((char*)workspace + 128, 0, 4));
  awq_set_error("a fused launch gave up waiting for what other workgroups hand over");
  return AWQ_ERR_HIP;
}

extern "C" int awq_gemv(const void* repacked, const void* scale, const void* zp, int64_t m, int64_t k, const void* x,
                        void* y, void* workspace, void* stream) {
  awq_linear_args u;
  memset(&u, 0, sizeof(u));
  u.repacked = repacked;
  u.scale = scale;
  u.zp = zp;
  u.m = m;
  u.k = k;
  u.x = x;
  u.y = y;
  u.workspace = workspace;
  return awq_gemv_fused(&u, stream);
}

extern "C" int64_t awq_gemm_workspace_bytes(int64_t m, int64_t k, int64_t M) { return gemm_workspace_bytes(m, k, M); }
extern "C" int awq_gemm_plan(int64_t m, int64_t k, int64_t M, int has_workspace) {
  return gemm_plan(m, k, M, has_workspace);
}

extern "C" int awq_gemm(const void* repacked, const void* scale, const void* zp, int64_t m, int64_t k, const void* x,
                        void* y, int64_t M, int32_t zp_integral, void* workspace, void* stream) {
  AWQ_REQUIRE(repacked && scale && zp && x && y, "NULL pointer");
  AWQ_REQUIRE(m > 0 && m % 128 == 0, "m must be a positive multiple of 128");
  if (zp_integral < 0) {
    std::vector<uint16_t> zph((size_t)(m / 128));
    AWQ_HIP_TRY(hipMemcpyAsync(zph.data(), zp, zph.size() * 2, hipMemcpyDeviceToHost, (hipStream_t)stream));
    AWQ_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    zp_integral = zp_all_integral(zph.data(), (int64_t)zph.size());
  }
  return launch_gemm(repacked, (const half_t*)scale, (const half_t*)zp, m, k, (const half_t*)x, (half_t*)y, M,
                     zp_integral != 0, EPI_STORE, nullptr, workspace, workspace ? gemm_workspace_bytes(m, k, M) : 0,
                     (hipStream_t)stream);
}

extern "C" int awq_rmsnorm(const void* x, const void* gamma, void* out, int64_t n, float eps, void* stream) {
  AWQ_REQUIRE(x && gamma && out, "NULL pointer");
  return launch_rmsnorm((const half_t*)x, (const half_t*)gamma, (half_t*)out, n, eps, (hipStream_t)stream);
}

extern "C" int awq_rope_kv_append(const void* qkv, const void* cos_t, const void* sin_t, void* q_out, void* k_cache,
                                  void* v_cache, int32_t n_heads, int64_t max_pos, int64_t pos, void* stream) {
  AWQ_REQUIRE(qkv && cos_t && sin_t && q_out && k_cache && v_cache, "NULL pointer");
  return launch_rope_kv_append((const half_t*)qkv, (const half_t*)cos_t, (const half_t*)sin_t, (half_t*)q_out,
                               (half_t*)k_cache, (half_t*)v_cache, n_heads, max_pos, kv_head_major(max_pos), pos, nullptr,
                               (hipStream_t)stream);
}

extern "C" int64_t awq_attention_workspace_bytes(int32_t n_heads, int64_t max_pos) {
  return attention_workspace_bytes(n_heads, max_pos);
}

extern "C" int awq_decode_attention(const void* q, const void* k_cache, const void* v_cache, void* ctx, int32_t n_heads,
                                    int64_t max_pos, int64_t L, void* workspace, void* stream) {
  AWQ_REQUIRE(q && k_cache && v_cache && ctx, "NULL pointer");
  return launch_attention((const half_t*)q, (const half_t*)k_cache, (const half_t*)v_cache, (half_t*)ctx, n_heads,
                          max_pos, kv_head_major(max_pos), L, nullptr, 0, 0, workspace, (hipStream_t)stream);
}

extern "C" int awq_decode_attention_static(const void* q, const void* k_cache, const void* v_cache, void* ctx,
                                           int32_t n_heads, int64_t max_pos, int64_t L, void* stream) {
  AWQ_REQUIRE(q && k_cache && v_cache && ctx, "NULL pointer");
  return launch_attention_static((const half_t*)q, (const half_t*)k_cache, (const half_t*)v_cache, (half_t*)ctx, n_heads,
                                 max_pos, L, (hipStream_t)stream);
}

extern "C" int awq_prefill_attention(const void* q, const void* k_cache, const void* v_cache, void* ctx,
                                     int32_t n_heads, int64_t max_pos, int64_t pos0, int64_t n_tokens,
                                     int32_t first_layer, void* stream) {
  AWQ_REQUIRE(q && k_cache && v_cache && ctx, "NULL pointer");
  return launch_prefill_attention((const half_t*)q, (const half_t*)k_cache, (const half_t*)v_cache, (half_t*)ctx,
                                  n_heads, max_pos, kv_head_major(max_pos), pos0, n_tokens, first_layer ? 0 : 1,
                                  (hipStream_t)stream);
}

extern "C" int awq_residual_add(const void* a, const void* b, void* out, int64_t n, void* stream) {
  AWQ_REQUIRE(a && b && out, "NULL pointer");
  return launch_residual((const half_t*)a, (const half_t*)b, (half_t*)out, n, (hipStream_t)stream);
}

extern "C" int awq_gelu(void* x, int64_t n, void* stream) {
  AWQ_REQUIRE(x != nullptr, "NULL pointer");
  return launch_gelu((half_t*)x, n, (hipStream_t)stream);
}

extern "C" int64_t awq_argmax_workspace_bytes(int64_t n) { return argmax_workspace_bytes(n); }

extern "C" int awq_logits_argmax(const void* logits, int64_t n, void* out_token, void* workspace, void* stream) {
  AWQ_REQUIRE(logits && out_token, "NULL pointer");
  return launch_argmax((const half_t*)logits, n, (int32_t*)out_token, workspace, nullptr, nullptr, (hipStream_t)stream);
}

extern "C" int awq_embed_gather(const void* packed, const void* scale, const void* zp, int64_t hidden, int64_t vocab,
                                int32_t tok, void* out, void* stream) {
  AWQ_REQUIRE(packed && scale && zp && out, "NULL pointer");
  return launch_embed((const uint8_t*)packed, (const half_t*)scale, (const half_t*)zp, hidden, vocab, tok, nullptr,
                      (half_t*)out, (hipStream_t)stream);
}
