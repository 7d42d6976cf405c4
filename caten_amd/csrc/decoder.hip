// Decoder session: Caten's Transformer (external/llm/layers.lisp:73-90) and the
// gpt2-generate loop (apps/gpt2/gpt2.lisp:97-113) as a device-resident pipeline.
//
// One decode step is a fixed sequence of fused launches whose only varying
// inputs -- the current token and the position -- live in device memory, so the
// sequence is captured ONCE as a hipGraph and replayed for every step without a
// host round trip: the argmax kernel writes the next token where the embedding
// kernel reads it and advances the position.  Per GPT-2 layer:
//   1. LayerNorm1 -> c_attn GEMV -> +bias, q to a buffer, k/v rows straight into
//      the KV cache at `pos` (the !assign of layers.lisp:30-31)
//   2. attention of the one query row over cache rows 0..pos (causal mask implicit)
//   3. c_proj GEMV + bias + residual
//   4. LayerNorm2 -> c_fc GEMV + bias -> GELU
//   5. mlp c_proj GEMV + bias + residual
// then ln_f -> lm_head GEMV and the argmax.  Llama-shaped models (not in the
// reference) use RMSNorm prologues, a fused wq|wk|wv matrix, a RoPE + cache-append
// kernel, GQA attention and a fused gate|up matrix whose SwiGLU is the prologue of
// the down projection.
//
// The reference pushes a whole prompt through one forward (s > 1).  Prompts of 8 or more rows
// run as one batch (MFMA GEMMs over the rows, see prefill()); shorter ones are fed row by row
// through the decode step (causal attention makes that the same function).  Either way only the
// last row runs lm_head and argmax.
#include <stdlib.h>
#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "common.h"
#include "decode_fused.h"

namespace cthip {

struct RawTensor {
  void *dev = nullptr;  // GGUF bytes on the device
  int type = 0;
  int64_t rows = 0, cols = 0;
  size_t nbytes = 0;
};

static size_t raw_nbytes(int type, int64_t n) {
  switch (type) {
    case CTHIP_F32: return (size_t)n * 4;
    case CTHIP_F16: return (size_t)n * 2;
    case CTHIP_Q8_0: return (size_t)((n + 31) / 32) * 34;
    case CTHIP_Q4_0: return (size_t)(n / 32) * 18;
    default: return 0;
  }
}

static const int kStepsPerGraph = 8;

struct Layer {
  // GPT-2
  float *ln1_g = nullptr, *ln1_b = nullptr, *ln2_g = nullptr, *ln2_b = nullptr;
  WMat *attn = nullptr, *proj = nullptr, *fc = nullptr, *fc2 = nullptr;
  float *attn_b = nullptr, *proj_b = nullptr, *fc_b = nullptr, *fc2_b = nullptr;
  // LayerNorm folded through c_attn / c_fc: S = W.gamma, C = W.beta + bias
  float *attn_s = nullptr, *attn_c = nullptr, *fc_s = nullptr, *fc_c = nullptr;
  // Llama: attn = wq|wk|wv, proj = wo, fc = gate|up, fc2 = down, ln1_g/ln2_g = rms weights
  bool fc_pairs = false;  // gate / up rows interleaved, SwiGLU in the gate|up launch
  float *k_cache = nullptr, *v_cache = nullptr;
  // option kv_cache 1: the cache as Q8_0 rows instead (quant and scale planes; k_cache / v_cache stay null)
  void *kq = nullptr, *kdq = nullptr, *vq = nullptr, *vdq = nullptr;
  // option kv_cache 2: the cache in pages (kvp.hip): device tables of page pointers and the host's copy of them
  float **k_pages = nullptr, **v_pages = nullptr;
  std::vector<float *> k_page_host, v_page_host;
  // three-launch decode layer: attn.c_proj by head and mlp.c_proj by 16-column slab (quant / scale planes)
  void *proj_hq = nullptr, *proj_hd = nullptr, *fc2_sq = nullptr, *fc2_sd = nullptr;
};

struct Decoder {
  cthip_decoder_config cfg;
  std::map<std::string, RawTensor> raw;
  std::vector<std::string> required;
  bool finalized = false;
  std::vector<Layer> layers;
  float *wte = nullptr, *wpe = nullptr, *lnf_g = nullptr, *lnf_b = nullptr;
  WMat *lm_head = nullptr;
  float *lm_s = nullptr, *lm_c = nullptr;  // ln_f folded through lm_head
  // activations
  float *x = nullptr, *q = nullptr, *kv_tmp = nullptr, *att = nullptr, *h = nullptr, *logits = nullptr;
  AttnSplit att_split = {1, nullptr, nullptr};  // the one-launch-per-Linear step: workgroups per head of its attention launch
  // device-resident loop state: [0] = current token, [1] = position
  int *tokpos = nullptr;
  int64_t *token64 = nullptr;
  int64_t *history = nullptr;
  int *hist_n = nullptr;
  int *ctrl = nullptr;        // [0] = token id that ends a sequence (-1 = none), [1] = the sequence has ended
  int *ctrl_host = nullptr;   // pinned copy of ctrl the host polls between graph launches
  hipEvent_t ctrl_ev = nullptr;
  // scratch of the argmax fused behind lm_head: one partial per wavefront
  float *am_val = nullptr;
  int *am_idx = nullptr;
  int position = 0;
  bool primed = false;  // a forward has left token/position on the device
  bool use_graph = true;
  // the three-launch decode layer (decode_fused.hip): second residual buffer, per-head partials of the
  // attention projection, per-XCD accumulators of the MLP projection
  bool fused = false;
  float *x2 = nullptr, *patt = nullptr;
  long long *pmlp = nullptr;
  // all layers of a step as one launch (decode_flow.hip): the tagged hand-over buffers and the launch's arguments
  bool flow = false;
  FlowArgs flow_args = {};
  // grouped-query layers (decode_gqa.hip): the attention projection has an accumulator set of its own
  bool fused_gqa = false;
  long long *pattn = nullptr;
  // KV cache kept as Q8_0 rows (kvq.hip); peek_f32: fp32 copy of one layer's cache for cthip_decoder_peek
  bool kvq = false;
  float *peek_f32 = nullptr;
  // KV cache in pages (kvp.hip)
  bool kvp = false;
  // [0]: the step as the session runs it at short contexts; [1]: three-launch layers at long contexts (long_from > 0):
  // the attention as a launch of its own with a head's keys shared by several workgroups, then the projection
  hipGraphExec_t g_step[2] = {nullptr, nullptr}, g_body[2] = {nullptr, nullptr}, g_multi[2] = {nullptr, nullptr};
  int long_from = 0;       // position from which [1] runs; 0 = never
  bool long_mode = false;  // which of the two queue_step queues
  int64_t weight_bytes = 0, vector_bytes = 0;
  std::vector<void *> owned;  // device blocks to free
};

static int kv_dim(const cthip_decoder_config &c) { return c.dim / c.n_heads * c.n_kv_heads; }

static void build_required(Decoder *d) {
  const cthip_decoder_config &c = d->cfg;
  char buf[128];
  if (c.arch == CTHIP_ARCH_GPT2) {
    // state-dict keys after remap-key (apps/gpt2/gpt2.lisp:52-70)
    d->required = {"wte.weight", "wpe.weight", "ln_f.affine", "ln_f.bias", "lm_head.weight"};
    static const char *per[] = {"ln_1.affine", "ln_1.bias", "attn.c_attn.weight", "attn.c_attn.bias",
                                "attn.c_proj.weight", "attn.c_proj.bias", "ln_2.affine", "ln_2.bias",
                                "mlp.c_fc.weight", "mlp.c_fc.bias", "mlp.c_proj.weight", "mlp.c_proj.bias"};
    for (int l = 0; l < c.n_layers; l++)
      for (const char *p : per) {
        snprintf(buf, sizeof(buf), "h.%d.%s", l, p);
        d->required.push_back(buf);
      }
  } else {
    d->required = {"tok_embeddings.weight", "norm.weight", "output.weight"};
    static const char *per[] = {"attention_norm.weight", "attention.wq.weight", "attention.wk.weight",
                                "attention.wv.weight", "attention.wo.weight", "ffn_norm.weight",
                                "feed_forward.w1.weight", "feed_forward.w2.weight", "feed_forward.w3.weight"};
    for (int l = 0; l < c.n_layers; l++)
      for (const char *p : per) {
        snprintf(buf, sizeof(buf), "layers.%d.%s", l, p);
        d->required.push_back(buf);
      }
  }
}

static int dev_alloc(Decoder *d, void **p, size_t bytes) {
  int rc = cthip_alloc(p, bytes);
  if (rc == 0) d->owned.push_back(*p);
  return rc;
}

// dequantise a raw tensor to an fp32 device vector owned by the session
static int to_f32(Decoder *d, const std::string &key, int64_t want_n, float **out) {
  auto it = d->raw.find(key);
  if (it == d->raw.end()) return fail(CTHIP_E_STATE, "decoder: tensor '%s' was not loaded", key.c_str());
  RawTensor &r = it->second;
  const int64_t n = r.rows * r.cols;
  if (n != want_n)
    return fail(CTHIP_E_BAD_ARG, "decoder: tensor '%s' has %lld elements, expected %lld", key.c_str(), (long long)n,
                (long long)want_n);
  int rc = dev_alloc(d, (void **)out, sizeof(float) * (size_t)n);
  if (rc) return rc;
  rc = cthip_dequant(r.type, r.dev, n, *out);
  if (rc) return rc;
  d->vector_bytes += 4 * n;
  return 0;
}

// pack one or more raw tensors (row-concatenated) into a weight matrix
// interleave: two parts of equal height are merged row by row (a0, b0, a1, b1, ...) instead of stacked
static int to_wmat(Decoder *d, const std::vector<std::string> &keys, int64_t want_rows, int64_t want_cols, WMat **out,
                   bool interleave = false) {
  std::vector<RawTensor *> parts;
  int64_t rows = 0;
  for (const std::string &k : keys) {
    auto it = d->raw.find(k);
    if (it == d->raw.end()) return fail(CTHIP_E_STATE, "decoder: tensor '%s' was not loaded", k.c_str());
    parts.push_back(&it->second);
    rows += it->second.rows;
    if (it->second.cols != want_cols || it->second.type != parts[0]->type)
      return fail(CTHIP_E_BAD_ARG, "decoder: tensor '%s' is (%lld,%lld) type %d; expected %lld columns of type %d",
                  k.c_str(), (long long)it->second.rows, (long long)it->second.cols, it->second.type,
                  (long long)want_cols, parts[0]->type);
  }
  if (rows != want_rows)
    return fail(CTHIP_E_BAD_ARG, "decoder: '%s' (+%zu) has %lld rows, expected %lld", keys[0].c_str(), keys.size() - 1,
                (long long)rows, (long long)want_rows);
  int rc;
  if (parts.size() == 1) {
    rc = wmat_create_impl(out, parts[0]->type, parts[0]->dev, rows, want_cols);
  } else {
    size_t total = 0;
    for (RawTensor *p : parts) total += p->nbytes;
    void *cat = nullptr;
    if ((rc = cthip_alloc(&cat, total))) return rc;
    if (interleave) {
      if (parts.size() != 2 || parts[0]->rows != parts[1]->rows || parts[0]->nbytes != parts[1]->nbytes)
        return fail(CTHIP_E_BAD_ARG, "decoder: '%s' cannot be interleaved with its partner", keys[0].c_str());
      const size_t rowbytes = parts[0]->nbytes / (size_t)parts[0]->rows;  // GGUF rows are contiguous runs of blocks
      for (int k = 0; k < 2; k++)
        CTHIP_CHECK(hipMemcpy2DAsync((char *)cat + k * rowbytes, 2 * rowbytes, parts[k]->dev, rowbytes, rowbytes,
                                     (size_t)parts[k]->rows, hipMemcpyDeviceToDevice, state().stream));
    } else {
      size_t off = 0;
      for (RawTensor *p : parts) {
        if ((rc = cthip_d2d((char *)cat + off, p->dev, p->nbytes))) return rc;
        off += p->nbytes;
      }
    }
    rc = wmat_create_impl(out, parts[0]->type, cat, rows, want_cols);
    cthip_free(cat);
  }
  if (rc) return rc;
  d->weight_bytes += (*out)->q_bytes + (*out)->d_bytes;
  if (!gemv_is_direct(*out)) d->use_graph = false;
  return 0;
}

// Paged cache: opens the pages that rows [0, rows) need and extends the layers' tables.  Called by the host before it
// queues work that reaches those rows; the tables' addresses stay what the captured graphs hold.
static int ensure_pages(Decoder *d, int rows) {
  if (!d->kvp) return 0;
  const cthip_decoder_config &c = d->cfg;
  const size_t want = (size_t)(rows + kKvPageRows - 1) / kKvPageRows;
  const size_t bytes = sizeof(float) * (size_t)kKvPageRows * kv_dim(c);
  for (Layer &L : d->layers) {
    const size_t have = L.k_page_host.size();
    if (have >= want) continue;
    for (size_t p = have; p < want; p++) {
      float *k = nullptr, *v = nullptr;
      int rc;
      if ((rc = dev_alloc(d, (void **)&k, bytes))) return rc;  // zero-filled, as the dense cache starts
      if ((rc = dev_alloc(d, (void **)&v, bytes))) return rc;
      L.k_page_host.push_back(k);
      L.v_page_host.push_back(v);
    }
    int rc;
    if ((rc = cthip_h2d(L.k_pages + have, L.k_page_host.data() + have, sizeof(float *) * (want - have)))) return rc;
    if ((rc = cthip_h2d(L.v_pages + have, L.v_page_host.data() + have, sizeof(float *) * (want - have)))) return rc;
  }
  return 0;
}

static int queue_step(Decoder *d, bool with_head, bool embed = true);
static int queue_head(Decoder *d);

// S = W.gamma and C = W.beta + bias for a LayerNorm that precedes the Linear W
static int make_fold(Decoder *d, const WMat *w, const float *gamma, const float *beta, const float *bias, float **S,
                     float **C) {
  int rc;
  if ((rc = dev_alloc(d, (void **)S, sizeof(float) * (size_t)w->rows))) return rc;
  if ((rc = dev_alloc(d, (void **)C, sizeof(float) * (size_t)w->rows))) return rc;
  GemvArgs a = {};
  a.x = gamma;
  a.y = *S;
  a.x_stride = w->cols;
  a.y_stride = w->rows;
  if ((rc = launch_gemv(w, a, 1))) return rc;
  GemvArgs b = {};
  b.x = beta;
  b.bias = bias;
  b.y = *C;
  b.x_stride = w->cols;
  b.y_stride = w->rows;
  return launch_gemv(w, b, 1);
}

static int finalize(Decoder *d) {
  if (d->finalized) return 0;
  const cthip_decoder_config &c = d->cfg;
  for (const std::string &k : d->required)
    if (!d->raw.count(k)) return fail(CTHIP_E_STATE, "decoder: tensor '%s' has not been loaded", k.c_str());
  const int D = c.dim, F = c.ffn, V = c.vocab, KD = kv_dim(c);
  int rc;
  char b[128];
  d->layers.resize(c.n_layers);
  auto key = [&](int l, const char *s) {
    snprintf(b, sizeof(b), c.arch == CTHIP_ARCH_GPT2 ? "h.%d.%s" : "layers.%d.%s", l, s);
    return std::string(b);
  };
#define TRY(e)                 \
  do {                         \
    if ((rc = (e))) return rc; \
  } while (0)
  if (c.arch == CTHIP_ARCH_GPT2) {
    TRY(to_f32(d, "wte.weight", (int64_t)V * D, &d->wte));
    TRY(to_f32(d, "wpe.weight", (int64_t)c.max_seq * D, &d->wpe));
    TRY(to_f32(d, "ln_f.affine", D, &d->lnf_g));
    TRY(to_f32(d, "ln_f.bias", D, &d->lnf_b));
    TRY(to_wmat(d, {"lm_head.weight"}, V, D, &d->lm_head));
    for (int l = 0; l < c.n_layers; l++) {
      Layer &L = d->layers[l];
      TRY(to_f32(d, key(l, "ln_1.affine"), D, &L.ln1_g));
      TRY(to_f32(d, key(l, "ln_1.bias"), D, &L.ln1_b));
      TRY(to_wmat(d, {key(l, "attn.c_attn.weight")}, 3 * D, D, &L.attn));
      TRY(to_f32(d, key(l, "attn.c_attn.bias"), 3 * D, &L.attn_b));
      TRY(to_wmat(d, {key(l, "attn.c_proj.weight")}, D, D, &L.proj));
      TRY(to_f32(d, key(l, "attn.c_proj.bias"), D, &L.proj_b));
      TRY(to_f32(d, key(l, "ln_2.affine"), D, &L.ln2_g));
      TRY(to_f32(d, key(l, "ln_2.bias"), D, &L.ln2_b));
      TRY(to_wmat(d, {key(l, "mlp.c_fc.weight")}, F, D, &L.fc));
      TRY(to_f32(d, key(l, "mlp.c_fc.bias"), F, &L.fc_b));
      TRY(to_wmat(d, {key(l, "mlp.c_proj.weight")}, D, F, &L.fc2));
      TRY(to_f32(d, key(l, "mlp.c_proj.bias"), D, &L.fc2_b));
      TRY(make_fold(d, L.attn, L.ln1_g, L.ln1_b, L.attn_b, &L.attn_s, &L.attn_c));
      TRY(make_fold(d, L.fc, L.ln2_g, L.ln2_b, L.fc_b, &L.fc_s, &L.fc_c));
    }
    TRY(make_fold(d, d->lm_head, d->lnf_g, d->lnf_b, nullptr, &d->lm_s, &d->lm_c));
  } else {
    TRY(to_f32(d, "tok_embeddings.weight", (int64_t)V * D, &d->wte));
    TRY(to_f32(d, "norm.weight", D, &d->lnf_g));
    TRY(to_wmat(d, {"output.weight"}, V, D, &d->lm_head));
    for (int l = 0; l < c.n_layers; l++) {
      Layer &L = d->layers[l];
      TRY(to_f32(d, key(l, "attention_norm.weight"), D, &L.ln1_g));
      TRY(to_wmat(d, {key(l, "attention.wq.weight"), key(l, "attention.wk.weight"), key(l, "attention.wv.weight")},
                  D + 2 * KD, D, &L.attn));
      TRY(to_wmat(d, {key(l, "attention.wo.weight")}, D, D, &L.proj));
      TRY(to_f32(d, key(l, "ffn_norm.weight"), D, &L.ln2_g));
      // gate and up rows interleaved when the GEMV variant keeps a row pair in one wavefront: SwiGLU then
      // happens in that launch's epilogue and the down projection reads ffn floats instead of 2 * ffn
      L.fc_pairs = gemv_pair_swiglu_ok(d->raw.at(key(l, "feed_forward.w1.weight")).type, 2 * (int64_t)F, D);
      TRY(to_wmat(d, {key(l, "feed_forward.w1.weight"), key(l, "feed_forward.w3.weight")}, 2 * F, D, &L.fc, L.fc_pairs));
      TRY(to_wmat(d, {key(l, "feed_forward.w2.weight")}, D, F, &L.fc2));
    }
  }
  // raw GGUF bytes are no longer needed
  for (auto &kv : d->raw) cthip_free(kv.second.dev);
  d->raw.clear();
  // embeddings are read one row per step; norms/biases were counted in to_f32, remove the tables
  d->vector_bytes -= 4 * (int64_t)V * D;
  if (c.arch == CTHIP_ARCH_GPT2) d->vector_bytes -= 4 * (int64_t)c.max_seq * D;

  d->kvq = state().kv_cache == 1;
  d->kvp = state().kv_cache == 2;
  if (d->kvq && KD % 32) return fail(CTHIP_E_UNSUPPORTED, "decoder: a Q8_0 KV cache needs rows of whole 32-element blocks, not %d", KD);
  if (d->kvp && KD % 4) return fail(CTHIP_E_UNSUPPORTED, "decoder: a paged KV cache needs rows of a multiple of four floats, not %d", KD);
  for (int l = 0; l < c.n_layers; l++) {
    Layer &L = d->layers[l];
    if (d->kvp) {  // tables of page pointers, all null: pages are opened as positions are reached (ensure_pages)
      const size_t np = (size_t)(c.max_seq + kKvPageRows - 1) / kKvPageRows;
      TRY(dev_alloc(d, (void **)&L.k_pages, sizeof(float *) * np));
      TRY(dev_alloc(d, (void **)&L.v_pages, sizeof(float *) * np));
      continue;
    }
    if (d->kvq) {  // zero quants and zero scales: rows of zeros, as the fp32 cache starts
      TRY(dev_alloc(d, &L.kq, (size_t)c.max_seq * KD));
      TRY(dev_alloc(d, &L.vq, (size_t)c.max_seq * KD));
      TRY(dev_alloc(d, &L.kdq, sizeof(unsigned short) * (size_t)c.max_seq * (KD / 32)));
      TRY(dev_alloc(d, &L.vdq, sizeof(unsigned short) * (size_t)c.max_seq * (KD / 32)));
      continue;
    }
    // merge-kv-cache creates (B, max_len, H, Dh) zeros once (layers.lisp:25-26)
    TRY(dev_alloc(d, (void **)&L.k_cache, sizeof(float) * (size_t)c.max_seq * KD));
    TRY(dev_alloc(d, (void **)&L.v_cache, sizeof(float) * (size_t)c.max_seq * KD));
  }
  const int hdim = c.arch == CTHIP_ARCH_GPT2 ? F : 2 * F;
  TRY(dev_alloc(d, (void **)&d->x, sizeof(float) * D));
  TRY(dev_alloc(d, (void **)&d->q, sizeof(float) * D));
  TRY(dev_alloc(d, (void **)&d->kv_tmp, sizeof(float) * 2 * KD));
  TRY(dev_alloc(d, (void **)&d->att, sizeof(float) * D));
  {
    // long contexts: the keys of a head shared by as many workgroups as give every compute unit one (at most 16):
    // all of a launch's workgroups are then resident together and ask for their rows at once
    const int Dh = D / c.n_heads;
    int ranges = c.max_seq >= 512 ? state().compute_units / c.n_heads : 1;
    ranges = ranges < 1 ? 1 : ranges > kAttnSplitMaxRanges ? kAttnSplitMaxRanges : ranges;
    if (state().attn_split > 1) ranges = state().attn_split;  // (a given number of ranges)
    if (ranges > 1 && state().attn_split) {
      TRY(dev_alloc(d, (void **)&d->att_split.part, sizeof(float) * (size_t)c.n_heads * ranges * (Dh + 2)));
      TRY(dev_alloc(d, (void **)&d->att_split.count, sizeof(int) * (size_t)c.n_heads));  // zero-filled
      d->att_split.ranges = ranges;
    }
  }
  TRY(dev_alloc(d, (void **)&d->h, sizeof(float) * hdim));
  TRY(dev_alloc(d, (void **)&d->logits, sizeof(float) * V));
  TRY(dev_alloc(d, (void **)&d->tokpos, 256));
  TRY(dev_alloc(d, (void **)&d->token64, 256));
  TRY(dev_alloc(d, (void **)&d->history, sizeof(int64_t) * (size_t)(c.max_seq + 1)));
  TRY(dev_alloc(d, (void **)&d->hist_n, 256));
  TRY(dev_alloc(d, (void **)&d->ctrl, 256));
  {
    const int none[2] = {-1, 0};
    TRY(cthip_h2d(d->ctrl, none, sizeof(none)));
    CTHIP_CHECK(hipHostMalloc((void **)&d->ctrl_host, 256, hipHostMallocDefault));
    CTHIP_CHECK(hipEventCreateWithFlags(&d->ctrl_ev, hipEventDisableTiming));
  }
  TRY(dev_alloc(d, (void **)&d->am_val, sizeof(float) * kGemvMaxWaves));
  TRY(dev_alloc(d, (void **)&d->am_idx, sizeof(int) * kGemvMaxWaves));

  {
    // A step reads every weight once.  Past the Infinity Cache (three quarters of it: the KV cache and the
    // activations live there too) nothing of that stream survives to the next step, so it is requested
    // non-temporally and stops evicting what the step does reuse.
    std::vector<WMat *> ws = {d->lm_head};
    for (Layer &L : d->layers) ws.insert(ws.end(), {L.attn, L.proj, L.fc, L.fc2});
    int64_t total = 0;
    for (WMat *w : ws) total += w ? w->q_bytes + w->d_bytes : 0;
    for (WMat *w : ws)
      if (w) w->stream = total > kInfinityCacheBytes / 4 * 3;
  }
  if (c.arch == CTHIP_ARCH_GPT2 && state().decode_flow && !d->kvq && !d->kvp) {
    bool ok = true;
    for (int l = 0; l < c.n_layers && ok; l++) {
      Layer &L = d->layers[l];
      ok = dec_flow_supported(L.attn->type, L.proj->type, L.fc->type, L.fc2->type, D, c.n_heads, F, c.n_layers);
    }
    if (ok) {
      const int H = c.n_heads, NM = F / 32, NL = c.n_layers;
      std::vector<FlowLayer> fl(NL);
      for (int l = 0; l < NL; l++) {
        Layer &L = d->layers[l];
        TRY(dec_relay_heads(L.fc2, 32, &L.fc2_sq, &L.fc2_sd));  // 32-column slabs: one per MLP workgroup
        d->owned.insert(d->owned.end(), {L.fc2_sq, L.fc2_sd});
        FlowLayer &f = fl[l];
        f.attn_q = L.attn->q;
        f.attn_d = (const unsigned short *)L.attn->d;
        f.attn_s = L.attn_s;
        f.attn_c = L.attn_c;
        f.proj_q = L.proj->q;
        f.proj_d = (const unsigned short *)L.proj->d;
        f.proj_b = L.proj_b;
        f.fc_q = L.fc->q;
        f.fc_d = (const unsigned short *)L.fc->d;
        f.fc_s = L.fc_s;
        f.fc_c = L.fc_c;
        f.fc2_sq = L.fc2_sq;
        f.fc2_sd = (const unsigned short *)L.fc2_sd;
        f.fc2_b = L.fc2_b;
        f.ln1_g = L.ln1_g;
        f.ln2_g = L.ln2_g;
        f.kc = L.k_cache;
        f.vc = L.v_cache;
      }
      FlowArgs &fa = d->flow_args;
      FlowLayer *dl = nullptr;
      TRY(dev_alloc(d, (void **)&dl, sizeof(FlowLayer) * NL));
      TRY(cthip_h2d(dl, fl.data(), sizeof(FlowLayer) * NL));
      fa.layers = dl;
      fa.n_layers = NL;
      fa.D = D;
      fa.H = H;
      fa.F = F;
      fa.NM = NM;
      fa.eps = c.eps;
      // zero-filled: no element carries a tag of any step (epochs start at 1)
      int cx, co, cxp;
      dec_flow_copies(&cx, &co, &cxp);
      const size_t per_layer = (size_t)D * (cx + 3 + co + cxp + NM);
      unsigned long long *ll = nullptr;
      TRY(dev_alloc(d, (void **)&ll, 8 * per_layer * NL));
      fa.X = ll;
      fa.QKV = fa.X + (size_t)cx * NL * D;
      fa.O = fa.QKV + (size_t)NL * 3 * D;
      fa.XP = fa.O + (size_t)co * NL * D;
      fa.PM = fa.XP + (size_t)cxp * NL * D;
      fa.x0 = d->x;
      fa.x_out = d->x;
      fa.tokpos = d->tokpos;
      TRY(dev_alloc(d, (void **)&fa.state, 256));
      if (state().decode_flow == 2)
        TRY(dev_alloc(d, (void **)&fa.trace, sizeof(long long) * 4 * (size_t)NL * dec_flow_grid(D, H, F)));
      const int st0[2] = {1, 0};
      TRY(cthip_h2d(fa.state, st0, sizeof(st0)));
      d->flow = true;
    }
  }
  // (a cache of Q8_0 rows keeps the three launches: the attention launch has a variant over the planes)
  if (c.arch == CTHIP_ARCH_GPT2 && state().decode_fused && !d->kvp && !d->flow &&
      dec_fused_supported(d->layers[0].attn->type, d->layers[0].proj->type, d->layers[0].fc->type,
                          d->layers[0].fc2->type, D, c.n_heads, F)) {
    // the per-XCD accumulators assume what gfx950 has: XCD ids 0..7
    int max_id = -1;
    TRY(dec_xcd_probe(&max_id));
    d->fused = max_id >= 0 && max_id < kDecXcds;
    for (int l = 0; l < c.n_layers && d->fused; l++) {
      Layer &L = d->layers[l];
      if (L.attn->type != d->layers[0].attn->type || L.proj->type != L.attn->type || L.fc->type != L.attn->type || L.fc2->type != L.attn->type)
        d->fused = false;
    }
    if (d->fused) {
      for (int l = 0; l < c.n_layers; l++) {
        Layer &L = d->layers[l];
        TRY(dec_relay_heads(L.proj, D / c.n_heads, &L.proj_hq, &L.proj_hd));
        TRY(dec_relay_slabs(L.fc2, &L.fc2_sq, &L.fc2_sd));
        for (void *p : {L.proj_hq, L.proj_hd, L.fc2_sq, L.fc2_sd})
          if (p) d->owned.push_back(p);
      }
      TRY(dev_alloc(d, (void **)&d->x2, sizeof(float) * D));
      TRY(dev_alloc(d, (void **)&d->patt, sizeof(float) * (size_t)c.n_heads * D));
      TRY(dev_alloc(d, (void **)&d->pmlp, sizeof(long long) * (size_t)kDecXcds * D));
    }
  }
  if (c.arch == CTHIP_ARCH_LLAMA && state().decode_fused && !d->kvq && !d->kvp &&
      gqa_fused_supported(d->layers[0].attn->type, d->layers[0].proj->type, d->layers[0].fc->type, d->layers[0].fc2->type,
                          D, c.n_heads, c.n_kv_heads, F)) {
    int max_id = -1;
    TRY(dec_xcd_probe(&max_id));
    d->fused_gqa = max_id >= 0 && max_id < kDecXcds;
    for (int l = 0; l < c.n_layers && d->fused_gqa; l++) {
      Layer &L = d->layers[l];
      if (L.attn->type != CTHIP_Q4_0 || L.proj->type != CTHIP_Q4_0 || L.fc->type != CTHIP_Q4_0 || L.fc2->type != CTHIP_Q4_0)
        d->fused_gqa = false;
    }
    if (d->fused_gqa) {
      for (int l = 0; l < c.n_layers; l++) {
        Layer &L = d->layers[l];
        TRY(gqa_relay_groups(L.proj, D / c.n_heads, &L.proj_hq, &L.proj_hd));
        TRY(gqa_relay_slabs(L.fc2, &L.fc2_sq, &L.fc2_sd));
        d->owned.insert(d->owned.end(), {L.proj_hq, L.proj_hd, L.fc2_sq, L.fc2_sd});
      }
      TRY(dev_alloc(d, (void **)&d->x2, sizeof(float) * D));
      TRY(dev_alloc(d, (void **)&d->pattn, sizeof(long long) * (size_t)kDecXcds * D));
      TRY(dev_alloc(d, (void **)&d->pmlp, sizeof(long long) * (size_t)kDecXcds * D));
      TRY(cthip_memset(d->pattn, 0, sizeof(long long) * (size_t)kDecXcds * D));
    }
  }
  // three-launch layers: from this position on the attention is a launch of its own (Q8_0 cache rows are a quarter of
  // the bytes, the repeated attention stays the cheaper one half as far again)
  if (!d->flow && (d->fused || d->fused_gqa) && d->att_split.ranges > 1 && state().attn_long_from > 0) {
    const int64_t from = d->kvq ? (int64_t)state().attn_long_from * 3 / 2 : state().attn_long_from;
    if (from < c.max_seq) d->long_from = (int)from;
  }
  if (!state().decoder_graph) d->use_graph = false;
  if (d->use_graph) {
    hipStream_t st = state().stream;
    // 0: one step with the head; 1: one step without (prompt rows fed one by one); 2: kStepsPerGraph steps
    // with their heads back to back (the device-resident loop: fewer graph launches per token)
    for (int pass = 0; pass < (d->long_from > 0 ? 6 : 3); pass++) {
      const int mode = pass / 3;
      d->long_mode = mode == 1;
      hipGraph_t g = nullptr;
      CTHIP_CHECK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
      // the device-resident loop (pass 2) only ever follows a head, which leaves the next input in place
      rc = queue_step(d, pass % 3 != 1, pass % 3 != 2);
      for (int k = 1; pass % 3 == 2 && k < kStepsPerGraph && !rc; k++) rc = queue_step(d, true, false);
      hipError_t e = hipStreamEndCapture(st, &g);
      if (rc) {
        if (g) (void)hipGraphDestroy(g);
        d->long_mode = false;
        return rc;
      }
      if (e != hipSuccess) return fail((int)e, "decoder: hipStreamEndCapture -> %s", hipGetErrorString(e));
      hipGraphExec_t ex = nullptr;
      e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
      (void)hipGraphDestroy(g);
      if (e != hipSuccess) return fail((int)e, "decoder: hipGraphInstantiate -> %s", hipGetErrorString(e));
      (pass % 3 == 0 ? d->g_step : pass % 3 == 1 ? d->g_body : d->g_multi)[mode] = ex;
    }
    d->long_mode = false;
  }
#undef TRY
  d->finalized = true;
  return 0;
}

// queues one decode step on the stream; token and position are read from d->tokpos
static int queue_step(Decoder *d, bool with_head, bool embed) {
  const cthip_decoder_config &c = d->cfg;
  const int D = c.dim, F = c.ffn, V = c.vocab, KD = kv_dim(c), Dh = c.dim / c.n_heads;
  const int *tok = d->tokpos, *pos = d->tokpos + 1;
  int rc;
#define TRY(e)                 \
  do {                         \
    if ((rc = (e))) return rc; \
  } while (0)
  const bool gpt2 = c.arch == CTHIP_ARCH_GPT2;
  // embed = false: the previous step's head has already gathered this step's input (queue_head)
  if (embed) TRY(launch_embedding(d->x, d->wte, nullptr, tok, 1, V, D, gpt2 ? d->wpe : nullptr, pos, c.max_seq));
  if (d->flow) {
    TRY(launch_dec_flow(d->flow_args));
    if (with_head) TRY(queue_head(d));
    return 0;
  }
  if (d->fused) {
    // Three launches per layer.  The residual stream alternates between d->x and d->x2 as "base + bias +
    // partials": each launch adds up what its predecessor left and block 0 stores the sum for the launch after.
    // four workgroups per head repeat the head's attention and share its slab of the projection: what one
    // compute unit must fetch bounds a launch (GPT-2 small: 182 -> 173 us / step; six or twelve: no further gain)
    const int replicas = 4;
    const int skip = state().decode_skip;  // knock-out timing only
    for (int l = 0; l < c.n_layers; l++) {
      Layer &L = d->layers[l];
      DecQkvArgs qa = {};
      qa.st.base = d->x;
      qa.st.bias = l ? d->layers[l - 1].fc2_b : nullptr;
      qa.st.iparts = d->pmlp;
      qa.st.gamma = L.ln1_g;
      qa.st.xout = d->x2;
      qa.st.eps = c.eps;
      qa.st.D = D;
      qa.wq = L.attn->q;
      qa.wd = (const unsigned short *)L.attn->d;
      qa.fold_s = L.attn_s;
      qa.fold_c = L.attn_c;
      qa.q = d->q;
      qa.kc = d->kvq ? d->kv_tmp : L.k_cache;  // Q8_0 rows: the new row is quantised by the attention launch
      qa.vc = d->kvq ? d->kv_tmp + D : L.v_cache;
      qa.kv_stride = d->kvq ? 0 : D;
      qa.pos = pos;
      qa.rows = 3 * D;
      if (!(skip & 1)) TRY(launch_dec_qkv(qa, L.attn->type, l > 0));
      DecAttnArgs aa = {};
      aa.q = d->q;
      aa.kc = L.k_cache;
      aa.vc = L.v_cache;
      aa.pos = pos;
      aa.pq = L.proj_hq;
      aa.pd = (const unsigned short *)L.proj_hd;
      aa.part = d->patt;
      aa.zero = d->pmlp;
      aa.zero_n16 = (int64_t)kDecXcds * D * 8 / 16;
      if (d->kvq) {
        DecAttnQ8Args a8 = {};
        a8.q = d->q;
        a8.newkv = d->kv_tmp;
        a8.kq = (signed char *)L.kq;
        a8.vq = (signed char *)L.vq;
        a8.kd = (unsigned short *)L.kdq;
        a8.vd = (unsigned short *)L.vdq;
        a8.pos = pos;
        a8.pq = aa.pq;
        a8.pd = aa.pd;
        a8.part = aa.part;
        a8.zero = aa.zero;
        a8.zero_n16 = aa.zero_n16;
        if (skip & 2) {
        } else if (d->long_mode) {  // rotation (none here), quantisation, append and attention, then the projection
          TRY(launch_attn_q8_step(d->att, d->q, d->kv_tmp, L.kq, L.kdq, L.vq, L.vdq, pos, c.n_heads, c.n_kv_heads, Dh, 0.0f, &d->att_split));
          aa.att_in = d->att;
          TRY(launch_dec_attn_proj(aa, L.attn->type, c.n_heads, D, replicas));
        } else {
          TRY(launch_dec_attn_proj_q8(a8, L.attn->type, c.n_heads, D, replicas));
        }
      } else if (!(skip & 2)) {
        if (d->long_mode) {
          TRY(launch_attn(d->att, d->q, L.k_cache, L.v_cache, 1, 0, pos, c.max_seq, c.n_heads, c.n_kv_heads, Dh, &d->att_split));
          aa.att_in = d->att;
        }
        TRY(launch_dec_attn_proj(aa, L.attn->type, c.n_heads, D, replicas));
      }
      DecMlpArgs ma = {};
      ma.st.base = d->x2;
      ma.st.bias = L.proj_b;
      ma.st.fparts = d->patt;
      ma.st.gamma = L.ln2_g;
      ma.st.xout = d->x;
      ma.st.eps = c.eps;
      ma.st.D = D;
      ma.wq = L.fc->q;
      ma.wd = (const unsigned short *)L.fc->d;
      ma.fold_s = L.fc_s;
      ma.fold_c = L.fc_c;
      ma.pq = L.fc2_sq;
      ma.pd = (const unsigned short *)L.fc2_sd;
      ma.accum = d->pmlp;
      if (!(skip & 4)) TRY(launch_dec_mlp(ma, L.attn->type, F, c.n_heads));
    }
    DecStage fin = {};
    fin.base = d->x;
    fin.bias = d->layers[c.n_layers - 1].fc2_b;
    fin.iparts = d->pmlp;
    fin.D = D;
    if (!(skip & 8)) TRY(launch_dec_sum(fin, d->x));
    if (with_head && !(skip & 16)) TRY(queue_head(d));
    return 0;
  }
  if (d->fused_gqa) {
    // The same three launches for grouped-query layers.  Both column Linears add into per-XCD accumulators:
    // pattn (attention projection, cleared by the qkv launch) and pmlp (down projection, cleared by the attention
    // launch); the residual stream alternates between d->x and d->x2 as "base + accumulators".
    // workgroups per query head: as many as fill the compute units once (32 heads: 8; measured 0.560 / 0.550 /
    // 0.540 / 0.620 ms per Llama-1.1B step with 2 / 4 / 8 / 16)
    int replicas = 4;
    while (replicas < 8 && c.n_heads * replicas * 2 <= state().compute_units && D % (replicas * 2) == 0) replicas *= 2;
    const int64_t acc16 = (int64_t)kDecXcds * D * 8 / 16;
    for (int l = 0; l < c.n_layers; l++) {
      Layer &L = d->layers[l];
      GqaQkvArgs qa = {};
      qa.st.base = d->x;
      qa.st.iparts = d->pmlp;
      qa.st.gamma = L.ln1_g;
      qa.st.xout = d->x2;
      qa.st.eps = c.eps;
      qa.st.D = D;
      qa.wq = L.attn->q;
      qa.wd = (const unsigned short *)L.attn->d;
      qa.q = d->q;
      qa.kc = L.k_cache;
      qa.vc = L.v_cache;
      qa.pos = pos;
      qa.rows = D + 2 * KD;
      qa.KD = KD;
      qa.DH = Dh;
      qa.log2_base = log2f(c.rope_base);
      qa.zero = d->pattn;
      qa.zero_n16 = acc16;
      TRY(launch_gqa_qkv(qa, l > 0));
      GqaAttnArgs aa = {};
      aa.q = d->q;
      aa.kc = L.k_cache;
      aa.vc = L.v_cache;
      aa.pos = pos;
      aa.pq = L.proj_hq;
      aa.pd = (const unsigned short *)L.proj_hd;
      aa.accum = d->pattn;
      aa.zero = d->pmlp;
      aa.zero_n16 = acc16;
      aa.D = D;
      aa.KD = KD;
      if (d->long_mode) {
        TRY(launch_attn(d->att, d->q, L.k_cache, L.v_cache, 1, 0, pos, c.max_seq, c.n_heads, c.n_kv_heads, Dh, &d->att_split));
        aa.att_in = d->att;
      }
      TRY(launch_gqa_attn_proj(aa, c.n_heads, c.n_kv_heads, replicas));
      GqaMlpArgs ma = {};
      ma.st.base = d->x2;
      ma.st.iparts = d->pattn;
      ma.st.gamma = L.ln2_g;
      ma.st.xout = d->x;
      ma.st.eps = c.eps;
      ma.st.D = D;
      ma.wq = L.fc->q;
      ma.wd = (const unsigned short *)L.fc->d;
      ma.gate_stride = L.fc_pairs ? 2 : 1;
      ma.up_off = L.fc_pairs ? 1 : F;
      ma.pq = L.fc2_sq;
      ma.pd = (const unsigned short *)L.fc2_sd;
      ma.accum = d->pmlp;
      TRY(launch_gqa_mlp(ma, F, c.n_kv_heads));
    }
    DecStage fin = {};
    fin.base = d->x;
    fin.bias = nullptr;
    fin.iparts = d->pmlp;
    fin.D = D;
    TRY(launch_dec_sum(fin, d->x));
    if (with_head) TRY(queue_head(d));
    return 0;
  }
  for (int l = 0; l < c.n_layers; l++) {
    Layer &L = d->layers[l];
    GemvArgs a = {};
    a.x = d->x;
    a.pro = gpt2 ? CTHIP_PRO_LAYERNORM : CTHIP_PRO_RMSNORM;
    a.norm_g = L.ln1_g;
    a.norm_b = L.ln1_b;
    a.eps = c.eps;
    a.bias = gpt2 ? L.attn_c : L.attn_b;
    a.fold_s = L.attn_s;
    a.bias0 = L.attn_b;
    a.y = d->q;
    a.split1 = D;
    a.split2 = D + KD;
    a.x_stride = D;
    a.y_stride = D;
    if (gpt2 && !d->kvq && !d->kvp) {
      a.y1 = L.k_cache;
      a.y2 = L.v_cache;
      a.pos = pos;
      a.pos_stride = KD;
    } else {
      a.y1 = d->kv_tmp;
      a.y2 = d->kv_tmp + KD;
      a.pos = nullptr;
      a.pos_stride = 0;
    }
    TRY(launch_gemv(L.attn, a, 1));
    if (d->kvq) {
      // the new row is in kv_tmp (k then v): one launch rotates q and k where the model rotates, quantises the row
      // into the cache at `pos` and attends over the Q8_0 rows
      TRY(launch_attn_q8_step(d->att, d->q, d->kv_tmp, L.kq, L.kdq, L.vq, L.vdq, pos, c.n_heads, c.n_kv_heads, Dh,
                              gpt2 ? 0.0f : c.rope_base, &d->att_split));
    } else if (d->kvp) {
      // the new row is in kv_tmp (k then v): one launch rotates q and k where the model rotates, copies the row into
      // its page and attends over the pages
      TRY(launch_attn_paged_step(d->att, d->q, d->kv_tmp, L.k_pages, L.v_pages, pos, c.n_heads, c.n_kv_heads, Dh,
                                 gpt2 ? 0.0f : c.rope_base, &d->att_split));
    } else if (!gpt2) {
      // q and the new key are rotated inside the attention launch, which also appends k / v at `pos`
      TRY(launch_attn_rope_append(d->att, d->q, L.k_cache, L.v_cache, d->kv_tmp, pos, c.n_heads, c.n_kv_heads, Dh,
                                  c.rope_base, &d->att_split));
    } else {
      TRY(launch_attn(d->att, d->q, L.k_cache, L.v_cache, 1, 0, pos, c.max_seq, c.n_heads, c.n_kv_heads, Dh, &d->att_split));
    }
    GemvArgs p = {};
    p.x = d->att;
    p.bias = L.proj_b;
    p.residual = d->x;
    p.y = d->x;
    p.x_stride = D;
    p.y_stride = D;
    TRY(launch_gemv(L.proj, p, 1));
    GemvArgs f = {};
    f.x = d->x;
    f.pro = gpt2 ? CTHIP_PRO_LAYERNORM : CTHIP_PRO_RMSNORM;
    f.norm_g = L.ln2_g;
    f.norm_b = L.ln2_b;
    f.eps = c.eps;
    f.bias = gpt2 ? L.fc_c : L.fc_b;
    f.fold_s = L.fc_s;
    f.bias0 = L.fc_b;
    f.act = gpt2 ? CTHIP_ACT_GELU : CTHIP_ACT_NONE;
    f.pair_swiglu = L.fc_pairs ? 1 : 0;
    f.y = d->h;
    f.x_stride = D;
    f.y_stride = (gpt2 || L.fc_pairs) ? F : 2 * F;
    TRY(launch_gemv(L.fc, f, 1));
    GemvArgs g = {};
    g.x = d->h;
    g.pro = (gpt2 || L.fc_pairs) ? CTHIP_PRO_NONE : CTHIP_PRO_SWIGLU;
    g.bias = L.fc2_b;
    g.residual = d->x;
    g.y = d->x;
    g.x_stride = (gpt2 || L.fc_pairs) ? F : 2 * F;
    g.y_stride = D;
    TRY(launch_gemv(L.fc2, g, 1));
  }
  if (with_head) TRY(queue_head(d));
#undef TRY
  return 0;
}

// ln_f -> lm_head GEMV on d->x, greedy token -> tokpos[0] and the history, position + 1
static int queue_head(Decoder *d) {
  const cthip_decoder_config &c = d->cfg;
  const bool gpt2 = c.arch == CTHIP_ARCH_GPT2;
  GemvArgs o = {};
  o.x = d->x;
  o.pro = gpt2 ? CTHIP_PRO_LAYERNORM : CTHIP_PRO_RMSNORM;
  o.norm_g = d->lnf_g;
  o.norm_b = d->lnf_b;
  o.eps = c.eps;
  o.bias = d->lm_c;
  o.fold_s = d->lm_s;
  o.bias0 = nullptr;
  o.y = d->logits;
  o.x_stride = c.dim;
  o.y_stride = c.vocab;
  // greedy token -> next step's input; position advances (apps/gpt2/gpt2.lisp:105-107)
  o.am_val = d->am_val;
  o.am_idx = d->am_idx;
  o.am_token64 = (long long *)d->token64;
  o.am_tok = d->tokpos;
  o.am_pos = d->tokpos + 1;
  o.am_hist = (long long *)d->history;
  o.am_hist_n = d->hist_n;
  o.am_ctrl = d->ctrl;
  // ... and its embedding rows become the next step's input, in the block that settles the token
  o.nx_out = d->x;
  o.nx_wte = d->wte;
  o.nx_wpe = gpt2 ? d->wpe : nullptr;
  o.nx_dim = c.dim;
  o.nx_vocab = c.vocab;
  o.nx_max_pos = c.max_seq;
  return launch_gemv(d->lm_head, o, 1);
}

// A prompt of s >= kPrefillMin rows as one batch (the reference's forward with s > 1): every Linear is
// an MFMA GEMM over the s rows (weights dequantised while staged), attention runs all s query rows
// against the cache under the causal mask; only the last row goes through lm_head.
static const int kPrefillMin = 8;
static int prefill(Decoder *d, const int *ids, int s, int n) {
  const cthip_decoder_config &c = d->cfg;
  const bool gpt2 = c.arch == CTHIP_ARCH_GPT2;
  const int D = c.dim, F = c.ffn, V = c.vocab, KD = kv_dim(c), Dh = c.dim / c.n_heads;
  const int QW = D + 2 * KD, HW = gpt2 ? F : 2 * F;
  const int prec = state().gemm_precision;
  int rc = 0;
  float *X = nullptr, *XN = nullptr, *QKV = nullptr, *Q = nullptr, *ATT = nullptr, *Hb = nullptr, *G = nullptr, *KF = nullptr, *VF = nullptr;
  int *ids_dev = nullptr;
  std::vector<void *> tmp;
  auto alloc = [&](void **p, size_t bytes) {
    int r = alloc_scratch(p, bytes);  // every temporary below is fully written before it is read
    if (r == 0) tmp.push_back(*p);
    return r;
  };
#define TRY(e)                \
  do {                        \
    if ((rc = (e))) goto done; \
  } while (0)
  TRY(alloc((void **)&X, sizeof(float) * (size_t)s * D));
  TRY(alloc((void **)&XN, sizeof(float) * (size_t)s * D));
  TRY(alloc((void **)&QKV, sizeof(float) * (size_t)s * QW));
  TRY(alloc((void **)&Q, sizeof(float) * (size_t)s * D));
  TRY(alloc((void **)&ATT, sizeof(float) * (size_t)s * D));
  TRY(alloc((void **)&Hb, sizeof(float) * (size_t)s * HW));
  if (!gpt2) TRY(alloc((void **)&G, sizeof(float) * (size_t)s * F));
  if (d->kvq || d->kvp) {
    TRY(alloc((void **)&KF, sizeof(float) * (size_t)(n + s) * KD));
    TRY(alloc((void **)&VF, sizeof(float) * (size_t)(n + s) * KD));
  }
  TRY(alloc((void **)&ids_dev, sizeof(int) * (size_t)s));
  TRY(cthip_h2d(ids_dev, ids, sizeof(int) * (size_t)s));
  {
    int tp[2] = {ids[s - 1], n};  // position base for the learned position rows
    TRY(cthip_h2d(d->tokpos, tp, sizeof(tp)));
  }
  TRY(launch_embedding(X, d->wte, nullptr, ids_dev, s, V, D, gpt2 ? d->wpe : nullptr, d->tokpos + 1, c.max_seq));
  {
    // A row-split Linear (attention projection, second MLP Linear) whose reduction axis was shared among several
    // workgroups per tile leaves partial tiles; what follows it is the residual add and the next norm, so one pass
    // over the rows does all three (launch_reduce_norm) instead of a reduction launch and a norm launch.
    auto norm = [&](float *y, const float *x, const float *g, const float *b) {
      return gpt2 ? cthip_layernorm(y, x, g, b, c.eps, s, D) : cthip_rmsnorm(y, x, g, c.eps, s, D);
    };
    // X += W.in + bias, then XN = norm(X) with (g, b); g == nullptr: no norm follows (after the last layer)
    auto linear_residual_norm = [&](const WMat *w, const float *in, const float *bias, const float *g, const float *b) {
      GemmDeferred df;
      const bool fuse = g != nullptr && reduce_norm_supported(D, 1);
      int r = launch_linear_gemm(X, w, in, s, bias, X, CTHIP_ACT_NONE, prec, fuse ? &df : nullptr);
      if (r) return r;
      if (df.ws) {
        if (reduce_norm_supported(D, df.ksplit)) {
          r = launch_reduce_norm(XN, X, df.ws, df.ksplit, (int64_t)s * D, bias, X, g, b, c.eps, s, D, !gpt2);
        } else {  // too many shares of too wide a row to hold at once: reduce, then normalise
          r = launch_splitk_reduce(X, df.ws, df.ksplit, s, D, bias, X);
          if (!r) r = norm(XN, X, g, b);
        }
        const int r2 = cthip_free(df.ws);  // stream-ordered: reused only by later work on this stream
        return r ? r : r2;
      }
      return g ? norm(XN, X, g, b) : 0;
    };
    TRY(norm(XN, X, d->layers[0].ln1_g, d->layers[0].ln1_b));
    for (int l = 0; l < c.n_layers; l++) {
      Layer &L = d->layers[l];
      if (d->kvq) {
        // attention of a prompt batch runs on fp32 rows: the cached rows [0, n) are widened into a temporary, the
        // batch's rows [n, n + s) join them (rotated where the model rotates) and are quantised into the cache
        TRY(launch_kvq_dequant(KF, L.kq, L.kdq, n, KD));
        TRY(launch_kvq_dequant(VF, L.vq, L.vdq, n, KD));
        TRY(launch_linear_gemm(QKV, L.attn, XN, s, L.attn_b, nullptr, CTHIP_ACT_NONE, prec));
        TRY(launch_qkv_split(Q, KF, VF, QKV, s, n, c.n_heads, c.n_kv_heads, Dh, gpt2 ? 0.0f : c.rope_base));
        TRY(launch_kvq_append(L.kq, L.kdq, KF + (int64_t)n * KD, KD, s, n, nullptr, KD));
        TRY(launch_kvq_append(L.vq, L.vdq, VF + (int64_t)n * KD, KD, s, n, nullptr, KD));
        TRY(launch_attn(ATT, Q, KF, VF, s, n, nullptr, n + s, c.n_heads, c.n_kv_heads, Dh));
      } else if (d->kvp) {
        // attention of a prompt batch runs on dense rows: the cached rows [0, n) are gathered out of their pages, the
        // batch's rows [n, n + s) join them (rotated where the model rotates) and are copied into their pages
        TRY(launch_kvp_gather(KF, L.k_pages, n, KD));
        TRY(launch_kvp_gather(VF, L.v_pages, n, KD));
        TRY(launch_linear_gemm(QKV, L.attn, XN, s, L.attn_b, nullptr, CTHIP_ACT_NONE, prec));
        TRY(launch_qkv_split(Q, KF, VF, QKV, s, n, c.n_heads, c.n_kv_heads, Dh, gpt2 ? 0.0f : c.rope_base));
        TRY(launch_kvp_append(L.k_pages, L.v_pages, KF + (int64_t)n * KD, VF + (int64_t)n * KD, KD, s, n, nullptr, KD));
        TRY(launch_attn(ATT, Q, KF, VF, s, n, nullptr, n + s, c.n_heads, c.n_kv_heads, Dh));
      } else {
      if (gpt2 && D % 128 == 0 && KD % 128 == 0) {
        // no rotation: the thirds of the fused projection go straight to the query rows and the cache rows
        const GemmRoute rt = {{Q, L.k_cache + (int64_t)n * KD, L.v_cache + (int64_t)n * KD}, {0, D, D + KD}, {D, KD, KD}};
        TRY(launch_linear_gemm(nullptr, L.attn, XN, s, L.attn_b, nullptr, CTHIP_ACT_NONE, prec, nullptr, &rt));
      } else {
        TRY(launch_linear_gemm(QKV, L.attn, XN, s, L.attn_b, nullptr, CTHIP_ACT_NONE, prec));
        TRY(launch_qkv_split(Q, L.k_cache, L.v_cache, QKV, s, n, c.n_heads, c.n_kv_heads, Dh, gpt2 ? 0.0f : c.rope_base));
      }
      TRY(launch_attn(ATT, Q, L.k_cache, L.v_cache, s, n, nullptr, n + s, c.n_heads, c.n_kv_heads, Dh));
      }
      TRY(linear_residual_norm(L.proj, ATT, L.proj_b, L.ln2_g, L.ln2_b));
      const float *hin = Hb;
      if (!gpt2 && L.fc_pairs && (2 * F) % 4 == 0) {  // SwiGLU in the epilogue of the gate|up launch
        TRY(launch_linear_gemm(G, L.fc, XN, s, L.fc_b, nullptr, kActSwigluPairs, prec));
        hin = G;
      } else {
        TRY(launch_linear_gemm(Hb, L.fc, XN, s, L.fc_b, nullptr, gpt2 ? CTHIP_ACT_GELU : CTHIP_ACT_NONE, prec));
        if (!gpt2) {
          if (L.fc_pairs) TRY(launch_swiglu_pairs(G, Hb, (int64_t)s * F));
          else TRY(launch_prologue(G, Hb, F, CTHIP_PRO_SWIGLU, nullptr, nullptr, 0.0f, 2 * (int64_t)F, s));
          hin = G;
        }
      }
      const bool last = l + 1 == c.n_layers;
      TRY(linear_residual_norm(L.fc2, hin, L.fc2_b, last ? nullptr : d->layers[l + 1].ln1_g, last ? nullptr : d->layers[l + 1].ln1_b));
    }
  }
  // the last row continues through the decode-step head
  TRY(cthip_d2d(d->x, X + (size_t)(s - 1) * D, sizeof(float) * D));
  {
    int tp[2] = {ids[s - 1], n + s - 1};
    TRY(cthip_h2d(d->tokpos, tp, sizeof(tp)));
  }
  TRY(queue_head(d));
#undef TRY
done:
  for (void *p : tmp) cthip_free(p);
  return rc;
}

// After a synchronising copy: did a workgroup of the one-launch step give up waiting?  The step's results are void
// then; the epoch moves on so that no tag of the failed step can match later.
static int flow_check(Decoder *d) {
  if (!d->flow) return 0;
  int st[2] = {0, 0};
  int rc = cthip_d2h(st, d->flow_args.state, sizeof(st));
  if (rc || !st[1]) return rc;
  const int next[2] = {st[0] + 2, 0};
  if ((rc = cthip_h2d(d->flow_args.state, next, sizeof(next)))) return rc;
  return fail(CTHIP_E_STATE, "decoder: a workgroup of the one-launch decode step waited for its input beyond the poll limit; "
                             "the step's results are void (are all %d workgroups resident at once?)",
              dec_flow_grid(d->cfg.dim, d->cfg.n_heads, d->cfg.ffn));
}

// `position`: where the step's row goes (what the host knows of it: never below the device's)
static int run_step(Decoder *d, bool with_head, int position) {
  const int mode = d->long_from > 0 && position >= d->long_from ? 1 : 0;
  if (d->use_graph) {
    CTHIP_CHECK(hipGraphLaunch((with_head ? d->g_step : d->g_body)[mode], state().stream));
    return 0;
  }
  d->long_mode = mode == 1;
  const int rc = queue_step(d, with_head);
  d->long_mode = false;
  return rc;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_decoder_create(void **dec, const cthip_decoder_config *cfg) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && cfg != nullptr);
  const cthip_decoder_config &c = *cfg;
  CTHIP_ARG(c.arch == CTHIP_ARCH_GPT2 || c.arch == CTHIP_ARCH_LLAMA);
  CTHIP_ARG(c.n_layers > 0 && c.dim > 0 && c.n_heads > 0 && c.ffn > 0 && c.vocab > 0 && c.max_seq > 0);
  CTHIP_ARG(c.dim % c.n_heads == 0);
  CTHIP_ARG(c.n_kv_heads > 0 && c.n_heads % c.n_kv_heads == 0);
  if (c.arch == CTHIP_ARCH_GPT2 && c.n_kv_heads != c.n_heads)
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_create: the GPT-2 shaped Transformer has n_kv_heads == n_heads");
  const int Dh = c.dim / c.n_heads;
  if (Dh != 32 && Dh != 64 && Dh != 128)
    return fail(CTHIP_E_UNSUPPORTED, "cthip_decoder_create: head_dim %d (supported: 32, 64, 128)", Dh);
  if (c.max_seq > 8192) return fail(CTHIP_E_UNSUPPORTED, "cthip_decoder_create: max_seq %d > 8192", c.max_seq);
  Decoder *d = new Decoder();
  d->cfg = c;
  build_required(d);
  *dec = d;
  return 0;
}

int cthip_decoder_destroy(void *dec) {
  if (!dec) return 0;
  Decoder *d = (Decoder *)dec;
  if (state().inited) (void)hipStreamSynchronize(state().stream);
  for (int mode = 0; mode < 2; mode++) {
    if (d->g_step[mode]) (void)hipGraphExecDestroy(d->g_step[mode]);
    if (d->g_body[mode]) (void)hipGraphExecDestroy(d->g_body[mode]);
    if (d->g_multi[mode]) (void)hipGraphExecDestroy(d->g_multi[mode]);
  }
  if (d->ctrl_host) (void)hipHostFree(d->ctrl_host);
  if (d->ctrl_ev) (void)hipEventDestroy(d->ctrl_ev);
  for (auto &kv : d->raw) cthip_free(kv.second.dev);
  for (void *p : d->owned) cthip_free(p);
  for (Layer &L : d->layers) {
    cthip_wmat_destroy(L.attn);
    cthip_wmat_destroy(L.proj);
    cthip_wmat_destroy(L.fc);
    cthip_wmat_destroy(L.fc2);
  }
  cthip_wmat_destroy(d->lm_head);
  delete d;
  return 0;
}

int cthip_decoder_load(void *dec, const char *key, int ggml_type, const void *host_raw, int64_t rows, int64_t cols) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && key != nullptr && host_raw != nullptr && rows > 0 && cols > 0);
  Decoder *d = (Decoder *)dec;
  if (d->finalized) return fail(CTHIP_E_STATE, "cthip_decoder_load: the session has already run; weights are frozen");
  bool known = false;
  for (const std::string &k : d->required)
    if (k == key) known = true;
  if (!known) return fail(CTHIP_E_BAD_ARG, "cthip_decoder_load: '%s' is not a tensor of this model", key);
  const size_t nbytes = raw_nbytes(ggml_type, rows * cols);
  if (nbytes == 0) return fail(CTHIP_E_UNSUPPORTED, "cthip_decoder_load: ggml type %d is not supported", ggml_type);
  if ((ggml_type == CTHIP_Q8_0 || ggml_type == CTHIP_Q4_0) && cols % 32)
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_load: '%s': quantised rows need cols %% 32 == 0", key);
  RawTensor r;
  r.type = ggml_type;
  r.rows = rows;
  r.cols = cols;
  r.nbytes = nbytes;
  int rc = cthip_alloc(&r.dev, nbytes);
  if (rc) return rc;
  rc = cthip_h2d(r.dev, host_raw, nbytes);
  if (rc) {
    cthip_free(r.dev);
    return rc;
  }
  auto it = d->raw.find(key);
  if (it != d->raw.end()) cthip_free(it->second.dev);
  d->raw[key] = r;
  return 0;
}

int cthip_decoder_missing(const void *dec) {
  const Decoder *d = (const Decoder *)dec;
  if (!d) return -1;
  if (d->finalized) return 0;
  int n = 0;
  for (const std::string &k : d->required)
    if (!d->raw.count(k)) n++;
  return n;
}

int cthip_decoder_forward(void *dec, const float *tokens, int s, int n, int64_t *token, float *logits_out) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && tokens != nullptr && token != nullptr);
  Decoder *d = (Decoder *)dec;
  const cthip_decoder_config &c = d->cfg;
  if (s < 1) return fail(CTHIP_E_BAD_ARG, "cthip_decoder_forward: s = %d; a forward needs at least one token", s);
  if (n < 0 || n + s > c.max_seq)
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_forward: positions %d..%d fall outside the KV cache (max_seq %d)", n,
                n + s - 1, c.max_seq);
  int rc = finalize(d);
  if (rc) return rc;
  if ((rc = ensure_pages(d, n + s))) return rc;
  int zero = 0;
  if ((rc = cthip_h2d(d->hist_n, &zero, sizeof(int)))) return rc;
  {
    const int none[2] = {-1, 0};
    if ((rc = cthip_h2d(d->ctrl, none, sizeof(none)))) return rc;
  }
  // ids arrive as floats (gpt2.lisp:95); one that equals no vocabulary index selects no row
  std::vector<int> ids(s);
  for (int i = 0; i < s; i++) {
    const float tf = tokens[i];
    ids[i] = (tf >= 0.0f && tf < (float)c.vocab && (float)(int)tf == tf) ? (int)tf : -1;
  }
  if (s >= kPrefillMin && state().prefill_gemm) {
    if ((rc = prefill(d, ids.data(), s, n))) return rc;
  } else {
    for (int i = 0; i < s; i++) {
      int tp[2] = {ids[i], n + i};
      if ((rc = cthip_h2d(d->tokpos, tp, sizeof(tp)))) return rc;
      if ((rc = run_step(d, i == s - 1, n + i))) return rc;
    }
  }
  if (logits_out && (rc = cthip_d2h(logits_out, d->logits, sizeof(float) * (size_t)c.vocab))) return rc;
  if ((rc = cthip_d2h(token, d->token64, sizeof(int64_t)))) return rc;
  if ((rc = flow_check(d))) return rc;
  d->position = n + s;
  d->primed = true;
  return 0;
}

// the loop behind cthip_decoder_generate / cthip_decoder_generate_until
static int generate_impl(Decoder *d, int steps, int eos, int64_t *tokens_out, int *n_generated) {
  if (!d->primed)
    return fail(CTHIP_E_STATE, "cthip_decoder_generate: run cthip_decoder_forward on a prompt first");
  if (d->position + steps > d->cfg.max_seq)
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_generate: %d more tokens from position %d overflow max_seq %d", steps,
                d->position, d->cfg.max_seq);
  if (n_generated) *n_generated = 0;
  if (steps == 0) return 0;
  int rc, zero = 0;
  if ((rc = ensure_pages(d, d->position + steps))) return rc;
  if ((rc = cthip_h2d(d->hist_n, &zero, sizeof(int)))) return rc;
  const int ctrl[2] = {eos, 0};
  if ((rc = cthip_h2d(d->ctrl, ctrl, sizeof(ctrl)))) return rc;
  hipStream_t st = state().stream;
  d->ctrl_host[1] = 0;
  bool copy_pending = false;
  int i = 0;
  auto ended = [&]() {
    // Looks at the last copy of the flag that has ARRIVED; never waits.  A step that runs after the sequence
    // has ended changes nothing, so launching a batch too many costs time only.
    if (eos < 0) return false;
    if (copy_pending && hipEventQuery(d->ctrl_ev) == hipSuccess) copy_pending = false;
    if (!copy_pending) {
      if (d->ctrl_host[1]) return true;
      if (hipMemcpyAsync(d->ctrl_host, d->ctrl, 2 * sizeof(int), hipMemcpyDeviceToHost, st) == hipSuccess &&
          hipEventRecord(d->ctrl_ev, st) == hipSuccess)
        copy_pending = true;
    }
    return false;
  };
  if (d->use_graph)
    for (; i + kStepsPerGraph <= steps && !ended(); i += kStepsPerGraph)
      CTHIP_CHECK(hipGraphLaunch(d->g_multi[d->long_from > 0 && d->position + i >= d->long_from ? 1 : 0], st));
  for (; i < steps && !ended(); i++)
    if ((rc = run_step(d, true, d->position + i))) return rc;
  int n = 0;
  if ((rc = cthip_d2h(&n, d->hist_n, sizeof(int)))) return rc;  // synchronises
  if ((rc = flow_check(d))) return rc;
  if (n < 0 || n > steps) return fail(CTHIP_E_STATE, "cthip_decoder_generate: the device reports %d tokens for %d steps", n, steps);
  if (n && (rc = cthip_d2h(tokens_out, d->history, sizeof(int64_t) * (size_t)n))) return rc;
  d->position += n;
  if (n_generated) *n_generated = n;
  return 0;
}

int cthip_decoder_generate(void *dec, int steps, int64_t *tokens_out) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && steps >= 0 && (steps == 0 || tokens_out != nullptr));
  return generate_impl((Decoder *)dec, steps, -1, tokens_out, nullptr);
}

int cthip_decoder_generate_until(void *dec, int max_steps, int64_t eos_token, int64_t *tokens_out, int *n_generated) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && max_steps >= 0 && (max_steps == 0 || tokens_out != nullptr) && n_generated != nullptr);
  Decoder *d = (Decoder *)dec;
  if (eos_token < 0 || eos_token >= d->cfg.vocab)
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_generate_until: token %lld is not in the vocabulary of %d", (long long)eos_token, d->cfg.vocab);
  return generate_impl(d, max_steps, (int)eos_token, tokens_out, n_generated);
}

int cthip_decoder_position(const void *dec) { return dec ? ((const Decoder *)dec)->position : -1; }

int cthip_decoder_layer_launches(void *dec) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr);
  Decoder *d = (Decoder *)dec;
  int rc = finalize(d);
  if (rc) return -1;
  if (d->flow) return 1;  // all layers are ONE launch
  if (d->fused || d->fused_gqa) return 3;  // (GPT-2 shapes: also over a cache of Q8_0 rows)
  return 5;  // (Q8_0 and paged caches too: rotation, quantisation / copy and append of the new row happen inside the attention launch)
}

int64_t cthip_decoder_step_bytes(const void *dec, int t) {
  const Decoder *d = (const Decoder *)dec;
  if (!d || !d->finalized) return -1;
  const cthip_decoder_config &c = d->cfg;
  const int64_t KD = kv_dim(c);
  int64_t emb = 4LL * c.dim * (c.arch == CTHIP_ARCH_GPT2 ? 2 : 1);
  // per element of a cache row: 4 bytes, or 1 + 2 / 32 as Q8_0
  int64_t kv_read = d->kvq ? 2LL * c.n_layers * t * (KD + KD / 32 * 2) : 2LL * c.n_layers * t * KD * 4;
  int64_t kv_write = d->kvq ? 2LL * c.n_layers * (KD + KD / 32 * 2) : 2LL * c.n_layers * KD * 4;
  return d->weight_bytes + d->vector_bytes + emb + kv_read + kv_write;
}

int cthip_decoder_peek(void *dec, const char *what, void **ptr, int64_t *n_floats) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(dec != nullptr && what != nullptr && ptr != nullptr);
  Decoder *d = (Decoder *)dec;
  int rc = finalize(d);
  if (rc) return rc;
  const cthip_decoder_config &c = d->cfg;
  int64_t n = 0;
  void *p = nullptr;
  int l = -1;
  if (!strcmp(what, "logits")) {
    p = d->logits;
    n = c.vocab;
  } else if (!strcmp(what, "x")) {
    p = d->x;
    n = c.dim;
  } else if (!strcmp(what, "flow_trace") && d->flow && d->flow_args.trace) {
    // int64 clock stamps [workgroups][n_layers][4]; n counts their bytes in units of four
    p = d->flow_args.trace;
    n = (int64_t)dec_flow_grid(c.dim, c.n_heads, c.ffn) * c.n_layers * 4 * 2;
  } else if ((sscanf(what, "k_cache.%d", &l) == 1 || sscanf(what, "v_cache.%d", &l) == 1) && l >= 0 && l < c.n_layers) {
    const bool key = what[0] == 'k';
    n = (int64_t)c.max_seq * kv_dim(c);
    if (d->kvp) {
      // pages: what the caller gets is the rows as one dense array (zeros where no page has been opened), in a buffer
      // that the next peek overwrites
      if (!d->peek_f32 && (rc = dev_alloc(d, (void **)&d->peek_f32, sizeof(float) * (size_t)n))) return rc;
      const Layer &L = d->layers[l];
      if ((rc = launch_kvp_gather(d->peek_f32, key ? L.k_pages : L.v_pages, c.max_seq, kv_dim(c)))) return rc;
      p = d->peek_f32;
    } else if (d->kvq) {
      // Q8_0 rows: what the caller gets is their fp32 value, in a buffer that the next peek overwrites
      if (!d->peek_f32 && (rc = dev_alloc(d, (void **)&d->peek_f32, sizeof(float) * (size_t)n))) return rc;
      const Layer &L = d->layers[l];
      if ((rc = launch_kvq_dequant(d->peek_f32, key ? L.kq : L.vq, key ? L.kdq : L.vdq, c.max_seq, kv_dim(c)))) return rc;
      p = d->peek_f32;
    } else {
      p = key ? d->layers[l].k_cache : d->layers[l].v_cache;
    }
  } else if ((sscanf(what, "k_cache_q8.%d", &l) == 1 || sscanf(what, "v_cache_q8.%d", &l) == 1) && d->kvq && l >= 0 && l < c.n_layers) {
    // the quant plane itself, int8[max_seq][KD]; n counts its bytes in units of four
    p = what[0] == 'k' ? d->layers[l].kq : d->layers[l].vq;
    n = (int64_t)c.max_seq * kv_dim(c) / 4;
  } else if ((sscanf(what, "k_cache_d.%d", &l) == 1 || sscanf(what, "v_cache_d.%d", &l) == 1) && d->kvq && l >= 0 && l < c.n_layers) {
    // the scale plane, fp16[max_seq][KD / 32]; n counts its bytes in units of four
    p = what[0] == 'k' ? d->layers[l].kdq : d->layers[l].vdq;
    n = (int64_t)c.max_seq * (kv_dim(c) / 32) / 2;
  } else {
    return fail(CTHIP_E_BAD_ARG, "cthip_decoder_peek: unknown buffer '%s'", what);
  }
  *ptr = p;
  if (n_floats) *n_floats = n;
  return 0;
}

}  // extern "C"
