// tl_stack.hip — the layer-list engine: a decoder described layer by layer (tl_stack_config) instead of by the fixed Llama
// block of tl_model.hip. It owns the bf16 weights, the per-layer FP32 caches and recurrent states and the chunk workspaces,
// and runs T tokens through all layers: T = 1 is the decode step (GEMVs, position and token id read from the device, so the
// step can be captured into a hipGraph by tl_model.hip like the Llama step), T > 1 a chunk of a prompt (MFMA GEMMs).
//
// Blocks  TL_BLOCK_POST_NORM  x += norm1(mixer(x)); x += norm2(ff(x))   -- the sublayers read x itself, RMS norm on their OUTPUT
//         TL_BLOCK_PARALLEL   h = norm1(x); x += mixer(h) + ff(h)       -- one Dynamic Tanh norm, both sublayers read its output;
//                             the norm of the NEXT block rides in the launch that finishes x (it is elementwise)
// Mixers  TL_MIXER_SWA    q | k (| v) = W h in one product; either the whole-projection q/k RMS norm with optional value mixing
//                         (tl_norm.hip), or rotary positions + per-head unit norm, values optionally the keys as projected
//                         (tl_rope.hip); k, v -> cache; windowed attention with softmax or sigmoid weights, optionally with
//                         the first keys kept visible (tl_swa.hip); W_o
//         TL_MIXER_DELTA  q | k | v | beta | a1 | g1 = W h in one product, a2 and g2 behind a1 and g1; convolution, unit norms
//                         and decay (delta_pre), the recurrence over a per-head state (delta_scan), gated head norm; W_o
// Feed-forward  TL_MLP_MOE  router (two kinds, tl_moe.hip) -> top experts (gated units) + optional shared expert, optionally
//                           gated per token;  TL_MLP_DENSE  one gated unit (it runs where a shared expert would)
// A layer may use an earlier layer's tensors (weights_of) with a cache or state of its own.
// The residual stream, norms, router, attention scores, caches and states are FP32; matrix operands of a prompt chunk are bf16
// (terms = 1) or the FP32-grade three-term split (terms = 3), see tl_dense.hip; the decode step's GEMVs are FP32 throughout.
//
// Cache and state: one allocation. Attention layers: K [max_positions][kv_heads * dim] and V [max_positions][kv_heads * vdim],
// flat by absolute position; a window only bounds what attention reads. Delta layers: S [heads][vdim][dim] and the
// convolution's last taps - 1 inputs. tl_stack_reset gives everything back (one sequence at a time): zeros are the state of
// an empty sequence.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <set>
#include <string>
#include <vector>

#include "tl_stack.h"

namespace {

struct Layer {
  tl_layer_spec sp;
  int wsrc = 0;                        // layer whose tensors this one uses (itself unless weights_of)
  int qd = 0, kd = 0, vd = 0, od = 0;  // q / k / v projection sizes, mixer output size (heads * vdim)
  int pd = 0;                          // rows of the first product (q | k | v, plus beta | a1 | g1 for the delta rule)
  int vmix_mode = 0;                   // 0 none, 1 first mixing layer, 2 mixes with the first
  bool rotary_path = false;            // tl_rope.hip prepares q / k (otherwise tl_norm.hip's qkv_post)
  uint16_t *wqkv = nullptr, *wo = nullptr;
  float *q_norm = nullptr, *k_norm = nullptr, *lambda = nullptr, *norm1 = nullptr, *norm2 = nullptr;
  float *norm1_b = nullptr, *norm1_alpha = nullptr;  // Dynamic Tanh
  float* pb = nullptr;                               // sigmoid bias per head
  double* freq = nullptr;                            // rotary frequencies
  float mscale = 1.0f;
  uint16_t *wa2 = nullptr, *wg2 = nullptr, *conv = nullptr;  // delta rule
  float *a_log = nullptr, *dt_bias = nullptr, *onorm = nullptr;
  uint16_t *router = nullptr, *gu = nullptr, *down = nullptr, *sgu = nullptr, *sdown = nullptr, *sg = nullptr;
  float* router_b = nullptr;
  float *kc = nullptr, *vc = nullptr;        // attention: caches
  float *state = nullptr, *hist = nullptr;   // delta rule: S and the convolution's history
  std::set<std::string> expect, optional;    // tensor names (without the "l<i>." prefix) still missing / accepted and ignored
};

}  // namespace

struct TlStack {
  tl_stack_config cfg;
  std::vector<Layer> layers;
  uint16_t *embed = nullptr, *head = nullptr;
  float *embed_norm = nullptr, *final_norm = nullptr, *final_b = nullptr, *final_alpha = nullptr;
  int got_globals = 0, need_globals = 0;
  std::vector<void*> allocs;
  bool finalized = false;
  int terms = 1;
  // tokens of a prompt that go through the layers together. Measured at width 4096 with 16 experts (top 4): 105.9 k tokens/s
  // at 512, 140.4 k at 1024, 171.6 k at 2048 -- the experts' grouped GEMMs see 4 x the tokens per expert, the dense ones
  // enough tiles for the 128 x 128 shape.
  int chunk = 2048;
  bool gemv_decode = true;
  bool fuse_router = true;  // TL_STACK_FUSE_ROUTER=0: the router as a launch of its own (A/B, tests)
  // One token through a parallel block: mixer and feed-forward read the same h and meet only in the residual sum, so the
  // feed-forward's launches go to a second stream (forked and joined by events; under capture they become a parallel branch
  // of the graph) and the step's critical path per layer is the longer of the two chains, not their sum. TL_STACK_FORK=0: one stream.
  bool fork = true;
  hipStream_t side = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  // workspaces for one chunk
  float *x = nullptr, *qkv = nullptr, *att = nullptr, *proj = nullptr, *v_first = nullptr, *xn = nullptr;
  float* h = nullptr;       // norm-first blocks: the normalised input both sublayers read
  float *dq = nullptr, *da = nullptr, *dg = nullptr, *dbeta = nullptr, *ddecay = nullptr;  // delta rule
  float *act_buf = nullptr, *eout = nullptr, *sact = nullptr, *sout = nullptr, *sgate = nullptr;
  float* wts = nullptr;
  float* swa_ws = nullptr;  // partial results of split attention launches (few tokens, long windows)
  unsigned* swa_cnt = nullptr;  // their arrival counters (zero between launches)
  int *ids = nullptr, *off = nullptr, *slot_of = nullptr;
  int max_qkv = 0, max_od = 0, max_vd = 0, max_top = 0, max_experts = 0, max_gu = 0, max_sff = 0;
  int max_dc = 0, max_da = 0, max_heads = 0;
  tl_stack_layer_hook hook = nullptr;
  void* hook_ctx = nullptr;
  size_t cache_bytes = 0;
  void* cache_base = nullptr;
};

namespace {

template <class T>
int dev_alloc(TlStack* st, T** p, size_t n) {
  void* q = nullptr;
  TL_HIP(hipMalloc(&q, sizeof(T) * (n ? n : 1)));
  st->allocs.push_back(q);
  *p = static_cast<T*>(q);
  return 0;
}

int upload_as_f32(float* dst, int type, const void* host, size_t n, hipStream_t s) {
  std::vector<float> wide(n);
  if (type == TL_BF16) {
    const uint16_t* b = static_cast<const uint16_t*>(host);
    for (size_t i = 0; i < n; ++i) {
      const uint32_t bits = (uint32_t)b[i] << 16;
      memcpy(&wide[i], &bits, 4);
    }
  } else {
    memcpy(wide.data(), host, n * 4);
  }
  TL_HIP(hipMemcpyAsync(dst, wide.data(), n * 4, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

// rows of `cols` bf16 values to every second row of dst (gate rows to the even, up rows to the odd rows of a gate|up matrix)
int upload_bf16_alternate(uint16_t* dst, const void* host, size_t rows, size_t cols, hipStream_t s) {
  TL_HIP(hipMemcpy2DAsync(dst, 2 * cols * 2, host, cols * 2, cols * 2, rows, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

int upload_bf16(uint16_t* dst, const void* host, size_t n, hipStream_t s) {
  TL_HIP(hipMemcpyAsync(dst, host, n * 2, hipMemcpyHostToDevice, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

bool shape_is(const long long* shape, int ndim, long long a, long long b = -1) {
  if (b < 0) {
    long long n = 1;
    for (int i = 0; i < ndim; ++i) n *= shape[i];
    return n == a && ndim <= 1;
  }
  return ndim == 2 && shape[0] == a && shape[1] == b;
}

}  // namespace

int tl_stack_create(const tl_stack_config* cfg, TlStack** out) {
  TL_REQUIRE(cfg && out && cfg->layers, "tl_stack_create: null argument");
  TL_REQUIRE(cfg->width > 0 && cfg->vocab > 0 && cfg->n_layers > 0 && cfg->max_positions > 0,
             "tl_stack_create: non-positive size in the configuration");
  TL_REQUIRE(cfg->norm == TL_NORM_RMS_ONE_PLUS || cfg->norm == TL_NORM_DYT, "tl_stack_create: norm kind %d", cfg->norm);
  TlStack* st = new TlStack();
  st->cfg = *cfg;
  st->layers.resize(cfg->n_layers);
  const size_t W = cfg->width;
  int first_mix = -1;
  int rc = 0;
  auto fail = [&](int code) {
    tl_stack_free(st);
    return code;
  };
#define CREATE_REQUIRE(cond, ...) \
  do {                            \
    if (!(cond)) {                \
      tl_set_error(__VA_ARGS__);  \
      return fail(2);             \
    }                             \
  } while (0)
  for (int i = 0; i < cfg->n_layers && rc == 0; ++i) {
    Layer& L = st->layers[i];
    L.sp = cfg->layers[i];
    const tl_layer_spec& sp = L.sp;
    const bool dyt = cfg->norm == TL_NORM_DYT;
    CREATE_REQUIRE(sp.mixer == TL_MIXER_SWA || sp.mixer == TL_MIXER_DELTA,
                   "tl_stack_create: layer %d has mixer kind %d; this engine has windowed attention (%d) and the gated delta rule (%d)",
                   i, sp.mixer, TL_MIXER_SWA, TL_MIXER_DELTA);
    CREATE_REQUIRE(sp.heads > 0 && sp.kv_heads > 0 && sp.heads % sp.kv_heads == 0 && sp.dim > 0 && sp.vdim > 0,
                   "tl_stack_create: layer %d: %d heads / %d key-value heads / sizes %d, %d", i, sp.heads, sp.kv_heads, sp.dim, sp.vdim);
    CREATE_REQUIRE((sp.block == TL_BLOCK_POST_NORM && !dyt) || (sp.block == TL_BLOCK_PARALLEL && dyt),
                   "tl_stack_create: layer %d: block kind %d with norm kind %d (post-norm blocks take the RMS norm, parallel "
                   "blocks the Dynamic Tanh norm)", i, sp.block, cfg->norm);
    CREATE_REQUIRE(sp.mlp == TL_MLP_NONE || sp.mlp == TL_MLP_MOE || sp.mlp == TL_MLP_DENSE,
                   "tl_stack_create: layer %d has feed-forward kind %d", i, sp.mlp);
    CREATE_REQUIRE(sp.mlp != TL_MLP_DENSE || sp.block == TL_BLOCK_PARALLEL, "tl_stack_create: layer %d: a dense feed-forward "
                   "runs in parallel blocks only", i);
    L.wsrc = i;
    if (sp.weights_of > 0) {
      CREATE_REQUIRE(sp.weights_of - 1 < i, "tl_stack_create: layer %d takes its tensors from layer %d, which is not an earlier "
                     "layer", i, sp.weights_of - 1);
      L.wsrc = st->layers[sp.weights_of - 1].wsrc;  // (a layer that itself borrows hands on the owner)
      tl_layer_spec a = sp, b = st->layers[L.wsrc].sp;
      a.weights_of = b.weights_of = 0;
      CREATE_REQUIRE(memcmp(&a, &b, sizeof(a)) == 0, "tl_stack_create: layer %d differs from layer %d whose tensors it uses", i, L.wsrc);
    }
    const bool own = L.wsrc == i;
    // ---- mixer ----
    if (sp.mixer == TL_MIXER_SWA) {
      CREATE_REQUIRE(!sp.values_are_keys || sp.vdim == sp.dim, "tl_stack_create: layer %d: values that are keys need vdim == dim", i);
      CREATE_REQUIRE(sp.rot_dims >= 0 && sp.rot_dims <= sp.dim && (sp.rot_dims & 1) == 0 && (sp.rot_dims == 0 || sp.rot_base > 0.0f),
                     "tl_stack_create: layer %d: %d rotating dimensions of %d, base %g", i, sp.rot_dims, sp.dim, sp.rot_base);
      CREATE_REQUIRE(sp.keep_first >= 0, "tl_stack_create: layer %d: %d kept first keys", i, sp.keep_first);
      L.rotary_path = sp.rot_dims > 0 || sp.qk_norm == TL_QK_NORM_HEAD_UNIT || sp.values_are_keys;
      CREATE_REQUIRE(!L.rotary_path || (sp.qk_norm != TL_QK_NORM_WHOLE && !sp.v_mix), "tl_stack_create: layer %d: rotation / "
                     "per-head norm / values-are-keys do not combine with the whole-projection norm or value mixing", i);
      CREATE_REQUIRE(sp.qk_norm >= TL_QK_NORM_NONE && sp.qk_norm <= TL_QK_NORM_HEAD_UNIT, "tl_stack_create: layer %d: q/k norm %d", i, sp.qk_norm);
      L.qd = sp.heads * sp.dim;
      L.kd = sp.kv_heads * sp.dim;
      L.vd = sp.kv_heads * sp.vdim;
      L.od = sp.heads * sp.vdim;
      L.pd = L.qd + L.kd + (sp.values_are_keys ? 0 : L.vd);
      if (sp.v_mix) {
        if (first_mix < 0) {
          first_mix = i;
          L.vmix_mode = 1;
        } else {
          L.vmix_mode = 2;
          CREATE_REQUIRE(st->layers[first_mix].vd == L.vd, "tl_stack_create: layer %d mixes %d values with the %d of layer %d", i,
                         L.vd, st->layers[first_mix].vd, first_mix);
        }
      }
      st->cache_bytes += sizeof(float) * (size_t)cfg->max_positions * (L.kd + L.vd);
      if (own) {
        L.expect.insert({"mix.q", "mix.k", "mix.o"});
        if (!sp.values_are_keys) L.expect.insert("mix.v");
        if (sp.qk_norm == TL_QK_NORM_WHOLE) L.expect.insert({"mix.q.norm", "mix.k.norm"});
        else L.optional.insert({"mix.q.norm", "mix.k.norm"});
        if (L.vmix_mode == 2) L.expect.insert("mix.vmix");
        else L.optional.insert("mix.vmix");
        if (sp.attn_weight == TL_ATTN_SIGMOID) L.expect.insert("mix.pb");
        if ((rc = dev_alloc(st, &L.q_norm, L.qd))) break;
        if ((rc = dev_alloc(st, &L.k_norm, L.kd))) break;
        if ((rc = dev_alloc(st, &L.lambda, 1))) break;
        if ((rc = dev_alloc(st, &L.pb, sp.heads))) break;
        if (sp.rot_dims > 0) {
          std::vector<double> f(sp.rot_dims / 2);
          tl_rotary_frequencies(sp.rot_dims, sp.rot_base, sp.rot_factor, sp.rot_original, sp.rot_fast, sp.rot_slow, f.data(), &L.mscale);
          if ((rc = dev_alloc(st, &L.freq, f.size()))) break;
          if (hipMemcpy(L.freq, f.data(), sizeof(double) * f.size(), hipMemcpyHostToDevice) != hipSuccess) {
            tl_set_error("tl_stack_create: upload of the rotary frequencies failed");
            return fail(1);
          }
        }
      }
    } else {
      CREATE_REQUIRE(sp.block == TL_BLOCK_PARALLEL, "tl_stack_create: layer %d: the delta rule runs in parallel blocks only", i);
      CREATE_REQUIRE(sp.conv_taps >= 1 && sp.conv_taps <= 64 && sp.decay_rank > 0 && sp.gate_rank > 0,
                     "tl_stack_create: layer %d: %d taps, inner sizes %d / %d", i, sp.conv_taps, sp.decay_rank, sp.gate_rank);
      CREATE_REQUIRE(sp.dim <= 256 && sp.vdim <= 512, "tl_stack_create: layer %d: key size %d above 256 or value size %d above 512", i,
                     sp.dim, sp.vdim);
      L.qd = sp.kv_heads * sp.dim;  // queries share the keys' heads
      L.kd = sp.kv_heads * sp.dim;
      L.vd = sp.heads * sp.vdim;
      L.od = sp.heads * sp.vdim;
      L.pd = L.qd + L.kd + L.vd + sp.heads + sp.decay_rank + sp.gate_rank;
      const int dc = L.qd + L.kd + L.vd, da = sp.heads * sp.dim;
      st->max_dc = dc > st->max_dc ? dc : st->max_dc;
      st->max_da = da > st->max_da ? da : st->max_da;
      st->cache_bytes += sizeof(float) * ((size_t)sp.heads * sp.vdim * sp.dim + (size_t)(sp.conv_taps - 1) * dc);
      if (own) {
        L.expect.insert({"mix.q", "mix.k", "mix.v", "mix.b", "mix.a1", "mix.g1", "mix.a2", "mix.g2", "mix.o", "mix.q.conv",
                         "mix.k.conv", "mix.v.conv", "mix.A_log", "mix.dt_bias", "mix.norm"});
        if ((rc = dev_alloc(st, &L.wa2, (size_t)da * sp.decay_rank))) break;
        if ((rc = dev_alloc(st, &L.wg2, (size_t)L.vd * sp.gate_rank))) break;
        if ((rc = dev_alloc(st, &L.conv, (size_t)dc * sp.conv_taps))) break;
        if ((rc = dev_alloc(st, &L.a_log, sp.heads))) break;
        if ((rc = dev_alloc(st, &L.dt_bias, da))) break;
        if ((rc = dev_alloc(st, &L.onorm, sp.vdim))) break;
      }
    }
    if (own) {
      if ((rc = dev_alloc(st, &L.wqkv, (size_t)L.pd * W))) break;
      if ((rc = dev_alloc(st, &L.wo, W * L.od))) break;
      if ((rc = dev_alloc(st, &L.norm1, W))) break;
      if ((rc = dev_alloc(st, &L.norm2, W))) break;
      L.expect.insert("norm1");
      if (dyt) {
        if ((rc = dev_alloc(st, &L.norm1_b, W))) break;
        if ((rc = dev_alloc(st, &L.norm1_alpha, 1))) break;
        L.expect.insert({"norm1.b", "norm1.alpha"});
      }
    }
    // ---- feed-forward ----
    if (sp.mlp == TL_MLP_MOE) {
      CREATE_REQUIRE(sp.experts > 0 && sp.top > 0 && sp.top <= sp.experts && sp.expert_ff > 0 && sp.shared_ff >= 0,
                     "tl_stack_create: layer %d: %d experts, top %d, sizes %d / %d", i, sp.experts, sp.top, sp.expert_ff, sp.shared_ff);
      CREATE_REQUIRE(sp.route == TL_ROUTE_TOP_LOGITS ||
                         (sp.route == TL_ROUTE_SOFTMAX_GROUPS && sp.route_groups > 0 && sp.experts % sp.route_groups == 0 &&
                          sp.route_keep > 0 && sp.route_keep <= sp.route_groups &&
                          (long long)sp.route_keep * (sp.experts / sp.route_groups) >= sp.top),
                     "tl_stack_create: layer %d: router kind %d, %d experts in %d groups, %d kept, top %d", i, sp.route, sp.experts,
                     sp.route_groups, sp.route_keep, sp.top);
      CREATE_REQUIRE(!sp.shared_gate || sp.shared_ff > 0, "tl_stack_create: layer %d: a gate without a shared expert", i);
      if (own) {
        if (sp.block == TL_BLOCK_POST_NORM) L.expect.insert("norm2");
        L.expect.insert("mlp.router");
        if (sp.route == TL_ROUTE_TOP_LOGITS) L.expect.insert("mlp.router.b");
        for (int e = 0; e < sp.experts; ++e)
          for (const char* k : {"gate", "up", "down"}) L.expect.insert("mlp.e" + std::to_string(e) + "." + k);
        if ((rc = dev_alloc(st, &L.router, (size_t)sp.experts * W))) break;
        if ((rc = dev_alloc(st, &L.router_b, sp.experts))) break;
        if ((rc = dev_alloc(st, &L.gu, (size_t)sp.experts * 2 * sp.expert_ff * W))) break;
        if ((rc = dev_alloc(st, &L.down, (size_t)sp.experts * W * sp.expert_ff))) break;
        if (sp.shared_ff) {
          L.expect.insert({"mlp.shared.gate", "mlp.shared.up", "mlp.shared.down"});
          if ((rc = dev_alloc(st, &L.sgu, (size_t)2 * sp.shared_ff * W))) break;
          if ((rc = dev_alloc(st, &L.sdown, W * sp.shared_ff))) break;
          if (sp.shared_gate) {
            L.expect.insert("mlp.shared.sg");
            if ((rc = dev_alloc(st, &L.sg, W))) break;
          }
        }
      }
      st->max_top = sp.top > st->max_top ? sp.top : st->max_top;
      st->max_experts = sp.experts > st->max_experts ? sp.experts : st->max_experts;
      st->max_gu = 2 * sp.expert_ff * sp.top > st->max_gu ? 2 * sp.expert_ff * sp.top : st->max_gu;
      st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
    } else if (sp.mlp == TL_MLP_DENSE) {
      CREATE_REQUIRE(sp.shared_ff > 0, "tl_stack_create: layer %d: a dense feed-forward of size %d", i, sp.shared_ff);
      if (own) {
        L.expect.insert({"mlp.gate", "mlp.up", "mlp.down"});
        if ((rc = dev_alloc(st, &L.sgu, (size_t)2 * sp.shared_ff * W))) break;
        if ((rc = dev_alloc(st, &L.sdown, W * sp.shared_ff))) break;
      }
      st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
    } else if (own) {
      L.optional.insert("norm2");
    }
    st->max_qkv = L.pd > st->max_qkv ? L.pd : st->max_qkv;
    st->max_od = L.od > st->max_od ? L.od : st->max_od;
    st->max_vd = L.vd > st->max_vd ? L.vd : st->max_vd;
    st->max_heads = sp.heads > st->max_heads ? sp.heads : st->max_heads;
  }
#undef CREATE_REQUIRE
  if (rc) return fail(rc);
  if ((rc = dev_alloc(st, &st->embed, (size_t)cfg->vocab * W)) || (rc = dev_alloc(st, &st->head, (size_t)cfg->vocab * W)) ||
      (rc = dev_alloc(st, &st->embed_norm, W)) || (rc = dev_alloc(st, &st->final_norm, W)) ||
      (rc = dev_alloc(st, &st->final_b, W)) || (rc = dev_alloc(st, &st->final_alpha, 1)))
    return fail(rc);
  st->need_globals = 1 | 2 | 8 | (cfg->embed_norm ? 4 : 0) | (cfg->norm == TL_NORM_DYT ? 16 | 32 : 0);
  if (const char* e = getenv("TL_STACK_CHUNK")) st->chunk = atoi(e) > 0 ? atoi(e) : st->chunk;
  if (const char* e = getenv("TL_STACK_GEMV")) st->gemv_decode = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FUSE_ROUTER")) st->fuse_router = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FORK")) st->fork = atoi(e) != 0;
  *out = st;
  return 0;
}

void tl_stack_free(TlStack* st) {
  if (!st) return;
  for (void* p : st->allocs) hipFree(p);
  hipFree(st->cache_base);
  if (st->ev_fork) hipEventDestroy(st->ev_fork);
  if (st->ev_join) hipEventDestroy(st->ev_join);
  if (st->side) hipStreamDestroy(st->side);
  delete st;
}

int tl_stack_set_tensor(TlStack* st, const char* name, int type, const long long* shape, int ndim, const void* host,
                        hipStream_t s) {
  TL_REQUIRE(st && name && host && (shape || ndim == 0), "tl_stack_set_tensor: null argument");
  TL_REQUIRE(!st->finalized, "tl_stack_set_tensor: model already finalized");
  TL_REQUIRE(type == TL_BF16 || type == TL_F32, "tl_stack_set_tensor: %s has type %d; bf16 (matrices, vectors) or f32 (vectors)",
             name, type);
  const long long W = st->cfg.width, V = st->cfg.vocab;
  const std::string n(name);
#define MATRIX(dst, r, c)                                                                                                   \
  do {                                                                                                                      \
    TL_REQUIRE(type == TL_BF16, "tl_stack_set_tensor: matrix %s must be bf16", name);                                       \
    TL_REQUIRE(shape_is(shape, ndim, (r), (c)), "tl_stack_set_tensor: %s is not %lld x %lld", name, (long long)(r),         \
               (long long)(c));                                                                                             \
    return upload_bf16((dst), host, (size_t)(r) * (size_t)(c), s);                                                          \
  } while (0)
#define PAIRED(dst, r, c)                                                                                                   \
  do {                                                                                                                      \
    TL_REQUIRE(type == TL_BF16, "tl_stack_set_tensor: matrix %s must be bf16", name);                                       \
    TL_REQUIRE(shape_is(shape, ndim, (r), (c)), "tl_stack_set_tensor: %s is not %lld x %lld", name, (long long)(r),         \
               (long long)(c));                                                                                             \
    return upload_bf16_alternate((dst), host, (size_t)(r), (size_t)(c), s);                                                 \
  } while (0)
#define VECTOR(dst, len)                                                                                                    \
  do {                                                                                                                      \
    TL_REQUIRE(shape_is(shape, ndim, (len)), "tl_stack_set_tensor: %s does not have %lld elements", name, (long long)(len)); \
    return upload_as_f32((dst), type, host, (size_t)(len), s);                                                              \
  } while (0)
  if (n == "embed") { st->got_globals |= 1; MATRIX(st->embed, V, W); }
  if (n == "head") { st->got_globals |= 2; MATRIX(st->head, V, W); }
  if (n == "embed.norm") { st->got_globals |= 4; VECTOR(st->embed_norm, W); }
  if (n == "final.norm") { st->got_globals |= 8; VECTOR(st->final_norm, W); }
  if (n == "final.norm.b") { st->got_globals |= 16; VECTOR(st->final_b, W); }
  if (n == "final.norm.alpha") { st->got_globals |= 32; VECTOR(st->final_alpha, 1); }
  int li = -1, used = 0;
  TL_REQUIRE(sscanf(name, "l%d.%n", &li, &used) == 1 && used > 0 && li >= 0 && li < st->cfg.n_layers,
             "tl_stack_set_tensor: no place for a tensor named %s", name);
  Layer& L = st->layers[li];
  const tl_layer_spec& sp = L.sp;
  const std::string r = n.substr(used);
  if (L.optional.count(r) && !L.expect.count(r)) {  // present in the checkpoint, not used by this configuration: checked, dropped
    return 0;
  }
  TL_REQUIRE(L.expect.erase(r) == 1, "tl_stack_set_tensor: no place for a tensor named %s in layer %d (unknown, given twice, or "
             "the layer uses another layer's tensors)", name, li);
  if (r == "norm1") VECTOR(L.norm1, W);
  if (r == "norm1.b") VECTOR(L.norm1_b, W);
  if (r == "norm1.alpha") VECTOR(L.norm1_alpha, 1);
  if (r == "norm2") VECTOR(L.norm2, W);
  if (r == "mix.q") MATRIX(L.wqkv, L.qd, W);
  if (r == "mix.k") MATRIX(L.wqkv + (size_t)L.qd * W, L.kd, W);
  if (r == "mix.v") MATRIX(L.wqkv + (size_t)(L.qd + L.kd) * W, L.vd, W);
  if (r == "mix.o") MATRIX(L.wo, W, L.od);
  if (r == "mix.q.norm") VECTOR(L.q_norm, L.qd);
  if (r == "mix.k.norm") VECTOR(L.k_norm, L.kd);
  if (r == "mix.vmix") VECTOR(L.lambda, 1);
  if (r == "mix.pb") VECTOR(L.pb, sp.heads);
  if (sp.mixer == TL_MIXER_DELTA) {
    const long long c0 = L.qd + L.kd + L.vd, da = (long long)sp.heads * sp.dim, taps = sp.conv_taps;
    if (r == "mix.b") MATRIX(L.wqkv + (size_t)c0 * W, sp.heads, W);
    if (r == "mix.a1") MATRIX(L.wqkv + (size_t)(c0 + sp.heads) * W, sp.decay_rank, W);
    if (r == "mix.g1") MATRIX(L.wqkv + (size_t)(c0 + sp.heads + sp.decay_rank) * W, sp.gate_rank, W);
    if (r == "mix.a2") MATRIX(L.wa2, da, sp.decay_rank);
    if (r == "mix.g2") MATRIX(L.wg2, L.vd, sp.gate_rank);
    if (r == "mix.q.conv") MATRIX(L.conv, L.qd, taps);
    if (r == "mix.k.conv") MATRIX(L.conv + (size_t)L.qd * taps, L.kd, taps);
    if (r == "mix.v.conv") MATRIX(L.conv + (size_t)(L.qd + L.kd) * taps, L.vd, taps);
    if (r == "mix.A_log") VECTOR(L.a_log, sp.heads);
    if (r == "mix.dt_bias") VECTOR(L.dt_bias, da);
    if (r == "mix.norm") VECTOR(L.onorm, sp.vdim);
  }
  if (sp.mlp == TL_MLP_DENSE) {
    const long long ff = sp.shared_ff;
    if (r == "mlp.gate") PAIRED(L.sgu, ff, W);  // gate | up interleaved by unit (DenseArgs::glu)
    if (r == "mlp.up") PAIRED(L.sgu + W, ff, W);
    if (r == "mlp.down") MATRIX(L.sdown, W, ff);
  }
  if (sp.mlp == TL_MLP_MOE) {
    const long long ff = sp.expert_ff, sff = sp.shared_ff;
    if (r == "mlp.router") MATRIX(L.router, sp.experts, W);
    if (r == "mlp.router.b") VECTOR(L.router_b, sp.experts);
    if (sff) {
      if (r == "mlp.shared.gate") PAIRED(L.sgu, sff, W);  // gate | up interleaved by unit (DenseArgs::glu)
      if (r == "mlp.shared.up") PAIRED(L.sgu + W, sff, W);
      if (r == "mlp.shared.down") MATRIX(L.sdown, W, sff);
      if (r == "mlp.shared.sg") {
        TL_REQUIRE(type == TL_BF16 && ((ndim == 2 && shape[0] == 1 && shape[1] == W) || (ndim == 1 && shape[0] == W)),
                   "tl_stack_set_tensor: %s is not a bf16 row of %lld", name, W);
        return upload_bf16(L.sg, host, (size_t)W, s);
      }
    }
    int e = -1, u2 = 0;
    if (sscanf(r.c_str(), "mlp.e%d.%n", &e, &u2) == 1 && u2 > 0 && e >= 0 && e < sp.experts) {
      const std::string k = r.substr(u2);
      uint16_t* gu = L.gu + (size_t)e * 2 * ff * W;
      if (k == "gate") PAIRED(gu, ff, W);
      if (k == "up") PAIRED(gu + W, ff, W);
      if (k == "down") MATRIX(L.down + (size_t)e * W * ff, W, ff);
    }
  }
  TL_REQUIRE(false, "tl_stack_set_tensor: no place for a tensor named %s in layer %d", name, li);
#undef MATRIX
#undef PAIRED
#undef VECTOR
}

int tl_stack_finalize(TlStack* st, hipStream_t s) {
  TL_REQUIRE(st, "tl_stack_finalize: null handle");
  if (st->finalized) return 0;
  TL_REQUIRE((st->got_globals & st->need_globals) == st->need_globals,
             "tl_stack_finalize: embed / head / final.norm (and their parts) missing (have mask %d of %d)", st->got_globals,
             st->need_globals);
  for (size_t i = 0; i < st->layers.size(); ++i)
    TL_REQUIRE(st->layers[i].expect.empty(), "tl_stack_finalize: layer %d lacks %zu tensors, the first is %s", (int)i,
               st->layers[i].expect.size(), st->layers[i].expect.begin()->c_str());
  const size_t W = st->cfg.width, C = st->chunk;
  TL_HIP(hipMalloc(&st->cache_base, st->cache_bytes));
  float* p = static_cast<float*>(st->cache_base);
  for (Layer& L : st->layers) {
    if (L.sp.mixer == TL_MIXER_SWA) {
      L.kc = p;
      p += (size_t)st->cfg.max_positions * L.kd;
      L.vc = p;
      p += (size_t)st->cfg.max_positions * L.vd;
    } else {
      L.state = p;
      p += (size_t)L.sp.heads * L.sp.vdim * L.sp.dim;
      L.hist = p;
      p += (size_t)(L.sp.conv_taps - 1) * (L.qd + L.kd + L.vd);
    }
  }
  TL_TRY(dev_alloc(st, &st->x, C * W));
  TL_TRY(dev_alloc(st, &st->h, C * W));
  TL_TRY(dev_alloc(st, &st->qkv, C * st->max_qkv));
  TL_TRY(dev_alloc(st, &st->att, C * st->max_od));
  TL_TRY(dev_alloc(st, &st->proj, C * W));
  TL_TRY(dev_alloc(st, &st->v_first, C * st->max_vd));
  TL_TRY(dev_alloc(st, &st->xn, C * W));
  if (st->max_dc) {
    TL_TRY(dev_alloc(st, &st->dq, C * st->max_dc));
    TL_TRY(dev_alloc(st, &st->da, C * st->max_da));
    TL_TRY(dev_alloc(st, &st->ddecay, C * st->max_da));
    TL_TRY(dev_alloc(st, &st->dg, C * st->max_od));
    TL_TRY(dev_alloc(st, &st->dbeta, C * st->max_heads));
  }
  {
    size_t ws = 1;
    for (const Layer& L : st->layers)
      for (int T = 1; T <= 4; ++T) {
        if (L.sp.mixer != TL_MIXER_SWA) continue;
        const size_t n = tl_swa_ws_floats(T, L.sp.heads, L.sp.vdim,
                                          tl_swa_splits(T, L.sp.window, st->cfg.max_positions, L.sp.keep_first));
        ws = n > ws ? n : ws;
      }
    TL_TRY(dev_alloc(st, &st->swa_ws, ws));
    const size_t heads = st->max_heads > 0 ? st->max_heads : 1;
    TL_TRY(dev_alloc(st, &st->swa_cnt, 4 * heads));
    TL_HIP(hipMemsetAsync(st->swa_cnt, 0, sizeof(unsigned) * 4 * heads, s));
  }
  if (st->max_top) {
    const size_t S = C * st->max_top;
    TL_TRY(dev_alloc(st, &st->ids, S));
    TL_TRY(dev_alloc(st, &st->wts, S));
    TL_TRY(dev_alloc(st, &st->slot_of, S));
    TL_TRY(dev_alloc(st, &st->off, (size_t)st->max_experts + 1));
    TL_TRY(dev_alloc(st, &st->eout, S * W));
  }
  if (st->max_top || st->max_sff) {
    TL_TRY(dev_alloc(st, &st->act_buf, C * st->max_gu / 2 + st->max_sff));
    TL_TRY(dev_alloc(st, &st->sgate, C));
    TL_TRY(dev_alloc(st, &st->sout, C * W));
    if (st->max_sff) TL_TRY(dev_alloc(st, &st->sact, C * st->max_sff));
  }
  bool any_parallel = false;
  for (const Layer& L : st->layers) any_parallel |= L.sp.block == TL_BLOCK_PARALLEL && L.sp.mlp != TL_MLP_NONE;
  if (st->fork && any_parallel) {
    TL_HIP(hipStreamCreateWithFlags(&st->side, hipStreamNonBlocking));
    TL_HIP(hipEventCreateWithFlags(&st->ev_fork, hipEventDisableTiming));
    TL_HIP(hipEventCreateWithFlags(&st->ev_join, hipEventDisableTiming));
  } else {
    st->fork = false;
  }
  st->finalized = true;
  return tl_stack_reset(st, s);
}

int tl_stack_reset(TlStack* st, hipStream_t s) {
  TL_REQUIRE(st && st->finalized, "tl_stack_reset: model not finalized");
  TL_HIP(hipMemsetAsync(st->cache_base, 0, st->cache_bytes, s));
  TL_HIP(hipStreamSynchronize(s));
  return 0;
}

int tl_stack_set_terms(TlStack* st, int terms) {
  TL_REQUIRE(st, "tl_stack_set_terms: null handle");
  TL_REQUIRE(terms == 1 || terms == 3, "tl_stack_set_terms: a layer-list model multiplies with 1 (bf16 activations) or 3 "
             "(FP32-grade) terms, not %d", terms);
  st->terms = terms;
  return 0;
}

int tl_stack_chunk(const TlStack* st) { return st->chunk; }
const float* tl_stack_residual(const TlStack* st) { return st->x; }
void tl_stack_set_layer_hook(TlStack* st, tl_stack_layer_hook hook, void* ctx) {
  st->hook = hook;
  st->hook_ctx = ctx;
}

int tl_stack_cache_ptr(TlStack* st, int which, int layer, void** out) {
  TL_REQUIRE(st && st->finalized && out, "tl_stack_cache_ptr: model not finalized");
  TL_REQUIRE(layer >= 0 && layer < (int)st->layers.size(), "tl_stack_cache_ptr: layer %d out of range", layer);
  const Layer& L = st->layers[layer];
  // attention: 0 keys, 1 values; delta rule: 0 the state S [heads][vdim][dim], 1 the convolution's history
  if (L.sp.mixer == TL_MIXER_SWA) *out = which == 0 ? L.kc : L.vc;
  else *out = which == 0 ? L.state : L.hist;
  return 0;
}

void tl_stack_bytes_per_token(const TlStack* st, int pos, double* weight_bytes, double* kv_bytes) {
  const double W = st->cfg.width;
  double wb = 2.0 * W /*embedding row*/ + 2.0 * W * st->cfg.vocab, kb = 0.0;
  for (const Layer& L : st->layers) {
    const tl_layer_spec& sp = L.sp;
    wb += 2.0 * W * (L.pd + L.od);
    if (sp.mlp == TL_MLP_MOE)
      wb += 2.0 * W * (sp.experts + 3.0 * sp.expert_ff * sp.top + 3.0 * sp.shared_ff + (sp.shared_gate ? 1.0 : 0.0));
    if (sp.mlp == TL_MLP_DENSE) wb += 2.0 * W * 3.0 * sp.shared_ff;
    if (sp.mixer == TL_MIXER_DELTA) {
      wb += 2.0 * ((double)sp.heads * sp.dim * sp.decay_rank + (double)L.vd * sp.gate_rank);
      kb += 2.0 * 4.0 * sp.heads * sp.vdim * sp.dim;  // the state is read and written
    } else {
      double seen = sp.window > 0 && pos + 1 > sp.window ? sp.window : pos + 1;
      if (sp.window > 0 && sp.keep_first > 0 && pos + 1 > sp.window)
        seen += sp.keep_first < pos + 1 - sp.window ? sp.keep_first : pos + 1 - sp.window;
      kb += 4.0 * (seen + 1.0) * (L.kd + L.vd);
    }
  }
  if (weight_bytes) *weight_bytes = wb;
  if (kv_bytes) *kv_bytes = kb;
}

namespace {

// One token is always FP32-grade: the decode step's GEMVs are, and where TL_STACK_GEMV=0 sends it through the chunk GEMMs
// instead (a test configuration) it takes three terms, whatever the chunks use; so the captured step never depends on a
// setting that may change after the capture.
inline int terms_for(const TlStack* st, int T) { return T == 1 ? 3 : st->terms; }

// y[T][rows] = x[T][cols] W^T for a chunk, or the GEMV for the one token of a decode step
int project(TlStack* st, const uint16_t* w, int rows, int cols, const float* x, int ldx, float* y, int ldy, int T,
            hipStream_t s, float softcap = 0.0f) {
  if (T == 1 && st->gemv_decode) return tl_launch_dense_gemv(w, rows, cols, x, y, s, softcap);
  DenseArgs d = {};
  d.w = w;
  d.rows = rows;
  d.cols = cols;
  d.x = x;
  d.ldx = ldx;
  d.y = y;
  d.ldy = ldy;
  d.T = T;
  d.terms = terms_for(st, T);
  d.softcap = softcap;
  return tl_launch_dense_gemm(d, s);
}

// The routed experts (and the shared expert) of layer L on the rows of `in` (x itself for a post-norm block, the normalised
// h for a parallel one). Leaves: one token -> everything summed (router weights, the shared expert and its gate) in
// one_token_out [W]; a chunk -> st->eout [T * top][W] to be weighted by st->wts, and the shared expert's output in st->sout
// (its per-token gate, if any, in st->sgate).
int moe_experts(TlStack* st, const Layer& L, const Layer& Wt, const float* in, int T, float* one_token_out, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ff = sp.expert_ff, sff = sp.shared_ff, S = T * sp.top;
  if (T == 1 && st->gemv_decode) {
    MoeDecodeArgs d = {};
    d.x = in;
    d.width = W;
    d.top = sp.top;
    d.ids = st->ids;
    d.wts = st->wts;
    d.gu = Wt.gu;
    d.down = Wt.down;
    d.ff = ff;
    d.limit = sp.expert_limit;
    d.sgu = Wt.sgu;
    d.sdown = Wt.sdown;
    d.sff = sff;
    d.slimit = sp.shared_limit;
    d.alpha = sp.act_alpha;
    d.up_add = sp.glu_up_add;
    d.sgate = sp.shared_gate ? st->sgate : nullptr;
    d.act = st->act_buf;
    d.y = one_token_out;
    return tl_launch_moe_decode(d, s);
  }
  TL_TRY(tl_launch_moe_plan(st->ids, S, sp.experts, st->off, st->slot_of, s));
  DenseArgs g = {};  // gate | up of every slot, grouped by expert: item p reads token slot_of[p] / top
  g.w = Wt.gu;
  g.rows = 2 * ff;
  g.cols = W;
  g.x = in;
  g.ldx = W;
  g.y = st->act_buf;  // the gated unit is applied in the epilogue: [S][ff]
  g.ldy = ff;
  g.T = S;
  g.terms = terms_for(st, T);
  g.x_rows = st->slot_of;
  g.x_div = sp.top;
  g.groups = sp.experts;
  g.group_off = st->off;
  g.glu = 1;
  g.glu_limit = sp.expert_limit;
  g.glu_alpha = sp.act_alpha;
  g.glu_up_add = sp.glu_up_add;
  TL_TRY(tl_launch_dense_gemm(g, s));
  DenseArgs d = {};  // down: item p writes the row of its slot, so that a token's choices lie side by side
  d.w = Wt.down;
  d.rows = W;
  d.cols = ff;
  d.x = st->act_buf;
  d.ldx = ff;
  d.y = st->eout;
  d.ldy = W;
  d.T = S;
  d.terms = terms_for(st, T);
  d.y_rows = st->slot_of;
  d.groups = sp.experts;
  d.group_off = st->off;
  TL_TRY(tl_launch_dense_gemm(d, s));
  if (sff) {
    DenseArgs u = {};  // the shared expert's gate | up with the gated unit in the epilogue, then its down projection
    u.w = Wt.sgu;
    u.rows = 2 * sff;
    u.cols = W;
    u.x = in;
    u.ldx = W;
    u.y = st->sact;
    u.ldy = sff;
    u.T = T;
    u.terms = terms_for(st, T);
    u.glu = 1;
    u.glu_limit = sp.shared_limit;
    u.glu_alpha = sp.act_alpha;
    u.glu_up_add = sp.glu_up_add;
    TL_TRY(tl_launch_dense_gemm(u, s));
    TL_TRY(project(st, Wt.sdown, W, sff, st->sact, sff, st->sout, W, T, s));
  }
  return 0;
}

RouterArgs router_args(TlStack* st, const Layer& L, const Layer& Wt, const float* in, int T) {
  const tl_layer_spec& sp = L.sp;
  RouterArgs r = {};
  r.x = in;
  r.T = T;
  r.width = st->cfg.width;
  r.experts = sp.experts;
  r.top = sp.top;
  r.w = Wt.router;
  r.b = sp.route == TL_ROUTE_TOP_LOGITS ? Wt.router_b : nullptr;
  r.ids = st->ids;
  r.wts = st->wts;
  r.kind = sp.route;
  r.groups = sp.route_groups;
  r.keep = sp.route_keep;
  if (sp.shared_gate) {
    r.gate_w = Wt.sg;
    r.gate_out = st->sgate;
  }
  return r;
}

// x += norm2(ff(x)) of a post-norm block
int moe_layer(TlStack* st, Layer& L, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const Layer& Wt = st->layers[L.wsrc];
  const int W = st->cfg.width;
  if (!st->fuse_router || sp.route != TL_ROUTE_TOP_LOGITS || sp.shared_gate)
    TL_TRY(tl_launch_router(router_args(st, L, Wt, st->x, T), s));  // (otherwise it rode in the x += N1 launch)
  ResidNormArgs n = {};
  n.x = st->x;
  n.T = T;
  n.width = W;
  n.w = Wt.norm2;
  n.eps = st->cfg.norm_eps;
  TL_REQUIRE(!sp.shared_gate, "layer-list engine: a gated shared expert runs in parallel blocks only");
  TL_TRY(moe_experts(st, L, Wt, st->x, T, st->proj, s));
  if (T == 1 && st->gemv_decode) {
    n.a = st->proj;
    return tl_launch_resid_norm(n, s);
  }
  if (sp.shared_ff) n.a = st->sout;
  n.slots = st->eout;
  n.slot_w = st->wts;
  n.top = sp.top;
  return tl_launch_resid_norm(n, s);
}

// ---- mixers: both read `in` [T][W] and leave their output in st->proj [T][W] ----
int swa_mixer(TlStack* st, Layer& L, const Layer& Wt, const float* in, int T, int start_pos, const int* pos_dev, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const tl_stack_config& c = st->cfg;
  const int W = c.width, ld = L.pd;
  TL_TRY(project(st, Wt.wqkv, ld, W, in, W, st->qkv, ld, T, s));
  if (L.rotary_path) {
    RotaryArgs r = {};
    r.qk = st->qkv;
    r.ld = ld;
    r.heads = sp.heads;
    r.kv_heads = sp.kv_heads;
    r.dim = sp.dim;
    r.rot_dims = sp.rot_dims;
    r.freq = Wt.freq;
    r.mscale = Wt.mscale;
    r.unit_norm = sp.qk_norm == TL_QK_NORM_HEAD_UNIT;
    r.eps = c.norm_eps;
    r.kc = L.kc;
    if (sp.values_are_keys) {
      r.vc = L.vc;
    } else {
      r.v_src = st->qkv + L.qd + L.kd;
      r.v_dst = L.vc;
      r.vd = L.vd;
    }
    r.T = T;
    r.start_pos = start_pos;
    r.pos_dev = pos_dev;
    TL_TRY(tl_launch_rotary(r, s));
  } else {
    QkvPostArgs q = {};
    q.qkv = st->qkv;
    q.ld = ld;
    q.qd = L.qd;
    q.kd = L.kd;
    q.vd = L.vd;
    q.q_norm = sp.qk_norm == TL_QK_NORM_WHOLE ? Wt.q_norm : nullptr;
    q.k_norm = sp.qk_norm == TL_QK_NORM_WHOLE ? Wt.k_norm : nullptr;
    q.eps = c.norm_eps;
    q.kc = L.kc;
    q.vc = L.vc;
    q.T = T;
    q.start_pos = start_pos;
    q.pos_dev = pos_dev;
    q.vmix = L.vmix_mode;
    q.v_first = st->v_first;
    q.lambda = Wt.lambda;
    TL_TRY(tl_launch_qkv_post(q, s));
  }
  SwaArgs a = {};
  a.q = st->qkv;
  a.ldq = ld;
  a.kc = L.kc;
  a.vc = L.vc;
  a.out = st->att;
  a.T = T;
  a.heads = sp.heads;
  a.kv_heads = sp.kv_heads;
  a.dim = sp.dim;
  a.vdim = sp.vdim;
  a.window = sp.window;
  a.scale = sp.scale;
  a.start_pos = start_pos;
  a.pos_dev = pos_dev;
  a.keep_first = sp.keep_first;
  a.sigmoid = sp.attn_weight == TL_ATTN_SIGMOID;
  a.head_bias = a.sigmoid ? Wt.pb : nullptr;
  a.nsplit = tl_swa_splits(T, sp.window, c.max_positions, sp.keep_first);
  a.ws = st->swa_ws;
  a.done_cnt = st->swa_cnt;
  TL_TRY(tl_launch_swa(a, s));
  return project(st, Wt.wo, W, L.od, st->att, L.od, st->proj, W, T, s);
}

int delta_mixer(TlStack* st, Layer& L, const Layer& Wt, const float* in, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ld = L.pd, dc = L.qd + L.kd + L.vd, da = sp.heads * sp.dim;
  TL_TRY(project(st, Wt.wqkv, ld, W, in, W, st->qkv, ld, T, s));  // q | k | v | beta | a1 | g1
  const float* a1 = st->qkv + dc + sp.heads;
  TL_TRY(project(st, Wt.wa2, da, sp.decay_rank, a1, ld, st->da, da, T, s));
  TL_TRY(project(st, Wt.wg2, L.vd, sp.gate_rank, a1 + sp.decay_rank, ld, st->dg, L.vd, T, s));
  DeltaPreArgs p = {};
  p.p = st->qkv;
  p.ld = ld;
  p.a = st->da;
  p.T = T;
  p.heads = sp.heads;
  p.kv_heads = sp.kv_heads;
  p.dim = sp.dim;
  p.vdim = sp.vdim;
  p.taps = sp.conv_taps;
  p.conv = Wt.conv;
  p.hist = L.hist;
  p.a_log = Wt.a_log;
  p.dt_bias = Wt.dt_bias;
  p.qkv = st->dq;
  p.beta = st->dbeta;
  p.g = st->ddecay;
  TL_TRY(tl_launch_delta_pre(p, s));
  DeltaScanArgs d = {};
  d.q = st->dq;
  d.k = st->dq + L.qd;
  d.ldq = dc;
  d.v = st->dq + L.qd + L.kd;
  d.ldv = dc;
  d.beta = st->dbeta;
  d.g = st->ddecay;
  d.state = L.state;
  d.o = st->att;
  d.T = T;
  d.heads = sp.heads;
  d.kv_heads = sp.kv_heads;
  d.dim = sp.dim;
  d.vdim = sp.vdim;
  TL_TRY(tl_launch_delta_scan(d, s));
  TL_TRY(tl_launch_gated_head_norm(st->att, st->dg, Wt.onorm, T, sp.heads, sp.vdim, st->cfg.norm_eps, s));
  return project(st, Wt.wo, W, L.od, st->att, L.od, st->proj, W, T, s);
}

DytParams dyt_of_layer(const Layer& Wt) { return DytParams{Wt.norm1_alpha, Wt.norm1, Wt.norm1_b}; }

// h = norm1(x) (already in st->h); x += mixer(h) + ff(h), and the next block's h in the same launch
int parallel_layer(TlStack* st, size_t li, int T, int start_pos, const int* pos_dev, hipStream_t s) {
  Layer& L = st->layers[li];
  const Layer& Wt = st->layers[L.wsrc];
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width;
  ResidSumArgs r = {};
  r.x = st->x;
  r.T = T;
  r.width = W;
  r.a = st->proj;
  const bool one = T == 1 && st->gemv_decode;
  const bool forked = st->fork && T == 1 && sp.mlp != TL_MLP_NONE;
  hipStream_t fs = forked ? st->side : s;  // the feed-forward's stream
  if (forked) {
    TL_HIP(hipEventRecord(st->ev_fork, s));
    TL_HIP(hipStreamWaitEvent(st->side, st->ev_fork, 0));
  }
  if (sp.mlp == TL_MLP_MOE) {
    TL_TRY(tl_launch_router(router_args(st, L, Wt, st->h, T), fs));
    TL_TRY(moe_experts(st, L, Wt, st->h, T, st->sout, fs));
    if (one) {
      r.b = st->sout;  // experts and shared expert already summed (the gate applied)
    } else {
      r.slots = st->eout;
      r.slot_w = st->wts;
      r.top = sp.top;
      if (sp.shared_ff) {
        r.b = st->sout;
        r.b_gate = sp.shared_gate ? st->sgate : nullptr;
      }
    }
  } else if (sp.mlp == TL_MLP_DENSE) {
    const int ff = sp.shared_ff;
    if (one) {
      MoeDecodeArgs d = {};  // the one gated unit runs where a shared expert would
      d.x = st->h;
      d.width = W;
      d.sgu = Wt.sgu;
      d.sdown = Wt.sdown;
      d.sff = ff;
      d.slimit = sp.shared_limit;
      d.alpha = sp.act_alpha;
      d.up_add = sp.glu_up_add;
      d.act = st->act_buf;
      d.y = st->sout;
      TL_TRY(tl_launch_moe_decode(d, fs));
    } else {
      DenseArgs u = {};
      u.w = Wt.sgu;
      u.rows = 2 * ff;
      u.cols = W;
      u.x = st->h;
      u.ldx = W;
      u.y = st->sact;
      u.ldy = ff;
      u.T = T;
      u.terms = terms_for(st, T);
      u.glu = 1;
      u.glu_limit = sp.shared_limit;
      u.glu_alpha = sp.act_alpha;
      u.glu_up_add = sp.glu_up_add;
      TL_TRY(tl_launch_dense_gemm(u, fs));
      TL_TRY(project(st, Wt.sdown, W, ff, st->sact, ff, st->sout, W, T, fs));
    }
    r.b = st->sout;
  }
  if (forked) TL_HIP(hipEventRecord(st->ev_join, st->side));
  if (sp.mixer == TL_MIXER_SWA) TL_TRY(swa_mixer(st, L, Wt, st->h, T, start_pos, pos_dev, s));
  else TL_TRY(delta_mixer(st, L, Wt, st->h, T, s));
  if (forked) TL_HIP(hipStreamWaitEvent(s, st->ev_join, 0));
  if (li + 1 < st->layers.size() && st->layers[li + 1].sp.block == TL_BLOCK_PARALLEL) {
    r.next = dyt_of_layer(st->layers[st->layers[li + 1].wsrc]);
    r.h = st->h;
  }
  return tl_launch_resid_sum(r, s);
}

}  // namespace

int tl_stack_forward(TlStack* st, const int* tokens_dev, int T, int start_pos, const int* pos_dev, const int* rows_dev,
                     int n_rows, float* logits_dev, hipStream_t s) {
  TL_REQUIRE(st && st->finalized && tokens_dev, "tl_stack_forward: model not finalized");
  TL_REQUIRE(T > 0 && T <= st->chunk, "tl_stack_forward: %d tokens outside (0, %d]", T, st->chunk);
  TL_REQUIRE(pos_dev || (start_pos >= 0 && start_pos + T <= st->cfg.max_positions),
             "tl_stack_forward: positions [%d, %d) outside the cache of %d", start_pos, start_pos + T, st->cfg.max_positions);
  TL_REQUIRE(n_rows >= 0 && n_rows <= T && (n_rows == 0 || logits_dev), "tl_stack_forward: bad logits request");
  const tl_stack_config& c = st->cfg;
  const int W = c.width;
  const bool dyt = c.norm == TL_NORM_DYT;
  if (c.embed_norm) {
    TL_TRY(tl_launch_embed_norm(st->embed, c.vocab, W, tokens_dev, T, st->embed_norm, c.norm_eps, st->x, s));
    if (dyt) TL_TRY(tl_launch_dyt_rows(st->x, W, nullptr, T, dyt_of_layer(st->layers[st->layers[0].wsrc]), st->h, s));
  } else {
    const DytParams first = dyt ? dyt_of_layer(st->layers[st->layers[0].wsrc]) : DytParams{};
    TL_TRY(tl_launch_embed_rows(st->embed, c.vocab, W, tokens_dev, T, st->x, first, st->h, s));
  }
  for (size_t li = 0; li < st->layers.size(); ++li) {
    Layer& L = st->layers[li];
    const tl_layer_spec& sp = L.sp;
    if (sp.block == TL_BLOCK_PARALLEL) {
      TL_TRY(parallel_layer(st, li, T, start_pos, pos_dev, s));
    } else {
      const Layer& Wt = st->layers[L.wsrc];
      TL_TRY(swa_mixer(st, L, Wt, st->x, T, start_pos, pos_dev, s));
      ResidNormArgs n = {};
      n.x = st->x;
      n.T = T;
      n.width = W;
      n.a = st->proj;
      n.w = Wt.norm1;
      n.eps = c.norm_eps;
      if (sp.mlp == TL_MLP_MOE && st->fuse_router && sp.route == TL_ROUTE_TOP_LOGITS && !sp.shared_gate) {
        n.route.w = Wt.router;  // the router reads the row this launch has just finished
        n.route.b = Wt.router_b;
        n.route.experts = sp.experts;
        n.route.top = sp.top;
        n.route.ids = st->ids;
        n.route.wts = st->wts;
      }
      TL_TRY(tl_launch_resid_norm(n, s));
      if (sp.mlp == TL_MLP_MOE) TL_TRY(moe_layer(st, L, T, s));
    }
    if (st->hook) {
      TL_HIP(hipStreamSynchronize(s));
      st->hook(st->hook_ctx, (int)li, st->x, T, W);
    }
  }
  if (n_rows > 0) {
    const int last = T - 1;
    const float* src = st->x;
    if (!rows_dev && n_rows == 1) src = st->x + (size_t)last * W;
    TL_REQUIRE(rows_dev || n_rows == 1 || n_rows == T, "tl_stack_forward: %d rows without a list", n_rows);
    if (dyt) TL_TRY(tl_launch_dyt_rows(src, W, rows_dev, n_rows, DytParams{st->final_alpha, st->final_norm, st->final_b}, st->xn, s));
    else TL_TRY(tl_launch_norm_rows(src, W, rows_dev, n_rows, st->final_norm, c.norm_eps, st->xn, s));
    TL_TRY(project(st, st->head, c.vocab, W, st->xn, W, logits_dev, c.vocab, n_rows, s, c.logit_softcap));
  }
  return 0;
}
