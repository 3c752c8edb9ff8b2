// tl_stack.hip — the layer-list engine: a decoder described layer by layer (tl_stack_config) instead of by the fixed Llama
// block of tl_model.hip. It owns the bf16 weights, the per-layer FP32 key/value caches and the chunk workspaces, and runs
// T tokens through all layers: T = 1 is the decode step (GEMVs, position and token id read from the device, so the step
// can be captured into a hipGraph by tl_model.hip like the Llama step), T > 1 a chunk of a prompt (MFMA GEMMs).
//
// A layer:  x += norm1(mixer(x));  x += norm2(ff(x))  -- the sublayers read x itself, the norm is on their OUTPUT
//   mixer TL_MIXER_SWA  q | k | v = W_qkv x (one product over the concatenated rows); RMS norm over the whole q and the whole
//                       k projection; optional value mixing with the values of the first mixing layer (same token);
//                       k, v -> cache; sliding-window attention without rotation (tl_swa.hip); W_o
//   ff    TL_MLP_MOE    router -> top experts (clamped gated units) weighted by the softmax over the chosen logits, plus an
//                       optional shared expert for every token
// The residual stream, norms, router, attention scores and the cache are FP32; matrix operands of a prompt chunk are bf16
// (terms = 1) or the FP32-grade three-term split (terms = 3), see tl_dense.hip; the decode step's GEMVs are FP32 throughout.
//
// Cache: per layer K [max_positions][kv_heads * dim] and V [max_positions][kv_heads * vdim], flat by absolute position; a
// window only bounds what attention reads. tl_stack_reset gives everything back (one sequence at a time).
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "tl_stack.h"

namespace {

struct Layer {
  tl_layer_spec sp;
  int qd = 0, kd = 0, vd = 0, od = 0;  // q / k / v projection sizes, attention output size (heads * vdim)
  int vmix_mode = 0;                   // 0 none, 1 first mixing layer, 2 mixes with the first
  uint16_t *wqkv = nullptr, *wo = nullptr;
  float *q_norm = nullptr, *k_norm = nullptr, *lambda = nullptr, *norm1 = nullptr, *norm2 = nullptr;
  uint16_t *router = nullptr, *gu = nullptr, *down = nullptr, *sgu = nullptr, *sdown = nullptr;
  float* router_b = nullptr;
  float *kc = nullptr, *vc = nullptr;
  size_t got = 0, need = 0;  // tensors received / expected
};

}  // namespace

struct TlStack {
  tl_stack_config cfg;
  std::vector<Layer> layers;
  uint16_t *embed = nullptr, *head = nullptr;
  float *embed_norm = nullptr, *final_norm = nullptr;
  int got_globals = 0;
  std::vector<void*> allocs;
  bool finalized = false;
  int terms = 1;
  // tokens of a prompt that go through the layers together. Measured at width 4096 with 16 experts (top 4): 105.9 k tokens/s
  // at 512, 140.4 k at 1024, 171.6 k at 2048 -- the experts' grouped GEMMs see 4 x the tokens per expert, the dense ones
  // enough tiles for the 128 x 128 shape.
  int chunk = 2048;
  bool gemv_decode = true;
  bool fuse_router = true;  // TL_STACK_FUSE_ROUTER=0: the router as a launch of its own (A/B, tests)
  // workspaces for one chunk
  float *x = nullptr, *qkv = nullptr, *att = nullptr, *proj = nullptr, *v_first = nullptr, *xn = nullptr;
  float *act_buf = nullptr, *eout = nullptr, *sact = nullptr, *sout = nullptr;
  float* wts = nullptr;
  float* swa_ws = nullptr;  // partial results of split attention launches (few tokens, long windows)
  unsigned* swa_cnt = nullptr;  // their arrival counters (zero between launches)
  int *ids = nullptr, *off = nullptr, *slot_of = nullptr;
  int max_qkv = 0, max_od = 0, max_vd = 0, max_top = 0, max_experts = 0, max_gu = 0, max_sff = 0;
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
  for (int i = 0; i < cfg->n_layers && rc == 0; ++i) {
    Layer& L = st->layers[i];
    L.sp = cfg->layers[i];
    const tl_layer_spec& sp = L.sp;
    if (sp.mixer != TL_MIXER_SWA) {
      tl_set_error("tl_stack_create: layer %d has mixer kind %d; this engine has sliding-window attention (%d)", i, sp.mixer,
                   TL_MIXER_SWA);
      return fail(2);
    }
    if (sp.heads <= 0 || sp.kv_heads <= 0 || sp.heads % sp.kv_heads != 0 || sp.dim <= 0 || sp.vdim <= 0) {
      tl_set_error("tl_stack_create: layer %d: %d heads / %d key-value heads / sizes %d, %d", i, sp.heads, sp.kv_heads, sp.dim,
                   sp.vdim);
      return fail(2);
    }
    L.qd = sp.heads * sp.dim;
    L.kd = sp.kv_heads * sp.dim;
    L.vd = sp.kv_heads * sp.vdim;
    L.od = sp.heads * sp.vdim;
    if (sp.v_mix) {
      if (first_mix < 0) {
        first_mix = i;
        L.vmix_mode = 1;
      } else {
        L.vmix_mode = 2;
        if (st->layers[first_mix].vd != L.vd) {
          tl_set_error("tl_stack_create: layer %d mixes %d values with the %d of layer %d", i, L.vd, st->layers[first_mix].vd,
                       first_mix);
          return fail(2);
        }
      }
    }
    L.need = 5 + (sp.qk_norm ? 2 : 0) + (L.vmix_mode == 2 ? 1 : 0);  // q k v o norm1 (+ the feed-forward's below)
    if ((rc = dev_alloc(st, &L.wqkv, (size_t)(L.qd + L.kd + L.vd) * W))) break;
    if ((rc = dev_alloc(st, &L.wo, W * L.od))) break;
    if ((rc = dev_alloc(st, &L.q_norm, L.qd))) break;
    if ((rc = dev_alloc(st, &L.k_norm, L.kd))) break;
    if ((rc = dev_alloc(st, &L.lambda, 1))) break;
    if ((rc = dev_alloc(st, &L.norm1, W))) break;
    if ((rc = dev_alloc(st, &L.norm2, W))) break;
    if (sp.mlp == TL_MLP_MOE) {
      if (sp.experts <= 0 || sp.top <= 0 || sp.top > sp.experts || sp.expert_ff <= 0 || sp.shared_ff < 0) {
        tl_set_error("tl_stack_create: layer %d: %d experts, top %d, sizes %d / %d", i, sp.experts, sp.top, sp.expert_ff,
                     sp.shared_ff);
        return fail(2);
      }
      L.need += 1 /*norm2*/ + 2 /*router, bias*/ + 3 * (size_t)sp.experts + (sp.shared_ff ? 3 : 0);
      if ((rc = dev_alloc(st, &L.router, (size_t)sp.experts * W))) break;
      if ((rc = dev_alloc(st, &L.router_b, sp.experts))) break;
      if ((rc = dev_alloc(st, &L.gu, (size_t)sp.experts * 2 * sp.expert_ff * W))) break;
      if ((rc = dev_alloc(st, &L.down, (size_t)sp.experts * W * sp.expert_ff))) break;
      if (sp.shared_ff) {
        if ((rc = dev_alloc(st, &L.sgu, (size_t)2 * sp.shared_ff * W))) break;
        if ((rc = dev_alloc(st, &L.sdown, W * sp.shared_ff))) break;
      }
      st->max_top = sp.top > st->max_top ? sp.top : st->max_top;
      st->max_experts = sp.experts > st->max_experts ? sp.experts : st->max_experts;
      st->max_gu = 2 * sp.expert_ff * sp.top > st->max_gu ? 2 * sp.expert_ff * sp.top : st->max_gu;
      st->max_sff = sp.shared_ff > st->max_sff ? sp.shared_ff : st->max_sff;
    } else if (sp.mlp != TL_MLP_NONE) {
      tl_set_error("tl_stack_create: layer %d has feed-forward kind %d", i, sp.mlp);
      return fail(2);
    }
    const int qkv = L.qd + L.kd + L.vd;
    st->max_qkv = qkv > st->max_qkv ? qkv : st->max_qkv;
    st->max_od = L.od > st->max_od ? L.od : st->max_od;
    st->max_vd = L.vd > st->max_vd ? L.vd : st->max_vd;
    st->cache_bytes += sizeof(float) * (size_t)cfg->max_positions * (L.kd + L.vd);
  }
  if (rc) return fail(rc);
  if ((rc = dev_alloc(st, &st->embed, (size_t)cfg->vocab * W)) || (rc = dev_alloc(st, &st->head, (size_t)cfg->vocab * W)) ||
      (rc = dev_alloc(st, &st->embed_norm, W)) || (rc = dev_alloc(st, &st->final_norm, W)))
    return fail(rc);
  if (const char* e = getenv("TL_STACK_CHUNK")) st->chunk = atoi(e) > 0 ? atoi(e) : st->chunk;
  if (const char* e = getenv("TL_STACK_GEMV")) st->gemv_decode = atoi(e) != 0;
  if (const char* e = getenv("TL_STACK_FUSE_ROUTER")) st->fuse_router = atoi(e) != 0;
  *out = st;
  return 0;
}

void tl_stack_free(TlStack* st) {
  if (!st) return;
  for (void* p : st->allocs) hipFree(p);
  hipFree(st->cache_base);
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
  int li = -1, used = 0;
  TL_REQUIRE(sscanf(name, "l%d.%n", &li, &used) == 1 && used > 0 && li >= 0 && li < st->cfg.n_layers,
             "tl_stack_set_tensor: no place for a tensor named %s", name);
  Layer& L = st->layers[li];
  const tl_layer_spec& sp = L.sp;
  const std::string r = n.substr(used);
  ++L.got;
  if (r == "norm1") VECTOR(L.norm1, W);
  if (r == "norm2") {
    if (sp.mlp == TL_MLP_NONE) --L.got;  // present but unused
    VECTOR(L.norm2, W);
  }
  if (r == "mix.q") MATRIX(L.wqkv, L.qd, W);
  if (r == "mix.k") MATRIX(L.wqkv + (size_t)L.qd * W, L.kd, W);
  if (r == "mix.v") MATRIX(L.wqkv + (size_t)(L.qd + L.kd) * W, L.vd, W);
  if (r == "mix.o") MATRIX(L.wo, W, L.od);
  if (r == "mix.q.norm") {
    if (!sp.qk_norm) --L.got;
    VECTOR(L.q_norm, L.qd);
  }
  if (r == "mix.k.norm") {
    if (!sp.qk_norm) --L.got;
    VECTOR(L.k_norm, L.kd);
  }
  if (r == "mix.vmix") {
    if (L.vmix_mode != 2) --L.got;  // the first mixing layer's coefficient is never read
    VECTOR(L.lambda, 1);
  }
  if (sp.mlp == TL_MLP_MOE) {
    const long long ff = sp.expert_ff, sff = sp.shared_ff;
    if (r == "mlp.router") MATRIX(L.router, sp.experts, W);
    if (r == "mlp.router.b") VECTOR(L.router_b, sp.experts);
    if (sff) {
      if (r == "mlp.shared.gate") PAIRED(L.sgu, sff, W);  // gate | up interleaved by unit (DenseArgs::glu)
      if (r == "mlp.shared.up") PAIRED(L.sgu + W, sff, W);
      if (r == "mlp.shared.down") MATRIX(L.sdown, W, sff);
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
  --L.got;
  TL_REQUIRE(false, "tl_stack_set_tensor: no place for a tensor named %s in layer %d", name, li);
#undef MATRIX
#undef PAIRED
#undef VECTOR
}

int tl_stack_finalize(TlStack* st, hipStream_t s) {
  TL_REQUIRE(st, "tl_stack_finalize: null handle");
  if (st->finalized) return 0;
  TL_REQUIRE(st->got_globals == 15, "tl_stack_finalize: embed / embed.norm / final.norm / head missing (mask %d)",
             st->got_globals);
  for (size_t i = 0; i < st->layers.size(); ++i)
    TL_REQUIRE(st->layers[i].got == st->layers[i].need, "tl_stack_finalize: layer %d received %zu of its %zu tensors", (int)i,
               st->layers[i].got, st->layers[i].need);
  const size_t W = st->cfg.width, C = st->chunk;
  TL_HIP(hipMalloc(&st->cache_base, st->cache_bytes));
  float* p = static_cast<float*>(st->cache_base);
  for (Layer& L : st->layers) {
    L.kc = p;
    p += (size_t)st->cfg.max_positions * L.kd;
    L.vc = p;
    p += (size_t)st->cfg.max_positions * L.vd;
  }
  TL_TRY(dev_alloc(st, &st->x, C * W));
  TL_TRY(dev_alloc(st, &st->qkv, C * st->max_qkv));
  TL_TRY(dev_alloc(st, &st->att, C * st->max_od));
  TL_TRY(dev_alloc(st, &st->proj, C * W));
  TL_TRY(dev_alloc(st, &st->v_first, C * st->max_vd));
  TL_TRY(dev_alloc(st, &st->xn, C * W));
  {
    size_t ws = 1;
    for (const Layer& L : st->layers)
      for (int T = 1; T <= 4; ++T) {
        const size_t n = tl_swa_ws_floats(T, L.sp.heads, L.sp.vdim, tl_swa_splits(T, L.sp.window, st->cfg.max_positions));
        ws = n > ws ? n : ws;
      }
    TL_TRY(dev_alloc(st, &st->swa_ws, ws));
    size_t heads = 1;
    for (const Layer& L : st->layers) heads = (size_t)L.sp.heads > heads ? (size_t)L.sp.heads : heads;
    TL_TRY(dev_alloc(st, &st->swa_cnt, 4 * heads));
    TL_HIP(hipMemsetAsync(st->swa_cnt, 0, sizeof(unsigned) * 4 * heads, s));
  }
  if (st->max_top) {
    const size_t S = C * st->max_top;
    TL_TRY(dev_alloc(st, &st->ids, S));
    TL_TRY(dev_alloc(st, &st->wts, S));
    TL_TRY(dev_alloc(st, &st->slot_of, S));
    TL_TRY(dev_alloc(st, &st->off, (size_t)st->max_experts + 1));
    TL_TRY(dev_alloc(st, &st->act_buf, C * st->max_gu / 2 + st->max_sff));
    TL_TRY(dev_alloc(st, &st->eout, S * W));
    if (st->max_sff) {
      TL_TRY(dev_alloc(st, &st->sact, C * st->max_sff));
      TL_TRY(dev_alloc(st, &st->sout, C * W));
    }
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
  *out = which == 0 ? st->layers[layer].kc : st->layers[layer].vc;
  return 0;
}

void tl_stack_bytes_per_token(const TlStack* st, int pos, double* weight_bytes, double* kv_bytes) {
  const double W = st->cfg.width;
  double wb = 2.0 * W /*embedding row*/ + 2.0 * W * st->cfg.vocab, kb = 0.0;
  for (const Layer& L : st->layers) {
    const tl_layer_spec& sp = L.sp;
    wb += 2.0 * W * (L.qd + L.kd + L.vd + L.od);
    if (sp.mlp == TL_MLP_MOE)
      wb += 2.0 * W * (sp.experts + 3.0 * sp.expert_ff * sp.top + 3.0 * sp.shared_ff);
    const double seen = sp.window > 0 && pos + 1 > sp.window ? sp.window : pos + 1;
    kb += 4.0 * (seen + 1.0) * (L.kd + L.vd);
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
            hipStream_t s) {
  if (T == 1 && st->gemv_decode) return tl_launch_dense_gemv(w, rows, cols, x, y, s);
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
  return tl_launch_dense_gemm(d, s);
}

int moe_layer(TlStack* st, Layer& L, int T, hipStream_t s) {
  const tl_layer_spec& sp = L.sp;
  const int W = st->cfg.width, ff = sp.expert_ff, sff = sp.shared_ff, S = T * sp.top;
  RouterArgs r = {};
  r.x = st->x;
  r.T = T;
  r.width = W;
  r.experts = sp.experts;
  r.top = sp.top;
  r.w = L.router;
  r.b = L.router_b;
  r.ids = st->ids;
  r.wts = st->wts;
  if (!st->fuse_router) TL_TRY(tl_launch_router(r, s));  // (otherwise it rode in the x += N1 launch)
  ResidNormArgs n = {};
  n.x = st->x;
  n.T = T;
  n.width = W;
  n.w = L.norm2;
  n.eps = st->cfg.norm_eps;
  if (T == 1 && st->gemv_decode) {
    MoeDecodeArgs d = {};
    d.x = st->x;
    d.width = W;
    d.top = sp.top;
    d.ids = st->ids;
    d.wts = st->wts;
    d.gu = L.gu;
    d.down = L.down;
    d.ff = ff;
    d.limit = sp.expert_limit;
    d.sgu = L.sgu;
    d.sdown = L.sdown;
    d.sff = sff;
    d.slimit = sp.shared_limit;
    d.alpha = sp.act_alpha;
    d.act = st->act_buf;
    d.y = st->proj;
    TL_TRY(tl_launch_moe_decode(d, s));
    n.a = st->proj;
    return tl_launch_resid_norm(n, s);
  }
  TL_TRY(tl_launch_moe_plan(st->ids, S, sp.experts, st->off, st->slot_of, s));
  DenseArgs g = {};  // gate | up of every slot, grouped by expert: item p reads token slot_of[p] / top
  g.w = L.gu;
  g.rows = 2 * ff;
  g.cols = W;
  g.x = st->x;
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
  TL_TRY(tl_launch_dense_gemm(g, s));
  DenseArgs d = {};  // down: item p writes the row of its slot, so that a token's choices lie side by side
  d.w = L.down;
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
    u.w = L.sgu;
    u.rows = 2 * sff;
    u.cols = W;
    u.x = st->x;
    u.ldx = W;
    u.y = st->sact;
    u.ldy = sff;
    u.T = T;
    u.terms = terms_for(st, T);
    u.glu = 1;
    u.glu_limit = sp.shared_limit;
    u.glu_alpha = sp.act_alpha;
    TL_TRY(tl_launch_dense_gemm(u, s));
    TL_TRY(project(st, L.sdown, W, sff, st->sact, sff, st->sout, W, T, s));
    n.a = st->sout;
  }
  n.slots = st->eout;
  n.slot_w = st->wts;
  n.top = sp.top;
  return tl_launch_resid_norm(n, s);
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
  TL_TRY(tl_launch_embed_norm(st->embed, c.vocab, W, tokens_dev, T, st->embed_norm, c.norm_eps, st->x, s));
  for (size_t li = 0; li < st->layers.size(); ++li) {
    Layer& L = st->layers[li];
    const tl_layer_spec& sp = L.sp;
    const int ld = L.qd + L.kd + L.vd;
    TL_TRY(project(st, L.wqkv, ld, W, st->x, W, st->qkv, ld, T, s));
    QkvPostArgs q = {};
    q.qkv = st->qkv;
    q.ld = ld;
    q.qd = L.qd;
    q.kd = L.kd;
    q.vd = L.vd;
    q.q_norm = sp.qk_norm ? L.q_norm : nullptr;
    q.k_norm = sp.qk_norm ? L.k_norm : nullptr;
    q.eps = c.norm_eps;
    q.kc = L.kc;
    q.vc = L.vc;
    q.T = T;
    q.start_pos = start_pos;
    q.pos_dev = pos_dev;
    q.vmix = L.vmix_mode;
    q.v_first = st->v_first;
    q.lambda = L.lambda;
    TL_TRY(tl_launch_qkv_post(q, s));
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
    a.nsplit = tl_swa_splits(T, sp.window, c.max_positions);
    a.ws = st->swa_ws;
    a.done_cnt = st->swa_cnt;
    TL_TRY(tl_launch_swa(a, s));
    TL_TRY(project(st, L.wo, W, L.od, st->att, L.od, st->proj, W, T, s));
    ResidNormArgs n = {};
    n.x = st->x;
    n.T = T;
    n.width = W;
    n.a = st->proj;
    n.w = L.norm1;
    n.eps = c.norm_eps;
    if (sp.mlp == TL_MLP_MOE && st->fuse_router) {  // the router reads the row this launch has just finished
      n.route.w = L.router;
      n.route.b = L.router_b;
      n.route.experts = sp.experts;
      n.route.top = sp.top;
      n.route.ids = st->ids;
      n.route.wts = st->wts;
    }
    TL_TRY(tl_launch_resid_norm(n, s));
    if (sp.mlp == TL_MLP_MOE) TL_TRY(moe_layer(st, L, T, s));
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
    TL_TRY(tl_launch_norm_rows(src, W, rows_dev, n_rows, st->final_norm, c.norm_eps, st->xn, s));
    TL_TRY(project(st, st->head, c.vocab, W, st->xn, W, logits_dev, c.vocab, n_rows, s));
  }
  return 0;
}
