// tl_stack_config.cpp — loader of the layer-list family (tl_registry.hpp): config.json -> tl_stack_config, model.safetensors
// -> tl_model_set_tensor_named. Every size and every constant that can differ between two models of the design is read from
// the file; what the design fixes (the gate's 1.702, the whole-projection query/key norm) is set here.
//
// config.json: {"architecture", "width", "vocab", "norm": {"eps"}, "layers": [{"type": "attention",
//   "mixer": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}, "v_mix"},
//   "mlp": null | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff", "limit"}, "shared": null | {"ff", "limit"}}}]}
#include <chrono>
#include <fstream>
#include <sstream>
#include <stdexcept>

#include "tl_json.hpp"
#include "tl_registry.hpp"
#include "tl_safetensors.hpp"

namespace tlhost {

namespace {

constexpr float kGateAlpha = 1.702f;   // g * sigmoid(1.702 g): fixed by the design
constexpr int kDefaultContext = 4096;  // cache rows when the caller names no context length

void hip_check(int rc, const std::string& what) {
  if (rc != 0) throw std::runtime_error("tlhip: " + what + ": " + tl_last_error());
}

int geti(const Json& o, const char* key) { return (int)o.at(key).as_int(key); }

tl_layer_spec layer_from_json(const Json& L, int index) {
  const std::string where = "layers[" + std::to_string(index) + "]";
  tl_layer_spec sp = {};
  const std::string& type = L.at("type").as_string("type");
  if (type != "attention") throw std::runtime_error(where + ": unknown layer type \"" + type + "\"");
  const Json& mx = L.at("mixer");
  sp.mixer = TL_MIXER_SWA;
  sp.heads = geti(mx, "heads");
  sp.kv_heads = geti(mx, "kv_heads");
  sp.dim = geti(mx, "dim");
  sp.vdim = geti(mx, "vdim");
  sp.scale = (float)mx.at("scale").as_double("scale");
  const Json* mask = mx.find("mask");
  sp.window = (mask && !mask->is_null()) ? geti(*mask, "size") : 0;
  const Json* vm = mx.find("v_mix");
  sp.v_mix = vm && vm->truthy();
  sp.qk_norm = 1;
  sp.act_alpha = kGateAlpha;
  const Json* ml = L.find("mlp");
  if (ml && !ml->is_null()) {
    const Json* kind = ml->find("kind");
    if (kind && kind->as_string("kind") != "moe")
      throw std::runtime_error(where + ": unknown feed-forward kind \"" + kind->str + "\"");
    sp.mlp = TL_MLP_MOE;
    sp.experts = geti(ml->at("router"), "experts");
    sp.top = geti(ml->at("router"), "top");
    sp.expert_ff = geti(ml->at("expert"), "ff");
    sp.expert_limit = (float)ml->at("expert").at("limit").as_double("limit");
    const Json* sh = ml->find("shared");
    if (sh && !sh->is_null()) {
      sp.shared_ff = geti(*sh, "ff");
      sp.shared_limit = (float)sh->at("limit").as_double("limit");
    }
  }
  return sp;
}

}  // namespace

void load_stack_folder(const std::string& dir, int device, int max_context, LoadedModel* out) {
  const auto t0 = std::chrono::steady_clock::now();
  std::ifstream in(dir + "/config.json");
  if (!in) throw std::runtime_error("cannot open " + dir + "/config.json");
  std::stringstream ss;
  ss << in.rdbuf();
  const Json cfg = Json::parse(ss.str());
  const Json& layers = cfg.at("layers");
  if (layers.kind != Json::ARRAY || layers.arr.empty()) throw std::runtime_error("config.json: \"layers\" is empty");
  std::vector<tl_layer_spec> specs;
  for (size_t i = 0; i < layers.arr.size(); ++i) specs.push_back(layer_from_json(layers.arr[i], (int)i));
  tl_stack_config sc = {};
  sc.width = geti(cfg, "width");
  sc.vocab = geti(cfg, "vocab");
  sc.n_layers = (int)specs.size();
  sc.max_positions = max_context > 0 ? max_context : kDefaultContext;
  sc.norm_eps = (float)cfg.at("norm").at("eps").as_double("norm.eps");
  sc.layers = specs.data();

  ModelConfig& mc = out->config;
  mc.architecture = cfg.at("architecture").as_string("architecture");
  mc.name = mc.architecture;
  mc.hidden_size = sc.width;
  mc.vocab_size = sc.vocab;
  mc.num_hidden_layers = sc.n_layers;
  mc.max_position_embeddings = sc.max_positions;
  mc.rms_norm_eps = sc.norm_eps;
  mc.num_attention_heads = specs[0].heads;
  mc.num_key_value_heads = specs[0].kv_heads;
  mc.intermediate_size = specs[0].expert_ff;
  mc.bos_token_id = -1;  // token ids in, token ids out: such a checkpoint carries no tokenizer
  mc.eos_token_id = -1;
  if (const Json* e = cfg.find("eos"))
    if (e->kind == Json::NUMBER) mc.eos_token_id = (int)e->as_int("eos");

  hip_check(tl_init(device), "tl_init");
  hip_check(tl_model_create_stack(&sc, &out->model), "tl_model_create_stack");
  try {
    SafeTensorsFile file;
    file.open(dir + "/model.safetensors");
    for (const SafeTensor& t : file.tensors()) {
      int type = -1;
      if (t.dtype == "BF16") type = TL_BF16;
      else if (t.dtype == "F32") type = TL_F32;
      else if (t.dtype == "I32" || t.dtype == "I64") continue;  // integer tables belong to other designs
      else throw std::runtime_error("tensor " + t.name + " has dtype " + t.dtype + "; this family holds BF16 (and F32 vectors)");
      hip_check(tl_model_set_tensor_named(out->model, t.name.c_str(), type, t.shape.data(), (int)t.shape.size(), t.data),
                "tl_model_set_tensor_named " + t.name);
      ++out->stats.tensors;
      out->stats.quantized_bytes += t.nbytes;
    }
    hip_check(tl_model_finalize(out->model), "tl_model_finalize");
  } catch (...) {
    tl_model_free(out->model);
    out->model = nullptr;
    throw;
  }
  out->multi_sequence = false;
  out->exact_terms = 3;
  out->serving_terms = 1;
  out->stats.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

}  // namespace tlhost
