// tl_registry.hpp — the model families the host layer can open, keyed by the architecture name a checkpoint carries.
//
// The reference has one family (the Llama block, read from a GGUF file: model_config.cpp:149-221, weight_management.cpp);
// this table is where another one is added: a name, how its checkpoint is recognised, and a loader that parses the
// configuration, creates the device model through the C-ABI and uploads the tensors. Session asks the table and keeps
// the resulting tl_model handle; everything after that (prefill, decode step, sampling, generation loops) goes through
// the same tl_model_* entry points for every family.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "tl_session.hpp"

namespace tlhost {

struct LoadedModel {
  tl_model* model = nullptr;
  ModelConfig config;
  LoadStats stats;
  std::unique_ptr<Tokenizer> tokenizer;  // null when the checkpoint carries none
  bool multi_sequence = false;           // the device model has the multi-sequence decode step (tl_model_batch_*)
  int exact_terms = 6;                   // tl_model_set_prefill terms that make the chunk GEMMs FP32-grade
  int serving_terms = 0;                 // ... and the family's default
};

struct ModelFamily {
  const char* name;       // architecture as checkpoints spell it
  const char* container;  // "gguf": one file; "folder": config.json + model.safetensors
  void (*load)(const std::string& path, int device, int max_context, LoadedModel* out);
};

const std::vector<ModelFamily>& model_families();
// nullptr when no family has that name (GGUF files of any *llama-like* architecture name go to the Llama family, as the
// reference reads every GGUF file through the llama.* keys)
const ModelFamily* find_model_family(const std::string& architecture, const std::string& container);
// `path`: a .gguf file, a folder holding config.json, or that config.json itself. Returns the architecture named there and
// sets *container and *resolved (the file or folder a loader takes).
std::string detect_architecture(const std::string& path, std::string* container, std::string* resolved);

// the loaders (tl_session.cpp, tl_stack_config.cpp)
void load_llama_gguf(const std::string& path, int device, int max_context, LoadedModel* out);
void load_stack_folder(const std::string& path, int device, int max_context, LoadedModel* out);

}  // namespace tlhost
