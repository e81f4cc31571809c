// A decoder assembled from parts as a ModelSpec says, and its weights.
//
// The model owns its parts and the order in which the layers run; it owns no cache.  forward() runs the
// tokens of one step and returns logits for the rows that are asked for
// (src/exec/dense_swiglu_model.rs:131-1041: embedding, the layers, final norm, row selection before the
// vocabulary projection).
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "parts.h"
#include "safetensors.h"

namespace vosti {

struct WeightError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// A tensor of the weight files: its shape and type rule, and every (part, local name) that gets it.
struct ExpectedTensor {
  ParamDecl decl;
  std::vector<std::pair<Part*, std::string>> owners;
};

class DecoderModel {
 public:
  DecoderModel(ModelSpec spec, Kernels& kernels);
  const ModelSpec& spec() const { return spec_; }
  Kernels& kernels() { return kernels_; }

  std::vector<Part*> parts();                               // every part, sub-parts included
  std::map<std::string, ExpectedTensor> expected_tensors();
  // Checks the folder against the model (one error lists missing, unexpected and misshapen tensors), then
  // loads tensor by tensor: floats become the compute type (a keep_f32 tensor stored in 32-bit stays so),
  // integers int32.
  void load_weights(const Checkpoint& ckpt);
  // Random weights from a seed, drawn on the GPU: every element is a function of (seed, tensor name, element
  // index), the values the Python package's random-weights mode stores for the same seed in the compute type.
  void random_weights(uint64_t seed);
  bool replayable();                                        // every part's launches depend on arrays on the GPU alone
  std::vector<CacheNeed> cache_needs();                     // one per schedule entry (None if it reads another's)
  // ids int32 [T]; caches: one per schedule entry; want_rows int32 [R] -> logits [R, vocab].
  Tensor forward(const Tensor& ids, StepContext& ctx, std::vector<CacheEntry>& caches, const Tensor& want_rows);

 private:
  ModelSpec spec_;
  Kernels& kernels_;
  std::unique_ptr<Embedding> embedding_;
  std::vector<std::unique_ptr<Block>> layers_;
  std::unique_ptr<Norm> final_norm_;
  std::unique_ptr<Head> head_;
  bool loaded_ = false;
};

// The seed of a tensor's stream: the first 8 bytes, little-endian, of BLAKE2b-64("<seed>:<name>").
uint64_t tensor_seed(uint64_t seed, const std::string& name);

// Uploads one stored tensor, converted as the rule above says.
Tensor upload_tensor(const StoredTensor& t, DType compute, bool keep_f32);

}  // namespace vosti
