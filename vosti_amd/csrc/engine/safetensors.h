// Reads safetensors files by mapping them: an 8-byte little-endian header length, a JSON header
// {name: {dtype, shape, data_offsets}}, then the tensors' bytes.  File mechanics follow the reference's
// helper (python/vosti_kernels/checkpoint.py:15-78): model.safetensors.index.json with its weight_map if
// present, else one model.safetensors; shard paths stay inside the model folder.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "../host/files.h"

namespace vosti {

struct StoredTensor {
  std::string dtype;               // as the file names it: BF16, F32, F16, I64, ...
  std::vector<int64_t> shape;
  const unsigned char* data = nullptr;
  size_t bytes = 0;
  std::string file;
};

class Checkpoint {
 public:
  explicit Checkpoint(const std::string& model_dir);
  ~Checkpoint();
  Checkpoint(const Checkpoint&) = delete;
  const std::map<std::string, StoredTensor>& entries() const { return entries_; }
  const std::string& dir() const { return dir_; }

 private:
  struct Mapping {
    void* base;
    size_t bytes;
  };
  void map_file(const std::string& path);
  std::string dir_;
  std::vector<Mapping> maps_;
  std::map<std::string, StoredTensor> entries_;
};

}  // namespace vosti
