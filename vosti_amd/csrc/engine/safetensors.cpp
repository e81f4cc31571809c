#include "safetensors.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <climits>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <set>
#include <sstream>

#include "gpu.h"
#include "../host/json.h"

namespace vosti {

static std::string real_path(const std::string& p) {
  char buf[PATH_MAX];
  if (!realpath(p.c_str(), buf)) throw EngineError("no such path: " + p);
  return buf;
}

static const std::map<std::string, int>& stored_sizes() {
  static const std::map<std::string, int> m = {{"F64", 8}, {"F32", 4}, {"F16", 2}, {"BF16", 2}, {"I64", 8}, {"I32", 4},
                                               {"I16", 2}, {"I8", 1},  {"U8", 1},  {"BOOL", 1}};
  return m;
}

Checkpoint::Checkpoint(const std::string& model_dir) : dir_(real_path(model_dir)) {
  const std::string index = dir_ + "/model.safetensors.index.json";
  std::set<std::string> files;
  if (file_exists(index)) {
    const Json j = Json::parse(read_text_file(index));
    const Json* wm = j.get("weight_map");
    if (!wm || wm->kind != Json::Object || wm->members.empty()) throw EngineError(index + " has no 'weight_map'");
    for (const auto& m : wm->members) files.insert(m.second.text);
  } else if (file_exists(dir_ + "/model.safetensors")) {
    files.insert("model.safetensors");
  } else {
    throw EngineError(dir_ + " holds neither model.safetensors nor model.safetensors.index.json");
  }
  for (const std::string& f : files) {
    const std::string joined = dir_ + "/" + f;
    if (!file_exists(joined)) throw EngineError("shard " + joined + " is missing");
    const std::string path = real_path(joined);
    if (path.compare(0, dir_.size() + 1, dir_ + "/") != 0) throw EngineError("shard '" + f + "' lies outside the model folder");
    map_file(path);
  }
}

Checkpoint::~Checkpoint() {
  for (const Mapping& m : maps_) munmap(m.base, m.bytes);
}

void Checkpoint::map_file(const std::string& path) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) throw EngineError("cannot open " + path);
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 0) {
    close(fd);
    throw EngineError("cannot read the size of " + path);
  }
  const size_t size = (size_t)st.st_size;
  if (size < 8) {
    close(fd);
    throw EngineError(path + " is too short for a safetensors file");
  }
  void* base = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (base == MAP_FAILED) throw EngineError("cannot map " + path);
  maps_.push_back({base, size});
  const unsigned char* p = static_cast<const unsigned char*>(base);
  uint64_t header_len = 0;
  for (int i = 7; i >= 0; --i) header_len = (header_len << 8) | p[i];
  if (header_len > size - 8) throw EngineError(path + ": the header is longer than the file");
  const Json header = Json::parse(std::string(reinterpret_cast<const char*>(p + 8), (size_t)header_len));
  const size_t data_start = 8 + (size_t)header_len;
  for (const auto& m : header.members) {
    if (m.first == "__metadata__") continue;
    const Json *dt = m.second.get("dtype"), *sh = m.second.get("shape"), *off = m.second.get("data_offsets");
    if (!dt || !sh || !off || off->items.size() != 2) throw EngineError(path + ": malformed entry for " + m.first);
    StoredTensor t;
    t.dtype = dt->text;
    // The header's numbers are the file's word, not ours: a negative or overflowing one must not become a
    // pointer outside the mapping.
    const uint64_t limit = (uint64_t)1 << 56;
    uint64_t n = 1;
    for (const Json& s : sh->items) {
      if (!s.is_int() || s.as_int() < 0) throw EngineError(path + ": " + m.first + " has a shape entry that is no size");
      const uint64_t d = (uint64_t)s.as_int();
      if (d != 0 && n > limit / d) throw EngineError(path + ": the shape of " + m.first + " is larger than any file");
      t.shape.push_back((int64_t)d);
      n *= d;
    }
    if (!off->items[0].is_int() || !off->items[1].is_int() || off->items[0].as_int() < 0 || off->items[1].as_int() < 0)
      throw EngineError(path + ": " + m.first + " has data offsets that are no sizes");
    const size_t b = (size_t)off->items[0].as_int(), e = (size_t)off->items[1].as_int();
    if (e < b || e > size - data_start) throw EngineError(path + ": " + m.first + " lies outside the file");
    auto it = stored_sizes().find(t.dtype);
    if (it != stored_sizes().end() && n * (uint64_t)it->second != (uint64_t)(e - b))
      throw EngineError(path + ": " + m.first + " has " + std::to_string(e - b) + " bytes, its shape needs " + std::to_string(n * (uint64_t)it->second));
    t.data = p + data_start + b;
    t.bytes = e - b;
    t.file = path;
    entries_[m.first] = std::move(t);
  }
}

}  // namespace vosti
