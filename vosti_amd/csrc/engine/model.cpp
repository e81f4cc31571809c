#include "model.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <set>
#include <sstream>

namespace vosti {

namespace {

void walk_parts(Part* p, std::vector<Part*>& out) {
  out.push_back(p);
  for (auto& c : p->children()) walk_parts(c.second, out);
}

struct Param {
  std::string path;
  Part* owner;
  ParamDecl decl;
};
void walk_params(Part* p, const std::string& prefix, std::vector<Param>& out) {
  for (const ParamDecl& d : p->params()) out.push_back({prefix + d.name, p, d});
  for (auto& c : p->children()) walk_params(c.second, prefix + c.first + ".", out);
}

std::string shape_text(const std::vector<int64_t>& s) {
  std::ostringstream o;
  o << "[";
  for (size_t i = 0; i < s.size(); ++i) o << (i ? ", " : "") << s[i];
  o << "]";
  return o.str();
}

std::string join(const std::vector<std::string>& v, const char* sep) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? sep : "") + v[i];
  return s;
}

bool is_float_type(const std::string& t) { return t == "F64" || t == "F32" || t == "F16" || t == "BF16"; }
bool is_int_type(const std::string& t) { return t == "I64" || t == "I32" || t == "I16" || t == "I8" || t == "U8" || t == "BOOL"; }

float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do { ++e; man <<= 1; } while (!(man & 0x400));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FF) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

uint16_t float_to_bf16(float f) {      // round to nearest, ties to even
  uint32_t b;
  std::memcpy(&b, &f, 4);
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40);   // NaN stays NaN
  b += 0x7FFFu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}

float load_float(const unsigned char* p, const std::string& t, int64_t i) {
  if (t == "F32") { float f; std::memcpy(&f, p + 4 * i, 4); return f; }
  if (t == "BF16") { uint16_t h; std::memcpy(&h, p + 2 * i, 2); uint32_t b = (uint32_t)h << 16; float f; std::memcpy(&f, &b, 4); return f; }
  if (t == "F16") { uint16_t h; std::memcpy(&h, p + 2 * i, 2); return half_to_float(h); }
  double d; std::memcpy(&d, p + 8 * i, 8); return (float)d;   // F64
}

int32_t load_int(const unsigned char* p, const std::string& t, int64_t i) {
  if (t == "I64") { int64_t v; std::memcpy(&v, p + 8 * i, 8); return (int32_t)v; }
  if (t == "I32") { int32_t v; std::memcpy(&v, p + 4 * i, 4); return v; }
  if (t == "I16") { int16_t v; std::memcpy(&v, p + 2 * i, 2); return v; }
  if (t == "I8") return (int8_t)p[i];
  return p[i];   // U8, BOOL
}

}  // namespace

Tensor upload_tensor(const StoredTensor& st, DType compute, bool keep_f32) {
  Tensor out;
  out.shape = st.shape;
  const bool flt = is_float_type(st.dtype);
  if (!flt && !is_int_type(st.dtype)) throw WeightError("unsupported stored type " + st.dtype);
  out.dtype = flt ? ((keep_f32 && st.dtype == "F32") ? DType::F32 : compute) : DType::I32;
  out.owner = std::make_shared<DeviceBuffer>(out.bytes());
  out.data = out.owner->data();
  const int64_t n = out.numel();
  const bool same = (out.dtype == DType::F32 && st.dtype == "F32") || (out.dtype == DType::BF16 && st.dtype == "BF16") ||
                    (out.dtype == DType::I32 && st.dtype == "I32");
  if (same) {
    hip_check(hipMemcpy(out.data, st.data, out.bytes(), hipMemcpyHostToDevice), "weight upload");
    return out;
  }
  // Converted on the host in pieces, so that a large tensor never has a second whole copy.
  const int64_t piece = 1 << 22;
  std::vector<uint32_t> staging((size_t)std::min(n, piece));
  for (int64_t at = 0; at < n; at += piece) {
    const int64_t m = std::min(piece, n - at);
    if (out.dtype == DType::F32) {
      float* d = reinterpret_cast<float*>(staging.data());
      for (int64_t i = 0; i < m; ++i) d[i] = load_float(st.data, st.dtype, at + i);
    } else if (out.dtype == DType::BF16) {
      uint16_t* d = reinterpret_cast<uint16_t*>(staging.data());
      for (int64_t i = 0; i < m; ++i) d[i] = float_to_bf16(load_float(st.data, st.dtype, at + i));
    } else {
      int32_t* d = reinterpret_cast<int32_t*>(staging.data());
      for (int64_t i = 0; i < m; ++i) d[i] = load_int(st.data, st.dtype, at + i);
    }
    hip_check(hipMemcpy(static_cast<char*>(out.data) + (size_t)at * dtype_bytes(out.dtype), staging.data(),
                        (size_t)m * dtype_bytes(out.dtype), hipMemcpyHostToDevice),
              "weight upload");
  }
  return out;
}

DecoderModel::DecoderModel(ModelSpec spec, Kernels& kernels) : spec_(std::move(spec)), kernels_(kernels) {
  spec_.validate();
  embedding_ = build_part<Embedding>("embedding", *spec_.embedding, kernels_);
  for (const LayerSpec& l : spec_.layers) layers_.push_back(build_block(l, kernels_));
  final_norm_ = build_part<Norm>("norm", *spec_.final_norm, kernels_);
  head_ = build_part<Head>("head", *spec_.head, kernels_);
}

std::vector<Part*> DecoderModel::parts() {
  std::vector<Part*> out;
  walk_parts(embedding_.get(), out);
  for (auto& l : layers_) walk_parts(l.get(), out);
  walk_parts(final_norm_.get(), out);
  walk_parts(head_.get(), out);
  return out;
}

std::map<std::string, ExpectedTensor> DecoderModel::expected_tensors() {
  std::map<std::string, ExpectedTensor> out;
  auto add = [&](const std::map<std::string, std::string>& names, Part* root, const std::string& prefix) {
    std::vector<Param> params;
    walk_params(root, prefix, params);
    for (const Param& p : params) {
      auto it = names.find(p.path);
      if (it == names.end()) throw ConfigError("the configuration gives no tensor name for parameter '" + p.path + "'");
      auto ins = out.emplace(it->second, ExpectedTensor{p.decl, {}});
      ExpectedTensor& e = ins.first->second;
      // Parameters that the description gives the same tensor name share one tensor.
      if (e.decl.shape != p.decl.shape)
        throw ConfigError("tensor '" + it->second + "' is shared by parameters of different shapes: " + shape_text(e.decl.shape) +
                          " and " + shape_text(p.decl.shape) + " ('" + p.path + "')");
      e.owners.emplace_back(p.owner, p.decl.name);
    }
  };
  add(spec_.names, embedding_.get(), "embedding.");
  add(spec_.names, final_norm_.get(), "final_norm.");
  add(spec_.names, head_.get(), "head.");
  for (size_t i = 0; i < layers_.size(); ++i) add(spec_.layers[i].names, layers_[i].get(), "");
  return out;
}

void DecoderModel::load_weights(const Checkpoint& ckpt) {
  const auto expected = expected_tensors();
  const auto& stored = ckpt.entries();
  std::vector<std::string> missing, unexpected, wrong;
  for (const auto& e : expected) {
    auto it = stored.find(e.first);
    if (it == stored.end()) {
      missing.push_back(e.first);
    } else if (it->second.shape != e.second.decl.shape) {
      wrong.push_back(e.first + ": file has " + shape_text(it->second.shape) + ", model needs " + shape_text(e.second.decl.shape));
    } else if (!is_float_type(it->second.dtype) && !is_int_type(it->second.dtype)) {
      wrong.push_back(e.first + ": unsupported stored type " + it->second.dtype);
    }
  }
  const std::set<std::string> ignorable(spec_.ignored_names.begin(), spec_.ignored_names.end());
  for (const auto& s : stored)
    if (!expected.count(s.first) && !ignorable.count(s.first)) unexpected.push_back(s.first);
  if (!missing.empty() || !unexpected.empty() || !wrong.empty()) {
    std::string msg = "weights in " + ckpt.dir() + " do not fit the model:";
    if (!missing.empty()) msg += "\n  missing (" + std::to_string(missing.size()) + "): " + join(missing, ", ");
    if (!unexpected.empty()) msg += "\n  unexpected (" + std::to_string(unexpected.size()) + "): " + join(unexpected, ", ");
    if (!wrong.empty()) msg += "\n  wrong shape or type (" + std::to_string(wrong.size()) + "): " + join(wrong, "; ");
    throw WeightError(msg);
  }
  // Part by part, so that a part that keeps its weights in another arrangement (projections stacked for
  // one launch) frees the pieces before the next part loads.  A tensor with several owners is uploaded once.
  std::map<Part*, std::vector<std::pair<std::string, std::string>>> wanted;     // part -> (local, tensor name)
  std::map<std::string, int> owners_left;
  for (const auto& e : expected)
    for (const auto& o : e.second.owners) {
      wanted[o.first].emplace_back(o.second, e.first);
      ++owners_left[e.first];
    }
  std::map<std::string, Tensor> live;
  for (Part* part : parts()) {
    auto w = wanted.find(part);
    if (w == wanted.end()) continue;
    std::map<std::string, Tensor> given;
    for (const auto& ln : w->second) {
      auto it = live.find(ln.second);
      if (it == live.end()) it = live.emplace(ln.second, upload_tensor(stored.at(ln.second), kernels_.dtype(), expected.at(ln.second).decl.keep_f32)).first;
      given[ln.first] = it->second;
      if (--owners_left[ln.second] == 0) live.erase(it);
    }
    part->load(given);
  }
  loaded_ = true;
}

// BLAKE2b (RFC 7693) with an 8-byte digest and no key, for inputs of any length.
static uint64_t blake2b_64(const unsigned char* in, size_t len) {
  static const uint64_t IV[8] = {0x6a09e667f3bcc908ull, 0xbb67ae8584caa73bull, 0x3c6ef372fe94f82bull, 0xa54ff53a5f1d36f1ull,
                                 0x510e527fade682d1ull, 0x9b05688c2b3e6c1full, 0x1f83d9abfb41bd6bull, 0x5be0cd19137e2179ull};
  static const unsigned char SIGMA[12][16] = {
      {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3},
      {11, 8, 12, 0, 5, 2, 15, 13, 10, 14, 3, 6, 7, 1, 9, 4}, {7, 9, 3, 1, 13, 12, 11, 14, 2, 6, 5, 10, 4, 0, 15, 8},
      {9, 0, 5, 7, 2, 4, 10, 15, 14, 1, 11, 12, 6, 8, 3, 13}, {2, 12, 6, 10, 0, 11, 8, 3, 4, 13, 7, 5, 15, 14, 1, 9},
      {12, 5, 1, 15, 14, 13, 4, 10, 0, 7, 6, 3, 9, 2, 8, 11}, {13, 11, 7, 14, 12, 1, 3, 9, 5, 0, 15, 4, 8, 6, 2, 10},
      {6, 15, 14, 9, 11, 3, 0, 8, 12, 2, 13, 7, 1, 4, 10, 5}, {10, 2, 8, 4, 7, 6, 1, 5, 15, 11, 9, 14, 3, 12, 13, 0},
      {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3}};
  auto rotr = [](uint64_t x, int n) { return (x >> n) | (x << (64 - n)); };
  uint64_t h[8];
  for (int i = 0; i < 8; ++i) h[i] = IV[i];
  h[0] ^= 0x01010000ull ^ 8;            // digest length 8, no key, fanout 1, depth 1
  size_t done = 0;
  for (;;) {
    const bool last = len - done <= 128;
    const size_t n = last ? len - done : 128;
    unsigned char block[128] = {0};
    std::memcpy(block, in + done, n);
    done += n;
    uint64_t m[16], v[16];
    for (int i = 0; i < 16; ++i) {
      m[i] = 0;
      for (int b = 7; b >= 0; --b) m[i] = (m[i] << 8) | block[8 * i + b];
    }
    for (int i = 0; i < 8; ++i) { v[i] = h[i]; v[i + 8] = IV[i]; }
    v[12] ^= (uint64_t)done;            // the bytes so far (below 2^64)
    if (last) v[14] = ~v[14];
    for (int r = 0; r < 12; ++r) {
      const unsigned char* s = SIGMA[r];
      auto G = [&](int a, int b, int c, int d, uint64_t x, uint64_t y) {
        v[a] = v[a] + v[b] + x; v[d] = rotr(v[d] ^ v[a], 32);
        v[c] = v[c] + v[d];     v[b] = rotr(v[b] ^ v[c], 24);
        v[a] = v[a] + v[b] + y; v[d] = rotr(v[d] ^ v[a], 16);
        v[c] = v[c] + v[d];     v[b] = rotr(v[b] ^ v[c], 63);
      };
      G(0, 4, 8, 12, m[s[0]], m[s[1]]);   G(1, 5, 9, 13, m[s[2]], m[s[3]]);
      G(2, 6, 10, 14, m[s[4]], m[s[5]]);  G(3, 7, 11, 15, m[s[6]], m[s[7]]);
      G(0, 5, 10, 15, m[s[8]], m[s[9]]);  G(1, 6, 11, 12, m[s[10]], m[s[11]]);
      G(2, 7, 8, 13, m[s[12]], m[s[13]]); G(3, 4, 9, 14, m[s[14]], m[s[15]]);
    }
    for (int i = 0; i < 8; ++i) h[i] ^= v[i] ^ v[i + 8];
    if (last) break;
  }
  return h[0];      // the digest's 8 bytes are h[0] in little-endian order
}

uint64_t tensor_seed(uint64_t seed, const std::string& name) {
  const std::string text = std::to_string(seed) + ":" + name;
  return blake2b_64(reinterpret_cast<const unsigned char*>(text.data()), text.size());
}

void DecoderModel::random_weights(uint64_t seed) {
  const auto expected = expected_tensors();
  std::map<Part*, std::map<std::string, Tensor>> given;
  for (const auto& e : expected) {
    const ParamDecl& d = e.second.decl;
    Tensor t;
    t.dtype = kernels_.dtype();
    t.shape = d.shape;
    t.owner = std::make_shared<DeviceBuffer>(t.bytes());
    t.data = t.owner->data();
    // As the kernel takes them: a normal value is a sum of four 16-bit uniforms times std * sqrt(3) / 65536.
    const float p0 = d.uniform ? (float)d.p0 : (float)(d.p0 * std::sqrt(3.0) / 65536.0);
    const float p1 = d.uniform ? (float)(d.p1 - d.p0) : 0.f;
    kernels_.fill_random(t, tensor_seed(seed, e.first), d.uniform ? 1 : 0, p0, p1);
    for (const auto& o : e.second.owners) given[o.first][o.second] = t;
  }
  hip_check(hipStreamSynchronize(kernels_.stream), "random weights");
  for (Part* part : parts()) {
    auto it = given.find(part);
    if (it != given.end()) part->load(it->second);
  }
  loaded_ = true;
}

bool DecoderModel::replayable() {
  for (Part* p : parts())
    if (!p->replayable()) return false;
  return true;
}

std::vector<CacheNeed> DecoderModel::cache_needs() {
  std::vector<CacheNeed> out;
  for (const ScheduleEntry& e : spec_.schedule) out.push_back(e.cache_from >= 0 ? CacheNeed{} : layers_[e.layer]->mixer().cache_need());
  return out;
}

Tensor DecoderModel::forward(const Tensor& ids, StepContext& ctx, std::vector<CacheEntry>& caches, const Tensor& want_rows) {
  if (!loaded_) throw EngineError("the model has no weights yet");
  if (caches.size() != spec_.schedule.size()) throw EngineError("one cache entry per schedule entry is needed");
  Tensor hidden = embedding_->forward(ids), residual;
  for (size_t i = 0; i < spec_.schedule.size(); ++i) {
    auto hr = layers_[spec_.schedule[i].layer]->forward(hidden, residual, ctx, caches[i]);
    hidden = hr.first;
    residual = hr.second;
  }
  if (want_rows.numel() == 0) return kernels_.empty({0, spec_.vocab_size});
  hidden = kernels_.gather_rows(hidden, want_rows);
  Tensor normed;
  if (residual.data == nullptr) {
    normed = final_norm_->forward(hidden);            // a model without layers
  } else {
    Tensor r = kernels_.gather_rows(residual, want_rows);
    normed = final_norm_->forward_add(hidden, r);
  }
  return head_->forward(normed);
}

}  // namespace vosti
