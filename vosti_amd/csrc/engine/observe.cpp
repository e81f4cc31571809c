#include "observe.h"

#include <sys/stat.h>
#include <unistd.h>

#include <climits>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "gpu.h"

namespace vosti {

namespace {
inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }

const uint32_t K256[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
    0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
    0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
    0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
    0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
    0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

void sha256_block(uint32_t h[8], const unsigned char* p) {
  uint32_t w[64];
  for (int i = 0; i < 16; ++i) w[i] = (uint32_t)p[4 * i] << 24 | (uint32_t)p[4 * i + 1] << 16 | (uint32_t)p[4 * i + 2] << 8 | p[4 * i + 3];
  for (int i = 16; i < 64; ++i) {
    const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
    const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
    w[i] = w[i - 16] + s0 + w[i - 7] + s1;
  }
  uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
  for (int i = 0; i < 64; ++i) {
    const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + K256[i] + w[i];
    const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
    hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
  }
  h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
}

std::string absolute_path(const std::string& p) {
  if (!p.empty() && p[0] == '/') return p;
  char buf[PATH_MAX];
  return getcwd(buf, sizeof buf) ? std::string(buf) + "/" + p : p;
}

void make_dirs(const std::string& path) {
  for (size_t i = 1; i <= path.size(); ++i)
    if (i == path.size() || path[i] == '/') (void)mkdir(path.substr(0, i).c_str(), 0777);
}
}  // namespace

std::string sha256_hex(const unsigned char* data, size_t len) {
  uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
  size_t done = 0;
  for (; done + 64 <= len; done += 64) sha256_block(h, data + done);
  unsigned char tail[128] = {0};
  const size_t rest = len - done;
  std::memcpy(tail, data + done, rest);
  tail[rest] = 0x80;
  const size_t blocks = rest + 9 <= 64 ? 1 : 2;
  const uint64_t bits = (uint64_t)len * 8;
  for (int i = 0; i < 8; ++i) tail[64 * blocks - 1 - i] = (unsigned char)(bits >> (8 * i));
  for (size_t b = 0; b < blocks; ++b) sha256_block(h, tail + 64 * b);
  char out[65];
  for (int i = 0; i < 8; ++i) std::snprintf(out + 8 * i, 9, "%08x", h[i]);
  return std::string(out, 64);
}

LogitsObserver::LogitsObserver() {
  if (const char* d = std::getenv("VOSTI_LOGITS_DIGEST"))
    if (*d) digest_path_ = d;
  if (const char* f = std::getenv("VOSTI_LOGITS_OBSERVER_DIR"))
    if (*f) folder_ = absolute_path(f);
}

void LogitsObserver::rows(const float* data, int64_t vocab, const std::vector<int>& row_indices, int64_t engine_step,
                          const std::string& source_dtype) {
  const int64_t call = calls_++;
  if (!folder_.empty()) make_dirs(folder_);
  const long pid = (long)getpid();
  for (size_t offset = 0; offset < row_indices.size(); ++offset) {
    const int index = row_indices[offset];
    const float* row = data + (int64_t)offset * vocab;
    const size_t bytes = (size_t)vocab * sizeof(float);
    const std::string sha = sha256_hex(reinterpret_cast<const unsigned char*>(row), bytes);
    if (!digest_path_.empty()) {
      std::FILE* f = std::fopen(digest_path_.c_str(), "a");
      if (!f) throw EngineError("cannot append to " + digest_path_);
      std::fprintf(f, "%d %s\n", index, sha.c_str());
      std::fclose(f);
    }
    if (folder_.empty()) continue;
    char name[96];
    std::snprintf(name, sizeof name, "row-%ld-%06lld-%04d.npy", pid, (long long)call, index);
    const std::string path = folder_ + "/" + name;
    std::FILE* f = std::fopen(path.c_str(), "wbx");
    if (!f) throw EngineError("cannot create " + path);
    // The .npy format, version 1.0: magic, a dictionary padded with spaces so that the data start at a multiple of 64.
    std::string dict = "{'descr': '<f4', 'fortran_order': False, 'shape': (" + std::to_string(vocab) + ",), }";
    while ((10 + dict.size() + 1) % 64) dict += ' ';
    dict += '\n';
    const unsigned char magic[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, (unsigned char)(dict.size() & 0xff), (unsigned char)(dict.size() >> 8)};
    std::fwrite(magic, 1, 10, f);
    std::fwrite(dict.data(), 1, dict.size(), f);
    std::fwrite(row, 1, bytes, f);
    std::fclose(f);
    // numpy's argmax: the first NaN if there is one, else the first largest value.
    bool finite = true;
    int64_t arg = 0;
    bool arg_nan = false;
    for (int64_t i = 0; i < vocab; ++i) {
      if (!std::isfinite(row[i])) finite = false;
      if (arg_nan) continue;
      if (std::isnan(row[i])) {
        arg = i;
        arg_nan = true;
      } else if (row[i] > row[arg]) {
        arg = i;
      }
    }
    std::string rec = "{\"argmax\":" + (vocab ? std::to_string(arg) : std::string("null")) + ",\"artifact\":\"" + name + "\",\"batch_index\":" +
                      std::to_string(index) + ",\"batch_size\":" + std::to_string(row_indices.size()) + ",\"byte_length\":" + std::to_string(bytes) +
                      ",\"call_sequence\":" + std::to_string(call) + ",\"engine_step\":" + std::to_string(engine_step) + ",\"finite\":" +
                      (finite ? "true" : "false") + ",\"numel\":" + std::to_string(vocab) + ",\"observed_dtype\":\"float32\"";
    const char* phase = std::getenv("VOSTI_LOGITS_OBSERVER_PHASE");
    if (phase && *phase) rec += std::string(",\"phase\":\"") + phase + "\"";
    rec += ",\"pid\":" + std::to_string(pid) + ",\"row_offset\":" + std::to_string(offset) + ",\"schema_version\":1,\"sha256\":\"" + sha +
           "\",\"shape\":[" + std::to_string(vocab) + "],\"source\":\"vosti_amd.engine\",\"source_dtype\":\"" + source_dtype + "\"}\n";
    const std::string index_path = folder_ + "/observer-" + std::to_string(pid) + ".jsonl";
    std::FILE* j = std::fopen(index_path.c_str(), "a");
    if (!j) throw EngineError("cannot append to " + index_path);
    std::fputs(rec.c_str(), j);
    std::fclose(j);
  }
}

}  // namespace vosti
