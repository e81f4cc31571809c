// What the engine can leave behind for comparisons between runs: a digest of every sampled logits row, or the
// rows themselves.
//
// The reference's determinism harness reads two artefacts at the sampling boundary
// (python/vosti_kernels/kernels.py:1020-1033, scripts/determinism_tests/logits_observer.py):
//
//   VOSTI_LOGITS_DIGEST=<file>          one line "<row index in the step> <sha256>" per sampled row, the hash taken
//                                       over the row as 32-bit floats;
//   VOSTI_LOGITS_OBSERVER_DIR=<folder>  every sampled row as a float32 .npy file row-<pid>-<call>-<row index>.npy
//                                       plus one JSON line per row in observer-<pid>.jsonl with its hash, shape,
//                                       argmax, the step, and the phase that VOSTI_LOGITS_OBSERVER_PHASE names.
//
// Both cost a device-to-host copy of the rows per step; they are instrumentation, off by default.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace vosti {

// SHA-256 (FIPS 180-4) of a byte string, as 64 hexadecimal digits.
std::string sha256_hex(const unsigned char* data, size_t len);

class LogitsObserver {
 public:
  LogitsObserver();       // reads VOSTI_LOGITS_DIGEST and VOSTI_LOGITS_OBSERVER_DIR
  bool active() const { return !digest_path_.empty() || !folder_.empty(); }
  // data: float32 [n, vocab], one row per sampled row of the step; row_indices: their places in the step.
  void rows(const float* data, int64_t vocab, const std::vector<int>& row_indices, int64_t engine_step, const std::string& source_dtype);

 private:
  std::string digest_path_, folder_;
  int64_t calls_ = 0;
};

}  // namespace vosti
