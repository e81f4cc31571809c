// Device memory, tensors and the kernel library as the native engine sees them.
//
// The engine is host code: it is compiled by the host compiler against the HIP runtime API and reaches
// the gfx950 kernels through the C entry points of libvosti_bf16.so or libvosti_f32.so, whichever the
// chosen precision names (both export the same names, so the library is picked at run time with dlopen).
// Every wrapper checks on the host that operand shapes and sizes are what the kernel's grid assumes
// before it launches: a kernel that reads out of bounds can take the GPU down.
#pragma once
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace vosti {

struct EngineError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

void hip_check(hipError_t e, const char* what);

enum class DType { BF16, F32, I32 };
inline int dtype_bytes(DType t) { return t == DType::BF16 ? 2 : 4; }
const char* dtype_name(DType t);

// Device memory that frees itself.
class DeviceBuffer {
 public:
  explicit DeviceBuffer(size_t bytes);
  ~DeviceBuffer();
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  void* data() const { return ptr_; }
  size_t bytes() const { return bytes_; }

 private:
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

// A contiguous row-major tensor on the GPU.  `owner` keeps weights alive; activations live in the step's
// arena and have none.
struct Tensor {
  void* data = nullptr;
  DType dtype = DType::BF16;
  std::vector<int64_t> shape;
  std::shared_ptr<DeviceBuffer> owner;

  int64_t numel() const {
    int64_t n = 1;
    for (int64_t s : shape) n *= s;
    return n;
  }
  int64_t dim(int i) const { return shape.at(i < 0 ? shape.size() + i : i); }
  size_t bytes() const { return (size_t)numel() * dtype_bytes(dtype); }
  bool defined() const { return data != nullptr || numel() == 0; }
  Tensor view(std::vector<int64_t> new_shape) const;         // same elements, another shape
  Tensor rows(int64_t first, int64_t count) const;           // rows [first, first + count) of the outer axis
  std::string describe() const;
};

// Memory for one step's activations: handed out front to back, all given back at once when the step is
// over.  Blocks are only ever appended, so the same sequence of requests gets the same addresses in
// every step, which a recorded graph relies on.  Nothing is allocated while a stream is capturing.
class Arena {
 public:
  void* take(size_t bytes);
  void reset() { block_ = 0; offset_ = 0; }
  // Where the next block would be handed out.  A recorded step's results lie below the mark taken at the end
  // of its recording; after a replay the cursor goes back there, so that what is taken next (a copy of the
  // logits, say) cannot lie on top of them.
  struct Mark {
    size_t block = 0, offset = 0;
  };
  Mark mark() const { return {block_, offset_}; }
  void restore(const Mark& m) { block_ = m.block; offset_ = m.offset; }
  void forbid_growth(bool on) { frozen_ = on; }
  size_t capacity() const;

 private:
  std::vector<std::unique_ptr<DeviceBuffer>> blocks_;
  size_t block_ = 0, offset_ = 0;
  bool frozen_ = false;
};

// The kernel library of one precision.
class Kernels {
 public:
  // `lib_dir`: the folder that holds libvosti_<name>.so; name is "bf16" or "f32".
  Kernels(const std::string& lib_dir, const std::string& name);
  ~Kernels();
  Kernels(const Kernels&) = delete;

  DType dtype() const { return dtype_; }
  const std::string& name() const { return name_; }
  hipStream_t stream = nullptr;      // every launch goes here
  Arena arena;                       // where results are put

  Tensor empty(std::vector<int64_t> shape) { return empty(std::move(shape), dtype_); }
  Tensor empty(std::vector<int64_t> shape, DType t);

  Tensor embedding(const Tensor& table, const Tensor& ids);
  Tensor rmsnorm(const Tensor& x, const Tensor& w, float eps);
  Tensor add_rmsnorm(const Tensor& x, Tensor& residual, const Tensor& w, float eps);
  Tensor swiglu(const Tensor& gate_up);
  Tensor gather_rows(const Tensor& x, const Tensor& rows);
  Tensor to_f32(const Tensor& x);
  // Columns [first, first + count) of a [rows, width] tensor as a tensor of their own.
  Tensor columns(const Tensor& x, int64_t first, int64_t count);
  // dst[:, dst_first : dst_first + count] = src[:, src_first : src_first + count], rows alike.
  void copy_columns(Tensor& dst, int64_t dst_first, const Tensor& src, int64_t src_first, int64_t count);
  void rope_tables(Tensor& cos, Tensor& sin, const Tensor& inv_freq);
  // Counter-based random fill: element i is a function of (seed, i); kind 0: a sum of four 16-bit uniforms
  // scaled by p0, kind 1: p0 + u * p1.
  void fill_random(Tensor& out, uint64_t seed, int kind, float p0, float p1);
  // act @ w^T, w [out, in].  workspace: float32 scratch; with enough of it (gemm_workspace_floats) some sizes
  // take a faster route to the same bits.
  Tensor gemm(const Tensor& act, const Tensor& w, const Tensor* workspace = nullptr);
  Tensor gemm_swiglu(const Tensor& act, const Tensor& w_gate_up, const Tensor* workspace = nullptr);
  // float32 elements of workspace with which gemm / gemm_swiglu take the route through chunk sums for these
  // sizes, or 0 where that route does not exist or is the slower one.
  int64_t gemm_workspace_floats(int64_t M, int64_t rows, int64_t K, bool swiglu = false) const;
  // Head norm, rotation and cache store of [T, (nq + 2 nkv) d] rows; returns q [T, nq, d] (nq > 0).
  Tensor qkv_post(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache, int page_size,
                  const Tensor* q_w, const Tensor* k_w, float eps, const Tensor* cos, const Tensor* sin,
                  const Tensor* positions, const Tensor* slots);
  int64_t attn_scratch_floats(int items, int nq, int d, int nseg) const;
  void paged_attention(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
                       const Tensor& block_table, const Tensor& cu_q, const Tensor& k_len, const Tensor& items, int mode,
                       float scale, int window, int max_k_len, int nseg, const Tensor* scratch);
  // Token ids per row: the largest logit, or a draw at temps[r] > 0 with the uniform number unis[r].
  void sample(Tensor& out, const Tensor& logits, const Tensor* temps, const Tensor* unis, Tensor& scratch);
  int sample_scratch_words(int rows) const;
  int segment_keys() const { return segment_keys_; }
  int item_rows() const { return item_rows_; }

 private:
  void call(int rc) const;
  void expect(const Tensor& t, const char* what, DType dtype, std::vector<int64_t> shape = {}) const;
  int norm_weight(const Tensor& w, const char* what, int64_t n) const;   // 1 if the weight is float32
  bool split(Tensor& out, const Tensor& act, const Tensor& w, bool swiglu, const Tensor* workspace);

  std::string name_;
  DType dtype_;
  void* handle_ = nullptr;
  int segment_keys_ = 0, item_rows_ = 0;
  struct Fn;
  std::unique_ptr<Fn> fn_;
};

}  // namespace vosti
