#include "gpu.h"

#include <dlfcn.h>

#include <sstream>

namespace vosti {

void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw EngineError(std::string(what) + ": " + hipGetErrorString(e));
}

const char* dtype_name(DType t) { return t == DType::BF16 ? "bfloat16" : (t == DType::F32 ? "float32" : "int32"); }

DeviceBuffer::DeviceBuffer(size_t bytes) : bytes_(bytes) {
  hip_check(hipMalloc(&ptr_, bytes ? bytes : 16), "device allocation");
}
DeviceBuffer::~DeviceBuffer() {
  if (ptr_) (void)hipFree(ptr_);
}

Tensor Tensor::view(std::vector<int64_t> new_shape) const {
  Tensor t = *this;
  t.shape = std::move(new_shape);
  if (t.numel() != numel()) throw EngineError("view of " + describe() + " with another number of elements");
  return t;
}

Tensor Tensor::rows(int64_t first, int64_t count) const {
  if (shape.empty() || first < 0 || count < 0 || first + count > shape[0]) throw EngineError("rows outside " + describe());
  Tensor t = *this;
  const int64_t row = shape[0] ? numel() / shape[0] : 0;
  t.data = static_cast<char*>(data) + (size_t)(first * row) * dtype_bytes(dtype);
  t.shape[0] = count;
  return t;
}

std::string Tensor::describe() const {
  std::ostringstream s;
  s << dtype_name(dtype) << "[";
  for (size_t i = 0; i < shape.size(); ++i) s << (i ? ", " : "") << shape[i];
  s << "]";
  return s.str();
}

// ------------------------------------------------------------------------------------------ arena
void* Arena::take(size_t bytes) {
  bytes = (bytes + 255) & ~(size_t)255;
  if (bytes == 0) bytes = 256;
  while (block_ < blocks_.size()) {
    if (offset_ + bytes <= blocks_[block_]->bytes()) {
      void* p = static_cast<char*>(blocks_[block_]->data()) + offset_;
      offset_ += bytes;
      return p;
    }
    ++block_;
    offset_ = 0;
  }
  if (frozen_) throw EngineError("a step that is being recorded asks for more activation memory than the step before it");
  const size_t min_block = (size_t)64 << 20;
  blocks_.push_back(std::make_unique<DeviceBuffer>(bytes > min_block ? bytes : min_block));
  offset_ = bytes;
  return blocks_.back()->data();
}

size_t Arena::capacity() const {
  size_t n = 0;
  for (const auto& b : blocks_) n += b->bytes();
  return n;
}

// ---------------------------------------------------------------------------------------- kernels
using P = void*;
using CP = const void*;
struct Kernels::Fn {
  const char* (*last_error)();
  int (*abi_version)();
  int (*elem_bytes)();
  int (*embedding)(P, CP, CP, int, int, int, hipStream_t);
  int (*rmsnorm)(P, CP, CP, int, int, int, int, int64_t, int64_t, float, hipStream_t);
  int (*add_rmsnorm)(P, P, CP, CP, int, int, int, float, hipStream_t);
  int (*swiglu)(P, CP, int, int, hipStream_t);
  int (*gather_rows)(P, CP, CP, int, int, hipStream_t);
  int (*cast_to_f32)(P, CP, int64_t, hipStream_t);
  int (*rope_tables)(P, P, CP, int, int, hipStream_t);
  int (*fill_random)(P, int64_t, uint64_t, int, float, float, hipStream_t);
  int (*gemm)(P, CP, CP, int, int, int, int64_t, int64_t, int, hipStream_t);
  int (*gemm_swiglu)(P, CP, CP, int, int, int, int64_t, int64_t, hipStream_t);
  int (*gemm_swiglu_supported)(int, int, int);
  int (*gemm_split)(P, CP, CP, int, int, int, int64_t, int64_t, int, P, int64_t, hipStream_t);
  int64_t (*gemm_split_floats)(int, int, int, int);
  int (*gemm_split_preferred)(int, int, int, int);
  int (*qkv_post)(CP, int64_t, P, P, P, CP, CP, int, CP, CP, int, CP, CP, int, int, int, int, int, float, hipStream_t);
  int (*paged_attention)(P, CP, CP, CP, CP, int, CP, CP, CP, int, int, int, P, int, int, int, int, int, int, float, hipStream_t);
  int (*sample)(P, CP, CP, CP, P, int, int, int64_t, hipStream_t);
  int (*sample_scratch_words)(int);
  int64_t (*attn_scratch_floats)(int, int, int, int);
  int (*attn_segment_keys)();
  int (*attn_item_rows)();
};

static constexpr int KERNEL_ABI = 13;

Kernels::Kernels(const std::string& lib_dir, const std::string& name) : name_(name), fn_(new Fn) {
  if (name == "bf16") dtype_ = DType::BF16;
  else if (name == "f32") dtype_ = DType::F32;
  else throw EngineError("unsupported element type '" + name + "'; use bf16 or f32");
  const std::string path = lib_dir + "/libvosti_" + name + ".so";
  handle_ = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!handle_) throw EngineError("the kernel library is missing: " + std::string(dlerror()) + " (build it: python -m vosti_amd.kernels.build)");
  auto sym = [&](const char* s) {
    void* p = dlsym(handle_, s);
    if (!p) throw EngineError(path + " lacks " + s + "; rebuild it");
    return p;
  };
#define VK(field, symbol) fn_->field = reinterpret_cast<decltype(fn_->field)>(sym(symbol))
  VK(last_error, "vk_last_error"); VK(abi_version, "vk_abi_version"); VK(elem_bytes, "vk_elem_bytes");
  if (fn_->abi_version() != KERNEL_ABI)
    throw EngineError(path + " has ABI " + std::to_string(fn_->abi_version()) + ", expected " + std::to_string(KERNEL_ABI) + "; rebuild it");
  if (fn_->elem_bytes() != dtype_bytes(dtype_)) throw EngineError(path + " was built for another element type");
  VK(embedding, "vk_embedding"); VK(rmsnorm, "vk_rmsnorm"); VK(add_rmsnorm, "vk_add_rmsnorm"); VK(swiglu, "vk_swiglu");
  VK(gather_rows, "vk_gather_rows"); VK(cast_to_f32, "vk_cast_to_f32"); VK(rope_tables, "vk_rope_tables"); VK(fill_random, "vk_fill_random");
  VK(gemm, "vk_gemm"); VK(gemm_swiglu, "vk_gemm_swiglu"); VK(gemm_swiglu_supported, "vk_gemm_swiglu_supported");
  VK(gemm_split, "vk_gemm_split"); VK(gemm_split_floats, "vk_gemm_split_floats"); VK(gemm_split_preferred, "vk_gemm_split_preferred");
  VK(qkv_post, "vk_qkv_post"); VK(paged_attention, "vk_paged_attention"); VK(sample, "vk_sample");
  VK(sample_scratch_words, "vk_sample_scratch_words"); VK(attn_scratch_floats, "vk_attn_scratch_floats");
  VK(attn_segment_keys, "vk_attn_segment_keys"); VK(attn_item_rows, "vk_attn_item_rows");
#undef VK
  segment_keys_ = fn_->attn_segment_keys();
  item_rows_ = fn_->attn_item_rows();
  hip_check(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "stream creation");
}

Kernels::~Kernels() {
  if (stream) (void)hipStreamDestroy(stream);
  // The library stays loaded: its code objects are registered with the runtime.
}

void Kernels::call(int rc) const {
  if (rc != 0) throw EngineError(fn_->last_error());
}

void Kernels::expect(const Tensor& t, const char* what, DType dtype, std::vector<int64_t> shape) const {
  if (t.data == nullptr && t.numel() != 0) throw EngineError(std::string(what) + " has no memory");
  if (t.dtype != dtype) throw EngineError(std::string(what) + " has type " + dtype_name(t.dtype) + ", expected " + dtype_name(dtype));
  if (!shape.empty() && t.shape != shape) {
    Tensor want;
    want.dtype = dtype;
    want.shape = shape;
    throw EngineError(std::string(what) + " is " + t.describe() + ", expected " + want.describe());
  }
}

int Kernels::norm_weight(const Tensor& w, const char* what, int64_t n) const {
  // A norm weight may be stored as elements or as float.
  if (w.dtype == DType::F32) {
    expect(w, what, DType::F32, {n});
    return 1;
  }
  expect(w, what, dtype_, {n});
  return 0;
}

Tensor Kernels::empty(std::vector<int64_t> shape, DType t) {
  Tensor out;
  out.dtype = t;
  out.shape = std::move(shape);
  for (int64_t s : out.shape)
    if (s < 0) throw EngineError("a tensor with a negative size");
  out.data = arena.take(out.bytes());
  return out;
}

Tensor Kernels::embedding(const Tensor& table, const Tensor& ids) {
  expect(table, "embedding table", dtype_);
  if (table.shape.size() != 2) throw EngineError("embedding table is " + table.describe());
  const int64_t V = table.dim(0), H = table.dim(1), T = ids.numel();
  expect(ids, "ids", DType::I32, {T});
  Tensor out = empty({T, H});
  call(fn_->embedding(out.data, table.data, ids.data, (int)T, (int)H, (int)V, stream));
  return out;
}

Tensor Kernels::rmsnorm(const Tensor& x, const Tensor& w, float eps) {
  expect(x, "norm input", dtype_);
  const int64_t H = x.dim(-1), rows = H ? x.numel() / H : 0;
  const int wf = norm_weight(w, "norm weight", H);
  Tensor out = empty(x.shape);
  call(fn_->rmsnorm(out.data, x.data, w.data, wf, (int)rows, (int)H, 1, H, H, eps, stream));
  return out;
}

Tensor Kernels::add_rmsnorm(const Tensor& x, Tensor& residual, const Tensor& w, float eps) {
  expect(x, "norm input", dtype_);
  if (x.shape.size() != 2) throw EngineError("norm input is " + x.describe());
  expect(residual, "residual", dtype_, x.shape);
  const int wf = norm_weight(w, "norm weight", x.dim(1));
  Tensor out = empty(x.shape);
  call(fn_->add_rmsnorm(out.data, residual.data, x.data, w.data, wf, (int)x.dim(0), (int)x.dim(1), eps, stream));
  return out;
}

Tensor Kernels::swiglu(const Tensor& gate_up) {
  expect(gate_up, "gate/up tensor", dtype_);
  if (gate_up.shape.size() != 2 || gate_up.dim(1) % 2) throw EngineError("swiglu: gate/up tensor is " + gate_up.describe());
  const int64_t T = gate_up.dim(0), I = gate_up.dim(1) / 2;
  Tensor out = empty({T, I});
  call(fn_->swiglu(out.data, gate_up.data, (int)T, (int)I, stream));
  return out;
}

Tensor Kernels::gather_rows(const Tensor& x, const Tensor& rows) {
  expect(x, "rows' source", dtype_);
  if (x.shape.size() != 2) throw EngineError("gather_rows: source is " + x.describe());
  const int64_t R = rows.numel();
  expect(rows, "row numbers", DType::I32, {R});
  Tensor out = empty({R, x.dim(1)});
  call(fn_->gather_rows(out.data, x.data, rows.data, (int)R, (int)x.dim(1), stream));
  return out;
}

Tensor Kernels::to_f32(const Tensor& x) {
  expect(x, "cast input", dtype_);
  Tensor out = empty(x.shape, DType::F32);
  call(fn_->cast_to_f32(out.data, x.data, x.numel(), stream));
  return out;
}

void Kernels::copy_columns(Tensor& dst, int64_t dst_first, const Tensor& src, int64_t src_first, int64_t count) {
  if (src.shape.size() != 2 || dst.shape.size() != 2 || src.dim(0) != dst.dim(0) || src.dtype != dst.dtype || count < 0 || src_first < 0 ||
      dst_first < 0 || src_first + count > src.dim(1) || dst_first + count > dst.dim(1))
    throw EngineError("copy_columns: " + std::to_string(count) + " columns from " + std::to_string(src_first) + " of " + src.describe() +
                      " to " + std::to_string(dst_first) + " of " + dst.describe());
  if (count == 0 || src.dim(0) == 0) return;
  const size_t e = (size_t)dtype_bytes(src.dtype);
  hip_check(hipMemcpy2DAsync(static_cast<char*>(dst.data) + (size_t)dst_first * e, (size_t)dst.dim(1) * e,
                             static_cast<const char*>(src.data) + (size_t)src_first * e, (size_t)src.dim(1) * e, (size_t)count * e,
                             (size_t)src.dim(0), hipMemcpyDeviceToDevice, stream),
            "copying columns");
}

Tensor Kernels::columns(const Tensor& x, int64_t first, int64_t count) {
  if (x.shape.size() != 2) throw EngineError("columns of " + x.describe());
  Tensor out = empty({x.dim(0), count}, x.dtype);
  copy_columns(out, 0, x, first, count);
  return out;
}

void Kernels::rope_tables(Tensor& cos, Tensor& sin, const Tensor& inv_freq) {
  const int64_t half = inv_freq.numel();
  expect(inv_freq, "inverse frequencies", DType::F32, {half});
  expect(cos, "cosine table", dtype_);
  if (cos.shape.size() != 2 || cos.dim(1) != half) throw EngineError("cosine table is " + cos.describe());
  expect(sin, "sine table", dtype_, cos.shape);
  call(fn_->rope_tables(cos.data, sin.data, inv_freq.data, (int)cos.dim(0), (int)half, stream));
}

int64_t Kernels::gemm_workspace_floats(int64_t M, int64_t rows, int64_t K, bool swiglu) const {
  if (!fn_->gemm_split_preferred((int)M, (int)rows, (int)K, swiglu ? 1 : 0)) return 0;
  return fn_->gemm_split_floats((int)M, (int)rows, (int)K, swiglu ? 1 : 0);
}

// Runs the product through chunk sums in the workspace if that is the faster route and it fits.
bool Kernels::split(Tensor& out, const Tensor& act, const Tensor& w, bool swiglu, const Tensor* workspace) {
  if (!workspace) return false;
  const int64_t M = act.dim(0), K = act.dim(1), rows = w.dim(0);
  const int64_t need = gemm_workspace_floats(M, rows, K, swiglu);
  if (need == 0 || workspace->dtype != DType::F32 || workspace->numel() < need) return false;
  call(fn_->gemm_split(out.data, act.data, w.data, (int)M, (int)rows, (int)K, K, out.dim(1), swiglu ? 1 : 0, workspace->data,
                       workspace->numel(), stream));
  return true;
}

void Kernels::fill_random(Tensor& out, uint64_t seed, int kind, float p0, float p1) {
  expect(out, "tensor to fill", dtype_);
  call(fn_->fill_random(out.data, out.numel(), seed, kind, p0, p1, stream));
}

Tensor Kernels::gemm(const Tensor& act, const Tensor& w, const Tensor* workspace) {
  expect(act, "activation", dtype_);
  expect(w, "weight", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 2 || act.dim(1) != w.dim(1))
    throw EngineError("gemm: activation " + act.describe() + " does not fit weight " + w.describe());
  const int64_t M = act.dim(0), K = act.dim(1), N = w.dim(0);
  Tensor out = empty({M, N});
  if (split(out, act, w, false, workspace)) return out;
  call(fn_->gemm(out.data, act.data, w.data, (int)M, (int)N, (int)K, K, N, 0, stream));
  return out;
}

Tensor Kernels::gemm_swiglu(const Tensor& act, const Tensor& w, const Tensor* workspace) {
  expect(act, "activation", dtype_);
  expect(w, "gate/up weight", dtype_);
  if (act.shape.size() != 2 || w.shape.size() != 2 || act.dim(1) != w.dim(1) || w.dim(0) % 2)
    throw EngineError("gemm_swiglu: activation " + act.describe() + " does not fit a gate/up weight " + w.describe());
  const int64_t M = act.dim(0), K = act.dim(1), I = w.dim(0) / 2;
  // One launch where the sizes allow it, else projection and activation one after the other: the same bits.
  if (!fn_->gemm_swiglu_supported((int)M, (int)I, (int)K)) return swiglu(gemm(act, w, workspace));
  Tensor out = empty({M, I});
  if (split(out, act, w, true, workspace)) return out;
  call(fn_->gemm_swiglu(out.data, act.data, w.data, (int)M, (int)I, (int)K, K, I, stream));
  return out;
}

Tensor Kernels::qkv_post(const Tensor& qkv, int nq, int nkv, int d, const Tensor* k_cache, const Tensor* v_cache,
                         int page_size, const Tensor* q_w, const Tensor* k_w, float eps, const Tensor* cos,
                         const Tensor* sin, const Tensor* positions, const Tensor* slots) {
  expect(qkv, "qkv", dtype_);
  const int64_t W = (int64_t)(nq + 2 * nkv) * d;
  if (qkv.shape.size() != 2 || qkv.dim(1) != W) throw EngineError("qkv_post: rows are " + qkv.describe() + ", expected width " + std::to_string(W));
  const int64_t T = qkv.dim(0);
  Tensor q_out;
  if (nq) q_out = empty({T, nq, d});
  int wf = 0;
  if (q_w) wf = norm_weight(*q_w, "q norm weight", d);
  if (k_w) {
    const int wf2 = norm_weight(*k_w, "k norm weight", d);
    if (q_w && wf2 != wf) throw EngineError("qkv_post: q and k norm weights must have the same type");
    wf = wf2;
  }
  int rot_half = 0;
  if (cos) {
    if (!sin || !positions) throw EngineError("qkv_post: a rotation needs cosines, sines and positions");
    expect(*cos, "cosine table", dtype_);
    if (cos->shape.size() != 2 || 2 * cos->dim(1) > d) throw EngineError("qkv_post: cosine table is " + cos->describe());
    expect(*sin, "sine table", dtype_, cos->shape);
    expect(*positions, "positions", DType::I32, {T});
    rot_half = (int)cos->dim(1);
  }
  if (nkv) {
    if (!k_cache || !v_cache || !slots) throw EngineError("qkv_post: a store needs both caches and slots");
    expect(*k_cache, "k cache", dtype_);
    if (k_cache->shape.size() != 4) throw EngineError("k cache is " + k_cache->describe());
    const int64_t pages = k_cache->dim(0);
    expect(*k_cache, "k cache", dtype_, {pages, nkv, page_size, d});
    expect(*v_cache, "v cache", dtype_, {pages, nkv, d, page_size});
    expect(*slots, "slots", DType::I32, {T});
  }
  call(fn_->qkv_post(qkv.data, W, nq ? q_out.data : nullptr, nkv ? k_cache->data : nullptr, nkv ? v_cache->data : nullptr,
                     q_w ? q_w->data : nullptr, k_w ? k_w->data : nullptr, wf, cos ? cos->data : nullptr,
                     cos ? sin->data : nullptr, rot_half, positions ? positions->data : nullptr,
                     slots ? slots->data : nullptr, (int)T, nq, nkv, d, page_size, eps, stream));
  return q_out;
}

int64_t Kernels::attn_scratch_floats(int items, int nq, int d, int nseg) const {
  return fn_->attn_scratch_floats(items, nq, d, nseg);
}

void Kernels::paged_attention(Tensor& out, const Tensor& q, const Tensor& k_cache, const Tensor& v_cache,
                              const Tensor& block_table, const Tensor& cu_q, const Tensor& k_len, const Tensor& items,
                              int mode, float scale, int window, int max_k_len, int nseg, const Tensor* scratch) {
  expect(q, "q", dtype_);
  expect(k_cache, "k cache", dtype_);
  expect(block_table, "block table", DType::I32);
  if (q.shape.size() != 3 || k_cache.shape.size() != 4 || block_table.shape.size() != 2)
    throw EngineError("attention: q " + q.describe() + ", k cache " + k_cache.describe() + ", block table " + block_table.describe());
  const int64_t T = q.dim(0), nq = q.dim(1), d = q.dim(2), pages = k_cache.dim(0), nkv = k_cache.dim(1), P = k_cache.dim(2);
  const int64_t S = block_table.dim(0), W = block_table.dim(1);
  expect(k_cache, "k cache", dtype_, {pages, nkv, P, d});
  expect(v_cache, "v cache", dtype_, {pages, nkv, d, P});
  expect(cu_q, "cu_q", DType::I32, {S + 1});
  expect(k_len, "k_len", DType::I32, {S});
  expect(out, "attention output", dtype_, q.shape);
  if (items.shape.size() != 2 || items.dim(1) != 2) throw EngineError("attention: items are " + items.describe());
  expect(items, "items", DType::I32);
  const int64_t n_items = items.dim(0);
  if (W * P < max_k_len)
    throw EngineError("attention: a block table of " + std::to_string(W) + " pages of " + std::to_string(P) + " does not cover " +
                      std::to_string(max_k_len) + " keys");
  void* sp = nullptr;
  if (mode == 1 || (mode >= 3 && mode <= 5) || mode == 7) {
    if (nseg < (max_k_len + segment_keys_ - 1) / segment_keys_)
      throw EngineError("attention: " + std::to_string(nseg) + " segments do not cover " + std::to_string(max_k_len) + " keys");
    const int64_t need = attn_scratch_floats((int)n_items, (int)nq, (int)d, nseg);
    if (!scratch || scratch->dtype != DType::F32 || scratch->numel() < need)
      throw EngineError("attention: scratch of " + std::to_string(need) + " floats needed");
    sp = scratch->data;
  }
  call(fn_->paged_attention(out.data, q.data, k_cache.data, v_cache.data, block_table.data, (int)W, cu_q.data, k_len.data,
                            items.data, (int)n_items, mode, nseg, sp, (int)T, (int)nq, (int)nkv, (int)d, (int)P, window, scale,
                            stream));
}

int Kernels::sample_scratch_words(int rows) const { return fn_->sample_scratch_words(rows); }

void Kernels::sample(Tensor& out, const Tensor& logits, const Tensor* temps, const Tensor* unis, Tensor& scratch) {
  expect(logits, "logits", dtype_);
  if (logits.shape.size() != 2) throw EngineError("logits are " + logits.describe());
  const int64_t R = logits.dim(0), V = logits.dim(1);
  expect(out, "sampled ids", DType::I32, {R});
  if (temps) {
    if (!unis) throw EngineError("sampling at a temperature needs uniform numbers");
    expect(*temps, "temperatures", DType::F32, {R});
    expect(*unis, "uniform numbers", DType::F32, {R});
  }
  if (scratch.dtype != DType::I32 || scratch.numel() < sample_scratch_words((int)R))
    throw EngineError("sampling: scratch of " + std::to_string(sample_scratch_words((int)R)) + " words needed");
  call(fn_->sample(out.data, logits.data, temps ? temps->data : nullptr, temps ? unis->data : nullptr, scratch.data, (int)R,
                   (int)V, V, stream));
}

}  // namespace vosti
