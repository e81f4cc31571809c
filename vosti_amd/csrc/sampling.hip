// Token selection from logit rows: greedy (the reference's sampler,
// python/vosti_kernels/kernels.py:1088-1104: argmax, first index on ties, a
// NaN counts as the maximum) and temperature sampling by inverse CDF.
//
// Two launches.  The first cuts every row into SAMPLE_BLOCKS contiguous ranges
// and finds each range's maximum and its first index.  The second, one
// workgroup of 1024 threads per row, merges them in range order; for
// temperature sampling thread t then owns the contiguous range [t*C, (t+1)*C)
// of the vocabulary, C = ceil(V/1024): its sum of exp((x - max)/T) runs over the
// range in ascending order, the 1024 sums are scanned serially in thread order,
// and the owner of the target walks its range again.  The result is a function
// of the row, the temperature and the uniform number only.
#include "common.h"
#include "sampling.h"

#include <mutex>

#define SAMPLE_BLOCKS 32
#define PARTIAL_THREADS 256
#define FINAL_THREADS 1024

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  const bool vn = v != v, bn = bv != bv;
  if (vn) return !bn || i < bi;
  if (bn) return false;
  return v > bv || (v == bv && i < bi);
}

__global__ __launch_bounds__(PARTIAL_THREADS) void argmax_partial_kernel(float* __restrict__ pval, int* __restrict__ pidx,
                                                                         const elem_t* __restrict__ logits, int V,
                                                                         int64_t row_stride) {
  __shared__ float s_val[PARTIAL_THREADS];
  __shared__ int s_idx[PARTIAL_THREADS];
  const int r = blockIdx.x, b = blockIdx.y, t = threadIdx.x;
  const elem_t* row = logits + r * row_stride;
  const int span = (V + SAMPLE_BLOCKS - 1) / SAMPLE_BLOCKS;
  const int lo = min(V, b * span), hi = min(V, lo + span);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + t; i < hi; i += PARTIAL_THREADS) {
    const float v = to_f32(row[i]);
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  }
  s_val[t] = bv;
  s_idx[t] = bi;
  __syncthreads();
  for (int off = PARTIAL_THREADS / 2; off > 0; off >>= 1) {
    if (t < off && better(s_val[t + off], s_idx[t + off], s_val[t], s_idx[t])) {
      s_val[t] = s_val[t + off];
      s_idx[t] = s_idx[t + off];
    }
    __syncthreads();
  }
  if (t == 0) {
    pval[r * SAMPLE_BLOCKS + b] = s_val[0];
    pidx[r * SAMPLE_BLOCKS + b] = s_idx[0];
  }
}

__global__ __launch_bounds__(FINAL_THREADS) void sample_final_kernel(int32_t* __restrict__ out,
                                                                     const float* __restrict__ pval,
                                                                     const int* __restrict__ pidx,
                                                                     const elem_t* __restrict__ logits,
                                                                     const float* __restrict__ temps,
                                                                     const float* __restrict__ uniforms, int V,
                                                                     int64_t row_stride) {
  __shared__ float s_sum[FINAL_THREADS];
  __shared__ float s_pre[FINAL_THREADS + 1];
  __shared__ int s_owner;
  const int r = blockIdx.x, t = threadIdx.x;
  const elem_t* row = logits + r * row_stride;
  const float temp = temps ? temps[r] : 0.f;
  // Every thread merges the ranges' maxima in range order: the same result in all.
  float vmax = -INFINITY;
  int imax = 0x7fffffff;
  for (int b = 0; b < SAMPLE_BLOCKS; ++b) {
    const float v = pval[r * SAMPLE_BLOCKS + b];
    const int i = pidx[r * SAMPLE_BLOCKS + b];
    if (i != 0x7fffffff && better(v, i, vmax, imax)) { vmax = v; imax = i; }
  }
  if (!(temp > 0.f) || vmax != vmax || vmax == INFINITY) {
    if (t == 0) out[r] = imax;
    return;
  }
  // ---- softmax(logits / temp) by inverse CDF ----
  const float zmax = vmax / temp;
  const int C = (V + FINAL_THREADS - 1) / FINAL_THREADS;
  const int lo = min(V, t * C), hi = min(V, lo + C);
  float sum = 0.f;
  for (int i = lo; i < hi; ++i) sum = sum + expf(to_f32(row[i]) / temp - zmax);
  s_sum[t] = sum;
  __syncthreads();
  if (t == 0) {
    float run = 0.f;
    for (int j = 0; j < FINAL_THREADS; ++j) {
      s_pre[j] = run;
      run = run + s_sum[j];
    }
    s_pre[FINAL_THREADS] = run;
    // Owner: the first thread whose range carries the target; if rounding puts
    // the target at or beyond the total, the last thread with a positive sum.
    const float target0 = uniforms[r] * run;
    int own = -1, last = 0;
    for (int j = 0; j < FINAL_THREADS; ++j) {
      if (s_sum[j] > 0.f) {
        last = j;
        if (own < 0 && target0 < s_pre[j + 1]) own = j;
      }
    }
    s_owner = own >= 0 ? own : last;
  }
  __syncthreads();
  if (t == s_owner) {
    const float target = uniforms[r] * s_pre[FINAL_THREADS];
    float run = s_pre[t];
    int pick = -1, last_pos = lo;
    for (int i = lo; i < hi; ++i) {
      const float e = expf(to_f32(row[i]) / temp - zmax);
      run = run + e;
      if (e > 0.f) last_pos = i;
      if (pick < 0 && target < run) pick = i;
    }
    out[r] = pick >= 0 ? pick : last_pos;
  }
}

extern "C" {

// Words (4 bytes each) of scratch that vk_sample needs for R rows.
int vk_sample_scratch_words(int R) { return 2 * R * SAMPLE_BLOCKS; }

// temps null: greedy for every row.  A row with temperature <= 0 is greedy.
int vk_sample(int32_t* out, const elem_t* logits, const float* temps, const float* uniforms, void* scratch, int R,
              int V, int64_t row_stride, hipStream_t st) {
  VK_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
  VK_REQUIRE(row_stride >= V, "sample: row stride %lld smaller than V=%d", (long long)row_stride, V);
  VK_REQUIRE(temps == nullptr || uniforms != nullptr, "sample: temperatures need uniform numbers");
  VK_REQUIRE(scratch != nullptr, "sample: scratch is missing");
  if (R == 0) return 0;
  float* pval = static_cast<float*>(scratch);
  int* pidx = reinterpret_cast<int*>(pval + (int64_t)R * SAMPLE_BLOCKS);
  argmax_partial_kernel<<<dim3(R, SAMPLE_BLOCKS), PARTIAL_THREADS, 0, st>>>(pval, pidx, logits, V, row_stride);
  if (vk_check_launch("sample (partial)")) return 1;
  sample_final_kernel<<<R, FINAL_THREADS, 0, st>>>(out, pval, pidx, logits, temps, uniforms, V, row_stride);
  return vk_check_launch("sample");
}

}  // extern "C"

// ---- the variant that allocates nothing (see sampling.h) ----
// The partial maxima of vk_sample's first kernel, for up to VK_SAMPLE_STATIC_MAX_ROWS rows, in device
// memory that belongs to the library: 8 bytes per (row, range).  Every GPU that the library runs on
// holds its own copy of this array at its own address, until the process ends.
static __device__ __align__(256) unsigned char scratch[(size_t)VK_SAMPLE_STATIC_MAX_ROWS * SAMPLE_BLOCKS * 8];

#define VK_MAX_DEVICES 64
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[VK_MAX_DEVICES];      // device address of `scratch`, per device; null until asked for

// The device address of `scratch` on the current device.  In host code the array's name is only a
// handle for the runtime, not an address a kernel can use: the address is asked for once per device.
static int static_scratch(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return vk_fail("sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= VK_MAX_DEVICES) return vk_fail("sample_static: device index %d is beyond %d", dev, VK_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return vk_fail("sample_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

extern "C" {

int vk_sample_static_max_rows(void) { return VK_SAMPLE_STATIC_MAX_ROWS; }

int vk_sample_static(int32_t* out, const elem_t* logits, const float* temps, const float* uniforms, int R, int V,
                     int64_t row_stride, hipStream_t st) {
  VK_REQUIRE(R >= 0 && V > 0, "sample_static: bad sizes R=%d V=%d", R, V);
  VK_REQUIRE(R <= VK_SAMPLE_STATIC_MAX_ROWS, "sample_static: %d rows are more than the %d that the library's own scratch holds",
             R, VK_SAMPLE_STATIC_MAX_ROWS);
  VK_REQUIRE(row_stride >= V, "sample_static: row stride %lld smaller than V=%d", (long long)row_stride, V);
  VK_REQUIRE(temps == nullptr || uniforms != nullptr, "sample_static: temperatures need uniform numbers");
  VK_REQUIRE(out != nullptr && logits != nullptr, "sample_static: out and logits are needed");
  if (R == 0) return 0;
  void* base = nullptr;
  if (static_scratch(&base)) return 1;
  // Nothing has to start at zero: the first kernel writes every word that the second one reads.
  float* pval = static_cast<float*>(base);
  int* pidx = reinterpret_cast<int*>(pval + (size_t)VK_SAMPLE_STATIC_MAX_ROWS * SAMPLE_BLOCKS);
  argmax_partial_kernel<<<dim3(R, SAMPLE_BLOCKS), PARTIAL_THREADS, 0, st>>>(pval, pidx, logits, V, row_stride);
  if (vk_check_launch("sample_static (partial)")) return 1;
  sample_final_kernel<<<R, FINAL_THREADS, 0, st>>>(out, pval, pidx, logits, temps, uniforms, V, row_stride);
  return vk_check_launch("sample_static");
}

}  // extern "C"
