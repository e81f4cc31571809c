// Token selection from logit rows: greedy (the reference's sampler,
// python/vosti_kernels/kernels.py:1088-1104: argmax, first index on ties, a
// NaN counts as the maximum) and temperature sampling by inverse CDF.
//
// One workgroup of 256 threads per row.  For temperature sampling thread t owns
// the contiguous range [t*C, (t+1)*C) of the vocabulary, C = ceil(V/256): its
// sum runs over the range in ascending order, the 256 sums are scanned serially
// in thread order, and the owner of the target walks its range again.  The
// result is a function of the row, the temperature and the uniform number only.
#include "common.h"

#define SAMPLE_THREADS 256

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  const bool vn = v != v, bn = bv != bv;
  if (vn) return !bn || i < bi;
  if (bn) return false;
  return v > bv || (v == bv && i < bi);
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(int32_t* __restrict__ out,
                                                                const elem_t* __restrict__ logits,
                                                                const float* __restrict__ temps,
                                                                const float* __restrict__ uniforms, int V,
                                                                int64_t row_stride) {
  __shared__ float s_val[SAMPLE_THREADS];
  __shared__ int s_idx[SAMPLE_THREADS];
  __shared__ float s_pre[SAMPLE_THREADS + 1];
  const int r = blockIdx.x, t = threadIdx.x;
  const elem_t* row = logits + r * row_stride;
  const float temp = temps ? temps[r] : 0.f;

  // ---- maximum and its first index ----
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = t; i < V; i += SAMPLE_THREADS) {
    const float v = to_f32(row[i]);
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  }
  s_val[t] = bv;
  s_idx[t] = bi;
  __syncthreads();
  for (int off = SAMPLE_THREADS / 2; off > 0; off >>= 1) {
    if (t < off && better(s_val[t + off], s_idx[t + off], s_val[t], s_idx[t])) {
      s_val[t] = s_val[t + off];
      s_idx[t] = s_idx[t + off];
    }
    __syncthreads();
  }
  const float vmax = s_val[0];
  const int imax = s_idx[0];
  if (!(temp > 0.f) || vmax != vmax || vmax == INFINITY) {
    if (t == 0) out[r] = imax;
    return;
  }
  // ---- softmax(logits / temp) by inverse CDF ----
  const float zmax = vmax / temp;
  const int C = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int lo = min(V, t * C), hi = min(V, lo + C);
  float sum = 0.f;
  for (int i = lo; i < hi; ++i) sum = sum + expf(to_f32(row[i]) / temp - zmax);
  __syncthreads();
  s_val[t] = sum;
  __syncthreads();
  __shared__ int s_owner;
  if (t == 0) {
    float run = 0.f;
    for (int j = 0; j < SAMPLE_THREADS; ++j) {
      s_pre[j] = run;
      run = run + s_val[j];
    }
    s_pre[SAMPLE_THREADS] = run;
    // Owner: the first thread whose range carries the target; if rounding puts
    // the target at or beyond the total, the last thread with a positive sum.
    const float target0 = uniforms[r] * run;
    int own = -1, last = 0;
    for (int j = 0; j < SAMPLE_THREADS; ++j) {
      if (s_val[j] > 0.f) {
        last = j;
        if (own < 0 && target0 < s_pre[j + 1]) own = j;
      }
    }
    s_owner = own >= 0 ? own : last;
  }
  __syncthreads();
  const float target = uniforms[r] * s_pre[SAMPLE_THREADS];
  const bool owner = t == s_owner;
  if (owner) {
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

// temps null: greedy for every row.  A row with temperature <= 0 is greedy.
int vk_sample(int32_t* out, const elem_t* logits, const float* temps, const float* uniforms, int R, int V,
              int64_t row_stride, hipStream_t st) {
  VK_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
  VK_REQUIRE(row_stride >= V, "sample: row stride %lld smaller than V=%d", (long long)row_stride, V);
  VK_REQUIRE(temps == nullptr || uniforms != nullptr, "sample: temperatures need uniform numbers");
  if (R == 0) return 0;
  sample_kernel<<<R, SAMPLE_THREADS, 0, st>>>(out, logits, temps, uniforms, V, row_stride);
  return vk_check_launch("sample");
}

}  // extern "C"
