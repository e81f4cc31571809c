// Row-wise and element-wise kernels: embedding, RMSNorm, residual-add RMSNorm,
// SwiGLU, row gather, casts, rotary tables and the counter-based weight filler.
//
// Formulas follow the reference's Triton kernels:
//   embedding            kernels/triton_kernels/embedding.py:57-84
//   RMSNorm              kernels/triton_kernels/rmsnorm.py:63-93   ((x*r)*w, fp32)
//   residual-add RMSNorm kernels/triton_kernels/rmsnorm_residual.py:73-125
//                        (the norm sees the unrounded fp32 sum)
//   SwiGLU               kernels/triton_kernels/silu_mul.py:64-87   (x*sigmoid(x)*y)
//   rotary tables        python/vosti_kernels/rotary.py:137-160
#include "common.h"
#include "vec.h"

#define NORM_THREADS 256

// ---------------------------------------------------------------- embedding
__global__ __launch_bounds__(256) void embedding_kernel(elem_t* __restrict__ out,
                                                        const elem_t* __restrict__ table,
                                                        const int32_t* __restrict__ ids, int H, int vec_ok) {
  const int t = blockIdx.x;
  const int64_t id = ids[t];
  const elem_t* src = table + id * (int64_t)H;
  elem_t* dst = out + (int64_t)t * H;
  if (vec_ok) {
    const u32x4* s = reinterpret_cast<const u32x4*>(src);
    u32x4* d = reinterpret_cast<u32x4*>(dst);
    const int nv = H / VK_VEC;
    for (int i = threadIdx.x; i < nv; i += blockDim.x) d[i] = s[i];
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = src[i];
  }
}

// ------------------------------------------------------------------ RMSNorm
// One workgroup per row.  Thread t owns the vectors t, t+256, ... of the row;
// its partial sum runs over them in that order, a wave butterfly follows, and
// the four wave sums are added in wave order.  The order depends on H alone.
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum_xor(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = red[0];
  s = s + red[1];
  s = s + red[2];
  s = s + red[3];
  return s;
}

template <int VEC, bool ADD>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_kernel(
    elem_t* __restrict__ out, elem_t* res_io, const elem_t* __restrict__ x, const void* __restrict__ w,
    int w_is_f32, int H, int heads, int64_t x_tok_stride, int64_t out_tok_stride, float eps) {
  extern __shared__ float smem[];
  float* row32 = smem;        // H floats: the unrounded row
  float* red = smem + H;      // 4 floats
  const int r = blockIdx.x;
  const int tok = r / heads, head = r - tok * heads;
  const elem_t* xr = x + tok * x_tok_stride + (int64_t)head * H;
  elem_t* outr = out + tok * out_tok_stride + (int64_t)head * H;
  elem_t* resr = ADD ? res_io + (int64_t)r * H : nullptr;

  float part = 0.f;
  const int nv = H / VEC;
  for (int v = threadIdx.x; v < nv; v += NORM_THREADS) {
    float a[VEC];
    load_elems(xr + v * VEC, a);
    if (ADD) {
      float b[VEC];
      load_elems(resr + v * VEC, b);
#pragma unroll
      for (int i = 0; i < VEC; ++i) a[i] = a[i] + b[i];
      store_elems(resr + v * VEC, a);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      row32[v * VEC + i] = a[i];
      part = part + a[i] * a[i];
    }
  }
  const float total = block_sum_256(part, red);
  const float var = total / (float)H;
  const float rr = rsqrtf(var + eps);
  for (int v = threadIdx.x; v < nv; v += NORM_THREADS) {
    float y[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const int c = v * VEC + i;
      y[i] = (row32[c] * rr) * load_weight(w, w_is_f32, c);
    }
    store_elems(outr + v * VEC, y);
  }
}

// The same computation with the row in registers: NV vectors of VEC elements per thread, for rows of up
// to NV * NORM_THREADS vectors.  The sums are taken in the order of rmsnorm_kernel, so the bits are the same.
template <int VEC, bool ADD, int NV>
__global__ __launch_bounds__(NORM_THREADS) void rmsnorm_reg_kernel(
    elem_t* __restrict__ out, elem_t* res_io, const elem_t* __restrict__ x, const void* __restrict__ w,
    int w_is_f32, int H, int heads, int64_t x_tok_stride, int64_t out_tok_stride, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const int tok = r / heads, head = r - tok * heads;
  const elem_t* xr = x + tok * x_tok_stride + (int64_t)head * H;
  elem_t* outr = out + tok * out_tok_stride + (int64_t)head * H;
  elem_t* resr = ADD ? res_io + (int64_t)r * H : nullptr;
  const int nv = H / VEC;

  float a[NV][VEC], wv[NV][VEC];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = threadIdx.x + j * NORM_THREADS;
    if (v < nv) {
      load_elems(xr + v * VEC, a[j]);
      if (w_is_f32) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) wv[j][i] = static_cast<const float*>(w)[v * VEC + i];
      } else {
        load_elems(static_cast<const elem_t*>(w) + v * VEC, wv[j]);
      }
    }
  }
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = threadIdx.x + j * NORM_THREADS;
    if (v < nv) {
      if (ADD) {
        float b[VEC];
        load_elems(resr + v * VEC, b);
#pragma unroll
        for (int i = 0; i < VEC; ++i) a[j][i] = a[j][i] + b[i];
        store_elems(resr + v * VEC, a[j]);
      }
#pragma unroll
      for (int i = 0; i < VEC; ++i) part = part + a[j][i] * a[j][i];
    }
  }
  const float total = block_sum_256(part, red);
  const float var = total / (float)H;
  const float rr = rsqrtf(var + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = threadIdx.x + j * NORM_THREADS;
    if (v < nv) {
      float y[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) y[i] = (a[j][i] * rr) * wv[j][i];
      store_elems(outr + v * VEC, y);
    }
  }
}

// ------------------------------------------------------------------- SwiGLU
template <int VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ gu,
                                                     int I) {
  const int t = blockIdx.y;
  const int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v * VEC >= I) return;
  const elem_t* g = gu + (int64_t)t * 2 * I + v * VEC;
  float a[VEC], b[VEC], y[VEC];
  load_elems(g, a);
  load_elems(g + I, b);
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    const float sig = 1.0f / (1.0f + expf(-a[i]));
    y[i] = (a[i] * sig) * b[i];
  }
  store_elems(out + (int64_t)t * I + v * VEC, y);
}

// -------------------------------------------------------------- row gather
__global__ __launch_bounds__(256) void gather_rows_kernel(elem_t* __restrict__ out, const elem_t* __restrict__ x,
                                                          const int32_t* __restrict__ rows, int H) {
  const int r = blockIdx.x;
  const elem_t* src = x + (int64_t)rows[r] * H;
  elem_t* dst = out + (int64_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = src[i];
}

// -------------------------------------------------------------------- casts
__global__ void cast_to_f32_kernel(float* __restrict__ out, const elem_t* __restrict__ in, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = to_f32(in[i]);
}
__global__ void cast_from_f32_kernel(elem_t* __restrict__ out, const float* __restrict__ in, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<elem_t>(in[i]);
}

// ------------------------------------------------------------ rotary tables
// angle = inv_freq[j] * float(p) in fp32; cos and sin in fp32, then stored as
// elements (rounded to bfloat16 in that build, as the reference's tables are).
__global__ void rope_tables_kernel(elem_t* __restrict__ cos_t, elem_t* __restrict__ sin_t,
                                   const float* __restrict__ inv_freq, int max_pos, int half) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)max_pos * half) return;
  const int p = (int)(i / half), j = (int)(i - (int64_t)p * half);
  const float ang = inv_freq[j] * (float)p;
  cos_t[i] = from_f32<elem_t>(cosf(ang));
  sin_t[i] = from_f32<elem_t>(sinf(ang));
}

// ------------------------------------------------------------ random filler
// Counter-based: element i of a tensor depends on (seed, i) only, and every
// operation is exact integer arithmetic followed by correctly rounded float
// operations, so a host implementation gives the same bits.
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// kind 0: approximately normal (sum of four 16-bit uniforms), value = (s - 131070) * p0
// kind 1: uniform, value = p0 + u * p1 with u = 24 bits * 2^-24
__global__ void fill_random_kernel(elem_t* __restrict__ out, int64_t n, uint64_t seed, int kind, float p0,
                                   float p1) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t z = mix64(seed ^ ((uint64_t)i * 0x9E3779B97F4A7C15ull));
  float v;
  if (kind == 0) {
    const int s = (int)(z & 0xFFFF) + (int)((z >> 16) & 0xFFFF) + (int)((z >> 32) & 0xFFFF) + (int)(z >> 48);
    v = (float)(s - 131070) * p0;
  } else {
    const float u = (float)(uint32_t)(z >> 40) * 5.9604644775390625e-08f;
    v = p0 + u * p1;
  }
  out[i] = from_f32<elem_t>(v);
}

// ------------------------------------------------------------- a yardstick
// Reads `n16` 16-byte vectors and keeps nothing: every wave has 16 KB in flight and does nothing else.  What
// this reaches on a buffer is what a kernel that must read that buffer once can reach at best; measurements
// price the projections against it (bench.py).
__global__ __launch_bounds__(512) void pull_kernel(const u32x4* __restrict__ p, int64_t n16, uint32_t* sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6);
  const int64_t first = wave * 1024;                   // this wave's 16 KB
  if (first >= n16) return;
  u32x4 v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t at = first + i * 64 + lane;
    v[i] = p[at < n16 ? at : n16 - 1];                  // the last wave's tail: the last vector again
  }
  u32x4 a = v[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) a ^= v[i];
  if ((a.x ^ a.y ^ a.z ^ a.w) == 0x5a17c0deu && a.x == 0x12345678u) sink[0] = a.y;      // never, in practice: keeps the loads
}

// ================================================================ host side
extern "C" {

int vk_embedding(elem_t* out, const elem_t* table, const int32_t* ids, int T, int H, int V, hipStream_t st) {
  VK_REQUIRE(T >= 0 && H > 0 && V > 0, "embedding: bad sizes T=%d H=%d V=%d", T, H, V);
  if (T == 0) return 0;
  embedding_kernel<<<T, 256, 0, st>>>(out, table, ids, H, H % VK_VEC == 0);
  return vk_check_launch("embedding");
}

static int norm_launch(bool add, elem_t* out, elem_t* res_io, const elem_t* x, const void* w, int w_is_f32,
                       int rows, int H, int heads, int64_t xs, int64_t os, float eps, hipStream_t st) {
  VK_REQUIRE(rows >= 0 && H > 0 && heads > 0, "rmsnorm: bad sizes rows=%d H=%d heads=%d", rows, H, heads);
  VK_REQUIRE(H <= 32768, "rmsnorm: row length %d exceeds the supported maximum of 32768", H);
  VK_REQUIRE(eps >= 0.f, "rmsnorm: eps must not be negative");
  if (rows == 0) return 0;
  const bool vec = (H % VK_VEC == 0) && (xs % VK_VEC == 0) && (os % VK_VEC == 0);
  const size_t smem = (size_t)(H + 4) * sizeof(float);
#define LAUNCH(VEC, ADD)                                                                              \
  do {                                                                                                \
    if (smem > 48 * 1024)                                                                             \
      (void)hipFuncSetAttribute((const void*)rmsnorm_kernel<VEC, ADD>,                                \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);               \
    rmsnorm_kernel<VEC, ADD><<<rows, NORM_THREADS, smem, st>>>(out, res_io, x, w, w_is_f32, H, heads, \
                                                               xs, os, eps);                          \
  } while (0)
#define LAUNCH_REG(ADD, NV)                                                                                    \
  rmsnorm_reg_kernel<VK_VEC, ADD, NV><<<rows, NORM_THREADS, 0, st>>>(out, res_io, x, w, w_is_f32, H, heads, xs, os, eps)
  const int nv = H / VK_VEC;
  if (vec && nv <= 4 * NORM_THREADS) {
    // The row fits the registers of a workgroup: no trip through LDS.
    if (add) {
      if (nv <= NORM_THREADS) LAUNCH_REG(true, 1); else if (nv <= 2 * NORM_THREADS) LAUNCH_REG(true, 2); else LAUNCH_REG(true, 4);
    } else {
      if (nv <= NORM_THREADS) LAUNCH_REG(false, 1); else if (nv <= 2 * NORM_THREADS) LAUNCH_REG(false, 2); else LAUNCH_REG(false, 4);
    }
  } else if (add) {
    if (vec) LAUNCH(VK_VEC, true); else LAUNCH(1, true);
  } else {
    if (vec) LAUNCH(VK_VEC, false); else LAUNCH(1, false);
  }
#undef LAUNCH_REG
#undef LAUNCH
  return vk_check_launch("rmsnorm");
}

// out[tok, head, :] = rmsnorm(x[tok, head, :]) for rows = tokens * heads rows of
// length H; token strides are in elements.
int vk_rmsnorm(elem_t* out, const elem_t* x, const void* w, int w_is_f32, int rows, int H, int heads,
               int64_t x_tok_stride, int64_t out_tok_stride, float eps, hipStream_t st) {
  return norm_launch(false, out, nullptr, x, w, w_is_f32, rows, H, heads, x_tok_stride, out_tok_stride, eps, st);
}

// residual += x (in fp32, stored rounded); normed = rmsnorm(unrounded sum).
int vk_add_rmsnorm(elem_t* normed, elem_t* residual_io, const elem_t* x, const void* w, int w_is_f32,
                   int rows, int H, float eps, hipStream_t st) {
  return norm_launch(true, normed, residual_io, x, w, w_is_f32, rows, H, 1, H, H, eps, st);
}

int vk_swiglu(elem_t* out, const elem_t* gate_up, int T, int I, hipStream_t st) {
  VK_REQUIRE(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
  VK_REQUIRE(T <= 65535 * 64, "swiglu: too many rows (%d)", T);
  if (T == 0) return 0;
  if (I % VK_VEC == 0) {
    dim3 grid((I / VK_VEC + 255) / 256, T);
    swiglu_kernel<VK_VEC><<<grid, 256, 0, st>>>(out, gate_up, I);
  } else {
    dim3 grid((I + 255) / 256, T);
    swiglu_kernel<1><<<grid, 256, 0, st>>>(out, gate_up, I);
  }
  return vk_check_launch("swiglu");
}

int vk_gather_rows(elem_t* out, const elem_t* x, const int32_t* rows, int R, int H, hipStream_t st) {
  VK_REQUIRE(R >= 0 && H > 0, "gather_rows: bad sizes R=%d H=%d", R, H);
  if (R == 0) return 0;
  gather_rows_kernel<<<R, 256, 0, st>>>(out, x, rows, H);
  return vk_check_launch("gather_rows");
}

int vk_cast_to_f32(float* out, const elem_t* in, int64_t n, hipStream_t st) {
  if (n <= 0) return 0;
  cast_to_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, in, n);
  return vk_check_launch("cast_to_f32");
}

int vk_cast_from_f32(elem_t* out, const float* in, int64_t n, hipStream_t st) {
  if (n <= 0) return 0;
  cast_from_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, in, n);
  return vk_check_launch("cast_from_f32");
}

int vk_rope_tables(elem_t* cos_t, elem_t* sin_t, const float* inv_freq, int max_pos, int half, hipStream_t st) {
  VK_REQUIRE(max_pos > 0 && half > 0, "rope_tables: bad sizes max_pos=%d half=%d", max_pos, half);
  const int64_t n = (int64_t)max_pos * half;
  rope_tables_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(cos_t, sin_t, inv_freq, max_pos, half);
  return vk_check_launch("rope_tables");
}

// The measurements' yardstick, no part of any model: reads `bytes` bytes at p (16-byte aligned) once and keeps
// nothing, so that a projection's time can be set against what a plain read of its weights takes on the same
// machine (bench.py's read_only_us).  `sink`: four bytes of device memory that are practically never written.
int vk_pull(const void* p, int64_t bytes, void* sink, hipStream_t st) {
  VK_REQUIRE(p != nullptr && sink != nullptr && ((uintptr_t)p % 16) == 0 && bytes >= 16, "pull: bad operands");
  const int64_t n16 = bytes / 16;
  const int64_t waves = (n16 + 1023) / 1024;
  VK_REQUIRE((waves + 7) / 8 <= 0x7fffffff, "pull: buffer too large");
  pull_kernel<<<(unsigned)((waves + 7) / 8), 512, 0, st>>>(static_cast<const u32x4*>(p), n16, static_cast<uint32_t*>(sink));
  return vk_check_launch("pull");
}

int vk_fill_random(elem_t* out, int64_t n, uint64_t seed, int kind, float p0, float p1, hipStream_t st) {
  VK_REQUIRE(kind == 0 || kind == 1, "fill_random: unknown kind %d", kind);
  if (n <= 0) return 0;
  VK_REQUIRE((n + 255) / 256 <= 0x7fffffff, "fill_random: tensor too large");
  fill_random_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, n, seed, kind, p0, p1);
  return vk_check_launch("fill_random");
}

}  // extern "C"
