// What happens to the q, k and v rows between the QKV projection and attention,
// in one launch: per-head RMSNorm of q and k, rotary position encoding of q and
// k, and the write of k and v into their pages.  Each step is optional, so the
// same kernel also serves as a plain head norm, a plain rotation or a plain
// cache store.
//
// Formulas (reference):
//   head norm  kernels/triton_kernels/qk_norm.py:67-95   y = x*rsqrt(mean(x^2)+eps)*w, rounded
//   rotation   kernels/triton_kernels/rope.py:78-123     y1 = x1*cos - x2*sin; y2 = x2*cos + x1*sin,
//              halves split at rot/2, on the rounded norm output, tables indexed by position
//   store      kernels/triton_kernels/store_kv_cache.py:89-120   slot -1 writes nothing
// The reference runs them as five launches (src/exec/dense_swiglu_decoder.rs:207-272).
//
// One wave per (token, head) at a time; lane l owns elements l, l+64, l+128, l+192.
#include "common.h"
#include "vec.h"

struct QkvPostArgs {
  const elem_t* qkv;      // [T, row_stride]: nq q heads, then nkv k heads, then nkv v heads, d each
  int64_t row_stride;
  elem_t* q_out;          // [T, nq, d]
  elem_t* kc;             // [pages, nkv, P, d]
  elem_t* vc;             // [pages, nkv, d, P]
  const void* q_w;        // [d] or null
  const void* k_w;        // [d] or null
  const elem_t* cos_t;    // [max_pos, rot_half] or null
  const elem_t* sin_t;
  const int32_t* positions;  // [T]
  const int32_t* slots;      // [T]: page * P + offset, or -1
  int w_is_f32, nq, nkv, d, P, rot_half;
  float eps;
};

// A workgroup has four waves and one token; wave w takes the heads first + w, first + w + 4, ... of the
// workgroup's `per_wave` * 4 heads, so that a long step does not start a workgroup per head.
__global__ __launch_bounds__(256) void qkv_post_kernel(QkvPostArgs a, int per_wave) {
  __shared__ float ybuf[4][256];
  const int tok = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* y = ybuf[wave];
  const int d = a.d, heads = a.nq + 2 * a.nkv;
  const int rh = a.rot_half;
  // With a rotation half of 64 or 128 elements the partner of an element is held by the same lane.
  const bool in_lane = rh % 64 == 0;
  const int shift = rh / 64;
  int64_t trow = 0;
  if (a.cos_t != nullptr) trow = (int64_t)a.positions[tok] * rh;
  const int slot = a.slots != nullptr ? a.slots[tok] : -1;
  for (int j = 0; j < per_wave; ++j) {
    const int hh = (blockIdx.y * per_wave + j) * 4 + wave;
    const bool live = hh < heads;            // the same number of barriers for every wave
    const int kind = hh < a.nq ? 0 : (hh < a.nq + a.nkv ? 1 : 2);   // q, k, v
    const elem_t* x = a.qkv + tok * a.row_stride + (int64_t)(live ? hh : 0) * d;
    const void* w = kind == 0 ? a.q_w : (kind == 1 ? a.k_w : nullptr);

    float xv[4];
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + 64 * i;
      xv[i] = c < d ? to_f32(x[c]) : 0.f;
      part = part + xv[i] * xv[i];
    }
    if (w != nullptr) {
      const float total = wave_sum_xor(part);
      const float rr = rsqrtf(total / (float)d + a.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < d) xv[i] = round_to_elem((xv[i] * rr) * load_weight(w, a.w_is_f32, c));
      }
    }
    const bool rotate = a.cos_t != nullptr && kind != 2;
    if (a.cos_t != nullptr && !in_lane) {
      if (rotate) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int c = lane + 64 * i;
          if (c < d) y[c] = xv[i];
        }
      }
      __syncthreads();
    }
    if (rotate) {
      float old[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) old[i] = xv[i];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < rh) {
          const float cs = to_f32(a.cos_t[trow + c]), sn = to_f32(a.sin_t[trow + c]);
          const float other = in_lane ? (i + shift < 4 ? old[(i + shift) & 3] : 0.f) : y[c + rh];
          xv[i] = old[i] * cs - other * sn;
        } else if (c < 2 * rh) {
          const float cs = to_f32(a.cos_t[trow + c - rh]), sn = to_f32(a.sin_t[trow + c - rh]);
          const float other = in_lane ? (i >= shift ? old[(i - shift) & 3] : 0.f) : y[c - rh];
          xv[i] = old[i] * cs + other * sn;
        }
      }
    }
    if (a.cos_t != nullptr && !in_lane) __syncthreads();    // y is free for the next head
    if (!live) continue;
    if (kind == 0) {
      elem_t* o = a.q_out + ((int64_t)tok * a.nq + hh) * d;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < d) o[c] = from_f32<elem_t>(xv[i]);
      }
      continue;
    }
    if (slot < 0) continue;
    const int page = slot / a.P, off = slot - page * a.P;
    if (kind == 1) {
      const int kh = hh - a.nq;
      elem_t* o = a.kc + (((int64_t)page * a.nkv + kh) * a.P + off) * d;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < d) o[c] = from_f32<elem_t>(xv[i]);
      }
    } else {
      const int kh = hh - a.nq - a.nkv;
      elem_t* o = a.vc + ((int64_t)page * a.nkv + kh) * d * a.P + off;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < d) o[(int64_t)c * a.P] = from_f32<elem_t>(xv[i]);
      }
    }
  }
}

// The same for head sizes 64, 128 and 256 with a full rotation (or none): a lane owns VK_VEC
// consecutive elements, so that rows are read and written 16 bytes per lane; the d / VK_VEC lanes of a
// head sit side by side, a wave holds 64 / (d / VK_VEC) heads of one token.  The sum of squares runs
// over a lane's elements in order, then as a butterfly over the head's lanes.
template <int LPH>     // lanes per head
__global__ __launch_bounds__(256) void qkv_post_vec_kernel(QkvPostArgs a, int per_wave) {
  constexpr int HPW = 64 / LPH;
  const int tok = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int d = a.d, heads = a.nq + 2 * a.nkv;
  const int j = lane % LPH, hsub = lane / LPH;
  int64_t trow = 0;
  if (a.cos_t != nullptr) trow = (int64_t)a.positions[tok] * a.rot_half;
  const int slot = a.slots != nullptr ? a.slots[tok] : -1;
  const int page = slot >= 0 ? slot / a.P : 0, off = slot >= 0 ? slot - page * a.P : 0;
  for (int it = 0; it < per_wave; ++it) {
    const int hh = ((blockIdx.y * per_wave + it) * 4 + wave) * HPW + hsub;
    const bool live = hh < heads;
    const int kind = hh < a.nq ? 0 : (hh < a.nq + a.nkv ? 1 : 2);   // q, k, v
    const elem_t* x = a.qkv + tok * a.row_stride + (int64_t)(live ? hh : 0) * d + j * VK_VEC;
    const void* w = kind == 0 ? a.q_w : (kind == 1 ? a.k_w : nullptr);
    float xv[VK_VEC];
    load_elems(x, xv);
    if (w != nullptr) {
      float part = 0.f;
#pragma unroll
      for (int e = 0; e < VK_VEC; ++e) part = part + xv[e] * xv[e];
#pragma unroll
      for (int m = 1; m < LPH; m <<= 1) part = part + __shfl_xor(part, m, VK_WAVE);
      const float rr = rsqrtf(part / (float)d + a.eps);
      float wv[VK_VEC];
      if (a.w_is_f32) {
#pragma unroll
        for (int e = 0; e < VK_VEC; ++e) wv[e] = static_cast<const float*>(w)[j * VK_VEC + e];
      } else {
        load_elems(static_cast<const elem_t*>(w) + j * VK_VEC, wv);
      }
#pragma unroll
      for (int e = 0; e < VK_VEC; ++e) xv[e] = round_to_elem((xv[e] * rr) * wv[e]);
    }
    if (a.cos_t != nullptr) {
      // The partner of element c is c +- d/2: the same place in the lane LPH/2 away.  Every lane takes
      // part in the exchange, also those of v heads, which keep their values.
      float other[VK_VEC], cs[VK_VEC], sn[VK_VEC];
#pragma unroll
      for (int e = 0; e < VK_VEC; ++e) other[e] = __shfl_xor(xv[e], LPH / 2, VK_WAVE);
      const int tcol = (j % (LPH / 2)) * VK_VEC;
      load_elems(a.cos_t + trow + tcol, cs);
      load_elems(a.sin_t + trow + tcol, sn);
      if (kind != 2) {
        if (j < LPH / 2) {
#pragma unroll
          for (int e = 0; e < VK_VEC; ++e) xv[e] = xv[e] * cs[e] - other[e] * sn[e];
        } else {
#pragma unroll
          for (int e = 0; e < VK_VEC; ++e) xv[e] = xv[e] * cs[e] + other[e] * sn[e];
        }
      }
    }
    if (!live) continue;
    if (kind == 0) {
      store_elems(a.q_out + ((int64_t)tok * a.nq + hh) * d + j * VK_VEC, xv);
    } else if (slot >= 0) {
      if (kind == 1) {
        store_elems(a.kc + (((int64_t)page * a.nkv + (hh - a.nq)) * a.P + off) * d + j * VK_VEC, xv);
      } else {
        elem_t* o = a.vc + (((int64_t)page * a.nkv + (hh - a.nq - a.nkv)) * d + j * VK_VEC) * a.P + off;
#pragma unroll
        for (int e = 0; e < VK_VEC; ++e) o[(int64_t)e * a.P] = from_f32<elem_t>(xv[e]);
      }
    }
  }
}

extern "C" {

// Null q_w / k_w: no norm for that kind.  Null cos_t: no rotation.  nkv == 0:
// only q rows (a plain norm and/or rotation of [T, nq, d]).  nq == 0: only the
// store.  Positions must lie below the tables' row count and slots inside the
// cache; the caller checks both on the host before the upload.
int vk_qkv_post(const elem_t* qkv, int64_t row_stride, elem_t* q_out, elem_t* kc, elem_t* vc, const void* q_w,
                const void* k_w, int w_is_f32, const elem_t* cos_t, const elem_t* sin_t, int rot_half,
                const int32_t* positions, const int32_t* slots, int T, int nq, int nkv, int d, int P, float eps,
                hipStream_t st) {
  VK_REQUIRE(T >= 0 && nq >= 0 && nkv >= 0 && nq + nkv > 0, "qkv_post: bad sizes T=%d nq=%d nkv=%d", T, nq, nkv);
  VK_REQUIRE(d > 0 && d <= 256, "qkv_post: head size %d must be in 1..256", d);
  VK_REQUIRE(row_stride >= (int64_t)(nq + 2 * nkv) * d, "qkv_post: row stride %lld too small", (long long)row_stride);
  VK_REQUIRE(cos_t == nullptr || (rot_half > 0 && 2 * rot_half <= d), "qkv_post: rotary width %d does not fit head size %d",
             2 * rot_half, d);
  VK_REQUIRE(cos_t == nullptr || positions != nullptr, "qkv_post: rotation needs positions");
  VK_REQUIRE(nkv == 0 || (slots != nullptr && kc != nullptr && vc != nullptr && P > 0), "qkv_post: store needs slots and caches");
  VK_REQUIRE(nq + 2 * nkv <= 65535, "qkv_post: too many heads");
  if (T == 0) return 0;
  QkvPostArgs a;
  a.qkv = qkv; a.row_stride = row_stride; a.q_out = q_out; a.kc = kc; a.vc = vc; a.q_w = q_w; a.k_w = k_w;
  a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.slots = slots; a.w_is_f32 = w_is_f32;
  a.nq = nq; a.nkv = nkv; a.d = d; a.P = P; a.rot_half = rot_half; a.eps = eps;
  // Few tokens: four waves' worth of heads per workgroup, for many workgroups; many tokens: all heads of a token.
  const int heads = nq + 2 * nkv;
  const int lph = d / VK_VEC;          // lanes per head in the kernel with 16-byte accesses
  const bool vec = (d == 64 || d == 128 || d == 256) && lph <= 64 && (cos_t == nullptr || 2 * rot_half == d) &&
                   row_stride % VK_VEC == 0 && ((uintptr_t)qkv % 16) == 0 && (q_out == nullptr || (uintptr_t)q_out % 16 == 0) &&
                   (kc == nullptr || (uintptr_t)kc % 16 == 0) && (cos_t == nullptr || ((uintptr_t)cos_t % 16 == 0 && (uintptr_t)sin_t % 16 == 0));
  if (vec) {
    const int hpw = 64 / lph, per_wg = 4 * hpw;
    const int per_wave = T >= 512 ? (heads + per_wg - 1) / per_wg : 1;
    const dim3 grid(T, (heads + per_wg * per_wave - 1) / (per_wg * per_wave));
    if (lph == 8) qkv_post_vec_kernel<8><<<grid, 256, 0, st>>>(a, per_wave);
    else if (lph == 16) qkv_post_vec_kernel<16><<<grid, 256, 0, st>>>(a, per_wave);
    else if (lph == 32) qkv_post_vec_kernel<32><<<grid, 256, 0, st>>>(a, per_wave);
    else qkv_post_vec_kernel<64><<<grid, 256, 0, st>>>(a, per_wave);
    return vk_check_launch("qkv_post");
  }
  const int per_wave = T >= 512 ? (heads + 3) / 4 : 1;
  qkv_post_kernel<<<dim3(T, (heads + 4 * per_wave - 1) / (4 * per_wave)), 256, 0, st>>>(a, per_wave);
  return vk_check_launch("qkv_post");
}

}  // extern "C"
