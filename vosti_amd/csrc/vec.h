// Vector loads and stores of elements, widened to float in registers.
#pragma once
#include "common.h"

// Number of elements in a 16-byte vector.
#ifdef VK_F32
#define VK_VEC 4
#else
#define VK_VEC 8
#endif

#ifdef VK_F32
__device__ __forceinline__ void load_elems(const elem_t* p, float (&out)[4]) {
  f32x4 v = *reinterpret_cast<const f32x4*>(p);
  out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
}
__device__ __forceinline__ void store_elems(elem_t* p, const float (&in)[4]) {
  f32x4 v = {in[0], in[1], in[2], in[3]};
  *reinterpret_cast<f32x4*>(p) = v;
}
#else
__device__ __forceinline__ void load_elems(const elem_t* p, float (&out)[8]) {
  bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = (float)v[i];
}
__device__ __forceinline__ void store_elems(elem_t* p, const float (&in)[8]) {
  bf16x8 v;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (__bf16)in[i];
  *reinterpret_cast<bf16x8*>(p) = v;
}
#endif

__device__ __forceinline__ void load_elems(const elem_t* p, float (&out)[1]) { out[0] = to_f32(p[0]); }
__device__ __forceinline__ void store_elems(elem_t* p, const float (&in)[1]) { p[0] = from_f32<elem_t>(in[0]); }

// Norm weights may be stored as elements or as float.
__device__ __forceinline__ float load_weight(const void* w, int is_f32, int i) {
  return is_f32 ? reinterpret_cast<const float*>(w)[i] : to_f32(reinterpret_cast<const elem_t*>(w)[i]);
}
