// Shared definitions of the gfx950 kernel library.
//
// The library is compiled twice from the same sources: once with -DVK_BF16
// (elements are bfloat16, the serving precision) and once with -DVK_F32
// (elements are float: the true 32-bit path, which uses fp32 MFMA and rounds
// nothing to a shorter type).  Both builds export the same C symbols.
//
// Every reduction in these kernels has an order that is a function of the
// model's sizes only, never of the number of rows in a launch or of which rows
// share a tile, so a row of a batch is bit-identical to the same row alone.
// All sources are compiled with -ffp-contract=off: a fused multiply-add
// appears only where __builtin_fmaf is written.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#if defined(VK_F32) == defined(VK_BF16)
#error "compile with exactly one of -DVK_BF16 or -DVK_F32"
#endif

#ifdef VK_F32
typedef float elem_t;
#define VK_ELEM_BYTES 4
#else
typedef __bf16 elem_t;
#define VK_ELEM_BYTES 2
#endif

#define VK_WAVE 64

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__bf16 x) { return (float)x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
// Round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
template <> __device__ __forceinline__ __bf16 from_f32<__bf16>(float x) { return (__bf16)x; }

// The value an element-typed store would hold, as a float.
__device__ __forceinline__ float round_to_elem(float x) { return to_f32(from_f32<elem_t>(x)); }

__device__ __forceinline__ float wave_sum_xor(float v) {
  // Butterfly: every lane ends with the same value; the order of the additions
  // is fixed by the lane pattern.
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, VK_WAVE);
  return v;
}

// The values of lanes l ^ 16 and l ^ 32 (what __shfl_xor gives), through the row and half swaps of
// gfx950, which stay in the vector unit instead of going through LDS.
__device__ __forceinline__ float lane_xor16(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  // Rows of 16 lanes r0 r1 r2 r3: the swap leaves (r0 r0 r2 r2, r1 r1 r3 r3).
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 16) ? r[0] : r[1]);
}
__device__ __forceinline__ float lane_xor32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  // Halves h0 h1: the swap leaves (h0 h0, h1 h1).
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}

__device__ __forceinline__ float wave_max_xor(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, VK_WAVE));
  return v;
}

// Host side -----------------------------------------------------------------
#ifdef __cplusplus
extern "C" {
#endif
// Text of the last error on this thread ("" if none).
const char* vk_last_error(void);
#ifdef __cplusplus
}
#endif

int vk_fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int vk_check_launch(const char* what);

#define VK_REQUIRE(cond, ...)             \
  do {                                    \
    if (!(cond)) return vk_fail(__VA_ARGS__); \
  } while (0)
