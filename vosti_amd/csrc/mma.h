// MFMA building blocks shared by the GEMM and attention kernels.
//
// A "slab" is 64 bytes of one row along the reduction axis: 32 bfloat16 or 16
// float.  In a 16-row operand tile, lane l holds the 16 bytes at byte offset
// 16*(l/16) of row l%16 of the slab.  mma_slab() multiplies a [16 x slab] tile
// by a [16 x slab] tile (both row-major along the reduction axis) and adds the
// [16 x 16] product to the accumulator.
//
// bfloat16: one v_mfma_f32_16x16x32_bf16; lane l supplies reduction indices
//           8*(l/16) .. 8*(l/16)+7.
// float:    four v_mfma_f32_16x16x4_f32 (true fp32 multiply-add); MFMA j takes
//           element j of every lane's four floats, i.e. reduction indices
//           {4*g + j : g = 0..3}.  The permutation is the same for both
//           operands, so the product is unchanged.
//
// Accumulator layout (both types): lane l holds rows 4*(l/16)+i, i = 0..3, of
// column l%16, where "row" indexes the first operand's rows and "column" the
// second operand's rows.
//
// Every kernel that must agree bitwise with another one reduces through
// mma_slab() with the same operand roles and the same slab order.
#pragma once
#include "common.h"

#ifdef VK_BF16
typedef bf16x8 frag_t;
#define VK_SLAB 32  // elements per slab
__device__ __forceinline__ f32x4 mma_slab(frag_t a, frag_t b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
#else
typedef f32x4 frag_t;
#define VK_SLAB 16
__device__ __forceinline__ f32x4 mma_slab(frag_t a, frag_t b, f32x4 c) {
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, c, 0, 0, 0);
  c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, c, 0, 0, 0);
  return c;
}
#endif

__device__ __forceinline__ frag_t zero_frag() {
  u32x4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(frag_t, z);
}

// 16 bytes at p if ok, else zeros.  p must be 16-byte aligned when ok.
__device__ __forceinline__ frag_t load_frag(const elem_t* p, bool ok) {
  return ok ? *reinterpret_cast<const frag_t*>(p) : zero_frag();
}
