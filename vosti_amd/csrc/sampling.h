// Exported entry points of the sampler (sampling.hip).  The same names exist in both builds of the
// library; ``elem_t`` is bfloat16 (2 bytes) or float.
#pragma once
#include "common.h"

#ifdef __cplusplus
extern "C" {
#endif

// Words (4 bytes each) of scratch that vk_sample needs for R rows.
int vk_sample_scratch_words(int R);

// out[r] = token of logits row r: argmax (first index on ties, a NaN counts as the maximum), or, where
// temps[r] > 0, a draw from softmax(logits / temps[r]) by inverse CDF with the uniform number
// uniforms[r].  temps null: greedy for every row.  scratch: vk_sample_scratch_words(R) words of device
// memory that the caller brings.
int vk_sample(int32_t* out, const elem_t* logits, const float* temps, const float* uniforms, void* scratch, int R,
              int V, int64_t row_stride, hipStream_t st);

// vk_sample without the scratch argument, for callers that cannot allocate device memory: code under
// HIP graph capture, tight serving loops, harnesses that forbid it.  It has no counterpart in the
// reference.  The partial results live in an array of the library's own, VK_SAMPLE_STATIC_MAX_ROWS * 256 bytes per GPU
// (256 KB), held from the first call on that GPU until the process ends; the call allocates and frees
// nothing.  More rows than VK_SAMPLE_STATIC_MAX_ROWS are refused with an error.  Every call on a GPU
// uses that GPU's one array: calls that overlap on one GPU (two streams, two host threads) race and
// may return wrong tokens; calls on one stream, or ordered by events, are safe.  Nothing in the array
// has to be cleared between calls.  The result is vk_sample's, bit for bit.
#define VK_SAMPLE_STATIC_MAX_ROWS 1024
int vk_sample_static_max_rows(void);
int vk_sample_static(int32_t* out, const elem_t* logits, const float* temps, const float* uniforms, int R, int V,
                     int64_t row_stride, hipStream_t st);

#ifdef __cplusplus
}
#endif
