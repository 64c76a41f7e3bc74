// Where the keys and values of a token lie inside a cache page (shared by the kernels that write the cache).
#pragma once
#include "common.h"

// Offsets of element e of the token at place t of a 64-position page of one kv head.  Layout 0 is
// row-major [position][d]; layout 1 is the fragment layout that the matrix-core attention kernels
// read (see attention_mfma.hip): keys in 16-position x 32-dim tiles, values in 32-position x 16-dim
// tiles with the positions in the order the score tiles come out of the MFMA.
__device__ __forceinline__ size_t k_offset(int layout, int t, int e, int d) {
  if (layout == 0) return (size_t)t * d + e;
  return ((size_t)((t >> 4) * (d >> 5) + (e >> 5)) * 64 + ((e & 31) >> 3) * 16 + (t & 15)) * 8 + (e & 7);
}
__device__ __forceinline__ size_t v_offset(int layout, int t, int e, int d) {
  if (layout == 0) return (size_t)t * d + e;
  const int tt = t & 31, w = tt & 15;
  return ((size_t)((t >> 5) * (d >> 4) + (e >> 4)) * 64 + (w >> 2) * 16 + (e & 15)) * 8 + ((tt >> 4) * 4 + (w & 3));
}

// The rotation of one pair, written with explicit roundings so that every kernel that rotates (the separate
// kernels for few and for many tokens, the projections' epilogue) gives the same bits.
__device__ __forceinline__ void rotate_pair(float x0, float x1, float c, float s, float& y0, float& y1) {
  y0 = fmaf(x0, c, -__fmul_rn(x1, s));
  y1 = fmaf(x0, s, __fmul_rn(x1, c));
}
