// Rotation of q and k by the position tables, and the write of k (rotated) and v into the
// paged cache, in one pass over the fused q|k|v rows.
//
// Pairing is half-split over the rotated width R: (j, j + R/2), y[j] = x[j] cos - x[j+R/2] sin,
// y[j+R/2] = x[j] sin + x[j+R/2] cos (llama3.rs:5367-5378); k is cached after the rotation and
// v as it is (llama3.rs:14307-14331).  Dimensions at or beyond R pass through unchanged.
#include "common.h"
#include "alice_hip.h"
#include "kv_layout.h"

// `interleaved`: the q and k heads of the qkv row come with the two elements of each rotated pair next to
// each other, (j, j + R/2) at 2j and 2j + 1 (the order in which a projection whose rows were permuted that
// way delivers them; only with R == d); the outputs are in the plain order either way.
// One block per token.  qkv row of row_w elements: [nH*d | nKV*d | nKV*d | ...]; with no pools
// only the q part is read.  cos/sin: [max_pos, R/2].
// Cache pools: [page][nKV][page_size][d]; the page of position p of sequence s is
// block_table[s * bt_stride + p / page_size].
template <typename T>
__global__ void rope_cache_kernel(const T* __restrict__ qkv, T* __restrict__ q_out,
                                  T* __restrict__ k_pool, T* __restrict__ v_pool,
                                  const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                  const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                  const int* __restrict__ block_table, int bt_stride, int row_w,
                                  int nH, int nKV, int d, int R, int page_size, int n_pages, int layout, int interleaved) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = R >> 1;
  const T* row = qkv + (size_t)t * row_w;
  const float* cs = cos_t ? cos_t + (size_t)pos * half : nullptr;
  const float* sn = sin_t ? sin_t + (size_t)pos * half : nullptr;

  T* kdst = nullptr;             // the page's region of kv head 0; head h adds h * page_size * d
  T* vdst = nullptr;
  const int tp = pos % page_size;  // place within the page
  if (k_pool) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    if (page >= 0 && page < n_pages) {
      const size_t base = (size_t)page * nKV * page_size * d;
      kdst = k_pool + base;
      vdst = v_pool + base;
    }
  }
  const int hd2 = d >> 1;        // work items per head: one per pair of the first/second half
  // blockIdx.y names the head this block handles: q heads, then k heads, then v heads.
  const int h = blockIdx.y;
  if (h < nH + nKV) {
    const bool is_q = h < nH;
    if (!is_q && !kdst) return;
    const T* src = row + (size_t)h * d;                     // k heads follow the q heads directly
    T* dst = is_q ? q_out + (size_t)t * nH * d + (size_t)h * d : kdst + (size_t)(h - nH) * page_size * d;
    // where element e goes: q rows are plain; k goes to its place in the page
    auto at = [&](int e) -> size_t { return is_q ? (size_t)e : k_offset(layout, tp, e, d); };
    for (int j = threadIdx.x; j < hd2; j += blockDim.x) {
      // the rotated pair (j, j + half) if j < half; elements at or beyond R pass through, spread over the items
      if (j < half) {
        float x0 = load_f32(src, interleaved ? 2 * j : j), x1 = load_f32(src, interleaved ? 2 * j + 1 : j + half);
        float c = cs ? cs[j] : 1.f, s = sn ? sn[j] : 0.f, y0, y1;
        rotate_pair(x0, x1, c, s, y0, y1);
        store_f32(dst, at(j), y0);
        store_f32(dst, at(j + half), y1);
      }
      for (int e = R + j; e < d; e += hd2) store_f32(dst, at(e), load_f32(src, e));
    }
  } else if (vdst) {
    const int hv = h - nH - nKV;
    const T* vsrc = row + (size_t)(nH + nKV + hv) * d;
    T* dst = vdst + (size_t)hv * page_size * d;
    for (int e = threadIdx.x; e < d; e += blockDim.x) dst[v_offset(layout, tp, e, d)] = vsrc[e];
  }
}

// The same for bfloat16 with the whole head rotated (R == d, d a multiple of 16), eight elements a thread:
// one block per token; an item is eight pairs (j .. j+7, j + d/2 ..) of a q or k head, or eight elements of
// a v head.  16-byte loads and stores except for values in the fragment layout, whose eight neighbours in
// memory are eight positions.
__global__ void rope_cache_vec_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out,
                                      bf16_t* __restrict__ k_pool, bf16_t* __restrict__ v_pool,
                                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                      const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                                      const int* __restrict__ block_table, int bt_stride, int row_w,
                                      int nH, int nKV, int d, int page_size, int n_pages, int layout, int interleaved) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int half = d >> 1;
  const bf16_t* row = qkv + (size_t)t * row_w;
  const float* cs = cos_t + (size_t)pos * half;
  const float* sn = sin_t + (size_t)pos * half;
  bf16_t* kdst = nullptr;
  bf16_t* vdst = nullptr;
  const int tp = pos % page_size;
  int heads = nH;
  if (k_pool) {
    const int page = block_table[(size_t)seq_of_token[t] * bt_stride + pos / page_size];
    if (page >= 0 && page < n_pages) {
      const size_t base = (size_t)page * nKV * page_size * d;
      kdst = k_pool + base;
      vdst = v_pool + base;
      heads = nH + nKV;
    }
  }
  const int per_head = half >> 3;                       // items of a rotated head
  const int rot_items = heads * per_head;
  const int v_items = vdst ? nKV * (d >> 3) : 0;
  for (int it = threadIdx.x; it < rot_items + v_items; it += blockDim.x) {
    if (it < rot_items) {
      const int h = it / per_head, j = (it % per_head) * 8;
      const bf16_t* src = row + (size_t)h * d;
      uint4 lo, hi;
      if (interleaved) {
        // pairs j .. j+7 lie at 2j .. 2j+15: even places are the first elements, odd places the second
        const uint4 a = *reinterpret_cast<const uint4*>(src + 2 * j), b = *reinterpret_cast<const uint4*>(src + 2 * j + 8);
        lo = uint4{(a.x & 0xffffu) | (a.y << 16), (a.z & 0xffffu) | (a.w << 16), (b.x & 0xffffu) | (b.y << 16), (b.z & 0xffffu) | (b.w << 16)};
        hi = uint4{(a.x >> 16) | (a.y & 0xffff0000u), (a.z >> 16) | (a.w & 0xffff0000u), (b.x >> 16) | (b.y & 0xffff0000u), (b.z >> 16) | (b.w & 0xffff0000u)};
      } else {
        lo = *reinterpret_cast<const uint4*>(src + j);
        hi = *reinterpret_cast<const uint4*>(src + j + half);
      }
      const float4 c0 = *reinterpret_cast<const float4*>(cs + j), c1 = *reinterpret_cast<const float4*>(cs + j + 4);
      const float4 s0 = *reinterpret_cast<const float4*>(sn + j), s1 = *reinterpret_cast<const float4*>(sn + j + 4);
      const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
      const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
      const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w}, hw[4] = {hi.x, hi.y, hi.z, hi.w};
      uint32_t ol[4], oh[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float a0 = bf16_bits_to_f32(lw[p] & 0xffffu), a1 = bf16_bits_to_f32(lw[p] >> 16);
        const float b0 = bf16_bits_to_f32(hw[p] & 0xffffu), b1 = bf16_bits_to_f32(hw[p] >> 16);
        float l0, h0, l1, h1;
        rotate_pair(a0, b0, c[2 * p], sv[2 * p], l0, h0);
        rotate_pair(a1, b1, c[2 * p + 1], sv[2 * p + 1], l1, h1);
        ol[p] = pack_bf16x2(l0, l1);
        oh[p] = pack_bf16x2(h0, h1);
      }
      bf16_t* dst;
      size_t o_lo, o_hi;
      if (h < nH) {
        dst = q_out + (size_t)t * nH * d + (size_t)h * d;
        o_lo = j;
        o_hi = j + half;
      } else {
        dst = kdst + (size_t)(h - nH) * page_size * d;
        o_lo = k_offset(layout, tp, j, d);
        o_hi = k_offset(layout, tp, j + half, d);
      }
      *reinterpret_cast<uint4*>(dst + o_lo) = uint4{ol[0], ol[1], ol[2], ol[3]};
      *reinterpret_cast<uint4*>(dst + o_hi) = uint4{oh[0], oh[1], oh[2], oh[3]};
    } else {
      const int vi = it - rot_items, hv = vi / (d >> 3), e = (vi % (d >> 3)) * 8;
      const bf16_t* vsrc = row + (size_t)(nH + nKV + hv) * d + e;
      bf16_t* dst = vdst + (size_t)hv * page_size * d;
      const uint4 v = *reinterpret_cast<const uint4*>(vsrc);
      if (layout == 0) {
        *reinterpret_cast<uint4*>(dst + (size_t)tp * d + e) = v;
      } else {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          dst[v_offset(layout, tp, e + 2 * p, d)].bits = (uint16_t)(w[p] & 0xffffu);
          dst[v_offset(layout, tp, e + 2 * p + 1, d)].bits = (uint16_t)(w[p] >> 16);
        }
      }
    }
  }
}

extern "C" int alice_rope_cache_write(const void* qkv, int dtype, void* q_out, void* k_pool, void* v_pool,
                                      const float* cos_t, const float* sin_t, const int* positions,
                                      const int* seq_of_token, const int* block_table, int bt_stride,
                                      int T, int row_width, int nH, int nKV, int d, int rotary_dim, int page_size,
                                      int n_pages, int kv_layout, int interleaved, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(dtype), "rope: unknown dtype %d", dtype);
  ALICE_CHECK(!interleaved || (rotary_dim == d && cos_t != nullptr), "rope: interleaved pairs need the whole head rotated");
  ALICE_CHECK(T >= 0 && nH >= 1 && nKV >= 0 && d >= 2 && d % 2 == 0, "rope: bad sizes T=%d nH=%d nKV=%d d=%d", T, nH, nKV, d);
  ALICE_CHECK(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0, "rope: rotated width %d must be even and at most head_dim %d", rotary_dim, d);
  ALICE_CHECK((cos_t == nullptr) == (sin_t == nullptr), "rope: cos and sin tables must come together");
  ALICE_CHECK(rotary_dim == 0 || cos_t != nullptr, "rope: a rotated width needs the tables");
  ALICE_CHECK((k_pool == nullptr) == (v_pool == nullptr), "rope: key and value pools must come together");
  ALICE_CHECK(k_pool == nullptr || (block_table && seq_of_token && page_size > 0 && n_pages > 0 && nKV >= 1),
              "rope: a cache write needs the block table, the token-to-sequence map and the page geometry");
  ALICE_CHECK(nH + 2 * nKV <= 65535, "rope: too many heads for one launch");
  ALICE_CHECK(row_width >= (nH + (k_pool ? 2 * nKV : 0)) * d, "rope: rows of %d elements are too short for the heads", row_width);
  ALICE_CHECK(kv_layout == 0 || (kv_layout == 1 && page_size == 64 && d % 32 == 0 && dtype == DT_BF16) || k_pool == nullptr,
              "rope: the fragment cache layout needs bfloat16, pages of 64 and head_dim %% 32 == 0");
  if (T == 0) return 0;
  // Many tokens: the vector kernel (a block per token).  Few: a block per token and head has more in flight.
  if (T >= 256 && dtype == DT_BF16 && rotary_dim == d && d % 16 == 0 && row_width % 8 == 0 && cos_t != nullptr &&
      ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)q_out & 15) == 0 && ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0 &&
      (k_pool == nullptr || (((uintptr_t)k_pool & 15) == 0 && ((uintptr_t)v_pool & 15) == 0))) {
    const int items = (nH + nKV) * (d / 16) + nKV * (d / 8);
    const int threads = items >= 256 ? 256 : (items >= 128 ? 128 : 64);
    rope_cache_vec_kernel<<<T, threads, 0, stream>>>((const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_pool, (bf16_t*)v_pool,
        cos_t, sin_t, positions, seq_of_token, block_table, bt_stride, row_width, nH, nKV, d, page_size, n_pages, kv_layout, interleaved);
    ALICE_LAUNCH_CHECK();
    return 0;
  }
  DISPATCH_DTYPE(dtype, TT, (rope_cache_kernel<TT><<<dim3(T, nH + (k_pool ? 2 * nKV : 0)), d >= 256 ? 128 : 64, 0, stream>>>(
      (const TT*)qkv, (TT*)q_out, (TT*)k_pool, (TT*)v_pool, cos_t, sin_t, positions, seq_of_token,
      block_table, bt_stride, row_width, nH, nKV, d, rotary_dim, page_size, n_pages, kv_layout, interleaved)));
  ALICE_LAUNCH_CHECK();
  return 0;
}
