// bfloat16 matrix products on the matrix cores (MFMA 16x16x32, 32-bit accumulation), reading
// weights in a fragment layout that is made once at load.
//
// Fragment layout of W[N, K] (bfloat16): tiles of 16 rows x 32 columns, stored tile by tile as
// [N/16][K/32][64 lanes][8 elements]; lane l = g*16 + r of a tile holds W[n0 + r][k0 + 8g .. 8g+7],
// which is exactly what lane l supplies to the MFMA as its part of the 16x32 operand.  A wave
// therefore loads a whole tile with one fully coalesced 1 KB read and no shuffle through LDS.
// N is padded to a multiple of 16 and K to a multiple of 32 with zeros.
//
// Operand roles: the weight tile is the MFMA's first operand (rows = output features n), the
// activations the second (columns = tokens m).  Lane l then holds D[n = 4*(l/16) + i][m = l%16],
// i = 0..3: four consecutive output features of one token, stored with one vector store.
//
// Two kernels share this: a weight-streaming kernel for up to 64 tokens (decode), whose four waves
// split the inner dimension and add their parts in a fixed order, and a tiled kernel for many
// tokens (prompts).  The math is the reference's y[r] = sum_c W[r,c] x[c] (gguf.rs:4063-4074) with the
// GeGLU (llama3.rs:14519-14534) and softcap (llama3.rs:14606-14611) epilogues.
//
// This header holds what the kernels' source files share: the operand types, the stores, and the rotation epilogue's
// helpers.  linear_mfma_stream.hip has the streaming kernel, linear_mfma_tiled.hip the tiled one, linear_mfma.hip the
// entry points; each is compiled on its own, which halves the time of a build.
#pragma once
#include "common.h"
#include "alice_hip.h"
#include "kv_layout.h"

// What the rotation epilogue needs: where q goes, the cache, the tables and the geometry.
struct RopeArgs {
  bf16_t* q_out;
  bf16_t* k_pool;
  bf16_t* v_pool;
  const float* cos_t;
  const float* sin_t;
  const int* positions;
  const int* seq_of_token;
  const int* block_table;
  int bt_stride, nH, nKV, d, page_size, n_pages, layout;
};

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// A weight fragment of zeros: k-tiles beyond a slice read it instead of the matrix, so that every load of
// the main loops is unconditional and nothing has to be patched after a load.
// (Not declared const: that would put it into the constant address space, and a pointer that may point
// into either space is dereferenced with the slower flat loads.)
static __device__ __align__(16) uint32_t g_zero_tile[256];

__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

// The activation fragment of token row `m` (clamped by the caller) at k-tile kt: 8 consecutive elements.
__device__ __forceinline__ u32x4 load_x_frag(const bf16_t* __restrict__ x, int row, bool row_ok, int K, int kt, int g) {
  const int k = kt * 32 + g * 8;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row_ok && k < K) v = *reinterpret_cast<const u32x4*>(x + (size_t)row * K + k);
  return v;
}

// The same fragment when the activations themselves are stored in fragment order
// ([M/16][K/32][64 lanes][8], what a decode step's producers write): one contiguous 1 KB read per wave.
__device__ __forceinline__ u32x4 load_x_frag_f(const bf16_t* __restrict__ x, int mtile, bool ok, int KT, int kt, int lane) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (ok) v = *reinterpret_cast<const u32x4*>(x + ((size_t)((size_t)mtile * KT + kt) * 64 + lane) * 8);
  return v;
}

template <int EPI, bool FULL>
__device__ __forceinline__ float epilogue1(float v, float p) {
  if (EPI == ALICE_EPI_SOFTCAP) return p * (FULL ? tanh_full(v / p) : tanh_fast(v / p));
  return v;
}

template <typename TO>
__device__ __forceinline__ void store4(TO* __restrict__ y, size_t row_off, int n, int N, f32x4 v) {
  if (n + 3 < N && (((size_t)row_off + n) & 3) == 0) {
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<f32x4*>((float*)y + row_off + n) = v;
    } else {
      uint32_t lo = pack_bf16x2(v[0], v[1]);
      uint32_t hi = pack_bf16x2(v[2], v[3]);
      uint2 pk = {lo, hi};
      *reinterpret_cast<uint2*>((bf16_t*)y + row_off + n) = pk;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) store_f32(y, row_off + n + i, v[i]);
  }
}

// Four consecutive output features of token m, stored in fragment order for the next matrix product
// (its inner dimension is this one's N): element (m, n) lies at
// ((m/16 * N/32 + n/32) * 64 + (n%32)/8 * 16 + m%16) * 8 + n%8.  N is a multiple of 32, n of 4.
__device__ __forceinline__ void store4_frag(bf16_t* __restrict__ y, int m, int n, int N, f32x4 v) {
  const size_t off = ((size_t)((size_t)(m >> 4) * (N >> 5) + (n >> 5)) * 64 + ((n & 31) >> 3) * 16 + (m & 15)) * 8 + (n & 7);
  uint2 pk = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  *reinterpret_cast<uint2*>(y + off) = pk;
}

// Row-major, or (bfloat16 only) fragment order.
template <typename TO>
__device__ __forceinline__ void store4_any(TO* __restrict__ y, int y_frag, int m, size_t row_off, int n, int N, f32x4 v) {
  if constexpr (sizeof(TO) == 2) {
    if (y_frag) { store4_frag((bf16_t*)y, m, n, N, v); return; }
  }
  store4(y, row_off, n, N, v);
}

// A token as the tiled kernel's rotation epilogue keeps it in LDS, and the elements per staged token there: 256
// features and 8 of padding (a token's stride is 132 words, so that neither 64 lanes on 16 tokens x 4 words nor 16
// tokens x 16 bytes meet in a bank).
struct RopeStagedToken {
  size_t page_base;
  int tp;
  bool valid, page_ok;
};
constexpr int ROPE_PITCH = 264;

// Where token m's keys and values go.
struct RopeToken {
  int pos, tp;
  bool page_ok;
  size_t page_base;
};
__device__ __forceinline__ RopeToken rope_token(const RopeArgs& ra, int m) {
  RopeToken t;
  t.pos = ra.positions[m];
  t.tp = t.pos % ra.page_size;
  const int page = ra.block_table[(size_t)ra.seq_of_token[m] * ra.bt_stride + t.pos / ra.page_size];
  t.page_ok = page >= 0 && page < ra.n_pages;
  t.page_base = (size_t)(t.page_ok ? page : 0) * ra.nKV * ra.page_size * ra.d;
  return t;
}
// The rotation epilogue for four consecutive output features n .. n+3 (in W's row order) of token m.  The
// rows of W are all q heads, all k heads, all v heads, the rows of every q and k head in pair order: the four
// features are two whole rotated pairs (or four elements of a value head).  The sums are rounded to bfloat16
// before the rotation, as they are when the projection and the rotation are separate kernels: both ways give
// the same bits.
// Which head features n .. n+3 belong to and where in it they lie: the same for every token of a tile, so the
// divisions by the head size are done once per tile, not per token.
struct RopeCol { int head, w; };
__device__ __forceinline__ RopeCol rope_col(const RopeArgs& ra, int n) { return RopeCol{n / ra.d, n % ra.d}; }

// The cosines and sines of the two pairs that the four features make (nothing for a value head).
struct RopeTrig { float2 c, s; };
__device__ __forceinline__ RopeTrig rope_trig(const RopeArgs& ra, const RopeToken& t, const RopeCol& col) {
  RopeTrig g{float2{1.f, 1.f}, float2{0.f, 0.f}};
  if (col.head < ra.nH + ra.nKV) {
    g.c = *reinterpret_cast<const float2*>(ra.cos_t + (size_t)t.pos * (ra.d >> 1) + (col.w >> 1));
    g.s = *reinterpret_cast<const float2*>(ra.sin_t + (size_t)t.pos * (ra.d >> 1) + (col.w >> 1));
  }
  return g;
}
__device__ __forceinline__ void rope_store4(const RopeArgs& ra, int m, const RopeToken& t, const RopeCol& col, f32x4 acc,
                                            const RopeTrig& tr) {
  const int d = ra.d, half = d >> 1;
  const int head = col.head, w = col.w;
  float x[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = round_to<bf16_t>(acc[e]);
  if (head < ra.nH + ra.nKV) {
    const int p0 = w >> 1;                                 // the pairs p0 and p0 + 1 of the head
    float l0, h0, l1, h1;
    rotate_pair(x[0], x[1], tr.c.x, tr.s.x, l0, h0);
    rotate_pair(x[2], x[3], tr.c.y, tr.s.y, l1, h1);
    const uint32_t lo = pack_bf16x2(l0, l1), hi = pack_bf16x2(h0, h1);
    if (head < ra.nH) {
      bf16_t* dst = ra.q_out + ((size_t)m * ra.nH + head) * d;
      *reinterpret_cast<uint32_t*>(dst + p0) = lo;
      *reinterpret_cast<uint32_t*>(dst + p0 + half) = hi;
    } else if (t.page_ok) {
      bf16_t* dst = ra.k_pool + t.page_base + (size_t)(head - ra.nH) * ra.page_size * d;
      *reinterpret_cast<uint32_t*>(dst + k_offset(ra.layout, t.tp, p0, d)) = lo;
      *reinterpret_cast<uint32_t*>(dst + k_offset(ra.layout, t.tp, p0 + half, d)) = hi;
    }
  } else if (t.page_ok) {
    bf16_t* dst = ra.v_pool + t.page_base + (size_t)(head - ra.nH - ra.nKV) * ra.page_size * d;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[v_offset(ra.layout, t.tp, w + e, d)] = f32_to_bf16(x[e]);
  }
}
__device__ __forceinline__ void rope_store4(const RopeArgs& ra, int m, const RopeToken& t, int n, f32x4 acc) {
  const RopeCol col = rope_col(ra, n);
  rope_store4(ra, m, t, col, acc, rope_trig(ra, t, col));
}

}  // namespace

// ---- what the source files of the matrix-core products call in each other
// The streaming kernel (at most 64 tokens): plain, GeGLU or softcap epilogue by `epi`, float32 or bfloat16 output.
int alice_mfma_stream(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                      int split, int x_frag, int y_frag, hipStream_t s);
// The same with the rotation and the cache write as its epilogue.
int alice_mfma_stream_rope(const void* x, const void* w, int M, int N, int K, int x_frag, hipStream_t s, const RopeArgs& ra);
// The tiled kernel (many tokens), and with the rotation epilogue.  force_wn 1 or 2: the wave tile of 16 or 32
// features whatever the cost rule says (0: the rule's choice).
int alice_mfma_tiled(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                     int split, int x_frag, int y_frag, int force_wn, hipStream_t s);
int alice_mfma_tiled_rope(const void* x, const void* w, int M, int N, int K, int x_frag, hipStream_t s, const RopeArgs& ra);
// The tiled kernel's tile: a wave's 16 wn output features x 16 tm tokens, kc k-tiles a stage, slices of the inner
// dimension.  split 0: the rule chooses the slices too (float32 sums without epilogue only), else they are given.
// Up to 64 tokens wn is 0 where the streaming kernel is the better one (always up to 32).
struct TiledPlan { int wn, tm, kc, split; };
TiledPlan alice_mfma_tiled_plan(int M, int N, int K, int epi, int y_dtype, int split, int x_frag);
int alice_mfma_tiled_narrow(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                            const TiledPlan& p, int y_frag, hipStream_t s, const RopeArgs& ra);
// The streaming kernel's choice of row tiles a block and what the launcher's cost rule says of a choice.
int alice_mfma_stream_row_tiles(int M, int N, int epi, int split, int K);
int alice_mfma_stream_row_tiles_base(int M, int N, int epi, int split, int K);
float alice_mfma_stream_cost(int M, int N, int K, int epi, int rt, int split);

// Calls FN<epilogue, output type>(...) for the run-time epilogue and output dtype.
#define ALICE_MFMA_BY_EPI(FN, ...)                                                                 \
  do {                                                                                             \
    if (y_dtype == DT_F32) {                                                                       \
      if (epi == ALICE_EPI_NONE) return FN<ALICE_EPI_NONE, float>(__VA_ARGS__);                    \
      if (epi == ALICE_EPI_GEGLU) return FN<ALICE_EPI_GEGLU, float>(__VA_ARGS__);                  \
      return FN<ALICE_EPI_SOFTCAP, float>(__VA_ARGS__);                                            \
    } else {                                                                                       \
      if (epi == ALICE_EPI_NONE) return FN<ALICE_EPI_NONE, bf16_t>(__VA_ARGS__);                   \
      if (epi == ALICE_EPI_GEGLU) return FN<ALICE_EPI_GEGLU, bf16_t>(__VA_ARGS__);                 \
      return FN<ALICE_EPI_SOFTCAP, bf16_t>(__VA_ARGS__);                                           \
    }                                                                                              \
  } while (0)
