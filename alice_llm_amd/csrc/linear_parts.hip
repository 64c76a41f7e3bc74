// The output projection of single-token attention with the combine of the key splits as its prologue: the
// attention kernel leaves, per (sequence, head, split), a maximum, a sum and an unnormalised output
// (attention_mfma.hip); combining them is a kernel of its own that reads and writes a few KB and costs a step of
// 26 layers as much as the projection itself.  Here every block of the projection combines what it needs by
// itself.  The inner dimension is cut into slices of at most 32 k-tiles, a block takes one slice of 64, 128 or 256
// output features, so it needs the combined output of a few heads of at most 16 sequences: it reads those parts
// (from the L2, where the attention kernel's blocks left them), scales and sums them in the order of the splits as
// the combine kernel does, rounds to bfloat16 and keeps them in LDS in fragment order; its first weight tiles are
// on their way meanwhile.  The sums over a slice go to
// y[slice][M][N] in float32, which the fused add + norm adds up (llama3.rs:5688-5700 for the projection).
#include "linear_mfma.h"

namespace {

constexpr int PARTS_MAX_TILES = 32;   // k-tiles a slice
constexpr int PARTS_MAX_SLICES = 16;  // slices of the inner dimension: each is a partial result that the add + norm sums
constexpr int PARTS_U = 8;            // weight k-tiles in flight per wave

__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }

template <int WN, int SR>
__global__ __launch_bounds__(256) void linear_parts_kernel(const float* __restrict__ parts, const bf16_t* __restrict__ wf,
                                                         float* __restrict__ y, int M, int N, int KT, int NT, int per,
                                                         int S, int D, int nH) {
  __shared__ __align__(16) u32x4 xs[PARTS_MAX_TILES * 64];             // the slice's activations, one token tile
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int kt0 = blockIdx.y * per;                                    // the slice's first k-tile
  const int k0 = kt0 * 32;
  int tile[WN];
  const bf16_t* wsrc[WN];
#pragma unroll
  for (int i = 0; i < WN; ++i) {
    tile[i] = (blockIdx.x * 4 + wave) * WN + i;
    wsrc[i] = wf + ((size_t)min(tile[i], NT - 1) * KT + kt0) * 512 + lane * 8;
  }
  // the first weight tiles: they come from memory, everything below from the L2
  u32x4 wk[PARTS_U][WN];
#pragma unroll
  for (int u = 0; u < PARTS_U; ++u)
#pragma unroll
    for (int i = 0; i < WN; ++i) wk[u][i] = *reinterpret_cast<const u32x4*>(wsrc[i] + (size_t)min(u, per - 1) * 512);
  __builtin_amdgcn_sched_barrier(0);

  // ---- the combined output of the slice: an item is eight consecutive features of one token.  A thread works
  // out the weights of its token's splits itself (the 32 threads of a token and head read the same maxima and sums),
  // so nothing but the loads stands between the kernel's start and the product; they are all in flight at once
  // (at most SR splits: with more, which single sequences at long contexts have, the combine stays a kernel).
  const size_t pstride = (size_t)(D + ALICE_ATTN_PARTS_HEAD);
  const int chunks = per * 4;
  for (int it = threadIdx.x; it < 16 * chunks; it += 256) {
    const int m = it / chunks, c = it % chunks;
    u32x4 packed = {0u, 0u, 0u, 0u};
    if (m < M) {
      const int k = k0 + c * 8, e0 = k % D;
      const float* pr = parts + ((size_t)m * nH + k / D) * S * pstride;
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      float ll = 0.f;
      float2 ml[SR];
      float4 v[SR][2];
#pragma unroll
      for (int q = 0; q < SR; ++q) {
        const float* src = pr + (size_t)min(q, S - 1) * pstride;
        ml[q] = *reinterpret_cast<const float2*>(src);
#pragma unroll
        for (int j = 0; j < 2; ++j) v[q][j] = *reinterpret_cast<const float4*>(src + ALICE_ATTN_PARTS_HEAD + e0 + 4 * j);
      }
      float mm = -INFINITY;
#pragma unroll
      for (int q = 0; q < SR; ++q) mm = fmaxf(mm, ml[q].x);
#pragma unroll
      for (int q = 0; q < SR; ++q) {
        const float f = (q < S && ml[q].x != -INFINITY) ? exp2_hw(ml[q].x - mm) : 0.f;
        ll += ml[q].y * f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          acc[4 * j] += v[q][j].x * f;
          acc[4 * j + 1] += v[q][j].y * f;
          acc[4 * j + 2] += v[q][j].z * f;
          acc[4 * j + 3] += v[q][j].w * f;
        }
      }
      const float sc = 1.f / ll;
#pragma unroll
      for (int j = 0; j < 4; ++j) packed[j] = pack_bf16x2(acc[2 * j] * sc, acc[2 * j + 1] * sc);
    }
    xs[(c >> 2) * 64 + (c & 3) * 16 + m] = packed;                     // k-tile c / 4, lane (c % 4) * 16 + m
  }
  __syncthreads();

  // ---- the product
  f32x4 acc[WN];
#pragma unroll
  for (int i = 0; i < WN; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int t0 = 0; t0 < per; t0 += PARTS_U) {
#pragma unroll
    for (int u = 0; u < PARTS_U; ++u) {
      const int t = t0 + u;
      if (t < per) {                                                   // the same for the whole block
        const u32x4 b = xs[t * 64 + lane];
#pragma unroll
        for (int i = 0; i < WN; ++i) acc[i] = mfma16(wk[u][i], b, acc[i]);
        if (t + PARTS_U < per) {
#pragma unroll
          for (int i = 0; i < WN; ++i) wk[u][i] = *reinterpret_cast<const u32x4*>(wsrc[i] + (size_t)(t + PARTS_U) * 512);
        }
      }
    }
  }
  if (r >= M) return;
  const size_t row_off = ((size_t)blockIdx.y * M + r) * N;
#pragma unroll
  for (int i = 0; i < WN; ++i)
    if (tile[i] < NT) store4(y, row_off, tile[i] * 16 + g * 4, N, acc[i]);
}

// Slices and tile for M tokens: at most PARTS_MAX_SLICES slices of whole k-tiles, at most PARTS_MAX_TILES of them,
// whose k-tiles lie in one head each (a head size of a multiple of 32); inner dimensions that this does not cover
// (beyond 16,384) are not taken.  Among the choices with at least three quarters of the most blocks
// that fit the chip once (256), the cheapest by what grows with them: every slice is one more partial result for the
// add + norm that follows (about 0.12 us), and every block reads its slice's parts anew (about 64 KB a microsecond).
struct PartsPlan { int wn, split; };
PartsPlan parts_plan(int M, int N, int nH, int D, int S) {
  PartsPlan none{0, 0};
  const int K = nH * D;
  if (M < 1 || M > 16 || S < 2 || S > 16 || D % 32 != 0 || N < 1) return none;
  const int KT = K / 32, NT = ceil_div(N, 16);
  int most = 0;
  for (int pass = 0; pass < 2; ++pass) {
    PartsPlan best = none;
    float best_cost = 1e30f;
    for (int split = 1; split <= KT; ++split) {
      if (KT % split != 0 || KT / split > PARTS_MAX_TILES || split > PARTS_MAX_SLICES) continue;
      for (int wn = 4; wn >= 1; wn >>= 1) {
        const int b = ceil_div(NT, 4 * wn) * split;
        if (b > 256) continue;
        if (pass == 0) { most = b > most ? b : most; continue; }
        if (4 * b < 3 * most) continue;
        const float cost = split * 0.12f + (float)M * S * (K / split + ALICE_ATTN_PARTS_HEAD * nH / (float)split) * 4.f / 65536.f;
        if (cost < best_cost) { best_cost = cost; best = PartsPlan{wn, split}; }
      }
    }
    if (pass == 1) return best;
  }
  return none;
}

}  // namespace

// The number of slices of the inner dimension (the first dimension of y) that alice_linear_parts uses for these
// sizes, or 0 where it does not cover them (the caller then combines the splits and projects separately).
extern "C" int alice_linear_parts_split(int M, int N, int nH, int d, int splits) { return parts_plan(M, N, nH, d, splits).split; }

extern "C" int alice_linear_parts(const float* parts, int splits, int nH, int d, const void* w, float* y, int M, int N,
                                  hipStream_t stream) {
  ALICE_CHECK(parts && w && y, "linear (attention parts): a pointer is missing");
  const PartsPlan p = parts_plan(M, N, nH, d, splits);
  ALICE_CHECK(p.split > 0, "linear (attention parts): %d tokens, %d heads of %d, %d splits and %d output features are not covered", M, nH, d, splits, N);
  ALICE_CHECK(((uintptr_t)parts & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0, "linear (attention parts): operands are not aligned");
  const int KT = nH * d / 32, NT = ceil_div(N, 16), per = KT / p.split;
  dim3 grid(ceil_div(NT, 4 * p.wn), p.split);
#define GO(WNV)                                                                                                       \
  do {                                                                                                                \
    if (splits <= 8) linear_parts_kernel<WNV, 8><<<grid, 256, 0, stream>>>(parts, (const bf16_t*)w, y, M, N, KT, NT, per, splits, d, nH); \
    else linear_parts_kernel<WNV, 16><<<grid, 256, 0, stream>>>(parts, (const bf16_t*)w, y, M, N, KT, NT, per, splits, d, nH); \
  } while (0)
  if (p.wn == 4) GO(4); else if (p.wn == 2) GO(2); else GO(1);
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}
