// The weight-streaming matrix product for up to 64 tokens (decode steps) on the matrix cores: the kernel, its launcher
// and the launcher's rules.  The layouts and the operand roles are described in linear_mfma.h.  y[r] = sum_c W[r,c] x[c]
// (gguf.rs:4063-4074) with the GeGLU (llama3.rs:14519-14534), softcap (llama3.rs:14606-14611) and rotation
// (llama3.rs:5367-5378) epilogues.  Included by one source file per epilogue (linear_mfma_stream_*.hip), so that the
// epilogues' instantiations compile side by side.
#pragma once
#include "linear_mfma.h"

namespace {

// ---------------------------------------------------------------- weight streaming, M <= 16*MT
// Block: NW waves on the same RT row tiles; wave w takes k-tiles kb + w, kb + w + NW, ...; the parts of
// waves 1.. go through LDS and wave 0 adds them in the order 1, 2, 3, ....  grid.x: groups of RT row
// tiles (for GeGLU: RT/2 gate tiles and the RT/2 up tiles that belong to them); grid.y: slices of the
// inner dimension, each writing its own partial sum y[slice][M][N] (slices > 1 only without epilogue).
//
// Every load of the main loop is unconditional: addresses beyond the matrix or the slice are clamped to
// valid ones and what they bring is replaced by zeros (weights) or lands in output columns that are never
// stored (tokens beyond M).  Only then does the compiler know how many loads are in flight and wait for the
// oldest alone (s_waitcnt vmcnt(n)); a load under a branch makes it wait for all of them.
template <int RT, int MT, int NW, int EPI, typename TO, bool FULL, bool XF, bool STREAM = false, int WINDOW = 0>
__global__ __launch_bounds__(NW * 64) void linear_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wf,
                                                            TO* __restrict__ y, int M, int N, int K, int KT, int NT,
                                                            int kt_per_slice, float epi, int y_frag, RopeArgs ra) {
  extern __shared__ __align__(16) float red[];            // [NW - 1][RT*MT][64][4]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int kb = blockIdx.y * kt_per_slice, ke = min(KT, kb + kt_per_slice);

  int tile[RT];
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    if (EPI == ALICE_EPI_GEGLU) tile[i] = (i & 1) ? (N / 16 + blockIdx.x * (RT / 2) + (i >> 1)) : (blockIdx.x * (RT / 2) + (i >> 1));
    else tile[i] = blockIdx.x * RT + i;
  }
  // where this lane reads its weight fragments (rows beyond the matrix: the last tile's, results unused)
  const bf16_t* wrow[RT];
#pragma unroll
  for (int i = 0; i < RT; ++i) wrow[i] = wf + (size_t)min(tile[i], NT - 1) * KT * 512 + lane * 8;
  f32x4 acc[RT][MT];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  bool row_ok[MT];
  int row[MT];
  const bf16_t* xrow[MT];        // this lane's place in the activations at k-tile 0
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    row[j] = j * 16 + r;
    row_ok[j] = row[j] < M;
    if constexpr (XF) xrow[j] = x + ((size_t)min(j, (M - 1) >> 4) * KT * 64 + lane) * 8;
    else xrow[j] = x + (size_t)min(row[j], M - 1) * K;
  }

  // A rolling window of U k-tiles per wave: wave w takes k-tiles kb + w, kb + w + NW, ...; as soon as a
  // tile's fragments have gone into the MFMAs their registers are refilled with the tile U steps ahead,
  // so U loads per operand stay in flight all the time.
  // The window is 4 (3 with eight or more products per k-tile), or 5 where the launcher finds that this leaves fewer
  // idle slots in a wave's last window (WINDOW; one or two products per k-tile only): 9 k-tiles a wave are two windows
  // of five with one idle slot instead of three of four with three, and 5 k-tiles one window and no loop (a 2B layer's
  // six kernels 54.0 -> 51.9 us), while 7 k-tiles are better off with two windows of four (9B down projection: 22.3
  // against 25.0 us).  Six and eight were slower everywhere.
  constexpr int U = WINDOW > 0 ? WINDOW : ((RT * MT >= 8) ? 3 : 4);
  u32x4 a[U][RT], b[U][MT];
  const bf16_t* zero = reinterpret_cast<const bf16_t*>(g_zero_tile) + lane * 8;
  auto fetch = [&](int kt, u32x4 (&aa)[RT], u32x4 (&bb)[MT]) {
    const bool kok = kt < ke;
    const int ktc = kok ? kt : 0;                           // past the slice: zero weights, any activations
    // STREAM: a matrix of 96 MB or more is read with the streaming hint (the 2B output head: 6.5 against 5.85 TB/s;
    // the 9B and 27B layers' matrices: 4 to 7 % faster).  Smaller ones are not: the hint cost the 2B down
    // projection (42 MB) 8 % and changed the others by 2 % either way.
#pragma unroll
    for (int i = 0; i < RT; ++i) {
      const u32x4* src = reinterpret_cast<const u32x4*>(kok ? wrow[i] + (size_t)ktc * 512 : zero);
      if constexpr (STREAM) aa[i] = __builtin_nontemporal_load(src);
      else aa[i] = *src;
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      if constexpr (XF) {
        bb[j] = *reinterpret_cast<const u32x4*>(xrow[j] + (size_t)ktc * 512);
      } else {
        // a row's last, partial k-tile: the weights are zero there, so any finite values do
        bb[j] = *reinterpret_cast<const u32x4*>(xrow[j] + min(ktc * 32 + g * 8, K - 8));
      }
    }
  };
  // Blocks start at different places of their k range and wrap around: all blocks read the same
  // activations, and in lockstep they would all ask the same L2 channel for the same line at once.
  const int J = (ke - kb + NW - 1) / NW;                    // k-tiles per wave (the last ones may be past the end)
  const int rot = J > 0 ? (int)(blockIdx.x % (unsigned)J) : 0;
  auto tile_at = [&](int t) {                               // t-th tile of this wave's rotated sequence
    int j = t + rot;
    if (j >= J) j -= J;
    return t < J ? kb + wave + j * NW : ke;                 // past the sequence: nothing to load
  };
#pragma unroll
  for (int u = 0; u < U; ++u) {
    fetch(tile_at(u), a[u], b[u]);
    __builtin_amdgcn_sched_barrier(0);       // slot by slot, oldest first: the loop waits for the oldest only
  }
  for (int t0 = 0; t0 + U < J; t0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[i][j] = mfma16(a[u][i], b[u][j], acc[i][j]);
      // The refill is issued here, U - 1 steps ahead of its use: the scheduler must not move it down to
      // the use (it would, to save registers).
      __builtin_amdgcn_sched_barrier(0);
      fetch(tile_at(t0 + U + u), a[u], b[u]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // the last window: nothing is left to fetch (slots past the end hold zero weights)
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j) acc[i][j] = mfma16(a[u][i], b[u][j], acc[i][j]);
  }

  // The waves' sums meet in LDS.  A tile of the output (a pair of tiles with GeGLU) has an owner among the waves,
  // in turn; every other wave leaves its sum of that tile in LDS (its place there: its index among the others), and
  // the owner adds them up in the order of the waves, its own in its place, and runs the epilogue of its tiles: the
  // same sums in the same order whoever owns a tile, and the epilogue's arithmetic and stores on all waves at once.
  constexpr int UNIT = EPI == ALICE_EPI_GEGLU ? 2 : 1;      // row tiles an owner takes together
  auto owner_of = [&](int i, int j) { return ((i / UNIT) * MT + j) % NW; };
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const int own = owner_of(i, j);
      if (wave != own) {
        const int slot = wave < own ? wave : wave - 1;
        *reinterpret_cast<f32x4*>(red + ((size_t)(slot * RT * MT + i * MT + j) * 64 + lane) * 4) = acc[i][j];
      }
    }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      if (wave != owner_of(i, j)) continue;
      const f32x4 mine = acc[i][j];
      f32x4 sum = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const int slot = w < wave ? w : w - 1;
        const f32x4 p = w == wave ? mine
                                  : *reinterpret_cast<const f32x4*>(red + ((size_t)(slot * RT * MT + i * MT + j) * 64 + lane) * 4);
        sum = w == 0 ? p : sum + p;
      }
      acc[i][j] = sum;
    }

  if constexpr (EPI == ALICE_EPI_ROPE) {
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      if (!row_ok[j]) continue;
      const RopeToken t = rope_token(ra, row[j]);
#pragma unroll
      for (int i = 0; i < RT; ++i)
        if (wave == owner_of(i, j) && tile[i] < NT) rope_store4(ra, row[j], t, tile[i] * 16 + g * 4, acc[i][j]);
    }
    return;
  }
  TO* yo = y + (size_t)blockIdx.y * M * N;                // the slice's partial sum
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (!row_ok[j]) continue;
    const size_t row_off = (size_t)row[j] * N;
    if (EPI == ALICE_EPI_GEGLU) {
#pragma unroll
      for (int p = 0; p < RT / 2; ++p) {
        if (wave != owner_of(2 * p, j)) continue;
        const int n = (blockIdx.x * (RT / 2) + p) * 16 + g * 4;
        f32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = gelu_tanh_f(acc[2 * p][j][i], FULL) * acc[2 * p + 1][j][i];
        if constexpr (sizeof(TO) == 2) {
          if (y_frag) { if (n < N) store4_frag((bf16_t*)yo, row[j], n, N, o); continue; }
        }
        store4(yo, row_off, n, N, o);
      }
    } else {
#pragma unroll
      for (int i = 0; i < RT; ++i) {
        if (wave != owner_of(i, j)) continue;
        const int n = tile[i] * 16 + g * 4;
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = epilogue1<EPI, FULL>(acc[i][j][e], epi);
        if constexpr (sizeof(TO) == 2) {
          if (y_frag) { if (n < N) store4_frag((bf16_t*)yo, row[j], n, N, o); continue; }
        }
        store4(yo, row_off, n, N, o);
      }
    }
  }
}

template <int RT, int MT, int EPI, typename TO>
int launch_skinny(const void* x, const void* w, void* y, int M, int N, int K, int split, float epi, int x_frag, int y_frag,
                  hipStream_t s, const RopeArgs& ra = RopeArgs{}) {
  const int KT = (K + 31) / 32, NT = (N * (EPI == ALICE_EPI_GEGLU ? 2 : 1) + 15) / 16;
  const int groups = EPI == ALICE_EPI_GEGLU ? ceil_div(N / 16, RT / 2) : ceil_div(NT, RT);
  const int per = ceil_div(KT, split);
  dim3 grid(groups, split);
  // Eight waves a block when the slice is long enough to give each of them work and the block count is
  // too low to fill the chip with four.
  const bool eight = (RT * MT <= 4) && per >= 32 && groups * split < 2048;
  const bool stream_w = x_frag && (size_t)NT * KT * 1024 >= ((size_t)96 << 20);
  // k-tiles per wave, and whether windows of five waste fewer slots than windows of four (see the kernel)
  const int nw = eight ? 8 : 4, J = ceil_div(min(per, KT), nw);
  const bool five = RT * MT <= 2 && x_frag && (ceil_div(J, 5) * 5 - J) < (ceil_div(J, 4) * 4 - J);
  // The reduction's LDS passes 64 KB with six row tiles and four token tiles: the kernel is told once.
#define SKINNY(NWV, THREADS, XFV, STREAMV, WINV)                                                                             \
  do {                                                                                                                         \
    auto kern = linear_skinny_kernel<RT, MT, NWV, EPI, TO, false, XFV, STREAMV, WINV>;                                        \
    if (lds > 48 * 1024) {                                                                                                     \
      static bool told = false;                                                                                                \
      if (!told) {                                                                                                             \
        ALICE_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, \
                    "linear: the device does not give a block %d bytes of LDS", (int)lds);                                     \
        told = true;                                                                                                           \
      }                                                                                                                        \
    }                                                                                                                          \
    kern<<<grid, THREADS, lds, s>>>((const bf16_t*)x, (const bf16_t*)w, (TO*)y, M, N, K, KT, NT, per, epi, y_frag, ra);       \
  } while (0)
#define BY_INPUT(NWV, THREADS)                                                        \
  do {                                                                                \
    if constexpr (RT * MT <= 2) {                                                     \
      if (five && stream_w) { SKINNY(NWV, THREADS, true, true, 5); break; }           \
      if (five) { SKINNY(NWV, THREADS, true, false, 5); break; }                      \
    }                                                                                 \
    if (stream_w) SKINNY(NWV, THREADS, true, true, 0);                                \
    else if (x_frag) SKINNY(NWV, THREADS, true, false, 0);                            \
    else SKINNY(NWV, THREADS, false, false, 0);                                       \
  } while (0)
  if (eight) {
    const size_t lds = (size_t)7 * RT * MT * 256 * sizeof(float);
    BY_INPUT(8, 512);
  } else {
    const size_t lds = (size_t)3 * RT * MT * 256 * sizeof(float);
    BY_INPUT(4, 256);
  }
#undef BY_INPUT
#undef SKINNY
  ALICE_LAUNCH_CHECK();
  return 0;
}

// Row tiles per block: few keep the chip full on narrow matrices, more amortise the activation reads
// on wide ones.  (GeGLU needs an even number: gate and up tiles come in pairs.)  Measured on the 2B
// shapes with the activations in fragment order.
int skinny_row_tiles_base(int M, int N, int epi, int split, int K) {
  const int tiles = ceil_div(N * (epi == ALICE_EPI_GEGLU ? 2 : 1), 16);
  if (tiles >= 4096) return 4;
  if (epi == ALICE_EPI_GEGLU) return 2;
  // Many tokens and slices of the inner dimension: more rows per block per read of the activations.
  if (M > 32 && split > 1 && tiles >= 64) return K >= 8192 ? 4 : 2;
  return tiles >= 1024 ? 2 : 1;
}

// What a choice of row tiles and slices costs, in units of one k-tile of one row tile read by a CU: the busiest of
// the 256 CUs runs ceil(blocks / 256) blocks one after the other (or side by side, sharing what it can load), each
// reading rt weight tiles and the token tiles' activations (which come from the L2: half the price) per k-tile,
// and every slice adds a partial result and shortens each wave's run.  Fitted to the 2B, 9B and 27B matrices at 1
// to 64 tokens: gate/up of the 2B shape at 64 tokens takes 27.5, 30.5 and 22.9 us with 2, 4 and 6 row tiles (576,
// 288 and 192 blocks: 3, 2 and 1 per CU), the 9B shape 57.5, 49.6 and 58.7 us, the 27B shape 168, 148 and 132 us.
float skinny_cost(int M, int N, int K, int epi, int rt, int split) {
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4), KT = (K + 31) / 32;
  const int groups = epi == ALICE_EPI_GEGLU ? ceil_div(N / 16, rt / 2) : ceil_div(ceil_div(N, 16), rt);
  return (float)ceil_div((long)groups * split, 256) * ceil_div(KT, split) * (rt + 0.5f * mt) + 20.f * split;
}

// Six row tiles a block where the cost above says so: gate/up by the cost alone, the other products only where
// six beat the rule above by 7 % (that rule is measured, the cost is a model).
int skinny_row_tiles(int M, int N, int epi, int split, int K) {
  const int base = skinny_row_tiles_base(M, N, epi, split, K);
  if (epi == ALICE_EPI_GEGLU) {
    int best = 2;
    for (int rt = 4; rt <= 6; rt += 2)
      if (skinny_cost(M, N, K, epi, rt, 1) < skinny_cost(M, N, K, epi, best, 1)) best = rt;
    return best;
  }
  if (epi != ALICE_EPI_NONE) return base;
  return skinny_cost(M, N, K, epi, 6, split) < 0.93f * skinny_cost(M, N, K, epi, base, split) ? 6 : base;
}

template <int EPI, typename TO>
int skinny_by_shape(const void* x, const void* w, void* y, int M, int N, int K, int split, float epi, int x_frag, int y_frag,
                    hipStream_t s) {
  const int rt = skinny_row_tiles(M, N, EPI, split, K);
#define GO(RT, MT) return launch_skinny<RT, MT, EPI, TO>(x, w, y, M, N, K, split, epi, x_frag, y_frag, s)
#define BY_RT(MT)                                                   \
  do {                                                              \
    if constexpr (EPI != ALICE_EPI_SOFTCAP) { if (rt == 6) GO(6, MT); } \
    if (rt == 4) GO(4, MT);                                         \
    if (rt == 2) GO(2, MT);                                         \
    if constexpr (EPI != ALICE_EPI_GEGLU) GO(1, MT);                \
  } while (0)
  if (M <= 16) BY_RT(1);
  if (M <= 32) BY_RT(2);
  BY_RT(4);
#undef BY_RT
#undef GO
  return 1;
}

}  // namespace
