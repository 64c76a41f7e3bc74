// The tiled matrix product for many tokens: the choice of its tile (wave tile width, tokens a block, k-tiles a stage,
// slices of the inner dimension) and the launches with the widest wave tile; the kernel is in linear_mfma_tiled.h, the
// launches with narrower tiles in linear_mfma_tiled_narrow.hip.
#include "linear_mfma_tiled.h"

namespace {

// Slices of the inner dimension for the widest tile: 128 tokens x 256 features a block, two blocks a CU.  Narrow
// outputs leave most of the chip idle; slices fill it.  Cost of s slices, relative to one block a CU running the
// whole inner dimension: the busiest CU runs n = ceil(blocks s / 256) blocks of 1/s the length, two at a time at
// 1.7 times the time of one; every extra slice writes and reads another [M, N] float32 partial result (both
// constants fitted to measurements at N = 2304, K = 2048 and 9216).
int tiled_split_wide(int M, int N, int K) {
  const int blocks = ceil_div(N, 256) * ceil_div(M, 128), KT = (K + 31) / 32;
  if (blocks >= 384) return 1;
  int best = 1;
  float best_cost = 1e30f;
  for (int s = 1; s <= 6; ++s) {
    if (s > 1 && KT / s < 16) break;
    const int n = ceil_div(blocks * s, 256);
    const float cost = (1.7f * (n / 2) + (n % 2)) / s + 3.6f * blocks / K * (s - 1);
    if (cost < best_cost * 0.97f) { best_cost = cost; best = s; }
  }
  return best;
}

// What a tile costs at a few hundred tokens, in microseconds without the fixed part (fitted to all tiles and slice
// counts at 96 to 1,024 tokens on the q|k|v, output, gate/up and down shapes of the 2B, 9B and 27B models; its
// choices are 3 % behind the best measured one on average).  A block takes its k-tiles one after the other, each at
// the slowest of: the wait for a stage's weights over the stage's k-tiles, the blocks' common share of the memory
// rate, the bytes through the CU's L1, and the products; the busiest CU runs ceil(B / 256) blocks, two at a time.
float tiled_cost(int M, int N, int K, int epi, int wn, int tm, int kc, int sp) {
  const int NT = ceil_div(N * (epi == ALICE_EPI_GEGLU ? 2 : 1), 16), KT = ceil_div(K, 32);
  const int gx = ceil_div(NT, 4 * wn), gy = ceil_div(M, 16 * tm), B = gx * gy * sp, kts = ceil_div(KT, sp);
  const int n = ceil_div(B, 256), res = n < 2 ? n : 2, conc = B < 512 ? B : 512;
  float t = kc >= 8 ? 0.12f : kc >= 4 ? 0.146f : 0.25f;
  t = fmaxf(t, (float)conc / gy * 4 * wn / 8000.f);
  t = fmaxf(t, 0.011f * (4 * wn + tm) * res);
  t = fmaxf(t, 0.008f * wn * tm * res);
  const float rounds = n == 1 ? 1.f : (n / 2) + (n % 2) * 0.6f;
  return rounds * kts * t + 0.1f * (sp > 1 ? sp : 0) * (float)M * N * 4e-6f;
}

template <int EPI, typename TO>
int launch_wide(const void* x, const void* w, void* y, int M, int N, int K, int split, float epi, int x_frag, int y_frag,
                hipStream_t s, int tm, const RopeArgs& ra) {
  if (x_frag) {
    if (tm == 8) return launch_tiled_as<EPI, TO, 8, true, 4, 2>(x, w, y, M, N, K, split, epi, y_frag, s, ra);
    return launch_tiled_as<EPI, TO, 4, true, 4, 2>(x, w, y, M, N, K, split, epi, y_frag, s, ra);
  }
  if (tm == 8) return launch_tiled_as<EPI, TO, 8, false, 4, 2>(x, w, y, M, N, K, split, epi, y_frag, s, ra);
  return launch_tiled_as<EPI, TO, 4, false, 4, 2>(x, w, y, M, N, K, split, epi, y_frag, s, ra);
}

bool narrow_built(int epi, int y_dtype) {
  return (epi == ALICE_EPI_NONE && y_dtype == DT_F32) || (epi == ALICE_EPI_GEGLU && y_dtype == DT_BF16) || epi == ALICE_EPI_ROPE;
}

}  // namespace

TiledPlan alice_mfma_tiled_plan(int M, int N, int K, int epi, int y_dtype, int split, int x_frag) {
  const int KT = ceil_div(K, 32), NT = ceil_div(N * (epi == ALICE_EPI_GEGLU ? 2 : 1), 16);
  const bool may_split = epi == ALICE_EPI_NONE && y_dtype == DT_F32;
  if (M <= 64) {
    // Up to 64 tokens: the streaming kernel, or the narrow tiles in blocks of 64 tokens with stages of eight
    // k-tiles.  Measured on 23 shapes at 33, 40, 48 and 64 tokens: the tiled kernel is 8 to 57 % faster where its
    // blocks come close to one a CU (the most blocks up to 256 over both tiles and the slice counts, the fewest
    // slices among equals), slower where they are few (48 to 80 blocks: 3 to 20 %) or more than 256, and no better
    // with the GeGLU epilogue below 190 blocks; with that rule the mean gain is 13 %, the worst case -3 %.
    // Up to 32 tokens the streaming kernel is the better one except for float32 sums over a long inner dimension
    // in slices (output and down projections: 2 to 17 % for the tiled kernel on eight shapes of 16 to 134 MB; a
    // matrix of 340 MB, which the streaming kernel reads with the streaming hint, is 4 to 10 % slower tiled).
    TiledPlan none{0, 4, 8, split > 0 ? split : 1};
    if (!(x_frag && narrow_built(epi, y_dtype))) return none;
    if (M <= 32 && !(may_split && K >= 4096 && (size_t)N * K < ((size_t)128 << 20))) return none;
    static const int slices[] = {1, 2, 3, 4, 6, 8, 12, 16};
    int best_b = 0, best_wn = 0, best_sp = 0;
    for (int wn = 2; wn >= 1; --wn) {
      if (epi == ALICE_EPI_GEGLU && wn == 1) continue;
      for (int sp : slices) {
        if (split > 0 ? sp != split : (sp > 1 && (!may_split || KT / sp < 8))) continue;
        const int b = ceil_div(NT, 4 * wn) * sp;
        if (b <= 256 && (b > best_b || (b == best_b && sp < best_sp))) { best_b = b; best_wn = wn; best_sp = sp; }
      }
    }
    if (best_b >= 190 || (M > 32 && epi != ALICE_EPI_GEGLU && best_b >= 96)) return TiledPlan{best_wn, 4, 8, best_sp};
    return none;
  }
  const int sp0 = split > 0 ? split : (may_split ? tiled_split_wide(M, N, K) : 1);
  // The widest tile: 128 tokens a block, or 64 when that leaves most of the chip without a block (measured at
  // N = 2304 and 4096: 216 and 256 blocks of 128 tokens beat twice as many of 64, 128 blocks do not; the same with
  // the rotation epilogue since its stores go through LDS).
  const bool high = ceil_div(NT, 16) * ceil_div(M, 128) * sp0 >= 192;
  const TiledPlan wide{4, high ? 8 : 4, 2, sp0};
  // Between 65 and 1,024 tokens (what the cost rule was fitted on) another tile is taken where the rule says it is
  // 8 % cheaper; the narrow tiles exist for activations in fragment order and for the layers' own products.
  if (!(x_frag && M <= 1024 && narrow_built(epi, y_dtype))) return wide;
  TiledPlan best = wide;
  float best_cost = tiled_cost(M, N, K, epi, wide.wn, wide.tm, wide.kc, wide.split) * 0.92f;
  static const int slices[] = {1, 2, 3, 4, 6, 8};
  for (int wn = 4; wn >= 1; wn >>= 1) {
    if (epi == ALICE_EPI_GEGLU && wn == 1) continue;
    for (int tm = 8; tm >= 4; tm >>= 1) {
      const int kc = wn == 4 ? 2 : 32 / tm;
      for (int sp : slices) {
        if (split > 0 ? sp != split : (sp > 1 && (!may_split || KT / sp < 16))) continue;
        const float c = tiled_cost(M, N, K, epi, wn, tm, kc, sp);
        if (c < best_cost) { best_cost = c; best = TiledPlan{wn, tm, kc, sp}; }
      }
    }
  }
  if (split > 0) best.split = split;
  return best;
}

int alice_mfma_tiled(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                     int split, int x_frag, int y_frag, int force_wn, hipStream_t s) {
  TiledPlan p = alice_mfma_tiled_plan(M, N, K, epi, y_dtype, split, x_frag);
  p.split = split;
  if (p.wn == 0) p = TiledPlan{4, 8, 2, split};              // up to 64 tokens and asked for by name: the widest tile
  if (force_wn) {
    ALICE_CHECK((force_wn == 1 || force_wn == 2) && x_frag && narrow_built(epi, y_dtype) && !(epi == ALICE_EPI_GEGLU && force_wn == 1),
                "linear: no tiled kernel with a wave tile of %d features for this epilogue, output type and activation layout", 16 * force_wn);
    p.wn = force_wn;
    if (M <= 64) p.tm = 4;
    p.kc = 32 / p.tm;
  }
  if (p.wn < 4) return alice_mfma_tiled_narrow(x, w, y, y_dtype, M, N, K, epi, epi_param, p, y_frag, s, RopeArgs{});
  const int tm = p.tm;
  ALICE_MFMA_BY_EPI(launch_wide, x, w, y, M, N, K, split, epi_param, x_frag, y_frag, s, tm, RopeArgs{});
}

int alice_mfma_tiled_rope(const void* x, const void* w, int M, int N, int K, int x_frag, hipStream_t s, const RopeArgs& ra) {
  TiledPlan p = alice_mfma_tiled_plan(M, N, K, ALICE_EPI_ROPE, DT_BF16, 1, x_frag);
  if (p.wn == 0) p = TiledPlan{4, 8, 2, 1};
  if (p.wn < 4) return alice_mfma_tiled_narrow(x, w, nullptr, DT_BF16, M, N, K, ALICE_EPI_ROPE, 0.f, p, 0, s, ra);
  return launch_wide<ALICE_EPI_ROPE, bf16_t>(x, w, nullptr, M, N, K, 1, 0.f, x_frag, 0, s, p.tm, ra);
}
