// The tiled matrix product with wave tiles of 16 or 32 output features (prompts of a few hundred tokens, where the
// widest tile makes fewer blocks than the chip has CUs): activations in fragment order; float32 sums (with slices of
// the inner dimension), the GeGLU epilogue to bfloat16, or the rotation epilogue.
#include "linear_mfma_tiled.h"

namespace {

template <int EPI, typename TO>
int launch_narrow(const void* x, const void* w, void* y, int M, int N, int K, float epi, const TiledPlan& p, int y_frag,
                  hipStream_t s, const RopeArgs& ra) {
  if constexpr (EPI != ALICE_EPI_GEGLU) {
    if (p.wn == 1 && p.tm == 8) return launch_tiled_as<EPI, TO, 8, true, 1, 4>(x, w, y, M, N, K, p.split, epi, y_frag, s, ra);
    if (p.wn == 1) return launch_tiled_as<EPI, TO, 4, true, 1, 8>(x, w, y, M, N, K, p.split, epi, y_frag, s, ra);
  }
  if (p.tm == 8) return launch_tiled_as<EPI, TO, 8, true, 2, 4>(x, w, y, M, N, K, p.split, epi, y_frag, s, ra);
  return launch_tiled_as<EPI, TO, 4, true, 2, 8>(x, w, y, M, N, K, p.split, epi, y_frag, s, ra);
}

}  // namespace

int alice_mfma_tiled_narrow(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                            const TiledPlan& p, int y_frag, hipStream_t s, const RopeArgs& ra) {
  ALICE_CHECK((p.wn == 1 || p.wn == 2) && (p.tm == 4 || p.tm == 8) && p.kc * p.tm == 32 && p.split >= 1,
              "linear: no tiled kernel for wave tile %d, %d tokens a block, %d k-tiles a stage", 16 * p.wn, 16 * p.tm, p.kc);
  if (epi == ALICE_EPI_ROPE) return launch_narrow<ALICE_EPI_ROPE, bf16_t>(x, w, nullptr, M, N, K, 0.f, p, 0, s, ra);
  if (epi == ALICE_EPI_NONE && y_dtype == DT_F32) return launch_narrow<ALICE_EPI_NONE, float>(x, w, y, M, N, K, epi_param, p, y_frag, s, ra);
  ALICE_CHECK(epi == ALICE_EPI_GEGLU && y_dtype == DT_BF16 && p.wn == 2 && p.split == 1,
              "linear: the narrow tiles take float32 sums, GeGLU to bfloat16 (32 features a wave) or the rotation epilogue");
  return launch_narrow<ALICE_EPI_GEGLU, bf16_t>(x, w, y, M, N, K, epi_param, p, y_frag, s, ra);
}
