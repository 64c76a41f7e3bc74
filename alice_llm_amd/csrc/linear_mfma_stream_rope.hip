// The streaming matrix product's instantiations with the rotation and the cache write as epilogue (see
// linear_mfma_stream.h).
#include "linear_mfma_stream.h"

int alice_mfma_stream_rope(const void* x, const void* w, int M, int N, int K, int x_frag, hipStream_t s, const RopeArgs& ra) {
  const int rt = skinny_row_tiles(M, N, ALICE_EPI_NONE, 1, K);
#define GO(RT, MT) return launch_skinny<RT, MT, ALICE_EPI_ROPE, bf16_t>(x, w, nullptr, M, N, K, 1, 0.f, x_frag, 0, s, ra)
#define BY_RT(MT)                \
  do {                           \
    if (rt >= 2) GO(2, MT);      \
    GO(1, MT);                   \
  } while (0)
  if (M <= 16) BY_RT(1);
  if (M <= 32) BY_RT(2);
  BY_RT(4);
#undef BY_RT
#undef GO
}
