// The streaming matrix product's instantiations with the rotation and the cache write as epilogue (see
// linear_mfma_stream.h).
#include "linear_mfma_stream.h"

int alice_mfma_stream_rope(const void* x, const void* w, int M, int N, int K, int x_frag, hipStream_t s, const RopeArgs& ra) {
  // one row tile a block while that gives every CU at most one block, two beyond (q|k|v of 8,192 rows at 32 tokens:
  // 20.0 against 24.6 us, at 8 tokens 17.2 against 17.8; of 4,096 rows two tiles are 25 % slower)
  const int rt = ceil_div(N, 16) > 256 ? 2 : 1;
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
