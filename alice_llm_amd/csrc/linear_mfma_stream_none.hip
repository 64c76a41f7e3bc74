// The streaming matrix product's instantiations with the none epilogue (see linear_mfma_stream.h).
#include "linear_mfma_stream.h"

int alice_mfma_stream_none(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, float epi_param, int split,
                           int x_frag, int y_frag, hipStream_t s) {
  if (y_dtype == DT_F32) return skinny_by_shape<ALICE_EPI_NONE, float>(x, w, y, M, N, K, split, epi_param, x_frag, y_frag, s);
  return skinny_by_shape<ALICE_EPI_NONE, bf16_t>(x, w, y, M, N, K, split, epi_param, x_frag, y_frag, s);
}
