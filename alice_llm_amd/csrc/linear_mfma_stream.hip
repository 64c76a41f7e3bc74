// The streaming matrix product's entry for the other source files: its rules, and the dispatch to the source file
// that holds the instantiations of the asked epilogue.
#include "linear_mfma_stream.h"

int alice_mfma_stream_none(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, float epi_param, int split,
                           int x_frag, int y_frag, hipStream_t s);
int alice_mfma_stream_geglu(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, float epi_param, int split,
                            int x_frag, int y_frag, hipStream_t s);
int alice_mfma_stream_softcap(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, float epi_param, int split,
                              int x_frag, int y_frag, hipStream_t s);

int alice_mfma_stream_row_tiles(int M, int N, int epi, int split, int K) { return skinny_row_tiles(M, N, epi, split, K); }
int alice_mfma_stream_row_tiles_base(int M, int N, int epi, int split, int K) { return skinny_row_tiles_base(M, N, epi, split, K); }
float alice_mfma_stream_cost(int M, int N, int K, int epi, int rt, int split) { return skinny_cost(M, N, K, epi, rt, split); }

int alice_mfma_stream(const void* x, const void* w, void* y, int y_dtype, int M, int N, int K, int epi, float epi_param,
                      int split, int x_frag, int y_frag, hipStream_t s) {
  if (epi == ALICE_EPI_NONE) return alice_mfma_stream_none(x, w, y, y_dtype, M, N, K, epi_param, split, x_frag, y_frag, s);
  if (epi == ALICE_EPI_GEGLU) return alice_mfma_stream_geglu(x, w, y, y_dtype, M, N, K, epi_param, split, x_frag, y_frag, s);
  return alice_mfma_stream_softcap(x, w, y, y_dtype, M, N, K, epi_param, split, x_frag, y_frag, s);
}
