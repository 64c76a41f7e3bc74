// Dispatch of the matrix product to its kernels.
#include "common.h"
#include "alice_hip.h"

int alice_linear_split_hint_frag(int M, int N, int K);
int alice_linear_frag(const void* x, int x_dtype, const void* w, void* y, int y_dtype, int M, int N, int K,
                      int epi, float epi_param, int split_k, int variant, int x_layout, int y_layout,
                      hipStream_t stream);

extern "C" int alice_linear_split_hint(int M, int N, int K, int w_layout) {
  return w_layout == ALICE_LAYOUT_FRAG16 ? alice_linear_split_hint_frag(M, N, K) : 1;
}

extern "C" int alice_linear(const void* x, int x_dtype, const void* w, int w_dtype, int w_layout, void* y,
                            int y_dtype, int M, int N, int K, int epilogue, float epi_param, int split_k,
                            int variant, int full_precision, int x_layout, int y_layout, hipStream_t stream) {
  ALICE_CHECK(x && w && y, "linear: null operand");
  ALICE_CHECK(split_k >= 1, "linear: split_k must be at least 1");
  if (w_layout == ALICE_LAYOUT_ROW) {
    ALICE_CHECK(variant == ALICE_LINEAR_AUTO || variant == ALICE_LINEAR_GENERIC,
                "linear: row-major weights run on the generic kernel only");
    ALICE_CHECK(split_k == 1, "linear: the generic kernel produces no partial sums");
    ALICE_CHECK(x_layout == ALICE_LAYOUT_ROW && y_layout == ALICE_LAYOUT_ROW, "linear: the generic kernel reads and writes rows");
    return alice_linear_generic(x, x_dtype, w, w_dtype, y, y_dtype, M, N, K, epilogue, epi_param,
                                full_precision, stream);
  }
  if (w_layout == ALICE_LAYOUT_FRAG16) {
    ALICE_CHECK(w_dtype == DT_BF16, "linear: the fragment layout holds bfloat16 only");
    ALICE_CHECK(variant != ALICE_LINEAR_GENERIC, "linear: the generic kernel reads row-major weights");
    return alice_linear_frag(x, x_dtype, w, y, y_dtype, M, N, K, epilogue, epi_param, split_k, variant, x_layout, y_layout,
                             stream);
  }
  alice_set_error("linear: unknown weight layout %d", w_layout);
  return 1;
}
