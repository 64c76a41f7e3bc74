// Entry points of the bfloat16 matrix products on the matrix cores: the conversion of a weight matrix into the
// fragment layout, the choice between the streaming and the tiled kernel, and the number of slices of the inner
// dimension.  The kernels are in linear_mfma_stream.hip and linear_mfma_tiled.hip, what they share in linear_mfma.h.
#include "linear_mfma.h"

namespace {

// ---------------------------------------------------------------- layout conversion
__global__ void to_frag16_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, int N, int K, int KT, size_t total) {
  const size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x;     // index in dst, in elements
  if (o >= total) return;
  const int e = o & 7;
  const int lane = (o >> 3) & 63;
  const size_t t = o >> 9;
  const int kt = (int)(t % KT);
  const int nt = (int)(t / KT);
  const int n = nt * 16 + (lane & 15), k = kt * 32 + (lane >> 4) * 8 + e;
  bf16_t z;
  z.bits = 0;
  dst[o] = (n < N && k < K) ? src[(size_t)n * K + k] : z;
}

}  // namespace

// Whether a matrix of `rows` x K with this epilogue can use the fragment layout.
extern "C" int alice_frag16_supported(int rows, int K, int epilogue) {
  if (K % 8 != 0) return 0;                                   // activations are read 8 at a time
  if (epilogue == ALICE_EPI_GEGLU && (rows % 32 != 0)) return 0;   // gate and up halves must be whole tiles
  return 1;
}

extern "C" int alice_to_frag16(const void* src, void* dst, int N, int K, hipStream_t stream) {
  ALICE_CHECK(N > 0 && K > 0, "to_frag16: bad sizes N=%d K=%d", N, K);
  const int KT = (K + 31) / 32, NT = (N + 15) / 16;
  const size_t total = (size_t)NT * KT * 512;
  to_frag16_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>((const bf16_t*)src, (bf16_t*)dst, N, K, KT, total);
  ALICE_LAUNCH_CHECK();
  return 0;
}

// The number of slices once six row tiles a block are a choice: half or twice the measured rule's number where the
// cost (with the row tiles that skinny_row_tiles would then pick) is 7 % lower.
static int skinny_split_with_six(int M, int N, int K, int split0) {
  const int KT = (K + 31) / 32;
  auto cost_at = [&](int sp) {
    return alice_mfma_stream_cost(M, N, K, ALICE_EPI_NONE, alice_mfma_stream_row_tiles(M, N, ALICE_EPI_NONE, sp, K), sp);
  };
  int best = split0;
  float best_cost = cost_at(split0) * 0.93f;
  for (int sp : {split0 / 2, split0 * 2}) {
    if (sp < 1 || sp > 16 || sp == split0 || (sp > 1 && KT / sp < 16)) continue;
    const float c = cost_at(sp);
    if (c < best_cost) { best_cost = c; best = sp; }
  }
  return best;
}

int alice_linear_split_hint_frag(int M, int N, int K) {
  // more than 64 tokens: the tiled kernel's own rule (activations in fragment order, as prompts bring them)
  if (M > 64) return alice_mfma_tiled_plan(M, N, K, ALICE_EPI_NONE, DT_F32, 0, 1).split;
  const int KT = (K + 31) / 32;
  const TiledPlan p = alice_mfma_tiled_plan(M, N, K, ALICE_EPI_NONE, DT_F32, 0, 1);
  if (p.wn != 0) return p.split;                             // the tiled kernel's narrow tiles are the better ones here
  if (M > 32) return skinny_split_with_six(M, N, K, KT >= 128 ? 4 : (KT >= 32 ? 2 : 1));
  const int groups = ceil_div(ceil_div(N, 16), alice_mfma_stream_row_tiles_base(M, N, ALICE_EPI_NONE, 1, K));
  int split = 1;
  // aim at about 1024 blocks, keep at least 16 k-tiles (4 per wave) per slice
  while (groups * split < 1024 && KT / (split * 2) >= 16 && split < 16) split *= 2;
  return skinny_split_with_six(M, N, K, split);
}

int alice_linear_frag(const void* x, int x_dtype, const void* w, void* y, int y_dtype, int M, int N, int K,
                      int epi, float epi_param, int split_k, int variant, int x_layout, int y_layout,
                      hipStream_t stream) {
  ALICE_CHECK(x_dtype == DT_BF16, "linear: the fragment layout needs bfloat16 activations");
  ALICE_CHECK(dtype_ok(y_dtype), "linear: unknown output dtype");
  ALICE_CHECK(M >= 0 && N > 0 && K > 0 && K % 8 == 0, "linear: bad sizes M=%d N=%d K=%d (K must be a multiple of 8)", M, N, K);
  ALICE_CHECK(epi != ALICE_EPI_GEGLU || N % 16 == 0, "linear: GeGLU in the fragment layout needs N %% 16 == 0, found %d", N);
  ALICE_CHECK(epi != ALICE_EPI_SOFTCAP || epi_param > 0.f, "linear: softcap must be positive");
  ALICE_CHECK(((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0, "linear: operands must be 16-byte aligned");
  ALICE_CHECK(x_layout == ALICE_LAYOUT_ROW || (x_layout == ALICE_LAYOUT_FRAG16 && K % 32 == 0),
              "linear: activations in fragment order need K %% 32 == 0, found K=%d", K);
  if (M == 0) return 0;
  // Up to 64 tokens stream the weights once; very wide matrices (the output head) have enough column
  // blocks for the tiled kernel, which shares the activations through LDS, from 33 tokens on (the 2B head: the same
  // time at 32 tokens, 228 against 277 us at 48; the streaming kernel 198 against 210 us at 17).
  bool skinny = variant == ALICE_LINEAR_SKINNY || (variant == ALICE_LINEAR_AUTO && M <= 64 && !(M > 32 && N >= 65536 && split_k == 1));
  // the tiled kernel's narrow tiles where its rule prefers them
  if (skinny && variant == ALICE_LINEAR_AUTO && alice_mfma_tiled_plan(M, N, K, epi, y_dtype, split_k, x_layout == ALICE_LAYOUT_FRAG16).wn != 0)
    skinny = false;
  ALICE_CHECK(!(variant == ALICE_LINEAR_SKINNY && M > 64), "linear: the streaming kernel takes at most 64 rows, found %d", M);
  ALICE_CHECK(split_k == 1 || (epi == ALICE_EPI_NONE && y_dtype == DT_F32),
              "linear: partial sums need no epilogue and float32 output");
  ALICE_CHECK(ceil_div(M, 128) <= 65535, "linear: too many rows for one launch (%d)", M);
  ALICE_CHECK(y_layout == ALICE_LAYOUT_ROW || (y_layout == ALICE_LAYOUT_FRAG16 && y_dtype == DT_BF16 && N % 32 == 0 &&
                                                split_k == 1 && epi != ALICE_EPI_SOFTCAP),
              "linear: output in fragment order needs bfloat16, N %% 32 == 0, no softcap and no partial sums");
  const int x_frag = x_layout == ALICE_LAYOUT_FRAG16, y_frag = y_layout == ALICE_LAYOUT_FRAG16;
  if (skinny) return alice_mfma_stream(x, w, y, y_dtype, M, N, K, epi, epi_param, split_k, x_frag, y_frag, stream);
  const int force_wn = variant == ALICE_LINEAR_TILED_W16 ? 1 : variant == ALICE_LINEAR_TILED_W32 ? 2 : 0;
  return alice_mfma_tiled(x, w, y, y_dtype, M, N, K, epi, epi_param, split_k, x_frag, y_frag, force_wn, stream);
}

extern "C" int alice_linear_rope_cache(const void* x, int x_layout, const void* w, int M, int K, void* q_out, void* k_pool,
                                       void* v_pool, const float* cos_t, const float* sin_t, const int* positions,
                                       const int* seq_of_token, const int* block_table, int bt_stride, int nH, int nKV,
                                       int d, int page_size, int n_pages, int kv_layout, hipStream_t stream) {
  ALICE_CHECK(M >= 0 && ceil_div(M, 128) <= 65535, "linear+rope: bad number of tokens %d", M);
  ALICE_CHECK(K > 0 && K % 8 == 0, "linear+rope: K must be a multiple of 8, found %d", K);
  ALICE_CHECK(nH >= 1 && nKV >= 1 && d >= 16 && d % 16 == 0, "linear+rope: bad heads nH=%d nKV=%d d=%d (d must be a multiple of 16)", nH, nKV, d);
  ALICE_CHECK(x && w && q_out && k_pool && v_pool && cos_t && sin_t && positions && seq_of_token && block_table,
              "linear+rope: a pointer is missing");
  ALICE_CHECK(((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)q_out & 15) == 0 && ((uintptr_t)cos_t & 7) == 0 &&
              ((uintptr_t)sin_t & 7) == 0 && ((uintptr_t)k_pool & 15) == 0 && ((uintptr_t)v_pool & 15) == 0,
              "linear+rope: operands are not aligned");
  ALICE_CHECK(x_layout == ALICE_LAYOUT_ROW || (x_layout == ALICE_LAYOUT_FRAG16 && K % 32 == 0),
              "linear+rope: activations in fragment order need K %% 32 == 0, found K=%d", K);
  ALICE_CHECK(page_size > 0 && n_pages > 0 && bt_stride > 0, "linear+rope: bad page geometry");
  ALICE_CHECK(kv_layout == 0 || (kv_layout == 1 && page_size == 64 && d % 32 == 0),
              "linear+rope: the fragment cache layout needs pages of 64 and head_dim %% 32 == 0");
  if (M == 0) return 0;
  const int N = (nH + 2 * nKV) * d;
  RopeArgs ra{(bf16_t*)q_out, (bf16_t*)k_pool, (bf16_t*)v_pool, cos_t, sin_t, positions, seq_of_token, block_table,
              bt_stride, nH, nKV, d, page_size, n_pages, kv_layout};
  const int x_frag = x_layout == ALICE_LAYOUT_FRAG16;
  if (M > 64 || alice_mfma_tiled_plan(M, N, K, ALICE_EPI_ROPE, DT_BF16, 1, x_frag).wn != 0)
    return alice_mfma_tiled_rope(x, w, M, N, K, x_frag, stream, ra);
  return alice_mfma_stream_rope(x, w, M, N, K, x_frag, stream, ra);
}
