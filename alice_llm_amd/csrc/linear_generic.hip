// Matrix product y[M, N] = x[M, K] . W[N, K]^T for every combination of 32-bit and bfloat16
// operands, with plain 32-bit fused multiply-adds and 32-bit accumulation: the kernel of the
// true 32-bit path, and the fallback of the bfloat16 path for shapes its MFMA kernels refuse.
//
// Weight layout and orientation as in the reference: row-major [out, in], y[r] = sum_c W[r,c] x[c]
// (gguf.rs:4063-4074, f32_matvec).  Epilogues: none; GeGLU gelu_tanh(gate) * up with W = [gate; up]
// stacked (llama3.rs:14519-14534); softcap cap * tanh(y / cap) (llama3.rs:14606-14611).
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16;

// A block computes a 64 x 64 tile.  Its 64 columns are two runs of 32: columns [n0, n0+32) and
// [n1, n1+32).  Without an epilogue n1 = n0 + 32; with GeGLU the first run are gate rows j0.. and
// the second the up rows N + j0.. of the stacked weight, so that a thread holds gate and up of the
// same output column.  The k loop runs in order, so a result does not depend on M or on the tile.
template <typename TA, typename TW, typename TO, int EPI, bool FULL>
__global__ __launch_bounds__(256) void linear_tiled_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                           TO* __restrict__ Y, int M, int N, int K, float epi) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Bs[BK][BN + 4];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * BM;
  const int wrows = EPI == ALICE_EPI_GEGLU ? 2 * N : N;      // rows of W
  int n0, n1;
  if (EPI == ALICE_EPI_GEGLU) { n0 = blockIdx.x * 32; n1 = N + n0; }
  else { n0 = blockIdx.x * 64; n1 = n0 + 32; }
  const int lim0 = EPI == ALICE_EPI_GEGLU ? N : wrows;       // first run must stay below this row

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int lr = tid >> 2, lk = (tid & 3) * 4;               // loader: row 0..63, k offset 0,4,8,12
  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int m = m0 + lr;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        As[lk + i][lr] = (m < M && k < K) ? load_f32(A, (size_t)m * K + k) : 0.f;
      }
      const int run = lr >> 5, c = lr & 31;
      const int n = (run ? n1 : n0) + c;
      const bool ok = run ? (n < wrows) : (n < lim0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + lk + i;
        Bs[lk + i][lr] = (ok && k < K) ? load_f32(W, (size_t)n * K + k) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
      b[0] = Bs[k][tx * 2];
      b[1] = Bs[k][tx * 2 + 1];
      b[2] = Bs[k][32 + tx * 2];
      b[3] = Bs[k][33 + tx * 2];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
    if (EPI == ALICE_EPI_GEGLU) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = n0 + tx * 2 + j;
        if (n < N) {
          float g = acc[i][j], u = acc[i][j + 2];
          store_f32(Y, (size_t)m * N + n, gelu_tanh_f(g, FULL) * u);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = (j < 2 ? n0 : n1) + tx * 2 + (j & 1);
        if (n < N) {
          float v = acc[i][j];
          if (EPI == ALICE_EPI_SOFTCAP) v = epi * (FULL ? tanh_full(v / epi) : tanh_fast(v / epi));
          store_f32(Y, (size_t)m * N + n, v);
        }
      }
    }
  }
}

// Up to 8 tokens: one wave per output feature streams that feature's weight row once (coalesced, four
// elements a lane a step) against all the tokens' activations; the lanes' partial sums meet in a fixed
// shuffle tree, so a token's result does not depend on the others.  For GeGLU the wave takes the gate
// row and the up row of its feature.
template <typename TA, typename TW, typename TO, int EPI, bool FULL, int MB>
__global__ __launch_bounds__(256) void linear_rows_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                          TO* __restrict__ Y, int M, int N, int K, float epi) {
  const int lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  constexpr int NR = EPI == ALICE_EPI_GEGLU ? 2 : 1;
  float acc[NR][MB];
#pragma unroll
  for (int r = 0; r < NR; ++r)
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[r][m] = 0.f;
  const int K4 = K & ~3;
  for (int k = lane * 4; k < K4; k += 256) {
    float w[NR][4];
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
      for (int e = 0; e < 4; ++e) w[r][e] = load_f32(W, (size_t)(n + r * N) * K + k + e);
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      if (m < M) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float xv = load_f32(A, (size_t)m * K + k + e);
#pragma unroll
          for (int r = 0; r < NR; ++r) acc[r][m] = fmaf(w[r][e], xv, acc[r][m]);
        }
      }
    }
  }
  if (lane < K - K4) {                                       // up to three columns beyond the last whole group of four
    const int k = K4 + lane;
#pragma unroll
    for (int m = 0; m < MB; ++m)
      if (m < M) {
        const float xv = load_f32(A, (size_t)m * K + k);
#pragma unroll
        for (int r = 0; r < NR; ++r) acc[r][m] = fmaf(load_f32(W, (size_t)(n + r * N) * K + k), xv, acc[r][m]);
      }
  }
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    if (m >= M) continue;
    float v[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) v[r] = wave_sum(acc[r][m]);
    if (lane == 0) {
      float o = v[0];
      if (EPI == ALICE_EPI_GEGLU) o = gelu_tanh_f(v[0], FULL) * v[NR - 1];
      if (EPI == ALICE_EPI_SOFTCAP) o = epi * (FULL ? tanh_full(o / epi) : tanh_fast(o / epi));
      store_f32(Y, (size_t)m * N + n, o);
    }
  }
}

template <typename TA, typename TW, typename TO, bool FULL>
int launch_rows(const void* x, const void* w, void* y, int M, int N, int K, int epi, float epi_param, hipStream_t stream) {
  const int grid = ceil_div(N, 4);
#define GO(E, MB) linear_rows_kernel<TA, TW, TO, E, FULL, MB><<<grid, 256, 0, stream>>>((const TA*)x, (const TW*)w, (TO*)y, M, N, K, epi_param)
#define BY_M(E) do { if (M <= 1) GO(E, 1); else if (M <= 2) GO(E, 2); else if (M <= 4) GO(E, 4); else GO(E, 8); } while (0)
  if (epi == ALICE_EPI_NONE) BY_M(ALICE_EPI_NONE);
  else if (epi == ALICE_EPI_GEGLU) BY_M(ALICE_EPI_GEGLU);
  else BY_M(ALICE_EPI_SOFTCAP);
#undef BY_M
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

template <typename TA, typename TW, typename TO, bool FULL>
int launch_tiled(const void* x, const void* w, void* y, int M, int N, int K, int epi, float epi_param,
                 hipStream_t stream) {
  dim3 grid(epi == ALICE_EPI_GEGLU ? ceil_div(N, 32) : ceil_div(N, 64), ceil_div(M, BM));
#define GO(E) linear_tiled_kernel<TA, TW, TO, E, FULL><<<grid, 256, 0, stream>>>((const TA*)x, (const TW*)w, (TO*)y, M, N, K, epi_param)
  if (epi == ALICE_EPI_NONE) GO(ALICE_EPI_NONE);
  else if (epi == ALICE_EPI_GEGLU) GO(ALICE_EPI_GEGLU);
  else GO(ALICE_EPI_SOFTCAP);
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

}  // namespace

int alice_linear_generic(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype,
                         int M, int N, int K, int epi, float epi_param, int full_precision,
                         hipStream_t stream) {
  ALICE_CHECK(dtype_ok(x_dtype) && dtype_ok(w_dtype) && dtype_ok(y_dtype), "linear: unknown dtype");
  ALICE_CHECK(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  ALICE_CHECK(epi == ALICE_EPI_NONE || epi == ALICE_EPI_GEGLU || epi == ALICE_EPI_SOFTCAP,
              "linear: unknown epilogue %d", epi);
  ALICE_CHECK(epi != ALICE_EPI_SOFTCAP || epi_param > 0.f, "linear: softcap must be positive");
  ALICE_CHECK(ceil_div(M, BM) <= 65535, "linear: M=%d has too many row tiles for one launch", M);
  if (M == 0) return 0;
  int rc = 0;
  const bool rows = M <= 8 && N >= 64;                       // few tokens: stream each weight row once
  DISPATCH_DTYPE(x_dtype, TA, DISPATCH_DTYPE(w_dtype, TW, DISPATCH_DTYPE(y_dtype, TO, {
    if (rows)
      rc = full_precision ? launch_rows<TA, TW, TO, true>(x, w, y, M, N, K, epi, epi_param, stream)
                          : launch_rows<TA, TW, TO, false>(x, w, y, M, N, K, epi, epi_param, stream);
    else
      rc = full_precision ? launch_tiled<TA, TW, TO, true>(x, w, y, M, N, K, epi, epi_param, stream)
                          : launch_tiled<TA, TW, TO, false>(x, w, y, M, N, K, epi, epi_param, stream);
  })));
  return rc;
}
