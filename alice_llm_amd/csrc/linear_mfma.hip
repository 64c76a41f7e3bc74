// bfloat16 matrix products on the matrix cores (MFMA 16x16x32, 32-bit accumulation), reading
// weights in a fragment layout that is made once at load.
//
// Fragment layout of W[N, K] (bfloat16): tiles of 16 rows x 32 columns, stored tile by tile as
// [N/16][K/32][64 lanes][8 elements]; lane l = g*16 + r of a tile holds W[n0 + r][k0 + 8g .. 8g+7],
// which is exactly what lane l supplies to the MFMA as its part of the 16x32 operand.  A wave
// therefore loads a whole tile with one fully coalesced 1 KB read and no shuffle through LDS.
// N is padded to a multiple of 16 and K to a multiple of 32 with zeros.
//
// Operand roles: the weight tile is the MFMA's first operand (rows = output features n), the
// activations the second (columns = tokens m).  Lane l then holds D[n = 4*(l/16) + i][m = l%16],
// i = 0..3: four consecutive output features of one token, stored with one vector store.
//
// Two kernels share this: a weight-streaming kernel for up to 64 tokens (decode), whose four waves
// split the inner dimension and add their parts in a fixed order, and a tiled kernel for many
// tokens (prompts).  The math is the reference's y[r] = sum_c W[r,c] x[c] (gguf.rs:4063-4074) with the
// GeGLU (llama3.rs:14519-14534) and softcap (llama3.rs:14606-14611) epilogues.
#include "common.h"
#include "alice_hip.h"
#include "kv_layout.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// A weight fragment of zeros: k-tiles beyond a slice read it instead of the matrix, so that every load of
// the main loops is unconditional and nothing has to be patched after a load.
// (Not declared const: that would put it into the constant address space, and a pointer that may point
// into either space is dereferenced with the slower flat loads.)
__device__ __align__(16) uint32_t g_zero_tile[256];

__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

// The activation fragment of token row `m` (clamped by the caller) at k-tile kt: 8 consecutive elements.
__device__ __forceinline__ u32x4 load_x_frag(const bf16_t* __restrict__ x, int row, bool row_ok, int K, int kt, int g) {
  const int k = kt * 32 + g * 8;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row_ok && k < K) v = *reinterpret_cast<const u32x4*>(x + (size_t)row * K + k);
  return v;
}

// The same fragment when the activations themselves are stored in fragment order
// ([M/16][K/32][64 lanes][8], what a decode step's producers write): one contiguous 1 KB read per wave.
__device__ __forceinline__ u32x4 load_x_frag_f(const bf16_t* __restrict__ x, int mtile, bool ok, int KT, int kt, int lane) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (ok) v = *reinterpret_cast<const u32x4*>(x + ((size_t)((size_t)mtile * KT + kt) * 64 + lane) * 8);
  return v;
}

template <int EPI, bool FULL>
__device__ __forceinline__ float epilogue1(float v, float p) {
  if (EPI == ALICE_EPI_SOFTCAP) return p * (FULL ? tanh_full(v / p) : tanh_fast(v / p));
  return v;
}

template <typename TO>
__device__ __forceinline__ void store4(TO* __restrict__ y, size_t row_off, int n, int N, f32x4 v) {
  if (n + 3 < N && (((size_t)row_off + n) & 3) == 0) {
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<f32x4*>((float*)y + row_off + n) = v;
    } else {
      uint32_t lo = pack_bf16x2(v[0], v[1]);
      uint32_t hi = pack_bf16x2(v[2], v[3]);
      uint2 pk = {lo, hi};
      *reinterpret_cast<uint2*>((bf16_t*)y + row_off + n) = pk;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) store_f32(y, row_off + n + i, v[i]);
  }
}

// Four consecutive output features of token m, stored in fragment order for the next matrix product
// (its inner dimension is this one's N): element (m, n) lies at
// ((m/16 * N/32 + n/32) * 64 + (n%32)/8 * 16 + m%16) * 8 + n%8.  N is a multiple of 32, n of 4.
__device__ __forceinline__ void store4_frag(bf16_t* __restrict__ y, int m, int n, int N, f32x4 v) {
  const size_t off = ((size_t)((size_t)(m >> 4) * (N >> 5) + (n >> 5)) * 64 + ((n & 31) >> 3) * 16 + (m & 15)) * 8 + (n & 7);
  uint2 pk = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  *reinterpret_cast<uint2*>(y + off) = pk;
}

// Row-major, or (bfloat16 only) fragment order.
template <typename TO>
__device__ __forceinline__ void store4_any(TO* __restrict__ y, int y_frag, int m, size_t row_off, int n, int N, f32x4 v) {
  if constexpr (sizeof(TO) == 2) {
    if (y_frag) { store4_frag((bf16_t*)y, m, n, N, v); return; }
  }
  store4(y, row_off, n, N, v);
}

// What the rotation epilogue needs: where q goes, the cache, the tables and the geometry.
struct RopeArgs {
  bf16_t* q_out;
  bf16_t* k_pool;
  bf16_t* v_pool;
  const float* cos_t;
  const float* sin_t;
  const int* positions;
  const int* seq_of_token;
  const int* block_table;
  int bt_stride, nH, nKV, d, page_size, n_pages, layout;
};

// A token as the tiled kernel's rotation epilogue keeps it in LDS, and the elements per staged token there: 256
// features and 8 of padding (a token's stride is 132 words, so that neither 64 lanes on 16 tokens x 4 words nor 16
// tokens x 16 bytes meet in a bank).
struct RopeStagedToken {
  size_t page_base;
  int tp;
  bool valid, page_ok;
};
constexpr int ROPE_PITCH = 264;

// Where token m's keys and values go.
struct RopeToken {
  int pos, tp;
  bool page_ok;
  size_t page_base;
};
__device__ __forceinline__ RopeToken rope_token(const RopeArgs& ra, int m) {
  RopeToken t;
  t.pos = ra.positions[m];
  t.tp = t.pos % ra.page_size;
  const int page = ra.block_table[(size_t)ra.seq_of_token[m] * ra.bt_stride + t.pos / ra.page_size];
  t.page_ok = page >= 0 && page < ra.n_pages;
  t.page_base = (size_t)(t.page_ok ? page : 0) * ra.nKV * ra.page_size * ra.d;
  return t;
}
// The rotation epilogue for four consecutive output features n .. n+3 (in W's row order) of token m.  The
// rows of W are all q heads, all k heads, all v heads, the rows of every q and k head in pair order: the four
// features are two whole rotated pairs (or four elements of a value head).  The sums are rounded to bfloat16
// before the rotation, as they are when the projection and the rotation are separate kernels: both ways give
// the same bits.
// Which head features n .. n+3 belong to and where in it they lie: the same for every token of a tile, so the
// divisions by the head size are done once per tile, not per token.
struct RopeCol { int head, w; };
__device__ __forceinline__ RopeCol rope_col(const RopeArgs& ra, int n) { return RopeCol{n / ra.d, n % ra.d}; }

// The cosines and sines of the two pairs that the four features make (nothing for a value head).
struct RopeTrig { float2 c, s; };
__device__ __forceinline__ RopeTrig rope_trig(const RopeArgs& ra, const RopeToken& t, const RopeCol& col) {
  RopeTrig g{float2{1.f, 1.f}, float2{0.f, 0.f}};
  if (col.head < ra.nH + ra.nKV) {
    g.c = *reinterpret_cast<const float2*>(ra.cos_t + (size_t)t.pos * (ra.d >> 1) + (col.w >> 1));
    g.s = *reinterpret_cast<const float2*>(ra.sin_t + (size_t)t.pos * (ra.d >> 1) + (col.w >> 1));
  }
  return g;
}
__device__ __forceinline__ void rope_store4(const RopeArgs& ra, int m, const RopeToken& t, const RopeCol& col, f32x4 acc,
                                            const RopeTrig& tr) {
  const int d = ra.d, half = d >> 1;
  const int head = col.head, w = col.w;
  float x[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = round_to<bf16_t>(acc[e]);
  if (head < ra.nH + ra.nKV) {
    const int p0 = w >> 1;                                 // the pairs p0 and p0 + 1 of the head
    float l0, h0, l1, h1;
    rotate_pair(x[0], x[1], tr.c.x, tr.s.x, l0, h0);
    rotate_pair(x[2], x[3], tr.c.y, tr.s.y, l1, h1);
    const uint32_t lo = pack_bf16x2(l0, l1), hi = pack_bf16x2(h0, h1);
    if (head < ra.nH) {
      bf16_t* dst = ra.q_out + ((size_t)m * ra.nH + head) * d;
      *reinterpret_cast<uint32_t*>(dst + p0) = lo;
      *reinterpret_cast<uint32_t*>(dst + p0 + half) = hi;
    } else if (t.page_ok) {
      bf16_t* dst = ra.k_pool + t.page_base + (size_t)(head - ra.nH) * ra.page_size * d;
      *reinterpret_cast<uint32_t*>(dst + k_offset(ra.layout, t.tp, p0, d)) = lo;
      *reinterpret_cast<uint32_t*>(dst + k_offset(ra.layout, t.tp, p0 + half, d)) = hi;
    }
  } else if (t.page_ok) {
    bf16_t* dst = ra.v_pool + t.page_base + (size_t)(head - ra.nH - ra.nKV) * ra.page_size * d;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[v_offset(ra.layout, t.tp, w + e, d)] = f32_to_bf16(x[e]);
  }
}
__device__ __forceinline__ void rope_store4(const RopeArgs& ra, int m, const RopeToken& t, int n, f32x4 acc) {
  const RopeCol col = rope_col(ra, n);
  rope_store4(ra, m, t, col, acc, rope_trig(ra, t, col));
}

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

  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j)
        *reinterpret_cast<f32x4*>(red + ((size_t)((wave - 1) * RT * MT + i * MT + j) * 64 + lane) * 4) = acc[i][j];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 0; w < NW - 1; ++w)
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        f32x4 p = *reinterpret_cast<const f32x4*>(red + ((size_t)(w * RT * MT + i * MT + j) * 64 + lane) * 4);
        acc[i][j] += p;
      }

  if constexpr (EPI == ALICE_EPI_ROPE) {
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      if (!row_ok[j]) continue;
      const RopeToken t = rope_token(ra, row[j]);
#pragma unroll
      for (int i = 0; i < RT; ++i)
        if (tile[i] < NT) rope_store4(ra, row[j], t, tile[i] * 16 + g * 4, acc[i][j]);
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

constexpr int WM = 8, WN = 4;   // a wave's tile: 8 x 4 MFMA tiles = 128 tokens x 64 output features

// ---------------------------------------------------------------- tiled, many tokens
// Block: 4 waves side by side along N; every wave computes 128 (or 64) tokens x 64 output features
// (8 x 4 MFMA tiles, 128 accumulator registers per lane) and streams its own weight tiles straight
// from memory.  The block's tokens x 64 inner elements of activations are staged once in LDS (in
// fragment order, so LDS reads and writes are linear) and read by all four waves.  Two stages are kept: while one is used for the
// MFMAs the next one's global loads are in flight, and one barrier per stage suffices.  The grid is
// one-dimensional and mapped so that the blocks that share weight tiles run on the same XCD (blocks
// are dealt to the eight XCDs round robin by their linear index).
constexpr int KC = 2;      // k-tiles per stage

// XF: the activations come in fragment order (a compile-time choice: as a run-time one it cost the
// row-major path a third of its speed).
template <int EPI, typename TO, bool FULL, int TM, bool XF>
__global__ __launch_bounds__(256, 2) void linear_tiled_lds_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wf,
                                                               TO* __restrict__ y, int M, int N, int K, int KT, int NT,
                                                               float epi, int gx, int gy, int kt_per_slice, int y_frag,
                                                               RopeArgs ra) {
  constexpr int XJ = TM / 4;                               // token tiles each wave stages
  // The rotation epilogue stages 64 tokens x 256 features in the same memory afterwards (ROPE_PITCH elements a token).
  constexpr int XS_WORDS = 2 * KC * TM * 64 * 4;
  constexpr int LDS_WORDS = (EPI == ALICE_EPI_ROPE && XS_WORDS < 64 * ROPE_PITCH / 2) ? 64 * ROPE_PITCH / 2 : XS_WORDS;
  __shared__ __align__(16) uint32_t xs_raw[LDS_WORDS];
  u32x4* xs = reinterpret_cast<u32x4*>(xs_raw);            // [2][KC][TM][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  // Blocks go to the XCDs round robin by index; XCD x works through the x-th eighth of the tiles in
  // column-major order, so that tiles with the same weight columns meet in one L2.
  const int id = blockIdx.x, xcd = id & 7, local = id >> 3;
  const int per = (gx * gy + 7) >> 3;
  const int item = xcd * per + local;
  if (local >= per || item >= gx * gy) return;
  const int bx = item / gy, by = item % gy;
  const int m0 = by * (16 * TM);
  int tile[WN];
#pragma unroll
  for (int i = 0; i < WN; ++i) {
    if (EPI == ALICE_EPI_GEGLU) {
      const int pair = (bx * 4 + wave) * (WN / 2) + (i >> 1);
      tile[i] = (i & 1) ? N / 16 + pair : pair;
      if (pair >= N / 16) tile[i] = NT;
    } else {
      tile[i] = (bx * 4 + wave) * WN + i;
    }
  }
  // Loads are unconditional (see the streaming kernel): rows and tiles beyond the matrix are clamped, and
  // k-tiles beyond the slice bring zero weights.
  const bf16_t* xsrc[XJ];        // this lane's place in the activations at k-tile 0, for the token tiles it stages
#pragma unroll
  for (int j = 0; j < XJ; ++j) {
    if constexpr (XF) xsrc[j] = x + ((size_t)min((m0 >> 4) + XJ * wave + j, (M - 1) >> 4) * KT * 64 + lane) * 8;
    else xsrc[j] = x + (size_t)min(m0 + (XJ * wave + j) * 16 + r, M - 1) * K;
  }
  const bf16_t* wsrc[WN];
#pragma unroll
  for (int i = 0; i < WN; ++i) wsrc[i] = wf + (size_t)min(tile[i], NT - 1) * KT * 512 + lane * 8;

  f32x4 acc[WN][TM];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 xr[KC][XJ], wk[KC][WN];
  const int kt_base = blockIdx.y * kt_per_slice, kt_end = min(KT, kt_base + kt_per_slice);
  auto stage_load = [&](int s) {
#pragma unroll
    for (int kc = 0; kc < KC; ++kc)
#pragma unroll
      for (int j = 0; j < XJ; ++j) {
        const int kt = max(0, min(kt_base + s * KC + kc, kt_end - 1));      // past the slice: the weights are zeros
        if constexpr (XF) xr[kc][j] = *reinterpret_cast<const u32x4*>(xsrc[j] + (size_t)kt * 512);
        else xr[kc][j] = *reinterpret_cast<const u32x4*>(xsrc[j] + min(kt * 32 + g * 8, K - 8));
      }
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int kc = 0; kc < KC; ++kc)
#pragma unroll
      for (int j = 0; j < XJ; ++j) xs[((buf * KC + kc) * TM + XJ * wave + j) * 64 + lane] = xr[kc][j];
  };
  const bf16_t* zero = reinterpret_cast<const bf16_t*>(g_zero_tile) + lane * 8;
  auto w_load = [&](int rel, u32x4 (&w)[WN]) {                // rel: k-tile relative to the slice
    const int kt = kt_base + rel;
    const bool kok = kt < kt_end;
#pragma unroll
    for (int i = 0; i < WN; ++i) w[i] = *reinterpret_cast<const u32x4*>(kok ? wsrc[i] + (size_t)kt * 512 : zero);
  };
  // blockIdx.y: the slice of the inner dimension this block sums (its own partial result y[slice][M][N])
  const int kt_lo = blockIdx.y * kt_per_slice, kt_hi = min(KT, kt_lo + kt_per_slice);
  const int S = (kt_hi - kt_lo + KC - 1) / KC;
  y += (size_t)blockIdx.y * M * N;
  stage_load(0);
  stage_store(0);
#pragma unroll
  for (int kc = 0; kc < KC; ++kc) {
    w_load(kc, wk[kc]);
    __builtin_amdgcn_sched_barrier(0);
  }
  // Loads run one stage ahead and are unconditional (a k-tile beyond the slice in the last, partial stage
  // reads the zero tile); the scheduling barriers keep them where they are issued, so that each wait is for
  // the oldest loads only.
  auto stage_mfma = [&](int s, bool more) {
    u32x4 xf[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) xf[j] = xs[(((s & 1) * KC) * TM + j) * 64 + lane];
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
      const int kt_next = kt_base + (s + 1) * KC + kc;       // what this k-tile's weight registers hold next
      const bool kok = kt_next < kt_end;
#pragma unroll
      for (int i = 0; i < WN; ++i) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          acc[i][j] = mfma16(wk[kc][i], xf[j], acc[i][j]);
          // this token tile's fragment has had its last use: read the next k-tile's into the same registers
          if (i == WN - 1 && kc + 1 < KC) xf[j] = xs[(((s & 1) * KC + kc + 1) * TM + j) * 64 + lane];
        }
        if (more) {
          // this weight tile's registers are free again: fetch the same tile of the next stage now, so that the
          // loads of a stage are spread over its products instead of arriving at the memory system in a burst
          __builtin_amdgcn_sched_barrier(0);
          wk[kc][i] = *reinterpret_cast<const u32x4*>(kok ? wsrc[i] + (size_t)kt_next * 512 : zero);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };
  for (int s = 0; s + 1 < S; ++s) {
    stage_load(s + 1);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    stage_mfma(s, true);
    stage_store((s + 1) & 1);
  }
  if (S > 0) {                   // the last stage has nothing to fetch
    __syncthreads();
    stage_mfma(S - 1, false);
  }

  if constexpr (EPI == ALICE_EPI_ROPE) {
    // The rotated values go to their places through LDS, 64 tokens at a time: a lane holds two pairs of a token
    // (4-byte pieces of 16 different rows of q or of the cache), eight such stores per token tile and wave (measured:
    // 4 to 6 % of the kernel against the staging below).  Staged, a token's 16 features of a weight tile become two runs of eight
    // neighbouring elements of a head (the low and the high halves of eight pairs; a value head's 16 elements as
    // they are), and every thread then moves 16-byte runs: along a token for q and for row-major caches, along 16
    // tokens for keys in fragment order (a 1 KB tile per wave when the tokens start at a multiple of 16), and for
    // values in fragment order eight tokens of one element at a time, which is that layout's 16-byte unit (when 32
    // tokens are consecutive places of one sequence from a multiple of 32 on; one by one otherwise).
    __shared__ RopeStagedToken tinfo[64];
    __shared__ int group_ok[2];
    bf16_t* stage = reinterpret_cast<bf16_t*>(xs_raw);
    const int tid = threadIdx.x;
    const int n_tile0 = bx * 4 * WN;
    const int head0 = n_tile0 * 16 / ra.d;
    const bool key_block = ra.layout == 1 && head0 >= ra.nH && head0 < ra.nH + ra.nKV;
    const bool value_block = ra.layout == 1 && head0 >= ra.nH + ra.nKV;
    // Every token's place first, then the cosines and sines one token tile ahead of their use: the loads of a
    // tile are independent and in flight together.
    RopeToken tk[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) tk[j] = rope_token(ra, min(m0 + j * 16 + r, M - 1));
    RopeCol col[WN];
#pragma unroll
    for (int i = 0; i < WN; ++i) col[i] = rope_col(ra, min(tile[i], NT - 1) * 16 + g * 4);
    RopeTrig tr[2][WN];
    auto trig = [&](int j, RopeTrig (&o)[WN]) {
#pragma unroll
      for (int i = 0; i < WN; ++i) o[i] = rope_trig(ra, tk[j], col[i]);
    };
    trig(0, tr[0]);
    auto emit = [&](int mb, int t, int c) {                  // run c (eight elements) of staged token t
      const int nt = n_tile0 + (c >> 1);
      const RopeStagedToken ti = tinfo[t];
      if (nt >= NT || !ti.valid) return;
      const int d = ra.d, head = nt * 16 / d, w0 = nt * 16 % d;
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + t * ROPE_PITCH + c * 8);
      if (head < ra.nH) {
        const int dim0 = (w0 >> 1) + (c & 1) * (d >> 1);
        *reinterpret_cast<u32x4*>(ra.q_out + ((size_t)(mb + t) * ra.nH + head) * d + dim0) = v;
      } else if (!ti.page_ok) {
        return;
      } else if (head < ra.nH + ra.nKV) {
        const int dim0 = (w0 >> 1) + (c & 1) * (d >> 1);
        bf16_t* dst = ra.k_pool + ti.page_base + (size_t)(head - ra.nH) * ra.page_size * d;
        *reinterpret_cast<u32x4*>(dst + k_offset(ra.layout, ti.tp, dim0, d)) = v;
      } else {
        const int dim0 = w0 + (c & 1) * 8;
        bf16_t* dst = ra.v_pool + ti.page_base + (size_t)(head - ra.nH - ra.nKV) * ra.page_size * d;
        if (ra.layout == 0) {
          *reinterpret_cast<u32x4*>(dst + (size_t)ti.tp * d + dim0) = v;
        } else {
          const bf16_t* e8 = stage + t * ROPE_PITCH + c * 8;
#pragma unroll
          for (int e = 0; e < 8; ++e) dst[v_offset(1, ti.tp, dim0 + e, d)] = e8[e];
        }
      }
    };
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int mb = m0 + (j & ~3) * 16;                     // the first of the 64 tokens being staged
      if ((j & 3) == 0) {
        __syncthreads();                                     // the memory's last readers are done
        if (tid < 64) {
          const int m = mb + tid, mc = min(m, M - 1), first = min(mb + (tid & 32), M - 1);
          const RopeToken t = rope_token(ra, mc);
          tinfo[tid] = RopeStagedToken{t.page_base, t.tp, m < M, t.page_ok};
          const int pos0 = ra.positions[first];
          const bool in_run = m < M && t.page_ok && ra.seq_of_token[mc] == ra.seq_of_token[first] &&
                              t.pos == pos0 + (tid & 31) && (pos0 & 31) == 0 && (ra.page_size & 31) == 0;
          const unsigned long long run = __ballot(in_run);
          if (tid == 0) {
            group_ok[0] = (run & 0xffffffffull) == 0xffffffffull;
            group_ok[1] = (run >> 32) == 0xffffffffull;
          }
        }
      }
      if (j + 1 < TM) trig(j + 1, tr[(j + 1) & 1]);
      uint32_t* row = reinterpret_cast<uint32_t*>(stage + ((j & 3) * 16 + r) * ROPE_PITCH + wave * (16 * WN));
#pragma unroll
      for (int i = 0; i < WN; ++i) {
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = round_to<bf16_t>(acc[i][j][e]);
        if (col[i].head < ra.nH + ra.nKV) {
          float l0, h0, l1, h1;
          rotate_pair(x[0], x[1], tr[j & 1][i].c.x, tr[j & 1][i].s.x, l0, h0);
          rotate_pair(x[2], x[3], tr[j & 1][i].c.y, tr[j & 1][i].s.y, l1, h1);
          row[i * 8 + g] = pack_bf16x2(l0, l1);              // pairs 2 g and 2 g + 1 of the tile's eight: the low halves
          row[i * 8 + 4 + g] = pack_bf16x2(h0, h1);          // and the high halves, eight elements on
        } else {
          row[i * 8 + 2 * g] = pack_bf16x2(x[0], x[1]);
          row[i * 8 + 2 * g + 1] = pack_bf16x2(x[2], x[3]);
        }
      }
      if ((j & 3) != 3) continue;
      __syncthreads();
      if (value_block) {
        // wave items: (32 tokens, a 16-element tile of a head); a lane takes element lane % 16 of the tokens
        // 4 (lane / 16) .. + 3 and the same 16 further on
#pragma unroll 1
        for (int it = 0; it < 8; ++it) {
          const int item = it * 4 + wave, grp = item >> 4, vt = item & 15, nt = n_tile0 + vt;
          if (nt >= NT) continue;
          const int d = ra.d, head = nt * 16 / d, e = nt * 16 % d + (lane & 15), a = lane >> 4;
          const bf16_t* src = stage + (grp * 32 + 4 * a) * ROPE_PITCH + vt * 16 + (lane & 15);
          const size_t head_off = (size_t)(head - ra.nH - ra.nKV) * ra.page_size * d;
          if (group_ok[grp]) {
            uint16_t h[8];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              h[q] = src[q * ROPE_PITCH].bits;
              h[4 + q] = src[(16 + q) * ROPE_PITCH].bits;
            }
            const u32x4 v = {h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16, h[4] | (uint32_t)h[5] << 16,
                             h[6] | (uint32_t)h[7] << 16};
            const RopeStagedToken ti = tinfo[grp * 32];
            *reinterpret_cast<u32x4*>(ra.v_pool + ti.page_base + head_off + v_offset(1, ti.tp + 4 * a, e, d)) = v;
          } else {
#pragma unroll
            for (int q = 0; q < 8; ++q) {
              const int t = grp * 32 + 4 * a + (q & 3) + 16 * (q >> 2);
              const RopeStagedToken ti = tinfo[t];
              if (ti.valid && ti.page_ok)
                ra.v_pool[ti.page_base + head_off + v_offset(1, ti.tp, e, d)] = src[((q & 3) + 16 * (q >> 2)) * ROPE_PITCH];
            }
          }
        }
      } else if (key_block) {
        // wave items: (16 tokens, 32 elements of one half of a head); a lane takes run lane / 16 of token lane % 16
#pragma unroll 1
        for (int it = 0; it < 8; ++it) {
          const int item = it * 4 + wave;
          emit(mb, 16 * (item >> 3) + (lane & 15), 8 * ((item >> 1) & 3) + 2 * (lane >> 4) + (item & 1));
        }
      } else {
#pragma unroll 2
        for (int k = 0; k < 8; ++k) emit(mb, (tid >> 5) + 8 * k, tid & 31);
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + j * 16 + r;
    if (m >= M) continue;
    const size_t row_off = (size_t)m * N;
    if (EPI == ALICE_EPI_GEGLU) {
#pragma unroll
      for (int p = 0; p < WN / 2; ++p) {
        if (tile[2 * p] >= NT) continue;
        const int n = tile[2 * p] * 16 + g * 4;
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = gelu_tanh_f(acc[2 * p][j][e], FULL) * acc[2 * p + 1][j][e];
        store4_any(y, y_frag, m, row_off, n, N, o);
      }
    } else {
#pragma unroll
      for (int i = 0; i < WN; ++i) {
        if (tile[i] >= NT) continue;
        const int n = tile[i] * 16 + g * 4;
        f32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = epilogue1<EPI, FULL>(acc[i][j][e], epi);
        store4_any(y, y_frag, m, row_off, n, N, o);
      }
    }
  }
}

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

template <int EPI, typename TO>
int launch_tiled(const void* x, const void* w, void* y, int M, int N, int K, int split, float epi, int x_frag, int y_frag,
                 hipStream_t s, const RopeArgs& ra = RopeArgs{}) {
  const int KT = (K + 31) / 32, NT = (N * (EPI == ALICE_EPI_GEGLU ? 2 : 1) + 15) / 16;
  const int per = ceil_div(KT, split);
  const int gx = EPI == ALICE_EPI_GEGLU ? ceil_div(N / 16, 4 * WN / 2) : ceil_div(NT, 4 * WN);
  int gy = ceil_div(M, 16 * WM);
  // 128 tokens a block, or 64 when that leaves most of the chip without a block (measured at N = 2304 and 4096:
  // 216 and 256 blocks of 128 tokens beat twice as many of 64, 128 blocks do not; the same with the rotation
  // epilogue since its stores go through LDS)
  const bool high = gx * gy * split >= 192 || M <= 64;
  if (!high) gy = ceil_div(M, 64);
  dim3 grid(8 * ceil_div(gx * gy, 8), split);
#define GO(TMV, XFV) \
  linear_tiled_lds_kernel<EPI, TO, false, TMV, XFV><<<grid, 256, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, (TO*)y, M, N, K, KT, NT, epi, gx, gy, per, y_frag, ra)
  if (x_frag) { if (high) GO(8, true); else GO(4, true); }
  else { if (high) GO(8, false); else GO(4, false); }
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" int alice_has_mfma_linear() { return 1; }

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
    return skinny_cost(M, N, K, ALICE_EPI_NONE, skinny_row_tiles(M, N, ALICE_EPI_NONE, sp, K), sp);
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
  if (M > 64) {
    // Tiled kernel: 128 tokens x 256 features a block, two blocks a CU.  Narrow outputs leave most of the
    // chip idle; slices of the inner dimension fill it.  Cost of s slices, relative to one block a CU
    // running the whole inner dimension: the busiest CU runs n = ceil(blocks s / 256) blocks of 1/s the
    // length, two at a time at 1.7 times the time of one; every extra slice writes and reads another
    // [M, N] float32 partial result (both constants fitted to measurements at N = 2304, K = 2048 and 9216).
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
  const int KT = (K + 31) / 32;
  if (M > 32) return skinny_split_with_six(M, N, K, KT >= 128 ? 4 : (KT >= 32 ? 2 : 1));
  const int groups = ceil_div(ceil_div(N, 16), skinny_row_tiles_base(M, N, ALICE_EPI_NONE, 1, K));
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
  ALICE_CHECK(!(variant == ALICE_LINEAR_SKINNY && M > 64), "linear: the streaming kernel takes at most 64 rows, found %d", M);
  ALICE_CHECK(split_k == 1 || (epi == ALICE_EPI_NONE && y_dtype == DT_F32 && true),
              "linear: partial sums need no epilogue and float32 output");
  ALICE_CHECK(ceil_div(M, 128) <= 65535, "linear: too many rows for one launch (%d)", M);
  ALICE_CHECK(y_layout == ALICE_LAYOUT_ROW || (y_layout == ALICE_LAYOUT_FRAG16 && y_dtype == DT_BF16 && N % 32 == 0 &&
                                                split_k == 1 && epi != ALICE_EPI_SOFTCAP),
              "linear: output in fragment order needs bfloat16, N %% 32 == 0, no softcap and no partial sums");
  const int x_frag = x_layout == ALICE_LAYOUT_FRAG16, y_frag = y_layout == ALICE_LAYOUT_FRAG16;
#define BY_EPI(FN, ...)                                                                            \
  do {                                                                                             \
    if (y_dtype == DT_F32) {                                                                       \
      if (epi == ALICE_EPI_NONE) return FN<ALICE_EPI_NONE, float>(__VA_ARGS__);                    \
      if (epi == ALICE_EPI_GEGLU) return FN<ALICE_EPI_GEGLU, float>(__VA_ARGS__);                  \
      return FN<ALICE_EPI_SOFTCAP, float>(__VA_ARGS__);                                            \
    } else {                                                                                       \
      if (epi == ALICE_EPI_NONE) return FN<ALICE_EPI_NONE, bf16_t>(__VA_ARGS__);                   \
      if (epi == ALICE_EPI_GEGLU) return FN<ALICE_EPI_GEGLU, bf16_t>(__VA_ARGS__);                 \
      return FN<ALICE_EPI_SOFTCAP, bf16_t>(__VA_ARGS__);                                           \
    }                                                                                              \
  } while (0)
  if (skinny) BY_EPI(skinny_by_shape, x, w, y, M, N, K, split_k, epi_param, x_frag, y_frag, stream);
  BY_EPI(launch_tiled, x, w, y, M, N, K, split_k, epi_param, x_frag, y_frag, stream, RopeArgs{});
#undef BY_EPI
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
  if (M > 64) return launch_tiled<ALICE_EPI_ROPE, bf16_t>(x, w, nullptr, M, N, K, 1, 0.f, x_frag, 0, stream, ra);
  const int rt = skinny_row_tiles(M, N, ALICE_EPI_NONE, 1, K);
#define GO(RT, MT) return launch_skinny<RT, MT, ALICE_EPI_ROPE, bf16_t>(x, w, nullptr, M, N, K, 1, 0.f, x_frag, 0, stream, ra)
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
