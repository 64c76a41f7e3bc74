// Embedding gather, the fused residual-add / RMSNorm pair, and the stand-alone softcap.
//
// Reference formulas: embedding row copy and sqrt(hidden) scale llama3.rs:13686-13703;
// RMSNorm llama3.rs:5244-5256 (here with the weight applied as offset + w); post norms
// before the residual add llama3.rs:14460-14470, 14543-14557; softcap llama3.rs:14606-14611.
#include "common.h"
#include "alice_hip.h"

// ---------------------------------------------------------------- embedding
// Row-major table [V, H]: out[t, :] = table[tok[t], :] * scale.  A token id outside the table
// gives a zero row (the host rejects such ids before the launch; this keeps the kernel in bounds).
template <typename TW>
__global__ void embed_rows_kernel(const int* __restrict__ tok, const TW* __restrict__ table,
                                  float* __restrict__ out, int H, int V, float scale) {
  const int t = blockIdx.x;
  const int id = tok[t];
  const bool ok = id >= 0 && id < V;
  const TW* row = table + (size_t)(ok ? id : 0) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    out[(size_t)t * H + i] = ok ? load_f32(row, i) * scale : 0.f;
}

// Table in the 16x32 fragment layout of the bfloat16 matrix kernels (see linear_mfma.hip):
// element (n, k) lies at ((n/16 * KT + k/32) * 64 + ((k%32)/8)*16 + n%16) * 8 + k%8, KT = Kp/32.
__global__ void embed_rows_frag_kernel(const int* __restrict__ tok, const bf16_t* __restrict__ table,
                                       float* __restrict__ out, int H, int V, int KT, float scale) {
  const int t = blockIdx.x;
  const int id = tok[t];
  const bool ok = id >= 0 && id < V;
  const int n = ok ? id : 0;
  const size_t tile_row = (size_t)(n >> 4) * KT;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    size_t off = ((tile_row + (i >> 5)) * 64 + (size_t)(((i & 31) >> 3) * 16 + (n & 15))) * 8 + (i & 7);
    out[(size_t)t * H + i] = ok ? bf16_to_f32(table[off]) * scale : 0.f;
  }
}

extern "C" int alice_embed(const int* tokens, const void* table, int table_dtype, int table_layout,
                           float* out, int T, int H, int V, float scale, hipStream_t stream) {
  ALICE_CHECK(T >= 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  ALICE_CHECK(dtype_ok(table_dtype), "embed: unknown table dtype %d", table_dtype);
  if (T == 0) return 0;
  if (table_layout == ALICE_LAYOUT_FRAG16) {
    ALICE_CHECK(table_dtype == DT_BF16, "embed: the fragment layout holds bfloat16 only");
    embed_rows_frag_kernel<<<T, 256, 0, stream>>>(tokens, (const bf16_t*)table, out, H, V, (H + 31) / 32, scale);
  } else {
    ALICE_CHECK(table_layout == ALICE_LAYOUT_ROW, "embed: unknown layout %d", table_layout);
    DISPATCH_DTYPE(table_dtype, TW, (embed_rows_kernel<TW><<<T, 256, 0, stream>>>(tokens, (const TW*)table, out, H, V, scale)));
  }
  ALICE_LAUNCH_CHECK();
  return 0;
}

// Where element (row r, column i) of a [T, H] bfloat16 output goes: row-major, or fragment order for the
// matrix-core kernels ([T/16][H/32][64][8], see linear_mfma.hip).
__device__ __forceinline__ size_t out_index(int layout, int r, int i, int H) {
  if (layout == 0) return (size_t)r * H + i;
  return ((size_t)((size_t)(r >> 4) * (H >> 5) + (i >> 5)) * 64 + ((i & 31) >> 3) * 16 + (r & 15)) * 8 + (i & 7);
}

// ---------------------------------------------------------------- residual add + norms
// One block per row r (source row rows ? rows[r] : r):
//   b   = sum over `n_partials` slices of `branch` (slice stride `partial_stride` elements)
//   b   = w_post ? b * rsqrt(mean(b^2) + eps_post) * (off_post + w_post) : b
//   x   = resid + b, written back to resid            (only when branch is given)
//   out = x * rsqrt(mean(x^2) + eps_pre) * (off_pre + w_pre)   (only when out is given;
//         out = x when w_pre is absent)
// All sums are 32-bit; FULL selects 1/sqrtf over the fast reciprocal square root.
template <typename TW, typename TO, bool FULL>
__global__ void add_norm_kernel(float* __restrict__ resid, const float* __restrict__ branch,
                                int n_partials, size_t partial_stride,
                                const TW* __restrict__ w_post, const TW* __restrict__ w_pre,
                                TO* __restrict__ out, const int* __restrict__ rows, int H,
                                float eps_post, float eps_pre, float off_post, float off_pre, int out_layout) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * H;
  float* x = resid + src;
  float ss_x = 0.f;
  if (branch) {
    const float* b = branch + src;
    float inv_b = 1.f;
    if (w_post) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = b[i];
        for (int p = 1; p < n_partials; ++p) v += b[i + p * partial_stride];
        ss += v * v;
      }
      ss = block_sum(ss, red);
      float mean = ss / (float)H;
      inv_b = FULL ? 1.f / sqrtf(mean + eps_post) : rsqrtf(mean + eps_post);
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float v = b[i];
      for (int p = 1; p < n_partials; ++p) v += b[i + p * partial_stride];
      if (w_post) v = v * inv_b * (off_post + load_f32(w_post, i));
      float xv = x[i] + v;
      x[i] = xv;
      ss_x += xv * xv;
    }
  } else if (out && w_pre) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float xv = x[i];
      ss_x += xv * xv;
    }
  }
  if (!out) return;
  TO* o = out;
  if (!w_pre) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) store_f32(o, out_index(out_layout, r, i, H), x[i]);
    return;
  }
  ss_x = block_sum(ss_x, red);
  float mean = ss_x / (float)H;
  float inv = FULL ? 1.f / sqrtf(mean + eps_pre) : rsqrtf(mean + eps_pre);
  // Each thread re-reads the elements it wrote itself above, so no barrier is needed.
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    store_f32(o, out_index(out_layout, r, i, H), x[i] * inv * (off_pre + load_f32(w_pre, i)));
}

// The same operation with a row held in registers (EPT elements per thread): every operand is read once
// and the three phases need no second trip through memory.  Used when the row fits.
//
// All loads come first, unconditionally (indices beyond the row are clamped to its last element and the
// values replaced by zeros afterwards; the launch leaves few such threads), and nothing is converted or
// used before the last one is issued: the operands are a few hundred KB that other kernels have just
// written, they come from memory, and every load that waits for an earlier one costs a round trip.
template <typename T> struct raw_of;
template <> struct raw_of<float> { typedef float type; };
template <> struct raw_of<bf16_t> { typedef uint16_t type; };
__device__ __forceinline__ float raw_to_f32(float v) { return v; }
__device__ __forceinline__ float raw_to_f32(uint16_t v) { return bf16_bits_to_f32(v); }

template <int EPT, int C, int CMAX>
__device__ __forceinline__ void load_partials(float (&t)[EPT][CMAX], const float* __restrict__ row, const int (&idx)[EPT],
                                              int p0, int n_partials, size_t partial_stride) {
#pragma unroll
  for (int j = 0; j < EPT; ++j)
#pragma unroll
    for (int p = 0; p < C; ++p) t[j][p] = row[idx[j] + (size_t)min(p0 + p, n_partials - 1) * partial_stride];
}

template <typename TW, typename TO, bool FULL, int EPT>
__global__ void add_norm_regs_kernel(float* __restrict__ resid, const float* __restrict__ branch,
                                     int n_partials, size_t partial_stride,
                                     const TW* __restrict__ w_post, const TW* __restrict__ w_pre,
                                     TO* __restrict__ out, const int* __restrict__ rows, int H,
                                     float eps_post, float eps_pre, float off_post, float off_pre, int out_layout) {
  typedef typename raw_of<TW>::type RW;
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * H;
  int idx[EPT];
  bool in_row[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    in_row[j] = i < H;
    idx[j] = min(i, H - 1);
  }
  // ---- loads
  constexpr int CMAX = EPT >= 8 ? 4 : 8;        // partial sums in flight per element (registers)
  float xv[EPT], bv[EPT], t[EPT][CMAX];
  RW wq_raw[EPT], wp_raw[EPT];
  const int chunk = n_partials <= 1 ? 1 : (n_partials <= 2 ? 2 : (n_partials <= 4 ? 4 : CMAX));
#pragma unroll
  for (int j = 0; j < EPT; ++j) xv[j] = resid[src + idx[j]];
  if (w_pre) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) wq_raw[j] = reinterpret_cast<const RW*>(w_pre)[idx[j]];
  }
  if (branch) {
    if (w_post) {
#pragma unroll
      for (int j = 0; j < EPT; ++j) wp_raw[j] = reinterpret_cast<const RW*>(w_post)[idx[j]];
    }
    if (chunk == 1) load_partials<EPT, 1, CMAX>(t, branch + src, idx, 0, n_partials, partial_stride);
    else if (chunk == 2) load_partials<EPT, 2, CMAX>(t, branch + src, idx, 0, n_partials, partial_stride);
    else if (chunk == 4) load_partials<EPT, 4, CMAX>(t, branch + src, idx, 0, n_partials, partial_stride);
    else load_partials<EPT, CMAX, CMAX>(t, branch + src, idx, 0, n_partials, partial_stride);
  }
  // ---- arithmetic
  float wq[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    xv[j] = in_row[j] ? xv[j] : 0.f;
    wq[j] = (w_pre && in_row[j]) ? raw_to_f32(wq_raw[j]) : 0.f;
    bv[j] = 0.f;
  }
  if (branch) {
    // partial sums are added in their order, CMAX at a time
    for (int p0 = 0; p0 < n_partials; p0 += CMAX) {
      if (p0 > 0) load_partials<EPT, CMAX, CMAX>(t, branch + src, idx, p0, n_partials, partial_stride);
#pragma unroll
      for (int j = 0; j < EPT; ++j)
#pragma unroll
        for (int p = 0; p < CMAX; ++p)
          if (p < chunk) bv[j] += (in_row[j] && p0 + p < n_partials) ? t[j][p] : 0.f;
    }
    if (w_post) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < EPT; ++j) ss += bv[j] * bv[j];
      ss = block_sum(ss, red);
      const float mean = ss / (float)H;
      const float inv_b = FULL ? 1.f / sqrtf(mean + eps_post) : rsqrtf(mean + eps_post);
#pragma unroll
      for (int j = 0; j < EPT; ++j) bv[j] = bv[j] * inv_b * (off_post + (in_row[j] ? raw_to_f32(wp_raw[j]) : 0.f));
    }
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      xv[j] += bv[j];
      if (in_row[j]) resid[src + idx[j]] = xv[j];
    }
  }
  if (!out) return;
  TO* o = out;
  float inv = 1.f;
  if (w_pre) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < EPT; ++j) ss += xv[j] * xv[j];      // elements beyond H are zero
    ss = block_sum(ss, red);
    const float mean = ss / (float)H;
    inv = FULL ? 1.f / sqrtf(mean + eps_pre) : rsqrtf(mean + eps_pre);
  }
#pragma unroll
  for (int j = 0; j < EPT; ++j)
    if (in_row[j]) store_f32(o, out_index(out_layout, r, idx[j], H), w_pre ? xv[j] * inv * (off_pre + wq[j]) : xv[j]);
}

// The same operation for many rows (prompts): one wave per row, four rows a block, four consecutive
// elements a lane at a time (H a multiple of 4, at most 256 * K4); or, for rows too wide for one wave's
// registers, two waves per row (WPR = 2, at most 512 * K4 elements: the first wave takes the first 256 * K4),
// whose sums meet in LDS.  Reduction orders differ from the block-per-row kernels by rounding only.
template <typename TW> __device__ __forceinline__ float4 load4_f32(const TW* p, int e);
template <> __device__ __forceinline__ float4 load4_f32<float>(const float* p, int e) { return *reinterpret_cast<const float4*>(p + e); }
template <> __device__ __forceinline__ float4 load4_f32<bf16_t>(const bf16_t* p, int e) {
  const uint2 v = *reinterpret_cast<const uint2*>(p + e);
  return float4{bf16_bits_to_f32(v.x & 0xffffu), bf16_bits_to_f32(v.x >> 16), bf16_bits_to_f32(v.y & 0xffffu), bf16_bits_to_f32(v.y >> 16)};
}

template <typename TW, typename TO, bool FULL, int K4, int WPR>
__global__ __launch_bounds__(256) void add_norm_rows_kernel(float* __restrict__ resid, const float* __restrict__ branch,
                                                            int n_partials, size_t partial_stride,
                                                            const TW* __restrict__ w_post, const TW* __restrict__ w_pre,
                                                            TO* __restrict__ out, int T, int H,
                                                            float eps_post, float eps_pre, float off_post, float off_pre,
                                                            int out_layout) {
  __shared__ float red[2][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, part = wave % WPR;
  const int r_own = blockIdx.x * (4 / WPR) + wave / WPR;
  if (WPR == 1 && r_own >= T) return;
  const bool row_ok = r_own < T;                              // two waves a row: every wave reaches the barriers
  const int r = row_ok ? r_own : T - 1;
  const size_t src = (size_t)r * H;
  int e[K4];
  bool ok[K4];
#pragma unroll
  for (int k = 0; k < K4; ++k) {
    const int i = ((part * K4 + k) * 64 + lane) * 4;
    ok[k] = i < H && row_ok;
    e[k] = min(i, H - 4);                                    // clamped: loads are unconditional
  }
  // the row's sum of squares from its waves' shares, the same addends in the same order in both
  auto row_sum = [&](float ss, int which) {
    ss = wave_sum(ss);
    if constexpr (WPR == 2) {
      if (lane == 0) red[which][wave] = ss;
      __syncthreads();
      ss = red[which][wave & ~1] + red[which][wave | 1];
    }
    return ss;
  };
  const float4 zero4 = {0.f, 0.f, 0.f, 0.f};
  float4 xv[K4], bv[K4];
#pragma unroll
  for (int k = 0; k < K4; ++k) xv[k] = *reinterpret_cast<const float4*>(resid + src + e[k]);
#pragma unroll
  for (int k = 0; k < K4; ++k) bv[k] = zero4;
  if (branch) {
    for (int p = 0; p < n_partials; ++p) {                   // partial sums in their order
      float4 t[K4];
#pragma unroll
      for (int k = 0; k < K4; ++k) t[k] = *reinterpret_cast<const float4*>(branch + (size_t)p * partial_stride + src + e[k]);
#pragma unroll
      for (int k = 0; k < K4; ++k) { bv[k].x += t[k].x; bv[k].y += t[k].y; bv[k].z += t[k].z; bv[k].w += t[k].w; }
    }
  }
#pragma unroll
  for (int k = 0; k < K4; ++k) {
    if (!ok[k]) { xv[k] = zero4; bv[k] = zero4; }
  }
  if (branch) {
    if (w_post) {
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < K4; ++k) ss += bv[k].x * bv[k].x + bv[k].y * bv[k].y + bv[k].z * bv[k].z + bv[k].w * bv[k].w;
      ss = row_sum(ss, 0);
      const float mean = ss / (float)H;
      const float inv_b = FULL ? 1.f / sqrtf(mean + eps_post) : rsqrtf(mean + eps_post);
#pragma unroll
      for (int k = 0; k < K4; ++k) {
        const float4 w = load4_f32<TW>(w_post, e[k]);
        bv[k].x = bv[k].x * inv_b * (off_post + w.x);
        bv[k].y = bv[k].y * inv_b * (off_post + w.y);
        bv[k].z = bv[k].z * inv_b * (off_post + w.z);
        bv[k].w = bv[k].w * inv_b * (off_post + w.w);
      }
    }
#pragma unroll
    for (int k = 0; k < K4; ++k) {
      xv[k].x += bv[k].x; xv[k].y += bv[k].y; xv[k].z += bv[k].z; xv[k].w += bv[k].w;
      if (ok[k]) *reinterpret_cast<float4*>(resid + src + e[k]) = xv[k];
    }
  }
  if (!out) return;
  float inv = 1.f;
  if (w_pre) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < K4; ++k) ss += xv[k].x * xv[k].x + xv[k].y * xv[k].y + xv[k].z * xv[k].z + xv[k].w * xv[k].w;
    ss = row_sum(ss, 1);
    const float mean = ss / (float)H;
    inv = FULL ? 1.f / sqrtf(mean + eps_pre) : rsqrtf(mean + eps_pre);
  }
#pragma unroll
  for (int k = 0; k < K4; ++k) {
    if (!ok[k]) continue;
    float4 o = xv[k];
    if (w_pre) {
      const float4 w = load4_f32<TW>(w_pre, e[k]);
      o = float4{xv[k].x * inv * (off_pre + w.x), xv[k].y * inv * (off_pre + w.y), xv[k].z * inv * (off_pre + w.z), xv[k].w * inv * (off_pre + w.w)};
    }
    const size_t at = out_index(out_layout, r, e[k], H);     // four consecutive elements are neighbours in both layouts
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<float4*>((float*)out + at) = o;
    } else {
      *reinterpret_cast<uint2*>((bf16_t*)out + at) = uint2{pack_bf16x2(o.x, o.y), pack_bf16x2(o.z, o.w)};
    }
  }
}

extern "C" int alice_add_norm(float* resid, const float* branch, int n_partials, long partial_stride,
                              const void* w_post, const void* w_pre, int w_dtype, void* out, int out_dtype,
                              const int* rows, int T, int H, float eps_post, float eps_pre,
                              float off_post, float off_pre, int full_precision, int out_layout, hipStream_t stream) {
  ALICE_CHECK(T >= 0 && H > 0, "add_norm: bad sizes T=%d H=%d", T, H);
  ALICE_CHECK(resid != nullptr, "add_norm: the residual stream is missing");
  ALICE_CHECK(dtype_ok(w_dtype) && dtype_ok(out_dtype), "add_norm: unknown dtype");
  ALICE_CHECK(!(rows && branch), "add_norm: a row gather cannot be combined with a residual add");
  ALICE_CHECK(n_partials >= 1 && n_partials <= 64, "add_norm: n_partials %d out of range", n_partials);
  ALICE_CHECK(out_layout == 0 || (out_layout == 1 && out && out_dtype == DT_BF16 && H % 32 == 0),
              "add_norm: output in fragment order needs bfloat16 and a width that is a multiple of 32");
  if (T == 0) return 0;
  // Rows up to 8192 wide are held in registers, 1 to 8 elements a thread; the block is just as wide as the
  // row needs (a multiple of 64 threads), so that few threads are beyond its end.  Few rows: many threads
  // with few elements each (the step waits for this kernel); many rows: fewer threads, more rows per CU.
  int threads = H >= 2048 ? 512 : 256, ept = 0;
  if (H <= 8192) {
    ept = H <= 256 ? 1 : (H <= 512 ? 2 : (H <= 4096 ? 4 : 8));
    threads = ceil_div(ceil_div(H, ept), 64) * 64;
  }
#define ARGS resid, branch, n_partials, (size_t)partial_stride, (const TW*)w_post, (const TW*)w_pre, (TO*)out, rows, H, \
             eps_post, eps_pre, off_post, off_pre, out_layout
  // Many rows, no gather: a wave per row (two from 4,097 elements on).  From 320 rows: below, a block per row
  // fills more of the chip (measured at 2,304 and 3,584 elements: up to 256 rows the block-per-row kernel is 0.5
  // to 6 us faster, from 384 rows on the wave-per-row kernel is, by half at 2,048 rows).
  const bool aligned = (((uintptr_t)resid | (uintptr_t)branch | (uintptr_t)out | (uintptr_t)w_post | (uintptr_t)w_pre) & 15) == 0;
  const int k4 = (!rows && aligned && T >= 320 && H % 4 == 0 && H >= 256 && H <= 8192 && (partial_stride % 4 == 0 || !branch)) ? ceil_div(H, 256) : 0;
#define ROWS(TW, TO, FULL, K4, WPR) add_norm_rows_kernel<TW, TO, FULL, K4, WPR><<<ceil_div(T, 4 / WPR), 256, 0, stream>>>(     \
    resid, branch, n_partials, (size_t)partial_stride, (const TW*)w_post, (const TW*)w_pre, (TO*)out, T, H, eps_post, eps_pre, \
    off_post, off_pre, out_layout)
#define LAUNCH(TW, TO, FULL)                                                                         \
  do {                                                                                               \
    if (k4 > 0 && k4 <= 4) ROWS(TW, TO, FULL, 4, 1);                                                 \
    else if (k4 > 4 && k4 <= 9) ROWS(TW, TO, FULL, 9, 1);                                            \
    else if (k4 > 9 && k4 <= 16) ROWS(TW, TO, FULL, 16, 1);                                          \
    else if (k4 > 16 && k4 <= 18) ROWS(TW, TO, FULL, 9, 2);                                          \
    else if (k4 > 18) ROWS(TW, TO, FULL, 16, 2);                                                     \
    else if (ept == 1) add_norm_regs_kernel<TW, TO, FULL, 1><<<T, threads, 0, stream>>>(ARGS);            \
    else if (ept == 2) add_norm_regs_kernel<TW, TO, FULL, 2><<<T, threads, 0, stream>>>(ARGS);       \
    else if (ept == 4) add_norm_regs_kernel<TW, TO, FULL, 4><<<T, threads, 0, stream>>>(ARGS);       \
    else if (ept == 8) add_norm_regs_kernel<TW, TO, FULL, 8><<<T, threads, 0, stream>>>(ARGS);       \
    else add_norm_kernel<TW, TO, FULL><<<T, threads, 0, stream>>>(ARGS);                             \
  } while (0)
  DISPATCH_DTYPE(w_dtype, TW, DISPATCH_DTYPE(out_dtype, TO, {
    if (full_precision) LAUNCH(TW, TO, true); else LAUNCH(TW, TO, false);
  }));
#undef LAUNCH
#undef ROWS
#undef ARGS
  ALICE_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------- softcap
template <bool FULL>
__global__ void softcap_kernel(float* __restrict__ x, size_t n, float cap) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * (FULL ? tanh_full(x[i] / cap) : tanh_fast(x[i] / cap));
}

extern "C" int alice_softcap(float* x, long n, float cap, int full_precision, hipStream_t stream) {
  ALICE_CHECK(n >= 0 && cap > 0.f, "softcap: bad arguments n=%ld cap=%g", n, (double)cap);
  if (n == 0) return 0;
  if (full_precision) softcap_kernel<true><<<ceil_div(n, 256), 256, 0, stream>>>(x, (size_t)n, cap);
  else softcap_kernel<false><<<ceil_div(n, 256), 256, 0, stream>>>(x, (size_t)n, cap);
  ALICE_LAUNCH_CHECK();
  return 0;
}
