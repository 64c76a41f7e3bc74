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

// The same operation with a row held in registers (EPT elements per thread): every operand is read
// once and the three phases need no second trip through memory.  Used when the row fits.
template <typename TW, typename TO, bool FULL, int EPT>
__global__ void add_norm_regs_kernel(float* __restrict__ resid, const float* __restrict__ branch,
                                     int n_partials, size_t partial_stride,
                                     const TW* __restrict__ w_post, const TW* __restrict__ w_pre,
                                     TO* __restrict__ out, const int* __restrict__ rows, int H,
                                     float eps_post, float eps_pre, float off_post, float off_pre, int out_layout) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t src = (size_t)(rows ? rows[r] : r) * H;
  float xv[EPT], bv[EPT], wq[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    xv[j] = i < H ? resid[src + i] : 0.f;
    wq[j] = (w_pre && i < H) ? load_f32(w_pre, i) : 0.f;
    bv[j] = 0.f;
  }
  if (branch) {
    float wp[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      wp[j] = (w_post && i < H) ? load_f32(w_post, i) : 0.f;
      if (i < H) {
        // partial sums are added in their order; eight loads are in flight at a time
        float v = 0.f;
        for (int p0 = 0; p0 < n_partials; p0 += 8) {
          float t[8];
#pragma unroll
          for (int p = 0; p < 8; ++p) t[p] = (p0 + p < n_partials) ? branch[src + i + (size_t)(p0 + p) * partial_stride] : 0.f;
#pragma unroll
          for (int p = 0; p < 8; ++p) v += t[p];
        }
        bv[j] = v;
      }
    }
    if (w_post) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < EPT; ++j) ss += bv[j] * bv[j];
      ss = block_sum(ss, red);
      const float mean = ss / (float)H;
      const float inv_b = FULL ? 1.f / sqrtf(mean + eps_post) : rsqrtf(mean + eps_post);
#pragma unroll
      for (int j = 0; j < EPT; ++j) bv[j] = bv[j] * inv_b * (off_post + wp[j]);
    }
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      xv[j] += bv[j];
      if (i < H) resid[src + i] = xv[j];
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
  for (int j = 0; j < EPT; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < H) store_f32(o, out_index(out_layout, r, i, H), w_pre ? xv[j] * inv * (off_pre + wq[j]) : xv[j]);
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
  // Rows up to 8192 wide are held in registers: 256 threads x 1..4 elements, then 1024 threads x 4 or 8.
  int threads = H >= 2048 ? 512 : 256, ept = 0;
  if (H <= 1024) { threads = 256; ept = H <= 256 ? 1 : (H <= 512 ? 2 : 4); }
  else if (H <= 4096) { threads = 1024; ept = 4; }
  else if (H <= 8192) { threads = 1024; ept = 8; }
  // Many rows: smaller blocks with more elements a thread keep more rows and more loads in flight on a CU.
  if (T >= 256 && H > 1024 && H <= 4096) { threads = H <= 2048 ? 256 : 512; ept = 8; }
#define ARGS resid, branch, n_partials, (size_t)partial_stride, (const TW*)w_post, (const TW*)w_pre, (TO*)out, rows, H, \
             eps_post, eps_pre, off_post, off_pre, out_layout
#define LAUNCH(TW, TO, FULL)                                                                         \
  do {                                                                                               \
    if (ept == 1) add_norm_regs_kernel<TW, TO, FULL, 1><<<T, threads, 0, stream>>>(ARGS);            \
    else if (ept == 2) add_norm_regs_kernel<TW, TO, FULL, 2><<<T, threads, 0, stream>>>(ARGS);       \
    else if (ept == 4) add_norm_regs_kernel<TW, TO, FULL, 4><<<T, threads, 0, stream>>>(ARGS);       \
    else if (ept == 8) add_norm_regs_kernel<TW, TO, FULL, 8><<<T, threads, 0, stream>>>(ARGS);       \
    else add_norm_kernel<TW, TO, FULL><<<T, threads, 0, stream>>>(ARGS);                             \
  } while (0)
  DISPATCH_DTYPE(w_dtype, TW, DISPATCH_DTYPE(out_dtype, TO, {
    if (full_precision) LAUNCH(TW, TO, true); else LAUNCH(TW, TO, false);
  }));
#undef LAUNCH
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
