// Attention over the paged cache for any head size up to 256, any head and group counts, in
// 32-bit arithmetic: the kernel of the true 32-bit path and the fallback of the bfloat16 path.
// One block per (query token, query head); used for prompts and for single decoded tokens alike.
//
// Order of operations as in the reference (llama3.rs:5622-5688): dot product, times scale, softcap
// cap * tanh(s / cap), then the softmax over the keys max(0, pos + 1 - window) .. pos (window keys,
// the query's own included, llama3.rs:5444-5451), then the weighted sum of the values; the kv head
// of query head h is h / (nH / nKV).  The softmax is computed chunk by chunk with a running maximum
// (the reference's online variant, llama3.rs:5568-5620).  A position term at the score stage is a
// parameter: with bias_slopes, head h's capped score of key k for the query at position p gets
// bias_slopes[h] * (k - p) added (a linear distance bias; the reference's models have none, so the
// product passes a null pointer).
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int CHUNK = 1024;
constexpr int THREADS = 256;

template <typename T, bool FULL>
__global__ __launch_bounds__(THREADS) void attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pool, const T* __restrict__ v_pool, T* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, int d, int page_size,
    float scale, float cap, int window, int DG, const float* __restrict__ bias_slopes) {
  __shared__ float qs[256];
  __shared__ float sc[CHUNK];
  __shared__ float red[17];
  __shared__ float part[THREADS];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int kvh = h / (nH / nKV);
  const float slope = bias_slopes ? bias_slopes[h] : 0.f;
  const int start = window > 0 ? max(0, pos + 1 - window) : 0;
  const int* bt = block_table + (size_t)seq * bt_stride;

  const T* qrow = q + ((size_t)t * nH + h) * d;
  for (int i = tid; i < d; i += THREADS) qs[i] = load_f32(qrow, i);
  __syncthreads();

  const int G = THREADS / DG;            // key groups in the value pass
  const int g = tid / DG, j = tid % DG;
  float acc = 0.f, m_run = -INFINITY, l_run = 0.f;

  for (int c0 = start; c0 <= pos; c0 += CHUNK) {
    const int n = min(CHUNK, pos + 1 - c0);
    float lmax = -INFINITY;
    for (int i = tid; i < n; i += THREADS) {
      const int kp = c0 + i;
      const int page = bt[kp / page_size];
      const T* krow = k_pool + (((size_t)page * nKV + kvh) * page_size + kp % page_size) * d;
      float s = 0.f;
      for (int e = 0; e < d; ++e) s = fmaf(qs[e], load_f32(krow, e), s);
      s *= scale;
      if (cap > 0.f) s = cap * (FULL ? tanh_full(s / cap) : tanh_fast(s / cap));
      if (bias_slopes) s = fmaf(slope, (float)(kp - pos), s);
      sc[i] = s;
      lmax = fmaxf(lmax, s);
    }
    const float m_new = fmaxf(m_run, block_max(lmax, red));
    const float corr = (m_run == -INFINITY) ? 0.f : (FULL ? expf(m_run - m_new) : __expf(m_run - m_new));
    float lsum = 0.f;
    for (int i = tid; i < n; i += THREADS) {
      float p = FULL ? expf(sc[i] - m_new) : __expf(sc[i] - m_new);
      sc[i] = p;
      lsum += p;
    }
    l_run = l_run * corr + block_sum(lsum, red);      // the barriers inside also publish sc[]
    m_run = m_new;
    acc *= corr;
    if (j < d) {
      for (int i = g; i < n; i += G) {
        const int kp = c0 + i;
        const int page = bt[kp / page_size];
        const T* vrow = v_pool + (((size_t)page * nKV + kvh) * page_size + kp % page_size) * d;
        acc = fmaf(sc[i], load_f32(vrow, j), acc);
      }
    }
    __syncthreads();                                   // sc[] is rewritten by the next chunk
  }
  part[tid] = acc;
  __syncthreads();
  if (tid < d) {
    float o = 0.f;
    for (int gg = 0; gg < G; ++gg) o += part[gg * DG + tid];
    store_f32(out + ((size_t)t * nH + h) * d, tid, o / l_run);
  }
}

}  // namespace

extern "C" int alice_attention_generic(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                                       const int* positions, const int* seq_of_token, const int* block_table,
                                       int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                                       float softcap, int window, const float* bias_slopes, int full_precision,
                                       hipStream_t stream) {
  ALICE_CHECK(dtype_ok(dtype), "attention: unknown dtype %d", dtype);
  ALICE_CHECK(T >= 0 && nH >= 1 && nKV >= 1 && nH % nKV == 0, "attention: bad head counts nH=%d nKV=%d", nH, nKV);
  ALICE_CHECK(d >= 1 && d <= 256, "attention: head_dim %d is outside 1..256, the range of this kernel", d);
  ALICE_CHECK(nH <= 65535, "attention: too many heads for one launch (%d)", nH);
  ALICE_CHECK(page_size > 0 && bt_stride > 0, "attention: bad page geometry");
  ALICE_CHECK(softcap >= 0.f && window >= 0, "attention: softcap and window must not be negative (0 turns them off)");
  if (T == 0) return 0;
  int DG = 1;
  while (DG < d) DG <<= 1;
  dim3 grid(T, nH);
  DISPATCH_DTYPE(dtype, TT, {
    if (full_precision)
      attn_generic_kernel<TT, true><<<grid, THREADS, 0, stream>>>((const TT*)q, (const TT*)k_pool, (const TT*)v_pool,
          (TT*)out, positions, seq_of_token, block_table, bt_stride, nH, nKV, d, page_size, scale, softcap, window, DG, bias_slopes);
    else
      attn_generic_kernel<TT, false><<<grid, THREADS, 0, stream>>>((const TT*)q, (const TT*)k_pool, (const TT*)v_pool,
          (TT*)out, positions, seq_of_token, block_table, bt_stride, nH, nKV, d, page_size, scale, softcap, window, DG, bias_slopes);
  });
  ALICE_LAUNCH_CHECK();
  return 0;
}
