// Choosing the next token from float32 logits [B, V] on the device: argmax, and
// temperature -> top-k -> top-p -> softmax -> inverse CDF with a given uniform number per row.
//
// Semantics of the reference's host functions (src/sampling.rs:10-123): temperature multiplies the
// logits by 1/T; top-k keeps the k largest, ties at the threshold kept (25-41); top-p keeps the
// shortest descending prefix whose cumulative probability exceeds p (45-74; here all values tied
// with the last kept one are kept as well); softmax subtracts the maximum (77-92); the draw is the
// first index whose cumulative probability exceeds u (114-123).  Argmax returns the lowest index
// among equal maxima (llama3.rs:18862-18872).  One block per row; every reduction has a fixed
// order, so a row's result depends on nothing but the row, u and the options.
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int ST = 1024;     // threads per row

__device__ __forceinline__ uint32_t order_key(float x) {
  uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Stage 1 (chunks > 1): block (row, chunk) scans its slice of the row and writes (value, index) to `part`;
// stage 2 runs the same kernel over the partial results.  The lowest index wins among equal values at
// both stages, so the result does not depend on the number of chunks.
__global__ __launch_bounds__(ST) void argmax_kernel(const float* __restrict__ vals, const int* __restrict__ idxs,
                                                    int* __restrict__ out, float* __restrict__ part_v,
                                                    int* __restrict__ part_i, int V, int chunks) {
  __shared__ float bv[ST / 64];
  __shared__ int bi[ST / 64];
  const float* row = vals + (size_t)blockIdx.x * V;
  const int* irow = idxs ? idxs + (size_t)blockIdx.x * V : nullptr;
  const int per = (V + chunks - 1) / chunks;
  const int lo = blockIdx.y * per, hi = min(V, lo + per);
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += ST) {
    float v = row[i];
    int id = irow ? irow[i] : i;
    if (v > best || (v == best && id < idx)) { best = v; idx = id; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(best, o, 64);
    int oi = __shfl_xor(idx, o, 64);
    if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
  }
  if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = best; bi[threadIdx.x >> 6] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < ST / 64; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
    if (chunks > 1) {
      part_v[(size_t)blockIdx.x * chunks + blockIdx.y] = best;
      part_i[(size_t)blockIdx.x * chunks + blockIdx.y] = idx;
    } else {
      out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
  }
}

__device__ __forceinline__ int block_count(int v, int* ired) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  __syncthreads();
  if (lane == 0) ired[wid] = v;
  __syncthreads();
  int t = 0;
  for (int w = 0; w < ST / 64; ++w) t += ired[w];
  return t;
}

// Inclusive prefix sum over the block in thread order; `total` gets the sum over all threads.
__device__ __forceinline__ float block_inclusive_scan(float v, float* wred, float* total) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    float n = __shfl_up(v, o, 64);
    if (lane >= o) v += n;
  }
  __syncthreads();
  if (lane == 63) wred[wid] = v;
  __syncthreads();
  float before = 0.f, all = 0.f;
  for (int w = 0; w < ST / 64; ++w) {
    if (w < wid) before += wred[w];
    all += wred[w];
  }
  *total = all;
  return before + v;
}

__global__ __launch_bounds__(ST) void sample_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                    const float* __restrict__ uniform, int V, float inv_t,
                                                    int top_k, float top_p) {
  __shared__ float red[17];
  __shared__ int ired[ST / 64];
  __shared__ float wred[ST / 64];
  __shared__ int pick[2];
  const float* row = logits + (size_t)blockIdx.x * V;
  const int per = (V + ST - 1) / ST;
  const int lo_i = min(V, (int)threadIdx.x * per), hi_i = min(V, lo_i + per);   // this thread's run of indices

  float lmax = -INFINITY;
  for (int i = lo_i; i < hi_i; ++i) lmax = fmaxf(lmax, row[i] * inv_t);
  const float m = block_max(lmax, red);

  // top-k: the k-th largest key by bisection on the key space (count of keys >= mid is monotone).
  uint32_t thr = 0;
  if (top_k > 0 && top_k < V) {
    uint32_t lo = 0, hi = 0xffffffffu;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      int c = 0;
      for (int i = lo_i; i < hi_i; ++i) c += order_key(row[i] * inv_t) >= mid;
      if (block_count(c, ired) >= top_k) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }
  // top-p: the largest threshold whose kept mass exceeds p times the whole (top-k filtered) mass.
  if (top_p < 1.f) {
    float z = 0.f;
    for (int i = lo_i; i < hi_i; ++i) {
      float x = row[i] * inv_t;
      if (order_key(x) >= thr) z += expf(x - m);
    }
    const float target = top_p * block_sum(z, red);
    uint32_t lo = thr, hi = 0xffffffffu;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      float s = 0.f;
      for (int i = lo_i; i < hi_i; ++i) {
        float x = row[i] * inv_t;
        if (order_key(x) >= mid) s += expf(x - m);
      }
      if (block_sum(s, red) > target) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }

  // inverse CDF in index order
  float mine = 0.f;
  int last_kept = -1;
  for (int i = lo_i; i < hi_i; ++i) {
    float x = row[i] * inv_t;
    if (order_key(x) >= thr) {
      float e = expf(x - m);
      mine += e;
      if (e > 0.f) last_kept = i;
    }
  }
  float total;
  const float incl = block_inclusive_scan(mine, wred, &total);
  const float before = incl - mine;
  const float target = uniform[blockIdx.x] * total;
  if (threadIdx.x == 0) { pick[0] = -1; pick[1] = -1; }
  __syncthreads();
  atomicMax(&pick[1], last_kept);                       // last index with a positive probability
  if (mine > 0.f && target >= before && target < incl) {
    float acc = before;
    int chosen = last_kept;
    for (int i = lo_i; i < hi_i; ++i) {
      float x = row[i] * inv_t;
      if (order_key(x) >= thr) {
        acc += expf(x - m);
        if (target < acc) { chosen = i; break; }
      }
    }
    pick[0] = chosen;                                   // at most one thread satisfies the condition
  }
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = pick[0] >= 0 ? pick[0] : max(pick[1], 0);
}

}  // namespace

// How many chunks a row is cut into; the workspace holds B * chunks floats and as many ints.
extern "C" int alice_argmax_chunks(int B, int V) {
  if (V < 16384) return 1;
  int c = 512 / (B > 0 ? B : 1);
  if (c > V / 8192) c = V / 8192;
  return c < 2 ? 1 : (c > 64 ? 64 : c);
}

extern "C" int alice_argmax(const float* logits, int* out, float* work_v, int* work_i, int B, int V, hipStream_t stream) {
  ALICE_CHECK(B >= 0 && V >= 1, "argmax: bad sizes B=%d V=%d", B, V);
  if (B == 0) return 0;
  const int chunks = alice_argmax_chunks(B, V);
  ALICE_CHECK(chunks == 1 || (work_v && work_i), "argmax: the workspace is missing");
  ALICE_CHECK(B <= 65535 * 32, "argmax: too many rows");
  if (chunks == 1) {
    argmax_kernel<<<dim3(B, 1), ST, 0, stream>>>(logits, nullptr, out, nullptr, nullptr, V, 1);
  } else {
    argmax_kernel<<<dim3(B, chunks), ST, 0, stream>>>(logits, nullptr, out, work_v, work_i, V, chunks);
    ALICE_LAUNCH_CHECK();
    argmax_kernel<<<dim3(B, 1), ST, 0, stream>>>(work_v, work_i, out, nullptr, nullptr, chunks, 1);
  }
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_sample(const float* logits, int* out, const float* uniform, int B, int V, float temperature,
                            int top_k, float top_p, hipStream_t stream) {
  ALICE_CHECK(B >= 0 && V >= 1, "sample: bad sizes B=%d V=%d", B, V);
  ALICE_CHECK(temperature > 0.f, "sample: temperature must be positive (use argmax for greedy)");
  ALICE_CHECK(top_k >= 0 && top_p > 0.f, "sample: top_k must not be negative and top_p must be positive");
  if (B == 0) return 0;
  sample_kernel<<<B, ST, 0, stream>>>(logits, out, uniform, V, 1.f / temperature, top_k, top_p);
  ALICE_LAUNCH_CHECK();
  return 0;
}
