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

// Inclusive prefix sum over the block in thread order; `excl` gets the previous thread's inclusive sum (bit for bit).
__device__ __forceinline__ float block_inclusive_scan(float v, float* wred, float* excl) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    float n = __shfl_up(v, o, 64);
    if (lane >= o) v += n;
  }
  float prev = __shfl_up(v, 1, 64);
  __syncthreads();
  if (lane == 63) wred[wid] = v;
  __syncthreads();
  float before = 0.f;
  for (int w = 0; w < wid; ++w) before += wred[w];
  // the thread before lane 0 is lane 63 of the wave before: its inclusive sum is (sum of waves < wid-1) + wred[wid-1],
  // which is how `before` was built
  *excl = lane == 0 ? before : before + prev;
  return before + v;
}

// ---- the sampling kernel: one block per row
//
// Every pass over the row is read by the whole block, four consecutive elements per thread per load where the
// vocabulary is a multiple of four.  The thresholds of top-k and top-p are found among the few largest logits:
// a pass counts the elements within fixed distances of the maximum, the elements inside the chosen distance
// (at most CAP) are collected in shared memory, and the first wave bisects the key space over that list.
// Probabilities enter these comparisons as 64-bit fixed point, so the sums do not depend on the order in
// which the list was filled.  A row whose kept set does not fit (a flat distribution, a huge k) takes the
// same bisection over the whole row instead.  The draw goes by index order: sums of tiles of TILE elements
// (a wave per tile), the tile in which the cumulative sum passes the target, and a scan of that tile alone.
constexpr int TILE = 4096;       // 4 consecutive elements per thread
constexpr int CAP = 4096;        // candidates held in shared memory
constexpr int NCUT = 12;
__device__ constexpr float kCut[NCUT] = {0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f, 8.f, 12.f, 16.f, 24.f, 32.f};

__device__ __forceinline__ float key_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// exp(x - m) <= 1 as 24.40 fixed point
__device__ __forceinline__ unsigned long long fixed_mass(float x, float m) {
  return (unsigned long long)(expf(x - m) * 0x1p40f);
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
  uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    unsigned long long other = ((unsigned long long)__shfl_xor(hi, o, 64) << 32) | __shfl_xor(lo, o, 64);
    v += other;
    lo = (uint32_t)v;
    hi = (uint32_t)(v >> 32);
  }
  return v;
}

// f(index, logit / T, valid) for every element of the row; every lane of the block runs every call (those past
// the end with valid = false), in an order that depends on nothing but the thread and V.
template <int VEC, class F>
__device__ __forceinline__ void for_row(const float* __restrict__ row, int V, float inv_t, F&& f) {
  const int tid = threadIdx.x;
  if constexpr (VEC == 4) {
    constexpr int U = 4;
    const int G = V >> 2;
    const float4* r4 = reinterpret_cast<const float4*>(row);
    for (int g0 = 0; g0 < G; g0 += ST * U) {
      float4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = r4[min(g0 + u * ST + tid, G - 1)];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int g = g0 + u * ST + tid;
        const bool ok = g < G;
        f(4 * g + 0, x[u].x * inv_t, ok);
        f(4 * g + 1, x[u].y * inv_t, ok);
        f(4 * g + 2, x[u].z * inv_t, ok);
        f(4 * g + 3, x[u].w * inv_t, ok);
      }
    }
  } else {
    constexpr int U = 8;
    for (int i0 = 0; i0 < V; i0 += ST * U) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = row[min(i0 + u * ST + tid, V - 1)];
#pragma unroll
      for (int u = 0; u < U; ++u) f(i0 + u * ST + tid, x[u] * inv_t, i0 + u * ST + tid < V);
    }
  }
}

template <int VEC>
__global__ __launch_bounds__(ST) void sample_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                    const float* __restrict__ uniform, int V, float inv_t,
                                                    int top_k, float top_p) {
  __shared__ float red[17];
  __shared__ int ired[ST / 64];
  __shared__ float wred[ST / 64];
  __shared__ float tile_sum[256];                         // sums of up to 256 tiles at a time
  __shared__ int pick[2];
  __shared__ float carry[2];
  __shared__ uint32_t list[CAP];
  __shared__ unsigned long long list_mass[CAP];
  __shared__ int wave_cnt[ST / 64][NCUT];
  __shared__ unsigned long long wave_mass[ST / 64];
  __shared__ int n_list;
  __shared__ uint32_t found[3];                           // threshold, top-k done, top-p done
  const float* row = logits + (size_t)blockIdx.x * V;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  float lmax = -INFINITY;
  for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) { lmax = fmaxf(lmax, ok ? x : -INFINITY); });
  const float m = block_max(lmax, red);
  const uint32_t key_m = order_key(m);

  const bool need_k = top_k > 0 && top_k < V, need_p = top_p < 1.f;
  uint32_t thr = 0;
  bool k_done = !need_k, p_done = !need_p;
  if (need_k || need_p) {
    // how many elements lie within each distance of the maximum (and, for top-p alone, the whole mass)
    int cnt[NCUT];
#pragma unroll
    for (int j = 0; j < NCUT; ++j) cnt[j] = 0;
    unsigned long long mass = 0;
    const bool whole_mass = !need_k;
    for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) {
      const float d = ok ? m - x : INFINITY;
#pragma unroll
      for (int j = 0; j < NCUT; ++j) cnt[j] += d <= kCut[j];
      if (whole_mass && ok) mass += fixed_mass(x, m);
    });
    if (whole_mass) mass = wave_sum_u64(mass);
#pragma unroll
    for (int j = 0; j < NCUT; ++j) {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) cnt[j] += __shfl_xor(cnt[j], o, 64);
    }
    if (lane == 0) {
#pragma unroll
      for (int j = 0; j < NCUT; ++j) wave_cnt[wave][j] = cnt[j];
      wave_mass[wave] = mass;
    }
    if (tid == 0) { n_list = 0; found[0] = 0; found[1] = 0; found[2] = 0; }
    __syncthreads();
    int cut = -1;                                         // top-k: the nearest distance that holds k; else the widest that fits
    unsigned long long z_row = 0;
    {
      for (int w = 0; w < ST / 64; ++w) z_row += wave_mass[w];
#pragma unroll
      for (int j = 0; j < NCUT; ++j) {
        int c = 0;
        for (int w = 0; w < ST / 64; ++w) c += wave_cnt[w][j];
        if (need_k) { if (cut < 0 && c >= top_k && c <= CAP) cut = j; if (cut < 0 && c > CAP) cut = -2; }
        else if (c >= 1 && c <= CAP) cut = j;
      }
    }
    if (cut >= 0) {
      float dcut = kCut[0];
#pragma unroll
      for (int j = 0; j < NCUT; ++j) if (j == cut) dcut = kCut[j];
      for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) {
        const bool c = ok && (m - x <= dcut);
        const unsigned long long mask = __ballot(c);
        if (mask) {
          const int leader = __ffsll((long long)mask) - 1;
          int base = 0;
          if (lane == leader) base = atomicAdd(&n_list, __popcll(mask));
          base = __shfl(base, leader, 64);
          const int pos = base + __popcll(mask & ((1ull << lane) - 1ull));
          if (c && pos < CAP) list[pos] = order_key(x);
        }
      });
      __syncthreads();
      if (wave == 0) {
        const int n = min(n_list, CAP);
        uint32_t kmin = 0xffffffffu;
        for (int j = lane; j < n; j += 64) kmin = min(kmin, list[j]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) kmin = min(kmin, (uint32_t)__shfl_xor(kmin, o, 64));
        uint32_t t = kmin;
        if (need_k) {
          uint32_t lo = kmin, hi = key_m;                 // count(list >= lo) = n >= k
          while (lo < hi) {
            const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
            int c = 0;
            for (int j0 = 0; j0 < n; j0 += 64) c += __popcll(__ballot(j0 + lane < n && list[min(j0 + lane, n - 1)] >= mid));
            if (c >= top_k) lo = mid; else hi = mid - 1;
          }
          t = lo;
        }
        bool p_ok = !need_p;
        if (need_p) {
          unsigned long long kept = 0;
          for (int j = lane; j < n; j += 64) {
            const unsigned long long w = fixed_mass(key_value(list[j]), m);
            list_mass[j] = w;
            if (list[j] >= t) kept += w;
          }
          kept = wave_sum_u64(kept);                      // the mass of the list at and above the threshold so far
          const unsigned long long z = need_k ? kept : z_row;
          const unsigned long long target = (unsigned long long)((double)top_p * (double)z);
          if (kept > target) {                            // else the nucleus reaches below the list
            uint32_t lo = t, hi = key_m;
            while (lo < hi) {
              const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
              unsigned long long sum = 0;
              for (int j = lane; j < n; j += 64) if (list[j] >= mid) sum += list_mass[j];
              sum = wave_sum_u64(sum);
              if (sum > target) lo = mid; else hi = mid - 1;
            }
            t = lo;
            p_ok = true;
          }
        }
        if (lane == 0) { found[0] = t; found[1] = 1; found[2] = p_ok; }
      }
      __syncthreads();
      if (found[1]) { k_done = true; if (found[2]) { p_done = true; thr = found[0]; } else if (need_k) thr = found[0]; }
    }
  }
  // ---- the same over the whole row, for what the list could not settle
  if (!k_done) {
    uint32_t lo = 0, hi = key_m;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      int c = 0;
      for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) { c += ok && order_key(x) >= mid; });
      if (block_count(c, ired) >= top_k) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }
  if (!p_done) {
    float z = 0.f;
    for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) { if (ok && order_key(x) >= thr) z += expf(x - m); });
    const float target = top_p * block_sum(z, red);
    uint32_t lo = thr, hi = key_m;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      float s = 0.f;
      for_row<VEC>(row, V, inv_t, [&](int, float x, bool ok) { if (ok && order_key(x) >= mid) s += expf(x - m); });
      if (block_sum(s, red) > target) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }

  // ---- inverse CDF in index order
  // pass 1: the kept mass of every tile (wave w takes tiles w, w + 16, ...; lanes in a fixed order), and the
  // last index with a positive probability
  const int n_tiles = (V + TILE - 1) / TILE;
  int last_kept = -1;
  if (tid == 0) { pick[0] = -1; pick[1] = -1; carry[0] = 0.f; carry[1] = 0.f; }
  __syncthreads();
  const float u = uniform[blockIdx.x];
  auto tile_mass = [&](int t) {
    float s = 0.f;
    const int base = t * TILE;
    auto take = [&](int i, float x) {
      if (order_key(x) >= thr) {
        const float e = expf(x - m);
        s += e;
        if (e > 0.f) last_kept = max(last_kept, i);
      }
    };
    if constexpr (VEC == 4) {
      const float4* r4 = reinterpret_cast<const float4*>(row);
      const int G = V >> 2;
#pragma unroll 4
      for (int q = 0; q < TILE / 256; ++q) {
        const int g = base / 4 + q * 64 + lane;
        const float4 x = r4[min(g, G - 1)];
        if (g < G) { take(4 * g, x.x * inv_t); take(4 * g + 1, x.y * inv_t); take(4 * g + 2, x.z * inv_t); take(4 * g + 3, x.w * inv_t); }
      }
    } else {
      for (int i = base + lane; i < min(V, base + TILE); i += 64) take(i, row[i] * inv_t);
    }
    return wave_sum(s);
  };
  // Two sweeps over the tiles in groups of 256: the first finds the total, the second the tile of the target;
  // a row of one group keeps its tile sums and needs no second sweep.
  for (int sweep = 0; sweep < 2; ++sweep) {
    const float target = sweep == 1 ? u * carry[0] : 0.f;
    const bool choose = sweep == 1 || n_tiles <= 256;
    float before_group = 0.f;
    for (int t0 = 0; t0 < n_tiles; t0 += 256) {
      const int t1 = min(n_tiles, t0 + 256);
      for (int t = t0 + wave; t < t1; t += ST / 64) {
        const float s = tile_mass(t);
        if (lane == 0) tile_sum[t - t0] = s;
      }
      __syncthreads();
      if (tid == 0) {
        float acc = before_group;
        for (int t = t0; t < t1; ++t) acc += tile_sum[t - t0];
        if (sweep == 0) carry[0] = acc;
        if (choose) {
          const float tgt = sweep == 1 ? target : u * acc;
          float run = before_group;
          for (int t = t0; t < t1; ++t) {
            const float next = run + tile_sum[t - t0];
            if (pick[0] < 0 && tgt < next) { pick[0] = t; carry[1] = run; }
            run = next;
          }
        }
        before_group = acc;
      }
      __syncthreads();
    }
    if (choose) break;
  }
  atomicMax(&pick[1], last_kept);
  __syncthreads();
  const int t_sel = pick[0], last_of_row = pick[1];
  const float target = u * carry[0];
  const float tile_before = carry[1];
  __syncthreads();
  if (t_sel < 0) {                                       // u * total rounded up to the total: the last kept token
    if (tid == 0) out[blockIdx.x] = max(last_of_row, 0);
    return;
  }
  // pass 2: the chosen tile, four consecutive elements per thread, block scan in index order
  if (tid == 0) { pick[0] = -1; pick[1] = -1; }
  const int base = t_sel * TILE + tid * 4;
  float e[4], mine = 0.f;
  int my_last = -1;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    e[j] = 0.f;
    if (base + j < V) {
      float x = row[base + j] * inv_t;
      if (order_key(x) >= thr) e[j] = expf(x - m);
    }
    if (e[j] > 0.f) my_last = base + j;
    mine += e[j];
  }
  float excl;
  const float incl = tile_before + block_inclusive_scan(mine, wred, &excl);
  const float before = tile_before + excl;
  if (my_last >= 0) atomicMax(&pick[1], my_last);
  if (target >= before && target < incl) {               // at most one thread: `before` is the thread before's `incl`
    float acc = before;
    int c = my_last;                                     // if rounding lets the run end early: its last positive one
    bool found = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!found && e[j] > 0.f) {
        acc += e[j];
        if (target < acc) { c = base + j; found = true; }
      }
    }
    pick[0] = c;
  }
  __syncthreads();
  // the tile's sum by waves and by the scan can differ in the last bit: past the scan's end means the tile's last
  if (tid == 0) out[blockIdx.x] = pick[0] >= 0 ? pick[0] : max(pick[1], 0);
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
  if (V % 4 == 0 && ((uintptr_t)logits & 15) == 0)
    sample_kernel<4><<<B, ST, 0, stream>>>(logits, out, uniform, V, 1.f / temperature, top_k, top_p);
  else
    sample_kernel<1><<<B, ST, 0, stream>>>(logits, out, uniform, V, 1.f / temperature, top_k, top_p);
  ALICE_LAUNCH_CHECK();
  return 0;
}
