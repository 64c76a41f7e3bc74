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

// ---- sampling: a row is cut into chunks, a block per chunk for every pass over the row, one block per row
// for what needs the whole row
//
//   chunk_max        the maximum of every chunk
//   chunk_count      how many elements of the chunk lie within fixed distances of the row's maximum (and, for
//                    top-p alone, the chunk's probability mass)
//   chunk_collect    the elements within the chosen distance (at most capg a row) go to the row's list
//   row_threshold    the thresholds of top-k and top-p by bisection on the key space over that list, held in
//                    shared memory (up to CAP candidates: one wave does it) or read from memory by the whole
//                    block; probabilities enter as 64-bit fixed point, so the sums do not depend on the
//                    order in which the list was filled.  A row whose kept set does not fit (a flat
//                    distribution, a huge k) takes the same bisection over the whole row instead.
//   tile_sum         the kept mass of every tile of TILE elements (a wave per tile, lanes in a fixed order)
//   draw             the tile in which the cumulative sum, in index order, passes the target, and a scan of it
//
// Without top-k and top-p only the first and the last two run.  Every pass reads four consecutive elements per
// thread per load where the vocabulary is a multiple of four.
constexpr int TILE = 4096;       // 4 consecutive elements per thread of the draw's scan
constexpr int CAP = 4096;        // candidates held in shared memory
constexpr int CAPG = 32768;      // candidates of a row's list in memory, at most (fewer for very many rows: list_room())
constexpr int NCUT = 12;
constexpr int SB = 256;          // threads of the per-chunk kernels
constexpr int NMC = 4;           // distances at which the mass inside is summed too (top-p alone)
__device__ constexpr int kMassCut[NMC] = {5, 7, 8, 9};   // indices into kCut: 4, 8, 10, 12
__device__ constexpr float kCut[NCUT] = {0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f, 8.f, 10.f, 12.f, 16.f, 24.f};

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

// Where a row's intermediate results live (all arrays are per row; `chunks` and `tiles` per row).
struct SampleWork {
  float* pmax;                   // [B][chunks]
  int* pcnt;                     // [B][chunks][NCUT]
  unsigned long long* pmass;     // [B][chunks][1 + NMC]: the chunk's mass, and its mass within kCut[kMassCut[i]] of the maximum
  uint32_t* cand;                // [B][capg]
  unsigned long long* cmass;     // [B][capg]: the candidates' masses, for lists too long for shared memory
  uint32_t* thr;                 // [B]
  float* tsum;                   // [B][tiles]
  int* tlast;                    // [B][tiles]
  int chunks, tiles, tiles_per_chunk, capg;
};

// f(index, logit / T, valid) for the elements [lo, hi) of a row (lo a multiple of four); every lane of the block
// runs every call (those past the end with valid = false), in an order that depends on nothing but the thread,
// the block's size NT and the range.
template <int VEC, int NT, class F>
__device__ __forceinline__ void for_range(const float* __restrict__ row, int lo, int hi, float inv_t, F&& f) {
  const int tid = threadIdx.x;
  if constexpr (VEC == 4) {
    constexpr int U = 4;
    const int G0 = lo >> 2, G = hi >> 2;
    const float4* r4 = reinterpret_cast<const float4*>(row);
    for (int g0 = G0; g0 < G; g0 += NT * U) {
      float4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = r4[min(g0 + u * NT + tid, G - 1)];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int g = g0 + u * NT + tid;
        const bool ok = g < G;
        f(4 * g + 0, x[u].x * inv_t, ok);
        f(4 * g + 1, x[u].y * inv_t, ok);
        f(4 * g + 2, x[u].z * inv_t, ok);
        f(4 * g + 3, x[u].w * inv_t, ok);
      }
    }
  } else {
    constexpr int U = 8;
    for (int i0 = lo; i0 < hi; i0 += NT * U) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = row[min(i0 + u * NT + tid, hi - 1)];
#pragma unroll
      for (int u = 0; u < U; ++u) f(i0 + u * NT + tid, x[u] * inv_t, i0 + u * NT + tid < hi);
    }
  }
}

// The row's maximum from its chunks' (every wave computes it for itself).
__device__ __forceinline__ float row_max(const SampleWork& w, int b) {
  float m = -INFINITY;
  for (int c = threadIdx.x & 63; c < w.chunks; c += 64) m = fmaxf(m, w.pmax[(size_t)b * w.chunks + c]);
  return wave_max(m);
}

template <int VEC>
__global__ __launch_bounds__(SB) void chunk_max_kernel(const float* __restrict__ logits, SampleWork w, int V, float inv_t) {
  __shared__ float red[17];
  const int b = blockIdx.y, c = blockIdx.x;
  const float* row = logits + (size_t)b * V;
  const int lo = c * w.tiles_per_chunk * TILE, hi = min(V, lo + w.tiles_per_chunk * TILE);
  float lmax = -INFINITY;
  for_range<VEC, SB>(row, lo, hi, inv_t, [&](int, float x, bool ok) { lmax = fmaxf(lmax, ok ? x : -INFINITY); });
  const float m = block_max(lmax, red);
  if (threadIdx.x == 0) {
    w.pmax[(size_t)b * w.chunks + c] = m;
  }
}

template <int VEC>
__global__ __launch_bounds__(SB) void chunk_count_kernel(const float* __restrict__ logits, SampleWork w, int V, float inv_t,
                                                         int whole_mass) {
  __shared__ int wave_cnt[SB / 64][NCUT];
  __shared__ unsigned long long wave_mass[SB / 64][1 + NMC];
  const int b = blockIdx.y, c = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* row = logits + (size_t)b * V;
  const int lo = c * w.tiles_per_chunk * TILE, hi = min(V, lo + w.tiles_per_chunk * TILE);
  const float m = row_max(w, b);
  int cnt[NCUT];
#pragma unroll
  for (int j = 0; j < NCUT; ++j) cnt[j] = 0;
  unsigned long long mass[1 + NMC];
#pragma unroll
  for (int i = 0; i <= NMC; ++i) mass[i] = 0;
  for_range<VEC, SB>(row, lo, hi, inv_t, [&](int, float x, bool ok) {
    const float d = ok ? m - x : INFINITY;
#pragma unroll
    for (int j = 0; j < NCUT; ++j) cnt[j] += d <= kCut[j];
    if (whole_mass && ok) {
      const unsigned long long e = fixed_mass(x, m);
      mass[0] += e;
#pragma unroll
      for (int i = 0; i < NMC; ++i) mass[1 + i] += d <= kCut[kMassCut[i]] ? e : 0ull;
    }
  });
  if (whole_mass) {
#pragma unroll
    for (int i = 0; i <= NMC; ++i) mass[i] = wave_sum_u64(mass[i]);
  }
#pragma unroll
  for (int j = 0; j < NCUT; ++j) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt[j] += __shfl_xor(cnt[j], o, 64);
  }
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < NCUT; ++j) wave_cnt[wave][j] = cnt[j];
#pragma unroll
    for (int i = 0; i <= NMC; ++i) wave_mass[wave][i] = mass[i];
  }
  __syncthreads();
  if (threadIdx.x < NCUT) {
    int t = 0;
    for (int v = 0; v < SB / 64; ++v) t += wave_cnt[v][threadIdx.x];
    w.pcnt[((size_t)b * w.chunks + c) * NCUT + threadIdx.x] = t;
  }
  if (threadIdx.x < 1 + NMC) {
    unsigned long long t = 0;
    for (int v = 0; v < SB / 64; ++v) t += wave_mass[v][threadIdx.x];
    w.pmass[((size_t)b * w.chunks + c) * (1 + NMC) + threadIdx.x] = t;
  }
}

// The row's counts per distance (and, for top-p alone, its mass and the masses within some distances) from the
// chunks', into tot[NCUT] and z[1 + NMC] in shared memory; then the distance whose elements become the list:
// for top-k the nearest that holds k; for top-p alone the nearest whose mass clearly exceeds p times the row's,
// else the widest that fits; -1 if none does.  All threads of the block call it (blockDim.x >= 256) and get the
// same answer.
__device__ __forceinline__ int choose_cut(const SampleWork& w, int b, bool need_k, int top_k, float top_p, int* tot,
                                          unsigned long long* z) {
  const int t = threadIdx.x;
  if (t < NCUT * 16) {
    const int j = t / 16, part = t % 16;
    int sum = 0;
    for (int c = part; c < w.chunks; c += 16) sum += w.pcnt[((size_t)b * w.chunks + c) * NCUT + j];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (part == 0) tot[j] = sum;
  }
  if (t >= NCUT * 16 && t < NCUT * 16 + 1 + NMC && !need_k) {
    unsigned long long sum = 0;
    for (int c = 0; c < w.chunks; ++c) sum += w.pmass[((size_t)b * w.chunks + c) * (1 + NMC) + (t - NCUT * 16)];
    z[t - NCUT * 16] = sum;
  }
  __syncthreads();
  int cut = -1;
  if (!need_k) {
    const unsigned long long target = (unsigned long long)((double)top_p * (double)z[0]);
#pragma unroll
    for (int i = 0; i < NMC; ++i) {
      const int c = tot[kMassCut[i]];
      if (cut == -1 && c >= 1 && c <= w.capg && z[1 + i] > target + (target >> 16)) cut = kMassCut[i];
    }
    if (cut >= 0) return cut;
  }
#pragma unroll
  for (int j = 0; j < NCUT; ++j) {
    const int c = tot[j];
    if (need_k) { if (cut == -1 && c >= top_k && c <= w.capg) cut = j; if (cut == -1 && c > w.capg) cut = -2; }
    else if (c >= 1 && c <= w.capg) cut = j;
  }
  return cut;
}

template <int VEC>
__global__ __launch_bounds__(SB) void chunk_collect_kernel(const float* __restrict__ logits, SampleWork w, int V, float inv_t,
                                                           int top_k, float top_p) {
  __shared__ int tot[NCUT];
  __shared__ unsigned long long z[1 + NMC];
  const int b = blockIdx.y, c = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const bool need_k = top_k > 0 && top_k < V;
  const int cut = choose_cut(w, b, need_k, top_k, top_p, tot, z);
  if (cut < 0) return;
  const float* row = logits + (size_t)b * V;
  const int lo = c * w.tiles_per_chunk * TILE, hi = min(V, lo + w.tiles_per_chunk * TILE);
  const float m = row_max(w, b);
  float dcut = kCut[0];
#pragma unroll
  for (int j = 0; j < NCUT; ++j) if (j == cut) dcut = kCut[j];
  // Where this chunk's candidates go in the row's list: after those of the chunks before it, whose numbers the
  // counting kernel left (no atomic on memory: thousands of them on one address took most of a millisecond).
  // Within the chunk a counter in shared memory hands out the places.
  __shared__ int before, fill;
  if (threadIdx.x == 0) { before = 0; fill = 0; }
  __syncthreads();
  {
    int mine = 0;
    for (int cc = threadIdx.x; cc < c; cc += SB) mine += w.pcnt[((size_t)b * w.chunks + cc) * NCUT + cut];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
    if (lane == 0 && mine) atomicAdd(&before, mine);
  }
  __syncthreads();
  uint32_t* list = w.cand + (size_t)b * w.capg + before;
  const int room = w.capg - before;
  for_range<VEC, SB>(row, lo, hi, inv_t, [&](int, float x, bool ok) {
    const bool in = ok && (m - x <= dcut);
    const unsigned long long mask = __ballot(in);
    if (mask) {
      const int leader = __ffsll((long long)mask) - 1;
      int base = 0;
      if (lane == leader) base = atomicAdd(&fill, __popcll(mask));
      base = __shfl(base, leader, 64);
      const int pos = base + __popcll(mask & ((1ull << lane) - 1ull));
      if (in && pos < room) list[pos] = order_key(x);
    }
  });
}

template <int VEC>
__global__ __launch_bounds__(ST) void row_threshold_kernel(const float* __restrict__ logits, SampleWork w, int V, float inv_t,
                                                           int top_k, float top_p) {
  __shared__ float red[17];
  __shared__ int ired[ST / 64];
  __shared__ uint32_t list[CAP];
  __shared__ unsigned long long list_mass[CAP];
  __shared__ int tot[NCUT];
  __shared__ unsigned long long z_sh[1 + NMC];
  __shared__ uint32_t found[3];                           // threshold, top-k done, top-p done
  const int b = blockIdx.x;
  const float* row = logits + (size_t)b * V;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float m = row_max(w, b);
  const uint32_t key_m = order_key(m);
  const bool need_k = top_k > 0 && top_k < V, need_p = top_p < 1.f;
  uint32_t thr = 0;
  bool k_done = !need_k, p_done = !need_p;
  if (tid == 0) { found[0] = 0; found[1] = 0; found[2] = 0; }
  const int cut = choose_cut(w, b, need_k, top_k, top_p, tot, z_sh);
  const int n = cut >= 0 ? min(tot[cut], w.capg) : 0;
  if (cut >= 0 && n > CAP) {
    // a long list: the same bisections by the whole block over the list in memory
    __shared__ unsigned long long wsum[ST / 64];
    __shared__ uint32_t wmin[ST / 64];
    const uint32_t* gl = w.cand + (size_t)b * w.capg;
    unsigned long long* gm = w.cmass + (size_t)b * w.capg;
    auto block_sum_u64 = [&](unsigned long long v) {
      v = wave_sum_u64(v);
      __syncthreads();
      if (lane == 0) wsum[wave] = v;
      __syncthreads();
      unsigned long long t = 0;
      for (int x = 0; x < ST / 64; ++x) t += wsum[x];
      return t;
    };
    uint32_t kmin = 0xffffffffu;
    for (int j = tid; j < n; j += ST) {
      const uint32_t key = gl[j];
      kmin = min(kmin, key);
      if (need_p) gm[j] = fixed_mass(key_value(key), m);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) kmin = min(kmin, (uint32_t)__shfl_xor(kmin, o, 64));
    if (lane == 0) wmin[wave] = kmin;
    __syncthreads();                                      // also: the masses are written
    for (int x = 0; x < ST / 64; ++x) kmin = min(kmin, wmin[x]);
    uint32_t t = kmin;
    if (need_k) {
      uint32_t lo = kmin, hi = key_m;
      while (lo < hi) {
        const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
        int c = 0;
        for (int j = tid; j < n; j += ST) c += gl[j] >= mid;
        if (block_count(c, ired) >= top_k) lo = mid; else hi = mid - 1;
      }
      t = lo;
    }
    k_done = true;
    thr = need_k ? t : 0u;
    if (need_p) {
      unsigned long long kept = 0;
      for (int j = tid; j < n; j += ST) if (gl[j] >= t) kept += gm[j];
      kept = block_sum_u64(kept);
      const unsigned long long z = need_k ? kept : z_sh[0];
      const unsigned long long target = (unsigned long long)((double)top_p * (double)z);
      if (kept > target) {
        uint32_t lo = t, hi = key_m;
        while (lo < hi) {
          const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
          unsigned long long sum = 0;
          for (int j = tid; j < n; j += ST) if (gl[j] >= mid) sum += gm[j];
          if (block_sum_u64(sum) > target) lo = mid; else hi = mid - 1;
        }
        thr = lo;
        p_done = true;
      }
    }
  } else if (cut >= 0) {
    for (int j = tid; j < n; j += ST) list[j] = w.cand[(size_t)b * w.capg + j];
    __syncthreads();
    if (wave == 0) {
      const unsigned long long z_row = z_sh[0];
      uint32_t kmin = 0xffffffffu;
      for (int j = lane; j < n; j += 64) kmin = min(kmin, list[j]);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) kmin = min(kmin, (uint32_t)__shfl_xor(kmin, o, 64));
      uint32_t t = kmin;
      if (need_k) {
        uint32_t lo = kmin, hi = key_m;                   // count(list >= lo) = n >= k
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
          const unsigned long long mass = fixed_mass(key_value(list[j]), m);
          list_mass[j] = mass;
          if (list[j] >= t) kept += mass;
        }
        kept = wave_sum_u64(kept);                        // the mass of the list at and above the threshold so far
        const unsigned long long z = need_k ? kept : z_row;
        const unsigned long long target = (unsigned long long)((double)top_p * (double)z);
        if (kept > target) {                              // else the nucleus reaches below the list
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
  // ---- the same over the whole row, for what the list could not settle
  if (!k_done) {
    uint32_t lo = 0, hi = key_m;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      int c = 0;
      for_range<VEC, ST>(row, 0, V, inv_t, [&](int, float x, bool ok) { c += ok && order_key(x) >= mid; });
      if (block_count(c, ired) >= top_k) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }
  if (!p_done) {
    float z = 0.f;
    for_range<VEC, ST>(row, 0, V, inv_t, [&](int, float x, bool ok) { if (ok && order_key(x) >= thr) z += expf(x - m); });
    const float target = top_p * block_sum(z, red);
    uint32_t lo = thr, hi = key_m;
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) >> 1);
      float s = 0.f;
      for_range<VEC, ST>(row, 0, V, inv_t, [&](int, float x, bool ok) { if (ok && order_key(x) >= mid) s += expf(x - m); });
      if (block_sum(s, red) > target) lo = mid; else hi = mid - 1;
    }
    thr = lo;
  }
  if (tid == 0) w.thr[b] = thr;
}

// The kept mass of every tile of the chunk (wave v takes the chunk's tiles v, v + 4, ...), and the last index with
// a positive probability in it (-1: none).
template <int VEC>
__global__ __launch_bounds__(SB) void tile_sum_kernel(const float* __restrict__ logits, SampleWork w, int V, float inv_t,
                                                      int filtered) {
  const int b = blockIdx.y, c = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* row = logits + (size_t)b * V;
  const float m = row_max(w, b);
  const uint32_t thr = filtered ? w.thr[b] : 0u;
  const int t_end = min(w.tiles, (c + 1) * w.tiles_per_chunk);
  for (int t = c * w.tiles_per_chunk + wave; t < t_end; t += SB / 64) {
    float s = 0.f;
    int last_kept = -1;
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
    s = wave_sum(s);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) last_kept = max(last_kept, __shfl_xor(last_kept, o, 64));
    if (lane == 0) {
      w.tsum[(size_t)b * w.tiles + t] = s;
      w.tlast[(size_t)b * w.tiles + t] = last_kept;
    }
  }
}

// Inverse CDF in index order: the running sums of the tiles (one thread, in order), the tile in which the sum
// passes u times the total, and a scan of that tile, four consecutive elements per thread.
__global__ __launch_bounds__(ST) void draw_kernel(const float* __restrict__ logits, int* __restrict__ out,
                                                  const float* __restrict__ uniform, SampleWork w, int V, float inv_t,
                                                  int filtered) {
  __shared__ float wred[ST / 64];
  __shared__ float prefix[1024];                          // inclusive running sums of up to 1024 tiles at a time
  __shared__ int pick[2];
  __shared__ float carry[2];
  const int b = blockIdx.x;
  const float* row = logits + (size_t)b * V;
  const int tid = threadIdx.x;
  const float m = row_max(w, b);
  const uint32_t thr = filtered ? w.thr[b] : 0u;
  const float u = uniform[b];
  const float* tsum = w.tsum + (size_t)b * w.tiles;
  int last_kept = -1;
  for (int t = tid; t < w.tiles; t += ST) last_kept = max(last_kept, w.tlast[(size_t)b * w.tiles + t]);
  if (tid == 0) { pick[0] = -1; pick[1] = -1; carry[0] = 0.f; carry[1] = 0.f; }
  __syncthreads();
  atomicMax(&pick[1], last_kept);
  // the total first (groups of 1024 tiles), then the tile of the target
  for (int sweep = 0; sweep < 2; ++sweep) {
    const float target = u * carry[0];
    float before_group = 0.f;
    for (int t0 = 0; t0 < w.tiles; t0 += 1024) {
      const int n = min(w.tiles - t0, 1024);
      __syncthreads();
      for (int t = tid; t < n; t += ST) prefix[t] = tsum[t0 + t];
      __syncthreads();
      if (tid == 0) {
        float acc = before_group;
        for (int t = 0; t < n; ++t) { acc += prefix[t]; prefix[t] = acc; }
        if (sweep == 0) carry[0] = acc;
      }
      __syncthreads();
      if (sweep == 1 || w.tiles <= 1024) {
        const float tgt = sweep == 1 ? target : u * carry[0];
        for (int t = tid; t < n; t += ST) {
          const float lo = t == 0 ? before_group : prefix[t - 1];
          if (tgt >= lo && tgt < prefix[t]) { pick[0] = t0 + t; carry[1] = lo; }   // at most one tile
        }
      }
      before_group = prefix[n - 1];
    }
    if (w.tiles <= 1024) break;
  }
  __syncthreads();
  const int t_sel = pick[0], last_of_row = pick[1];
  const float target = u * carry[0];
  const float tile_before = carry[1];
  __syncthreads();
  if (t_sel < 0) {                                       // u * total rounded up to the total: the last kept token
    if (tid == 0) out[b] = max(last_of_row, 0);
    return;
  }
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
    bool hit = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (!hit && e[j] > 0.f) {
        acc += e[j];
        if (target < acc) { c = base + j; hit = true; }
      }
    }
    pick[0] = c;
  }
  __syncthreads();
  // the tile's sum by waves and by the scan can differ in the last bit: past the scan's end means the tile's last
  if (tid == 0) out[b] = pick[0] >= 0 ? pick[0] : max(pick[1], 0);
}

// How long a row's list may be: 32,768 candidates, fewer (down to what fits shared memory) when the lists of
// all rows would take more than 200 MB.
__host__ inline int list_room(int B) {
  long room = (16L << 20) / (B > 0 ? B : 1);
  return (int)(room > CAPG ? CAPG : (room < CAP ? CAP : room));
}

// chunks, tiles and tiles per chunk of a call
__host__ inline void sample_shape(int B, int V, int* chunks, int* tiles, int* per) {
  *tiles = (V + TILE - 1) / TILE;
  *per = ((long)B * *tiles + 1023) / 1024;
  if (*per < 1) *per = 1;
  *chunks = (*tiles + *per - 1) / *per;
}

}  // namespace

// How many chunks a row is cut into; the workspace holds B * chunks floats and as many ints, which is never more
// than ALICE_ARGMAX_MAX_PARTIALS of each: the bound that sizes the static workspace of alice_argmax_static.
extern "C" int alice_argmax_chunks(int B, int V) {
  if (V < 16384) return 1;
  int c = ALICE_ARGMAX_MAX_PARTIALS / (B > 0 ? B : 1);
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

// ---- argmax without a workspace argument
//
// The chunk maxima of the two-stage argmax live in a file-scope device array instead of a buffer that the caller
// allocates.  Every GPU holds its own copy of the array at its own address, which the host learns once per
// device from hipGetSymbolAddress (in host code the array's name is only a stand-in, not a device address).
// Nothing in the array has to start at zero: stage one writes every pair that stage two reads.
static_assert(ALICE_ARGMAX_STATIC_MAX_PAIRS >= ALICE_ARGMAX_MAX_PARTIALS,
              "the static workspace must hold what the chunk rule can ask for");
static __device__ __align__(256) unsigned char argmax_scratch[ALICE_ARGMAX_STATIC_MAX_PAIRS * 8];

namespace {
constexpr int MAX_DEVICES = 64;
void* g_argmax_scratch_ptr[MAX_DEVICES] = {};       // per device, set once; a pointer store is atomic on the host

// The address of the current device's copy of the array; nullptr (and the error set) on failure.
void* argmax_scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    alice_set_error("argmax (static): no current device, or a device number beyond %d", MAX_DEVICES - 1);
    return nullptr;
  }
  void* p = __atomic_load_n(&g_argmax_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p) return p;
  hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_scratch));
  if (e != hipSuccess || !p) {
    alice_set_error("argmax (static): hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    return nullptr;
  }
  __atomic_store_n(&g_argmax_scratch_ptr[dev], p, __ATOMIC_RELEASE);   // two threads racing here store the same address
  return p;
}
}  // namespace

extern "C" int alice_argmax_static_init() { return argmax_scratch_of_current_device() ? 0 : 1; }

extern "C" int alice_argmax_static(const float* logits, int* out, int B, int V, hipStream_t stream) {
  ALICE_CHECK(B >= 0 && V >= 1, "argmax: bad sizes B=%d V=%d", B, V);
  if (B == 0) return 0;
  ALICE_CHECK(logits && out, "argmax (static): logits and out must be given");
  ALICE_CHECK(B <= 65535 * 32, "argmax: too many rows");
  const int chunks = alice_argmax_chunks(B, V);
  if (chunks == 1) {
    argmax_kernel<<<dim3(B, 1), ST, 0, stream>>>(logits, nullptr, out, nullptr, nullptr, V, 1);
    ALICE_LAUNCH_CHECK();
    return 0;
  }
  ALICE_CHECK((long)B * chunks <= ALICE_ARGMAX_STATIC_MAX_PAIRS,
              "argmax (static): %d rows in %d chunks need %ld partial results, the static workspace holds %d",
              B, chunks, (long)B * chunks, ALICE_ARGMAX_STATIC_MAX_PAIRS);
  void* scratch = argmax_scratch_of_current_device();
  if (!scratch) return 1;
  float* work_v = reinterpret_cast<float*>(scratch);
  int* work_i = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(scratch) + (size_t)ALICE_ARGMAX_STATIC_MAX_PAIRS * 4);
  argmax_kernel<<<dim3(B, chunks), ST, 0, stream>>>(logits, nullptr, out, work_v, work_i, V, chunks);
  ALICE_LAUNCH_CHECK();
  argmax_kernel<<<dim3(B, 1), ST, 0, stream>>>(work_v, work_i, out, nullptr, nullptr, chunks, 1);
  ALICE_LAUNCH_CHECK();
  return 0;
}

// Number of 32-bit words of workspace a call needs.
extern "C" long alice_sample_workspace(int B, int V) {
  int chunks, tiles, per;
  sample_shape(B > 0 ? B : 1, V, &chunks, &tiles, &per);
  const long rows = B > 0 ? B : 1;
  // pmass and cmass first (8-byte elements), then the 4-byte arrays
  const long capg = list_room(B);
  return rows * chunks * 2 * (1 + NMC) + rows * capg * 2 + rows * chunks + rows * chunks * NCUT + rows * capg + rows + rows * tiles * 2 + 16;
}

extern "C" int alice_sample(const float* logits, int* out, const float* uniform, void* work, int B, int V,
                            float temperature, int top_k, float top_p, hipStream_t stream) {
  ALICE_CHECK(B >= 0 && V >= 1, "sample: bad sizes B=%d V=%d", B, V);
  ALICE_CHECK(temperature > 0.f, "sample: temperature must be positive (use argmax for greedy)");
  ALICE_CHECK(top_k >= 0 && top_p > 0.f, "sample: top_k must not be negative and top_p must be positive");
  ALICE_CHECK(B <= 65535, "sample: %d rows are more than one launch takes", B);
  ALICE_CHECK(work != nullptr && ((uintptr_t)work & 7) == 0, "sample: the workspace is missing or not 8-byte aligned");
  if (B == 0) return 0;
  SampleWork w;
  sample_shape(B, V, &w.chunks, &w.tiles, &w.tiles_per_chunk);
  w.capg = list_room(B);
  const size_t rows = (size_t)B;
  w.pmass = (unsigned long long*)work;
  w.cmass = w.pmass + rows * w.chunks * (1 + NMC);
  w.pmax = (float*)(w.cmass + rows * w.capg);
  w.pcnt = (int*)(w.pmax + rows * w.chunks);
  w.cand = (uint32_t*)(w.pcnt + rows * w.chunks * NCUT);
  w.thr = w.cand + rows * w.capg;
  w.tsum = (float*)(w.thr + rows);
  w.tlast = (int*)(w.tsum + rows * w.tiles);
  const float inv_t = 1.f / temperature;
  const bool need_k = top_k > 0 && top_k < V, need_p = top_p < 1.f;
  const int filtered = need_k || need_p;
  const dim3 cgrid(w.chunks, B);
#define GO(VEC)                                                                                                             \
  do {                                                                                                                      \
    chunk_max_kernel<VEC><<<cgrid, SB, 0, stream>>>(logits, w, V, inv_t);                                                   \
    if (filtered) {                                                                                                         \
      chunk_count_kernel<VEC><<<cgrid, SB, 0, stream>>>(logits, w, V, inv_t, need_k ? 0 : 1);                               \
      chunk_collect_kernel<VEC><<<cgrid, SB, 0, stream>>>(logits, w, V, inv_t, top_k, top_p);                                   \
      row_threshold_kernel<VEC><<<B, ST, 0, stream>>>(logits, w, V, inv_t, top_k, top_p);                                   \
    }                                                                                                                       \
    tile_sum_kernel<VEC><<<cgrid, SB, 0, stream>>>(logits, w, V, inv_t, filtered);                                          \
  } while (0)
  if (V % 4 == 0 && ((uintptr_t)logits & 15) == 0) GO(4); else GO(1);
#undef GO
  ALICE_LAUNCH_CHECK();
  draw_kernel<<<B, ST, 0, stream>>>(logits, out, uniform, w, V, inv_t, filtered);
  ALICE_LAUNCH_CHECK();
  return 0;
}
