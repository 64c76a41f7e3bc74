// bfloat16 attention over the paged cache on the matrix cores (MFMA 16x16x32, 32-bit softmax),
// for prompts (flash-style, causal, windowed) and for single decoded tokens (keys split over
// blocks, parts combined in a fixed order).
//
// Order of operations as in the reference (llama3.rs:5622-5688): dot product, times scale, softcap
// cap * tanh(s / cap), mask to the keys max(0, pos + 1 - window) .. pos (llama3.rs:5444-5451),
// softmax with a running maximum (llama3.rs:5568-5620), weighted sum of the values; the kv head of
// query head h is h / (nH / nKV).
//
// Cache layout ("fragment" layout, written by rope_cache_write): a page holds 64 positions of one kv
// head.  Keys:   [key tile t (4)][d tile (d/32)][lane 64][8]: lane g*16 + r holds K[16 t + r][32 dt + 8g ..+8].
// Values: [key block b (2)][dv tile (d/16)][lane 64][8]: lane g*16 + r, element j holds
//         V[32 b + 16 (j/4) + 4 g + j%4][16 dvt + r].
// With keys as the MFMA's first operand and queries as the second, lane l of the score tile holds
// S[key 4(l/16) + i][query l%16]; two such tiles, rounded to bfloat16, are exactly the second operand
// of the value product in the key order that the value layout above stores, so the probabilities
// never move between lanes.  Each lane keeps the running maximum and sum of its query column.
#include <type_traits>
#include "common.h"
#include "alice_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }   // one instruction; exp2(-inf) = 0
__device__ __forceinline__ float rcp_fast(float x) { return __builtin_amdgcn_rcpf(x); }

constexpr float LOG2E = 1.4426950408889634f;
constexpr float RAISE = 8.f;   // how far a maximum may outgrow the softmax's exponent base before the base follows

// Constants of the score pipeline.  A raw dot product s becomes, in the base-2 domain in which the
// softmax runs (2^y = e^score):
//   with softcap:  y = cap log2e tanh(s scale / cap),  tanh(x) = 1 - 2 / (2^(2 log2e x) + 1)
//   without:       y = s scale log2e
struct ScoreConsts {
  float c_in, c_out;
  __device__ __forceinline__ ScoreConsts(float scale, float cap) {
    if (cap > 0.f) { c_in = scale / cap * 2.f * LOG2E; c_out = cap * LOG2E; }
    else { c_in = scale * LOG2E; c_out = 0.f; }
  }
};
// max / sum over the four lanes that hold the same query column (l, l^16, l^32, l^48), with gfx950's
// lane-swap instructions: permlane32_swap(v, v) gives (value of the lane's copy in the lower half, in
// the upper half), permlane16_swap(v, v) the same for the even and odd rows of 16 lanes.
__device__ __forceinline__ float col_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float col_sum(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);                 // the same two addends in the same order in every lane
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Running state of NB query tiles (16 query columns each) against the keys seen so far.
template <int DT, int NB>
struct Core {
  u32x4 q[NB][DT];          // query fragments: lane (col, g) holds Q[col][32 dt + 8g ..+8]
  f32x4 o[NB][2 * DT];      // output^T tiles: lane holds O[dv 16 t + 4(l/16) + i][col l%16]
  float m[NB], l[NB];       // running maximum and sum of this lane's column

  __device__ __forceinline__ void init() {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      m[b] = -INFINITY;
      l[b] = 0.f;
#pragma unroll
      for (int t = 0; t < 2 * DT; ++t) o[b][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }

  // The fragments of one block of 32 keys: kpage/vpage point at the page of one kv head, kb is the block
  // within the page (0/1).
  // ONCE: the tile is read once per step by one wave (single tokens): loaded with the streaming hint.
  template <bool ONCE = false>
  __device__ __forceinline__ static u32x4 load_tile(const bf16_t* p) {
    if constexpr (ONCE) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    else return *reinterpret_cast<const u32x4*>(p);
  }
  template <bool ONCE = false>
  __device__ __forceinline__ static void load_k(const bf16_t* __restrict__ kpage, int kb, int lane, u32x4 (&kf)[2][DT]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        kf[t][dt] = load_tile<ONCE>(kpage + ((size_t)((kb * 2 + t) * DT + dt) * 64 + lane) * 8);
  }
  template <bool ONCE = false>
  __device__ __forceinline__ static void load_v(const bf16_t* __restrict__ vpage, int kb, int lane, u32x4 (&vf)[2 * DT]) {
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t)
      vf[t] = load_tile<ONCE>(vpage + ((size_t)(kb * 2 * DT + t) * 64 + lane) * 8);
  }

  // Scores of one block of 32 keys from loaded key fragments; key0 is the absolute position of its first
  // key.  pos[b]: the position of this lane's query column in tile b (negative: no query).  Keys outside
  // [pos + 1 - window, pos] are masked.  Updates the running maximum (base-2 domain, common to the four
  // lanes of a column), rescales the output, adds to this lane's own share of the running sum (the lanes
  // of a column are added up once, in finish()), and returns the probabilities as the second operand of
  // the value product.
  template <bool SOFTCAP>
  __device__ __forceinline__ void scores(const u32x4 (&kf)[2][DT], int key0, const int* pos, int window, ScoreConsts k,
                                         int lane, u32x4 (&p)[NB]) {
    f32x4 s[NB][2];
#pragma unroll
    for (int b = 0; b < NB; ++b) s[b][0] = s[b][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int b = 0; b < NB; ++b) s[b][t] = mfma16(kf[t][dt], q[b][dt], s[b][t]);
    softmax_step<SOFTCAP>(s, key0, pos, window, k, lane, p);
  }

  // The same with the key and value fragments of the block in LDS (laid out as in the cache: keys
  // [2][DT][64 lanes][8], values [2 DT][64 lanes][8]).
  template <bool SOFTCAP>
  __device__ __forceinline__ void compute_lds(const u32x4* __restrict__ kl, const u32x4* __restrict__ vl, int key0,
                                              const int* pos, int window, ScoreConsts k, int lane) {
    // All reads of a phase are issued before its products (the scheduling barriers keep them there: left alone,
    // the compiler reads one fragment at a time into the same registers and waits for each).  The first half of
    // the values is read before the softmax arithmetic and arrives during it.
    u32x4 f[2 * DT];
#pragma unroll
    for (int i = 0; i < 2 * DT; ++i) f[i] = kl[i * 64 + lane];              // keys: tile i / DT, d tile i % DT
    __builtin_amdgcn_sched_barrier(0);
    f32x4 s[NB][2];
#pragma unroll
    for (int b = 0; b < NB; ++b) s[b][0] = s[b][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        s[b][0] = mfma16(f[dt], q[b][dt], s[b][0]);
        s[b][1] = mfma16(f[DT + dt], q[b][dt], s[b][1]);
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < DT; ++t) f[t] = vl[t * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
    u32x4 p[NB];
    softmax_step<SOFTCAP>(s, key0, pos, window, k, lane, p);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = DT; t < 2 * DT; ++t) f[t] = vl[t * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t)
#pragma unroll
      for (int b = 0; b < NB; ++b) o[b][t] = mfma16(f[t], p[b], o[b][t]);
  }

  // From the raw dot products of 32 keys to their probabilities (see scores()).
  template <bool SOFTCAP>
  __device__ __forceinline__ void softmax_step(f32x4 (&s)[NB][2], int key0, const int* pos, int window, ScoreConsts k,
                                               int lane, u32x4 (&p)[NB]) {
    const int g = lane >> 4;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      // key visible iff lo <= key <= pos, i.e. (unsigned)(key - lo) <= (unsigned)(pos - lo); no query: span 0 and rel > 0
      const int lo = window > 0 ? max(pos[b] + 1 - window, 0) : 0;
      const unsigned span = pos[b] >= 0 ? (unsigned)(pos[b] - lo) : 0u;
      const int rel0 = pos[b] >= 0 ? key0 + g * 4 - lo : 1 << 30;
      // Most blocks lie wholly inside every query's range: no masking then (a column without a query takes what
      // comes; nothing of it is ever stored).
      const bool all_seen = __all(pos[b] < 0 || (key0 >= lo && key0 + 31 <= pos[b]));
      float mx = -INFINITY;
      auto transform = [&](auto masked) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = s[b][t][i] * k.c_in;
            if (SOFTCAP) v = fmaf(-2.f * k.c_out, rcp_fast(exp2_fast(v) + 1.f), k.c_out);
            if (decltype(masked)::value) v = ((unsigned)(rel0 + t * 16 + i) <= span) ? v : -INFINITY;
            s[b][t][i] = v;
            mx = fmaxf(mx, v);
          }
      };
      if (all_seen) transform(std::false_type{}); else transform(std::true_type{});
      // The exponent base follows the maximum only when the maximum has outgrown it by more than RAISE (in
      // base-2 exponent units): probabilities then reach 2^RAISE at most, which float32 sums and bfloat16
      // operands hold as well as values up to 1, and the output is rescaled in a few blocks instead of in most.
      const float seen = col_max(mx);
      const bool raise = seen > m[b] + RAISE;
      const float m_new = raise ? seen : m[b];
      const float base = (m_new == -INFINITY) ? 0.f : m_new;                    // all masked so far: every p is 0
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = exp2_fast(s[b][t][i] - base);
          s[b][t][i] = e;
          sum += e;
        }
      p[b] = u32x4{pack2(s[b][0][0], s[b][0][1]), pack2(s[b][0][2], s[b][0][3]),
                   pack2(s[b][1][0], s[b][1][1]), pack2(s[b][1][2], s[b][1][3])};
      if (__any(raise)) {                                                       // the whole wave or none of it
        const float corr = raise ? exp2_fast(m[b] - base) : 1.f;               // m[b] = -inf gives 0
        l[b] *= corr;
#pragma unroll
        for (int t = 0; t < 2 * DT; ++t) o[b][t] *= corr;
      }
      l[b] += sum;
      m[b] = m_new;
    }
  }

  // Adds the value product of output tiles [t0, t0 + N) from their loaded fragments.
  template <int N>
  __device__ __forceinline__ void accumulate(const u32x4 (&vf)[N], int t0, const u32x4 (&p)[NB]) {
#pragma unroll
    for (int t = 0; t < N; ++t)
#pragma unroll
      for (int b = 0; b < NB; ++b) o[b][t0 + t] = mfma16(vf[t], p[b], o[b][t0 + t]);
  }

  template <bool SOFTCAP>
  __device__ __forceinline__ void compute(const u32x4 (&kf)[2][DT], const u32x4 (&vf)[2 * DT], int key0, const int* pos,
                                          int window, ScoreConsts k, int lane) {
    u32x4 p[NB];
    scores<SOFTCAP>(kf, key0, pos, window, k, lane, p);
    accumulate<2 * DT>(vf, 0, p);
  }

  // The lanes of a column hold shares of its running sum: add them up (same order in every lane).
  __device__ __forceinline__ void finish() {
#pragma unroll
    for (int b = 0; b < NB; ++b) l[b] = col_sum(l[b]);
  }
};

// Where output element (token or sequence b, column c of nH * D) goes: row-major, or fragment order for the
// output projection ([rows/16][nH*D/32][64][8]; four consecutive columns from a multiple of four are neighbours
// in both).
__device__ __forceinline__ size_t decode_out_index(int layout, int b, int c, int width) {
  if (layout == 0) return (size_t)b * width + c;
  return ((size_t)((size_t)(b >> 4) * (width >> 5) + (c >> 5)) * 64 + ((c & 31) >> 3) * 16 + (b & 15)) * 8 + (c & 7);
}

// ---------------------------------------------------------------- prompts
// grid: (tiles of 64 query tokens, sequences, kv heads x passes); 4 waves, wave w takes tokens
// 16 w .. 16 w + 15 of the tile for GH query heads of one kv head (a pass); the passes of a kv head's
// group are separate blocks.  Tiles are taken from the end of the prompt backwards: the last tiles see
// the most keys, and starting them first shortens the tail.  With one head per wave (GH = 1) there are
// registers for two sets of key/value fragments, and the next block's loads fly during the current
// block's arithmetic.
template <int DT, int GH, bool SOFTCAP>
__global__ __launch_bounds__(256, GH == 1 ? 2 : 1) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    bf16_t* __restrict__ out, const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, float scale, float cap, int window,
    int out_layout) {
  constexpr int D = DT * 32;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;
  const int group = nH / nKV, passes = (group + GH - 1) / GH;
  const int b = blockIdx.y, kvh = blockIdx.z / passes, h0 = (blockIdx.z % passes) * GH;
  const int t_begin = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_begin;
  const int tile = (int)gridDim.x - 1 - (int)blockIdx.x;
  const int first = tile * 64 + wave * 16;                  // this wave's first token within the sequence's new tokens
  if (first >= n_new) return;
  const int start_len = context_lens[b] - n_new;
  const int my_tok = first + col;
  const bool tok_ok = my_tok < n_new;
  const int my_pos = tok_ok ? start_len + my_tok : -1;
  const int last_pos = start_len + min(first + 15, n_new - 1);
  const int first_key = window > 0 ? max(0, start_len + first + 1 - window) : 0;
  const int* bt = block_table + (size_t)b * bt_stride;
  const size_t page_elems = (size_t)64 * D;
  const ScoreConsts sc(scale, cap);

  Core<DT, GH> c;
  c.init();
  int pos[GH];
#pragma unroll
  for (int hh = 0; hh < GH; ++hh) {
    const int head = kvh * group + h0 + hh;
    const bool ok = tok_ok && (h0 + hh) < group;
    pos[hh] = ok ? my_pos : -1;
    const bf16_t* qrow = q + ((size_t)(t_begin + (tok_ok ? my_tok : 0)) * nH + (ok ? head : kvh * group)) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      c.q[hh][dt] = u32x4{0u, 0u, 0u, 0u};
      if (ok) c.q[hh][dt] = *reinterpret_cast<const u32x4*>(qrow + dt * 32 + g * 8);
    }
  }
  const int kb_begin = first_key >> 5, kb_end = last_pos >> 5;
  auto fetch = [&](int kb32, u32x4 (&kf)[2][DT], u32x4 (&vf)[2 * DT]) {
    const int page = bt[kb32 >> 1];
    Core<DT, GH>::load_k(k_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, kf);
    Core<DT, GH>::load_v(v_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, vf);
  };
  if constexpr (GH == 1) {
    // Two waves per SIMD (256 registers each) hide each other's waits.  Keys and the first half of the values
    // are fetched together; the second half of the values goes into the registers that the keys leave.
    int page_next = kb_begin <= kb_end ? bt[kb_begin >> 1] : 0;     // one block ahead, through the scalar cache
    for (int kb32 = kb_begin; kb32 <= kb_end; ++kb32) {
      const int page = page_next;
      page_next = bt[min(kb32 + 1, kb_end) >> 1];
      const bf16_t* vp = v_pool + ((size_t)page * nKV + kvh) * page_elems + ((size_t)(kb32 & 1) * 2 * DT * 64 + lane) * 8;
      u32x4 kf[2][DT], va[DT], vb[DT], p[1];
      Core<DT, GH>::load_k(k_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, kf);
#pragma unroll
      for (int t = 0; t < DT; ++t) va[t] = *reinterpret_cast<const u32x4*>(vp + (size_t)t * 512);
      c.template scores<SOFTCAP>(kf, kb32 << 5, pos, window, sc, lane, p);
#pragma unroll
      for (int t = 0; t < DT; ++t) vb[t] = *reinterpret_cast<const u32x4*>(vp + (size_t)(DT + t) * 512);
      c.template accumulate<DT>(va, 0, p);
      c.template accumulate<DT>(vb, DT, p);
    }
  } else {
    u32x4 kf[2][DT], vf[2 * DT];
    for (int kb32 = kb_begin; kb32 <= kb_end; ++kb32) {
      fetch(kb32, kf, vf);                                       // the values are in flight during the scores
      c.template compute<SOFTCAP>(kf, vf, kb32 << 5, pos, window, sc, lane);
    }
  }
  c.finish();
#pragma unroll
  for (int hh = 0; hh < GH; ++hh) {
    if (pos[hh] < 0) continue;
    const int head = kvh * group + h0 + hh;
    const float inv = 1.f / c.l[hh];
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t) {
      const f32x4 v = c.o[hh][t] * inv;
      uint2 pk = {pack2(v[0], v[1]), pack2(v[2], v[3])};
      *reinterpret_cast<uint2*>(out + decode_out_index(out_layout, t_begin + my_tok, head * D + t * 16 + g * 4, nH * D)) = pk;
    }
  }
}

// Prompts, second form: a block of four waves takes one tile of 16 query tokens of one head and the waves
// split its keys into four contiguous runs, as the single-token kernel below does; the parts are
// combined in LDS in the order 0, 1, 2, 3.  A single long prompt then gives thousands of short waves
// instead of a few hundred long ones, which is what fills the chip.
// grid: (tiles of 16 query tokens, taken from the end backwards; sequences; query heads).
template <int DT, bool SOFTCAP>
__global__ __launch_bounds__(256, 2) void attn_prefill_split_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    bf16_t* __restrict__ out, const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, float scale, float cap, int window,
    int out_layout) {
  constexpr int D = DT * 32;
  __shared__ float sm[4][16], sl[4][16];
  extern __shared__ __align__(16) float so[];                // [3 waves][16 columns][D + 4]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;
  const int group = nH / nKV;
  const int b = blockIdx.y, head = blockIdx.z, kvh = head / group;
  const int t_begin = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_begin;
  const int first = ((int)gridDim.x - 1 - (int)blockIdx.x) * 16;
  if (first >= n_new) return;                                // the whole block
  const int start_len = context_lens[b] - n_new;
  const int my_tok = first + col;
  const bool tok_ok = my_tok < n_new;
  int pos[1] = {tok_ok ? start_len + my_tok : -1};
  const int last_pos = start_len + min(first + 15, n_new - 1);
  const int first_key = window > 0 ? max(0, start_len + first + 1 - window) : 0;
  const int kb_first = first_key >> 5, kb_last = last_pos >> 5;
  const int per = (kb_last - kb_first + 4) / 4;              // ceil(blocks / 4)
  const int my_first = kb_first + wave * per, my_last = min(kb_last, my_first + per - 1);
  const int* bt = block_table + (size_t)b * bt_stride;
  const size_t page_elems = (size_t)64 * D;
  const ScoreConsts sc(scale, cap);

  Core<DT, 1> c;
  c.init();
  {
    const bf16_t* qrow = q + ((size_t)(t_begin + (tok_ok ? my_tok : 0)) * nH + head) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      c.q[0][dt] = u32x4{0u, 0u, 0u, 0u};
      if (tok_ok) c.q[0][dt] = *reinterpret_cast<const u32x4*>(qrow + dt * 32 + g * 8);
    }
  }
  // The page number of the next block of keys is read (through the scalar cache: the whole wave asks for the
  // same one) while this block is computed.
  int page_next = my_first <= my_last ? bt[my_first >> 1] : 0;
  for (int kb32 = my_first; kb32 <= my_last; ++kb32) {
    const int page = page_next;
    page_next = bt[min(kb32 + 1, my_last) >> 1];
    const bf16_t* vp = v_pool + ((size_t)page * nKV + kvh) * page_elems + ((size_t)(kb32 & 1) * 2 * DT * 64 + lane) * 8;
    u32x4 kf[2][DT], va[DT], vb[DT], p[1];
    Core<DT, 1>::load_k(k_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, kf);
#pragma unroll
    for (int t = 0; t < DT; ++t) va[t] = *reinterpret_cast<const u32x4*>(vp + (size_t)t * 512);
    c.template scores<SOFTCAP>(kf, kb32 << 5, pos, window, sc, lane, p);
#pragma unroll
    for (int t = 0; t < DT; ++t) vb[t] = *reinterpret_cast<const u32x4*>(vp + (size_t)(DT + t) * 512);   // into the keys' registers
    c.template accumulate<DT>(va, 0, p);
    c.template accumulate<DT>(vb, DT, p);
  }
  c.finish();
  if (g == 0) { sm[wave][col] = c.m[0]; sl[wave][col] = c.l[0]; }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t)
      *reinterpret_cast<f32x4*>(&so[((size_t)(wave - 1) * 16 + col) * (D + 4) + t * 16 + g * 4]) = c.o[0][t];
  }
  __syncthreads();
  if (wave != 0 || !tok_ok) return;
  // wave 0 adds the parts of waves 1..3 to its own, each scaled to the common maximum
  float mm = fmaxf(fmaxf(sm[0][col], sm[1][col]), fmaxf(sm[2][col], sm[3][col]));
  float f[4], ll = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = (sm[w][col] == -INFINITY) ? 0.f : exp2_fast(sm[w][col] - mm);
    ll += sl[w][col] * f[w];
  }
  const float inv = 1.f / ll;
#pragma unroll
  for (int t = 0; t < 2 * DT; ++t) {
    f32x4 v = c.o[0][t] * f[0];
#pragma unroll
    for (int w = 1; w < 4; ++w)
      v += *reinterpret_cast<const f32x4*>(&so[((size_t)(w - 1) * 16 + col) * (D + 4) + t * 16 + g * 4]) * f[w];
    v *= inv;
    uint2 pk = {pack2(v[0], v[1]), pack2(v[2], v[3])};
    *reinterpret_cast<uint2*>(out + decode_out_index(out_layout, t_begin + my_tok, head * D + t * 16 + g * 4, nH * D)) = pk;
  }
}

// Prompts, third form: the NW (4 or 8) waves of a block share every block of 32 keys and values through LDS.
// A block takes the heads of one kv head (1, 2 or 4 of them at a time: HB) for 16 NW / HB tokens; wave w takes
// head w % HB and tokens 16 (w / HB) .. +15 of the block's.  A block of keys and values is a contiguous copy
// of the cache's fragment order, so filling LDS and reading fragments from it are both linear.  Two buffers:
// the next block is on its way from memory into registers while this one is computed, and one barrier a
// step suffices.  Against whole tiles per wave, memory traffic falls by the number of waves.
// grid: (tiles of 16 NW / HB tokens, from the end backwards; sequences; kv heads x passes over the group).
template <int DT, bool SOFTCAP, int NW, int KS>
__global__ __launch_bounds__(64 * NW * KS, NW * KS == 4 ? 2 : 1) void attn_prefill_shared_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    bf16_t* __restrict__ out, const int* __restrict__ cu_seqlens, const int* __restrict__ context_lens,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, float scale, float cap, int window, int HB,
    int out_layout, int xcd_map) {
  // KS = 2: two sets of NW waves, the second takes the later half of the block's keys (its own buffers in LDS);
  // at the end the first set adds the second's part to its own, each scaled to the common maximum.  Halves the
  // longest block's run when there are too few blocks to fill the chip.
  constexpr int D = DT * 32;
  constexpr int NT = 64 * NW;                                // threads of a set
  constexpr int PIECES = 4 * DT * 64;                        // 16-byte pieces of a block: keys, then values
  constexpr int CH = (PIECES + NT - 1) / NT;                 // pieces per thread
  extern __shared__ __align__(16) uint32_t kv_raw[];         // [KS sets][2 buffers][keys 2 DT KB | values 2 DT KB]
  const int lane = threadIdx.x & 63, wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int set = wave_all / NW, wave = wave_all % NW, tid = threadIdx.x % NT;
  u32x4* kv = reinterpret_cast<u32x4*>(kv_raw) + (size_t)set * 2 * PIECES;
  const int col = lane & 15, g = lane >> 4;
  const int group = nH / nKV, passes = (group + HB - 1) / HB;
  // Which (tile, sequence, kv head) this block takes.  The hardware deals blocks to the eight XCDs round robin by
  // their linear index.  With more blocks than CUs (xcd_map), blocks that read the same keys and values are made
  // to meet in one XCD's L2: with Z = kv heads x passes dividing 8, XCD x takes z = x / (8 / Z); with 8 dividing
  // Z, the Z / 8 values from x Z / 8 on.  (Measured on the 2B, 9B and 27B head shapes at 1,024 to 6,000 tokens: 25
  // to 65 % faster wherever there are more blocks than CUs, 2 to 6 % slower where all blocks run at once.)
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if (xcd_map) {
    const int X = gridDim.x, Y = gridDim.y, Z = gridDim.z;
    const long lin = bx + (long)X * (by + (long)Y * bz);
    const int xcd = (int)(lin & 7);
    const long slot = lin >> 3;
    long r;
    if (8 % Z == 0) { const int per = 8 / Z; bz = xcd / per; r = slot * per + xcd % per; }
    else { const int per = Z / 8; bz = xcd * per + (int)(slot % per); r = slot / per; }
    bx = (int)(r % X);
    by = (int)(r / X);
  }
  const int b = by, kvh = bz / passes, hh = (bz % passes) * HB + wave % HB;
  const int tokens = 16 * NW / HB;
  const int t_begin = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t_begin;
  const int tile = (int)gridDim.x - 1 - bx;
  const int block_first = tile * tokens;                     // first token of the block among the sequence's new ones
  if (block_first >= n_new) return;                          // the whole block
  const int start_len = context_lens[b] - n_new;
  const int first = block_first + (wave / HB) * 16;
  const bool wave_ok = first < n_new && hh < group;
  const int my_tok = first + col;
  const bool tok_ok = wave_ok && my_tok < n_new;
  int pos[1] = {tok_ok ? start_len + my_tok : -1};
  const int* bt = block_table + (size_t)b * bt_stride;
  const size_t page_elems = (size_t)64 * D;
  const ScoreConsts sc(scale, cap);
  // the block's run of key blocks, this set's part of it, and this wave's own within that
  const int block_last_pos = start_len + min(block_first + tokens, n_new) - 1;
  const int run_begin = (window > 0 ? max(0, start_len + block_first + 1 - window) : 0) >> 5, run_end = block_last_pos >> 5;
  const int steps = (run_end - run_begin + KS) / KS;         // of the first set: ceil(blocks / KS)
  const int kb_begin = run_begin + set * steps, kb_end = min(run_end, kb_begin + steps - 1);
  const int my_begin = max(kb_begin, (window > 0 ? max(0, start_len + first + 1 - window) : 0) >> 5);
  const int my_end = wave_ok ? min(kb_end, (start_len + min(first + 15, n_new - 1)) >> 5) : -1;

  Core<DT, 1> c;
  c.init();
  {
    const bf16_t* qrow = q + ((size_t)(t_begin + (tok_ok ? my_tok : 0)) * nH + kvh * group + (hh < group ? hh : 0)) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      c.q[0][dt] = u32x4{0u, 0u, 0u, 0u};
      if (tok_ok) c.q[0][dt] = *reinterpret_cast<const u32x4*>(qrow + dt * 32 + g * 8);
    }
  }
  // piece j of a thread: piece tid + NT j of the block.  Loads are unconditional: past the set's last block
  // (or, for an empty second set, before its first) a block of the run is fetched again, and a piece past the
  // end is the last piece.
  u32x4 st[CH];
  auto fetch = [&](int kb32) {
    kb32 = min(min(kb32, max(kb_end, kb_begin)), run_end);
    const int page = bt[kb32 >> 1];
    const u32x4* kp = reinterpret_cast<const u32x4*>(k_pool + ((size_t)page * nKV + kvh) * page_elems) + (size_t)(kb32 & 1) * 2 * DT * 64;
    const u32x4* vp = reinterpret_cast<const u32x4*>(v_pool + ((size_t)page * nKV + kvh) * page_elems) + (size_t)(kb32 & 1) * 2 * DT * 64;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int piece = min(tid + NT * j, PIECES - 1);
      st[j] = *(piece < 2 * DT * 64 ? kp + piece : vp + (piece - 2 * DT * 64));
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int piece = tid + NT * j;
      if (PIECES % NT == 0 || piece < PIECES) kv[(size_t)buf * PIECES + piece] = st[j];
    }
  };
  fetch(kb_begin);
  put(0);
  __syncthreads();
  for (int it = 0; it < steps; ++it) {                       // both sets take the same number of steps
    const int kb32 = kb_begin + it, buf = it & 1;
    fetch(kb32 + 1);
    if (kb32 >= my_begin && kb32 <= my_end) {
      const u32x4* kl = kv + (size_t)buf * PIECES;
      c.template compute_lds<SOFTCAP>(kl, kl + 2 * DT * 64, kb32 << 5, pos, window, sc, lane);
    }
    put(buf ^ 1);
    __syncthreads();
  }
  c.finish();
  if constexpr (KS == 2) {
    // the second set leaves its part where the key buffers were (everyone is past the last barrier of the loop)
    float* so = reinterpret_cast<float*>(kv_raw);            // [NW waves][16 columns][D + 4], then maxima and sums
    float* sm = so + NW * 16 * (D + 4);
    float* sl = sm + NW * 16;
    if (set == 1) {
      if (g == 0) { sm[wave * 16 + col] = c.m[0]; sl[wave * 16 + col] = c.l[0]; }
#pragma unroll
      for (int t = 0; t < 2 * DT; ++t)
        *reinterpret_cast<f32x4*>(&so[((size_t)wave * 16 + col) * (D + 4) + t * 16 + g * 4]) = c.o[0][t];
    }
    __syncthreads();
    if (set == 1 || !tok_ok) return;
    const float m1 = sm[wave * 16 + col], l1 = sl[wave * 16 + col];
    const float mm = fmaxf(c.m[0], m1);
    const float f0 = (c.m[0] == -INFINITY) ? 0.f : exp2_fast(c.m[0] - mm), f1 = (m1 == -INFINITY) ? 0.f : exp2_fast(m1 - mm);
    const float inv = 1.f / (c.l[0] * f0 + l1 * f1);
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t) {
      f32x4 v = c.o[0][t] * f0 + *reinterpret_cast<const f32x4*>(&so[((size_t)wave * 16 + col) * (D + 4) + t * 16 + g * 4]) * f1;
      v *= inv;
      uint2 pk = {pack2(v[0], v[1]), pack2(v[2], v[3])};
      *reinterpret_cast<uint2*>(out + decode_out_index(out_layout, t_begin + my_tok, (kvh * group + hh) * D + t * 16 + g * 4, nH * D)) = pk;
    }
    return;
  }
  if (!tok_ok) return;
  const float inv = 1.f / c.l[0];
#pragma unroll
  for (int t = 0; t < 2 * DT; ++t) {
    const f32x4 v = c.o[0][t] * inv;
    uint2 pk = {pack2(v[0], v[1]), pack2(v[2], v[3])};
    *reinterpret_cast<uint2*>(out + decode_out_index(out_layout, t_begin + my_tok, (kvh * group + hh) * D + t * 16 + g * 4, nH * D)) = pk;
  }
}

// ---------------------------------------------------------------- single tokens, keys split over blocks
// grid: (sequences, kv heads, splits).  The query tile's 16 columns are the query heads of the kv head's
// group (group <= 16).  The sequence's 32-key blocks are dealt out in contiguous runs to the
// splits * 4 waves; every wave keeps a running (max, sum, output); the block's four waves are combined
// in LDS in the order 0, 1, 2, 3 and the split's result goes to `parts`:
// [sequence][head][split][4 + D] = (max, sum, two unused, unnormalised output).  With one split the output is final.
template <int DT, bool SOFTCAP>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    bf16_t* __restrict__ out, float* __restrict__ parts, const int* __restrict__ context_lens,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, float scale, float cap, int window, int splits,
    int out_layout) {
  constexpr int D = DT * 32;
  __shared__ float sm[4][16], sl[4][16];
  extern __shared__ __align__(16) float so[];            // [4 waves][group][D + 4]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 15, g = lane >> 4;
  const int b = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int group = nH / nKV;
  const int pos = context_lens[b] - 1;
  const int first_key = window > 0 ? max(0, pos + 1 - window) : 0;
  const int kb_first = first_key >> 5, kb_last = pos >> 5;
  const int n_blocks = kb_last - kb_first + 1;
  const int workers = splits * 4, me = split * 4 + wave;
  const int per = (n_blocks + workers - 1) / workers;
  const int my_first = kb_first + me * per, my_last = min(kb_last, my_first + per - 1);
  const int* bt = block_table + (size_t)b * bt_stride;
  const size_t page_elems = (size_t)64 * D;

  Core<DT, 1> c;
  c.init();
  const ScoreConsts sc(scale, cap);
  const bool head_ok = col < group;
  int cpos[1] = {head_ok ? pos : -1};
  {
    const bf16_t* qrow = q + ((size_t)b * nH + kvh * group + (head_ok ? col : 0)) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      c.q[0][dt] = u32x4{0u, 0u, 0u, 0u};
      if (head_ok) c.q[0][dt] = *reinterpret_cast<const u32x4*>(qrow + dt * 32 + g * 8);
    }
  }
  // Two sets of fragment registers: while one block of keys is computed, the next one's loads are in flight.
  // The page numbers are read one step before the tiles they name, through the scalar cache (the indices are
  // the same for the whole wave): a wait for them is no wait for the tiles in flight.
  {
    u32x4 kf0[2][DT], vf0[2 * DT], kf1[2][DT], vf1[2 * DT];
    auto page_of = [&](int kb32) { return bt[min(kb32, my_last) >> 1]; };
    auto fetch = [&](int kb32, int page, u32x4 (&kf)[2][DT], u32x4 (&vf)[2 * DT]) {
      Core<DT, 1>::template load_k<true>(k_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, kf);
      Core<DT, 1>::template load_v<true>(v_pool + ((size_t)page * nKV + kvh) * page_elems, kb32 & 1, lane, vf);
    };
    int page_a = 0, page_b = 0;
    if (my_first <= my_last) {
      page_a = page_of(my_first);
      page_b = page_of(my_first + 1);
      fetch(my_first, page_a, kf0, vf0);
    }
    for (int kb32 = my_first; kb32 <= my_last; kb32 += 2) {
      if (kb32 + 1 <= my_last) fetch(kb32 + 1, page_b, kf1, vf1);
      page_a = page_of(kb32 + 2);
      page_b = page_of(kb32 + 3);
      c.template compute<SOFTCAP>(kf0, vf0, kb32 << 5, cpos, window, sc, lane);
      if (kb32 + 1 <= my_last) {
        if (kb32 + 2 <= my_last) fetch(kb32 + 2, page_a, kf0, vf0);
        c.template compute<SOFTCAP>(kf1, vf1, (kb32 + 1) << 5, cpos, window, sc, lane);
      }
    }
  }
  // combine the four waves
  c.finish();
  if (g == 0) { sm[wave][col] = c.m[0]; sl[wave][col] = c.l[0]; }
  if (head_ok) {
#pragma unroll
    for (int t = 0; t < 2 * DT; ++t)
      *reinterpret_cast<f32x4*>(&so[((size_t)wave * group + col) * (D + 4) + t * 16 + g * 4]) = c.o[0][t];
  }
  __syncthreads();
  // thread -> (head column hc, dims): 256 threads cover 16 columns x D dims
  for (int idx = threadIdx.x; idx < 16 * D; idx += 256) {
    const int hc = idx / D, e = idx % D;
    if (hc >= group) continue;
    float mm = fmaxf(fmaxf(sm[0][hc], sm[1][hc]), fmaxf(sm[2][hc], sm[3][hc]));
    float acc = 0.f, ll = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = (sm[w][hc] == -INFINITY) ? 0.f : exp2_fast(sm[w][hc] - mm);     // maxima are base-2 exponents
      acc += so[((size_t)w * group + hc) * (D + 4) + e] * f;
      ll += sl[w][hc] * f;
    }
    const int head = kvh * group + hc;
    if (splits == 1) {
      out[decode_out_index(out_layout, b, head * D + e, nH * D)] = f32_to_bf16(acc / ll);
    } else {
      float* pr = parts + (((size_t)b * nH + head) * splits + split) * (D + ALICE_ATTN_PARTS_HEAD);
      pr[ALICE_ATTN_PARTS_HEAD + e] = acc;
      if (e == 0) { pr[0] = mm; pr[1] = ll; }
    }
  }
}

// Combines the splits of one (sequence, head): grid (sequences * heads).  The first wave fetches every
// split's maximum and sum at once and leaves the weights in LDS; then each thread sums its elements over the
// splits in the order 0, 1, ..., eight loads in flight at a time (a loop of dependent round trips to memory
// would cost more than the arithmetic).
__global__ void attn_decode_reduce_kernel(const float* __restrict__ parts, bf16_t* __restrict__ out, int D, int splits,
                                          int nH, int out_layout) {
  __shared__ float fs[65];
  const int PS = D + ALICE_ATTN_PARTS_HEAD;
  const float* pr = parts + (size_t)blockIdx.x * splits * PS;
  const int t = threadIdx.x;
  if (t < 64) {
    const float m = t < splits ? pr[(size_t)t * PS] : -INFINITY;
    const float l = t < splits ? pr[(size_t)t * PS + 1] : 0.f;
    const float mm = wave_max(m);
    const float f = (m == -INFINITY) ? 0.f : exp2_fast(m - mm);
    const float ll = wave_sum(l * f);
    fs[t] = f;
    if (t == 0) fs[64] = ll;
  }
  __syncthreads();
  const float inv = 1.f / fs[64];
  for (int e = t; e < D; e += blockDim.x) {
    float acc = 0.f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
      float v[8];
#pragma unroll
      for (int p = 0; p < 8; ++p) v[p] = (s0 + p < splits) ? pr[(size_t)(s0 + p) * PS + ALICE_ATTN_PARTS_HEAD + e] : 0.f;
#pragma unroll
      for (int p = 0; p < 8; ++p) acc += v[p] * fs[min(s0 + p, 63)];
    }
    out[decode_out_index(out_layout, blockIdx.x / nH, (blockIdx.x % nH) * D + e, nH * D)] = f32_to_bf16(acc * inv);
  }
}

}  // namespace

// Head sizes the matrix-core kernels and the fragment cache layout cover.
extern "C" int alice_attention_mfma_supported(int d) { return d == 64 || d == 128 || d == 256; }

extern "C" int alice_attention_prefill(const void* q, const void* k_pool, const void* v_pool, void* out,
                                       const int* cu_seqlens, const int* context_lens, const int* block_table,
                                       int bt_stride, int B, int max_new, int nH, int nKV, int d, int page_size,
                                       float scale, float softcap, int window, int variant, int out_layout, hipStream_t stream) {
  ALICE_CHECK(alice_attention_mfma_supported(d), "attention (matrix cores): head_dim %d is not covered (64, 128 or 256)", d);
  ALICE_CHECK(out_layout == 0 || (out_layout == 1 && (nH * d) % 32 == 0), "attention: unknown output layout %d", out_layout);
  ALICE_CHECK(nKV >= 1 && nH % nKV == 0, "attention: bad head counts nH=%d nKV=%d", nH, nKV);
  ALICE_CHECK(page_size == 64, "attention (matrix cores): pages must hold 64 positions, found %d", page_size);
  ALICE_CHECK(B >= 0 && max_new >= 0 && B <= 65535 && nKV <= 65535, "attention: bad batch B=%d", B);
  ALICE_CHECK(softcap >= 0.f && window >= 0 && bt_stride > 0, "attention: bad softcap, window or block table");
  if (B == 0 || max_new == 0) return 0;
  const int group = nH / nKV;
  // Two heads a wave halve the key/value reads.
  const long waves2 = (long)ceil_div(max_new, 64) * B * nKV * ceil_div(group, 2) * 4;
  const int gh = group % 2 == 0 ? 2 : 1;
  ALICE_CHECK(variant >= 0 && variant <= 5, "attention: unknown variant %d", variant);
  ALICE_CHECK((long)nKV * ceil_div(group, gh) <= 65535, "attention: too many heads for one launch");
  dim3 grid(ceil_div(max_new, 64), B, nKV * ceil_div(group, gh));
#define GO(DT, GH)                                                                                                          \
  do {                                                                                                                      \
    if (softcap > 0.f)                                                                                                      \
      attn_prefill_kernel<DT, GH, true><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, out_layout);     \
    else                                                                                                                    \
      attn_prefill_kernel<DT, GH, false><<<grid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, out_layout);     \
  } while (0)
#define GOS(DT)                                                                                                             \
  do {                                                                                                                      \
    dim3 sgrid(ceil_div(max_new, 16), B, nH);                                                                               \
    const size_t lds = (size_t)3 * 16 * (DT * 32 + 4) * sizeof(float);                                                      \
    if (softcap > 0.f)                                                                                                      \
      attn_prefill_split_kernel<DT, true><<<sgrid, 256, lds, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, out_layout);     \
    else                                                                                                                    \
      attn_prefill_split_kernel<DT, false><<<sgrid, 256, lds, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, out_layout);     \
  } while (0)
  // Few waves (one prompt of a few thousand tokens): split every tile's keys over four waves.  Many: whole
  // tiles per wave, two heads a wave where the group is even.
#define GOL(DT, NW, KS)                                                                                                     \
  do {                                                                                                                      \
    const int hb = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);                                                           \
    ALICE_CHECK((long)nKV * ceil_div(group, hb) <= 65535, "attention: too many heads for one launch");                      \
    dim3 lgrid(ceil_div(max_new, 16 * NW / hb), B, nKV * ceil_div(group, hb));                                              \
    const long blocks = (long)lgrid.x * lgrid.y * lgrid.z;                                                                  \
    const int xcd_map = blocks > 256 && blocks % 8 == 0 && (8 % lgrid.z == 0 || lgrid.z % 8 == 0);                          \
    const size_t lds = (size_t)KS * 2 * 4 * DT * 1024;                                                                      \
    static bool prepared = false;                                                                                           \
    if (lds > 65536 && !prepared) {                                                                                         \
      ALICE_CHECK(hipFuncSetAttribute((const void*)attn_prefill_shared_kernel<DT, true, NW, KS>,                            \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess &&                \
                  hipFuncSetAttribute((const void*)attn_prefill_shared_kernel<DT, false, NW, KS>,                           \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,                  \
                  "attention: the device does not give a block %d bytes of LDS", (int)lds);                                 \
      prepared = true;                                                                                                      \
    }                                                                                                                       \
    if (softcap > 0.f)                                                                                                      \
      attn_prefill_shared_kernel<DT, true, NW, KS><<<lgrid, 64 * NW * KS, lds, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, hb, out_layout, xcd_map); \
    else                                                                                                                    \
      attn_prefill_shared_kernel<DT, false, NW, KS><<<lgrid, 64 * NW * KS, lds, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, \
          (bf16_t*)out, cu_seqlens, context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, hb, out_layout, xcd_map); \
  } while (0)
  // Which form (measured on Gemma 2 shapes): with many blocks, four waves sharing their keys; with fewer, eight
  // (half as many blocks, half the key traffic); with too few blocks to fill the chip, the keys of a block split
  // over two sets of four waves, or one tile's keys split over a block's waves.  Small heads spend their time in
  // the softmax arithmetic and gain nothing from sharing.
  if (variant == ALICE_PREFILL_AUTO && d >= 128) {
    const int hb = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
    const long per_tile = (long)B * nKV * ceil_div(group, hb);
    if (per_tile * ceil_div(max_new, 64 / hb) >= 2048) variant = ALICE_PREFILL_SHARED4;
    else if (per_tile * ceil_div(max_new, 128 / hb) >= 192) variant = ALICE_PREFILL_SHARED8;
    else if (per_tile * ceil_div(max_new, 64 / hb) >= 192 && max_new >= 1024) variant = ALICE_PREFILL_SHARED4X2;
  }
  if (variant == ALICE_PREFILL_SHARED4 || variant == ALICE_PREFILL_SHARED8 || variant == ALICE_PREFILL_SHARED4X2) {
    if (variant == ALICE_PREFILL_SHARED4) { if (d == 64) GOL(2, 4, 1); else if (d == 128) GOL(4, 4, 1); else GOL(8, 4, 1); }
    else if (variant == ALICE_PREFILL_SHARED8) { if (d == 64) GOL(2, 8, 1); else if (d == 128) GOL(4, 8, 1); else GOL(8, 8, 1); }
    else { if (d == 64) GOL(2, 4, 2); else if (d == 128) GOL(4, 4, 2); else GOL(8, 4, 2); }
    ALICE_LAUNCH_CHECK();
    return 0;
  }
  const bool split = variant == ALICE_PREFILL_SPLIT || (variant == ALICE_PREFILL_AUTO && waves2 < 4096);
  if (split) {
    ALICE_CHECK(nH <= 65535, "attention: too many heads for one launch");
    if (d == 64) GOS(2); else if (d == 128) GOS(4); else GOS(8);
  } else {
    if (d == 64) { if (gh == 2) GO(2, 2); else GO(2, 1); }
    else if (d == 128) { if (gh == 2) GO(4, 2); else GO(4, 1); }
    else { if (gh == 2) GO(8, 2); else GO(8, 1); }
  }
#undef GOL
#undef GOS
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}

// Number of float32 elements `parts` must hold for a decode call.
extern "C" long alice_attention_decode_workspace(int B, int nH, int d, int splits) {
  return splits <= 1 ? 0 : (long)B * nH * splits * (d + ALICE_ATTN_PARTS_HEAD);
}

extern "C" int alice_attention_decode(const void* q, const void* k_pool, const void* v_pool, void* out, float* parts,
                                      const int* context_lens, const int* block_table, int bt_stride, int B, int nH,
                                      int nKV, int d, int page_size, float scale, float softcap, int window, int splits,
                                      int out_layout, hipStream_t stream) {
  ALICE_CHECK(alice_attention_mfma_supported(d), "attention (matrix cores): head_dim %d is not covered (64, 128 or 256)", d);
  ALICE_CHECK(nKV >= 1 && nH % nKV == 0 && nH / nKV <= 16, "attention (decode): %d query heads per kv head are more than the 16 this kernel takes", nKV ? nH / nKV : 0);
  ALICE_CHECK(page_size == 64, "attention (matrix cores): pages must hold 64 positions, found %d", page_size);
  ALICE_CHECK(B >= 0 && nKV <= 65535 && splits >= 1 && splits <= 64, "attention: bad batch B=%d or splits=%d", B, splits);
  ALICE_CHECK(splits == 1 || parts != nullptr, "attention: split keys need the workspace");
  ALICE_CHECK(out != nullptr || splits > 1, "attention: without an output the keys must be split (the parts are the result)");
  ALICE_CHECK(softcap >= 0.f && window >= 0 && bt_stride > 0, "attention: bad softcap, window or block table");
  ALICE_CHECK(out_layout == 0 || out_layout == 1, "attention: unknown output layout %d", out_layout);
  if (B == 0) return 0;
  dim3 grid(B, nKV, splits);
  const size_t lds = (size_t)4 * (nH / nKV) * (d + 4) * sizeof(float);
  // 16 query heads on a kv head of size 256 take 65 KB for the waves' parts: beyond what a block gets unasked
  // (the attribute is the kernel's and is told once; a smaller launch is not affected by it)
#define GO1(DT, CAP)                                                                                                        \
  do {                                                                                                                      \
    auto kern = attn_decode_kernel<DT, CAP>;                                                                                \
    if (lds > 48 * 1024) {                                                                                                  \
      static bool told = false;                                                                                             \
      if (!told) {                                                                                                          \
        ALICE_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 4 * 16 * (DT * 32 + 4) * (int)sizeof(float)) == hipSuccess, \
                    "attention (decode): the device does not give a block %d bytes of LDS", (int)lds);                      \
        told = true;                                                                                                        \
      }                                                                                                                     \
    }                                                                                                                       \
    kern<<<grid, 256, lds, stream>>>((const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, (bf16_t*)out, parts,   \
                                     context_lens, block_table, bt_stride, nH, nKV, scale, softcap, window, splits, out_layout); \
  } while (0)
#define GO(DT)                          \
  do {                                  \
    if (softcap > 0.f) GO1(DT, true);   \
    else GO1(DT, false);                \
  } while (0)
  if (d == 64) GO(2); else if (d == 128) GO(4); else GO(8);
#undef GO
#undef GO1
  ALICE_LAUNCH_CHECK();
  if (splits > 1 && out != nullptr) {
    attn_decode_reduce_kernel<<<B * nH, d <= 64 ? 64 : 128, 0, stream>>>(parts, (bf16_t*)out, d, splits, nH, out_layout);
    ALICE_LAUNCH_CHECK();
  }
  return 0;
}
