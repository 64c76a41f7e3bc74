// The tiled matrix product for many tokens (prompts) on the matrix cores: the kernel, shared by the source files
// that instantiate it (the widest wave tile in linear_mfma_tiled.hip, the narrower ones in
// linear_mfma_tiled_narrow.hip).  The layouts and the operand roles are described in linear_mfma.h.
// y[r] = sum_c W[r,c] x[c] (gguf.rs:4063-4074) with the GeGLU (llama3.rs:14519-14534), softcap
// (llama3.rs:14606-14611) and rotation (llama3.rs:5367-5378) epilogues.
#pragma once
#include "linear_mfma.h"

namespace {

constexpr int WM = 8;   // a wave's tile: up to 8 x 4 MFMA tiles = 128 tokens x 64 output features

// ---------------------------------------------------------------- tiled, many tokens
// Block: 4 waves side by side along N; every wave computes 16 TM (128 or 64) tokens x 16 WN (64, 32 or 16)
// output features (at most 8 x 4 MFMA tiles, 128 accumulator registers per lane) and streams its own weight
// tiles straight from memory.  The block's tokens x 64 inner elements of activations are staged once in LDS (in
// fragment order, so LDS reads and writes are linear) and read by all four waves.  Two stages are kept: while one is used for the
// MFMAs the next one's global loads are in flight, and one barrier per stage suffices.  The grid is
// one-dimensional and mapped so that the blocks that share weight tiles run on the same XCD (blocks
// are dealt to the eight XCDs round robin by their linear index).
// KC: k-tiles per stage.  A wave has the weights of one stage in flight, KC WN KB: two k-tiles with the widest
// tile, which is enough when the chip is full of blocks (long prompts); with a few hundred tokens there are
// fewer blocks than the chip has room for, narrower tiles make more of them, and deeper stages (KC TM = 32: the
// two stages of activations fill 64 KB of LDS) keep as many bytes on their way per wave as the wide tile does.

// XF: the activations come in fragment order (a compile-time choice: as a run-time one it cost the
// row-major path a third of its speed).
template <int EPI, typename TO, bool FULL, int TM, bool XF, int WN, int KC>
__global__ __launch_bounds__(256, 2) void linear_tiled_lds_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wf,
                                                               TO* __restrict__ y, int M, int N, int K, int KT, int NT,
                                                               float epi, int gx, int gy, int kt_per_slice, int y_frag,
                                                               RopeArgs ra) {
  constexpr int XJ = TM / 4;                               // token tiles each wave stages
  // The rotation epilogue stages 64 tokens x 256 features in the same memory afterwards (ROPE_PITCH elements a token).
  constexpr int XS_WORDS = 2 * KC * TM * 64 * 4;
  constexpr int LDS_WORDS = (EPI == ALICE_EPI_ROPE && WN == 4 && XS_WORDS < 64 * ROPE_PITCH / 2) ? 64 * ROPE_PITCH / 2 : XS_WORDS;
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

  if constexpr (EPI == ALICE_EPI_ROPE && WN != 4) {
    // narrow tiles (a few hundred tokens): every lane stores its own pairs, as the streaming kernel does
    RopeCol col[WN];
#pragma unroll
    for (int i = 0; i < WN; ++i) col[i] = rope_col(ra, min(tile[i], NT - 1) * 16 + g * 4);
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + j * 16 + r;
      if (m >= M) continue;
      const RopeToken t = rope_token(ra, m);
#pragma unroll
      for (int i = 0; i < WN; ++i)
        if (tile[i] < NT) rope_store4(ra, m, t, col[i], acc[i][j], rope_trig(ra, t, col[i]));
    }
    return;
  } else if constexpr (EPI == ALICE_EPI_ROPE) {
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


// Launches the kernel with the plan's tile for the grid that goes with it.
template <int EPI, typename TO, int TM, bool XF, int WN, int KC>
int launch_tiled_as(const void* x, const void* w, void* y, int M, int N, int K, int split, float epi, int y_frag, hipStream_t s,
                    const RopeArgs& ra) {
  const int KT = (K + 31) / 32, NT = (N * (EPI == ALICE_EPI_GEGLU ? 2 : 1) + 15) / 16;
  const int per = ceil_div(KT, split);
  const int gx = EPI == ALICE_EPI_GEGLU ? ceil_div(N / 16, 4 * WN / 2) : ceil_div(NT, 4 * WN);
  const int gy = ceil_div(M, 16 * TM);
  dim3 grid(8 * ceil_div(gx * gy, 8), split);
  linear_tiled_lds_kernel<EPI, TO, false, TM, XF, WN, KC><<<grid, 256, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, (TO*)y, M, N, K, KT, NT,
                                                                             epi, gx, gy, per, y_frag, ra);
  ALICE_LAUNCH_CHECK();
  return 0;
}

}  // namespace
