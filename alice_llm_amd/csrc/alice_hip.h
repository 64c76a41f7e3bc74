// C interface of the HIP library (gfx950).  Every function takes raw device pointers and a HIP
// stream, checks its arguments on the host before it launches anything, and returns 0 on success;
// otherwise alice_last_error() describes the problem.  dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#define ALICE_ABI_VERSION 6

#define ALICE_EPI_NONE 0
#define ALICE_EPI_GEGLU 1     // W = [gate; up] stacked, y = gelu_tanh(gate x) * (up x)
#define ALICE_EPI_SOFTCAP 2   // y = cap * tanh(y / cap)
#define ALICE_EPI_ROPE 3      // internal: rotation and cache write (alice_linear_rope_cache)

#define ALICE_LAYOUT_ROW 0     // row-major [N, K]
#define ALICE_LAYOUT_FRAG16 1  // bfloat16 in 16x32 MFMA fragments, see linear_mfma.hip

#define ALICE_PREFILL_AUTO 0    // prompt attention: chosen by the grid's size
#define ALICE_PREFILL_TILES 1   // a wave takes whole tiles of 16 queries (two heads where the group is even)
#define ALICE_PREFILL_SPLIT 2   // the four waves of a block split one tile's keys
#define ALICE_PREFILL_SHARED4 3 // the four waves of a block share each block of keys and values through LDS
#define ALICE_PREFILL_SHARED8 4 // the same with eight waves
#define ALICE_PREFILL_SHARED4X2 5 // two sets of four waves, each with half of the block's keys

#define ALICE_LINEAR_AUTO 0
#define ALICE_LINEAR_GENERIC 1
#define ALICE_LINEAR_SKINNY 2
#define ALICE_LINEAR_MFMA 3
#define ALICE_LINEAR_TILED_W16 4   // the tiled kernel with a wave tile of 16 output features (activations in fragment order)
#define ALICE_LINEAR_TILED_W32 5   // the same with 32

#ifdef __cplusplus
extern "C" {
#endif

const char* alice_last_error();
int alice_abi_version();
// Digest of the sources and flags this library was built from; the bindings compare it with the sources beside them.
const char* alice_source_digest();
int alice_device_arch(char* out, int cap);

int alice_embed(const int* tokens, const void* table, int table_dtype, int table_layout, float* out,
                int T, int H, int V, float scale, hipStream_t stream);

int alice_add_norm(float* resid, const float* branch, int n_partials, long partial_stride,
                   const void* w_post, const void* w_pre, int w_dtype, void* out, int out_dtype,
                   const int* rows, int T, int H, float eps_post, float eps_pre, float off_post,
                   float off_pre, int full_precision, int out_layout, hipStream_t stream);

int alice_softcap(float* x, long n, float cap, int full_precision, hipStream_t stream);

// y[M, N] = x[M, K] . W^T with an optional epilogue.  `variant` forces a kernel (tests); AUTO picks.
// For GEGLU, W has 2N rows.  `split_k` > 1 asks for partial sums y[split_k][M][N] in float32
// (no epilogue), to be added up by the consumer (alice_add_norm's n_partials).
// x_layout / y_layout: ALICE_LAYOUT_ROW, or ALICE_LAYOUT_FRAG16 for activations stored in fragment order
// ([M/16][K/32][64][8], bfloat16, rows padded to 16), which the producers of a decode step write.
int alice_linear(const void* x, int x_dtype, const void* w, int w_dtype, int w_layout, void* y, int y_dtype,
                 int M, int N, int K, int epilogue, float epi_param, int split_k, int variant,
                 int full_precision, int x_layout, int y_layout, hipStream_t stream);
// How many partial sums AUTO would like for this shape (1 = none).
int alice_linear_split_hint(int M, int N, int K, int w_layout);

// Rearranges a row-major bfloat16 [N, K] matrix into the fragment layout ([Np/16][Kp/32][64][8],
// zero padded); dst holds Np * Kp elements with Np = ceil16(N), Kp = ceil32(K).
int alice_to_frag16(const void* src, void* dst, int N, int K, hipStream_t stream);
int alice_frag16_supported(int rows, int K, int epilogue);

int alice_rope_cache_write(const void* qkv, int dtype, void* q_out, void* k_pool, void* v_pool,
                           const float* cos_t, const float* sin_t, const int* positions,
                           const int* seq_of_token, const int* block_table, int bt_stride, int T,
                           int row_width, int nH, int nKV, int d, int rotary_dim, int page_size, int n_pages,
                           int kv_layout, int interleaved, hipStream_t stream);

// The fused q|k|v projection with the rotation and the cache write as its epilogue (single tokens: the
// streaming kernel; more than 64 tokens: the tiled one): x [M, K] (row-major or fragment order), W in the fragment layout with the rows of every q and k
// head in pair order (rows j and j + d/2 of a head at 2j and 2j + 1).  Writes what alice_linear followed by
// alice_rope_cache_write (interleaved) would: q_out [M, nH * d] and the token's keys and values in the cache.
int alice_linear_rope_cache(const void* x, int x_layout, const void* w, int M, int K, void* q_out, void* k_pool,
                            void* v_pool, const float* cos_t, const float* sin_t, const int* positions,
                            const int* seq_of_token, const int* block_table, int bt_stride, int nH, int nKV, int d,
                            int page_size, int n_pages, int kv_layout, hipStream_t stream);

// bias_slopes: null, or nH floats: head h's capped score of key k for the query at position p gets
// bias_slopes[h] * (k - p) added before the softmax (a linear distance bias at the score stage).
int alice_attention_generic(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                            const int* positions, const int* seq_of_token, const int* block_table,
                            int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                            float softcap, int window, const float* bias_slopes, int full_precision,
                            hipStream_t stream);

// bfloat16 attention on the matrix cores over a cache in the fragment layout (kv_layout 1 of
// alice_rope_cache_write): prompts, and single tokens with the keys split over `splits` blocks.
int alice_attention_mfma_supported(int d);
int alice_attention_prefill(const void* q, const void* k_pool, const void* v_pool, void* out,
                            const int* cu_seqlens, const int* context_lens, const int* block_table,
                            int bt_stride, int B, int max_new, int nH, int nKV, int d, int page_size,
                            float scale, float softcap, int window, int variant, int out_layout, hipStream_t stream);
long alice_attention_decode_workspace(int B, int nH, int d, int splits);
// out may be absent when splits > 1: the splits are then left in `parts`, [B][nH][splits][ALICE_ATTN_PARTS_HEAD + d]
// = (maximum as a base-2 exponent, sum, two unused, unnormalised output: the output starts at a multiple of 16
// bytes), for alice_linear_parts to combine.
#define ALICE_ATTN_PARTS_HEAD 4
int alice_attention_decode(const void* q, const void* k_pool, const void* v_pool, void* out, float* parts,
                           const int* context_lens, const int* block_table, int bt_stride, int B, int nH,
                           int nKV, int d, int page_size, float scale, float softcap, int window, int splits,
                           int out_layout, hipStream_t stream);

// The output projection straight from the parts of alice_attention_decode (at most 16 sequences and 16 splits, weights in the
// fragment layout, [N, nH d]): y[slices][M][N] float32 partial sums, slices = alice_linear_parts_split(...), which
// is 0 where the sizes are not covered.
int alice_linear_parts_split(int M, int N, int nH, int d, int splits);
int alice_linear_parts(const float* parts, int splits, int nH, int d, const void* w, float* y, int M, int N,
                       hipStream_t stream);

// Lowest index among equal maxima.
int alice_argmax_chunks(int B, int V);
int alice_argmax(const float* logits, int* out, float* work_v, int* work_i, int B, int V, hipStream_t stream);
// The same argmax with no workspace argument and no allocation of any kind: the chunk maxima go to a device
// array inside the library (ALICE_ARGMAX_STATIC_MAX_PAIRS pairs of a float and an int, 4 KB, which every GPU
// that the library runs on holds until the process ends; it is the most that the chunk rule of
// alice_argmax_chunks ever asks for, ALICE_ARGMAX_MAX_PARTIALS, so no number of rows or vocabulary is too large).  It has no counterpart in the reference; it is for
// callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It calls no hipMalloc, hipFree or allocating library routine; the caller passes logits and out
// as for alice_argmax.  Rows x chunks beyond the maximum are refused with an error (a check that the chunk rule
// keeps from firing; missing pointers and bad sizes are refused the same way).  All
// calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race;
// calls on one stream follow each other and are safe.  alice_argmax_static_init() resolves the array's address
// for the current device ahead of the first call (the first call on a device does it otherwise).
#define ALICE_ARGMAX_MAX_PARTIALS 512
#define ALICE_ARGMAX_STATIC_MAX_PAIRS ALICE_ARGMAX_MAX_PARTIALS
int alice_argmax_static_init();
int alice_argmax_static(const float* logits, int* out, int B, int V, hipStream_t stream);
// temperature -> top-k (0: off) -> top-p (>= 1: off) -> softmax -> first index whose cumulative
// probability exceeds uniform[row].  work: alice_sample_workspace(B, V) 32-bit words, 8-byte aligned.
long alice_sample_workspace(int B, int V);
int alice_sample(const float* logits, int* out, const float* uniform, void* work, int B, int V, float temperature,
                 int top_k, float top_p, hipStream_t stream);

#ifdef __cplusplus
}

// internal
int alice_linear_generic(const void* x, int x_dtype, const void* w, int w_dtype, void* y, int y_dtype,
                         int M, int N, int K, int epi, float epi_param, int full_precision,
                         hipStream_t stream);
#endif
