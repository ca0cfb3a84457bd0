// C interface of the kernel library (loaded from Python through ctypes).
//
// Conventions: every function returns 0 on success; otherwise fsie_last_error() describes the
// refusal (sizes a kernel does not take are refused here, never computed wrongly).  Pointers are
// device pointers unless said otherwise.  `dtype` is the type of activations and matrices:
// 0 = float32, 1 = bfloat16.  All work is queued on `stream`; nothing synchronises.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define FSIE_GEMM_SKINNY_MAX_M 8
#define FSIE_GEMM_MFMA_SKINNY_MAX_M 64
#define FSIE_GEMM_MFMA_WIDE_MAX_M 128  // the product that shares x through LDS, on a fragment-ordered weight: eight tiles of 16 rows
#define FSIE_GEMM_MFMA_SKINNY_BEST_M 16  // above this the library product is faster on MI355X
#define FSIE_GEMM_MAX_SPLITS 16          // most slices of K a product may leave as partial sums

// one attention work item = 8 int32
#define FSIE_ATTN_ITEM_INTS 8
#define FSIE_ATTN_ITEM_SEQ 0      // row of the block table
#define FSIE_ATTN_ITEM_QROW 1     // first query row (token index within the step)
#define FSIE_ATTN_ITEM_NQ 2       // query tokens in the tile (0 = padding item, skipped)
#define FSIE_ATTN_ITEM_POS 3      // absolute position of the first query token
#define FSIE_ATTN_ITEM_KBEGIN 4   // first key
#define FSIE_ATTN_ITEM_KEND 5     // one past the last key
#define FSIE_ATTN_ITEM_PARTIAL 6  // -1: write the output; >= 0: first partial slot of the tile
// one merge item = 4 int32: {output row, first partial slot, number of splits, slot stride}
#define FSIE_ATTN_MERGE_INTS 4

#ifdef __cplusplus
extern "C" {
#endif

const char* fsie_last_error(void);
int fsie_version(void);
// Name of the architecture the device code was built for and of the device present.
int fsie_device_info(char* arch_out, int arch_len, int* n_compute_units);
// Compute units of the current device; 0 if there is no device to ask.
int fsie_device_compute_units(void);

int fsie_embedding(const void* table, int dtype, const int32_t* ids, float* out, int n_tokens, int hidden,
                   int vocab, hipStream_t stream);
int fsie_rmsnorm(float* residual, const void* delta, const float* weight, void* out, const int32_t* rows,
                 int n_rows, int hidden, float eps, int dtype, int write_back, int n_parts, int total_rows,
                 hipStream_t stream);
// RMSNorm of a plain tensor (no residual stream): every row holds `groups` runs of `width` values
// (strides in elements), each run normalised by itself; `out` may be `x`.
int fsie_rmsnorm_plain(const void* x, int64_t x_stride, const float* weight, void* out, int64_t out_stride, int n_rows,
                       int groups, int width, float eps, int dtype, hipStream_t stream);
// Rows slots[0..n) of a table of n_slots rows of row_bytes set to zero; a negative slot is skipped.
int fsie_zero_rows(void* table, const int32_t* slots, int n, int64_t row_bytes, int n_slots, hipStream_t stream);
// Pages pages[0..n) (negative: skipped) of two pools of [planes][n_pages][page_bytes] set to zero.
int fsie_zero_pages(void* pool_a, void* pool_b, const int32_t* pages, int n, int planes, int n_pages,
                    int64_t page_bytes, hipStream_t stream);
// Counter-based random values (the random-weights mode): see elementwise.hip.
int fsie_random_fill(void* out, int64_t n, uint64_t key, int kind, float std, hipStream_t stream);
int fsie_swiglu(const void* x, void* out, int n_tokens, int inter, int dtype, hipStream_t stream);
int fsie_residual_add(float* residual, const void* delta, int64_t total, int dtype, hipStream_t stream);
int fsie_bias_add(void* y, const float* bias, int rows, int cols, int dtype, hipStream_t stream);

int fsie_rope_kv_write(void* qkv, const int32_t* positions, const int32_t* slots, const double* inv_freq,
                       const float* bias, void* k_pool, void* v_pool, int n_tokens, int n_heads, int n_kv, int head_dim,
                       int rotary_dim, int page_size, int64_t pool_slots, int dtype, hipStream_t stream);

// the same with the whole head rotated by the cosines and sines of fsie_rope_table (head_dim % 8 == 0);
// parts (or null): the projection as n_parts float32 partial sums [n_parts][n_tokens][width], added in
// order; qkv then only receives the q heads
int fsie_rope_kv_write_table(void* qkv, const float* cos_sin, const int32_t* slots, const float* bias, void* k_pool,
                             void* v_pool, int n_tokens, int n_heads, int n_kv, int head_dim, int page_size,
                             int64_t pool_slots, int dtype, const float* parts, int n_parts, hipStream_t stream);

// table [n_tokens, half, 2] float32: cos and sin of positions[t] * inv_freq[i]
int fsie_rope_table(const int32_t* positions, const double* inv_freq, int n_tokens, int half, float* table,
                    hipStream_t stream);

int fsie_gemm(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, int dtype,
              int out_f32, int kind, hipStream_t stream);

// True float32 on the matrix cores (v_mfma_f32_16x16x4_f32) for up to 64 rows: the 32-bit path's decoding.
int fsie_gemm_mfma_fp32(const float* x, const float* w, const float* bias, float* y, int M, int N, int K, int waves,
                        hipStream_t stream);

int fsie_gemm_mfma_skinny(const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                          int out_f32, int waves, int blocks, int epilogue, int splits, hipStream_t stream);

int fsie_gemm_mfma_skinny_rope(const void* x, const void* w, const float* bias, void* y, int M, int K,
                               const int32_t* positions, const int32_t* slots, const double* inv_freq,
                               const float* cos_sin, void* k_pool,
                               void* v_pool, int n_heads, int n_kv, int head_dim, int page_size, int64_t pool_slots,
                               hipStream_t stream);

// 17 to 64 rows (any number up to 64 is taken): X shared through LDS, float32 result or partial sums
int fsie_gemm_mfma_wide_slice(int K, int splits);
int fsie_gemm_mfma_wide_best_splits(int M, int N, int K);
// (frags: w is the copy of the matrix in the order of the A fragments, made by fsie_fragment_order)
int fsie_gemm_mfma_wide(const void* x, const void* w, float* y, int M, int N, int K, int splits, int waves,
                        int blocks, int frags, hipStream_t stream);
// the rows of w are gate and up in turn: y is bfloat16 [M, N / 2], silu(gate) * up
int fsie_gemm_mfma_wide_swiglu(const void* x, const void* w, void* y, int M, int N, int K, int waves, int blocks,
                               int frags, hipStream_t stream);
// A bfloat16 matrix [N, K] (K a multiple of 32) copied so that the 64 16-byte units of a block of 16
// rows and 32 values of K lie together in the order of the lanes that hold them: a wave's load of W
// is then one piece of 1 KB.  The copy has fsie_fragment_order_size values (N rounded up to 16 rows).
// whether they take M rows of this shape (65 to FSIE_GEMM_MFMA_WIDE_MAX_M rows: only some launch shapes on a
// fragment-ordered weight)
int fsie_gemm_mfma_wide_takes(int M, int N, int K, int splits, int gate_up, int frags);
int64_t fsie_fragment_order_size(int N, int K);
int fsie_fragment_order(const void* w, void* out, int N, int K, hipStream_t stream);

int fsie_attention_scalar(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                          const int32_t* block_tables, int max_pages, const int32_t* items, int n_items,
                          void* out, float* partials, int n_heads, int n_kv, int head_dim, int page_size,
                          int window, float scale, int dtype, hipStream_t stream);
int fsie_attention_merge(const float* partials, const int32_t* merges, int n_merges, void* out, int n_heads,
                         int head_dim, int dtype, hipStream_t stream);
int fsie_attention_scalar_tile_tokens(int n_heads, int n_kv);

int fsie_attention_mfma(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                        const int32_t* block_tables, int max_pages, const int32_t* items, int n_items, void* out,
                        float* partials, int n_heads, int n_kv, int head_dim, int page_size, int window, float scale,
                        int large, int waves, hipStream_t stream);
// the same for a step of one token a request, from the q/k/v product's partial sums: bias, rotation and the
// write into the pools happen in the kernel
int fsie_attention_mfma_qkv_ok(int head_dim, int page_size);
int fsie_attention_mfma_qkv(const float* sums, int n_parts, int n_tokens, const float* bias, const float* cos_sin,
                            const int32_t* slots, void* k_pool, void* v_pool, int64_t pool_slots,
                            const int32_t* block_tables, int max_pages, const int32_t* items, int n_items, void* out,
                            float* partials, int n_heads, int n_kv, int head_dim, int page_size, int window,
                            float scale, int waves, hipStream_t stream);
int fsie_attention_mfma_lds_ok(int head_dim, int page_size);
int fsie_attention_mfma_lds(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                            const int32_t* block_tables, int max_pages, const int32_t* items, const int32_t* groups,
                            int n_groups, void* out, int n_heads, int n_kv, int head_dim, int page_size, int window,
                            float scale, hipStream_t stream);
int fsie_attention_mfma_tiles(int head_dim, int large);
int fsie_attention_mfma_max_waves(int head_dim);

// ---- an entry point that allocates nothing --------------------------------------------------
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// fsie_attention_scalar / fsie_attention_mfma (small items) followed by fsie_attention_merge, as one
// call, with the partial records of the key splits kept in a buffer of FSIE_STATIC_SCRATCH_BYTES
// that the library itself holds on every GPU it runs on (a file-scope device array; nothing is
// allocated or freed, here or in any routine called from here).  The caller passes the inputs, the
// tables and the output as for those entry points; `n_partial_slots` is one more than the largest
// partial slot that `items` and `merges` name (slot = one query token of one split); a step that
// needs more than the buffer holds is refused with an error, never computed.  The two tables lie in
// device memory, which this call does not wait for: it runs the kernels on copies of them (kept in
// the same buffer, behind the records, and counted against its size) in which an item or merge that
// names a slot at or beyond `n_partial_slots` does nothing, so a wrong table leaves rows of `out`
// unwritten and never reaches memory outside the buffer.  `mfma` != 0: the
// matrix-core kernel (bfloat16), else the float32-arithmetic kernel.  Every call on a GPU uses
// that GPU's one buffer, which keeps the last call's contents: calls that overlap on one GPU
// (different streams, or threads) race; calls on one stream are ordered and safe.  Nothing needs
// clearing between calls: an item writes every record that a merge reads.
#define FSIE_STATIC_SCRATCH_BYTES (16 * 1024 * 1024)
int64_t fsie_static_scratch_bytes(void);
int fsie_attention_split_static(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                const int32_t* block_tables, int max_pages, const int32_t* items, int n_items,
                                const int32_t* merges, int n_merges, int n_partial_slots, void* out, int n_heads,
                                int n_kv, int head_dim, int page_size, int window, float scale, int dtype, int mfma,
                                int waves, hipStream_t stream);

int fsie_sample(const float* logits, int n_rows, int vocab, const float* temperature, const int32_t* top_k,
                const float* top_p, const double* uniform, int32_t* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
