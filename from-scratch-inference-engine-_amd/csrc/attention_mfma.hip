// Entry point of the matrix-core attention (bfloat16): picks the instantiation for the head size.
#include "attention_mfma_impl.h"

namespace fsie_attn {
LaunchFn table_a(int hdt, int large);
LaunchFn table_b(int hdt, int large);
LaunchFn table_c(int hdt, int large);
LaunchFn table_d(int hdt, int large);
LaunchQkvFn table_a_qkv(int hdt);
LaunchQkvFn table_b_qkv(int hdt);
LaunchQkvFn table_c_qkv(int hdt);
LaunchQkvFn table_d_qkv(int hdt);
}  // namespace fsie_attn

// Waves that a workgroup of the small variant may use to split an item's keys.
extern "C" int fsie_attention_mfma_max_waves(int head_dim) {
    if (head_dim <= 0 || head_dim % 16 || head_dim > 256) return 0;
    return head_dim <= 64 ? 16 : (head_dim <= 128 ? 8 : 4);
}

// Query tiles of 16 rows that one wave of the `large` variant holds for this head size.
extern "C" int fsie_attention_mfma_tiles(int head_dim, int large) {
    if (head_dim <= 0 || head_dim % 16 || head_dim > 256) return 0;
    if (!large) return 1;
    return 2;
}

// bfloat16 only; head_dim a multiple of 16 up to 256; page_size a multiple of 4.
// large = 0: items of at most 16 rows (tokens x heads of a group); large = 1: up to 16 * tiles rows.
// `waves` waves of a workgroup split each item's keys (at most 4 for large items).
extern "C" int fsie_attention_mfma(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                   const int32_t* block_tables, int max_pages, const int32_t* items, int n_items,
                                   void* out, float* partials, int n_heads, int n_kv, int head_dim, int page_size,
                                   int window, float scale, int large, int waves, hipStream_t stream) {
    FSIE_REQUIRE(n_items >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
                 "attention_mfma: heads %d must be a positive multiple of kv heads %d", n_heads, n_kv);
    FSIE_REQUIRE(head_dim > 0 && head_dim % 16 == 0 && head_dim <= 256,
                 "attention_mfma: head_dim %d must be a multiple of 16 up to 256", head_dim);
    FSIE_REQUIRE(page_size > 0 && page_size % 4 == 0, "attention_mfma: page_size %d must be a multiple of 4", page_size);
    FSIE_REQUIRE(max_pages > 0, "attention_mfma: empty block table");
    // the kernel divides a key's position by the page size with one multiplication, exact below this
    FSIE_REQUIRE((static_cast<int64_t>(max_pages) + 8) * page_size * page_size < (int64_t{1} << 32),
                 "attention_mfma: %d pages of %d keys are more than the kernel can address", max_pages, page_size);
    FSIE_REQUIRE(q_stride % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0,
                 "attention_mfma: query rows must be 16-byte aligned");
    if (n_items == 0) return 0;
    const int hdt = head_dim / 16;
    fsie_attn::LaunchFn fn = hdt <= 4 ? fsie_attn::table_a(hdt, large)
                           : hdt <= 8 ? fsie_attn::table_b(hdt, large)
                           : hdt <= 12 ? fsie_attn::table_c(hdt, large) : fsie_attn::table_d(hdt, large);
    FSIE_REQUIRE(fn != nullptr, "attention_mfma: no kernel for head_dim %d", head_dim);
    return fn(q, q_stride, k_pool, v_pool, block_tables, max_pages, items, n_items, out, partials, n_heads, n_kv,
              page_size, window, scale, waves, stream);
}

// Whether fsie_attention_mfma_qkv has a kernel for these sizes.
extern "C" int fsie_attention_mfma_qkv_ok(int head_dim, int page_size) {
    return head_dim > 0 && head_dim % 32 == 0 && head_dim <= 256 && page_size > 0 && page_size % 8 == 0;
}

// Attention for a step of one token a request (every item has one query row per head), straight from
// the q/k/v product's float32 partial sums [n_parts][n_tokens][(n_heads + 2 n_kv) head_dim]: the kernel adds
// them up, adds `bias` (or null), rotates queries and keys by cos_sin [n_tokens][head_dim / 2][2],
// scores the new key from registers and writes it and the value to slots[t] of the pools (negative,
// or not below pool_slots: not written).  Otherwise as fsie_attention_mfma with large = 0.
extern "C" int fsie_attention_mfma_qkv(const float* sums, int n_parts, int n_tokens, const float* bias,
                                       const float* cos_sin, const int32_t* slots, void* k_pool, void* v_pool,
                                       int64_t pool_slots, const int32_t* block_tables, int max_pages,
                                       const int32_t* items, int n_items, void* out, float* partials, int n_heads,
                                       int n_kv, int head_dim, int page_size, int window, float scale, int waves,
                                       hipStream_t stream) {
    FSIE_REQUIRE(n_items >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
                 "attention_mfma_qkv: heads %d must be a positive multiple of kv heads %d", n_heads, n_kv);
    FSIE_REQUIRE(fsie_attention_mfma_qkv_ok(head_dim, page_size),
                 "attention_mfma_qkv: head_dim %d must be a multiple of 32 up to 256 and page_size %d a multiple of 8",
                 head_dim, page_size);
    FSIE_REQUIRE(max_pages > 0, "attention_mfma_qkv: empty block table");
    FSIE_REQUIRE((static_cast<int64_t>(max_pages) + 8) * page_size * page_size < (int64_t{1} << 32),
                 "attention_mfma_qkv: %d pages of %d keys are more than the kernel can address", max_pages, page_size);
    FSIE_REQUIRE(n_parts >= 1 && n_tokens >= 1 && pool_slots >= 0, "attention_mfma_qkv: bad sizes parts=%d T=%d",
                 n_parts, n_tokens);
    FSIE_REQUIRE(sums && cos_sin && slots && k_pool && v_pool && block_tables && items && out,
                 "attention_mfma_qkv: missing operand");
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(sums) % 16 == 0 && reinterpret_cast<uintptr_t>(bias) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0 && reinterpret_cast<uintptr_t>(k_pool) % 4 == 0,
                 "attention_mfma_qkv: sums and bias must be 16-byte aligned, the cosines and sines 8-byte");
    if (n_items == 0) return 0;
    const int hdt = head_dim / 16;
    fsie_attn::LaunchQkvFn fn = hdt <= 4 ? fsie_attn::table_a_qkv(hdt)
                              : hdt <= 8 ? fsie_attn::table_b_qkv(hdt)
                              : hdt <= 12 ? fsie_attn::table_c_qkv(hdt) : fsie_attn::table_d_qkv(hdt);
    FSIE_REQUIRE(fn != nullptr, "attention_mfma_qkv: no kernel for head_dim %d", head_dim);
    fsie_attn::QkvSums f;
    f.sums = sums;
    f.bias = bias;
    f.cos_sin = cos_sin;
    f.slots = slots;
    f.k_out = static_cast<bf16_t*>(k_pool);
    f.v_out = static_cast<bf16_t*>(v_pool);
    f.width = (n_heads + 2 * n_kv) * head_dim;
    f.part_stride = static_cast<int64_t>(n_tokens) * f.width;
    f.pool_slots = pool_slots;
    f.n_parts = n_parts;
    return fn(f, k_pool, v_pool, block_tables, max_pages, items, n_items, out, partials, n_heads, n_kv, page_size,
              window, scale, waves, stream);
}
