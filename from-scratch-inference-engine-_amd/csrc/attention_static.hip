// Split-key attention and its merge with the partial records in a buffer that the library owns:
// an entry point that allocates nothing, for callers that cannot allocate.
#include "common.h"
#include "api.h"

#include <atomic>

namespace {

// Partial records of the key splits: per slot and head, head_dim weighted sums, the maximum and
// the denominator, all float32.  One array per GPU that the library runs on, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress; the device
// address that kernels and copies take is kept in g_scratch[device].
static __device__ __align__(256) unsigned char scratch[FSIE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
// (several host threads may make their first call at once: every one of them gets the same
// address from the runtime, so the store needs to be atomic and nothing more)
std::atomic<void*> g_scratch[kMaxDevices];

// The items and merges come from device memory that this entry point cannot read on the host
// without waiting for the device.  A record that names a partial slot at or beyond the caller's
// `n_partial_slots` would write or read past what was checked against the buffer's size; so the
// tables are copied into the buffer, behind the partial records, with every such record turned
// into one that does nothing (an item of no query tokens, a merge of no splits), and the kernels
// read the copies.
__global__ __launch_bounds__(256) void bounded_tables_kernel(const int32_t* __restrict__ items, int n_items,
                                                             const int32_t* __restrict__ merges, int n_merges,
                                                             int slot_limit, int32_t* __restrict__ items_out,
                                                             int32_t* __restrict__ merges_out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_items) {
        const int32_t* it = items + static_cast<int64_t>(i) * FSIE_ATTN_ITEM_INTS;
        int32_t* o = items_out + static_cast<int64_t>(i) * FSIE_ATTN_ITEM_INTS;
        const int64_t base = it[FSIE_ATTN_ITEM_PARTIAL];
        const int64_t nq = it[FSIE_ATTN_ITEM_NQ];
        const bool ok = base < 0 || base + (nq > 0 ? nq : 0) <= slot_limit;
#pragma unroll
        for (int j = 0; j < FSIE_ATTN_ITEM_INTS; ++j) o[j] = it[j];
        if (!ok) o[FSIE_ATTN_ITEM_NQ] = 0;
    } else if (i - n_items < n_merges) {
        const int m = i - n_items;
        const int32_t* mi = merges + static_cast<int64_t>(m) * FSIE_ATTN_MERGE_INTS;
        int32_t* o = merges_out + static_cast<int64_t>(m) * FSIE_ATTN_MERGE_INTS;
        const int64_t first = mi[1], n = mi[2], stride = mi[3];
        const bool ok = n <= 0 || (first >= 0 && stride >= 0 && first + (n - 1) * stride < slot_limit);
        o[0] = mi[0], o[1] = mi[1], o[2] = ok ? mi[2] : 0, o[3] = mi[3];
    }
}

// The device address of this GPU's array: asked once per device, with that device current.
int scratch_of_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    FSIE_REQUIRE(e == hipSuccess, "attention_split_static: hipGetDevice: %s", hipGetErrorString(e));
    FSIE_REQUIRE(dev >= 0 && dev < kMaxDevices, "attention_split_static: device %d is beyond the %d this library keeps",
                 dev, kMaxDevices);
    void* p = g_scratch[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        FSIE_REQUIRE(e == hipSuccess && p != nullptr, "attention_split_static: hipGetSymbolAddress: %s",
                     hipGetErrorString(e));
        g_scratch[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return 0;
}

}  // namespace

extern "C" int64_t fsie_static_scratch_bytes(void) { return FSIE_STATIC_SCRATCH_BYTES; }

extern "C" int fsie_attention_split_static(const void* q, int64_t q_stride, const void* k_pool, const void* v_pool,
                                           const int32_t* block_tables, int max_pages, const int32_t* items,
                                           int n_items, const int32_t* merges, int n_merges, int n_partial_slots,
                                           void* out, int n_heads, int n_kv, int head_dim, int page_size, int window,
                                           float scale, int dtype, int mfma, int waves, hipStream_t stream) {
    FSIE_REQUIRE(n_items >= 0 && n_merges >= 0 && n_partial_slots >= 0, "attention_split_static: negative counts");
    FSIE_REQUIRE(n_heads > 0 && head_dim > 0, "attention_split_static: bad sizes");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "attention_split_static: unknown dtype %d", dtype);
    FSIE_REQUIRE(!mfma || dtype == FSIE_BF16, "attention_split_static: the matrix-core kernel takes bfloat16 only");
    // the buffer holds the partial records and, behind them, the bounded copies of the two tables
    const int64_t records = (static_cast<int64_t>(n_partial_slots) * n_heads * (head_dim + 2) * sizeof(float) + 255) / 256 * 256;
    const int64_t item_bytes = (static_cast<int64_t>(n_items) * FSIE_ATTN_ITEM_INTS * sizeof(int32_t) + 255) / 256 * 256;
    const int64_t merge_bytes = static_cast<int64_t>(n_merges) * FSIE_ATTN_MERGE_INTS * sizeof(int32_t);
    const int64_t need = records + item_bytes + merge_bytes;
    FSIE_REQUIRE(need <= FSIE_STATIC_SCRATCH_BYTES,
                 "attention_split_static: %d partial slots of %d heads of %d with %d items and %d merges need %lld "
                 "bytes, the library's buffer has %lld", n_partial_slots, n_heads, head_dim, n_items, n_merges,
                 static_cast<long long>(need), static_cast<long long>(FSIE_STATIC_SCRATCH_BYTES));
    FSIE_REQUIRE(n_merges == 0 || n_partial_slots > 0, "attention_split_static: merges without partial slots");
    void* base = nullptr;
    if (int rc = scratch_of_current_device(&base)) return rc;
    float* partials = static_cast<float*>(base);
    int32_t* items_in = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(base) + records);
    int32_t* merges_in = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(base) + records + item_bytes);
    if (n_items + n_merges > 0) {
        bounded_tables_kernel<<<(n_items + n_merges + 255) / 256, 256, 0, stream>>>(items, n_items, merges, n_merges,
                                                                                    n_partial_slots, items_in, merges_in);
        FSIE_CHECK_LAUNCH("attention_split_static: bounded_tables");
    }
    // nothing has to start at zero: an item writes the whole record of every slot that a merge
    // reads, and a merge reads no other slot
    int rc = mfma ? fsie_attention_mfma(q, q_stride, k_pool, v_pool, block_tables, max_pages, items_in, n_items, out,
                                        partials, n_heads, n_kv, head_dim, page_size, window, scale, 0, waves, stream)
                  : fsie_attention_scalar(q, q_stride, k_pool, v_pool, block_tables, max_pages, items_in, n_items, out,
                                          partials, n_heads, n_kv, head_dim, page_size, window, scale, dtype, stream);
    if (rc) return rc;
    return fsie_attention_merge(partials, merges_in, n_merges, out, n_heads, head_dim, dtype, stream);
}
