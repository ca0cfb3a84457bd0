// Split-key attention and its merge with the partial records in a buffer that the library owns:
// an entry point that allocates nothing, for callers that cannot allocate.
#include "common.h"
#include "api.h"

namespace {

// Partial records of the key splits: per slot and head, head_dim weighted sums, the maximum and
// the denominator, all float32.  One array per GPU that the library runs on, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress; the device
// address that kernels and copies take is kept in g_scratch[device].
static __device__ __align__(256) unsigned char scratch[FSIE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void* g_scratch[kMaxDevices] = {nullptr};

// The device address of this GPU's array: asked once per device, with that device current.
int scratch_of_current_device(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    FSIE_REQUIRE(e == hipSuccess, "attention_split_static: hipGetDevice: %s", hipGetErrorString(e));
    FSIE_REQUIRE(dev >= 0 && dev < kMaxDevices, "attention_split_static: device %d is beyond the %d this library keeps",
                 dev, kMaxDevices);
    if (g_scratch[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        FSIE_REQUIRE(e == hipSuccess && p != nullptr, "attention_split_static: hipGetSymbolAddress: %s",
                     hipGetErrorString(e));
        g_scratch[dev] = p;
    }
    *ptr = g_scratch[dev];
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
    const int64_t need = static_cast<int64_t>(n_partial_slots) * n_heads * (head_dim + 2) * sizeof(float);
    FSIE_REQUIRE(need <= FSIE_STATIC_SCRATCH_BYTES,
                 "attention_split_static: %d partial slots of %d heads of %d need %lld bytes, the library's buffer "
                 "has %lld", n_partial_slots, n_heads, head_dim, static_cast<long long>(need),
                 static_cast<long long>(FSIE_STATIC_SCRATCH_BYTES));
    FSIE_REQUIRE(n_merges == 0 || n_partial_slots > 0, "attention_split_static: merges without partial slots");
    void* base = nullptr;
    if (int rc = scratch_of_current_device(&base)) return rc;
    float* partials = static_cast<float*>(base);
    // nothing has to start at zero: an item writes the whole record of every slot that a merge
    // reads, and a merge reads no other slot
    int rc = mfma ? fsie_attention_mfma(q, q_stride, k_pool, v_pool, block_tables, max_pages, items, n_items, out,
                                        partials, n_heads, n_kv, head_dim, page_size, window, scale, 0, waves, stream)
                  : fsie_attention_scalar(q, q_stride, k_pool, v_pool, block_tables, max_pages, items, n_items, out,
                                          partials, n_heads, n_kv, head_dim, page_size, window, scale, dtype, stream);
    if (rc) return rc;
    return fsie_attention_merge(partials, merges, n_merges, out, n_heads, head_dim, dtype, stream);
}
