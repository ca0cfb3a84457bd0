// Rotary position encoding on q and k, fused with the q/k/v bias and with the write of k (rotated)
// and v into the pages of the cache.  One block per token.  The v columns of the row itself are
// left without the bias: only the cache is read afterwards.
//
// Page layout: keys [page][kv_head][slot in page][head_dim]; values transposed,
// [page][kv_head][head_dim][slot in page], so that the matrix-core attention kernel reads
// consecutive keys of one dimension with one load.
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxHalf = 256;  // head_dim <= 512

// angle = position * inv_freq in float64, as the plain formula has it, reduced in float64 to
// [-pi, pi]; there float32 sine and cosine are within a few 1e-7 of the float64 ones.
__device__ __forceinline__ void rotation(double pos, double inv_freq, float* c, float* s) {
    const double ang = pos * inv_freq;
    const double turns = rint(ang * 0.15915494309189535);  // 1 / (2 pi)
    const double red = fma(-turns, 6.283185307179586, ang) - turns * 2.4492935982947064e-16;  // 2 pi = hi + lo
    sincosf(static_cast<float>(red), s, c);
}

// No LDS and no barrier: every thread rotates whole pairs, and a pair of a k head goes to the row
// and to its cache slot from the same registers; the values are copied in a loop of their own.
template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(kThreads) void rope_kv_write_kernel(
    T* __restrict__ qkv, const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
    const double* __restrict__ inv_freq, const float* __restrict__ bias, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int n_heads, int n_kv, int head_dim, int rotary_half, int page_size, int write_kv,
    int64_t pool_slots) {
    const int t = blockIdx.x;
    const int q_dim = n_heads * head_dim;
    const int kv_dim = n_kv * head_dim;
    T* row = qkv + static_cast<int64_t>(t) * (q_dim + 2 * kv_dim);
    int slot = (write_kv && slots) ? slots[t] : -1;
    if (slot >= pool_slots) slot = -1;
    const int64_t page = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot % page_size : 0;

    // values first: their loads do not wait for the position
    if (slot >= 0) {
        const T* v = row + q_dim + kv_dim;
        for (int idx = threadIdx.x; idx < kv_dim; idx += blockDim.x) {
            const int kvh = idx / head_dim;
            const int d = idx - kvh * head_dim;
            const int64_t head = (page * n_kv + kvh) * page_size * head_dim;
            v_pool[head + static_cast<int64_t>(d) * page_size + off] =
                HAS_BIAS ? from_float<T>(to_float(v[idx]) + bias[q_dim + kv_dim + idx]) : v[idx];
        }
    }

    // q and k heads (k heads follow the q heads directly in a row): add the bias, rotate the
    // pairs (i, i + rotary_half) of the first 2*rotary_half dimensions
    const double pos = static_cast<double>(positions[t]);
    const int n_rot_heads = n_heads + n_kv;
    const int n_pairs = n_rot_heads * rotary_half;
    constexpr int PB = 8;  // pairs in flight per thread
    for (int base = threadIdx.x; base < n_pairs; base += blockDim.x * PB) {
        // loads only, from clamped places and without a branch, so that they all go out before
        // the first of them is waited for
        float x1[PB], x2[PB], b1[PB], b2[PB];
        double freq[PB];
        int which[PB];
#pragma unroll
        for (int u = 0; u < PB; ++u) {
            const int idx = min(base + u * static_cast<int>(blockDim.x), n_pairs - 1);
            const int h = idx / rotary_half;
            const int i = idx - h * rotary_half;
            const T* head = row + h * head_dim;
            which[u] = i;
            freq[u] = inv_freq[i];
            x1[u] = to_float(head[i]);
            x2[u] = to_float(head[i + rotary_half]);
            b1[u] = HAS_BIAS ? bias[h * head_dim + i] : 0.f;
            b2[u] = HAS_BIAS ? bias[h * head_dim + i + rotary_half] : 0.f;
        }
        float c = 1.f, s = 0.f;
#pragma unroll
        for (int u = 0; u < PB; ++u) {
            const int idx = base + u * blockDim.x;
            // the same angle for the whole batch when blockDim is a multiple of rotary_half
            if (u == 0 || which[u] != which[u - 1]) rotation(pos, freq[u], &c, &s);
            if (idx >= n_pairs) continue;
            const int h = idx / rotary_half;
            const int i = which[u];
            const float a1 = x1[u] + b1[u], a2 = x2[u] + b2[u];
            const T r1 = from_float<T>(a1 * c - a2 * s);
            const T r2 = from_float<T>(a2 * c + a1 * s);
            T* head = row + h * head_dim;
            head[i] = r1;
            head[i + rotary_half] = r2;
            if (h >= n_heads && slot >= 0) {
                T* dst = k_pool + ((page * n_kv + (h - n_heads)) * page_size + off) * head_dim;
                dst[i] = r1;
                dst[i + rotary_half] = r2;
            }
        }
    }
    // dimensions beyond the rotary ones only take the bias
    const int rest = head_dim - 2 * rotary_half;
    if (rest > 0) {
        for (int idx = threadIdx.x; idx < n_rot_heads * rest; idx += blockDim.x) {
            const int h = idx / rest;
            const int d = 2 * rotary_half + (idx - h * rest);
            T* head = row + h * head_dim;
            const T v = HAS_BIAS ? from_float<T>(to_float(head[d]) + bias[h * head_dim + d]) : head[d];
            head[d] = v;
            if (h >= n_heads && slot >= 0) k_pool[((page * n_kv + (h - n_heads)) * page_size + off) * head_dim + d] = v;
        }
    }
}

// table[t][i] = (cos, sin) of positions[t] * inv_freq[i]: the angles of a step are the same in
// every layer, so a step computes them once and the layers' kernels read them.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ inv_freq,
                                  float2* __restrict__ table, int half) {
    const int t = blockIdx.x;
    const double pos = static_cast<double>(positions[t]);
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float c, s;
        rotation(pos, inv_freq[i], &c, &s);
        table[static_cast<int64_t>(t) * half + i] = float2{c, s};
    }
}

}  // namespace

extern "C" int fsie_rope_table(const int32_t* positions, const double* inv_freq, int n_tokens, int half,
                               float* table, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && half > 0 && half <= kMaxHalf, "rope_table: bad sizes T=%d half=%d", n_tokens, half);
    FSIE_REQUIRE(positions && inv_freq && table, "rope_table: missing operand");
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(table) % 8 == 0, "rope_table: the table must be 8-byte aligned");
    if (n_tokens == 0) return 0;
    rope_table_kernel<<<n_tokens, half < 64 ? 64 : (half < 256 ? half : 256), 0, stream>>>(
        positions, inv_freq, reinterpret_cast<float2*>(table), half);
    FSIE_CHECK_LAUNCH("rope_table");
    return 0;
}

extern "C" int fsie_rope_kv_write(void* qkv, const int32_t* positions, const int32_t* slots,
                                  const double* inv_freq, const float* bias, void* k_pool, void* v_pool, int n_tokens,
                                  int n_heads, int n_kv, int head_dim, int rotary_dim, int page_size,
                                  int64_t pool_slots, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0, "rope_kv_write: bad sizes");
    FSIE_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim / 2 <= kMaxHalf,
                 "rope_kv_write: head_dim %d must be even and <= %d", head_dim, 2 * kMaxHalf);
    FSIE_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
                 "rope_kv_write: rotary_dim %d must be even and within head_dim %d", rotary_dim, head_dim);
    FSIE_REQUIRE(rotary_dim == 0 || inv_freq, "rope_kv_write: no frequency table");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "rope_kv_write: unknown dtype %d", dtype);
    const int write_kv = (k_pool && v_pool && slots) ? 1 : 0;
    FSIE_REQUIRE(!write_kv || (page_size > 0 && pool_slots > 0), "rope_kv_write: bad page geometry");
    if (n_tokens == 0) return 0;
#define FSIE_ROPE_LAUNCH(T, B)                                                                                   \
    rope_kv_write_kernel<T, B><<<n_tokens, kThreads, 0, stream>>>(                                               \
        static_cast<T*>(qkv), positions, slots, inv_freq, bias, static_cast<T*>(k_pool), static_cast<T*>(v_pool), \
        n_heads, n_kv, head_dim, rotary_dim / 2, page_size, write_kv, pool_slots)
    if (dtype == FSIE_F32) {
        if (bias) FSIE_ROPE_LAUNCH(float, true); else FSIE_ROPE_LAUNCH(float, false);
    } else {
        if (bias) FSIE_ROPE_LAUNCH(bf16_t, true); else FSIE_ROPE_LAUNCH(bf16_t, false);
    }
#undef FSIE_ROPE_LAUNCH
    FSIE_CHECK_LAUNCH("rope_kv_write");
    return 0;
}
