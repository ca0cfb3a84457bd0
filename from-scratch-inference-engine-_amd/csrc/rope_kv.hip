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

// Four values in 16 (float32) or 8 (bfloat16) bytes.
template <typename T>
struct Quad;
template <>
struct Quad<float> {
    static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <>
struct Quad<bf16_t> {
    static __device__ __forceinline__ float4 load(const bf16_t* p) {
        const uint2 w = *reinterpret_cast<const uint2*>(p);
        return float4{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                      __uint_as_float(w.y & 0xffff0000u)};
    }
    static __device__ __forceinline__ void store(bf16_t* p, float4 v) {
        *reinterpret_cast<uint2*>(p) = uint2{pack2_bf16(v.x, v.y), pack2_bf16(v.z, v.w)};
    }
};

// The same work with the cosines and sines read from the step's table [T][head_dim / 2][2] and four
// pairs a thread: no trigonometry, 8- and 16-byte accesses.  The whole head is rotated; head_dim is
// a multiple of 8.  A block takes TOK consecutive tokens: 1, or 8 for long batches (prompt portions).
// Values lie transposed in a page, [head_dim][slot]: a token alone writes 2 bytes per dimension, and
// the tokens of one 32-byte run would come from blocks on different dies, each of which would hand
// its bytes of the run to memory separately.  Eight tokens whose slots are consecutive and start at
// a multiple of 8 (a portion of a prompt) write 16 bytes per dimension at once.
// PARTS: the projection comes as float32 partial sums parts[n_parts][n_tokens][width] of a product
// whose inner dimension was cut into slices; they are added in the order of the slices, and qkv
// only receives the q heads (TOK == 1).
template <typename T, bool HAS_BIAS, int TOK, bool PARTS = false>
__global__ __launch_bounds__(kThreads) void rope_kv_write_table_kernel(
    T* __restrict__ qkv, const float* __restrict__ cos_sin, const int32_t* __restrict__ slots,
    const float* __restrict__ bias, T* __restrict__ k_pool, T* __restrict__ v_pool, int n_tokens, int n_heads,
    int n_kv, int head_dim, int page_size, int write_kv, int64_t pool_slots, const float* __restrict__ parts = nullptr,
    int n_parts = 0) {
    const int t0 = blockIdx.x * TOK;
    const int n_here = min(TOK, n_tokens - t0);
    const int half = head_dim / 2;
    const int q_dim = n_heads * head_dim;
    const int kv_dim = n_kv * head_dim;
    const int width = q_dim + 2 * kv_dim;
    int slot[TOK];
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
        slot[j] = (write_kv && j < n_here) ? slots[t0 + j] : -1;
        if (slot[j] >= pool_slots) slot[j] = -1;
    }
    // the blocks of a token (gridDim.y of them; more than one only where the partial sums make a token
    // heavy) share its columns
    const int first = threadIdx.x + blockIdx.y * kThreads;
    const int stride = kThreads * gridDim.y;
    // four consecutive columns of token t
    auto load4 = [&](int t, int col) -> float4 {
        if constexpr (PARTS) {
            const float* p = parts + static_cast<int64_t>(t) * width + col;
            const int64_t step = static_cast<int64_t>(n_tokens) * width;
            float4 acc = *reinterpret_cast<const float4*>(p);
#pragma unroll 4
            for (int s = 1; s < n_parts; ++s) {
                const float4 v = *reinterpret_cast<const float4*>(p + s * step);
                acc = float4{acc.x + v.x, acc.y + v.y, acc.z + v.z, acc.w + v.w};
            }
            return acc;
        } else {
            return Quad<T>::load(qkv + static_cast<int64_t>(t) * width + col);
        }
    };

    // ---- values
    bool run = !PARTS && TOK == 8 && n_here == 8 && slot[0] >= 0 && slot[0] % 8 == 0 && page_size % 8 == 0;
#pragma unroll
    for (int j = 1; j < TOK; ++j) run = run && slot[j] == slot[0] + j;
    if (TOK == 8 && run) {
        const int64_t page = slot[0] / page_size;
        const int off = slot[0] % page_size;
        for (int idx = first; idx < kv_dim; idx += stride) {  // lanes over the dimensions: rows read whole
            const int kvh = idx / head_dim;
            const int d = idx - kvh * head_dim;
            const float b = HAS_BIAS ? bias[q_dim + kv_dim + idx] : 0.f;
            float x[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                x[j] = to_float(qkv[static_cast<int64_t>(t0 + j) * width + q_dim + kv_dim + idx]) + b;
            T* dst = v_pool + ((page * n_kv + kvh) * head_dim + d) * page_size + off;
            Quad<T>::store(dst, float4{x[0], x[1], x[2], x[3]});
            Quad<T>::store(dst + 4, float4{x[4], x[5], x[6], x[7]});
        }
    } else {
#pragma unroll
        for (int j = 0; j < TOK; ++j) {
            if (slot[j] < 0) continue;
            const int64_t page = slot[j] / page_size;
            const int off = slot[j] % page_size;
            for (int idx = first * 4; idx < kv_dim; idx += stride * 4) {
                const int kvh = idx / head_dim;
                const int d = idx - kvh * head_dim;
                float4 x = load4(t0 + j, q_dim + kv_dim + idx);
                if (HAS_BIAS) {
                    const float4 b = *reinterpret_cast<const float4*>(bias + q_dim + kv_dim + idx);
                    x = float4{x.x + b.x, x.y + b.y, x.z + b.z, x.w + b.w};
                }
                T* dst = v_pool + ((page * n_kv + kvh) * head_dim + d) * page_size + off;
                dst[0] = from_float<T>(x.x);
                dst[page_size] = from_float<T>(x.y);
                dst[2 * page_size] = from_float<T>(x.z);
                dst[3 * page_size] = from_float<T>(x.w);
            }
        }
    }

    // ---- q and k heads: unit u of a token = four pairs of one head.  The block's (token, unit) pairs are
    // dealt to the threads of its gridDim.y blocks token by token, so that neighbouring threads take
    // neighbouring units of one token's row
    const int quads = half / 4;
    const int n_units = (n_heads + n_kv) * quads;
    for (int w = first; w < n_units * n_here; w += stride) {
        const int j = TOK == 1 ? 0 : w / n_units;
        const int u = TOK == 1 ? w : w - j * n_units;
        const int h = u / quads;
        const int i = (u - h * quads) * 4;
        float4 b1{0.f, 0.f, 0.f, 0.f}, b2{0.f, 0.f, 0.f, 0.f};
        if (HAS_BIAS) {
            b1 = *reinterpret_cast<const float4*>(bias + h * head_dim + i);
            b2 = *reinterpret_cast<const float4*>(bias + h * head_dim + i + half);
        }
        const int t = t0 + j;
        T* head = qkv + static_cast<int64_t>(t) * width + h * head_dim;
        float4 a1 = load4(t, h * head_dim + i), a2 = load4(t, h * head_dim + i + half);
        a1 = float4{a1.x + b1.x, a1.y + b1.y, a1.z + b1.z, a1.w + b1.w};
        a2 = float4{a2.x + b2.x, a2.y + b2.y, a2.z + b2.z, a2.w + b2.w};
        const float4* cs = reinterpret_cast<const float4*>(cos_sin + static_cast<int64_t>(t) * head_dim);
        const float4 c01 = cs[i / 2], c23 = cs[i / 2 + 1];  // (cos, sin) of pairs i, i + 1 and i + 2, i + 3
        const float4 r1{a1.x * c01.x - a2.x * c01.y, a1.y * c01.z - a2.y * c01.w, a1.z * c23.x - a2.z * c23.y,
                        a1.w * c23.z - a2.w * c23.w};
        const float4 r2{a2.x * c01.x + a1.x * c01.y, a2.y * c01.z + a1.y * c01.w, a2.z * c23.x + a1.z * c23.y,
                        a2.w * c23.z + a1.w * c23.w};
        if (!PARTS || h < n_heads) {
            Quad<T>::store(head + i, r1);
            Quad<T>::store(head + i + half, r2);
        }
        int sl = slot[0];
#pragma unroll
        for (int q = 1; q < TOK; ++q) sl = j == q ? slot[q] : sl;
        if (h >= n_heads && sl >= 0) {
            const int64_t page = sl / page_size;
            const int off = sl % page_size;
            T* dst = k_pool + ((page * n_kv + (h - n_heads)) * page_size + off) * head_dim;
            Quad<T>::store(dst + i, r1);
            Quad<T>::store(dst + i + half, r2);
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

// The rotation with cosines and sines from `cos_sin` ([n_tokens, head_dim / 2, 2] float32, made by
// fsie_rope_table): the whole head is rotated, head_dim a multiple of 8.
// parts (or null): float32 [n_parts][n_tokens][width], the projection as partial sums of a product cut
// along its inner dimension; qkv then only receives the rotated q heads (k and v go to the pools).
extern "C" int fsie_rope_kv_write_table(void* qkv, const float* cos_sin, const int32_t* slots, const float* bias,
                                        void* k_pool, void* v_pool, int n_tokens, int n_heads, int n_kv, int head_dim,
                                        int page_size, int64_t pool_slots, int dtype, const float* parts, int n_parts,
                                        hipStream_t stream) {
    FSIE_REQUIRE(!parts || (n_parts >= 1 && n_parts <= FSIE_GEMM_MAX_SPLITS && reinterpret_cast<uintptr_t>(parts) % 16 == 0),
                 "rope_kv_write_table: 1 to %d aligned partial sums, got %d", FSIE_GEMM_MAX_SPLITS, n_parts);
    FSIE_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0, "rope_kv_write_table: bad sizes");
    FSIE_REQUIRE(head_dim > 0 && head_dim % 8 == 0, "rope_kv_write_table: head_dim %d must be a multiple of 8", head_dim);
    FSIE_REQUIRE(cos_sin && reinterpret_cast<uintptr_t>(cos_sin) % 16 == 0, "rope_kv_write_table: no aligned table");
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && (!bias || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
                     (!k_pool || reinterpret_cast<uintptr_t>(k_pool) % 16 == 0),
                 "rope_kv_write_table: operands must be 16-byte aligned");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "rope_kv_write_table: unknown dtype %d", dtype);
    const int write_kv = (k_pool && v_pool && slots) ? 1 : 0;
    FSIE_REQUIRE(!write_kv || (page_size > 0 && pool_slots > 0), "rope_kv_write_table: bad page geometry");
    if (n_tokens == 0) return 0;
    // eight tokens a block where there are enough blocks left to fill the device, four blocks a run of eight
    // tokens: the kernel is made of loads that wait for memory, so it wants many waves on every unit
    // blocks a token: so many that the device's units all have one (64 tokens of 4,608 columns in 7 partial
    // sums on MI355X: 9.0 us with one block a token)
    const int units = fsie_compute_units();
    const int per_token = n_tokens > 0 && units > n_tokens ? (units / n_tokens > 8 ? 8 : units / n_tokens) : 1;
    const dim3 parts_grid(static_cast<unsigned>(n_tokens), static_cast<unsigned>(per_token));
#define FSIE_ROPE_PARTS(T, B)                                                                                     \
    rope_kv_write_table_kernel<T, B, 1, true><<<parts_grid, kThreads, 0, stream>>>(                               \
        static_cast<T*>(qkv), cos_sin, slots, bias, static_cast<T*>(k_pool), static_cast<T*>(v_pool), n_tokens,   \
        n_heads, n_kv, head_dim, page_size, write_kv, pool_slots, parts, n_parts)
    if (parts) {
        if (dtype == FSIE_F32) {
            if (bias) FSIE_ROPE_PARTS(float, true); else FSIE_ROPE_PARTS(float, false);
        } else {
            if (bias) FSIE_ROPE_PARTS(bf16_t, true); else FSIE_ROPE_PARTS(bf16_t, false);
        }
        FSIE_CHECK_LAUNCH("rope_kv_write_table");
        return 0;
    }
#undef FSIE_ROPE_PARTS
#define FSIE_ROPE_LAUNCH(T, B)                                                                                    \
    do {                                                                                                          \
        if (n_tokens >= 1024)                                                                                     \
            rope_kv_write_table_kernel<T, B, 8><<<dim3((n_tokens + 7) / 8, 4), kThreads, 0, stream>>>(            \
                static_cast<T*>(qkv), cos_sin, slots, bias, static_cast<T*>(k_pool), static_cast<T*>(v_pool),     \
                n_tokens, n_heads, n_kv, head_dim, page_size, write_kv, pool_slots);                              \
        else                                                                                                      \
            rope_kv_write_table_kernel<T, B, 1><<<n_tokens, kThreads, 0, stream>>>(                               \
                static_cast<T*>(qkv), cos_sin, slots, bias, static_cast<T*>(k_pool), static_cast<T*>(v_pool),     \
                n_tokens, n_heads, n_kv, head_dim, page_size, write_kv, pool_slots);                              \
    } while (0)
    if (dtype == FSIE_F32) {
        if (bias) FSIE_ROPE_LAUNCH(float, true); else FSIE_ROPE_LAUNCH(float, false);
    } else {
        if (bias) FSIE_ROPE_LAUNCH(bf16_t, true); else FSIE_ROPE_LAUNCH(bf16_t, false);
    }
#undef FSIE_ROPE_LAUNCH
    FSIE_CHECK_LAUNCH("rope_kv_write_table");
    return 0;
}
