// Embedding gather, RMSNorm (alone, fused with the residual sum, or over chosen rows), SiLU*up
// and the plain residual sum.  The residual stream is float32 in both precisions; T is the
// type of activations and matrices (float or bfloat16).
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWideNormRows = 128;  // up to so many rows (half the device's units), RMSNorm runs in workgroups of 1,024 threads

// out[t, :] = table[ids[t], :] as float32.  An id outside the table gives a row of zeros; the
// host refuses such ids before the launch.
template <typename T>
__global__ void embedding_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                 float* __restrict__ out, int hidden, int vocab) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* dst = out + static_cast<int64_t>(t) * hidden;
    if (id < 0 || id >= vocab) {
        for (int j = threadIdx.x; j < hidden; j += blockDim.x) dst[j] = 0.f;
        return;
    }
    const T* src = table + static_cast<int64_t>(id) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) dst[j] = to_float(src[j]);
}

// One block per output row r; source row = rows ? rows[r] : r.
//   v = residual[row] (+ delta[row]);  if write_back: residual[row] = v
//   out[r] = (v * rsqrt(mean(v^2) + eps)) * weight
// Sum of squares, scale and the residual sum are float32.  With n_parts > 0 the delta is the sum,
// taken in order, of n_parts float32 arrays [total_rows, hidden] that lie one after the other
// (partial sums of a matrix product whose inner dimension was cut).
template <typename T>
__global__ void rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                               const float* __restrict__ weight, T* __restrict__ out,
                               const int32_t* __restrict__ rows, int hidden, float eps,
                               int write_back, int n_parts, int64_t part_stride) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const T* del = (delta && !n_parts) ? delta + row * hidden : nullptr;
    const float* parts = n_parts ? reinterpret_cast<const float*>(delta) + row * hidden : nullptr;
    auto delta_at = [&](int j) {
        if (del) return to_float(del[j]);
        float d = 0.f;
        for (int s = 0; s < n_parts; ++s) d += parts[s * part_stride + j];
        return d;
    };
    const bool has_delta = del || parts;
    float sum_sq = 0.f;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = res[j];
        if (has_delta) v += delta_at(j);
        if (write_back) res[j] = v;
        sum_sq += v * v;
    }
    const float total = block_sum(sum_sq, scratch);
    const float scale = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    T* dst = out + static_cast<int64_t>(r) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) {
        float v = res[j];
        if (has_delta && !write_back) v += delta_at(j);
        dst[j] = from_float<T>((v * scale) * weight[j]);
    }
}

// The same for hidden % 4 == 0 and hidden <= 1024 * ITERS: the row stays in registers between
// the two passes and moves with 16-byte (float32) and 8- or 16-byte (T) accesses.
template <typename T>
struct Pack4;
template <>
struct Pack4<float> {
    static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <>
struct Pack4<bf16_t> {
    static __device__ __forceinline__ float4 load(const bf16_t* p) {
        const uint2 w = *reinterpret_cast<const uint2*>(p);
        return float4{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                      __uint_as_float(w.y & 0xffff0000u)};
    }
    static __device__ __forceinline__ void store(bf16_t* p, float4 v) {
        uint2 w;
        w.x = static_cast<uint32_t>(float_to_bf16_bits(v.x)) | (static_cast<uint32_t>(float_to_bf16_bits(v.y)) << 16);
        w.y = static_cast<uint32_t>(float_to_bf16_bits(v.z)) | (static_cast<uint32_t>(float_to_bf16_bits(v.w)) << 16);
        *reinterpret_cast<uint2*>(p) = w;
    }
};

// four elements per thread, grid = (tokens, quads / threads): no loop, one load per thread
template <typename T>
__global__ void embedding_vec_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids,
                                     float* __restrict__ out, int hidden, int vocab) {
    const int t = blockIdx.x;
    const int j = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (j >= hidden) return;
    const int id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    const float4 v = Pack4<T>::load(table + static_cast<int64_t>(ok ? id : 0) * hidden + j);
    Pack4<float>::store(out + static_cast<int64_t>(t) * hidden + j, ok ? v : float4{0.f, 0.f, 0.f, 0.f});
}

// DELTA: 0 = none, 1 = one array of T, 2 to 9 = that many float32 partial sums, added in
// order (every load of the row goes out before anything waits); -1 = `n_parts` of them (any other
// number: a loop, four loads ahead).
template <typename T, int ITERS, int DELTA, bool WRITE_BACK, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_vec_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                                               const float* __restrict__ weight, T* __restrict__ out,
                                                               const int32_t* __restrict__ rows, int hidden, float eps,
                                                               int64_t part_stride, int n_parts) {
    __shared__ float scratch[16];
    constexpr bool HAS_DELTA = DELTA != 0;
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const T* del = DELTA == 1 ? delta + row * hidden : nullptr;
    const float* parts = (DELTA > 1 || DELTA < 0) ? reinterpret_cast<const float*>(delta) + row * hidden : nullptr;
    // every load of the row goes out before anything waits: places past the end read the last
    // quad again and are masked out of the sum and the stores
    float4 v[ITERS], d[ITERS], w[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = min((it * THREADS + static_cast<int>(threadIdx.x)) * 4, hidden - 4);
        v[it] = Pack4<float>::load(res + j);
        if (DELTA == 1) d[it] = Pack4<T>::load(del + j);
        if (DELTA > 1) {
            float4 p[DELTA > 1 ? DELTA : 1];
#pragma unroll
            for (int s = 0; s < DELTA; ++s) p[s] = Pack4<float>::load(parts + s * part_stride + j);
            d[it] = p[0];
#pragma unroll
            for (int s = 1; s < DELTA; ++s) {
                d[it].x += p[s].x;
                d[it].y += p[s].y;
                d[it].z += p[s].z;
                d[it].w += p[s].w;
            }
        }
        if (DELTA < 0) {
            float4 a = Pack4<float>::load(parts + j);
#pragma unroll 4
            for (int s = 1; s < n_parts; ++s) {
                const float4 p = Pack4<float>::load(parts + s * part_stride + j);
                a.x += p.x;
                a.y += p.y;
                a.z += p.z;
                a.w += p.w;
            }
            d[it] = a;
        }
        w[it] = Pack4<float>::load(weight + j);
    }
    float sum_sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (it * THREADS + threadIdx.x) * 4;
        if (HAS_DELTA) {
            v[it].x += d[it].x;
            v[it].y += d[it].y;
            v[it].z += d[it].z;
            v[it].w += d[it].w;
        }
        if (j < hidden) {
            if (WRITE_BACK) Pack4<float>::store(res + j, v[it]);
            sum_sq += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
        }
    }
    const float total = block_sum(sum_sq, scratch);
    const float scale = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    T* dst = out + static_cast<int64_t>(r) * hidden;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (it * THREADS + threadIdx.x) * 4;
        if (j < hidden) {
            Pack4<T>::store(dst + j, float4{(v[it].x * scale) * w[it].x, (v[it].y * scale) * w[it].y,
                                            (v[it].z * scale) * w[it].z, (v[it].w * scale) * w[it].w});
        }
    }
}

struct NormCall {
    float* residual;
    const void* delta;
    const float* weight;
    void* out;
    const int32_t* rows;
    int n_rows, hidden;
    float eps;
    int write_back;
    int n_parts;          // 0: delta (if any) is one array of the output's type
    int64_t part_stride;  // elements between the partial sums
    hipStream_t stream;
};

template <typename T, int ITERS, int DELTA, int THREADS>
void launch_rmsnorm_delta(const NormCall& c) {
    const T* d = static_cast<const T*>(c.delta);
    T* o = static_cast<T*>(c.out);
    if (c.write_back) {
        rmsnorm_vec_kernel<T, ITERS, DELTA, DELTA != 0, THREADS><<<c.n_rows, THREADS, 0, c.stream>>>(
            c.residual, d, c.weight, o, c.rows, c.hidden, c.eps, c.part_stride, c.n_parts);
    } else {
        rmsnorm_vec_kernel<T, ITERS, DELTA, false, THREADS><<<c.n_rows, THREADS, 0, c.stream>>>(
            c.residual, d, c.weight, o, c.rows, c.hidden, c.eps, c.part_stride, c.n_parts);
    }
}

template <typename T, int ITERS, int THREADS = kThreads>
void launch_rmsnorm_vec(const NormCall& c) {
    if (!c.delta) return launch_rmsnorm_delta<T, ITERS, 0, THREADS>(c);
    switch (c.n_parts) {
        case 0: return launch_rmsnorm_delta<T, ITERS, 1, THREADS>(c);
        case 2: return launch_rmsnorm_delta<T, ITERS, 2, THREADS>(c);
        case 3: return launch_rmsnorm_delta<T, ITERS, 3, THREADS>(c);
        case 4: return launch_rmsnorm_delta<T, ITERS, 4, THREADS>(c);
        case 5: return launch_rmsnorm_delta<T, ITERS, 5, THREADS>(c);
        case 6: return launch_rmsnorm_delta<T, ITERS, 6, THREADS>(c);
        case 7: return launch_rmsnorm_delta<T, ITERS, 7, THREADS>(c);
        case 8: return launch_rmsnorm_delta<T, ITERS, 8, THREADS>(c);
        case 9: return launch_rmsnorm_delta<T, ITERS, 9, THREADS>(c);
        default: return launch_rmsnorm_delta<T, ITERS, -1, THREADS>(c);
    }
}

template <typename T>
void launch_rmsnorm(const NormCall& c) {
    const bool aligned = c.hidden % 4 == 0 && reinterpret_cast<uintptr_t>(c.residual) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(c.weight) % 16 == 0 && reinterpret_cast<uintptr_t>(c.delta) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(c.out) % 16 == 0 && c.part_stride % 4 == 0;
    // a thread holds `iters` quads of the row: as many as the row needs, so that a row of 5,120
    // values asks for five quads a thread and not for eight of which three repeat the last one
    const int per_iter = kThreads * 4;
    const int iters = (c.hidden + per_iter - 1) / per_iter;
    // Decoding (up to 128 rows): a row and its partial sums (nine of them at hidden 3584 are 129 KB) come
    // through one compute unit, which draws the more the more waves ask (some 50 GB/s with four waves,
    // 125 with sixteen): workgroups of 1,024 threads, one or two quads a thread.
    if (aligned && c.n_rows <= kWideNormRows && c.hidden >= 2048 && c.hidden <= 8192) {
        if (c.hidden <= 4096) launch_rmsnorm_vec<T, 1, 1024>(c);
        else launch_rmsnorm_vec<T, 2, 1024>(c);
        return;
    }
    if (aligned && c.hidden >= 4 && iters <= 8) {
        switch (iters) {
            case 1: launch_rmsnorm_vec<T, 1>(c); break;
            case 2: launch_rmsnorm_vec<T, 2>(c); break;
            case 3: launch_rmsnorm_vec<T, 3>(c); break;
            case 4: launch_rmsnorm_vec<T, 4>(c); break;
            case 5: launch_rmsnorm_vec<T, 5>(c); break;
            case 6: launch_rmsnorm_vec<T, 6>(c); break;
            case 7: launch_rmsnorm_vec<T, 7>(c); break;
            default: launch_rmsnorm_vec<T, 8>(c); break;
        }
    } else {
        rmsnorm_kernel<T><<<c.n_rows, kThreads, 0, c.stream>>>(c.residual, static_cast<const T*>(c.delta), c.weight,
                                                             static_cast<T*>(c.out), c.rows, c.hidden, c.eps,
                                                             c.write_back, c.n_parts, c.part_stride);
    }
}

// out[t, j] = silu(x[t, 2j]) * x[t, 2j + 1]; x is [T, 2*inter] with gate and up interleaved.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t total, int inter) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const float g = to_float(x[2 * i]);
    const float u = to_float(x[2 * i + 1]);
    out[i] = from_float<T>((g / (1.0f + expf(-g))) * u);
}

// four outputs per thread: 8 inputs in 16 (bfloat16) or 32 (float32) bytes
template <typename T>
__global__ void swiglu_vec_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t quads) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= quads) return;
    const float4 a = Pack4<T>::load(x + 8 * i), b = Pack4<T>::load(x + 8 * i + 4);
    Pack4<T>::store(out + 4 * i, float4{(a.x / (1.0f + expf(-a.x))) * a.y, (a.z / (1.0f + expf(-a.z))) * a.w,
                                        (b.x / (1.0f + expf(-b.x))) * b.y, (b.z / (1.0f + expf(-b.z))) * b.w});
}

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ residual, const T* __restrict__ delta, int64_t total) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) residual[i] += to_float(delta[i]);
}

template <typename T>
__global__ void bias_add_kernel(T* __restrict__ y, const float* __restrict__ bias, int64_t total, int cols) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) y[i] = from_float<T>(to_float(y[i]) + bias[i % cols]);
}

// Rows of a table set to zero: row slots[i] of [n_slots, row_bytes / 4] words, negative = none.
__global__ void zero_rows_kernel(uint32_t* __restrict__ table, const int32_t* __restrict__ slots, int64_t row_words,
                                 int n_slots) {
    const int slot = slots[blockIdx.x];
    if (slot < 0 || slot >= n_slots) return;
    uint32_t* row = table + static_cast<int64_t>(slot) * row_words;
    for (int64_t i = static_cast<int64_t>(blockIdx.y) * blockDim.x + threadIdx.x; i < row_words;
         i += static_cast<int64_t>(gridDim.y) * blockDim.x)
        row[i] = 0u;
}

// Pages pages[i] (negative = none) of two pools set to zero in every plane: the pools are
// [planes][n_pages][page_words] words each.
template <typename V>
__global__ void zero_pages_kernel(uint32_t* __restrict__ a, uint32_t* __restrict__ b, const int32_t* __restrict__ pages,
                                  int64_t page_words, int64_t plane_words, int n_pages) {
    const int page = pages[blockIdx.x];
    if (page < 0 || page >= n_pages) return;
    uint32_t* pool = (blockIdx.z & 1) ? b : a;
    V* dst = reinterpret_cast<V*>(pool + (blockIdx.z >> 1) * plane_words + static_cast<int64_t>(page) * page_words);
    const int64_t n = page_words / static_cast<int64_t>(sizeof(V) / 4);
    V zero;
    memset(&zero, 0, sizeof(V));
    for (int64_t i = static_cast<int64_t>(blockIdx.y) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.y) * blockDim.x)
        dst[i] = zero;
}

// Counter-based random values, a pure function of (key, element index): see fsie_random_fill.
__device__ __forceinline__ uint64_t splitmix_output(uint64_t key, uint64_t number) {
    uint64_t x = key + (number + 1) * 0x9E3779B97F4A7C15ull;
    uint64_t z = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void random_fill_kernel(void* __restrict__ out, int64_t n, uint64_t key, int kind, float std) {
#pragma clang fp contract(off)  // a product and a sum stay two roundings, as on the host
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const uint64_t a = splitmix_output(key, 2 * static_cast<uint64_t>(i));
        if (kind == 2) {
            static_cast<int32_t*>(out)[i] = static_cast<int32_t>((a >> 17) & 0x7FFF);
            continue;
        }
        const uint64_t b = splitmix_output(key, 2 * static_cast<uint64_t>(i) + 1);
        int total = 0;
#pragma unroll
        for (int shift = 0; shift < 64; shift += 16)
            total += static_cast<int>((a >> shift) & 0xFFFF) + static_cast<int>((b >> shift) & 0xFFFF);
        // single float32 operations, written out here so that the pragma above covers them (the
        // library's rounding-mode wrappers are compiled where contraction is allowed): the host
        // computes the same bits
        const float z = static_cast<float>(total - 4 * 65535) * __uint_as_float(0x379cc471u);
        const float v = z * std;
        const float shifted = v + 1.0f;
        static_cast<float*>(out)[i] = kind == 1 ? shifted : v;
    }
}

// RMSNorm of a plain tensor, no residual stream: every row of x holds `groups` runs of `width`
// values, each normalised by itself (a whole row, or the heads of a row); one wave a run.
template <typename T>
__global__ void rmsnorm_plain_kernel(const T* __restrict__ x, int64_t x_stride, const float* __restrict__ weight,
                                     T* __restrict__ out, int64_t out_stride, int64_t n_runs, int groups, int width,
                                     float eps) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int64_t run = static_cast<int64_t>(blockIdx.x) * (blockDim.x / FSIE_WAVE) + threadIdx.x / FSIE_WAVE;
    if (run >= n_runs) return;
    const int64_t row = run / groups;
    const int g = static_cast<int>(run % groups);
    const T* src = x + row * x_stride + static_cast<int64_t>(g) * width;
    T* dst = out + row * out_stride + static_cast<int64_t>(g) * width;
    float sum = 0.f;
    for (int i = lane; i < width; i += FSIE_WAVE) {
        const float v = to_float(src[i]);
        sum += v * v;
    }
    sum = wave_sum(sum);
    const float r = 1.0f / sqrtf(sum / static_cast<float>(width) + eps);
    for (int i = lane; i < width; i += FSIE_WAVE) dst[i] = from_float<T>(to_float(src[i]) * r * weight[i]);
}

}  // namespace

extern "C" int fsie_zero_rows(void* table, const int32_t* slots, int n, int64_t row_bytes, int n_slots,
                              hipStream_t stream) {
    FSIE_REQUIRE(n >= 0 && n_slots >= 0 && row_bytes >= 0 && row_bytes % 4 == 0,
                 "zero_rows: bad sizes n=%d slots=%d row_bytes=%lld", n, n_slots, static_cast<long long>(row_bytes));
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(table) % 4 == 0, "zero_rows: the table must be 4-byte aligned");
    if (n == 0 || row_bytes == 0) return 0;
    const int64_t words = row_bytes / 4;
    const dim3 grid(n, static_cast<unsigned>(ceil_div64(words, 4 * kThreads) > 64 ? 64 : ceil_div64(words, 4 * kThreads)));
    zero_rows_kernel<<<grid, kThreads, 0, stream>>>(static_cast<uint32_t*>(table), slots, words, n_slots);
    FSIE_CHECK_LAUNCH("zero_rows");
    return 0;
}

// out[i] for i in [0, n): kind 0: std * z_i, kind 1: 1 + std * z_i (float32), kind 2: 15 random bits
// (int32), where z_i is the centred, scaled sum of the eight 16-bit fields of the SplitMix64 outputs
// number 2i and 2i + 1 of the sequence that starts at `key` (close to a standard normal).
extern "C" int fsie_random_fill(void* out, int64_t n, uint64_t key, int kind, float std, hipStream_t stream) {
    FSIE_REQUIRE(n >= 0 && kind >= 0 && kind <= 2, "random_fill: bad arguments n=%lld kind=%d", static_cast<long long>(n), kind);
    if (n == 0) return 0;
    const int64_t blocks = ceil_div64(n, kThreads);
    random_fill_kernel<<<static_cast<unsigned>(blocks > 65536 ? 65536 : blocks), kThreads, 0, stream>>>(out, n, key, kind, std);
    FSIE_CHECK_LAUNCH("random_fill");
    return 0;
}

extern "C" int fsie_zero_pages(void* pool_a, void* pool_b, const int32_t* pages, int n, int planes, int n_pages,
                               int64_t page_bytes, hipStream_t stream) {
    FSIE_REQUIRE(n >= 0 && planes > 0 && n_pages > 0 && page_bytes > 0 && page_bytes % 4 == 0,
                 "zero_pages: bad sizes n=%d planes=%d pages=%d page_bytes=%lld (pages are whole 4-byte words)", n,
                 planes, n_pages, static_cast<long long>(page_bytes));
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(pool_a) % 16 == 0 && reinterpret_cast<uintptr_t>(pool_b) % 16 == 0,
                 "zero_pages: the pools must be 16-byte aligned");
    if (n == 0) return 0;
    const int64_t page_words = page_bytes / 4;
    const bool quads = page_bytes % 16 == 0;
    const int64_t chunks = ceil_div64(quads ? page_words / 4 : page_words, kThreads);
    const dim3 grid(n, static_cast<unsigned>(chunks > 16 ? 16 : chunks), 2 * planes);
    if (quads) {
        zero_pages_kernel<uint4><<<grid, kThreads, 0, stream>>>(static_cast<uint32_t*>(pool_a), static_cast<uint32_t*>(pool_b),
                                                               pages, page_words, page_words * n_pages, n_pages);
    } else {
        zero_pages_kernel<uint32_t><<<grid, kThreads, 0, stream>>>(static_cast<uint32_t*>(pool_a),
                                                                  static_cast<uint32_t*>(pool_b), pages, page_words,
                                                                  page_words * n_pages, n_pages);
    }
    FSIE_CHECK_LAUNCH("zero_pages");
    return 0;
}

extern "C" int fsie_rmsnorm_plain(const void* x, int64_t x_stride, const float* weight, void* out, int64_t out_stride,
                                  int n_rows, int groups, int width, float eps, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_rows >= 0 && groups > 0 && width > 0, "rmsnorm_plain: bad sizes rows=%d groups=%d width=%d", n_rows,
                 groups, width);
    FSIE_REQUIRE(x_stride >= static_cast<int64_t>(groups) * width && out_stride >= static_cast<int64_t>(groups) * width,
                 "rmsnorm_plain: a row is shorter than its %d runs of %d", groups, width);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "rmsnorm_plain: unknown dtype %d", dtype);
    const int64_t runs = static_cast<int64_t>(n_rows) * groups;
    if (runs == 0) return 0;
    const int per_block = kThreads / FSIE_WAVE;
    const unsigned grid = static_cast<unsigned>(ceil_div64(runs, per_block));
    if (dtype == FSIE_F32) {
        rmsnorm_plain_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<const float*>(x), x_stride, weight,
                                                                   static_cast<float*>(out), out_stride, runs, groups,
                                                                   width, eps);
    } else {
        rmsnorm_plain_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), x_stride, weight,
                                                                    static_cast<bf16_t*>(out), out_stride, runs, groups,
                                                                    width, eps);
    }
    FSIE_CHECK_LAUNCH("rmsnorm_plain");
    return 0;
}

extern "C" int fsie_embedding(const void* table, int dtype, const int32_t* ids, float* out,
                              int n_tokens, int hidden, int vocab, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes T=%d H=%d V=%d",
                 n_tokens, hidden, vocab);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "embedding: unknown dtype %d", dtype);
    if (n_tokens == 0) return 0;
    const bool vec = hidden % 4 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    const dim3 vgrid(n_tokens, static_cast<unsigned>(ceil_div64(hidden / 4, kThreads)));
    if (dtype == FSIE_F32) {
        if (vec) embedding_vec_kernel<float><<<vgrid, kThreads, 0, stream>>>(static_cast<const float*>(table), ids, out, hidden, vocab);
        else embedding_kernel<float><<<n_tokens, kThreads, 0, stream>>>(static_cast<const float*>(table), ids, out, hidden, vocab);
    } else {
        if (vec) embedding_vec_kernel<bf16_t><<<vgrid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(table), ids, out, hidden, vocab);
        else embedding_kernel<bf16_t><<<n_tokens, kThreads, 0, stream>>>(static_cast<const bf16_t*>(table), ids, out, hidden, vocab);
    }
    FSIE_CHECK_LAUNCH("embedding");
    return 0;
}

// n_parts > 0: delta is n_parts float32 arrays [total_rows, hidden], one after the other, whose sum
// (taken in order) is the delta; total_rows is the number of rows of the residual.
extern "C" int fsie_rmsnorm(float* residual, const void* delta, const float* weight, void* out,
                            const int32_t* rows, int n_rows, int hidden, float eps, int dtype,
                            int write_back, int n_parts, int total_rows, hipStream_t stream) {
    FSIE_REQUIRE(n_parts >= 0 && n_parts <= FSIE_GEMM_MAX_SPLITS && n_parts != 1,
                 "rmsnorm: the delta comes whole or in 2..%d parts, not %d", FSIE_GEMM_MAX_SPLITS, n_parts);
    FSIE_REQUIRE(n_parts == 0 || (delta && total_rows > 0), "rmsnorm: parts without a delta or a row count");
    FSIE_REQUIRE(n_rows >= 0 && hidden > 0, "rmsnorm: bad sizes rows=%d H=%d", n_rows, hidden);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "rmsnorm: unknown dtype %d", dtype);
    FSIE_REQUIRE(!(write_back && rows), "rmsnorm: write_back cannot be combined with a row list");
    FSIE_REQUIRE(!(write_back && !delta), "rmsnorm: write_back without a delta");
    if (n_rows == 0) return 0;
    const NormCall call{residual, delta, weight, out, rows, n_rows, hidden, eps, write_back, n_parts,
                        static_cast<int64_t>(total_rows) * hidden, stream};
    if (dtype == FSIE_F32) {
        launch_rmsnorm<float>(call);
    } else {
        launch_rmsnorm<bf16_t>(call);
    }
    FSIE_CHECK_LAUNCH("rmsnorm");
    return 0;
}

extern "C" int fsie_swiglu(const void* x, void* out, int n_tokens, int inter, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", n_tokens, inter);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "swiglu: unknown dtype %d", dtype);
    const int64_t total = static_cast<int64_t>(n_tokens) * inter;
    if (total == 0) return 0;
    const bool vec = total % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    const int64_t work = vec ? total / 4 : total;
    const unsigned grid = static_cast<unsigned>(ceil_div64(work, kThreads));
    if (dtype == FSIE_F32) {
        if (vec) swiglu_vec_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<const float*>(x), static_cast<float*>(out), work);
        else swiglu_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<const float*>(x), static_cast<float*>(out), total, inter);
    } else {
        if (vec) swiglu_vec_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<bf16_t*>(out), work);
        else swiglu_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), static_cast<bf16_t*>(out), total, inter);
    }
    FSIE_CHECK_LAUNCH("swiglu");
    return 0;
}

extern "C" int fsie_residual_add(float* residual, const void* delta, int64_t total, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(total >= 0, "residual_add: negative size");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "residual_add: unknown dtype %d", dtype);
    if (total == 0) return 0;
    const unsigned grid = static_cast<unsigned>(ceil_div64(total, kThreads));
    if (dtype == FSIE_F32) {
        residual_add_kernel<float><<<grid, kThreads, 0, stream>>>(residual, static_cast<const float*>(delta), total);
    } else {
        residual_add_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(residual, static_cast<const bf16_t*>(delta), total);
    }
    FSIE_CHECK_LAUNCH("residual_add");
    return 0;
}

extern "C" int fsie_bias_add(void* y, const float* bias, int rows, int cols, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(rows >= 0 && cols > 0, "bias_add: bad sizes %d x %d", rows, cols);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "bias_add: unknown dtype %d", dtype);
    const int64_t total = static_cast<int64_t>(rows) * cols;
    if (total == 0) return 0;
    const unsigned grid = static_cast<unsigned>(ceil_div64(total, kThreads));
    if (dtype == FSIE_F32) {
        bias_add_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<float*>(y), bias, total, cols);
    } else {
        bias_add_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<bf16_t*>(y), bias, total, cols);
    }
    FSIE_CHECK_LAUNCH("bias_add");
    return 0;
}
