// Next-token choice on the device, one block per row of float32 logits.
//
//   temperature <= 0 : argmax, ties to the smallest index.
//   temperature  > 0 : temperature -> top-k -> top-p -> inverse CDF against a uniform number u
//                      that the host supplies per row.
// The kept set is the one a sort by logit would give (all tokens tied with the last kept one are
// kept); the draw walks the kept tokens in vocabulary order: first i with u * mass < cumulative.
// Thresholds are found by bisection over the order-preserving integer image of the float logits,
// each probe being one deterministic block reduction, so no sort and no atomics are needed.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / FSIE_WAVE;

__device__ __forceinline__ uint32_t order_key(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = FSIE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, FSIE_WAVE);
    return v;
}

__device__ double block_sum_f64(double v, double* scratch) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1), wave = threadIdx.x / FSIE_WAVE;
    v = wave_sum_f64(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    double total = 0.0;
    for (int w = 0; w < kWaves; ++w) total += scratch[w];
    return total;
}

struct Best {
    float value;
    int index;
};

__device__ __forceinline__ Best better(Best a, Best b) {
    if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
    return a;
}

__device__ Best block_argmax(const float* row, int vocab, float* sval, int* sidx) {
    Best best{-INFINITY, 0x7fffffff};
    auto take = [&](float v, int i) {
        if (best.index == 0x7fffffff || v > best.value) best = Best{v, i};  // strict: lowest index of a stripe wins
    };
    int done = 0;
    if (reinterpret_cast<uintptr_t>(row) % 16 == 0) {
        // 16-byte loads, four of them in flight per thread
        const int quads = vocab / 4;
        constexpr int U = 4;
        for (int q0 = threadIdx.x; q0 < quads; q0 += blockDim.x * U) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = min(q0 + u * static_cast<int>(blockDim.x), quads - 1);
                v[u] = *reinterpret_cast<const float4*>(row + 4 * q);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = q0 + u * blockDim.x;
                if (q < quads) {
                    take(v[u].x, 4 * q);
                    take(v[u].y, 4 * q + 1);
                    take(v[u].z, 4 * q + 2);
                    take(v[u].w, 4 * q + 3);
                }
            }
        }
        done = quads * 4;
    }
    for (int i = done + threadIdx.x; i < vocab; i += blockDim.x) take(row[i], i);
#pragma unroll
    for (int off = FSIE_WAVE / 2; off > 0; off >>= 1) {
        Best other{__shfl_xor(best.value, off, FSIE_WAVE), __shfl_xor(best.index, off, FSIE_WAVE)};
        best = better(best, other);
    }
    const int lane = threadIdx.x & (FSIE_WAVE - 1), wave = threadIdx.x / FSIE_WAVE;
    __syncthreads();
    if (lane == 0) {
        sval[wave] = best.value;
        sidx[wave] = best.index;
    }
    __syncthreads();
    Best total{sval[0], sidx[0]};
    for (int w = 1; w < kWaves; ++w) total = better(total, Best{sval[w], sidx[w]});
    return total;
}

// weight of token i under the row's temperature; mx is the row maximum
__device__ __forceinline__ double token_weight(float logit, float mx, float inv_temp) {
    return static_cast<double>(expf((logit - mx) * inv_temp));
}

__global__ __launch_bounds__(kThreads) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                          const float* __restrict__ temperature,
                                                          const int32_t* __restrict__ top_k,
                                                          const float* __restrict__ top_p,
                                                          const double* __restrict__ uniform,
                                                          int32_t* __restrict__ out) {
    __shared__ float sval[kWaves];
    __shared__ int sidx[kWaves];
    __shared__ double sdbl[kWaves];
    __shared__ double seg_prefix[kThreads + 1];
    __shared__ int chosen;

    const int r = blockIdx.x;
    const float* row = logits + static_cast<int64_t>(r) * vocab;
    const Best top = block_argmax(row, vocab, sval, sidx);
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[r] = top.index;
        return;
    }
    const float mx = top.value;
    const float inv_temp = 1.0f / temp;
    const uint32_t key_max = order_key(mx);
    uint32_t cut = 0;  // tokens with key >= cut are kept

    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < vocab) {
        // largest key t with count(key >= t) >= k
        uint32_t lo = 0, hi = key_max;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo) / 2 + ((hi - lo) & 1);
            double cnt = 0.0;
            for (int i = threadIdx.x; i < vocab; i += blockDim.x) cnt += order_key(row[i]) >= mid ? 1.0 : 0.0;
            cnt = block_sum_f64(cnt, sdbl);
            if (cnt >= static_cast<double>(k)) lo = mid; else hi = mid - 1;
        }
        cut = lo;
    }
    const float p = top_p ? top_p[r] : 1.f;
    if (p < 1.f) {
        double kept = 0.0;
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
            const float v = row[i];
            if (order_key(v) >= cut) kept += token_weight(v, mx, inv_temp);
        }
        kept = block_sum_f64(kept, sdbl);
        const double target = static_cast<double>(p) * kept;
        // largest key t >= cut with mass(key >= t) >= target
        uint32_t lo = cut, hi = key_max;
        while (lo < hi) {
            const uint32_t mid = lo + (hi - lo) / 2 + ((hi - lo) & 1);
            double mass = 0.0;
            for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
                const float v = row[i];
                if (order_key(v) >= mid) mass += token_weight(v, mx, inv_temp);
            }
            mass = block_sum_f64(mass, sdbl);
            if (mass >= target) lo = mid; else hi = mid - 1;
        }
        cut = lo;
    }

    // inverse CDF in vocabulary order: thread t owns the tokens [t*seg, (t+1)*seg)
    const int seg = (vocab + kThreads - 1) / kThreads;
    const int begin = min(threadIdx.x * seg, vocab), end = min(begin + seg, vocab);
    double mine = 0.0;
    for (int i = begin; i < end; ++i) {
        const float v = row[i];
        if (order_key(v) >= cut) mine += token_weight(v, mx, inv_temp);
    }
    seg_prefix[threadIdx.x + 1] = mine;
    if (threadIdx.x == 0) {
        seg_prefix[0] = 0.0;
        chosen = -1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int t = 1; t <= kThreads; ++t) seg_prefix[t] += seg_prefix[t - 1];
    }
    __syncthreads();
    const double threshold = uniform[r] * seg_prefix[kThreads];
    if (mine > 0.0 && seg_prefix[threadIdx.x] <= threshold && threshold < seg_prefix[threadIdx.x + 1]) {
        double cum = seg_prefix[threadIdx.x];
        int pick = -1, last_kept = -1;
        for (int i = begin; i < end; ++i) {
            const float v = row[i];
            if (order_key(v) < cut) continue;
            last_kept = i;
            cum += token_weight(v, mx, inv_temp);
            if (threshold < cum) {
                pick = i;
                break;
            }
        }
        chosen = pick >= 0 ? pick : last_kept;  // rounding at the segment's end
    }
    __syncthreads();
    if (threadIdx.x == 0) out[r] = chosen >= 0 ? chosen : top.index;
}

}  // namespace

extern "C" int fsie_sample(const float* logits, int n_rows, int vocab, const float* temperature,
                           const int32_t* top_k, const float* top_p, const double* uniform, int32_t* out,
                           hipStream_t stream) {
    FSIE_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", n_rows, vocab);
    FSIE_REQUIRE(!temperature || uniform, "sample: temperatures given without uniform numbers");
    if (n_rows == 0) return 0;
    sample_kernel<<<n_rows, kThreads, 0, stream>>>(logits, vocab, temperature, top_k, top_p, uniform, out);
    FSIE_CHECK_LAUNCH("sample");
    return 0;
}
