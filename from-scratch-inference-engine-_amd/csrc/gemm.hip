// Y[M, N] = X[M, K] . W[N, K]^T (+ bias[N]) with float32 accumulation.
//
// Two kernels, both for float32 and bfloat16 storage:
//   * gemm_tiled   - LDS-tiled FMA kernel, any M/N/K.  It is the whole of the 32-bit path
//                    (true float32 products and sums) and the library-free fallback in bfloat16.
//   * gemm_skinny  - for a few rows (decode): every wave streams whole rows of W once with
//                    16-byte loads and reduces over the wave; bound by the read of W.
// A row's sum order depends on K only, never on how many other rows the call has.
#include "common.h"
#include "api.h"

namespace {

// ------------------------------------------------------------------------------ tiled
constexpr int TM = 64, TN = 64, TK = 16;

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                         const float* __restrict__ bias, OutT* __restrict__ y,
                                                         int M, int N, int K) {
    __shared__ float xs[TK][TM + 4];
    __shared__ float ws[TK][TN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    // two levels of float32 sums: runs of kFlush products are added up on their own and then
    // added to the total, so that the rounding error grows with sqrt(kFlush) + sqrt(K / kFlush)
    // instead of sqrt(K) (K reaches 18944 in a 7B model)
    constexpr int kFlush = 256;
    float acc[4][4], total[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = total[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += TK) {
        if (k0 > 0 && k0 % kFlush == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    total[i][j] += acc[i][j];
                    acc[i][j] = 0.f;
                }
        }
        // 64 rows x 16 k per operand: 1024 elements, 4 per thread; k is the fast index in memory
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * 256;
            const int r = idx / TK, kk = idx % TK;
            const int k = k0 + kk;
            const int m = m0 + r, n = n0 + r;
            xs[kk][r] = (m < M && k < K) ? to_float(x[static_cast<int64_t>(m) * K + k]) : 0.f;
            ws[kk][r] = (n < N && k < K) ? to_float(w[static_cast<int64_t>(n) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = total[i][j] + acc[i][j];
            if (bias) v += bias[n];
            y[static_cast<int64_t>(m) * N + n] = from_float<OutT>(v);
        }
    }
}

// ------------------------------------------------------------------------------ skinny
template <typename T>
struct Vec;  // 16 bytes of T
template <>
struct Vec<float> {
    static constexpr int N = 4;
    float4 raw;
    __device__ __forceinline__ float get(int i) const { return reinterpret_cast<const float*>(&raw)[i]; }
};
template <>
struct Vec<bf16_t> {
    static constexpr int N = 8;
    uint4 raw;
    __device__ __forceinline__ float get(int i) const {
        const uint32_t word = reinterpret_cast<const uint32_t*>(&raw)[i >> 1];
        return __uint_as_float((i & 1) ? (word & 0xffff0000u) : (word << 16));
    }
};

constexpr int kSkinnyWaves = 4;  // waves per block
constexpr int kSkinnyCols = 2;   // output columns per wave

// M <= MT rows.  VECTOR = 1: K is a multiple of the vector width and rows are 16-byte aligned.
template <typename T, typename OutT, int MT, int VECTOR>
__global__ __launch_bounds__(kSkinnyWaves* FSIE_WAVE) void gemm_skinny_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias, OutT* __restrict__ y,
    int M, int N, int K) {
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int n0 = (blockIdx.x * kSkinnyWaves + wave) * kSkinnyCols;
    if (n0 >= N) return;  // whole wave leaves together
    float acc[MT][kSkinnyCols];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < kSkinnyCols; ++c) acc[m][c] = 0.f;

    if (VECTOR) {
        constexpr int V = Vec<T>::N;
        for (int k = lane * V; k < K; k += FSIE_WAVE * V) {
            Vec<T> wv[kSkinnyCols];
#pragma unroll
            for (int c = 0; c < kSkinnyCols; ++c) {
                const int n = min(n0 + c, N - 1);  // a column past the end repeats the last one
                wv[c].raw = *reinterpret_cast<const decltype(wv[c].raw)*>(w + static_cast<int64_t>(n) * K + k);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    Vec<T> xv;
                    xv.raw = *reinterpret_cast<const decltype(xv.raw)*>(x + static_cast<int64_t>(m) * K + k);
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const float xi = xv.get(i);
#pragma unroll
                        for (int c = 0; c < kSkinnyCols; ++c) acc[m][c] = fmaf(xi, wv[c].get(i), acc[m][c]);
                    }
                }
            }
        }
    } else {
        for (int k = lane; k < K; k += FSIE_WAVE) {
            float wv[kSkinnyCols];
#pragma unroll
            for (int c = 0; c < kSkinnyCols; ++c) {
                const int n = min(n0 + c, N - 1);
                wv[c] = to_float(w[static_cast<int64_t>(n) * K + k]);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m < M) {
                    const float xi = to_float(x[static_cast<int64_t>(m) * K + k]);
#pragma unroll
                    for (int c = 0; c < kSkinnyCols; ++c) acc[m][c] = fmaf(xi, wv[c], acc[m][c]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int c = 0; c < kSkinnyCols; ++c) {
            const float v = wave_sum(acc[m][c]);
            const int n = n0 + c;
            if (lane == 0 && m < M && n < N) {
                y[static_cast<int64_t>(m) * N + n] = from_float<OutT>(bias ? v + bias[n] : v);
            }
        }
    }
}

template <typename T, typename OutT>
int launch_tiled(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, hipStream_t stream) {
    dim3 grid(static_cast<unsigned>(ceil_div64(N, TN)), static_cast<unsigned>(ceil_div64(M, TM)));
    gemm_tiled_kernel<T, OutT><<<grid, 256, 0, stream>>>(static_cast<const T*>(x), static_cast<const T*>(w), bias,
                                                         static_cast<OutT*>(y), M, N, K);
    FSIE_CHECK_LAUNCH("gemm_tiled");
    return 0;
}

template <typename T, typename OutT, int MT>
int launch_skinny_mt(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, hipStream_t stream) {
    const unsigned grid = static_cast<unsigned>(ceil_div64(N, kSkinnyWaves * kSkinnyCols));
    const bool aligned = (K % Vec<T>::N == 0) && (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(w) % 16 == 0);
    if (aligned) {
        gemm_skinny_kernel<T, OutT, MT, 1><<<grid, kSkinnyWaves * FSIE_WAVE, 0, stream>>>(
            static_cast<const T*>(x), static_cast<const T*>(w), bias, static_cast<OutT*>(y), M, N, K);
    } else {
        gemm_skinny_kernel<T, OutT, MT, 0><<<grid, kSkinnyWaves * FSIE_WAVE, 0, stream>>>(
            static_cast<const T*>(x), static_cast<const T*>(w), bias, static_cast<OutT*>(y), M, N, K);
    }
    FSIE_CHECK_LAUNCH("gemm_skinny");
    return 0;
}

template <typename T, typename OutT>
int launch_skinny(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, hipStream_t stream) {
    if (M <= 1) return launch_skinny_mt<T, OutT, 1>(x, w, bias, y, M, N, K, stream);
    if (M <= 2) return launch_skinny_mt<T, OutT, 2>(x, w, bias, y, M, N, K, stream);
    if (M <= 4) return launch_skinny_mt<T, OutT, 4>(x, w, bias, y, M, N, K, stream);
    return launch_skinny_mt<T, OutT, 8>(x, w, bias, y, M, N, K, stream);
}

}  // namespace

// kind: 0 = choose by M, 1 = tiled, 2 = skinny (M <= 8).  out_f32: write float32 whatever dtype.
extern "C" int fsie_gemm(const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                         int dtype, int out_f32, int kind, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gemm: unknown dtype %d", dtype);
    FSIE_REQUIRE(kind >= 0 && kind <= 2, "gemm: unknown kind %d", kind);
    FSIE_REQUIRE(!(kind == 2 && M > FSIE_GEMM_SKINNY_MAX_M), "gemm: skinny kernel takes at most %d rows, got %d",
                 FSIE_GEMM_SKINNY_MAX_M, M);
    if (M == 0) return 0;
    const bool skinny = kind == 2 || (kind == 0 && M <= FSIE_GEMM_SKINNY_MAX_M);
    if (dtype == FSIE_F32) {
        return skinny ? launch_skinny<float, float>(x, w, bias, y, M, N, K, stream)
                      : launch_tiled<float, float>(x, w, bias, y, M, N, K, stream);
    }
    if (out_f32) {
        return skinny ? launch_skinny<bf16_t, float>(x, w, bias, y, M, N, K, stream)
                      : launch_tiled<bf16_t, float>(x, w, bias, y, M, N, K, stream);
    }
    return skinny ? launch_skinny<bf16_t, bf16_t>(x, w, bias, y, M, N, K, stream)
                  : launch_tiled<bf16_t, bf16_t>(x, w, bias, y, M, N, K, stream);
}
