// Y[M, N] = X[M, K] . W[N, K]^T (+ bias) for bfloat16 operands and few rows (decode: M <= 64),
// on the matrix cores.  The product is computed transposed, D[n, m] = sum_k W[n, k] X[m, k], so
// that the big operand W streams from HBM straight into the A registers of
// v_mfma_f32_16x16x32_bf16 (16 bytes of one row per lane, no conversion, no LDS) and the small
// operand X comes from cache.  The kernel is bound by the read of W.
//
// One workgroup owns 16 rows of W (16 output columns); its waves split K in steps of 32,
// interleaved, and the partial tiles are summed through LDS in the fixed order of the waves, so
// the result does not depend on the batch or on timing.
#include "common.h"
#include "api.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

union Frag {
    uint4 raw;
    bf16x8 v;
};

constexpr int kStep = 32;  // k per MFMA

template <int MT, int WAVES, typename OutT>
__global__ __launch_bounds__(WAVES * FSIE_WAVE) void gemm_mfma_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    OutT* __restrict__ y, int M, int N, int K) {
    __shared__ float red[WAVES > 1 ? (WAVES - 1) * MT * FSIE_WAVE * 4 : 1];
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int row = lane & 15;  // row of the A tile (n) and column of the B tile (m)
    const int kg = lane >> 4;   // which 8 of the 32 k values this lane holds
    const int n0 = blockIdx.x * 16;
    const int n = min(n0 + row, N - 1);
    const bf16_t* wp = w + static_cast<int64_t>(n) * K + kg * 8;
    const bf16_t* xp[MT];
    bool x_ok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + row;
        x_ok[t] = m < M;
        xp[t] = x + static_cast<int64_t>(x_ok[t] ? m : 0) * K + kg * 8;
    }
    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int n_steps = (K + kStep - 1) / kStep;
    constexpr int U = 4;  // steps in flight per wave
    for (int s0 = wave; s0 < n_steps; s0 += WAVES * U) {
        Frag a[U], b[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = (s0 + u * WAVES) * kStep;
            const bool ok = k0 + kg * 8 < K;  // K is a multiple of 8: a lane's 8 values are all in or all out
            a[u].raw = ok ? *reinterpret_cast<const uint4*>(wp + k0) : uint4{0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                b[u][t].raw = (ok && x_ok[t]) ? *reinterpret_cast<const uint4*>(xp[t] + k0) : uint4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u].v, b[u][t].v, acc[t], 0, 0, 0);
            }
        }
    }

    if (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) red[(((wave - 1) * MT + t) * 4 + r) * FSIE_WAVE + lane] = acc[t][r];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int wv = 0; wv < WAVES - 1; ++wv)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] += red[((wv * MT + t) * 4 + r) * FSIE_WAVE + lane];
    }
    // lane holds D[n0 + 4*kg + r][m = 16*t + row]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + row;
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int nn = n0 + kg * 4 + r;
            if (nn < N) {
                const float v = bias ? acc[t][r] + bias[nn] : acc[t][r];
                y[static_cast<int64_t>(m) * N + nn] = from_float<OutT>(v);
            }
        }
    }
}

template <int MT, int WAVES, typename OutT>
int launch(const void* x, const void* w, const float* bias, void* y, int M, int N, int K, hipStream_t stream) {
    const unsigned grid = static_cast<unsigned>((N + 15) / 16);
    gemm_mfma_skinny_kernel<MT, WAVES, OutT><<<grid, WAVES * FSIE_WAVE, 0, stream>>>(
        static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), bias, static_cast<OutT*>(y), M, N, K);
    FSIE_CHECK_LAUNCH("gemm_mfma_skinny");
    return 0;
}

template <int MT, typename OutT>
int launch_waves(int waves, const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                 hipStream_t stream) {
    switch (waves) {
        case 1: return launch<MT, 1, OutT>(x, w, bias, y, M, N, K, stream);
        case 2: return launch<MT, 2, OutT>(x, w, bias, y, M, N, K, stream);
        case 4: return launch<MT, 4, OutT>(x, w, bias, y, M, N, K, stream);
        case 8: return launch<MT, 8, OutT>(x, w, bias, y, M, N, K, stream);
        default: return launch<MT, 16, OutT>(x, w, bias, y, M, N, K, stream);
    }
}

template <typename OutT>
int launch_tiles(int mt, int waves, const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                 hipStream_t stream) {
    switch (mt) {
        case 1: return launch_waves<1, OutT>(waves, x, w, bias, y, M, N, K, stream);
        case 2: return launch_waves<2, OutT>(waves, x, w, bias, y, M, N, K, stream);
        case 3: return launch_waves<3, OutT>(waves, x, w, bias, y, M, N, K, stream);
        default: return launch_waves<4, OutT>(waves, x, w, bias, y, M, N, K, stream);
    }
}

}  // namespace

// bfloat16 only.  M <= 64, K a multiple of 8, x and w 16-byte aligned.  waves: 0 = choose.
extern "C" int fsie_gemm_mfma_skinny(const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                                     int out_f32, int waves, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(M <= FSIE_GEMM_MFMA_SKINNY_MAX_M, "gemm_mfma_skinny: at most %d rows, got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    FSIE_REQUIRE(K % 8 == 0, "gemm_mfma_skinny: K=%d must be a multiple of 8", K);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_skinny: operands must be 16-byte aligned");
    FSIE_REQUIRE(waves == 0 || waves == 1 || waves == 2 || waves == 4 || waves == 8 || waves == 16,
                 "gemm_mfma_skinny: waves must be 0, 1, 2, 4, 8 or 16");
    if (M == 0) return 0;
    const int mt = (M + 15) / 16;
    if (waves == 0) {
        // enough waves to keep 256 compute units busy with loads in flight, but at least two
        // k steps of work per wave
        const int blocks = (N + 15) / 16;
        const int steps = (K + kStep - 1) / kStep;
        waves = 1;
        while (waves < 16 && blocks * waves < 4096 && steps / (waves * 2) >= 2) waves *= 2;
        if (mt >= 3 && waves > 8) waves = 8;  // LDS of the reduction
    }
    return out_f32 ? launch_tiles<float>(mt, waves, x, w, bias, y, M, N, K, stream)
                   : launch_tiles<bf16_t>(mt, waves, x, w, bias, y, M, N, K, stream);
}
