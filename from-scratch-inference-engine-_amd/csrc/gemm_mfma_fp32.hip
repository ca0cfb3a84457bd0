// Y[M, N] = X[M, K] . W[N, K]^T (+ bias) in true float32 on the matrix cores, for up to 64 rows
// (the 32-bit path's decoding): v_mfma_f32_16x16x4_f32 multiplies and adds float32 values as they
// are, no reduced-precision mode.  As in the bfloat16 product for few rows, the product is
// computed transposed, D[n, m] = sum_k W[n, k] X[m, k]: W streams from HBM straight into the A
// operands (16 bytes, four values of k, per lane), X comes from cache through a buffer descriptor
// that ends with its last row, the waves of a workgroup split K and their partial tiles are added
// through LDS in the fixed order of the waves: a row's sums depend on K and on the launch shape
// that N and K give, never on the other rows of the batch.
#include "common.h"
#include "api.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// MT tiles of 16 rows of X; WAVES waves split K in steps of 16 values (4 per lane group), U steps in flight.
template <int MT, int WAVES>
__global__ __launch_bounds__(WAVES * FSIE_WAVE) void gemm_mfma_fp32_kernel(const float* __restrict__ x,
                                                                          const float* __restrict__ w,
                                                                          const float* __restrict__ bias,
                                                                          float* __restrict__ y, int M, int N, int K) {
    constexpr int U = MT >= 3 ? 2 : 4;
    __shared__ float red[WAVES > 1 ? (WAVES - 1) * MT * FSIE_WAVE * 4 : 1];
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int row = lane & 15;  // row of the A tile (n) and column of the B tile (m)
    const int kg = lane >> 4;   // which 4 of a step's 16 k values this lane holds
    const int n0 = blockIdx.x * 16;
    const float* wp = w + static_cast<int64_t>(min(n0 + row, N - 1)) * K;  // rows past the end repeat the last; never written
    const __amdgpu_buffer_rsrc_t x_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(x), 0, M * K * static_cast<int>(sizeof(float)), 0x00020000);
    int xo[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xo[t] = (t * 16 + row) * K * static_cast<int>(sizeof(float));
    // two levels of float32 sums: a run of kFlush passes of the loop (some hundreds of products) is
    // summed on its own and then added to the total, so that the rounding error grows with the
    // square roots of the run and of the number of runs, not of K (K reaches 18944 in a 7B model)
    constexpr int kFlush = 8;
    floatx4 acc[MT], total[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = total[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int n_steps = (K + 15) / 16;
    int pass = 0;
    for (int s0 = wave; s0 < n_steps; s0 += WAVES * U, ++pass) {
        if (pass > 0 && pass % kFlush == 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                total[t] += acc[t];
                acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
            }
        }
        float4 a[U];
        u32x4 b[U][MT];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = (s0 + u * WAVES) * 16 + kg * 4;
            ok[u] = k0 < K;  // K is a multiple of 4: a lane's four values are all in or all out
            const int k0c = ok[u] ? k0 : 0;
            a[u] = *reinterpret_cast<const float4*>(wp + k0c);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                b[u][t] = __builtin_amdgcn_raw_buffer_load_b128(x_rows, xo[t] + k0c * static_cast<int>(sizeof(float)), 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) a[u] = float4{0.f, 0.f, 0.f, 0.f};
            const float av[4] = {a[u].x, a[u].y, a[u].z, a[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], __uint_as_float(b[u][t][j]), acc[t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] += total[t];
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
    // lane holds D[n0 + 4 kg + r][m = 16 t + row]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + row;
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int nn = n0 + kg * 4 + r;
            if (nn < N) y[static_cast<int64_t>(m) * N + nn] = bias ? acc[t][r] + bias[nn] : acc[t][r];
        }
    }
}

template <int MT>
int launch_mt(int waves, const float* x, const float* w, const float* bias, float* y, int M, int N, int K,
              hipStream_t stream) {
    const unsigned groups = static_cast<unsigned>((N + 15) / 16);
    switch (waves) {
        case 1: gemm_mfma_fp32_kernel<MT, 1><<<groups, 64, 0, stream>>>(x, w, bias, y, M, N, K); break;
        case 2: gemm_mfma_fp32_kernel<MT, 2><<<groups, 128, 0, stream>>>(x, w, bias, y, M, N, K); break;
        case 4: gemm_mfma_fp32_kernel<MT, 4><<<groups, 256, 0, stream>>>(x, w, bias, y, M, N, K); break;
        default: gemm_mfma_fp32_kernel<MT, 8><<<groups, 512, 0, stream>>>(x, w, bias, y, M, N, K); break;
    }
    FSIE_CHECK_LAUNCH("gemm_mfma_fp32");
    return 0;
}

}  // namespace

// float32 operands and result.  1 <= M <= 64, K a multiple of 4, x and w 16-byte aligned.
// waves: 1, 2, 4 or 8 waves of a workgroup split K; 0 = choose.
extern "C" int fsie_gemm_mfma_fp32(const float* x, const float* w, const float* bias, float* y, int M, int N, int K,
                                   int waves, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_fp32: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(M <= FSIE_GEMM_MFMA_SKINNY_MAX_M, "gemm_mfma_fp32: at most %d rows, got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    FSIE_REQUIRE(K % 4 == 0, "gemm_mfma_fp32: K=%d must be a multiple of 4", K);
    FSIE_REQUIRE(static_cast<int64_t>(M) * K * 4 < (int64_t{1} << 31),
                 "gemm_mfma_fp32: x of %d x %d is more than the kernel's 32-bit offsets take", M, K);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_fp32: operands must be 16-byte aligned");
    FSIE_REQUIRE(waves == 0 || waves == 1 || waves == 2 || waves == 4 || waves == 8,
                 "gemm_mfma_fp32: waves must be 0, 1, 2, 4 or 8");
    if (M == 0) return 0;
    if (waves == 0) {
        const int groups = (N + 15) / 16;
        const int steps = (K + 15) / 16;
        waves = 1;
        while (waves < 8 && groups * waves < 1024) waves *= 2;
        while (waves > 1 && steps < 4 * waves) waves /= 2;
    }
    switch ((M + 15) / 16) {
        case 1: return launch_mt<1>(waves, x, w, bias, y, M, N, K, stream);
        case 2: return launch_mt<2>(waves, x, w, bias, y, M, N, K, stream);
        case 3: return launch_mt<3>(waves, x, w, bias, y, M, N, K, stream);
        default: return launch_mt<4>(waves, x, w, bias, y, M, N, K, stream);
    }
}
