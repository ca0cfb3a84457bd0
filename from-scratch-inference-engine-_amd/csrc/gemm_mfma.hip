// Y[M, N] = X[M, K] . W[N, K]^T (+ bias) for bfloat16 operands and few rows (decode: M <= 64),
// on the matrix cores.  The product is computed transposed, D[n, m] = sum_k W[n, k] X[m, k], so
// that the big operand W streams from HBM straight into the A registers of
// v_mfma_f32_16x16x32_bf16 (16 bytes of one row per lane, no conversion, no LDS) and the small
// operand X comes from cache.  The kernel is bound by the read of W.
//
// One workgroup owns one, two or four blocks of 16 rows of W (16 output columns each), which share
// the X fragments; its waves split K in pairs of 32-wide steps, interleaved, and the partial
// tiles are summed through LDS in the fixed order of the waves, so the result does not depend on
// the batch or on timing.
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

enum Epilogue { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_ROPE = 2 };

// What the rotary epilogue needs: W is a fused q/k/v projection (n_heads + 2 n_kv heads of
// head_dim rows); the kernel adds the bias, rotates the q and k heads by positions[m] * inv_freq
// (rotate-half over the whole head), writes q into the rows of y and k (rotated) and v into the
// cache pages at slots[m] (negative or >= pool_slots: not stored).
struct RopeArgs {
    const int32_t* positions;
    const int32_t* slots;
    const double* inv_freq;  // head_dim / 2 entries; null = no rotation
    bf16_t* k_pool;          // [pages][n_kv][page_size][head_dim]; null = nothing stored
    bf16_t* v_pool;          // [pages][n_kv][head_dim][page_size]
    int n_heads, n_kv, head_dim, page_size;
    int64_t pool_slots;
};

// angle = position * inv_freq in float64, reduced in float64 to [-pi, pi], then float32 sine and
// cosine (the same as the stand-alone rotary kernel).
__device__ __forceinline__ void rotation(double pos, double inv_freq, float* c, float* s) {
    const double ang = pos * inv_freq;
    const double turns = rint(ang * 0.15915494309189535);
    const double red = fma(-turns, 6.283185307179586, ang) - turns * 2.4492935982947064e-16;
    sincosf(static_cast<float>(red), s, c);
}

// MT = tiles of 16 rows of X, NB = blocks of 16 rows of W per workgroup (they share the X
// fragments), WAVES = waves of the workgroup, which split K.
// EPI_SWIGLU: the rows of W are gate and up interleaved; the output has N/2 columns,
// y[m, j] = silu(d[2j]) * d[2j + 1], computed in float32 from the accumulators.
// EPI_ROPE: see RopeArgs.  A block of 16 rows of a q or k head then holds rows 8b..8b+7 of the
// head's first half and the same of its second half, so that both members of every rotary pair
// (i, i + head_dim/2) lie in one accumulator tile, 32 lanes apart.
// blockIdx.y selects a slice of K of `k_slice` values (a multiple of 64); with more than one slice
// the kernel writes float32 partial sums y[slice][m][n] without bias, for the consumer to add up
// in the order of the slices.
template <int MT, int NB, int WAVES, typename OutT, int EPI>
__global__ __launch_bounds__(WAVES * FSIE_WAVE) void gemm_mfma_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    OutT* __restrict__ y, int M, int N, int K, int k_slice, RopeArgs rope) {
    constexpr bool SWIGLU = EPI == EPI_SWIGLU;
    __shared__ float red[WAVES > 1 ? (WAVES - 1) * NB * MT * FSIE_WAVE * 4 : 1];
    const int lane = threadIdx.x & (FSIE_WAVE - 1);
    const int wave = threadIdx.x / FSIE_WAVE;
    const int row = lane & 15;  // row of the A tile (n) and column of the B tile (m)
    const int kg = lane >> 4;   // which 8 of the 32 k values this lane holds
    const int n0 = blockIdx.x * (16 * NB);
    const bf16_t* wp[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        int n = n0 + b * 16 + row;
        if (EPI == EPI_ROPE) {
            const int per_head = rope.head_dim / 16;
            const int block = blockIdx.x * NB + b;
            const int head = block / per_head, sub = block - head * per_head;
            if (head < rope.n_heads + rope.n_kv) {
                n = head * rope.head_dim + sub * 8 + (row < 8 ? row : rope.head_dim / 2 + row - 8);
            }
        }
        n = min(n, N - 1);  // rows past the end repeat the last one; never written
        wp[b] = w + static_cast<int64_t>(n) * K + kg * 8;
    }
    const bf16_t* xp[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        // rows of X past the end read the last row again: their columns of D are never written
        xp[t] = x + static_cast<int64_t>(min(t * 16 + row, M - 1)) * K + kg * 8;
    }
    floatx4 acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[b][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // k steps of 32; a wave takes pairs of steps (128 bytes of every row), pairs interleaved over the waves
    const int k_begin = blockIdx.y * k_slice;
    const int k_end = min(K, k_begin + k_slice);
    const int n_pairs = (k_end - k_begin + 2 * kStep - 1) / (2 * kStep);
    constexpr int U = (NB * MT >= 8) ? 1 : 2;  // pairs in flight per wave (more cost occupancy and lost 10-30 %)
    for (int p0 = wave; p0 < n_pairs; p0 += WAVES * U) {
        // loads without branches, so that they all go out before the first wait: a step past the
        // end of K reads step 0 again and its A fragments are zeroed afterwards
        Frag a[U][2][NB], b[U][2][MT];
        bool ok[U][2];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int k0 = k_begin + ((p0 + u * WAVES) * 2 + h) * kStep;
                ok[u][h] = k0 + kg * 8 < k_end;  // K is a multiple of 8: a lane's 8 values are all in or all out
                const int k0c = ok[u][h] ? k0 : 0;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) a[u][h][nb].raw = *reinterpret_cast<const uint4*>(wp[nb] + k0c);
#pragma unroll
                for (int t = 0; t < MT; ++t) b[u][h][t].raw = *reinterpret_cast<const uint4*>(xp[t] + k0c);
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    if (!ok[u][h]) a[u][h][nb].raw = uint4{0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < MT; ++t)
                        acc[nb][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][h][nb].v, b[u][h][t].v, acc[nb][t], 0, 0, 0);
                }
    }

    if (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        red[((((wave - 1) * NB + nb) * MT + t) * 4 + r) * FSIE_WAVE + lane] = acc[nb][t][r];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int wv = 0; wv < WAVES - 1; ++wv)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[nb][t][r] += red[(((wv * NB + nb) * MT + t) * 4 + r) * FSIE_WAVE + lane];
    }
    // lane holds D[n0 + 16 nb + 4 kg + r][m = 16 t + row]
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + row;
            if (m >= M) continue;
            if (gridDim.y > 1) {
                float* part = reinterpret_cast<float*>(y) + (static_cast<int64_t>(blockIdx.y) * M + m) * N;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int nn = n0 + nb * 16 + kg * 4 + r;
                    if (nn < N) part[nn] = acc[nb][t][r];
                }
                continue;
            }
            if (EPI == EPI_ROPE) {
                const int per_head = rope.head_dim / 16;
                const int block = blockIdx.x * NB + nb;
                if (block * 16 >= N) continue;  // N is a multiple of 16 here
                const int head = block / per_head, sub = block - head * per_head;
                const int rot_heads = rope.n_heads + rope.n_kv;
                const int half = rope.head_dim / 2;
                int slot = (rope.k_pool && rope.slots) ? rope.slots[m] : -1;
                if (slot >= rope.pool_slots) slot = -1;
                const int64_t page = slot >= 0 ? slot / rope.page_size : 0;
                const int off = slot >= 0 ? slot % rope.page_size : 0;
                if (head < rot_heads) {
                    // tile rows 0..7: dimensions i = 8 sub + (0..7); rows 8..15: i + half
                    const bool second = kg >= 2;
                    const int i0 = sub * 8 + (kg & 1) * 4;
                    const int col0 = head * rope.head_dim + i0 + (second ? half : 0);
                    const double pos = static_cast<double>(rope.positions[m]);
                    bf16_t res[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float mine = acc[nb][t][r] + (bias ? bias[col0 + r] : 0.f);
                        const float other = __shfl_xor(mine, 32, FSIE_WAVE);
                        float c = 1.f, sn = 0.f;
                        if (rope.inv_freq) rotation(pos, rope.inv_freq[i0 + r], &c, &sn);
                        // first half: x1 c - x2 s; second half: x2 c + x1 s
                        res[r] = from_float<bf16_t>(second ? mine * c + other * sn : mine * c - other * sn);
                    }
                    if (head < rope.n_heads) {
                        bf16_t* dst = reinterpret_cast<bf16_t*>(y) + static_cast<int64_t>(m) * N + col0;
#pragma unroll
                        for (int r = 0; r < 4; ++r) dst[r] = res[r];
                    } else if (slot >= 0) {
                        bf16_t* dst = rope.k_pool +
                                      ((page * rope.n_kv + (head - rope.n_heads)) * rope.page_size + off) * rope.head_dim +
                                      (col0 - head * rope.head_dim);
#pragma unroll
                        for (int r = 0; r < 4; ++r) dst[r] = res[r];
                    }
                } else if (slot >= 0) {
                    const int kvh = head - rot_heads;
                    const int d0 = sub * 16 + kg * 4;
                    const int col0 = head * rope.head_dim + d0;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float v = acc[nb][t][r] + (bias ? bias[col0 + r] : 0.f);
                        rope.v_pool[((page * rope.n_kv + kvh) * rope.head_dim + d0 + r) * rope.page_size + off] =
                            from_float<bf16_t>(v);
                    }
                }
                continue;
            }
            if (SWIGLU) {
#pragma unroll
                for (int r = 0; r < 4; r += 2) {
                    const int nn = n0 + nb * 16 + kg * 4 + r;  // even: a gate row, nn + 1 its up row
                    if (nn + 1 < N) {
                        const float g = acc[nb][t][r], u = acc[nb][t][r + 1];
                        y[static_cast<int64_t>(m) * (N / 2) + nn / 2] = from_float<OutT>((g / (1.0f + expf(-g))) * u);
                    }
                }
                continue;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int nn = n0 + nb * 16 + kg * 4 + r;
                if (nn < N) {
                    const float v = bias ? acc[nb][t][r] + bias[nn] : acc[nb][t][r];
                    y[static_cast<int64_t>(m) * N + nn] = from_float<OutT>(v);
                }
            }
        }
}

struct Call {
    const void* x;
    const void* w;
    const float* bias;
    void* y;
    int M, N, K;
    int splits;  // slices of K, each a workgroup row of its own (partial sums out) when > 1
    hipStream_t stream;
    RopeArgs rope;
};

template <int MT, int NB, int WAVES, typename OutT, int EPI>
int launch(const Call& c) {
    const int k_slice = c.splits > 1 ? ((c.K + c.splits - 1) / c.splits + 63) / 64 * 64 : c.K;
    const dim3 grid(static_cast<unsigned>((c.N + 16 * NB - 1) / (16 * NB)),
                    static_cast<unsigned>(c.splits > 1 ? c.splits : 1));
    gemm_mfma_skinny_kernel<MT, NB, WAVES, OutT, EPI><<<grid, WAVES * FSIE_WAVE, 0, c.stream>>>(
        static_cast<const bf16_t*>(c.x), static_cast<const bf16_t*>(c.w), c.bias, static_cast<OutT*>(c.y), c.M, c.N,
        c.K, k_slice, c.rope);
    FSIE_CHECK_LAUNCH("gemm_mfma_skinny");
    return 0;
}

template <int MT, int NB, typename OutT, int EPI>
int launch_waves(int waves, const Call& c) {
    switch (waves) {
        case 1: return launch<MT, NB, 1, OutT, EPI>(c);
        case 2: return launch<MT, NB, 2, OutT, EPI>(c);
        case 4: return launch<MT, NB, 4, OutT, EPI>(c);
        case 8: return launch<MT, NB, 8, OutT, EPI>(c);
        default:
            if constexpr (MT * NB <= 4) return launch<MT, NB, 16, OutT, EPI>(c);
            return launch<MT, NB, 8, OutT, EPI>(c);
    }
}

template <int MT, typename OutT, int EPI>
int launch_blocks(int nb, int waves, const Call& c) {
    switch (nb) {
        case 1: return launch_waves<MT, 1, OutT, EPI>(waves, c);
        case 2: return launch_waves<MT, 2, OutT, EPI>(waves, c);
        default: return launch_waves<MT, 4, OutT, EPI>(waves, c);
    }
}

template <typename OutT, int EPI>
int launch_tiles(int mt, int nb, int waves, const Call& c) {
    switch (mt) {
        case 1: return launch_blocks<1, OutT, EPI>(nb, waves, c);
        case 2: return launch_blocks<2, OutT, EPI>(nb, waves, c);
        case 3: return launch_blocks<3, OutT, EPI>(nb, waves, c);
        default: return launch_blocks<4, OutT, EPI>(nb, waves, c);
    }
}

}  // namespace

// bfloat16 only.  M <= 64, K a multiple of 8, x and w 16-byte aligned.
// waves (K split inside a workgroup) and blocks (16-row blocks of W per workgroup): 0 = choose.
// epilogue: 0 = y = d (+ bias); 1 = SiLU*up over interleaved gate/up rows (N even, no bias, y is [M, N/2]).
// splits > 1: K is cut into that many slices, each summed by workgroups of its own; y is then
// float32 [splits, M, N], partial sums without bias, which the consumer adds in the order of the slices
// (fsie_rmsnorm takes them as its delta).  Every slice must hold at least 64 values of K.
extern "C" int fsie_gemm_mfma_skinny(const void* x, const void* w, const float* bias, void* y, int M, int N, int K,
                                     int out_f32, int waves, int blocks, int epilogue, int splits,
                                     hipStream_t stream) {
    FSIE_REQUIRE(splits >= 1 && splits <= FSIE_GEMM_MAX_SPLITS, "gemm_mfma_skinny: splits must be 1..%d, got %d",
                 FSIE_GEMM_MAX_SPLITS, splits);
    FSIE_REQUIRE(splits == 1 || (epilogue == 0 && !bias && out_f32),
                 "gemm_mfma_skinny: partial sums are float32, without bias or epilogue");
    FSIE_REQUIRE(splits == 1 || ((K + splits - 1) / splits + 63) / 64 * 64 * (splits - 1) < K,
                 "gemm_mfma_skinny: K=%d is too short for %d slices", K, splits);
    FSIE_REQUIRE(epilogue == 0 || epilogue == 1, "gemm_mfma_skinny: unknown epilogue %d", epilogue);
    FSIE_REQUIRE(epilogue == 0 || (N % 2 == 0 && !bias && !out_f32),
                 "gemm_mfma_skinny: the SiLU*up epilogue needs an even N, no bias and a bfloat16 result");
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(M <= FSIE_GEMM_MFMA_SKINNY_MAX_M, "gemm_mfma_skinny: at most %d rows, got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    FSIE_REQUIRE(K % 8 == 0, "gemm_mfma_skinny: K=%d must be a multiple of 8", K);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_skinny: operands must be 16-byte aligned");
    FSIE_REQUIRE(waves == 0 || waves == 1 || waves == 2 || waves == 4 || waves == 8 || waves == 16,
                 "gemm_mfma_skinny: waves must be 0, 1, 2, 4, 8 or 16");
    FSIE_REQUIRE(blocks == 0 || blocks == 1 || blocks == 2 || blocks == 4, "gemm_mfma_skinny: blocks must be 0, 1, 2 or 4");
    if (M == 0) return 0;
    const int mt = (M + 15) / 16;
    const int pairs = ((K + splits - 1) / splits + 2 * kStep - 1) / (2 * kStep);
    if (blocks == 0) {
        // more than a few rows of X: two blocks of W share each X fragment where N still leaves
        // enough workgroups for the chip (measured on MI355X: 5.2 against 4.4 TB/s at N = 37888)
        blocks = (M > 4 && static_cast<int64_t>(N) * splits >= 14336) ? 2 : 1;
    }
    if (waves == 0) {
        // split K inside the workgroup until about a thousand waves stream W; a single row of X
        // gains from more loads in flight even at large N
        const int groups = (N + 16 * blocks - 1) / (16 * blocks) * splits;
        waves = 1;
        while (waves < 16 && groups * waves < 1024) waves *= 2;
        if (M <= 4 && waves < 8) waves = 8;
        while (waves > 1 && pairs < 2 * waves) waves /= 2;
    }
    if (mt * blocks > 4 && waves > 8) waves = 8;  // LDS of the reduction
    const Call call{x, w, bias, y, M, N, K, splits, stream, RopeArgs{}};
    if (epilogue == 1) return launch_tiles<bf16_t, EPI_SWIGLU>(mt, blocks, waves, call);
    return out_f32 ? launch_tiles<float, EPI_PLAIN>(mt, blocks, waves, call)
                   : launch_tiles<bf16_t, EPI_PLAIN>(mt, blocks, waves, call);
}

// The fused q/k/v projection of an attention layer with the position encoding in its epilogue:
// y[m, :] (bfloat16, [M, N], N = (n_heads + 2 n_kv) * head_dim) receives the q heads, with bias
// and rotated; the k heads (bias, rotated) and v heads (bias) go only to the cache pages at
// slots[m] (their columns of y are left unwritten).  head_dim a multiple of 16, the rotation over
// the whole head (inv_freq: head_dim / 2 float64 entries, or null for none).  k_pool null: nothing
// is stored.  M <= 64, K a multiple of 8.
extern "C" int fsie_gemm_mfma_skinny_rope(const void* x, const void* w, const float* bias, void* y, int M, int K,
                                          const int32_t* positions, const int32_t* slots, const double* inv_freq,
                                          void* k_pool, void* v_pool, int n_heads, int n_kv, int head_dim,
                                          int page_size, int64_t pool_slots, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && K > 0 && n_heads > 0 && n_kv > 0, "gemm_mfma_skinny_rope: bad sizes");
    FSIE_REQUIRE(M <= FSIE_GEMM_MFMA_SKINNY_MAX_M, "gemm_mfma_skinny_rope: at most %d rows, got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    FSIE_REQUIRE(K % 8 == 0, "gemm_mfma_skinny_rope: K=%d must be a multiple of 8", K);
    FSIE_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "gemm_mfma_skinny_rope: head_dim %d must be a multiple of 16",
                 head_dim);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_skinny_rope: operands must be 16-byte aligned");
    FSIE_REQUIRE(positions, "gemm_mfma_skinny_rope: no positions");
    const bool store = k_pool != nullptr;
    FSIE_REQUIRE(!store || (v_pool && slots && page_size > 0 && pool_slots > 0),
                 "gemm_mfma_skinny_rope: a cache needs both pools, slots and a page geometry");
    if (M == 0) return 0;
    const int N = (n_heads + 2 * n_kv) * head_dim;
    const int mt = (M + 15) / 16;
    const int pairs = (K + 2 * kStep - 1) / (2 * kStep);
    const int blocks = 1;
    int waves = 1;
    while (waves < 16 && (N / 16) * waves < 1024) waves *= 2;
    if (M <= 4 && waves < 8) waves = 8;
    while (waves > 1 && pairs < 2 * waves) waves /= 2;
    if (mt * blocks > 4 && waves > 8) waves = 8;  // LDS of the reduction
    const Call call{x, w, bias, y, M, N, K, 1, stream,
                    RopeArgs{positions, slots, inv_freq, static_cast<bf16_t*>(store ? k_pool : nullptr),
                             static_cast<bf16_t*>(store ? v_pool : nullptr), n_heads, n_kv, head_dim,
                             store ? page_size : 1, store ? pool_slots : 0}};
    return launch_tiles<bf16_t, EPI_ROPE>(mt, blocks, waves, call);
}
