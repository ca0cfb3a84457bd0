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
#pragma once

#include "common.h"
#include "api.h"

namespace fsie_mm {


typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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
    const float* cos_sin;    // [M][head_dim / 2][2]: cos and sin of positions[m] * inv_freq[i], computed once
                             // for all layers of a step; null = the epilogue computes them
    bf16_t* k_pool;          // [pages][n_kv][page_size][head_dim]; null = nothing stored
    bf16_t* v_pool;          // [pages][n_kv][head_dim][page_size]
    int n_heads, n_kv, head_dim, page_size;
    int64_t pool_slots;
    int pairs_per_wg;  // rotary pairs (rows i and i + head_dim / 2 of a head) a workgroup owns: 1..8 * NB
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
// EPI_ROPE: see RopeArgs.  The rows of W are taken in pairs (i, i + head_dim/2) of a head, numbered
// through all heads; a workgroup owns `pairs_per_wg` consecutive pairs, eight to a block: tile rows
// 0..7 are the first members, rows 8..15 the second, so that both members of a pair lie in one
// accumulator tile, 32 lanes apart.  A block that is not full repeats the workgroup's last pair
// (the same addresses again: no further memory traffic) and does not write the repeats.  The
// number of pairs a workgroup owns is the host's choice: it spreads the rows evenly over the
// compute units, whose memory pipelines bound a product this small.
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
            const int half = rope.head_dim / 2;
            const int base = blockIdx.x * rope.pairs_per_wg;
            const int here = min(rope.pairs_per_wg, N / 2 - base);  // at least 1: the grid covers N / 2 pairs
            const int pair = base + min(b * 8 + (row & 7), here - 1);
            const int head = pair / half;
            n = head * rope.head_dim + (pair - head * half) + (row < 8 ? 0 : half);
        }
        n = min(n, N - 1);  // rows past the end repeat the last one; never written
        wp[b] = w + static_cast<int64_t>(n) * K;
    }
    // X is read through a buffer descriptor that ends with row M - 1: a lane whose row lies past
    // the end gets zeros and asks the memory for nothing (its columns of D are never written).
    // With one row (decoding a single request) 4 lanes of 64 fetch; reading the last row again
    // instead costs as many requests to the cache as a full tile.
    const __amdgpu_buffer_rsrc_t x_rows = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(x), 0, M * K * static_cast<int>(sizeof(bf16_t)), 0x00020000);
    int xo[MT];  // byte offset of this lane's row
#pragma unroll
    for (int t = 0; t < MT; ++t) xo[t] = (t * 16 + row) * K * static_cast<int>(sizeof(bf16_t));
    floatx4 acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[b][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // What the rotary epilogue reads from memory (positions, slots, bias, frequencies) is asked for
    // here, so that it arrives while W streams: the epilogue runs after the other waves have left,
    // and every microsecond of it is added to the kernel's time.  Every wave asks (no branch lies
    // around the loads, so nothing waits for them here); a table that does not exist is replaced
    // by the start of W, and what is read there is dropped.
    float e_bias[NB][4];
    double e_freq[NB][4];
    float2 e_cs[NB][MT][4];
    int e_pos[MT], e_slot[MT];
    if (EPI == EPI_ROPE) {
        const int half = rope.head_dim / 2;
        const int base = blockIdx.x * rope.pairs_per_wg;
        const int here = min(rope.pairs_per_wg, N / 2 - base);
        const float* bias_src = bias ? bias : reinterpret_cast<const float*>(w);
        const double* freq_src = rope.inv_freq ? rope.inv_freq : reinterpret_cast<const double*>(w);
        const bool stores = rope.k_pool && rope.slots;
        const int32_t* slot_src = stores ? rope.slots : rope.positions;
        const float2* cs_src = reinterpret_cast<const float2*>(rope.cos_sin ? rope.cos_sin : reinterpret_cast<const float*>(w));
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int pair = base + min(nb * 8 + (kg & 1) * 4 + r, here - 1);
                const int head = pair / half;
                const int i = pair - head * half;
                const float b = bias_src[bias ? head * rope.head_dim + i + (kg >= 2 ? half : 0) : 0];
                const double f = freq_src[rope.inv_freq ? i : 0];
                e_bias[nb][r] = bias ? b : 0.f;
                e_freq[nb][r] = f;
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const int m = min(t * 16 + row, M - 1);
                    e_cs[nb][t][r] = cs_src[rope.cos_sin ? m * half + i : 0];
                }
            }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = min(t * 16 + row, M - 1);
            e_pos[t] = rope.positions[m];
            const int sl = slot_src[m];
            e_slot[t] = stores ? sl : -1;
        }
    }

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
                const int k0 = k_begin + ((p0 + u * WAVES) * 2 + h) * kStep + kg * 8;
                ok[u][h] = k0 < k_end;  // K is a multiple of 8: a lane's 8 values are all in or all out
                const int k0c = ok[u][h] ? k0 : k_begin;  // the slice's first 8 values: always inside the row
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) a[u][h][nb].raw = *reinterpret_cast<const uint4*>(wp[nb] + k0c);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const u32x4 got = __builtin_amdgcn_raw_buffer_load_b128(
                        x_rows, xo[t] + k0c * static_cast<int>(sizeof(bf16_t)), 0, 0);
                    b[u][h][t].raw = uint4{got.x, got.y, got.z, got.w};
                }
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
                // tile row 4 kg + r: pair (kg & 1) * 4 + r of block nb, first member for kg < 2, second else
                const int half = rope.head_dim / 2;
                const int rot_heads = rope.n_heads + rope.n_kv;
                const int base = blockIdx.x * rope.pairs_per_wg;
                const int here = min(rope.pairs_per_wg, N / 2 - base);
                const bool second = kg >= 2;
                int slot = e_slot[t];
                if (slot >= rope.pool_slots) slot = -1;
                const int64_t page = slot >= 0 ? slot / rope.page_size : 0;
                const int off = slot >= 0 ? slot % rope.page_size : 0;
                const double pos = static_cast<double>(e_pos[t]);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int lp = nb * 8 + (kg & 1) * 4 + r;
                    const bool mine_to_write = lp < here;  // a repeat of the last pair otherwise
                    const int pair = base + min(lp, here - 1);
                    const int head = pair / half;
                    const int i = pair - head * half;
                    const int d = i + (second ? half : 0);  // dimension within the head
                    const int col = head * rope.head_dim + d;
                    const float mine = acc[nb][t][r] + e_bias[nb][r];
                    const float other = __shfl_xor(mine, 32, FSIE_WAVE);  // every lane takes part
                    if (head < rot_heads) {
                        float c = 1.f, sn = 0.f;
                        if (rope.cos_sin) {
                            c = e_cs[nb][t][r].x;
                            sn = e_cs[nb][t][r].y;
                        } else if (rope.inv_freq) {
                            rotation(pos, e_freq[nb][r], &c, &sn);
                        }
                        // first half: x1 c - x2 s; second half: x2 c + x1 s
                        const bf16_t res = from_float<bf16_t>(second ? mine * c + other * sn : mine * c - other * sn);
                        if (!mine_to_write) continue;
                        if (head < rope.n_heads) {
                            reinterpret_cast<bf16_t*>(y)[static_cast<int64_t>(m) * N + col] = res;
                        } else if (slot >= 0) {
                            rope.k_pool[((page * rope.n_kv + (head - rope.n_heads)) * rope.page_size + off) * rope.head_dim + d] = res;
                        }
                    } else if (mine_to_write && slot >= 0) {
                        rope.v_pool[((page * rope.n_kv + (head - rot_heads)) * rope.head_dim + d) * rope.page_size + off] =
                            from_float<bf16_t>(mine);
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
    const unsigned groups = EPI == EPI_ROPE ? (c.N / 2 + c.rope.pairs_per_wg - 1) / c.rope.pairs_per_wg
                                            : (c.N + 16 * NB - 1) / (16 * NB);
    const dim3 grid(groups, static_cast<unsigned>(c.splits > 1 ? c.splits : 1));
    gemm_mfma_skinny_kernel<MT, NB, WAVES, OutT, EPI><<<grid, WAVES * FSIE_WAVE, 0, c.stream>>>(
        static_cast<const bf16_t*>(c.x), static_cast<const bf16_t*>(c.w), c.bias, static_cast<OutT*>(c.y), c.M, c.N,
        c.K, k_slice, c.rope);
    FSIE_CHECK_LAUNCH("gemm_mfma_skinny");
    return 0;
}

// waves: 1, 2, 4, 8 or 16 (16 only while the reduction's LDS allows: MT * NB <= 4)
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

// blocks of 16 rows of W per workgroup: 1 or 2
template <int MT, typename OutT, int EPI>
int launch_blocks(int nb, int waves, const Call& c) {
    if (nb == 1) return launch_waves<MT, 1, OutT, EPI>(waves, c);
    return launch_waves<MT, 2, OutT, EPI>(waves, c);
}

// Entry points of the instantiation files (one translation unit each, compiled side by side).
int launch_f32(int mt, int blocks, int waves, const Call& c);      // float32 result or partial sums, up to 64 rows
int launch_bf16(int blocks, int waves, const Call& c);             // bfloat16 result, up to 16 rows
int launch_swiglu(int blocks, int waves, const Call& c);           // SiLU*up epilogue, up to 16 rows
int launch_rope(int mt, int waves, const Call& c);                 // q/k/v + rotary epilogue, up to 64 rows; two blocks a
                                                                   // workgroup (9 to 16 pairs) for one tile of x only

}  // namespace fsie_mm
