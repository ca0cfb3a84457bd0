// Y[M, N] = X[M, K] . W[N, K]^T for bfloat16 operands and 17 to 64 rows of X, float32 results:
// the weight-streaming matrix-core product for batches whose X no longer comes cheaply from cache.
//
// As in the product for few rows, D[n, m] = sum_k W[n, k] X[m, k]: W streams from HBM straight
// into the A registers of v_mfma_f32_16x16x32_bf16.  With up to four tiles of 16 rows of X, reading
// the B fragments from memory would move several times the bytes of W through every compute
// unit's memory pipeline, which is what bounds it (some 50 GB/s a unit).  So the waves of a workgroup
// take different blocks of 16 rows of W (none splits K) and share X: a stage of KS values of K of
// all rows of X is laid into LDS once per workgroup, in the order of the B fragments, and every
// wave reads its fragments from there.
//
// Pipeline of a stage s (one barrier a stage):
//   global loads of X for stage s+1 (to registers), then of W for stage s+1;
//   B fragments of stage s from LDS, products with the W of stage s (loaded a stage ago);
//   X of stage s+1 from registers to the other LDS buffer (waits for the X loads only: they were
//   issued before the W loads and the counter is in order); barrier.
// The last stage runs outside the loop, so that no branch lies around a batch of loads.
//
// blockIdx.y selects a slice of K (a multiple of KS); with more than one slice y is
// [slices][M][N], float32 partial sums for the consumer to add in the order of the slices.
//
// W may also come in the order of the A fragments (fsie_fragment_order): the 64 16-byte units of a
// block of 16 rows and a step of 32 values of K lie together, in the order of the lanes that hold
// them, block after block along K and then along N.  A wave's load is then one piece of 1 KB
// instead of 16 pieces of 64 bytes, and W can be read with streaming (non-temporal) loads.  Measured
// on MI355X with kernels that only read 272 MB (N = 37888, K = 3584): rows, plain loads 48 us
// (this kernel's product takes as long); rows, streaming loads 52; fragment order, plain 46.5;
// fragment order, streaming 41.3.
#include "common.h"
#include "api.h"

// 32-wide steps of K per stage (a stage is what the pipeline keeps in flight per wave and lays into
// LDS).  Measured on MI355X with 2, 4 and 8 (8 holds at most 32 rows in the 64 KB of static LDS): the
// gate/up shape (N = 37888, K = 3584) does not care (32 rows: 57 to 62 us for the best launch shape of
// each), so it is not the memory latency that bounds it there; the down shape (N = 3584, K = 18944 in
// 8 slices, 8 rows) takes 29.6 / 25.6 / 29.0 us.
#ifndef FSIE_WIDE_STEPS
#define FSIE_WIDE_STEPS 4
#endif

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

extern __shared__ u32x4 wide_dynamic_lds[];
constexpr int kStaticLds = 64 * 1024;
// bytes of the two buffers of a stage of X of `mt` tiles of 16 rows
constexpr int wide_lds_bytes(int mt, int steps) { return 2 * (4 * steps * (16 * mt + 1) + 1) * 16; }
typedef const __attribute__((address_space(1))) u32x4* GlobalVec;

union Frag {
    u32x4 q;
    bf16x8 v;
};

// MT tiles of 16 rows of X; WAVES waves of NB blocks of 16 rows of W each per workgroup (a wave's
// blocks share the B fragments it reads from LDS: with four tiles of X one block a wave would be
// bound by those reads); STEPS 32-wide MFMA steps per stage (KS = 32 * STEPS values of K).
// SWIGLU: the rows of W are gate and up interleaved and y is bfloat16 [M, N / 2], silu(gate) * up
// from the accumulators (a lane holds rows 4 kg .. 4 kg + 3 of a block: two pairs); one slice only.
template <int MT, int WAVES, int STEPS, int NB, bool SWIGLU, bool FRAGS>
__global__ __launch_bounds__(WAVES * 64) void gemm_mfma_wide_kernel(const bf16_t* __restrict__ x,
                                                                   const bf16_t* __restrict__ w,
                                                                   float* __restrict__ y, int M, int N, int K,
                                                                   int k_slice) {
    constexpr int KS = 32 * STEPS;
    constexpr int ROWS = 16 * MT;             // rows of X in LDS (rows past M repeat the last one)
    constexpr int UNITS = ROWS * 4 * STEPS;   // 16-byte units of a stage of X
    constexpr int THREADS = WAVES * 64;
    constexpr int PER_THREAD = (UNITS + THREADS - 1) / THREADS;
    constexpr int PITCH = ROWS + 1;           // units between consecutive (step, k group) runs: the
                                              // odd pitch spreads a staging wave's writes over the banks
    constexpr int SPARE = 4 * STEPS * PITCH;  // where threads without a unit of their own write
    // the two buffers of a stage of X: static up to seven tiles (58 KB); eight tiles (66 KB) take the LDS
    // that the launch asks for beyond the 64 KB a kernel may declare
    constexpr int BUF = 4 * STEPS * PITCH + 1;
    constexpr bool DYNAMIC = wide_lds_bytes(MT, STEPS) > kStaticLds;
    __shared__ u32x4 xs_static[DYNAMIC ? 1 : 2 * BUF];
    u32x4* const xs0 = DYNAMIC ? wide_dynamic_lds : xs_static;
    u32x4* const xs[2] = {xs0, xs0 + BUF};

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = lane & 15;  // row of the A tile (n) and column of the B tile (m)
    const int kg = lane >> 4;   // which 8 of a step's 32 k values this lane holds
    const int n0 = (blockIdx.x * WAVES + wave) * 16 * NB;
    const int k_begin = blockIdx.y * k_slice;
    const int k_end = min(K, k_begin + k_slice);
    const int n_stages = (k_end - k_begin) / KS;  // the host makes every slice a multiple of KS

    // rows of W past the end repeat the last one; their results are never written
    // W_STEP: values between a lane's fragments of consecutive steps
    constexpr int W_STEP = FRAGS ? 512 : 32;
    const bf16_t* wp[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        if constexpr (FRAGS)  // blocks past the end repeat the last one (the copy is padded to whole blocks)
            wp[nb] = w + (static_cast<int64_t>(min(n0 / 16 + nb, (N - 1) / 16)) * (K / 32) + k_begin / 32) * 512 + lane * 8;
        else
            wp[nb] = w + static_cast<int64_t>(min(n0 + nb * 16 + row, N - 1)) * K + k_begin + kg * 8;
    }
    auto load_w = [](const bf16_t* p) -> u32x4 {
        if constexpr (FRAGS) return __builtin_nontemporal_load((GlobalVec)p);
        else return *(GlobalVec)p;
    };
    // staging: unit u = (row of X, j = step * 4 + k group); consecutive threads take consecutive
    // 16 bytes of a row
    const bf16_t* xsrc[PER_THREAD];
    int xdst[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
        const int u = threadIdx.x + i * THREADS;
        const int uc = u < UNITS ? u : 0;  // a thread without a unit reads unit 0 and writes the spare place:
        const int m = uc / (4 * STEPS), j = uc - m * (4 * STEPS);  // no branch around loads or stores
        xsrc[i] = x + static_cast<int64_t>(min(m, M - 1)) * K + k_begin + j * 8;
        xdst[i] = u < UNITS ? j * PITCH + m : SPARE;
    }

    floatx4 acc[NB][MT];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[nb][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    if (n_stages <= 0) return;

    u32x4 xr[PER_THREAD];
    Frag wa[STEPS][NB], wb[STEPS][NB];  // the W fragments of even and odd stages
    // stage 0
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) xr[i] = *(GlobalVec)(xsrc[i]);
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) wa[s][nb].q = load_w(wp[nb] + s * W_STEP);
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) xs[0][xdst[i]] = xr[i];
    __syncthreads();

    auto products = [&](int buf, const Frag (&wc)[STEPS][NB]) {
        const u32x4* xb = xs[buf] + kg * PITCH + row;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            Frag b[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) b[t].q = xb[s * 4 * PITCH + t * 16];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[nb][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[s][nb].v, b[t].v, acc[nb][t], 0, 0, 0);
        }
    };
    // A stage that is not the last: fetch the next one (X first, then W into `wn`), work on this
    // one (`wc`, LDS buffer `buf`), hand the next X to the other buffer.  No branch lies around
    // the loads and no register is copied, so the wait before the products counts exactly the
    // loads issued after this stage's W.
    auto stage = [&](int buf, const Frag (&wc)[STEPS][NB], Frag (&wn)[STEPS][NB], int k1) {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) xr[i] = *(GlobalVec)(xsrc[i] + k1);
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) wn[s][nb].q = load_w(wp[nb] + k1 * (W_STEP / 32) + s * W_STEP);
        __builtin_amdgcn_sched_barrier(0);
        products(buf, wc);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) xs[buf ^ 1][xdst[i]] = xr[i];
        __syncthreads();
    };
    int st = 0;  // even here: stage st lies in buffer 0, its W in wa
    for (; st + 2 < n_stages; st += 2) {
        stage(0, wa, wb, (st + 1) * KS);
        stage(1, wb, wa, (st + 2) * KS);
    }
    if (st + 1 < n_stages) {
        stage(0, wa, wb, (st + 1) * KS);
        products(1, wb);
    } else {
        products(0, wa);
    }

    // lane holds D[n0 + 16 nb + 4 kg + r][m = 16 t + row]
    if constexpr (SWIGLU) {
        uint32_t* out = reinterpret_cast<uint32_t*>(y);  // two bfloat16 results a store: columns nn / 2 and nn / 2 + 1
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int m = t * 16 + row;
                const int nn = n0 + nb * 16 + kg * 4;  // a multiple of 4: gate, up, gate, up
                if (m >= M || nn >= N) continue;      // N is a multiple of 4 here (checked by the host)
                const float g0 = acc[nb][t][0], u0 = acc[nb][t][1], g1 = acc[nb][t][2], u1 = acc[nb][t][3];
                out[(static_cast<int64_t>(m) * (N / 2) + nn / 2) / 2] =
                    pack2_bf16((g0 / (1.0f + expf(-g0))) * u0, (g1 / (1.0f + expf(-g1))) * u1);
            }
        return;
    }
    float* part = y + static_cast<int64_t>(blockIdx.y) * M * N;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = t * 16 + row;
            if (m >= M) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int nn = n0 + nb * 16 + kg * 4 + r;
                if (nn < N) part[static_cast<int64_t>(m) * N + nn] = acc[nb][t][r];
            }
        }
}

template <int MT, int WAVES, int STEPS, int NB, bool SWIGLU, bool FRAGS>
int launch(const bf16_t* x, const bf16_t* w, float* y, int M, int N, int K, int splits, int k_slice,
           hipStream_t stream) {
    const int rows = 16 * NB * WAVES;
    const dim3 grid(static_cast<unsigned>((N + rows - 1) / rows), static_cast<unsigned>(splits));
    constexpr int lds = wide_lds_bytes(MT, STEPS);
    constexpr int dynamic = lds > kStaticLds ? lds : 0;
    if constexpr (dynamic > 0) {
        static const hipError_t allowed = hipFuncSetAttribute(
            reinterpret_cast<const void*>(&gemm_mfma_wide_kernel<MT, WAVES, STEPS, NB, SWIGLU, FRAGS>),
            hipFuncAttributeMaxDynamicSharedMemorySize, dynamic);
        if (allowed != hipSuccess) {
            fsie_set_error("gemm_mfma_wide: %d bytes of LDS for %d rows: %s", dynamic, M, hipGetErrorString(allowed));
            return 1;
        }
    }
    gemm_mfma_wide_kernel<MT, WAVES, STEPS, NB, SWIGLU, FRAGS><<<grid, WAVES * 64, dynamic, stream>>>(x, w, y, M, N, K, k_slice);
    FSIE_CHECK_LAUNCH("gemm_mfma_wide");
    return 0;
}

template <int WAVES, int STEPS, int NB, bool SWIGLU, bool FRAGS>
int launch_mt(int mt, const bf16_t* x, const bf16_t* w, float* y, int M, int N, int K, int splits, int k_slice,
              hipStream_t stream) {
    switch (mt) {
        case 1: return launch<1, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
        case 2: return launch<2, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
#if FSIE_WIDE_STEPS <= 4
        case 3: return launch<3, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
        case 4: return launch<4, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
        default:
            // five to eight tiles of X (65 to 128 rows): on a fragment-ordered weight, two row blocks a
            // wave, four waves and more
            if constexpr (FRAGS && NB == 2 && WAVES >= 4) {
                if (mt == 8) return launch<8, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
                if (mt == 5) return launch<5, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
                if (mt == 6) return launch<6, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
                if (mt == 7) return launch<7, WAVES, STEPS, NB, SWIGLU, FRAGS>(x, w, y, M, N, K, splits, k_slice, stream);
            }
            fsie_set_error("gemm_mfma_wide: %d rows only on a fragment-ordered weight with two row blocks a wave and "
                           "at least four waves (N = %d in %d slices gives %d blocks, %d waves)", M, N, splits, NB, WAVES);
            return 1;
#else
        default: fsie_set_error("gemm_mfma_wide: stages of %d steps hold at most 32 rows", STEPS); return 1;
#endif
    }
}

template <bool SWIGLU, bool FRAGS>
int launch_shape_of(int mt, int waves, int blocks, const bf16_t* x, const bf16_t* w, float* y, int M, int N, int K,
                    int splits, int k_slice, hipStream_t stream) {
    if constexpr (SWIGLU && FRAGS) {  // gate/up of 17 rows and more: any number of waves that deals the rows evenly
        if (blocks == 2 && waves == 3) return launch_mt<3, FSIE_WIDE_STEPS, 2, true, true>(mt, x, w, y, M, N, K, splits, k_slice, stream);
        if (blocks == 2 && waves == 5) return launch_mt<5, FSIE_WIDE_STEPS, 2, true, true>(mt, x, w, y, M, N, K, splits, k_slice, stream);
        if (blocks == 2 && waves == 6) return launch_mt<6, FSIE_WIDE_STEPS, 2, true, true>(mt, x, w, y, M, N, K, splits, k_slice, stream);
        if (blocks == 2 && waves == 7) return launch_mt<7, FSIE_WIDE_STEPS, 2, true, true>(mt, x, w, y, M, N, K, splits, k_slice, stream);
    }
    if (blocks == 2) {
        if (waves == 8) return launch_mt<8, FSIE_WIDE_STEPS, 2, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
        if (waves == 2) return launch_mt<2, FSIE_WIDE_STEPS, 2, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
        return launch_mt<4, FSIE_WIDE_STEPS, 2, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
    }
    if (waves == 8) return launch_mt<8, FSIE_WIDE_STEPS, 1, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
    if (waves == 2) return launch_mt<2, FSIE_WIDE_STEPS, 1, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
    return launch_mt<4, FSIE_WIDE_STEPS, 1, SWIGLU, FRAGS>(mt, x, w, y, M, N, K, splits, k_slice, stream);
}

// One thread a 16-byte unit of the copy: unit ((block, step), lane) holds the 8 values at row
// 16 block + (lane & 15), k = 32 step + 8 (lane >> 4); rows past N are zeros.
__global__ __launch_bounds__(256) void fragment_order_kernel(const u32x4* __restrict__ w, u32x4* __restrict__ out,
                                                             int N, int K, int64_t units) {
    const int64_t u = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (u >= units) return;
    const int lane = static_cast<int>(u & 63);
    const int64_t bs = u >> 6;
    const int steps = K / 32;
    const int64_t block = bs / steps;
    const int step = static_cast<int>(bs - block * steps);
    const int64_t n = block * 16 + (lane & 15);
    u32x4 v = {0u, 0u, 0u, 0u};
    if (n < N) v = w[(n * K + step * 32 + (lane >> 4) * 8) / 8];
    out[u] = v;
}

// Waves a workgroup and row blocks a wave where the caller leaves them open (0).
void launch_shape(int mt, int N, int splits, int& waves, int& blocks, bool gate_up = false, bool frags = false) {
    if (gate_up && mt >= 2 && waves == 0 && blocks == 0) {
        // 17 rows and more, one slice: the products and the reads of x from LDS bound a workgroup, so
        // a compute unit with two workgroups takes twice as long as one with one, and a unit draws
        // only so much from memory, so every unit should have one.  Two blocks a wave, and the fewest
        // waves a workgroup that still give at most one workgroup a unit (MI355X, 256 units, 64 rows,
        // fragment-ordered W: N = 37888, K = 3584 in 237 workgroups of five waves 48.9 us, in 148 of eight
        // 52.7, in 296 of four 62.3; N = 27648, K = 5120 in 216 of four waves 48.9, in 288 of three 70.8,
        // in 173 of five 61.0; N = 55296, K = 5120 in 247 of seven 87.5, in 216 of eight 86.8, in 288 of six
        // 129.9; N = 19456, K = 2048 in 203 of three 18.7, in 152 of four 20.6, in 304 of two 22.2).
        // Five, six and seven waves exist only for fragment-ordered weights.
        const int units = fsie_compute_units();
        blocks = 2;
        for (waves = 2; waves < 8; ++waves)
            if ((N + 32 * waves - 1) / (32 * waves) <= units) break;
        if (!frags && waves != 2 && waves != 4) waves = waves < 4 ? 4 : 8;
        if (waves == 2 && (N + 31) / 32 * 2 <= units) blocks = 1;  // a small N: twice the workgroups of one block a wave
        return;
    }
    if (blocks == 0) {
        // three or four tiles of X: two blocks of W a wave share the B fragments read from LDS,
        // where that still leaves a workgroup for most compute units (measured on MI355X, 64 rows,
        // N = 3584, K = 18944 in 8 slices: 33.6 against 37.7 us)
        blocks = (mt >= 3 && static_cast<int64_t>((N + 127) / 128) * splits >= 128) ? 2 : 1;
        // gate and up of one or two tiles at a very large N: two blocks a wave once that still gives
        // every compute unit a workgroup and a half (N = 55296, K = 5120, 8 rows: 107 against 112 us;
        // N = 27648: 56.6 against 52.5, N = 37888: 65 against 54, so not there)
        const int units = fsie_compute_units();
        if (gate_up && mt < 3 && units > 0 && static_cast<int64_t>((N + 127) / 128) * 2 >= 3 * static_cast<int64_t>(units))
            blocks = 2;
    }
    if (waves == 0) {
        // eight waves a workgroup halve the reads of X, but only a large N leaves enough
        // workgroups for them (64 rows: N = 152064 242 against 261 us; N = 3584, K = 18944 in 8
        // slices 39.6 against 38.1); with two blocks a wave, four waves (N = 152064: 236 against 260)
        const int64_t groups4 = static_cast<int64_t>((N + 63) / 64) * splits;
        waves = (groups4 >= 1024 && blocks == 1) ? 8 : 4;
        // one tile of X at a large N of a fragment-ordered W: nothing to share, and two waves a workgroup stream best (N = 152064,
        // K = 3584, fragment-ordered: 8 rows 168 us with two waves, 171 with four, 179 with eight; one row
        // 164 / 168 / 177; N = 152064, K = 5120, 8 rows: 247 / 249 / 259)
        if (frags && mt == 1 && groups4 >= 1024 && blocks == 1) waves = 2;  // (on rows: 215 / 195 / 194)
        // two waves a workgroup where that deals the waves more evenly to the compute units (N =
        // 5120 in 8 slices: 640 workgroups of four waves put 12 waves on the fullest of 256 units,
        // 1280 of two put 10; K = 13824, 8 rows: 26.7 against 29.8 us)
        const int units = fsie_compute_units();
        if (waves == 4 && blocks == 1 && units > 0) {
            const int64_t fullest4 = (groups4 + units - 1) / units * 4;
            const int64_t fullest2 = (static_cast<int64_t>((N + 31) / 32) * splits + units - 1) / units * 2;
            if (fullest2 < fullest4) waves = 2;
        }
    }
}

}  // namespace

// The length of a slice of K for `splits` slices, or 0 if K cannot be cut that way: K and every
// slice must be a multiple of the stage (128 values), and no slice may be empty.
extern "C" int fsie_gemm_mfma_wide_slice(int K, int splits) {
    constexpr int kStage = 32 * FSIE_WIDE_STEPS;
    if (K <= 0 || splits < 1 || splits > FSIE_GEMM_MAX_SPLITS || K % kStage) return 0;
    const int slice = ((K + splits - 1) / splits + kStage - 1) / kStage * kStage;
    if (static_cast<int64_t>(slice) * (splits - 1) >= K) return 0;
    return slice;
}

// Into how many slices of K a product of M rows that leaves partial sums is best cut (1: not at
// all, or this kernel does not take K).  A slice is at least 512 long.
// Up to 16 rows: as many slices as K gives, up to 8: many short workgroups, several a compute unit
// (N = K = 3584 on MI355X, 8 rows: 7 slices 7.4 us, 6 7.2, 4 9.3, the few-rows kernel's 4 8.4; the
// norm that then adds 7 parts instead of 4 takes 0.6 us longer, which leaves 0.03 ms of a decode
// step of 28 layers; with a norm that loops over the parts instead of asking for all at once it
// cost 0.07 ms more than it brought).
// From 17 rows on the workgroups keep a compute unit busy by themselves (the reads of x from LDS
// and the matrix instructions grow with the rows): two of them with up to 32 rows, one beyond, and
// what counts is that all workgroups run at once and leave few units idle: the cut that gives the
// most workgroups the device has room for
// (32 rows on 256 units: N = 3584, K = 18944 in 9 slices, 504 workgroups, 28.1 us against 29.2 in 8
// and 38.5 in 4; N = 5120, K = 13824 in 6 slices, 480 workgroups, 29.2 against 35.2 in 8;
// 64 rows: N = 3584, K = 18944 in 9 slices, 252 workgroups, 32.4 us against 33.2 in 8;
// N = 5120, K = 13824 in 6 slices, 240 workgroups, 32.4 against 43.5 in 8, 320 workgroups;
// N = 5120, K = 27648 in 6 slices 60.4 against 75.3; N = K = 5120 in 6 slices 17.4 against 21.6).
extern "C" int fsie_gemm_mfma_wide_best_splits(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 1;
    const int mt = (M + 15) / 16;
    const int units = fsie_compute_units();
    if (mt <= 1 || units <= 0) {
        for (int s = 8; s >= 2; --s)
            if (K / s >= 512 && fsie_gemm_mfma_wide_slice(K, s) > 0) return s;
        return 1;
    }
    int best = 1;
    int64_t best_groups = 0;
    bool best_fits = false;
    for (int s = 2; s <= FSIE_GEMM_MAX_SPLITS; ++s) {
        if (K / s < 512 || fsie_gemm_mfma_wide_slice(K, s) <= 0) continue;
        int waves = 0, blocks = 0;
        launch_shape(mt, N, s, waves, blocks);
        const int rows = 16 * blocks * waves;
        const int64_t groups = static_cast<int64_t>((N + rows - 1) / rows) * s;
        const bool fits = groups <= static_cast<int64_t>(units) * (mt == 2 ? 2 : 1);
        // among the cuts that fit, the most workgroups (of equals, the more slices: shorter ones);
        // if none fits, the fewest workgroups
        const bool better = best == 1 || (fits && !best_fits) || (fits == best_fits && (fits ? groups >= best_groups : groups < best_groups));
        if (better) best = s, best_groups = groups, best_fits = fits;
    }
    // The partial sums are bytes too: S * rows * N * 4, written and read again.  At four tiles of X
    // they can weigh a quarter of the weights (N = 4608, K = 3584 in seven slices: 8.3 MB beside
    // 33 MB): beyond a fifth, the fewest slices whose workgroups still number four fifths of the
    // units (there three: a decode step of 64 requests at that shape 4.01 ms against 4.04; at two
    // and three tiles seven slices stay faster, 3.51 against 3.58 ms at 32 rows, and at N = 7168,
    // K = 5120 the sums of the rule's four slices are a tenth and the rule's choice the fastest).
    if (mt == 4 && best > 2 && 4.0 * best * 64 * N > 0.2 * 2.0 * N * K) {
        for (int s = 2; s < best; ++s) {
            if (K / s < 512 || fsie_gemm_mfma_wide_slice(K, s) <= 0) continue;
            int waves = 0, blocks = 0;
            launch_shape(mt, N, s, waves, blocks);
            const int rows = 16 * blocks * waves;
            if (static_cast<int64_t>((N + rows - 1) / rows) * s * 5 >= static_cast<int64_t>(units) * 4) return s;
        }
    }
    return best;
}

// bfloat16 operands, float32 result: y is [M, N] (splits == 1) or [splits, M, N] partial sums.
// 1 <= M <= 64; K a multiple of 128 that `splits` slices of whole stages cover (see above);
// x and w 16-byte aligned.  waves: 2, 4 or 8 waves per workgroup; blocks: 1 or 2 blocks of 16 rows
// of W per wave; 0 = choose.
// frags: w is the copy that fsie_fragment_order made of the [N, K] matrix.
extern "C" int fsie_gemm_mfma_wide(const void* x, const void* w, float* y, int M, int N, int K, int splits,
                                   int waves, int blocks, int frags, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_wide: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(M <= (frags ? FSIE_GEMM_MFMA_WIDE_MAX_M : FSIE_GEMM_MFMA_SKINNY_MAX_M),
                 "gemm_mfma_wide: at most %d rows (%d on a fragment-ordered weight), got %d", FSIE_GEMM_MFMA_SKINNY_MAX_M,
                 FSIE_GEMM_MFMA_WIDE_MAX_M, M);
    const int k_slice = fsie_gemm_mfma_wide_slice(K, splits);
    FSIE_REQUIRE(k_slice > 0, "gemm_mfma_wide: K=%d cannot be cut into %d slices of whole stages of 128", K, splits);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_wide: operands must be 16-byte aligned");
    FSIE_REQUIRE(waves == 0 || waves == 2 || waves == 4 || waves == 8, "gemm_mfma_wide: waves must be 0, 2, 4 or 8");
    FSIE_REQUIRE(blocks == 0 || blocks == 1 || blocks == 2, "gemm_mfma_wide: blocks must be 0, 1 or 2");
    if (M == 0) return 0;
    const int mt = (M + 15) / 16;
    launch_shape(mt, N, splits, waves, blocks, false, frags != 0);
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* wq = static_cast<const bf16_t*>(w);
    if (frags) return launch_shape_of<false, true>(mt, waves, blocks, xp, wq, y, M, N, K, splits, k_slice, stream);
    return launch_shape_of<false, false>(mt, waves, blocks, xp, wq, y, M, N, K, splits, k_slice, stream);
}

// The same product with the rows of w as gate and up in turn: y is bfloat16 [M, N / 2], silu(gate) * up.
// N a multiple of 4; one slice of K.
extern "C" int fsie_gemm_mfma_wide_swiglu(const void* x, const void* w, void* y, int M, int N, int K, int waves,
                                          int blocks, int frags, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_mfma_wide_swiglu: bad sizes M=%d N=%d K=%d", M, N, K);
    FSIE_REQUIRE(M <= (frags ? FSIE_GEMM_MFMA_WIDE_MAX_M : FSIE_GEMM_MFMA_SKINNY_MAX_M),
                 "gemm_mfma_wide_swiglu: at most %d rows (%d on a fragment-ordered weight), got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, FSIE_GEMM_MFMA_WIDE_MAX_M, M);
    FSIE_REQUIRE(N % 4 == 0, "gemm_mfma_wide_swiglu: N=%d must be a multiple of 4 (gate and up rows in turn)", N);
    const int k_slice = fsie_gemm_mfma_wide_slice(K, 1);
    FSIE_REQUIRE(k_slice > 0, "gemm_mfma_wide_swiglu: K=%d must be a multiple of the stage of %d", K, 32 * FSIE_WIDE_STEPS);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(y) % 4 == 0,
                 "gemm_mfma_wide_swiglu: operands must be 16-byte aligned, the result 4-byte");
    FSIE_REQUIRE(waves == 0 || waves == 2 || waves == 4 || waves == 8 || (frags && blocks == 2 && waves >= 2 && waves <= 8),
                 "gemm_mfma_wide_swiglu: waves must be 0, 2, 4 or 8 (2 to 8 with two blocks a wave on a fragment-ordered weight)");
    FSIE_REQUIRE(blocks == 0 || blocks == 1 || blocks == 2, "gemm_mfma_wide_swiglu: blocks must be 0, 1 or 2");
    if (M == 0) return 0;
    const int mt = (M + 15) / 16;
    launch_shape(mt, N, 1, waves, blocks, true, frags != 0);
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* wq = static_cast<const bf16_t*>(w);
    float* yp = static_cast<float*>(y);
    if (frags) return launch_shape_of<true, true>(mt, waves, blocks, xp, wq, yp, M, N, K, 1, k_slice, stream);
    return launch_shape_of<true, false>(mt, waves, blocks, xp, wq, yp, M, N, K, 1, k_slice, stream);
}

// The copy of a bfloat16 matrix w [N, K] in the order of the matrix instruction's A fragments, for
// the products above with frags set: out holds ceil(N / 16) * 16 * K values (fsie_fragment_order_size),
// the rows past N zeros.  K a multiple of 32; w and out 16-byte aligned and distinct.
extern "C" int64_t fsie_fragment_order_size(int N, int K) {
    if (N <= 0 || K <= 0 || K % 32) return 0;
    return static_cast<int64_t>((N + 15) / 16) * 16 * K;
}

extern "C" int fsie_fragment_order(const void* w, void* out, int N, int K, hipStream_t stream) {
    FSIE_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "fragment_order: N=%d, K=%d: K must be a multiple of 32", N, K);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && w != out,
                 "fragment_order: both matrices must be 16-byte aligned, and two");
    const int64_t units = fsie_fragment_order_size(N, K) / 8;
    FSIE_REQUIRE((units + 255) / 256 <= 0x7fffffff, "fragment_order: N=%d, K=%d is too large", N, K);
    fragment_order_kernel<<<static_cast<unsigned>((units + 255) / 256), 256, 0, stream>>>(
        static_cast<const u32x4*>(w), static_cast<u32x4*>(out), N, K, units);
    FSIE_CHECK_LAUNCH("fragment_order");
    return 0;
}

// Whether the products above take M rows of this shape: up to 64 always; 65 to FSIE_GEMM_MFMA_WIDE_MAX_M only
// on a fragment-ordered weight and where the launch shape they would choose has two row blocks a wave
// and at least four waves a workgroup (the kernels of five to seven tiles exist for those only).
// gate_up: the SiLU*up product (one slice).
extern "C" int fsie_gemm_mfma_wide_takes(int M, int N, int K, int splits, int gate_up, int frags) {
    if (M <= 0 || N <= 0 || fsie_gemm_mfma_wide_slice(K, gate_up ? 1 : splits) <= 0) return 0;
    if (gate_up && N % 4) return 0;
    if (M <= FSIE_GEMM_MFMA_SKINNY_MAX_M) return 1;
    if (!frags || M > FSIE_GEMM_MFMA_WIDE_MAX_M || FSIE_WIDE_STEPS > 4) return 0;
    int waves = 0, blocks = 0;
    launch_shape((M + 15) / 16, N, gate_up ? 1 : splits, waves, blocks, gate_up != 0, true);
    return blocks == 2 && waves >= 4;
}
