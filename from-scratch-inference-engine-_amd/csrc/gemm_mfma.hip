// Entry points of the weight-streaming matrix-core products (kernel: gemm_mfma_impl.h): checks and
// the choice of the launch shape.
#include "gemm_mfma_impl.h"

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
    FSIE_REQUIRE(K <= (1 << 23), "gemm_mfma_skinny: K=%d is more than the kernel's 32-bit offsets into x take", K);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_skinny: operands must be 16-byte aligned");
    FSIE_REQUIRE(waves == 0 || waves == 1 || waves == 2 || waves == 4 || waves == 8 || waves == 16,
                 "gemm_mfma_skinny: waves must be 0, 1, 2, 4, 8 or 16");
    FSIE_REQUIRE(blocks == 0 || blocks == 1 || blocks == 2, "gemm_mfma_skinny: blocks must be 0, 1 or 2");
    FSIE_REQUIRE(out_f32 || M <= FSIE_GEMM_MFMA_SKINNY_BEST_M,
                 "gemm_mfma_skinny: bfloat16 results for at most %d rows (float32 results up to %d), got %d",
                 FSIE_GEMM_MFMA_SKINNY_BEST_M, FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    if (M == 0) return 0;
    const int mt = (M + 15) / 16;
    const int pairs = ((K + splits - 1) / splits + 2 * fsie_mm::kStep - 1) / (2 * fsie_mm::kStep);
    if (blocks == 0) {
        // more than two rows of X: two blocks of W share each X fragment where N still leaves
        // enough workgroups for the chip (measured on MI355X at N = 37888: 5.2 against 4.4 TB/s
        // with 8 rows, 49 against 58 us with 4)
        blocks = (M > 2 && static_cast<int64_t>(N) * splits >= 14336) ? 2 : 1;
    }
    if (waves == 0) {
        // split K inside the workgroup until some eight hundred waves stream W (N = 3584,
        // K = 18944 in four slices, 8 rows: 27.9 us with 896 waves, 32.7 with 1792; N = 27648,
        // K = 5120, 8 rows: 58.4 us with 864 waves, 66.5 with 1728; with 64 rows 1792 are
        // better, 6.19 against 6.42 ms for a whole decode step of a 7B model); one or two
        // rows of X gain from more loads in flight even at large N (four waves where N alone gives
        // two thousand workgroups: 177 against 181 us at N = 152064; two from 896 workgroups on)
        const int groups = (N + 16 * blocks - 1) / (16 * blocks) * splits;
        waves = 1;
        const int enough = M <= 16 ? 832 : 1024;  // more rows of X: more waves to share the products
        while (waves < 16 && groups * waves < enough) waves *= 2;
        const int few_rows_waves = groups >= 2048 ? 4 : (groups >= 896 ? 2 : 8);
        if (M <= 2 && waves < few_rows_waves) waves = few_rows_waves;
        while (waves > 1 && pairs < 2 * waves) waves /= 2;
    }
    if (mt * blocks > 4 && waves > 8) waves = 8;  // LDS of the reduction
    const fsie_mm::Call call{x, w, bias, y, M, N, K, splits, stream, fsie_mm::RopeArgs{}};
    if (epilogue == 1) return fsie_mm::launch_swiglu(blocks, waves, call);
    return out_f32 ? fsie_mm::launch_f32(mt, blocks, waves, call) : fsie_mm::launch_bf16(blocks, waves, call);
}

// The fused q/k/v projection of an attention layer with the position encoding in its epilogue:
// y[m, :] (bfloat16, [M, N], N = (n_heads + 2 n_kv) * head_dim) receives the q heads, with bias
// and rotated; the k heads (bias, rotated) and v heads (bias) go only to the cache pages at
// slots[m] (their columns of y are left unwritten).  head_dim a multiple of 16, the rotation over
// the whole head (inv_freq: head_dim / 2 float64 entries, or null for none).  k_pool null: nothing
// is stored.  M <= 64, K a multiple of 8.
extern "C" int fsie_gemm_mfma_skinny_rope(const void* x, const void* w, const float* bias, void* y, int M, int K,
                                          const int32_t* positions, const int32_t* slots, const double* inv_freq,
                                          const float* cos_sin, void* k_pool, void* v_pool, int n_heads, int n_kv,
                                          int head_dim,
                                          int page_size, int64_t pool_slots, hipStream_t stream) {
    FSIE_REQUIRE(M >= 0 && K > 0 && n_heads > 0 && n_kv > 0, "gemm_mfma_skinny_rope: bad sizes");
    FSIE_REQUIRE(M <= FSIE_GEMM_MFMA_SKINNY_MAX_M, "gemm_mfma_skinny_rope: at most %d rows, got %d",
                 FSIE_GEMM_MFMA_SKINNY_MAX_M, M);
    FSIE_REQUIRE(K % 8 == 0, "gemm_mfma_skinny_rope: K=%d must be a multiple of 8", K);
    FSIE_REQUIRE(K <= (1 << 23), "gemm_mfma_skinny_rope: K=%d is more than the kernel's 32-bit offsets into x take", K);
    FSIE_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "gemm_mfma_skinny_rope: head_dim %d must be a multiple of 16",
                 head_dim);
    FSIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "gemm_mfma_skinny_rope: operands must be 16-byte aligned");
    FSIE_REQUIRE(positions, "gemm_mfma_skinny_rope: no positions");
    FSIE_REQUIRE(!cos_sin || reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0,
                 "gemm_mfma_skinny_rope: the table of cosines and sines must be 8-byte aligned");
    const bool store = k_pool != nullptr;
    FSIE_REQUIRE(!store || (v_pool && slots && page_size > 0 && pool_slots > 0),
                 "gemm_mfma_skinny_rope: a cache needs both pools, slots and a page geometry");
    if (M == 0) return 0;
    const int N = (n_heads + 2 * n_kv) * head_dim;
    const int mt = (M + 15) / 16;
    const int pairs = (K + 2 * fsie_mm::kStep - 1) / (2 * fsie_mm::kStep);
    // Rotary pairs a workgroup owns: 8 (one block of 16 rows).  A product this small is bound by
    // what a compute unit's memory pipeline gives, so the busiest unit sets the time: where eight
    // pairs a workgroup would leave some units two workgroups and others one (N = 4608 on 256
    // units: 288 workgroups), the pairs are dealt evenly instead, 9 to 16 a workgroup, in two blocks
    // of which the second is partly filled.
    const int total_pairs = N / 2;
    const int units = fsie_compute_units();
    int pairs_per_wg = 8;
    // Up to 6 rows of x, a product large enough for it: two workgroups of four waves a unit, each with
    // 4 to 8 pairs (two waves a SIMD hide each other's waits; MI355X, 256 units, N = 4608, K = 3584: 5
    // pairs, 461 workgroups: 10.0 us at one row, 11.0 at four, where 8 pairs take 11.8 and 13.0 and 9
    // pairs 11.6 and 11.7; N = 7168, K = 5120: 7 pairs, 512 workgroups: 15.8 and 16.8 against 17.1 and
    // 18.6 for 8 pairs; at 8 rows 12.1 against 12.0 and 19.0 against 19.5, at 16 rows 15.6 against 12.9)
    const int two_each = units > 0 ? (total_pairs + 2 * units - 1) / (2 * units) : 0;
    const bool two_a_unit = mt == 1 && M <= 6 && units > 0 && total_pairs >= 8 * units && two_each <= 8;
    if (two_a_unit) {
        pairs_per_wg = two_each;
    } else if (mt == 1 && M > 4 && units > 0 && total_pairs > 8 * units && total_pairs <= 16 * units) {
        pairs_per_wg = (total_pairs + units - 1) / units;
    }
    const int blocks = pairs_per_wg > 8 ? 2 : 1;
    const int groups = (total_pairs + pairs_per_wg - 1) / pairs_per_wg;
    int waves = 1;
    // (more waves than this only add to the reduction: 12.6 us with four against 14.1 with eight
    // at N = 4608, K = 3584 and one row)
    while (waves < 16 && groups * waves < 1024) waves *= 2;
    if (two_a_unit) waves = 4;
    while (waves > 1 && pairs < 2 * waves) waves /= 2;
    if (mt * blocks > 4 && waves > 8) waves = 8;  // LDS of the reduction
    const fsie_mm::Call call{x, w, bias, y, M, N, K, 1, stream,
                               fsie_mm::RopeArgs{positions, slots, inv_freq, cos_sin, static_cast<bf16_t*>(store ? k_pool : nullptr),
                                                   static_cast<bf16_t*>(store ? v_pool : nullptr), n_heads, n_kv, head_dim,
                                                   store ? page_size : 1, store ? pool_slots : 0, pairs_per_wg}};
    return fsie_mm::launch_rope(mt, waves, call);
}
