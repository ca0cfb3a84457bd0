// Instantiations of the weight-streaming matrix-core product with the q/k/v + rotary + cache-write
// epilogue: one block of 16 rows of W per workgroup (two for up to 16 rows of x, where the host
// spreads the rows over the compute units), up to 64 rows of x.
#include "gemm_mfma_impl.h"

namespace fsie_mm {

int launch_rope(int mt, int waves, const Call& c) {
    if (c.rope.pairs_per_wg > 8) return launch_waves<1, 2, bf16_t, EPI_ROPE>(waves, c);  // the host asks this for mt == 1 only
    switch (mt) {
        case 1: return launch_waves<1, 1, bf16_t, EPI_ROPE>(waves, c);
        case 2: return launch_waves<2, 1, bf16_t, EPI_ROPE>(waves, c);
        case 3: return launch_waves<3, 1, bf16_t, EPI_ROPE>(waves, c);
        default: return launch_waves<4, 1, bf16_t, EPI_ROPE>(waves, c);
    }
}

}  // namespace fsie_mm
