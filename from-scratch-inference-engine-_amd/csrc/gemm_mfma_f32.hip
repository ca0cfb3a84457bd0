// Instantiations of the weight-streaming matrix-core product with float32 results (logits, partial
// sums of a cut inner dimension): up to 64 rows.
#include "gemm_mfma_impl.h"

namespace fsie_mm {

int launch_f32(int mt, int blocks, int waves, const Call& c) {
    switch (mt) {
        case 1: return launch_blocks<1, float, EPI_PLAIN>(blocks, waves, c);
        case 2: return launch_blocks<2, float, EPI_PLAIN>(blocks, waves, c);
        case 3: return launch_blocks<3, float, EPI_PLAIN>(blocks, waves, c);
        default: return launch_blocks<4, float, EPI_PLAIN>(blocks, waves, c);
    }
}

}  // namespace fsie_mm
