// Instantiations of the weight-streaming matrix-core product with bfloat16 results, plain and with
// the SiLU*up epilogue: up to 16 rows (decoding).
#include "gemm_mfma_impl.h"

namespace fsie_mm {

int launch_bf16(int blocks, int waves, const Call& c) { return launch_blocks<1, bf16_t, EPI_PLAIN>(blocks, waves, c); }

int launch_swiglu(int blocks, int waves, const Call& c) { return launch_blocks<1, bf16_t, EPI_SWIGLU>(blocks, waves, c); }

}  // namespace fsie_mm
