// Instantiations of the matrix-core attention kernel for head_dim = 16 * (1 .. 4):
// one query tile per wave for decoding and short portions, 4 tiles for long portions.
#include "attention_mfma_impl.h"

namespace fsie_attn {

LaunchFn table_a(int hdt, int large) {
    switch (hdt) {
        case 1: return large ? launch<1, 2> : launch<1, 1>;
        case 2: return large ? launch<2, 2> : launch<2, 1>;
        case 3: return large ? launch<3, 2> : launch<3, 1>;
        case 4: return large ? launch<4, 2> : launch<4, 1>;
        default: return nullptr;
    }
}

LaunchQkvFn table_a_qkv(int hdt) {
    switch (hdt) {
        case 2: return launch_qkv<2>;
        case 4: return launch_qkv<4>;
        default: return nullptr;
    }
}

}  // namespace fsie_attn
