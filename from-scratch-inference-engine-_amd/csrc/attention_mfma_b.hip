// Instantiations of the matrix-core attention kernel for head_dim = 16 * (5 .. 8):
// one query tile per wave for decoding and short portions, 4 tiles for long portions.
#include "attention_mfma_impl.h"

namespace fsie_attn {

LaunchFn table_b(int hdt, int large) {
    switch (hdt) {
        case 5: return large ? launch<5, 2> : launch<5, 1>;
        case 6: return large ? launch<6, 2> : launch<6, 1>;
        case 7: return large ? launch<7, 2> : launch<7, 1>;
        case 8: return large ? launch<8, 2> : launch<8, 1>;
        default: return nullptr;
    }
}

LaunchQkvFn table_b_qkv(int hdt) {
    switch (hdt) {
        case 6: return launch_qkv<6>;
        case 8: return launch_qkv<8>;
        default: return nullptr;
    }
}

}  // namespace fsie_attn
