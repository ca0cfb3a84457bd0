// Instantiations of the matrix-core attention kernel for head_dim = 16 * (13 .. 16):
// one query tile per wave for decoding and short portions, 2 tiles for long portions.
#include "attention_mfma_impl.h"

namespace fsie_attn {

LaunchFn table_d(int hdt, int large) {
    switch (hdt) {
        case 13: return large ? launch<13, 2> : launch<13, 1>;
        case 14: return large ? launch<14, 2> : launch<14, 1>;
        case 15: return large ? launch<15, 2> : launch<15, 1>;
        case 16: return large ? launch<16, 2> : launch<16, 1>;
        default: return nullptr;
    }
}

LaunchQkvFn table_d_qkv(int hdt) {
    switch (hdt) {
        case 14: return launch_qkv<14>;
        case 16: return launch_qkv<16>;
        default: return nullptr;
    }
}

}  // namespace fsie_attn
