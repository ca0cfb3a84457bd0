// Instantiations of the matrix-core attention kernel for head_dim = 16 * (9 .. 12):
// one query tile per wave for decoding and short portions, 2 tiles for long portions.
#include "attention_mfma_impl.h"

namespace fsie_attn {

LaunchFn table_c(int hdt, int large) {
    switch (hdt) {
        case 9: return large ? launch<9, 2> : launch<9, 1>;
        case 10: return large ? launch<10, 2> : launch<10, 1>;
        case 11: return large ? launch<11, 2> : launch<11, 1>;
        case 12: return large ? launch<12, 2> : launch<12, 1>;
        default: return nullptr;
    }
}

LaunchQkvFn table_c_qkv(int hdt) {
    switch (hdt) {
        case 10: return launch_qkv<10>;
        case 12: return launch_qkv<12>;
        default: return nullptr;
    }
}

}  // namespace fsie_attn
