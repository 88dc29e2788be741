// Activation functions of the feed-forward block, shared by the kernels that fuse them.
#pragma once
#include "ojk_common.h"

// ACT 0 = SiLU  g / (1 + exp(-g))  (crates/ojas-cpu/src/cpu_math.rs:486), 1 = GELU, tanh form (:497-501).
__device__ __forceinline__ float ffn_act(float g, uint act) {
    if (act == 1u) {
        const float c = 0.7978845608028654f, a = 0.044715f;
        return 0.5f * g * (1.0f + tanhf(c * g * (1.0f + a * g * g)));
    }
    return g / (1.0f + expf(-g));
}
