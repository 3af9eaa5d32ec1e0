// The gated activation of one element as the stand-alone Op::GatedAct evaluates it (act_fn and
// gated_act_fn, crates/infr-cpu/src/kernels.rs:6578-6597): shared by that kernel and by the
// small-batch quantizer when a plan folds the op into it.
#pragma once

#include "device_common.hpp"

namespace infr {

__device__ __forceinline__ float act_fn(int act, float g) {
    switch (act) {
    case 1: return 0.5f * g * (1.0f + tanhf(0.7978846f * (g + 0.044715f * g * g * g)));
    case 2: return 1.0f / (1.0f + expf(-g));
    default: return g / (1.0f + expf(-g));
    }
}

__device__ __forceinline__ float gated_act_fn(int act, bool has_clamp, float l, float gate, float up) {
    if (has_clamp) {
        gate = gate < l ? gate : l;
        up = up < -l ? -l : (up > l ? l : up);
    }
    return act_fn(act, gate) * up;
}

}  // namespace infr
