// The activations that products may apply to their sums before they store them, and that the
// element-wise kernel applies in place: one definition, so that both round alike.
#pragma once

#include "common.h"

namespace lc {

enum : int { ACT_NONE = 0, ACT_GELU_TANH = 1, ACT_RELU_SQUARED = 2, ACT_SIGMOID_GATE = 3 };

__device__ __forceinline__ float activate(float z, int kind) {
    if (kind == ACT_GELU_TANH) {
        const float inner = 0.7978845608028654f * fmaf(0.044715f * z, z * z, z);   // sqrt(2/pi) (z + 0.044715 z^3)
        return 0.5f * z * (1.f + tanhf(inner));
    }
    if (kind == ACT_RELU_SQUARED) {
        const float r = fmaxf(z, 0.f);
        return r * r;
    }
    return z;
}

__device__ __forceinline__ float sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

}  // namespace lc
