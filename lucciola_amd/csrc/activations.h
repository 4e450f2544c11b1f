// The activations that products may apply to their sums before they store them, and that the
// element-wise kernel applies in place: one definition, so that both round alike.
#pragma once

#include "common.h"

namespace lc {

// ACT_SIGMOID_GATE: times sigmoid of the gate's entry at the output's place; ACT_SIGMOID_GROUP_GATE: times
// sigmoid of ONE gate entry per row and group (a number per token and head)
enum : int { ACT_NONE = 0, ACT_GELU_TANH = 1, ACT_RELU_SQUARED = 2, ACT_SIGMOID_GATE = 3, ACT_SIGMOID_GROUP_GATE = 4,
             ACT_XIELU = 5 };

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

// xIELU with its two numbers already through softplus: z > 0: a z^2 + z/2;  z <= 0: b (e^z - 1 - z) + z/2
// (a = softplus(p), b = 1/2 + softplus(q)).
__device__ __forceinline__ float xielu(float z, float a, float b) {
    if (z > 0.f) return fmaf(a * z, z, 0.5f * z);
    return fmaf(b, expm1f(z) - z, 0.5f * z);
}

}  // namespace lc
