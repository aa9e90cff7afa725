// Activation formulas that more than one kernel file uses.
#pragma once

#include "common.h"

// A gated unit with bounded inputs: g' = min(g, limit), u' = clamp(u, -limit, limit),
// y = g' * sigmoid(alpha * (g' + cubic * g'^3)) * (u' + offset).  float32.  cubic = 0 is the plain sigmoid gate;
// alpha = 2 sqrt(2 / pi), cubic = 0.044715 is the tanh form of gelu, 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))),
// since 0.5 (1 + tanh z) = sigmoid(2 z).
__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha, float offset, float cubic = 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    const float inner = cubic != 0.f ? fmaf(cubic * g * g, g, g) : g;
    return g / (1.0f + expf(-alpha * inner)) * (u + offset);
}
