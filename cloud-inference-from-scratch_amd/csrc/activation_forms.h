// Activation formulas that more than one kernel file uses.
#pragma once

#include "common.h"

// A gated unit with bounded inputs: g' = min(g, limit), u' = clamp(u, -limit, limit),
// y = g' * sigmoid(alpha * g') * (u' + offset).  float32.
__device__ __forceinline__ float clamped_glu(float g, float u, float limit, float alpha, float offset) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + offset);
}
