// A short causal convolution over time on one channel of a step's float32 projections, shared by the
// mixers that run their projections through one (attention with convolved q/k/v, the state-space
// mixer): y_t = sum_j taps[c, j] x_(t - K + 1 + j), the last column of the taps being the current
// token's.  Inputs from before the step come from the request's tail: its last K - 1 inputs, oldest
// first, [K - 1, C] per state slot, zeros at a sequence's start.
#pragma once

#include "common.h"

namespace lc {

constexpr int SHORT_CONV_MAX_TAPS = 16;

// Channel c (column c of proj) of token t, the `local`-th token of its request in this step.
// proj [T, cols]; taps [C, K]; tail [K - 1, C] of the request's slot.
__device__ __forceinline__ float short_conv(const float* __restrict__ proj, size_t cols, int t, int local, int c,
                                            const float* __restrict__ taps, int K,
                                            const float* __restrict__ tail, int C) {
    float y = 0.f;
    for (int back = K - 1; back >= 0; --back) {       // oldest input first: the order of the sum is fixed
        const float x = back <= local ? proj[(size_t)(t - back) * cols + c]
                                      : tail[(size_t)((K - 1) - (back - local)) * C + c];
        y = fmaf(taps[(size_t)c * K + (K - 1 - back)], x, y);
    }
    return y;
}

}  // namespace lc
