// A norm as a kernel argument: what it does to a row and with which numbers.
#pragma once

enum CelegNormMode { CELEG_NORM_NONE = 0, CELEG_NORM_RMS = 2, CELEG_NORM_LAYER = 3, CELEG_NORM_TANH = 4 };

struct CelegNorm {
    const float* w;     // [width] scale, or null
    const float* b;     // [width] bias, or null
    float eps;
    int mode;           // CelegNormMode; NONE: the row passes as it is (w and b still apply if given);
                        // TANH: no statistics, every value becomes tanh(alpha * x) before w and b
    float alpha;        // TANH only
    float gain;         // what the normed row is multiplied by as a whole (after w and b)
};
