// A norm as a kernel argument: what it does to a row and with which numbers.
#pragma once

enum CelegNormMode { CELEG_NORM_NONE = 0, CELEG_NORM_RMS = 2, CELEG_NORM_LAYER = 3 };

struct CelegNorm {
    const float* w;     // [width] scale, or null
    const float* b;     // [width] bias, or null
    float eps;
    int mode;           // CelegNormMode; NONE: the row passes as it is (w and b still apply if given)
};
