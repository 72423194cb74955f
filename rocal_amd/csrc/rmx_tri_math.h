// Coordinate and coefficient law of the triangular (antialiased) resize, shared by its kernels. Every function is the
// fp32 arithmetic of the reference's device kernel, operation for operation (rocal_hip_kernels.cpp:487-589).
#pragma once
#include "rmx_device.h"

namespace rmx {

struct TriAxis {
    float ratio, radius, fscale, offset;
    int ksize;
};

RMX_DEV TriAxis tri_axis(float ratio, float fscale) {
    TriAxis t;
    t.ratio = ratio;
    t.radius = ratio > 1.0f ? ratio : 1.0f;
    t.fscale = fscale;
    t.offset = (ratio - 1) * 0.5f - t.radius;
    t.ksize = (int)ceilf(t.radius * 2);
    return t;
}

RMX_DEV void tri_loc(const TriAxis &t, int d, float lo, int &loc, float &w0) {
    float raw = (float)d * t.ratio;
    raw = raw + t.offset;
    raw = raw + lo;
    loc = (int)ceilf(raw);
    w0 = (float)loc - raw;
}

RMX_DEV float tri_coeff(float w0, float radius, int k, float fscale) {
    float c = 1 - fabsf((w0 - radius + (float)k) * fscale);
    return c < 0 ? 0 : c;
}

}  // namespace rmx
