// 1-D Winograd F(6,3) transforms shared by the transform kernels and the fused kernels.
#pragma once

namespace {

// ---- 1-D transforms (the matrices of winoF63ZC/winoF63ZC.cpp:28-78,
// :137-166 and :181-228, factored by common sub-expressions) ---------------

__device__ __forceinline__ void bt8(const float d[8], float o[8]) {
    o[0] = (d[0] - d[6]) + 5.25f * (d[4] - d[2]);
    o[7] = (d[7] - d[1]) + 5.25f * (d[3] - d[5]);
    const float t1 = (d[2] + d[6]) - 4.25f * d[4];
    const float t2 = (d[1] + d[5]) - 4.25f * d[3];
    o[1] = t1 + t2;
    o[2] = t1 - t2;
    const float p1 = (d[6] + 0.25f * d[2]) - 1.25f * d[4];
    const float p2 = (0.5f * d[1] - 2.5f * d[3]) + 2.0f * d[5];
    o[3] = p1 + p2;
    o[4] = p1 - p2;
    const float q1 = (d[6] + 4.0f * d[2]) - 5.0f * d[4];
    const float q2 = (2.0f * d[1] - 2.5f * d[3]) + 0.5f * d[5];
    o[5] = q1 + q2;
    o[6] = q1 - q2;
}

__device__ __forceinline__ void at6(const float m[8], float s[6]) {
    const float a = m[1] + m[2], b = m[1] - m[2];
    const float c = m[3] + m[4], d = m[3] - m[4];
    const float e = m[5] + m[6], f = m[5] - m[6];
    s[0] = (m[0] + a) + (c + 32.0f * e);
    s[1] = (b + 2.0f * d) + 16.0f * f;
    s[2] = (a + 4.0f * c) + 8.0f * e;
    s[3] = (b + 8.0f * d) + 4.0f * f;
    s[4] = (a + 16.0f * c) + 2.0f * e;
    s[5] = ((b + 32.0f * d) + f) + m[7];
}

__device__ __forceinline__ void g8(const float g[3], float w[8]) {
    const float c29 = (float)(-2.0 / 9), c90 = (float)(1.0 / 90), c180 = (float)(1.0 / 180);
    const float s02 = g[0] + g[2];
    w[0] = g[0];
    w[1] = (s02 + g[1]) * c29;
    w[2] = (s02 - g[1]) * c29;
    const float e = g[0] + 4.0f * g[2], two = 2.0f * g[1];
    w[3] = (e + two) * c90;
    w[4] = (e - two) * c90;
    const float h = g[2] + 4.0f * g[0];
    w[5] = (h + two) * c180;
    w[6] = (h - two) * c180;
    w[7] = g[2];
}

}  // namespace
