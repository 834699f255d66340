// Real spherical-harmonic basis of degree <= 5 at one direction, shared by the kernels that evaluate it.
#pragma once
#include "common.h"

namespace pmesh {

// v[0 .. (L+1)^2) = basis values at the direction of (x, y, z), in the reference's ordering
// (picasso/math_utils.py:16-59): cartesian closed forms on the unit vector.  The normalisation is scale-free;
// the zero vector evaluates at (1, 0, 0) like atan2(0, 0) = 0 does.
__device__ __forceinline__ void sph_harm_at(float x, float y, float z, int L, float *v)
{
    // scale-free normalisation; the zero vector evaluates at (1,0,0) like atan2(0,0) = 0 does
    const float mx = fmaxf(fabsf(x), fmaxf(fabsf(y), fabsf(z)));
    if (mx > 0.f && mx < INFINITY) {
        x /= mx; y /= mx; z /= mx;
        const float inv = 1.0f / sqrtf(x * x + y * y + z * z);
        x *= inv; y *= inv; z *= inv;
    } else {
        x = 1.f; y = 0.f; z = 0.f;
    }
    const float PI = 3.14159265358979323846f;
    const float x2 = x * x, y2 = y * y, z2 = z * z, xy = x * y;
    const float c2 = x2 - y2, s2 = 2.f * xy;                      // sin^2(th) cos/sin(2 phi)
    const float c3 = x * (x2 - 3.f * y2), s3 = y * (3.f * x2 - y2);  // sin^3(th) cos/sin(3 phi)
    v[0] = 0.5f * sqrtf(1.f / PI);
    if (L >= 1) {
        const float a = 0.5f * sqrtf(1.5f / PI);
        v[1] = a * x; v[2] = 0.5f * sqrtf(3.f / PI) * z; v[3] = a * y;
    }
    if (L >= 2) {
        const float a = 0.25f * sqrtf(7.5f / PI), b = 0.5f * sqrtf(7.5f / PI);
        v[4] = a * c2; v[5] = b * x * z; v[6] = 0.25f * sqrtf(5.f / PI) * (3.f * z2 - 1.f);
        v[7] = a * s2; v[8] = b * y * z;
    }
    if (L >= 3) {
        const float a = 0.125f * sqrtf(35.f / PI), b = 0.25f * sqrtf(52.5f / PI), d = 0.125f * sqrtf(21.f / PI);
        const float t = 5.f * z2 - 1.f;
        v[9] = a * c3; v[10] = b * z * c2; v[11] = d * x * t;
        v[12] = 0.25f * sqrtf(7.f / PI) * z * (5.f * z2 - 3.f);
        v[13] = a * s3; v[14] = b * z * s2; v[15] = d * y * t;
    }
    if (L >= 4) {
        const float c4 = x2 * x2 - 6.f * x2 * y2 + y2 * y2, s4 = 4.f * xy * c2;
        const float a = 0.1875f * sqrtf(17.5f / PI), b = 0.375f * sqrtf(35.f / PI);
        const float d = 0.375f * sqrtf(2.5f / PI), e = 0.375f * sqrtf(5.f / PI);
        const float t2 = 7.f * z2 - 1.f, t1 = z * (7.f * z2 - 3.f);
        v[16] = a * c4; v[17] = b * z * c3; v[18] = d * c2 * t2; v[19] = e * x * t1;
        v[20] = 0.1875f * sqrtf(1.f / PI) * (35.f * z2 * z2 - 30.f * z2 + 3.f);
        v[21] = a * s4; v[22] = b * z * s3; v[23] = d * s2 * t2; v[24] = e * y * t1;
    }
    if (L >= 5) {
        const float c4 = x2 * x2 - 6.f * x2 * y2 + y2 * y2, s4 = 4.f * xy * c2;
        const float c5 = x * (x2 * x2 - 10.f * x2 * y2 + 5.f * y2 * y2);
        const float s5 = y * (5.f * x2 * x2 - 10.f * x2 * y2 + y2 * y2);
        const float a = 0.09375f * sqrtf(77.f / PI), b = 0.1875f * sqrtf(192.5f / PI);
        const float d = 0.03125f * sqrtf(385.f / PI), e = 0.125f * sqrtf(577.5f / PI);
        const float g = 0.0625f * sqrtf(82.5f / PI);
        const float t3 = 9.f * z2 - 1.f, t2 = z * (3.f * z2 - 1.f), t1 = 21.f * z2 * z2 - 14.f * z2 + 1.f;
        v[25] = a * c5; v[26] = b * z * c4; v[27] = d * c3 * t3; v[28] = e * c2 * t2; v[29] = g * x * t1;
        v[30] = 0.0625f * sqrtf(11.f / PI) * z * (63.f * z2 * z2 - 70.f * z2 + 15.f);
        v[31] = a * s5; v[32] = b * z * s4; v[33] = d * s3 * t3; v[34] = e * s2 * t2; v[35] = g * y * t1;
    }
}

// The (L + 1)^2 basis values of a point to memory, degree by degree with compile-time indices: a copy loop over a
// run-time count would index the value array dynamically and push it out of the registers into private memory.
template <int D>
__device__ __forceinline__ void sph_store_degree(float *o, const float (&v)[36])
{
#pragma unroll
    for (int i = D * D; i < (D + 1) * (D + 1); ++i) o[i] = v[i];
}

__device__ __forceinline__ void sph_store(float *o, const float (&v)[36], int L)
{
    sph_store_degree<0>(o, v);
    if (L >= 1) sph_store_degree<1>(o, v);
    if (L >= 2) sph_store_degree<2>(o, v);
    if (L >= 3) sph_store_degree<3>(o, v);
    if (L >= 4) sph_store_degree<4>(o, v);
    if (L >= 5) sph_store_degree<5>(o, v);
}

}  // namespace pmesh
