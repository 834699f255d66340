// Fp32-accurate products on the fp16 matrix cores: an operand is split into two fp16 pieces (both rounded to nearest,
// x = x1 + x2 + e with |e| <= 2^-23 |x|), a product is the sum of three piece products accumulated in fp32, and an
// exact power-of-two scale keeps the operand inside fp16's range.  Shared by the facet2facet and facet2vertex kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace pmesh {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Eight fp32 values -> two packed fp16x8 pieces, both rounded to nearest; the remainder x - x1 is exact in
// fp32.  Written out as instructions: left to the compiler, the FMA that produced x may be folded into ONE of
// the two conversions of x1 it emits (a mixed-precision FMA rounds the exact product once), and in a near-tie
// the piece that is multiplied and the piece the remainder was taken from then differ by one fp16 ulp.
__device__ __forceinline__ void split8h(const float (&x)[8], u32x4 &p1, u32x4 &p2)
{
    const float neg1 = -1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // hi = {f16(a), f16(b)};  ra = a - hi.lo, rb = b - hi.hi (mixed-precision FMAs reading one half of hi
        // each, exact);  lo = {f16(ra), f16(rb)}: four instructions per pair
        unsigned hi, lo;
        float ra, rb;
        asm("v_cvt_pk_f16_f32 %0, %4, %5\n\t"
            "s_nop 0\n\t"
            "v_fma_mix_f32 %1, %0, %6, %4 op_sel:[0,0,0] op_sel_hi:[1,0,0]\n\t"
            "v_fma_mix_f32 %2, %0, %6, %5 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
            "v_cvt_pk_f16_f32 %3, %1, %2"
            : "=&v"(hi), "=&v"(ra), "=&v"(rb), "=&v"(lo)
            : "v"(x[2 * j]), "v"(x[2 * j + 1]), "v"(neg1));
        p1[j] = hi;
        p2[j] = lo;
    }
}

__device__ __forceinline__ f32x16 mfma_f16(const u32x4 &a, const u32x4 &b, const f32x16 &c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Maxima over the wavefront without a trip through LDS: four data-parallel-primitive steps leave the maximum of each
// row of 16 lanes in all of its lanes (lane ^ 1, lane ^ 2, mirror of 8, mirror of 16), one lane of each row is read
// into a scalar register.  All 64 lanes must be active.
template <int CTRL> __device__ __forceinline__ int hdpp(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
__device__ __forceinline__ int hrow_max(int v)
{
    int t;
    t = hdpp<0xB1>(v); v = t > v ? t : v;
    t = hdpp<0x4E>(v); v = t > v ? t : v;
    t = hdpp<0x141>(v); v = t > v ? t : v;
    t = hdpp<0x140>(v); v = t > v ? t : v;
    return v;
}
__device__ __forceinline__ int hwave_max(int v)
{
    v = hrow_max(v);
    const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    const int ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}
__device__ __forceinline__ float hrow_fmax(float m)
{
    m = fmaxf(m, __builtin_bit_cast(float, hdpp<0xB1>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, hdpp<0x4E>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, hdpp<0x141>(__builtin_bit_cast(int, m))));
    m = fmaxf(m, __builtin_bit_cast(float, hdpp<0x140>(__builtin_bit_cast(int, m))));
    return m;
}
__device__ __forceinline__ float hwave_fmax(float m)
{
    const int v = __builtin_bit_cast(int, hrow_fmax(m));
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(v, 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(v, 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(v, 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(v, 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Power of two s with s * m < 2^14 for a bound m >= 0 (s = 1 for m = 0 or non-finite m); *inv = 1 / s.
__device__ __forceinline__ float pow2_scale(float m, float *inv)
{
    int e = (int)((__builtin_bit_cast(unsigned, m) >> 23) & 0xFFu);      // biased exponent: m < 2^(e - 126)
    if (e == 0 || e == 255) { *inv = 1.0f; return 1.0f; }
    e = e < 40 ? 40 : (e > 215 ? 215 : e);                                // keep both s and 1/s normal numbers
    *inv = __builtin_bit_cast(float, (unsigned)(e - 13) << 23);           // 2^(e - 140)
    return __builtin_bit_cast(float, (unsigned)(267 - e) << 23);          // 2^(140 - e):  s * m < 2^14
}

}  // namespace pmesh
