// Shared host/device helpers of libpicasso_mesh (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <initializer_list>

namespace pmesh {

constexpr int kWave = 64;
constexpr int kBlock = 256;  // threads per workgroup of the row kernels (4 wavefronts)

// Error plumbing: fail() formats into a thread-local buffer and returns a non-zero code.
int fail(const char *fmt, ...);
void clear_error();

#define PM_REQUIRE(cond, ...)                       \
    do {                                            \
        if (!(cond)) return ::pmesh::fail(__VA_ARGS__); \
    } while (0)

#define PM_LAUNCHED(name)                                                              \
    do {                                                                               \
        hipError_t e__ = hipGetLastError();                                            \
        if (e__ != hipSuccess)                                                         \
            return ::pmesh::fail("%s: kernel launch failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

// Switches that route an op to another kernel family than the default (tests compare the families; benchmarks time
// the variants).  Read from the environment ONCE, at the first call into the library, and again only when
// pmesh_reload_options() is called: PMESH_F2F_GENERIC, PMESH_F2F_BF16X3, PMESH_F2F_HALF, PMESH_F2V_VALU,
// PMESH_DENSE_FP32MFMA (each "1" to set).
struct Options {
    bool f2f_generic;        // facet2facet on the shape-generic fp32-MFMA kernels
    bool f2f_bf16x3;         // 16 coefficients: the three-piece bf16 kernels instead of the two-piece fp16 ones
    bool f2f_half;           // 16 coefficients: one fp16 piece per operand (results within 1e-3)
    bool f2v_valu;           // facet2vertex on the vector-ALU kernels
    bool f2v_fp32mfma;       // facet2vertex forward: the filter combination on the fp32 matrix instruction instead of split fp16
    bool point_conv_two_passes;   // point convolution backward: input and filter gradient as separate passes
    bool dense_fp32mfma;     // pointwise tail on the fp32 matrix instruction
};
const Options &options();

// Every index the kernels compute must fit int32 element counts times channels in int64;
// grids are 1-D and must stay below 2^31 workgroups.
inline bool grid_ok(int64_t blocks) { return blocks >= 0 && blocks < (int64_t(1) << 31); }

// How one feature row of `n_items` vector items is spread over the lanes of a workgroup:
// a power-of-two group of `lpr` lanes owns one row, kBlock/lpr rows are in flight per
// workgroup, a group loops when the row has more items than lanes.
struct RowShape {
    int items;     // vector items per row (channels / V)
    int lpr;       // lanes per row, power of two in [1, kBlock]
    int lpr_log2;
    int rpb;       // rows per workgroup = kBlock / lpr
};

inline RowShape row_shape(int items)
{
    RowShape s;
    s.items = items;
    s.lpr_log2 = 0;
    while ((1 << s.lpr_log2) < items && (1 << s.lpr_log2) < kBlock) ++s.lpr_log2;
    s.lpr = 1 << s.lpr_log2;
    s.rpb = kBlock / s.lpr;
    return s;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of persistent workgroups of a reduction kernel that also accumulates filter
// gradients: a function of the problem only (never of the device), so that the summation
// order -- and with it every output bit -- is the same on any GPU.
inline int persistent_blocks(int64_t rows, int rows_per_block)
{
    int64_t b = ceil_div(rows, int64_t(rows_per_block) * 8);
    if (b < 1) b = 1;
    if (b > 1024) b = 1024;
    return int(b);
}

#ifdef __HIPCC__
// V consecutive floats as registers; V = 4 moves 16 bytes per lane per access.
template <int V> struct Pack { float v[V]; };

template <int V> __device__ __forceinline__ Pack<V> ldp(const float *p)
{
    Pack<V> r;
    if constexpr (V == 4) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else if constexpr (V == 2) {
        const float2 t = *reinterpret_cast<const float2 *>(p);
        r.v[0] = t.x; r.v[1] = t.y;
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) r.v[i] = p[i];
    }
    return r;
}

template <int V> __device__ __forceinline__ void stp(float *p, const Pack<V> &r)
{
    if constexpr (V == 4) {
        *reinterpret_cast<float4 *>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
    } else if constexpr (V == 2) {
        *reinterpret_cast<float2 *>(p) = make_float2(r.v[0], r.v[1]);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) p[i] = r.v[i];
    }
}

template <int V> __device__ __forceinline__ Pack<V> zero_pack()
{
    Pack<V> r;
#pragma unroll
    for (int i = 0; i < V; ++i) r.v[i] = 0.f;
    return r;
}
#endif  // __HIPCC__

}  // namespace pmesh
