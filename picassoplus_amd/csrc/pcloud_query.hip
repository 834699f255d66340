// Point-cloud branch, part 1: neighbour queries, farthest point sampling and the kernel-bin builders
// (picasso/point/pi_modules/source/nnquery_gpu.cu, sample_gpu.cu, buildkernel_gpu.cu).
//
// The reference runs every query kernel with ONE workgroup per batch sample (its threads walk the sample's queries,
// each scanning the whole sample).  Here a query is a thread of a chip-wide grid: it finds its sample in the running
// totals and scans that sample's database points, which all lanes of a wavefront read at the same address.  The
// outputs are the reference's: neighbours of a query in ascending database order, the first nn_sample of them.
// Distances are compared in float32 with every operation rounded on its own (no fused multiply-add), so the integer
// outputs do not depend on how a compiler contracts the expression.
#include "common.h"
#include "../../include/picasso_mesh.h"
#include <cmath>

namespace pmesh {

struct SampleRange {
    int q0, d0, d1;      // first query of the sample, its database range
};

// sample of query j: the first b with j < nv_query[b] (inclusive running totals)
__device__ __forceinline__ bool sample_of(int64_t j, const int *__restrict__ nvq, const int *__restrict__ nvd, int B, SampleRange &s)
{
    int b = 0;
    while (b < B && j >= nvq[b]) ++b;
    if (b >= B) return false;
    s.q0 = b ? nvq[b - 1] : 0;
    s.d0 = b ? nvd[b - 1] : 0;
    s.d1 = nvd[b];
    return true;
}

__device__ __forceinline__ float sq_dist(float qx, float qy, float qz, const float *__restrict__ p, float &dx, float &dy, float &dz)
{
#pragma clang fp contract(off)
    dx = p[0] - qx;
    dy = p[1] - qy;
    dz = p[2] - qz;
    return (dx * dx + dy * dy) + dz * dz;
}

// MODE 0: sphere (sqrt(d2) < size), 1: cube (|dx|, |dy|, |dz| < size / 2)
template <int MODE> __device__ __forceinline__ bool is_neighbour(float d2, float dx, float dy, float dz, float size)
{
#pragma clang fp contract(off)
    if constexpr (MODE == 0) return sqrtf(d2) < size;
    const float half = size / 2;
    return fabsf(dx) < half && fabsf(dy) < half && fabsf(dz) < half;
}

// count[j] = min(nn_sample, number of neighbours of query j)
template <int MODE>
__global__ __launch_bounds__(kBlock) void point_count_k(const float *__restrict__ db, const float *__restrict__ query,
                                                        const int *__restrict__ nvd, const int *__restrict__ nvq, int B,
                                                        int64_t Np, int64_t Mp, float size, int nn_sample, int *__restrict__ count)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= Mp) return;
    SampleRange s;
    int cnt = 0;
    if (sample_of(j, nvq, nvd, B, s)) {
        const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
        const int64_t d1 = s.d1 < Np ? s.d1 : Np;
        for (int64_t k = s.d0; k < d1 && cnt < nn_sample; ++k) {
            float dx, dy, dz;
            const float d2 = sq_dist(qx, qy, qz, db + k * 3, dx, dy, dz);
            cnt += is_neighbour<MODE>(d2, dx, dy, dz, size) ? 1 : 0;
        }
    }
    count[j] = cnt;
}

// pairs of query j at [cnt_info[j-1], cnt_info[j]): (query, database point[, cell of the cube grid]); sphere: distances
template <int MODE>
__global__ __launch_bounds__(kBlock) void point_fill_k(const float *__restrict__ db, const float *__restrict__ query,
                                                       const int *__restrict__ nvd, const int *__restrict__ nvq, int B,
                                                       int64_t Np, int64_t Mp, float size, int grid_size,
                                                       const int64_t *__restrict__ cnt_info, int64_t Nout,
                                                       int *__restrict__ nn_index, float *__restrict__ nn_dist)
{
#pragma clang fp contract(off)
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= Mp) return;
    SampleRange s;
    if (!sample_of(j, nvq, nvd, B, s)) return;
    int64_t at = j ? cnt_info[j - 1] : 0, end = cnt_info[j];
    if (at < 0) at = 0;
    if (end > Nout) end = Nout;
    const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
    const int64_t d1 = s.d1 < Np ? s.d1 : Np;
    for (int64_t k = s.d0; k < d1 && at < end; ++k) {
        float dx, dy, dz;
        const float d2 = sq_dist(qx, qy, qz, db + k * 3, dx, dy, dz);
        if (!is_neighbour<MODE>(d2, dx, dy, dz, size)) continue;
        if constexpr (MODE == 0) {
            nn_index[at * 2] = (int)j;
            nn_index[at * 2 + 1] = (int)k;
            nn_dist[at] = sqrtf(d2);
        } else {
            const float half = size / 2, cell = size / (float)grid_size;
            const int xi = (int)((dx + half) / cell), yi = (int)((dy + half) / cell), zi = (int)((dz + half) / cell);
            nn_index[at * 3] = (int)j;
            nn_index[at * 3 + 1] = (int)k;
            nn_index[at * 3 + 2] = (xi * grid_size + yi) * grid_size + zi;
        }
        ++at;
    }
}

// the three nearest database points of the query's sample; an earlier point wins a tie
__global__ __launch_bounds__(kBlock) void point_knn3_k(const float *__restrict__ db, const float *__restrict__ query,
                                                       const int *__restrict__ nvd, const int *__restrict__ nvq, int B,
                                                       int64_t Np, int64_t Mp, int *__restrict__ nn_index, float *__restrict__ nn_dist)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= Mp) return;
    SampleRange s;
    if (!sample_of(j, nvq, nvd, B, s)) {
        for (int i = 0; i < 3; ++i) { nn_index[j * 3 + i] = 0; nn_dist[j * 3 + i] = INFINITY; }
        return;
    }
    const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
    float b1 = INFINITY, b2 = INFINITY, b3 = INFINITY;
    int i1 = s.d0, i2 = s.d0, i3 = s.d0;
    const int64_t d1 = s.d1 < Np ? s.d1 : Np;
    for (int64_t k = s.d0; k < d1; ++k) {
        float dx, dy, dz;
        const float d2 = sq_dist(qx, qy, qz, db + k * 3, dx, dy, dz);
        if (d2 < b1) { b3 = b2; i3 = i2; b2 = b1; i2 = i1; b1 = d2; i1 = (int)k; }
        else if (d2 < b2) { b3 = b2; i3 = i2; b2 = d2; i2 = (int)k; }
        else if (d2 < b3) { b3 = d2; i3 = (int)k; }
    }
    nn_index[j * 3] = i1; nn_index[j * 3 + 1] = i2; nn_index[j * 3 + 2] = i3;
    nn_dist[j * 3] = sqrtf(b1); nn_dist[j * 3 + 1] = sqrtf(b2); nn_dist[j * 3 + 2] = sqrtf(b3);
}

// Farthest point sampling: one workgroup of 1024 threads per sample.  temp[k] = squared distance of point k to the
// chosen set; every round updates it against the last chosen point and takes the arg-max (lowest index among equals).
constexpr int kFpsThreads = 1024;
__global__ __launch_bounds__(kFpsThreads) void point_fps_k(const float *__restrict__ xyz, const int *__restrict__ nv_in,
                                                           const int *__restrict__ nv_out, int B, int64_t Np, int64_t Mp,
                                                           float *__restrict__ temp, int *__restrict__ index_out)
{
#pragma clang fp contract(off)
    __shared__ float s_best[kFpsThreads / 64];
    __shared__ int s_idx[kFpsThreads / 64];
    __shared__ int s_cur;
    const int b = blockIdx.x;
    if (b >= B) return;
    const int n0 = b ? nv_in[b - 1] : 0, n1 = nv_in[b] < Np ? nv_in[b] : (int)Np;
    const int m0 = b ? nv_out[b - 1] : 0, m1 = nv_out[b] < Mp ? nv_out[b] : (int)Mp;
    const int N = n1 - n0, M = m1 - m0;
    if (M <= 0) return;
    for (int k = threadIdx.x; k < N; k += kFpsThreads) temp[n0 + k] = 1e38f;
    int cur = n0;
    if (threadIdx.x == 0) index_out[m0] = N > 0 ? n0 : 0;
    if (N <= 0) {
        for (int j = 1 + threadIdx.x; j < M; j += kFpsThreads) index_out[m0 + j] = 0;
        return;
    }
    __syncthreads();
    for (int j = 1; j < M; ++j) {
        const float x1 = xyz[(int64_t)cur * 3], y1 = xyz[(int64_t)cur * 3 + 1], z1 = xyz[(int64_t)cur * 3 + 2];
        float best = -1.f;
        int besti = n0;
        for (int k = threadIdx.x; k < N; k += kFpsThreads) {
            const float *p = xyz + (int64_t)(n0 + k) * 3;
            const float dx = p[0] - x1, dy = p[1] - y1, dz = p[2] - z1;
            const float d = (dx * dx + dy * dy) + dz * dz;
            const float td = temp[n0 + k];
            const float d2 = d < td ? d : td;
            if (d2 != td) temp[n0 + k] = d2;
            if (d2 > best) { best = d2; besti = n0 + k; }
        }
        // arg-max over the workgroup: larger value, then lower index
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(besti, o, 64);
            if (ob > best || (ob == best && oi < besti)) { best = ob; besti = oi; }
        }
        if ((threadIdx.x & 63) == 0) { s_best[threadIdx.x >> 6] = best; s_idx[threadIdx.x >> 6] = besti; }
        __syncthreads();
        if (threadIdx.x == 0) {
            float bb = s_best[0];
            int bi = s_idx[0];
            for (int w = 1; w < kFpsThreads / 64; ++w)
                if (s_best[w] > bb || (s_best[w] == bb && s_idx[w] < bi)) { bb = s_best[w]; bi = s_idx[w]; }
            s_cur = bi;
            index_out[m0 + j] = bi;
        }
        __syncthreads();
        cur = s_cur;
    }
}

// continuous bin coordinates of a neighbour pair in an (n azimuth, p elevation, q radial) spherical kernel
struct BinCoord {
    float alpha, beta, gamma, dist;
};
__device__ __forceinline__ BinCoord bin_coord(const float *__restrict__ db, const float *__restrict__ query,
                                              const int *__restrict__ nn_index, const float *__restrict__ nn_dist, int64_t pair,
                                              int64_t Np, int64_t Mp, int n, int p, int q, float radius)
{
    const float kPi = 3.14159265358979323846f;
    int o = nn_index[pair * 2], i = nn_index[pair * 2 + 1];
    o = o < 0 ? 0 : (o >= Mp ? (int)Mp - 1 : o);
    i = i < 0 ? 0 : (i >= Np ? (int)Np - 1 : i);
    const float dx = db[(int64_t)i * 3] - query[(int64_t)o * 3], dy = db[(int64_t)i * 3 + 1] - query[(int64_t)o * 3 + 1],
                dz = db[(int64_t)i * 3 + 2] - query[(int64_t)o * 3 + 2];
    BinCoord c;
    c.dist = nn_dist[pair];
    const float d2 = sqrtf(dx * dx + dy * dy);
    float theta = atan2f(dy, dx), phi = atan2f(dz, d2);
    theta = theta < kPi ? theta : -kPi;
    theta = theta > -kPi ? theta : -kPi;
    theta += kPi;
    phi = phi < kPi / 2 ? phi : kPi / 2;
    phi = phi > -kPi / 2 ? phi : -kPi / 2;
    phi += kPi / 2;
    c.alpha = theta * (float)n / 2 / kPi;
    c.beta = phi * (float)p / kPi;
    c.gamma = c.dist * (float)q / radius;
    return c;
}
__device__ __forceinline__ int clamp_bin(float v, int n)
{
    const int i = (int)v;
    return i < n - 1 ? (i < 0 ? 0 : i) : n - 1;
}

__global__ __launch_bounds__(kBlock) void point_sph3d_k(const float *__restrict__ db, const float *__restrict__ query,
                                                        const int *__restrict__ nn_index, const float *__restrict__ nn_dist,
                                                        int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q, float radius,
                                                        int *__restrict__ filt_index)
{
    const int64_t pair = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (pair >= Nout) return;
    const BinCoord c = bin_coord(db, query, nn_index, nn_dist, pair, Np, Mp, n, p, q, radius);
    int f = 0;
    if ((double)c.dist > 0.3 * (double)radius)
        f = clamp_bin(c.gamma, q) * p * n + clamp_bin(c.beta, p) * n + clamp_bin(c.alpha, n) + 1;
    filt_index[pair] = f;
}

__global__ __launch_bounds__(kBlock) void point_fuzzy_sph3d_k(const float *__restrict__ db, const float *__restrict__ query,
                                                              const int *__restrict__ nn_index, const float *__restrict__ nn_dist,
                                                              int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q, float radius,
                                                              int *__restrict__ filt_index, float *__restrict__ filt_coeff)
{
    const int64_t pair = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (pair >= Nout) return;
    const BinCoord c = bin_coord(db, query, nn_index, nn_dist, pair, Np, Mp, n, p, q, radius);
    const float self = fmaxf(0.f, 1.f - c.dist / radius);
    const int ni = clamp_bin(c.alpha, n), p0 = clamp_bin(c.beta, p), qi = clamp_bin(c.gamma, q);
    const float b0 = c.beta - (float)p0;
    const int p1 = b0 < 0.5f ? (p0 - 1 > 0 ? p0 - 1 : 0) : (p0 + 1 < p - 1 ? p0 + 1 : p - 1);
    const bool single = p0 == p1;
    const float w1 = single ? 0.f : fabsf(b0 - 0.5f), w0 = 1.f - w1;
    filt_index[pair * 3] = 0;
    filt_coeff[pair * 3] = self;
    filt_index[pair * 3 + 1] = qi * p * n + p0 * n + ni + 1;
    filt_coeff[pair * 3 + 1] = w0 * (1.f - self);
    filt_index[pair * 3 + 2] = single ? 0 : qi * p * n + p1 * n + ni + 1;
    filt_coeff[pair * 3 + 2] = single ? 0.f : w1 * (1.f - self);
}

}  // namespace pmesh

using namespace pmesh;

#define PM_QUERY_DIMS(name)                                                                                             \
    PM_REQUIRE(B >= 0 && Np >= 0 && Mp >= 0 && Np <= INT32_MAX && Mp <= INT32_MAX, name ": bad sizes");                 \
    if (Mp == 0) return 0;                                                                                              \
    PM_REQUIRE(database && query && nv_database && nv_query, name ": null pointer");                                    \
    PM_REQUIRE(grid_ok(ceil_div(Mp, kBlock)), name ": grid too large")

extern "C" int pmesh_point_range_count(const float *database, const float *query, const int32_t *nv_database,
                                       const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float radius, int nn_sample,
                                       int32_t *count, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(radius > 0 && nn_sample > 0, "point_range_count: radius and nn_sample must be positive");
    PM_QUERY_DIMS("point_range_count");
    PM_REQUIRE(count, "point_range_count: null pointer");
    point_count_k<0><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        database, query, nv_database, nv_query, B, Np, Mp, radius, nn_sample, count);
    PM_LAUNCHED("point_range_count");
    return 0;
}

extern "C" int pmesh_point_range_fill(const float *database, const float *query, const int32_t *nv_database,
                                      const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float radius, const int64_t *cnt_info,
                                      int64_t Nout, int32_t *nn_index, float *nn_dist, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(radius > 0 && Nout >= 0, "point_range_fill: bad arguments");
    PM_QUERY_DIMS("point_range_fill");
    if (Nout == 0) return 0;
    PM_REQUIRE(cnt_info && nn_index && nn_dist, "point_range_fill: null pointer");
    point_fill_k<0><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        database, query, nv_database, nv_query, B, Np, Mp, radius, 1, cnt_info, Nout, nn_index, nn_dist);
    PM_LAUNCHED("point_range_fill");
    return 0;
}

extern "C" int pmesh_point_cube_count(const float *database, const float *query, const int32_t *nv_database,
                                      const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float length, int nn_sample,
                                      int32_t *count, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(length > 0 && nn_sample > 0, "point_cube_count: length and nn_sample must be positive");
    PM_QUERY_DIMS("point_cube_count");
    PM_REQUIRE(count, "point_cube_count: null pointer");
    point_count_k<1><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        database, query, nv_database, nv_query, B, Np, Mp, length, nn_sample, count);
    PM_LAUNCHED("point_cube_count");
    return 0;
}

extern "C" int pmesh_point_cube_fill(const float *database, const float *query, const int32_t *nv_database,
                                     const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float length, int grid_size,
                                     const int64_t *cnt_info, int64_t Nout, int32_t *nn_index, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(length > 0 && grid_size > 0 && Nout >= 0, "point_cube_fill: bad arguments");
    PM_QUERY_DIMS("point_cube_fill");
    if (Nout == 0) return 0;
    PM_REQUIRE(cnt_info && nn_index, "point_cube_fill: null pointer");
    point_fill_k<1><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        database, query, nv_database, nv_query, B, Np, Mp, length, grid_size, cnt_info, Nout, nn_index, nullptr);
    PM_LAUNCHED("point_cube_fill");
    return 0;
}

extern "C" int pmesh_point_knn3(const float *database, const float *query, const int32_t *nv_database, const int32_t *nv_query,
                                int B, int64_t Np, int64_t Mp, int32_t *nn_index, float *nn_dist, pmesh_stream_t stream)
{
    clear_error();
    PM_QUERY_DIMS("point_knn3");
    PM_REQUIRE(nn_index && nn_dist, "point_knn3: null pointer");
    point_knn3_k<<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(database, query, nv_database, nv_query,
                                                                                            B, Np, Mp, nn_index, nn_dist);
    PM_LAUNCHED("point_knn3");
    return 0;
}

extern "C" int pmesh_point_fps(const float *xyz, const int32_t *nv_in, const int32_t *nv_out, int B, int64_t Np, int64_t Mp,
                               float *temp, int32_t *index_out, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(B >= 0 && B <= 65535 * 32 && Np >= 0 && Mp >= 0 && Np <= INT32_MAX && Mp <= INT32_MAX, "point_fps: bad sizes");
    if (B == 0 || Mp == 0) return 0;
    PM_REQUIRE(xyz && nv_in && nv_out && temp && index_out, "point_fps: null pointer");
    point_fps_k<<<dim3((unsigned)B), dim3(kFpsThreads), 0, (hipStream_t)stream>>>(xyz, nv_in, nv_out, B, Np, Mp, temp, index_out);
    PM_LAUNCHED("point_fps");
    return 0;
}

#define PM_KERNEL_DIMS(name)                                                                                           \
    PM_REQUIRE(radius > 0, name ": radius must be positive");                                                           \
    PM_REQUIRE(n > 2 && n % 2 == 0 && p > 0 && p % 2 == 0 && q > 0, name ": need n > 2, n and p even, p, q > 0");        \
    PM_REQUIRE(Nout >= 0 && Np >= 0 && Mp >= 0 && Np <= INT32_MAX && Mp <= INT32_MAX, name ": bad sizes");               \
    if (Nout == 0) return 0;                                                                                            \
    PM_REQUIRE(Np > 0 && Mp > 0 && database && query && nn_index && nn_dist && filt_index, name ": null pointer");       \
    PM_REQUIRE(grid_ok(ceil_div(Nout, kBlock)), name ": grid too large")

extern "C" int pmesh_point_sph3d_kernel(const float *database, const float *query, const int32_t *nn_index, const float *nn_dist,
                                        int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q, float radius,
                                        int32_t *filt_index, pmesh_stream_t stream)
{
    clear_error();
    PM_KERNEL_DIMS("point_sph3d_kernel");
    point_sph3d_k<<<dim3((unsigned)ceil_div(Nout, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(database, query, nn_index, nn_dist, Nout,
                                                                                               Np, Mp, n, p, q, radius, filt_index);
    PM_LAUNCHED("point_sph3d_kernel");
    return 0;
}

extern "C" int pmesh_point_fuzzy_sph3d_kernel(const float *database, const float *query, const int32_t *nn_index,
                                              const float *nn_dist, int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q,
                                              float radius, int32_t *filt_index, float *filt_coeff, pmesh_stream_t stream)
{
    clear_error();
    PM_KERNEL_DIMS("point_fuzzy_sph3d_kernel");
    PM_REQUIRE(filt_coeff, "point_fuzzy_sph3d_kernel: null pointer");
    point_fuzzy_sph3d_k<<<dim3((unsigned)ceil_div(Nout, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        database, query, nn_index, nn_dist, Nout, Np, Mp, n, p, q, radius, filt_index, filt_coeff);
    PM_LAUNCHED("point_fuzzy_sph3d_kernel");
    return 0;
}
