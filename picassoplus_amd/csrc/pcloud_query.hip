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
#include "rows_internal.h"
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

// ---------------------------------------------------------------------------------------------------------------
// The range and cube searches over a cell grid.  The scans above cost queries x sample size; here the database
// points are sorted into cells at least as wide as the search reaches (radius, or half the cube's edge), so a
// query looks at the 27 cells around its own.  The outputs are the scans': the same float32 test decides who is
// a neighbour, and of a query's neighbours the nn_sample lowest database indices are kept, in ascending order (the
// fill step inserts every neighbour it meets into the query's sorted output segment).
//
// One grid serves all samples: cell (b, x, y, z) of sample b over the bounding box of all finite database
// coordinates; at most kGridMaxCells cells and kGridMaxAxis per axis, the cell edge h grows until that holds.
// h >= 1.01 x reach, and a cell coordinate carries an error below 2 * kGridMaxAxis * 2^-23 cells, so two points
// whose coordinates differ by less than the reach lie at most one cell apart on every axis; a search that reaches
// further than the grid was built for widens its window instead.  Points that belong to no sample sort behind the
// last cell; coordinates that are not finite never pass the distance test, whichever cell they fall into.
constexpr int kGridMaxCells = 1 << 20;
constexpr int kGridMaxAxis = 4096;
constexpr int kGridKeyBits = 21;                        // keys 0 .. kGridMaxCells
constexpr float kGridSlack = 1.01f;

struct PointGrid {                                      // head of a grid workspace
    float ox, oy, oz, inv_h;
    int nx, ny, nz, cells;                              // cells per sample = nx * ny * nz
    int lo[3], hi[3];                                   // bounding box, floats as order-preserving integers
};
constexpr size_t kGridHead = 256;
static_assert(sizeof(PointGrid) <= kGridHead, "grid head");

__device__ __forceinline__ int ordered_int(float f)
{
    const int i = __float_as_int(f);
    return i >= 0 ? i : i ^ 0x7fffffff;
}
__device__ __forceinline__ float ordered_float(int i) { return __int_as_float(i >= 0 ? i : i ^ 0x7fffffff); }

// empties the cells and the bounding box
__global__ __launch_bounds__(kBlock) void grid_clear_k(PointGrid *__restrict__ G, int2 *__restrict__ cells)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < kGridMaxCells) cells[i] = make_int2(0, 0);
    if (i == 0)
        for (int a = 0; a < 3; ++a) { G->lo[a] = INT32_MAX; G->hi[a] = INT32_MIN; }
}

__device__ __forceinline__ bool finite3(float x, float y, float z) { return fabsf(x) < INFINITY && fabsf(y) < INFINITY && fabsf(z) < INFINITY; }

constexpr int kBboxPer = 16;                            // points per thread of the bounding-box pass
__global__ __launch_bounds__(kBlock) void grid_bbox_k(const float *__restrict__ db, const int *__restrict__ nvd, int B, int64_t Np,
                                                      PointGrid *__restrict__ G)
{
    __shared__ int s_lo[3][kBlock / 64], s_hi[3][kBlock / 64];
    int lo[3] = {INT32_MAX, INT32_MAX, INT32_MAX}, hi[3] = {INT32_MIN, INT32_MIN, INT32_MIN};
    const int64_t n = B > 0 ? (nvd[B - 1] < Np ? nvd[B - 1] : Np) : 0;
    const int64_t k0 = (int64_t)blockIdx.x * kBlock * kBboxPer + threadIdx.x;
    for (int i = 0; i < kBboxPer; ++i) {
        const int64_t k = k0 + (int64_t)i * kBlock;
        if (k >= n) break;
        const float x = db[k * 3], y = db[k * 3 + 1], z = db[k * 3 + 2];
        if (!finite3(x, y, z)) continue;
        const int v[3] = {ordered_int(x), ordered_int(y), ordered_int(z)};
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            lo[a] = v[a] < lo[a] ? v[a] : lo[a];
            hi[a] = v[a] > hi[a] ? v[a] : hi[a];
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const int l = __shfl_xor(lo[a], o, 64), h = __shfl_xor(hi[a], o, 64);
            lo[a] = l < lo[a] ? l : lo[a];
            hi[a] = h > hi[a] ? h : hi[a];
        }
        if ((threadIdx.x & 63) == 0) { s_lo[a][threadIdx.x >> 6] = lo[a]; s_hi[a][threadIdx.x >> 6] = hi[a]; }
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const int a = threadIdx.x;
        int l = s_lo[a][0], h = s_hi[a][0];
        for (int w = 1; w < kBlock / 64; ++w) {
            l = s_lo[a][w] < l ? s_lo[a][w] : l;
            h = s_hi[a][w] > h ? s_hi[a][w] : h;
        }
        if (l <= h) {
            atomicMin(&G->lo[a], l);
            atomicMax(&G->hi[a], h);
        }
    }
}

// origin, cell edge and cell counts from the bounding box (one thread)
__global__ void grid_dims_k(PointGrid *__restrict__ G, int B, float reach, int64_t per_sample)
{
    if (blockIdx.x || threadIdx.x) return;
    float o[3] = {0.f, 0.f, 0.f}, ext[3] = {0.f, 0.f, 0.f};
    for (int a = 0; a < 3; ++a)
        if (G->lo[a] <= G->hi[a]) {
            o[a] = ordered_float(G->lo[a]);
            ext[a] = ordered_float(G->hi[a]) - o[a];
        }
    float h = reach * kGridSlack;
    if (reach < 0.f && finite3(ext[0], ext[1], ext[2])) {
        // no search radius to go by (nearest-neighbour queries): about -reach cells per database point of a sample.
        // Axes shorter than the edge that comes out get one cell and leave the product to the others.
        const float target = fmaxf(-reach * (float)per_sample, 1.f);
        bool on[3] = {ext[0] > 0.f, ext[1] > 0.f, ext[2] > 0.f};
        h = 0.f;
        for (int it = 0; it < 4; ++it) {
            float vol = 1.f;
            int act = 0;
            for (int a = 0; a < 3; ++a)
                if (on[a]) { vol *= ext[a]; ++act; }
            if (!act) break;
            h = powf(vol / target, 1.0f / (float)act);
            bool again = false;
            for (int a = 0; a < 3; ++a)
                if (on[a] && ext[a] < h) { on[a] = false; again = true; }
            if (!again) break;
        }
        if (!(h > 0.f)) h = fmaxf(fmaxf(ext[0], ext[1]), fmaxf(ext[2], 1e-30f));     // all points in one place
    }
    int n[3] = {1, 1, 1};
    bool fits = false;
    if (h > 0.f && h < INFINITY && finite3(ext[0], ext[1], ext[2]))
        for (int it = 0; it < 400 && !fits && h < INFINITY; ++it) {
            double total = (double)(B > 0 ? B : 1);
            bool axis = true;
            for (int a = 0; a < 3; ++a) {
                const float c = floorf(ext[a] / h);
                axis = axis && c < (float)kGridMaxAxis;
                n[a] = (int)fminf(c, (float)kGridMaxAxis) + 1;
                total *= (double)n[a];
            }
            fits = axis && total <= (double)kGridMaxCells;
            if (!fits) h *= 1.26f;
        }
    if (!fits) {                                        // one cell per sample: every query looks at its whole sample
        n[0] = n[1] = n[2] = 1;
        G->inv_h = 0.f;
    } else {
        G->inv_h = 1.0f / h;
    }
    G->ox = o[0]; G->oy = o[1]; G->oz = o[2];
    G->nx = n[0]; G->ny = n[1]; G->nz = n[2];
    G->cells = n[0] * n[1] * n[2];
}

// cell coordinate of a database point, inside the grid whatever the value
__device__ __forceinline__ int grid_coord(float p, float o, float inv_h, int n)
{
    float v = floorf((p - o) * inv_h);
    v = fmaxf(v, 0.f);                                  // (also what a NaN becomes)
    v = fminf(v, (float)(n - 1));
    return (int)v;
}

__global__ __launch_bounds__(kBlock) void grid_keys_k(const float *__restrict__ db, const int *__restrict__ nvd, int B, int64_t Np,
                                                      const PointGrid *__restrict__ G, unsigned *__restrict__ keys,
                                                      int *__restrict__ ids)
{
    const int64_t k = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (k >= Np) return;
    int b = 0;
    while (b < B && k >= nvd[b]) ++b;
    unsigned key = (unsigned)kGridMaxCells;
    if (b < B) {
        const int x = grid_coord(db[k * 3], G->ox, G->inv_h, G->nx), y = grid_coord(db[k * 3 + 1], G->oy, G->inv_h, G->ny),
                  z = grid_coord(db[k * 3 + 2], G->oz, G->inv_h, G->nz);
        key = (unsigned)(b * G->cells + (x * G->ny + y) * G->nz + z);
    }
    keys[k] = key;
    ids[k] = (int)k;
}

// [first, last) sorted position of every occupied cell, and the sorted points as (x, y, z, database index)
__global__ __launch_bounds__(kBlock) void grid_cells_k(const float *__restrict__ db, const unsigned *__restrict__ keys,
                                                       const int *__restrict__ ids, int64_t Np, int2 *__restrict__ cells,
                                                       float4 *__restrict__ pts)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= Np) return;
    const unsigned key = keys[i];
    const int id = ids[i];
    pts[i] = make_float4(db[(int64_t)id * 3], db[(int64_t)id * 3 + 1], db[(int64_t)id * 3 + 2], __int_as_float(id));
    if (key >= (unsigned)kGridMaxCells) return;
    if (i == 0 || keys[i - 1] != key) cells[key].x = (int)i;
    if (i == Np - 1 || keys[i + 1] != key) cells[key].y = (int)i + 1;
}

// cells a query looks at on one axis: its own and `reach` cells to either side, cut to the grid (empty if c0 > c1)
struct GridSpan {
    int c0, c1;
};
__device__ __forceinline__ GridSpan grid_span(float q, float o, float inv_h, int n, int reach)
{
    float v = floorf((q - o) * inv_h);
    v = fmaxf(v, -2.f - (float)reach);                  // (a NaN query ends up outside and finds nothing, as in the scan)
    v = fminf(v, (float)(n + 1 + reach));
    const int c = (int)v;
    GridSpan s;
    s.c0 = c - reach > 0 ? c - reach : 0;
    s.c1 = c + reach < n - 1 ? c + reach : n - 1;
    return s;
}
__device__ __forceinline__ int grid_reach(float size, int mode, float inv_h)
{
    const float need = (mode == 0 ? size : size / 2) * kGridSlack * inv_h - 1e-3f;
    const float r = ceilf(fminf(need, (float)kGridMaxAxis));
    return r > 1.f ? (int)r : 1;
}

// Visits the database points of sample b in the cells around (qx, qy, qz).  The (x, y) columns of those cells are dealt
// out to the `lanes` lanes that share the query (`sub`: which of them I am); the cells of a column follow each other
// in the sort order, so a column's points are one run, read four at a time.  f(point) returns false to stop this lane.
template <int MODE, typename F>
__device__ __forceinline__ void grid_visit(const PointGrid *__restrict__ G, const int2 *__restrict__ cells,
                                           const float4 *__restrict__ pts, int b, float qx, float qy, float qz, float size,
                                           int sub, int lanes, F f)
{
    const float inv_h = G->inv_h;
    const int nx = G->nx, ny = G->ny, nz = G->nz, reach = grid_reach(size, MODE, inv_h);
    const GridSpan sx = grid_span(qx, G->ox, inv_h, nx, reach), sy = grid_span(qy, G->oy, inv_h, ny, reach),
                   sz = grid_span(qz, G->oz, inv_h, nz, reach);
    if (sx.c0 > sx.c1 || sy.c0 > sy.c1 || sz.c0 > sz.c1) return;
    const int wy = sy.c1 - sy.c0 + 1, ncol = (sx.c1 - sx.c0 + 1) * wy;
    const int2 *mine = cells + (int64_t)b * G->cells;
    for (int c = sub; c < ncol; c += lanes) {
        const int x = sx.c0 + c / wy, y = sy.c0 + c % wy;
        const int2 *col = mine + (x * ny + y) * nz;
        int s = INT32_MAX, e = 0;
        for (int z = sz.c0; z <= sz.c1; ++z) {
            const int2 r = col[z];
            if (r.y > r.x) {
                s = r.x < s ? r.x : s;
                e = r.y > e ? r.y : e;
            }
        }
        for (int i = s; i < e; i += 4) {
            float4 p[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) p[u] = pts[i + u < e ? i + u : e - 1];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i + u < e && !f(p[u])) return;
        }
    }
}

__device__ __forceinline__ float sq_dist(float qx, float qy, float qz, const float4 &p, float &dx, float &dy, float &dz)
{
#pragma clang fp contract(off)
    dx = p.x - qx;
    dy = p.y - qy;
    dz = p.z - qz;
    return (dx * dx + dy * dy) + dz * dz;
}

// sample of query j and its index b
__device__ __forceinline__ int sample_index(int64_t j, const int *__restrict__ nvq, int B)
{
    int b = 0;
    while (b < B && j >= nvq[b]) ++b;
    return b;
}

// kQLanes neighbouring lanes share a query: the searches are chains of dependent fetches (cell, then its points), and
// a chip-wide grid of one thread per query would leave most of the latency uncovered.
constexpr int kQLanes = 8;
constexpr int kQPerBlock = kBlock / kQLanes;

template <int MODE>
__global__ __launch_bounds__(kBlock) void point_count_grid_k(const PointGrid *__restrict__ G, const int2 *__restrict__ cells,
                                                             const float4 *__restrict__ pts, const float *__restrict__ query,
                                                             const int *__restrict__ nvq, int B, int64_t Mp, float size,
                                                             int nn_sample, int *__restrict__ count)
{
    const int64_t j = (int64_t)blockIdx.x * kQPerBlock + threadIdx.x / kQLanes;
    const int sub = threadIdx.x % kQLanes;
    const bool valid = j < Mp;
    const int b = valid ? sample_index(j, nvq, B) : B;
    int cnt = 0;
    if (b < B) {
        const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
        grid_visit<MODE>(G, cells, pts, b, qx, qy, qz, size, sub, kQLanes, [&](const float4 &p) {
            float dx, dy, dz;
            const float d2 = sq_dist(qx, qy, qz, p, dx, dy, dz);
            cnt += is_neighbour<MODE>(d2, dx, dy, dz, size) ? 1 : 0;
            return cnt < nn_sample;
        });
    }
    // (every lane of the wavefront is here: none has left the kernel)
#pragma unroll
    for (int o = 1; o < kQLanes; o <<= 1) {
        const int other = __shfl_xor(cnt, o, 64);
        cnt = (int)((int64_t)cnt + other < nn_sample ? cnt + other : nn_sample);
    }
    if (valid && sub == 0) count[j] = cnt;
}

// One lane's way to fill a query's segment, for the queries with more neighbours than the workgroup's buffers hold:
// the database indices to keep are held sorted (in `seg`: the query's buffer if they fit, else its segment of nn_index)
// while the neighbours come in; once all places are taken a neighbour replaces the largest index if it is lower.  The
// other columns follow from the final indices.
template <int MODE>
__device__ void fill_by_insertion(const PointGrid *__restrict__ G, const int2 *__restrict__ cells, const float4 *__restrict__ pts,
                                  const float *__restrict__ db, int b, int64_t j, float qx, float qy, float qz, int64_t Np,
                                  float size, int grid_size, int64_t at, int64_t m, int *seg, int step, int *nn_index,
                                  float *nn_dist)
{
#pragma clang fp contract(off)
    constexpr int W = MODE == 0 ? 2 : 3;                // seg[step * t]: database index of the query's t-th pair so far
    int64_t filled = 0;
    int last = -1;                                      // the largest index kept so far
    grid_visit<MODE>(G, cells, pts, b, qx, qy, qz, size, 0, 1, [&](const float4 &p) {
        float dx, dy, dz;
        const float d2 = sq_dist(qx, qy, qz, p, dx, dy, dz);
        if (!is_neighbour<MODE>(d2, dx, dy, dz, size)) return true;
        const int id = __float_as_int(p.w);
        if (filled == m && id > last) return true;
        const int64_t top = filled < m ? filled++ : m - 1;
        int64_t pos = top;
        int newlast = id;
        while (pos > 0) {
            const int prev = seg[step * (pos - 1)];
            if (prev < id) break;
            if (pos == top) newlast = prev;
            seg[step * pos] = prev;
            --pos;
        }
        seg[step * pos] = id;
        last = newlast;
        return true;
    });
    for (int64_t t = 0; t < filled; ++t) {
        const int kept = seg[step * t];
        const int id = kept < 0 ? 0 : (kept >= Np ? (int)Np - 1 : kept);
        float dx, dy, dz;
        const float d2 = sq_dist(qx, qy, qz, db + (int64_t)id * 3, dx, dy, dz);
        nn_index[(at + t) * W] = (int)j;
        nn_index[(at + t) * W + 1] = kept;
        if constexpr (MODE == 0) {
            nn_dist[at + t] = sqrtf(d2);
        } else {
            const float half = size / 2, cell = size / (float)grid_size;
            const int xi = (int)((dx + half) / cell), yi = (int)((dy + half) / cell), zi = (int)((dz + half) / cell);
            nn_index[(at + t) * W + 2] = (xi * grid_size + yi) * grid_size + zi;
        }
    }
}

// Pairs of query j at [cnt_info[j-1], cnt_info[j]): its lanes drop the neighbours they meet into a buffer of the
// workgroup (database index; distance or kernel cell), then every neighbour finds its place by counting the lower
// indices, and the first m = cnt_info[j] - cnt_info[j-1] places are written.  A query with more neighbours than the
// buffer holds, of which it keeps at most half a buffer: the m-th lowest of the indices that did get in bounds the
// m-th lowest of all from above, so the walk is repeated for the neighbours up to that index only (up to three
// times; each round leaves out at least half a buffer of what the round before let in).  A query that keeps ALL of
// more neighbours than the buffer holds sorts them through its output segment (below).  What is left -- a long
// segment that is still only part of the neighbours -- is filled by one lane (fill_by_insertion).
constexpr int kFillCap = 128;
constexpr int kFillRounds = 4;
template <int MODE>
__global__ __launch_bounds__(kBlock) void point_fill_grid_k(const PointGrid *__restrict__ G, const int2 *__restrict__ cells,
                                                            const float4 *__restrict__ pts, const float *__restrict__ db,
                                                            const float *__restrict__ query, const int *__restrict__ nvq, int B,
                                                            int64_t Np, int64_t Mp, float size, int grid_size,
                                                            const int64_t *__restrict__ cnt_info, int64_t Nout,
                                                            int *__restrict__ nn_index, float *__restrict__ nn_dist)
{
#pragma clang fp contract(off)
    constexpr int W = MODE == 0 ? 2 : 3;
    // a query's buffer: kFillCap indices, then as many distances / kernel cells; as one array of indices where all
    // neighbours are kept (below)
    constexpr int kRow = 2 * (kFillCap + 1);
    __shared__ int s_buf[kQPerBlock][kRow];
    int *s_id_q = &s_buf[threadIdx.x / kQLanes][0];
    unsigned *s_val_q = reinterpret_cast<unsigned *>(s_id_q + kFillCap + 1);
    __shared__ int s_cnt[kQPerBlock], s_thr[kQPerBlock];
    const int q = threadIdx.x / kQLanes, sub = threadIdx.x % kQLanes;
    const int64_t j = (int64_t)blockIdx.x * kQPerBlock + q;
    const bool valid = j < Mp;
    const int b = valid ? sample_index(j, nvq, B) : B;
    int64_t at = 0, m = 0;
    float qx = 0.f, qy = 0.f, qz = 0.f;
    if (b < B) {
        int64_t end = cnt_info[j];
        at = j ? cnt_info[j - 1] : 0;
        if (at < 0) at = 0;
        if (end > Nout) end = Nout;
        m = end > at ? end - at : 0;
        qx = query[j * 3]; qy = query[j * 3 + 1]; qz = query[j * 3 + 2];
    }
    // a segment longer than a query's buffer is left to point_fill_long_k: -1 in its first place says so
    bool later = m > kRow;
    // (the lanes of a query sit in one wavefront, and every lane of the wavefront stays until the last exchange)
    auto lanes_meet = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    int thr = INT32_MAX;                                // neighbours above this index are not among the m lowest
    int total = 0;
    bool open = m > 0 && !later, all_kept = false;
    for (int round = 0; round < kFillRounds; ++round) {
        if (!__builtin_amdgcn_ballot_w64(open)) break;
        if (open && sub == 0) s_cnt[q] = 0;
        lanes_meet();
        if (open)
            grid_visit<MODE>(G, cells, pts, b, qx, qy, qz, size, sub, kQLanes, [&](const float4 &p) {
                float dx, dy, dz;
                const float d2 = sq_dist(qx, qy, qz, p, dx, dy, dz);
                if (!is_neighbour<MODE>(d2, dx, dy, dz, size)) return true;
                const int id = __float_as_int(p.w);
                if (id > thr) return true;
                const int slot = atomicAdd(&s_cnt[q], 1);
                if (slot < kFillCap) {
                    s_id_q[slot] = id;
                    if constexpr (MODE == 0) {
                        s_val_q[slot] = __float_as_uint(sqrtf(d2));
                    } else {
                        const float half = size / 2, cell = size / (float)grid_size;
                        const int xi = (int)((dx + half) / cell), yi = (int)((dy + half) / cell), zi = (int)((dz + half) / cell);
                        s_val_q[slot] = (unsigned)((xi * grid_size + yi) * grid_size + zi);
                    }
                }
                return true;
            });
        lanes_meet();
        bool narrow = false;
        if (open) {
            total = s_cnt[q];
            if (total <= kFillCap) open = false;
            else if (round == 0 && total == m) { open = false; all_kept = true; }
            else if (m > kFillCap / 2 || round == kFillRounds - 1) { open = false; later = true; }
            else narrow = true;
        }
        if (__builtin_amdgcn_ballot_w64(narrow)) {
            if (narrow)
                for (int e = sub; e < kFillCap; e += kQLanes) {
                    const int id = s_id_q[e];
                    int rank = 0;
                    for (int f = 0; f < kFillCap; ++f) rank += s_id_q[f] < id ? 1 : 0;
                    if (rank == m - 1) s_thr[q] = id;
                }
            lanes_meet();
            if (narrow) thr = s_thr[q];
        }
    }
    // More neighbours than the buffer holds, all of them kept (and at most kRow of them): their indices go into the
    // query's whole buffer in the order met, then every entry of that list finds its place by counting the lower
    // indices in it.
    if (__builtin_amdgcn_ballot_w64(all_kept)) {
        if (all_kept && sub == 0) s_cnt[q] = 0;
        lanes_meet();
        if (all_kept)
            grid_visit<MODE>(G, cells, pts, b, qx, qy, qz, size, sub, kQLanes, [&](const float4 &p) {
                float dx, dy, dz;
                const float d2 = sq_dist(qx, qy, qz, p, dx, dy, dz);
                if (!is_neighbour<MODE>(d2, dx, dy, dz, size)) return true;
                const int slot = atomicAdd(&s_cnt[q], 1);
                if (slot < m) s_id_q[slot] = __float_as_int(p.w);
                return true;
            });
        lanes_meet();
        // (a second walk with the counting inside would make every lane of the wavefront wait through the count of
        // every neighbour any lane meets; the list itself is walked instead, and a neighbour's distance or cell comes
        // from its coordinates)
        if (all_kept)
            for (int e = sub; e < (int)m; e += kQLanes) {
                const int id = s_id_q[e];
                int r0 = 0, r1 = 0;
                int f = 0;
                for (; f + 2 <= (int)m; f += 2) {
                    const int2 two = *reinterpret_cast<const int2 *>(s_id_q + f);
                    r0 += two.x < id ? 1 : 0;
                    r1 += two.y < id ? 1 : 0;
                }
                if (f < (int)m) r0 += s_id_q[f] < id ? 1 : 0;
                const int rank = r0 + r1;
                const int64_t row = id < 0 ? 0 : (id >= Np ? Np - 1 : id);
                float dx, dy, dz;
                const float d2 = sq_dist(qx, qy, qz, db + row * 3, dx, dy, dz);
                nn_index[(at + rank) * W] = (int)j;
                nn_index[(at + rank) * W + 1] = id;
                if constexpr (MODE == 0) {
                    nn_dist[at + rank] = sqrtf(d2);
                } else {
                    const float half = size / 2, cell = size / (float)grid_size;
                    const int xi = (int)((dx + half) / cell), yi = (int)((dy + half) / cell), zi = (int)((dz + half) / cell);
                    nn_index[(at + rank) * W + 2] = (xi * grid_size + yi) * grid_size + zi;
                }
            }
    }
    if (m <= 0 || all_kept) return;
    if (later) {
        if (sub == 0) nn_index[at * W] = -1;
        return;
    }
    for (int e = sub; e < total; e += kQLanes) {
        const int id = s_id_q[e];
        int rank = 0;
        for (int f = 0; f < total; ++f) rank += s_id_q[f] < id ? 1 : 0;
        if (rank >= m) continue;
        nn_index[(at + rank) * W] = (int)j;
        nn_index[(at + rank) * W + 1] = id;
        if constexpr (MODE == 0) nn_dist[at + rank] = __uint_as_float(s_val_q[e]);
        else nn_index[(at + rank) * W + 2] = (int)s_val_q[e];
    }
}

// The segments point_fill_grid_k left (first place = -1): a wavefront per query, up to kLongCap neighbours in its
// buffer (index; distance or kernel cell), places by counting the lower indices as above; beyond that, one lane's
// sorted insertion.  A workgroup looks at kBlock queries and its wavefronts share out the marked ones.
constexpr int kLongCap = 4096;
template <int MODE>
__global__ __launch_bounds__(kBlock) void point_fill_long_k(const PointGrid *__restrict__ G, const int2 *__restrict__ cells,
                                                            const float4 *__restrict__ pts, const float *__restrict__ db,
                                                            const float *__restrict__ query, const int *__restrict__ nvq, int B,
                                                            int64_t Np, int64_t Mp, float size, int grid_size,
                                                            const int64_t *__restrict__ cnt_info, int64_t Nout,
                                                            int *nn_index, float *nn_dist)
{
#pragma clang fp contract(off)
    constexpr int W = MODE == 0 ? 2 : 3, NW = kBlock / 64;
    __shared__ int s_id[NW][kLongCap];
    __shared__ unsigned s_val[NW][kLongCap];
    __shared__ int s_list[kBlock], s_n, s_cnt[NW];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_n = 0;
    __syncthreads();
    {
        const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
        if (j < Mp && sample_index(j, nvq, B) < B) {
            int64_t at = j ? cnt_info[j - 1] : 0, end = cnt_info[j];
            if (at < 0) at = 0;
            if (end > Nout) end = Nout;
            if (end > at && nn_index[at * W] == -1) s_list[atomicAdd(&s_n, 1)] = (int)threadIdx.x;
        }
    }
    __syncthreads();
    const int n = s_n;
    for (int i = w; i < n; i += NW) {
        const int64_t j = (int64_t)blockIdx.x * kBlock + s_list[i];
        const int b = sample_index(j, nvq, B);
        int64_t at = j ? cnt_info[j - 1] : 0, end = cnt_info[j];
        if (at < 0) at = 0;
        if (end > Nout) end = Nout;
        const int64_t m = end - at;
        const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
        if (lane == 0) s_cnt[w] = 0;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        grid_visit<MODE>(G, cells, pts, b, qx, qy, qz, size, lane, 64, [&](const float4 &p) {
            float dx, dy, dz;
            const float d2 = sq_dist(qx, qy, qz, p, dx, dy, dz);
            if (!is_neighbour<MODE>(d2, dx, dy, dz, size)) return true;
            const int slot = atomicAdd(&s_cnt[w], 1);
            if (slot < kLongCap) {
                s_id[w][slot] = __float_as_int(p.w);
                if constexpr (MODE == 0) {
                    s_val[w][slot] = __float_as_uint(sqrtf(d2));
                } else {
                    const float half = size / 2, cell = size / (float)grid_size;
                    const int xi = (int)((dx + half) / cell), yi = (int)((dy + half) / cell), zi = (int)((dz + half) / cell);
                    s_val[w][slot] = (unsigned)((xi * grid_size + yi) * grid_size + zi);
                }
            }
            return true;
        });
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int total = s_cnt[w];
        if (total > kLongCap) {
            if (lane == 0)
                fill_by_insertion<MODE>(G, cells, pts, db, b, j, qx, qy, qz, Np, size, grid_size, at, m, nn_index + at * W + 1, W,
                                        nn_index, nn_dist);
            continue;
        }
        for (int e = lane; e < total; e += 64) {
            const int id = s_id[w][e];
            int rank = 0;
            for (int f = 0; f < total; ++f) rank += s_id[w][f] < id ? 1 : 0;
            if (rank >= m) continue;
            nn_index[(at + rank) * W] = (int)j;
            nn_index[(at + rank) * W + 1] = id;
            if constexpr (MODE == 0) nn_dist[at + rank] = __uint_as_float(s_val[w][e]);
            else nn_index[(at + rank) * W + 2] = (int)s_val[w][e];
        }
        // (a segment with fewer neighbours than places keeps its mark otherwise)
        if (lane == 0 && total == 0) nn_index[at * W] = (int)j;
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

// The three nearest over the cell grid, same result as the scan above: kQLanes lanes share a query and deal out the
// (x, y) columns of a window of cells around it; each keeps its three best by (squared distance, database index), the
// lists are merged, and the window grows until the third best is closer than anything outside it can be (a point in a
// cell r + 1 or more cells away on some axis is at least r cell edges away) or until it covers the sample's grid.
struct Near3 {
    float d[3];
    int i[3];
};
__device__ __forceinline__ bool nearer(float d, int i, float b, int j) { return d < b || (d == b && i < j); }
__device__ __forceinline__ void near3_insert(Near3 &n, float d, int i)
{
    if (nearer(d, i, n.d[0], n.i[0])) {
        n.d[2] = n.d[1]; n.i[2] = n.i[1]; n.d[1] = n.d[0]; n.i[1] = n.i[0]; n.d[0] = d; n.i[0] = i;
    } else if (nearer(d, i, n.d[1], n.i[1])) {
        n.d[2] = n.d[1]; n.i[2] = n.i[1]; n.d[1] = d; n.i[1] = i;
    } else if (nearer(d, i, n.d[2], n.i[2])) {
        n.d[2] = d; n.i[2] = i;
    }
}

__global__ __launch_bounds__(kBlock) void point_knn3_grid_k(const PointGrid *__restrict__ G, const int2 *__restrict__ cells,
                                                            const float4 *__restrict__ pts, const float *__restrict__ query,
                                                            const int *__restrict__ nvd, const int *__restrict__ nvq, int B,
                                                            int64_t Mp, int *__restrict__ nn_index, float *__restrict__ nn_dist)
{
    const int64_t j = (int64_t)blockIdx.x * kQPerBlock + threadIdx.x / kQLanes;
    const int sub = threadIdx.x % kQLanes;
    const bool valid = j < Mp;
    const int b = valid ? sample_index(j, nvq, B) : B;
    if (b >= B) {
        // (all lanes of a query leave together; the lanes of the other queries do not wait for them)
        if (valid && sub == 0)
            for (int i = 0; i < 3; ++i) { nn_index[j * 3 + i] = 0; nn_dist[j * 3 + i] = INFINITY; }
        return;
    }
    const int first = b ? nvd[b - 1] : 0;               // what the scan reports in the places it cannot fill
    const float qx = query[j * 3], qy = query[j * 3 + 1], qz = query[j * 3 + 2];
    const float inv_h = G->inv_h, h = inv_h > 0.f ? 1.0f / inv_h : INFINITY;
    const int n[3] = {G->nx, G->ny, G->nz};
    const float q[3] = {qx, qy, qz}, o[3] = {G->ox, G->oy, G->oz};
    int c[3], r = 1;
    bool sane = true;
    for (int a = 0; a < 3; ++a) {
        float v = floorf((q[a] - o[a]) * inv_h);
        sane = sane && v == v;
        v = fminf(fmaxf(v, -4.f * kGridMaxAxis), 4.f * kGridMaxAxis);
        c[a] = sane ? (int)v : 0;
        const int out = c[a] < 0 ? -c[a] : (c[a] > n[a] - 1 ? c[a] - (n[a] - 1) : 0);       // cells between me and the grid
        r = out > r ? out : r;
    }
    if (!sane) r = 8 * kGridMaxAxis;                    // a query that is not a number is no nearer to anything: every cell
    const int2 *mine = cells + (int64_t)b * G->cells;
    Near3 best;
    for (;;) {
        for (int i = 0; i < 3; ++i) { best.d[i] = INFINITY; best.i[i] = first; }
        int lo[3], hi[3];
        bool all = true;
        for (int a = 0; a < 3; ++a) {
            lo[a] = c[a] - r > 0 ? c[a] - r : 0;
            hi[a] = c[a] + r < n[a] - 1 ? c[a] + r : n[a] - 1;
            all = all && c[a] - r <= 0 && c[a] + r >= n[a] - 1;
        }
        const int wy = hi[1] - lo[1] + 1, ncol = (hi[0] - lo[0] + 1) * wy;
        for (int k = sub; k < ncol; k += kQLanes) {
            const int x = lo[0] + k / wy, y = lo[1] + k % wy;
            const int2 *col = mine + (x * n[1] + y) * n[2];
            int s = INT32_MAX, e = 0;
            for (int z = lo[2]; z <= hi[2]; ++z) {
                const int2 rg = col[z];
                if (rg.y > rg.x) {
                    s = rg.x < s ? rg.x : s;
                    e = rg.y > e ? rg.y : e;
                }
            }
            for (int i = s; i < e; i += 4) {
                float4 p[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) p[u] = pts[i + u < e ? i + u : e - 1];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (i + u < e) {
                        float dx, dy, dz;
                        const float d2 = sq_dist(qx, qy, qz, p[u], dx, dy, dz);
                        near3_insert(best, d2, __float_as_int(p[u].w));
                    }
            }
        }
        // the lanes of the query exchange their lists (all eight are here together)
#pragma unroll
        for (int step = 1; step < kQLanes; step <<= 1) {
            Near3 other;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                other.d[i] = __shfl_xor(best.d[i], step, 64);
                other.i[i] = __shfl_xor(best.i[i], step, 64);
            }
#pragma unroll
            for (int i = 0; i < 3; ++i)
                if (other.d[i] < INFINITY) near3_insert(best, other.d[i], other.i[i]);
        }
        if (all || sqrtf(best.d[2]) < ((float)r - 0.01f) * h) break;
        r = r + 1 > r + r / 2 ? r + 1 : r + r / 2;
    }
    if (sub == 0) {
        for (int i = 0; i < 3; ++i) {
            nn_index[j * 3 + i] = best.i[i];
            nn_dist[j * 3 + i] = sqrtf(best.d[i]);
        }
    }
}

// Farthest point sampling: one workgroup of 1024 threads per sample.  Every round updates the squared distance of
// each point to the chosen set against the last chosen point and takes the arg-max (lowest index among equals).
// A sample of at most 1024 * kFpsPer points lives in registers for the whole run (thread t holds points t, t + 1024,
// ... and their distances), the round's winner is found by every thread from the wavefronts' candidates in LDS, and
// its owner hands the coordinates to the others through LDS: two barriers and no global memory access per round
// (a round over global memory -- the distances in `temp`, the winner's coordinates fetched by all -- takes seven
// times as long; 512 threads with twice the points each: 5.2 instead of 4.35 ms).  Larger samples run that slower form.
constexpr int kFpsThreads = 1024;
constexpr int kFpsPer = 16;
constexpr int kFpsWaves = kFpsThreads / 64;
static_assert(kFpsWaves <= 16 && (kFpsWaves & (kFpsWaves - 1)) == 0, "the wavefronts' candidates of a round are compared within one row of 16 lanes");
__global__ __launch_bounds__(kFpsThreads) void point_fps_k(const float *__restrict__ xyz, const int *__restrict__ nv_in,
                                                           const int *__restrict__ nv_out, int B, int64_t Np, int64_t Mp,
                                                           float *__restrict__ temp, int *__restrict__ index_out)
{
#pragma clang fp contract(off)
    __shared__ float s_best[kFpsThreads / 64];
    __shared__ int s_idx[kFpsThreads / 64];
    __shared__ int s_cur;
    __shared__ float s_xyz[3];
    const int b = blockIdx.x;
    if (b >= B) return;
    const int n0 = b ? nv_in[b - 1] : 0, n1 = nv_in[b] < Np ? nv_in[b] : (int)Np;
    const int m0 = b ? nv_out[b - 1] : 0, m1 = nv_out[b] < Mp ? nv_out[b] : (int)Mp;
    const int N = n1 - n0, M = m1 - m0;
    if (M <= 0) return;
    if (threadIdx.x == 0) index_out[m0] = N > 0 ? n0 : 0;
    if (N <= 0) {
        for (int j = 1 + threadIdx.x; j < M; j += kFpsThreads) index_out[m0 + j] = 0;
        return;
    }
    // arg-max over a wavefront: larger value, then lower index.  Within rows of 16 lanes the candidates move through
    // DPP operands (lane pairs, quad halves, mirrored halves of 8 and 16: every lane of a row ends up with the row's
    // winner; all lanes of the wavefront are active here), across the four rows through the LDS crossbar.
    auto take_better = [](float &best, int &besti, float ob, int oi) {
        const bool take = ob > best || (ob == best && oi < besti);
        best = take ? ob : best;
        besti = take ? oi : besti;
    };
    auto row_argmax = [&](float &best, int &besti) {
#define PM_FPS_DPP(ctrl)                                                                                                  \
    take_better(best, besti, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, best), ctrl, 0xF, 0xF, true)), \
                __builtin_amdgcn_update_dpp(0, besti, ctrl, 0xF, 0xF, true))
        PM_FPS_DPP(0xB1);
        PM_FPS_DPP(0x4E);
        PM_FPS_DPP(0x141);
        PM_FPS_DPP(0x140);
#undef PM_FPS_DPP
    };
    auto wave_argmax = [&](float &best, int &besti) {
        row_argmax(best, besti);
#pragma unroll
        for (int o = 16; o <= 32; o <<= 1) take_better(best, besti, __shfl_xor(best, o, 64), __shfl_xor(besti, o, 64));
    };
    if (N <= kFpsThreads * kFpsPer) {
        const int per = (N + kFpsThreads - 1) / kFpsThreads;      // points of the busiest thread
        float px[kFpsPer], py[kFpsPer], pz[kFpsPer], td[kFpsPer];
#pragma unroll
        for (int i = 0; i < kFpsPer; ++i) {
            const int k = threadIdx.x + i * kFpsThreads;
            const bool in = k < N;
            const float *p = xyz + (int64_t)(n0 + (in ? k : 0)) * 3;
            px[i] = p[0]; py[i] = p[1]; pz[i] = p[2];
            td[i] = in ? 1e38f : -1.f;                            // (a distance is never below zero: no point there wins)
        }
        float x1 = xyz[(int64_t)n0 * 3], y1 = xyz[(int64_t)n0 * 3 + 1], z1 = xyz[(int64_t)n0 * 3 + 2];
        for (int j = 1; j < M; ++j) {
            float best = -1.f;
            int besti = n0;
#pragma unroll
            for (int i = 0; i < kFpsPer; ++i) {
                if (i < per) {
                    const float dx = px[i] - x1, dy = py[i] - y1, dz = pz[i] - z1;
                    const float d = (dx * dx + dy * dy) + dz * dz;
                    const float d2 = d < td[i] ? d : td[i];
                    td[i] = d2;
                    const bool up = d2 > best;
                    best = up ? d2 : best;
                    besti = up ? n0 + (int)threadIdx.x + i * kFpsThreads : besti;
                }
            }
            wave_argmax(best, besti);
            if ((threadIdx.x & 63) == 0) { s_best[threadIdx.x >> 6] = best; s_idx[threadIdx.x >> 6] = besti; }
            __syncthreads();
            // lane l looks at the candidate of wavefront l % kFpsWaves; the row exchange leaves the winner in every lane
            float bb = s_best[threadIdx.x & (kFpsWaves - 1)];
            int bi = s_idx[threadIdx.x & (kFpsWaves - 1)];
            row_argmax(bb, bi);
            if (threadIdx.x == 0) index_out[m0 + j] = bi;
            const int rel = bi - n0;
            if ((rel & (kFpsThreads - 1)) == (int)threadIdx.x) {  // my point: its slot is rel / kFpsThreads
                float cx = px[0], cy = py[0], cz = pz[0];
#pragma unroll
                for (int i = 1; i < kFpsPer; ++i)
                    if (i == rel / kFpsThreads) { cx = px[i]; cy = py[i]; cz = pz[i]; }
                s_xyz[0] = cx; s_xyz[1] = cy; s_xyz[2] = cz;
            }
            __syncthreads();
            x1 = s_xyz[0]; y1 = s_xyz[1]; z1 = s_xyz[2];
        }
        return;
    }
    for (int k = threadIdx.x; k < N; k += kFpsThreads) temp[n0 + k] = 1e38f;
    int cur = n0;
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
        wave_argmax(best, besti);
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

// grid workspace: head, cells, sorted points, then the sort's buffers (keys in/out, ids in/out, temporary storage)
static size_t grid_slot(int64_t Np) { return (((size_t)Np * 4) + 255) & ~size_t(255); }
static size_t grid_search_bytes(int64_t Np) { return kGridHead + (size_t)kGridMaxCells * sizeof(int2) + 4 * grid_slot(Np); }

extern "C" size_t pmesh_point_grid_workspace_bytes(int64_t Np)
{
    if (Np < 0) Np = 0;
    return grid_search_bytes(Np) + 4 * grid_slot(Np) + ((sort_pairs_temp_bytes(Np, kGridKeyBits) + 255) & ~size_t(255));
}

extern "C" int pmesh_point_grid_build(const float *database, const int32_t *nv_database, int B, int64_t Np, float reach,
                                      void *grid, size_t grid_bytes, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(B > 0 && B <= kGridMaxCells && Np > 0 && Np <= INT32_MAX, "point_grid_build: bad sizes");
    PM_REQUIRE(reach > 0 || (reach < 0 && reach >= -64.f), "point_grid_build: the reach of the searches must be positive (or -c for c cells per point)");
    PM_REQUIRE(database && nv_database && grid, "point_grid_build: null pointer");
    PM_REQUIRE(((uintptr_t)grid & 255) == 0, "point_grid_build: the workspace must be aligned to 256 bytes");
    PM_REQUIRE(grid_bytes >= pmesh_point_grid_workspace_bytes(Np), "point_grid_build: workspace too small (%zu bytes)", grid_bytes);
    hipStream_t st = (hipStream_t)stream;
    char *base = (char *)grid;
    PointGrid *G = (PointGrid *)base;
    int2 *cells = (int2 *)(base + kGridHead);
    float4 *pts = (float4 *)(base + kGridHead + (size_t)kGridMaxCells * sizeof(int2));
    char *sortb = base + grid_search_bytes(Np);
    const size_t slot = grid_slot(Np);
    unsigned *keys_in = (unsigned *)sortb, *keys_out = (unsigned *)(sortb + slot);
    int *ids_in = (int *)(sortb + 2 * slot), *ids_out = (int *)(sortb + 3 * slot);
    void *temp = sortb + 4 * slot;
    const unsigned pb = (unsigned)ceil_div(Np, kBlock);
    grid_clear_k<<<dim3(kGridMaxCells / kBlock), dim3(kBlock), 0, st>>>(G, cells);
    grid_bbox_k<<<dim3((unsigned)ceil_div(Np, (int64_t)kBlock * kBboxPer)), dim3(kBlock), 0, st>>>(database, nv_database, B, Np, G);
    grid_dims_k<<<dim3(1), dim3(64), 0, st>>>(G, B, reach, ceil_div(Np, (int64_t)B));
    grid_keys_k<<<dim3(pb), dim3(kBlock), 0, st>>>(database, nv_database, B, Np, G, keys_in, ids_in);
    PM_LAUNCHED("point_grid_build");
    const hipError_t e = sort_pairs(temp, sort_pairs_temp_bytes(Np, kGridKeyBits), keys_in, keys_out, ids_in, ids_out, Np,
                                    kGridKeyBits, st);
    PM_REQUIRE(e == hipSuccess, "point_grid_build: radix sort failed: %s", hipGetErrorString(e));
    grid_cells_k<<<dim3(pb), dim3(kBlock), 0, st>>>(database, keys_out, ids_out, Np, cells, pts);
    PM_LAUNCHED("point_grid_build");
    return 0;
}

#define PM_GRID_PARTS(name)                                                                                             \
    PM_REQUIRE(grid && Np > 0, name ": no grid");                                                                       \
    const PointGrid *G = (const PointGrid *)grid;                                                                       \
    const int2 *cells = (const int2 *)((const char *)grid + kGridHead);                                                 \
    const float4 *pts = (const float4 *)((const char *)grid + kGridHead + (size_t)kGridMaxCells * sizeof(int2))

extern "C" int pmesh_point_range_count_grid(const void *grid, const float *database, const float *query,
                                            const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                            float radius, int nn_sample, int32_t *count, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(radius > 0 && nn_sample > 0, "point_range_count: radius and nn_sample must be positive");
    PM_QUERY_DIMS("point_range_count");
    PM_REQUIRE(count, "point_range_count: null pointer");
    PM_GRID_PARTS("point_range_count");
    point_count_grid_k<0><<<dim3((unsigned)ceil_div(Mp, kQPerBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, query, nv_query, B, Mp, radius, nn_sample, count);
    PM_LAUNCHED("point_range_count");
    return 0;
}

extern "C" int pmesh_point_range_fill_grid(const void *grid, const float *database, const float *query,
                                           const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                           float radius, const int64_t *cnt_info, int64_t Nout, int32_t *nn_index, float *nn_dist,
                                           pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(radius > 0 && Nout >= 0, "point_range_fill: bad arguments");
    PM_QUERY_DIMS("point_range_fill");
    if (Nout == 0) return 0;
    PM_REQUIRE(cnt_info && nn_index && nn_dist, "point_range_fill: null pointer");
    PM_GRID_PARTS("point_range_fill");
    point_fill_grid_k<0><<<dim3((unsigned)ceil_div(Mp, kQPerBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, database, query, nv_query, B, Np, Mp, radius, 1, cnt_info, Nout, nn_index, nn_dist);
    point_fill_long_k<0><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, database, query, nv_query, B, Np, Mp, radius, 1, cnt_info, Nout, nn_index, nn_dist);
    PM_LAUNCHED("point_range_fill");
    return 0;
}

extern "C" int pmesh_point_cube_count_grid(const void *grid, const float *database, const float *query,
                                           const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                           float length, int nn_sample, int32_t *count, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(length > 0 && nn_sample > 0, "point_cube_count: length and nn_sample must be positive");
    PM_QUERY_DIMS("point_cube_count");
    PM_REQUIRE(count, "point_cube_count: null pointer");
    PM_GRID_PARTS("point_cube_count");
    point_count_grid_k<1><<<dim3((unsigned)ceil_div(Mp, kQPerBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, query, nv_query, B, Mp, length, nn_sample, count);
    PM_LAUNCHED("point_cube_count");
    return 0;
}

extern "C" int pmesh_point_cube_fill_grid(const void *grid, const float *database, const float *query,
                                          const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                          float length, int grid_size, const int64_t *cnt_info, int64_t Nout, int32_t *nn_index,
                                          pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(length > 0 && grid_size > 0 && Nout >= 0, "point_cube_fill: bad arguments");
    PM_QUERY_DIMS("point_cube_fill");
    if (Nout == 0) return 0;
    PM_REQUIRE(cnt_info && nn_index, "point_cube_fill: null pointer");
    PM_GRID_PARTS("point_cube_fill");
    point_fill_grid_k<1><<<dim3((unsigned)ceil_div(Mp, kQPerBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, database, query, nv_query, B, Np, Mp, length, grid_size, cnt_info, Nout, nn_index, nullptr);
    point_fill_long_k<1><<<dim3((unsigned)ceil_div(Mp, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, database, query, nv_query, B, Np, Mp, length, grid_size, cnt_info, Nout, nn_index, nullptr);
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

extern "C" int pmesh_point_knn3_grid(const void *grid, const float *database, const float *query, const int32_t *nv_database,
                                     const int32_t *nv_query, int B, int64_t Np, int64_t Mp, int32_t *nn_index, float *nn_dist,
                                     pmesh_stream_t stream)
{
    clear_error();
    PM_QUERY_DIMS("point_knn3_grid");
    PM_REQUIRE(nn_index && nn_dist, "point_knn3_grid: null pointer");
    PM_GRID_PARTS("point_knn3_grid");
    point_knn3_grid_k<<<dim3((unsigned)ceil_div(Mp, kQPerBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        G, cells, pts, query, nv_database, nv_query, B, Mp, nn_index, nn_dist);
    PM_LAUNCHED("point_knn3_grid");
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
