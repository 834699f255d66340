// One round of quadric-error mesh decimation (the producer of vt_replace / vt_map): the arithmetic kernels and the
// serial vertex clustering, in a deterministic re-specification of picasso/mesh/pi_modules/source/decimate_gpu.cu.
//
// The reference accumulates vertex quadrics with float atomics, sorts with unstable comparators and clusters on the
// host in whatever order the sorts leave ties in, so its vt_replace / vt_map change from run to run.  Here every
// sum runs in a fixed order and every sort has a total order:
//   vertex quadric   face contributions in ascending (facet, corner) order (vertex CSR), then boundary-edge
//                    contributions in ascending (vi, vj) order (a second CSR over the boundary edges' endpoints)
//   candidate edges  unique (vi < vj) pairs, ordered by (sample, cost, a 32-bit mix of (vi, vj), vi, vj): the mix keeps
//                    the many equal-cost edges of flat regions from lining up along the vertex numbering
//   clustering       the reference's two greedy passes over that order (clusterVertices, decimate_gpu.cu:561-614)
// The sorts, scans and compactions between these steps are index plumbing done by the caller (radix sorts of
// integer keys); this file holds what computes.
#include "common.h"
#include "../../include/picasso_mesh.h"
#include <vector>

// Every product and sum of this file is rounded on its own (no fused multiply-adds): the quadrics and costs are then
// the float32 values that the same expressions give anywhere, and the contraction order that follows from the costs
// can be checked against a float32 restatement from the mesh alone.
#pragma clang fp contract(off)

namespace pmesh {

constexpr float kAreaMagnitude = 100.0f;        // areas in dm^2 for inputs in metres (decimate_gpu.cu:16)
constexpr float kRrefEps = 2.220446049250313e-16f;
constexpr float kRcondEps = 1e-6f;

// plane (n, d) -> the ten distinct entries of [n; d] [n; d]^T in the order q11 q12 q13 q22 q23 q33 q14 q24 q34 q44
__device__ __forceinline__ void plane_quadric(const float n[3], float d, float (&Q)[10])
{
    Q[0] = n[0] * n[0]; Q[1] = n[0] * n[1]; Q[2] = n[0] * n[2];
    Q[3] = n[1] * n[1]; Q[4] = n[1] * n[2]; Q[5] = n[2] * n[2];
    Q[6] = n[0] * d;    Q[7] = n[1] * d;    Q[8] = n[2] * d;
    Q[9] = d * d;
}

// Quadric of every vertex from its incident facets (decimate_gpu.cu:220-247), summed in adjacency order.
// geometry rows: unit normal, plane offset d, area.  rowptr / colidx: vertex CSR of `face` (entries 3 f + corner).
__global__ __launch_bounds__(kBlock) void vertex_quadric_k(const float *__restrict__ geometry, const int *__restrict__ rowptr,
                                                           const int *__restrict__ colidx, float *__restrict__ quadric,
                                                           int64_t Nv, int use_area)
{
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= Nv) return;
    float S[10];
#pragma unroll
    for (int i = 0; i < 10; ++i) S[i] = 0.f;
    for (int e = rowptr[v]; e < rowptr[v + 1]; ++e) {
        const float *g = geometry + (int64_t)(colidx[e] / 3) * 5;
        const float n[3] = {g[0], g[1], g[2]};
        float Q[10];
        plane_quadric(n, g[3], Q);
        const float w = use_area ? g[4] * kAreaMagnitude / 3 : 1.0f;
#pragma unroll
        for (int i = 0; i < 10; ++i) S[i] += Q[i] * w;
    }
#pragma unroll
    for (int i = 0; i < 10; ++i) quadric[v * 10 + i] = S[i];
}

// Weighted quadric of every boundary edge (an edge that belongs to one facet): the plane through the edge
// perpendicular to that facet (decimate_gpu.cu:304-362).  rows: (nb, 10); each row is added to both end points.
__global__ __launch_bounds__(kBlock) void boundary_quadric_k(const float *__restrict__ vertex, const float *__restrict__ geometry,
                                                             const int *__restrict__ edge_vi, const int *__restrict__ edge_vj,
                                                             const int *__restrict__ edge_face, float *__restrict__ rows,
                                                             int64_t nb, int D, int use_area, float wgt_bnd)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= nb) return;
    const float *pi = vertex + (int64_t)edge_vi[i] * D, *pj = vertex + (int64_t)edge_vj[i] * D;
    const float *n = geometry + (int64_t)edge_face[i] * 5;
    const float dx[3] = {pj[0] - pi[0], pj[1] - pi[1], pj[2] - pi[2]};
    float b[3] = {n[1] * dx[2] - n[2] * dx[1], n[2] * dx[0] - n[0] * dx[2], n[0] * dx[1] - n[1] * dx[0]};
    float len = sqrtf(b[0] * b[0] + b[1] * b[1] + b[2] * b[2]);
    len = len > 1e-20f ? len : 1e-20f;
    b[0] /= len; b[1] /= len; b[2] /= len;
    const float d = -(b[0] * pi[0] + b[1] * pi[1] + b[2] * pi[2]);
    const float w = use_area ? (dx[0] * dx[0] + dx[1] * dx[1] + dx[2] * dx[2]) * kAreaMagnitude * wgt_bnd : wgt_bnd;
    float Q[10];
    plane_quadric(b, d, Q);
#pragma unroll
    for (int k = 0; k < 10; ++k) rows[i * 10 + k] = Q[k] * w;
}

// x^T A x + 2 b.x + c
__device__ __forceinline__ float quadric_error(const float x[3], const float A[3][3], const float b[3], float c)
{
    return ((x[0] * A[0][0] + x[1] * A[1][0] + x[2] * A[2][0]) * x[0] + (x[0] * A[0][1] + x[1] * A[1][1] + x[2] * A[2][1]) * x[1] +
            (x[0] * A[0][2] + x[1] * A[1][2] + x[2] * A[2][2]) * x[2]) +
           (x[0] * b[0] + x[1] * b[1] + x[2] * b[2]) * 2 + c;
}

// One step of the elimination at row I, column J (both fixed at compile time, so that the 3 x 7 matrix lives in
// registers): the largest entry of the column from row I down becomes the pivot; a column whose candidates are all
// negligible is cleared and left.  Returns whether a pivot was taken.
template <int I, int J>
__device__ __forceinline__ bool rref_step(float (&M)[3][7], float tol)
{
    float p = fabsf(M[I][J]);
    int k = I;
#pragma unroll
    for (int r = I + 1; r < 3; ++r)
        if (p < fabsf(M[r][J])) { p = fabsf(M[r][J]); k = r; }
    if (p <= tol) {
#pragma unroll
        for (int r = I; r < 3; ++r) M[r][J] = 0.f;
        return false;
    }
#pragma unroll
    for (int r = I + 1; r < 3; ++r)
        if (k == r) {
#pragma unroll
            for (int c = J; c < 7; ++c) { const float t = M[I][c]; M[I][c] = M[r][c]; M[r][c] = t; }
        }
    const float pivot = M[I][J];
#pragma unroll
    for (int c = J; c < 7; ++c) M[I][c] = M[I][c] / pivot;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
        if (r == I) continue;
        const float f = M[r][J];
#pragma unroll
        for (int c = J; c < 7; ++c) M[r][c] -= f * M[I][c];
    }
    return true;
}

// column J with `i` rows done so far (i <= J)
template <int J>
__device__ __forceinline__ void rref_column(float (&M)[3][7], float tol, int &i)
{
    if (i == 0) i += rref_step<0, J>(M, tol);
    else if (J >= 1 && i == 1) i += rref_step<1, (J >= 1 ? J : 1)>(M, tol);
    else if (J >= 2 && i == 2) i += rref_step<2, (J >= 2 ? J : 2)>(M, tol);
}

// Reduced row echelon form of [A | b | I] with partial pivoting and the negligible-column rule of the reference's
// RrefDim3 (decimate_gpu.cu:79-193): x = -A^-1 b, and the reciprocal condition number 1 / (|A|_inf |A^-1|_inf).
__device__ __forceinline__ float solve3(const float A[3][3], const float b[3], float (&x)[3])
{
    float M[3][7];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            M[r][c] = A[r][c];
            M[r][c + 4] = r == c ? 1.f : 0.f;
        }
        M[r][3] = b[r];
    }
    float normA = 0.f;
#pragma unroll
    for (int r = 0; r < 3; ++r) normA = fmaxf(normA, fabsf(M[r][0]) + fabsf(M[r][1]) + fabsf(M[r][2]));
    const float tol = kRrefEps * 7 * normA;
    int i = 0;                                        // rows done; the columns are walked until three are
    rref_column<0>(M, tol, i);
    rref_column<1>(M, tol, i);
    rref_column<2>(M, tol, i);
    rref_column<3>(M, tol, i);
    rref_column<4>(M, tol, i);
    rref_column<5>(M, tol, i);
    rref_column<6>(M, tol, i);
    x[0] = -M[0][3]; x[1] = -M[1][3]; x[2] = -M[2][3];
    float normInv = 0.f;
#pragma unroll
    for (int r = 0; r < 3; ++r) normInv = fmaxf(normInv, fabsf(M[r][4]) + fabsf(M[r][5]) + fabsf(M[r][6]));
    return 1.0f / (normA * normInv);
}

// Cost of contracting each candidate edge (decimate_gpu.cu:365-404): the error of the summed quadric at its
// minimiser when the 3 x 3 system is well conditioned, else the smaller of the errors at the two end points.
__global__ __launch_bounds__(kBlock) void edge_cost_k(const float *__restrict__ vertex, const float *__restrict__ quadric,
                                                      const int *__restrict__ edge_vi, const int *__restrict__ edge_vj,
                                                      float *__restrict__ cost, int64_t ne, int D)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= ne) return;
    const int vi = edge_vi[e], vj = edge_vj[e];
    float Q[10];
#pragma unroll
    for (int k = 0; k < 10; ++k) Q[k] = quadric[(int64_t)vi * 10 + k] + quadric[(int64_t)vj * 10 + k];
    const float A[3][3] = {{Q[0], Q[1], Q[2]}, {Q[1], Q[3], Q[4]}, {Q[2], Q[4], Q[5]}};
    const float b[3] = {Q[6], Q[7], Q[8]};
    float x[3];
    const float rcond = solve3(A, b, x);
    if (rcond > kRcondEps) {
        cost[e] = quadric_error(x, A, b, Q[9]);
    } else {
        const float ei = quadric_error(vertex + (int64_t)vi * D, A, b, Q[9]), ej = quadric_error(vertex + (int64_t)vj * D, A, b, Q[9]);
        cost[e] = ei < ej ? ei : ej;
    }
}

// ----------------------------------------------------------------------------------------
// Candidate edges from the vertex adjacency, without a sort of the whole edge list: the edges (v, w), v < w, of the
// facets around v are exactly those whose lower end is v, so one thread per vertex collects the other corners w > v
// of its row's facets, orders them, and writes the distinct ones -- which leaves the batch's unique edges in
// ascending (vi, vj) order (decimate_gpu.cu:250-297 sorts all 3 Nf facet edges instead).  With each edge: how many
// facet sides hold it (1 = boundary edge) and the lowest facet that does.
// A row's candidates (two per adjacency entry) are ordered in LDS up to kEdgeLocal of them, beyond that
// in the row's own segment of `spill` (4 ints per adjacency entry, 12 Nf in all; only touched when some row is that
// long: without a spill area such a row raises *need_spill and is left out, and the caller comes back with one).
constexpr int kEdgeLocal = 32;          // candidates of a row ordered in LDS (rows of up to 16 adjacency entries)
constexpr int kEdgeBlock = 128;         // threads per workgroup: 2 x 32 x 128 ints of LDS

struct EdgeRow {
    int n;          // candidates w > v, ordered ascending by (w, facet); -1 = too long for LDS and no spill area
    int *w, *f;
    int stride;     // element i of the lists sits at w[i * stride]
};

__device__ __forceinline__ void edge_row_collect(const int *__restrict__ face, const int *__restrict__ rowptr,
                                                 const int *__restrict__ colidx, int64_t Nv, int v, int *lw, int *lf,
                                                 int *__restrict__ spill, EdgeRow &row)
{
    const int e0 = rowptr[v], e1 = rowptr[v + 1];
    const bool big = 2 * (e1 - e0) > kEdgeLocal;
    if (big && !spill) {
        row.n = -1;                      // the caller comes back with a spill area
        return;
    }
    row.w = big ? spill + 4 * (int64_t)e0 : lw;
    row.f = big ? spill + 4 * (int64_t)e0 + 2 * (e1 - e0) : lf;
    row.stride = big ? 1 : kEdgeBlock;
    const int sd = row.stride;
    int n = 0;
    for (int e = e0; e < e1; ++e) {
        const int en = colidx[e], fc = en / 3, c = en - 3 * fc;
#pragma unroll
        for (int d = 1; d <= 2; ++d) {
            const int w = face[3 * (int64_t)fc + (c + d) % 3];
            if (w > v && w < Nv) {
                // insertion by (w, facet): rows are short
                int i = n++;
                while (i > 0 && (row.w[(i - 1) * sd] > w || (row.w[(i - 1) * sd] == w && row.f[(i - 1) * sd] > fc))) {
                    row.w[i * sd] = row.w[(i - 1) * sd];
                    row.f[i * sd] = row.f[(i - 1) * sd];
                    --i;
                }
                row.w[i * sd] = w;
                row.f[i * sd] = fc;
            }
        }
    }
    row.n = n;
}

// counts[v] = distinct edges whose lower end is v, counts[Nv + v] = those held by exactly one facet side
__global__ __launch_bounds__(kEdgeBlock) void edge_list_count_k(const int *__restrict__ face, const int *__restrict__ rowptr,
                                                                const int *__restrict__ colidx, int64_t Nv, int *__restrict__ counts,
                                                                int *__restrict__ spill, int *__restrict__ need_spill)
{
    __shared__ int lw[kEdgeLocal * kEdgeBlock], lf[kEdgeLocal * kEdgeBlock];
    const int64_t v = (int64_t)blockIdx.x * kEdgeBlock + threadIdx.x;
    if (v >= Nv) return;
    EdgeRow row;
    edge_row_collect(face, rowptr, colidx, Nv, (int)v, lw + threadIdx.x, lf + threadIdx.x, spill, row);
    if (row.n < 0) *need_spill = 1;
    const int sd = row.stride;
    int distinct = 0, single = 0;
    for (int i = 0; i < row.n;) {
        int j = i + 1;
        while (j < row.n && row.w[j * sd] == row.w[i * sd]) ++j;
        ++distinct;
        single += (j - i) == 1;
        i = j;
    }
    counts[v] = distinct;
    counts[Nv + v] = single;
}

// offsets = exclusive running totals of counts
__global__ __launch_bounds__(kEdgeBlock) void edge_list_fill_k(const int *__restrict__ face, const int *__restrict__ rowptr,
                                                               const int *__restrict__ colidx, int64_t Nv, const int *__restrict__ offsets,
                                                               int *__restrict__ edge_vi, int *__restrict__ edge_vj,
                                                               int *__restrict__ bnd_vi, int *__restrict__ bnd_vj,
                                                               int *__restrict__ bnd_face, int *__restrict__ spill)
{
    __shared__ int lw[kEdgeLocal * kEdgeBlock], lf[kEdgeLocal * kEdgeBlock];
    const int64_t v = (int64_t)blockIdx.x * kEdgeBlock + threadIdx.x;
    if (v >= Nv) return;
    EdgeRow row;
    edge_row_collect(face, rowptr, colidx, Nv, (int)v, lw + threadIdx.x, lf + threadIdx.x, spill, row);
    const int sd = row.stride;
    int o = offsets[v], ob = offsets[Nv + v];
    for (int i = 0; i < row.n;) {
        int j = i + 1;
        while (j < row.n && row.w[j * sd] == row.w[i * sd]) ++j;
        edge_vi[o] = (int)v;
        edge_vj[o] = row.w[i * sd];
        ++o;
        if (j - i == 1) {
            bnd_vi[ob] = (int)v;
            bnd_vj[ob] = row.w[i * sd];
            bnd_face[ob] = row.f[i * sd];
            ++ob;
        }
        i = j;
    }
}

// ----------------------------------------------------------------------------------------
// The two greedy passes of the vertex clustering on the device, with the result of the serial host routine below.
//
// First pass (disjoint pairs, cheapest edge first).  For a total order of the edges the serial greedy choice is the
// fixed point of: an edge both of whose end points are free, and which is the first such edge at BOTH of them, is
// chosen; its end points are covered; repeat.  Every round costs two sweeps over the edge list (propose with an
// integer atomic minimum per end point, select).  A budget that runs out stops the serial pass after its first
// n_remove choices, which are the n_remove lowest-ranked edges of the fixed point: the caller cuts the chosen set
// by rank.
// Second pass (runs only when the first one did not exhaust the budget, i.e. after a MAXIMAL matching: no edge has
// two free end points).  A free vertex then joins the cluster of the covered end of its first edge in the order
// whose cluster has a representative other than vertex 0, and vertices that join never enable others to (all their
// neighbours are covered already): one atomic minimum per edge finds each free vertex's edge, the caller cuts by
// rank again, one sweep applies.
// All atomics are integer minima / additions: the result does not depend on their order.
constexpr int kNoEdge = 0x7FFFFFFF;

__global__ __launch_bounds__(kBlock) void fill_int_k(int *__restrict__ p, int v, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = v;
}

// status[1] <- 1 if an edge is not (vi < vj) inside [0, Nv): such an edge takes no part (the serial routine refuses it)
__global__ __launch_bounds__(kBlock) void match_check_k(const int *__restrict__ evi, const int *__restrict__ evj, int64_t E,
                                                        int64_t Nv, int *__restrict__ status)
{
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= E) return;
    const int a = evi[r], b = evj[r];
    if (!(a >= 0 && a < b && b < Nv)) status[1] = 1;
}

__global__ __launch_bounds__(kBlock) void match_propose_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                          const int *__restrict__ rank, int64_t E, int64_t Nv,
                                                          const int *__restrict__ state, int *__restrict__ best)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    const int a = evi[e], b = evj[e];
    if (!(a >= 0 && a < b && b < Nv)) return;
    if (state[a] | state[b]) return;
    const int r = rank[e];
    atomicMin(best + a, r);
    atomicMin(best + b, r);
}

__global__ __launch_bounds__(kBlock) void match_select_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                         const int *__restrict__ rank, int64_t E, int64_t Nv,
                                                         int *__restrict__ state, const int *__restrict__ best,
                                                         int *__restrict__ chosen)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    const int a = evi[e], b = evj[e];
    if (!(a >= 0 && a < b && b < Nv)) return;
    const int r = rank[e];
    if (best[a] == r && best[b] == r) {
        chosen[e] = 1;
        state[a] = 1;
        state[b] = 1;
    }
}

// status[0] <- 1 if an edge with two free end points is left
__global__ __launch_bounds__(kBlock) void match_left_k(const int *__restrict__ evi, const int *__restrict__ evj, int64_t E,
                                                       int64_t Nv, const int *__restrict__ state, int *__restrict__ status)
{
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= E) return;
    const int a = evi[r], b = evj[r];
    if (!(a >= 0 && a < b && b < Nv)) return;
    if (!(state[a] | state[b])) status[0] = 1;
}

__global__ __launch_bounds__(kBlock) void contract_pairs_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                           const int *__restrict__ keep, int64_t E, int *__restrict__ vt_replace)
{
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= E || !keep[r]) return;
    vt_replace[evi[r]] = -evj[r];          // vi is contracted into vj (decimate_gpu.cu:568-585)
    vt_replace[evj[r]] = 1;
}

// One 64-bit sort key per candidate edge: the sample of vi (number of running totals <= vi, fewer than 128 samples) in
// the top byte, below it the cost as an integer that orders like the float (-0 = +0, NaN above everything), the 24-bit
// mix of the end points at the bottom.
__global__ __launch_bounds__(kBlock) void contraction_keys_k(const float *__restrict__ cost, const int *__restrict__ evi,
                                                             const int *__restrict__ evj, const int *__restrict__ nv_cumsum, int B,
                                                             int64_t E, int64_t *__restrict__ keys)
{
    __shared__ int s_end[128];
    if (threadIdx.x < 128) s_end[threadIdx.x] = (int)threadIdx.x < B ? nv_cumsum[threadIdx.x] : INT32_MAX;
    __syncthreads();
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    const int a = evi[e], b = evj[e];
    const float c = cost[e] + 0.0f;
    const int64_t bits = __float_as_int(c);
    int64_t ordered = bits >= 0 ? bits : -(bits + 2147483648LL) - 1;     // negative floats: larger magnitude, lower
    if (c != c) ordered = 2147483647;
    uint32_t h = (uint32_t)a * 0x9E3779B1u + (uint32_t)b * 0x85EBCA77u;
    h ^= h >> 15;
    h *= 0x2C1B3C6Du;
    h ^= h >> 12;
    h *= 0x297A2D39u;
    h ^= h >> 15;
    int lo = 0, hi = B;                                                  // first running total above vi
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (s_end[mid] <= a) lo = mid + 1;
        else hi = mid;
    }
    keys[e] = ((int64_t)lo << 56) | ((ordered + 2147483648LL) << 24) | (int64_t)(h >> 8);
}

// the contraction order turned round: rank[perm[i]] = i, edge_sample[perm[i]] = sample[i]
__global__ __launch_bounds__(kBlock) void cluster_ranks_k(const int64_t *__restrict__ perm, const int *__restrict__ sample, int64_t E,
                                                          int *__restrict__ rank, int *__restrict__ edge_sample)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= E) return;
    const int64_t e = perm[i];
    if (e < 0 || e >= E) return;
    rank[e] = (int)i;
    edge_sample[e] = sample[i];
}

__global__ __launch_bounds__(kBlock) void cluster_flags_by_rank_k(const int *__restrict__ flags, const int *__restrict__ rank, int64_t E,
                                                                  int *__restrict__ by_rank)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    const int r = rank[e];
    if (r >= 0 && r < E) by_rank[r] = flags[e] != 0;
}

// flagged edges ahead of sample b in the contraction order (run: inclusive running total of the flags in that order)
__device__ __forceinline__ int flagged_before(const int *__restrict__ run, const int64_t *__restrict__ first, int b)
{
    const int64_t at = first[b];
    return at > 0 ? run[at - 1] : 0;
}

// keeps a flagged edge when it is among the first allowance[sample] flagged edges of its sample
__global__ __launch_bounds__(kBlock) void cluster_cut_k(const int *__restrict__ flags, const int *__restrict__ rank,
                                                        const int *__restrict__ edge_sample, const int *__restrict__ run,
                                                        const int64_t *__restrict__ first, const int *__restrict__ allowance, int64_t E,
                                                        int B, int *__restrict__ keep)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    int k = 0;
    const int b = edge_sample[e], r = rank[e];
    if (flags[e] && b >= 0 && b < B && r >= 0 && r < E) k = run[r] - flagged_before(run, first, b) <= allowance[b];
    keep[e] = k;
}

__global__ __launch_bounds__(kBlock) void cluster_budget_k(const int *__restrict__ run, const int64_t *__restrict__ first,
                                                           const int *__restrict__ allowance, int B, int *__restrict__ open,
                                                           int *__restrict__ left)
{
    const int b = blockIdx.x * kBlock + threadIdx.x;
    if (b >= B) return;
    const int taken = flagged_before(run, first, b + 1) - flagged_before(run, first, b), a = allowance[b];
    open[b] = taken < a;
    left[b] = a - (taken < a ? taken : a);
}

// the covered and the free end of an edge with exactly one covered end, and the covered end's representative
__device__ __forceinline__ bool attach_ends(int a, int b, const int *__restrict__ vt_replace, int &rep, int &fr)
{
    const int ra = vt_replace[a], rb = vt_replace[b];
    const bool ca = ra != 0, cb = rb != 0;
    if (ca == cb) return false;
    fr = ca ? b : a;
    const int cov = ca ? a : b, rc = ca ? ra : rb;
    rep = rc < 0 ? -rc : cov;
    return rep != 0;                        // -0 cannot say 'contracted into vertex 0'
}

__global__ __launch_bounds__(kBlock) void attach_propose_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                           const int *__restrict__ rank, const int *__restrict__ sample,
                                                           const int *__restrict__ open, int64_t E, int64_t Nv,
                                                           const int *__restrict__ vt_replace, int *__restrict__ first_edge)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E || !open[sample[e]]) return;
    const int a = evi[e], b = evj[e];
    if (!(a >= 0 && a < b && b < Nv)) return;
    int rep, fr;
    if (attach_ends(a, b, vt_replace, rep, fr)) atomicMin(first_edge + fr, rank[e]);
}

__global__ __launch_bounds__(kBlock) void attach_flag_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                        const int *__restrict__ rank, const int *__restrict__ sample,
                                                        const int *__restrict__ open, int64_t E, int64_t Nv,
                                                        const int *__restrict__ vt_replace, const int *__restrict__ first_edge,
                                                        int *__restrict__ attaches)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E) return;
    int flag = 0;
    const int a = evi[e], b = evj[e];
    if (open[sample[e]] && a >= 0 && a < b && b < Nv) {
        int rep, fr;
        if (attach_ends(a, b, vt_replace, rep, fr)) flag = first_edge[fr] == rank[e];
    }
    attaches[e] = flag;
}

// first_edge tells the free end of a kept edge (vt_replace is being written here and can no longer say)
__global__ __launch_bounds__(kBlock) void attach_apply_k(const int *__restrict__ evi, const int *__restrict__ evj,
                                                         const int *__restrict__ rank, const int *__restrict__ keep, int64_t E,
                                                         const int *__restrict__ first_edge, const int *__restrict__ pairs,
                                                         int *__restrict__ vt_replace)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= E || !keep[e]) return;
    const int a = evi[e], b = evj[e];
    const int fr = first_edge[a] == rank[e] ? a : b, cov = fr == a ? b : a;
    const int rc = pairs[cov];              // the first pass's entry of the covered end: not written by this kernel
    const int rep = rc < 0 ? -rc : cov;
    vt_replace[fr] = -rep;
    atomicAdd(vt_replace + rep, 1);
}

// ----------------------------------------------------------------------------------------
// After the clustering: the facets over the clusters' representatives, which of them collapse (two corners in one
// cluster), which vertices keep a facet (decimate_gpu.cu:487-496), and -- once the caller has the running totals of
// the kept vertices -- the output numbering of vertices and facets (:519-549).
__global__ __launch_bounds__(kBlock) void simplify_faces_k(const int *__restrict__ face, const int *__restrict__ vt_replace,
                                                           int64_t Nf, int64_t Nv, int *__restrict__ new_face,
                                                           unsigned char *__restrict__ degenerate, int *__restrict__ alive,
                                                           int *__restrict__ kept)
{
    const int64_t f = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (f >= Nf) return;
    int c[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int v = face[3 * f + j];
        const int r = (v >= 0 && v < Nv) ? vt_replace[v] : 0;
        c[j] = r < 0 ? -r : v;
        new_face[3 * f + j] = c[j];
    }
    const bool dg = c[0] == c[1] || c[0] == c[2] || c[1] == c[2];
    degenerate[f] = dg ? 1 : 0;
    alive[f] = dg ? 0 : 1;
    if (!dg) {
#pragma unroll
        for (int j = 0; j < 3; ++j)
            if (c[j] >= 0 && c[j] < Nv) kept[c[j]] = 1;          // (every writer writes 1)
    }
}

// kept_total = inclusive running total of kept
__global__ __launch_bounds__(kBlock) void simplify_vertex_map_k(const int *__restrict__ kept, const int *__restrict__ kept_total,
                                                                int64_t Nv, int *__restrict__ vt_map)
{
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v < Nv) vt_map[v] = kept[v] ? kept_total[v] - 1 : -1;
}

__global__ __launch_bounds__(kBlock) void simplify_face_out_k(const int *__restrict__ new_face, const unsigned char *__restrict__ degenerate,
                                                              const int *__restrict__ kept_total, int64_t Nf, int64_t Nv,
                                                              int *__restrict__ face_out)
{
    const int64_t f = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (f >= Nf) return;
    const bool dg = degenerate[f] != 0;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const int c = new_face[3 * f + j];
        face_out[3 * f + j] = (dg || c < 0 || c >= Nv) ? c : kept_total[c] - 1;       // corners of a live facet are kept vertices
    }
}

}  // namespace pmesh

using namespace pmesh;

extern "C" int pmesh_simplify_faces(const int32_t *face, const int32_t *vt_replace, int64_t Nf, int64_t Nv, int32_t *new_face,
                                    uint8_t *degenerate, int32_t *alive, int32_t *kept, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nf >= 0 && Nv >= 0 && Nv <= INT32_MAX && Nf <= INT32_MAX / 3, "simplify_faces: bad sizes");
    hipStream_t st = (hipStream_t)stream;
    if (Nv > 0) {
        PM_REQUIRE(kept, "simplify_faces: null pointer");
        fill_int_k<<<dim3((unsigned)ceil_div(Nv, kBlock)), dim3(kBlock), 0, st>>>(kept, 0, Nv);
    }
    if (Nf == 0) return 0;
    PM_REQUIRE(face && vt_replace && new_face && degenerate && alive && kept, "simplify_faces: null pointer");
    simplify_faces_k<<<dim3((unsigned)ceil_div(Nf, kBlock)), dim3(kBlock), 0, st>>>(face, vt_replace, Nf, Nv, new_face, degenerate, alive, kept);
    PM_LAUNCHED("simplify_faces");
    return 0;
}

extern "C" int pmesh_simplify_renumber(const int32_t *new_face, const uint8_t *degenerate, const int32_t *kept,
                                       const int32_t *kept_total, int64_t Nf, int64_t Nv, int32_t *vt_map, int32_t *face_out,
                                       pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nf >= 0 && Nv >= 0 && Nv <= INT32_MAX && Nf <= INT32_MAX / 3, "simplify_renumber: bad sizes");
    hipStream_t st = (hipStream_t)stream;
    if (Nv > 0) {
        PM_REQUIRE(kept && kept_total && vt_map, "simplify_renumber: null pointer");
        simplify_vertex_map_k<<<dim3((unsigned)ceil_div(Nv, kBlock)), dim3(kBlock), 0, st>>>(kept, kept_total, Nv, vt_map);
    }
    if (Nf > 0) {
        PM_REQUIRE(new_face && degenerate && kept_total && face_out, "simplify_renumber: null pointer");
        simplify_face_out_k<<<dim3((unsigned)ceil_div(Nf, kBlock)), dim3(kBlock), 0, st>>>(new_face, degenerate, kept_total, Nf, Nv, face_out);
    }
    PM_LAUNCHED("simplify_renumber");
    return 0;
}

extern "C" int pmesh_edge_list_count(const int32_t *face, const int32_t *rowptr, const int32_t *colidx, int64_t Nv, int64_t Nf,
                                     int32_t *counts, int32_t *spill, int32_t *need_spill, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nv <= INT32_MAX && Nf >= 0 && Nf <= INT32_MAX / 6, "edge_list_count: bad sizes");
    if (Nv == 0) return 0;
    PM_REQUIRE(face && rowptr && colidx && counts && need_spill, "edge_list_count: null pointer");
    edge_list_count_k<<<dim3((unsigned)ceil_div(Nv, kEdgeBlock)), dim3(kEdgeBlock), 0, (hipStream_t)stream>>>(face, rowptr, colidx, Nv, counts, spill, need_spill);
    PM_LAUNCHED("edge_list_count");
    return 0;
}

extern "C" int pmesh_edge_list_fill(const int32_t *face, const int32_t *rowptr, const int32_t *colidx, int64_t Nv, int64_t Nf,
                                    const int32_t *offsets, int32_t *edge_vi, int32_t *edge_vj, int32_t *bnd_vi, int32_t *bnd_vj,
                                    int32_t *bnd_face, int32_t *spill, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nv <= INT32_MAX && Nf >= 0 && Nf <= INT32_MAX / 6, "edge_list_fill: bad sizes");
    if (Nv == 0) return 0;
    PM_REQUIRE(face && rowptr && colidx && offsets, "edge_list_fill: null pointer");      // (the lists may be empty)
    edge_list_fill_k<<<dim3((unsigned)ceil_div(Nv, kEdgeBlock)), dim3(kEdgeBlock), 0, (hipStream_t)stream>>>(
        face, rowptr, colidx, Nv, offsets, edge_vi, edge_vj, bnd_vi, bnd_vj, bnd_face, spill);
    PM_LAUNCHED("edge_list_fill");
    return 0;
}

extern "C" int pmesh_cluster_match(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank, int64_t n_edges,
                                   int64_t Nv, int32_t *state, int32_t *best, int32_t *chosen, int32_t *status, int rounds,
                                   pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge && Nv >= 0 && Nv <= INT32_MAX && rounds >= 1 && rounds <= 64,
               "cluster_match: bad sizes");
    PM_REQUIRE(status, "cluster_match: null status");
    hipStream_t st = (hipStream_t)stream;
    fill_int_k<<<dim3(1), dim3(kBlock), 0, st>>>(status, 0, 2);
    PM_LAUNCHED("cluster_match(status)");
    if (n_edges == 0 || Nv == 0) return 0;
    PM_REQUIRE(edge_vi && edge_vj && edge_rank && state && best && chosen, "cluster_match: null pointer");
    const dim3 ge((unsigned)ceil_div(n_edges, kBlock)), gv((unsigned)ceil_div(Nv, kBlock)), blk(kBlock);
    match_check_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, n_edges, Nv, status);
    for (int i = 0; i < rounds; ++i) {
        fill_int_k<<<gv, blk, 0, st>>>(best, kNoEdge, Nv);
        match_propose_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, edge_rank, n_edges, Nv, state, best);
        match_select_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, edge_rank, n_edges, Nv, state, best, chosen);
    }
    match_left_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, n_edges, Nv, state, status);
    PM_LAUNCHED("cluster_match");
    return 0;
}

extern "C" int pmesh_cluster_contract_pairs(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *keep, int64_t n_edges,
                                            int32_t *vt_replace, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge, "cluster_contract_pairs: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(edge_vi && edge_vj && keep && vt_replace, "cluster_contract_pairs: null pointer");
    contract_pairs_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(edge_vi, edge_vj, keep, n_edges, vt_replace);
    PM_LAUNCHED("cluster_contract_pairs");
    return 0;
}

extern "C" int pmesh_cluster_ranks(const int64_t *order, const int32_t *order_sample, int64_t n_edges, int32_t *edge_rank,
                                   int32_t *edge_sample, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge, "cluster_ranks: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(order && order_sample && edge_rank && edge_sample, "cluster_ranks: null pointer");
    cluster_ranks_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(order, order_sample, n_edges, edge_rank, edge_sample);
    PM_LAUNCHED("cluster_ranks");
    return 0;
}

extern "C" int pmesh_cluster_flags_by_rank(const int32_t *flags, const int32_t *edge_rank, int64_t n_edges, int32_t *by_rank,
                                           pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge, "cluster_flags_by_rank: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(flags && edge_rank && by_rank, "cluster_flags_by_rank: null pointer");
    cluster_flags_by_rank_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(flags, edge_rank, n_edges, by_rank);
    PM_LAUNCHED("cluster_flags_by_rank");
    return 0;
}

extern "C" int pmesh_cluster_cut(const int32_t *flags, const int32_t *edge_rank, const int32_t *edge_sample, const int32_t *run,
                                 const int64_t *first, const int32_t *allowance, int64_t n_edges, int B, int32_t *keep,
                                 int32_t *sample_open, int32_t *left, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge && B >= 0, "cluster_cut: bad sizes");
    if (n_edges == 0 || B == 0) return 0;
    PM_REQUIRE(flags && edge_rank && edge_sample && run && first && allowance && keep, "cluster_cut: null pointer");
    PM_REQUIRE((sample_open == nullptr) == (left == nullptr), "cluster_cut: sample_open and left come together");
    hipStream_t st = (hipStream_t)stream;
    cluster_cut_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, st>>>(flags, edge_rank, edge_sample, run, first, allowance, n_edges, B, keep);
    if (sample_open) cluster_budget_k<<<dim3((unsigned)ceil_div(B, kBlock)), dim3(kBlock), 0, st>>>(run, first, allowance, B, sample_open, left);
    PM_LAUNCHED("cluster_cut");
    return 0;
}

extern "C" int pmesh_cluster_attach_propose(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank,
                                            const int32_t *edge_sample, const int32_t *sample_open, int64_t n_edges, int64_t Nv,
                                            const int32_t *vt_replace, int32_t *first_edge, int32_t *attaches,
                                            pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge && Nv >= 0 && Nv <= INT32_MAX, "cluster_attach_propose: bad sizes");
    if (n_edges == 0 || Nv == 0) return 0;
    PM_REQUIRE(edge_vi && edge_vj && edge_rank && edge_sample && sample_open && vt_replace && first_edge && attaches, "cluster_attach_propose: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const dim3 ge((unsigned)ceil_div(n_edges, kBlock)), gv((unsigned)ceil_div(Nv, kBlock)), blk(kBlock);
    fill_int_k<<<gv, blk, 0, st>>>(first_edge, kNoEdge, Nv);
    attach_propose_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, edge_rank, edge_sample, sample_open, n_edges, Nv, vt_replace, first_edge);
    attach_flag_k<<<ge, blk, 0, st>>>(edge_vi, edge_vj, edge_rank, edge_sample, sample_open, n_edges, Nv, vt_replace, first_edge, attaches);
    PM_LAUNCHED("cluster_attach_propose");
    return 0;
}

extern "C" int pmesh_cluster_attach(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank, const int32_t *keep,
                                    int64_t n_edges, const int32_t *first_edge, const int32_t *pairs, int32_t *vt_replace,
                                    pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges < kNoEdge, "cluster_attach: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(edge_vi && edge_vj && edge_rank && keep && first_edge && pairs && vt_replace && pairs != vt_replace, "cluster_attach: null or aliased pointer");
    attach_apply_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(edge_vi, edge_vj, edge_rank, keep, n_edges, first_edge, pairs, vt_replace);
    PM_LAUNCHED("cluster_attach");
    return 0;
}

extern "C" int pmesh_vertex_quadrics(const float *geometry, const int32_t *rowptr, const int32_t *colidx, float *quadric,
                                     int64_t Nv, int use_area, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nv <= INT32_MAX, "vertex_quadrics: bad vertex count");
    if (Nv == 0) return 0;
    PM_REQUIRE(geometry && rowptr && colidx && quadric, "vertex_quadrics: null pointer");
    vertex_quadric_k<<<dim3((unsigned)ceil_div(Nv, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(geometry, rowptr, colidx, quadric, Nv, use_area);
    PM_LAUNCHED("vertex_quadrics");
    return 0;
}

extern "C" int pmesh_boundary_quadrics(const float *vertex, const float *geometry, const int32_t *edge_vi, const int32_t *edge_vj,
                                       const int32_t *edge_face, float *rows, int64_t n_edges, int vertex_stride, int use_area,
                                       float wgt_bnd, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges <= INT32_MAX && vertex_stride >= 3, "boundary_quadrics: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(vertex && geometry && edge_vi && edge_vj && edge_face && rows, "boundary_quadrics: null pointer");
    boundary_quadric_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(
        vertex, geometry, edge_vi, edge_vj, edge_face, rows, n_edges, vertex_stride, use_area, wgt_bnd);
    PM_LAUNCHED("boundary_quadrics");
    return 0;
}

extern "C" int pmesh_edge_costs(const float *vertex, const float *quadric, const int32_t *edge_vi, const int32_t *edge_vj,
                                float *cost, int64_t n_edges, int vertex_stride, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges <= INT32_MAX && vertex_stride >= 3, "edge_costs: bad sizes");
    if (n_edges == 0) return 0;
    PM_REQUIRE(vertex && quadric && edge_vi && edge_vj && cost, "edge_costs: null pointer");
    edge_cost_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(vertex, quadric, edge_vi, edge_vj, cost,
                                                                                                   n_edges, vertex_stride);
    PM_LAUNCHED("edge_costs");
    return 0;
}

extern "C" int pmesh_contraction_keys(const float *cost, const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *nv_cumsum,
                                      int64_t n_edges, int B, int64_t *keys, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && n_edges <= INT32_MAX && B >= 0 && B < 128, "contraction_keys: bad sizes (at most 127 samples)");
    if (n_edges == 0) return 0;
    PM_REQUIRE(cost && edge_vi && edge_vj && keys && (nv_cumsum || B == 0), "contraction_keys: null pointer");
    contraction_keys_k<<<dim3((unsigned)ceil_div(n_edges, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(cost, edge_vi, edge_vj, nv_cumsum, B,
                                                                                                         n_edges, keys);
    PM_LAUNCHED("contraction_keys");
    return 0;
}

// HOST arrays.  The candidate edges of ONE sample in contraction order, its vertex range [vt_start, vt_start + vt_num)
// and the number of vertices to remove; vt_replace (whole batch, zero on entry for this sample's range) receives
// -representative for contracted vertices and the member count for representatives.
extern "C" int pmesh_cluster_vertices_host(const int32_t *edge_vi, const int32_t *edge_vj, int64_t n_edges, int32_t vt_start,
                                           int32_t vt_num, int32_t n_remove, int32_t *vt_replace)
{
    clear_error();
    PM_REQUIRE(n_edges >= 0 && vt_num >= 0, "cluster_vertices_host: bad sizes");
    if (n_edges == 0 || n_remove <= 0) return 0;
    PM_REQUIRE(edge_vi && edge_vj && vt_replace, "cluster_vertices_host: null pointer");
    std::vector<char> covered((size_t)vt_num, 0);
    auto in_range = [&](int v) { return v >= vt_start && v - vt_start < vt_num; };
    int removed = 0;
    // first pass: disjoint pairs, cheapest edges first; vi is contracted into vj (decimate_gpu.cu:568-585)
    for (int64_t i = 0; i < n_edges && removed < n_remove; ++i) {
        const int vi = edge_vi[i], vj = edge_vj[i];
        PM_REQUIRE(in_range(vi) && in_range(vj), "cluster_vertices_host: edge (%d, %d) outside the sample's vertex range", vi, vj);
        if (vi != vj && vj != 0 && !covered[vi - vt_start] && !covered[vj - vt_start]) {   // -0 cannot say 'contracted into vertex 0'
            vt_replace[vi] = -vj;
            vt_replace[vj] += 1;
            covered[vi - vt_start] = covered[vj - vt_start] = 1;
            ++removed;
        }
    }
    // second pass: a vertex still free joins the cluster of a covered neighbour, cheapest edges first (:587-613).
    // (An edge joins its FREE end to its covered end whichever of the two positions they are in; the reference
    // takes only a pair member in second position for the swap and otherwise contracts a covered vertex into a
    // free one, which leaves a chain vt_replace -> vt_replace that the pooling kernels cannot follow.)
    for (int64_t i = 0; i < n_edges && removed < n_remove; ++i) {
        int a = edge_vi[i], b = edge_vj[i];
        const bool ca = covered[a - vt_start] != 0, cb = covered[b - vt_start] != 0;
        if (ca == cb || a == b) continue;                           // both covered, or both free (the first pass ran out of budget)
        if (cb) { const int t = a; a = b; b = t; }        // a: covered, b: free
        if (vt_replace[a] < 0) a = -vt_replace[a];        // representative of a's cluster
        if (a == 0) continue;                             // -0 cannot say 'contracted into vertex 0'
        vt_replace[b] = -a;
        vt_replace[a] += 1;
        covered[b - vt_start] = 2;
        ++removed;
    }
    return 0;
}
