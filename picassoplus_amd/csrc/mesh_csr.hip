// Sorted adjacency (CSR) builders.  The scatter ops of the mesh-conv path are run as segmented
// reductions over these arrays; a stable radix sort of (row key, entry id) pairs gives every
// row its entries in ascending order, which fixes the summation order of every reduction.
#include "common.h"
#include "../../include/picasso_mesh.h"
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace pmesh {

// key of entry e = 3*facet + corner: the row it lands in, or n_rows when it lands nowhere
__global__ __launch_bounds__(kBlock) void vertex_keys_k(const int *__restrict__ face,
                                                        const int *__restrict__ vtmap, int64_t n_entries,
                                                        int64_t n_vtmap, int64_t n_rows,
                                                        unsigned *__restrict__ keys, int *__restrict__ vals)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= n_entries) return;
    int64_t key = face[e];
    if (vtmap) key = (key >= 0 && key < n_vtmap) ? vtmap[key] : -1;
    keys[e] = (key >= 0 && key < n_rows) ? (unsigned)key : (unsigned)n_rows;
    vals[e] = (int)e;
}

// key of fine vertex v: the coarse row of its cluster, or n_coarse when it has none
__global__ __launch_bounds__(kBlock) void cluster_keys_k(const int *__restrict__ vtrep,
                                                         const int *__restrict__ vtmap, int64_t n_fine,
                                                         int64_t n_coarse, unsigned *__restrict__ keys,
                                                         int *__restrict__ vals)
{
    const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (v >= n_fine) return;
    const int rp = vtrep[v];
    const int64_t rep = rp < 0 ? -(int64_t)rp : v;
    int64_t key = (rep < n_fine) ? vtmap[rep] : -1;
    keys[v] = (key >= 0 && key < n_coarse) ? (unsigned)key : (unsigned)n_coarse;
    vals[v] = (int)v;
}

// key of entry i of a strided index array: the row keys[i * stride] names, or n_rows when it names none
__global__ __launch_bounds__(kBlock) void index_keys_k(const int *__restrict__ src, int stride, int64_t n, int64_t n_rows,
                                                       unsigned *__restrict__ keys, int *__restrict__ vals)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int64_t key = src[i * stride];
    keys[i] = (key >= 0 && key < n_rows) ? (unsigned)key : (unsigned)n_rows;
    vals[i] = (int)i;
}

// rowptr[r] = first sorted position whose key is >= r, for r in [0, n_rows]
__global__ __launch_bounds__(kBlock) void rowptr_k(const unsigned *__restrict__ sorted_keys, int64_t n,
                                                   int64_t n_rows, int *__restrict__ rowptr)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i > n) return;
    const int64_t lo = (i == 0) ? 0 : (int64_t)sorted_keys[i - 1] + 1;
    const int64_t hi = (i == n) ? n_rows : (int64_t)sorted_keys[i];
    for (int64_t r = lo; r <= hi && r <= n_rows; ++r) rowptr[r] = (int)i;
}

// key of facet f: its number of texture points, capped at 15
__global__ __launch_bounds__(kBlock) void facet_keys_k(const int *__restrict__ cum, int64_t Nf, int T,
                                                       unsigned *__restrict__ keys, int *__restrict__ vals)
{
    const int64_t f = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (f >= Nf) return;
    int a = f ? cum[f - 1] : 0, b = cum[f];
    a = a < 0 ? 0 : (a > T ? T : a);
    b = b < 0 ? 0 : (b > T ? T : b);
    const int K = b > a ? b - a : 0;
    keys[f] = (unsigned)(K < 15 ? K : 15);
    vals[f] = (int)f;
}

static int key_bits(int64_t n_rows)
{
    int b = 1;
    while (b < 32 && (int64_t(1) << b) <= n_rows) ++b;
    return b;
}

static size_t align_up(size_t x) { return (x + 255) & ~size_t(255); }

static size_t sort_temp_bytes(int64_t n, int bits)
{
    size_t bytes = 0;
    unsigned *k = nullptr;
    int *v = nullptr;
    if (n > 0) (void)rocprim::radix_sort_pairs(nullptr, bytes, k, k, v, v, (size_t)n, 0, bits);
    return bytes;
}

// the same stable sort for the other sources of the library (rows_internal.h)
size_t sort_pairs_temp_bytes(int64_t n, int bits) { return sort_temp_bytes(n, bits); }
hipError_t sort_pairs(void *temp, size_t temp_bytes, const unsigned *keys_in, unsigned *keys_out, const int *vals_in,
                      int *vals_out, int64_t n, int bits, hipStream_t st)
{
    if (n <= 0) return hipSuccess;
    return rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in, vals_out, (size_t)n, 0, bits, st);
}

static size_t csr_workspace(int64_t n, int64_t n_rows)
{
    return 3 * align_up((size_t)n * 4) + align_up(sort_temp_bytes(n, key_bits(n_rows))) + 256;
}

// sort (keys, vals) already written into ws slots 0 and 2; sorted ids go to `ids_out`
static int sort_and_rowptr(const char *name, int64_t n, int64_t n_rows, int *rowptr, int *ids_out, void *ws,
                           size_t ws_bytes, hipStream_t st)
{
    char *base = (char *)ws;
    const size_t slot = align_up((size_t)n * 4);
    unsigned *keys_in = (unsigned *)base, *keys_out = (unsigned *)(base + slot);
    int *vals_in = (int *)(base + 2 * slot);
    void *temp = base + 3 * slot;
    const int bits = key_bits(n_rows);
    size_t temp_bytes = sort_temp_bytes(n, bits);
    PM_REQUIRE(3 * slot + temp_bytes <= ws_bytes, "%s: workspace too small (%zu bytes)", name, ws_bytes);
    hipError_t e = rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, vals_in, ids_out, (size_t)n, 0, bits, st);
    PM_REQUIRE(e == hipSuccess, "%s: radix sort failed: %s", name, hipGetErrorString(e));
    rowptr_k<<<dim3((unsigned)ceil_div(n + 1, kBlock)), dim3(kBlock), 0, st>>>(keys_out, n, n_rows, rowptr);
    PM_LAUNCHED(name);
    return 0;
}

__global__ __launch_bounds__(kBlock) void fill_int_k(int *__restrict__ p, int64_t n, int value)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = value;
}

// ----------------------------------------------------------------------------------------
// Composition of two decimation steps' cluster maps (A: fine -> middle, B: middle -> coarse) into fine -> coarse
// maps, in three passes.  rep < 0: contracted into vertex -rep; rep >= 0: number of vertices contracted into
// this one.  Index values outside their arrays are ignored rather than followed.
__global__ __launch_bounds__(kBlock) void clusters_copy_k(const int *__restrict__ rep_a, const int *__restrict__ rep_b,
                                                          int *__restrict__ rep_out, int *__restrict__ owner,
                                                          int64_t nv_a, int64_t nv_b)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < nv_a) rep_out[i] = rep_a[i];
    if (i < nv_b) owner[i] = rep_b[i];
}

// owner[vo] = the fine vertex that survives step A as middle vertex vo, for the vo that survive step B too
// (contracted vo keep their negative entry).
__global__ __launch_bounds__(kBlock) void clusters_owner_k(const int *__restrict__ map_a, const int *__restrict__ rep_b,
                                                           int *__restrict__ owner, int64_t nv_a, int64_t nv_b)
{
    const int64_t vi = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (vi >= nv_a) return;
    const int vo = map_a[vi];
    if (vo >= 0 && vo < nv_b && rep_b[vo] >= 0) owner[vo] = (int)vi;
}

// A fine vertex whose middle-level representative is contracted by step B moves to the fine vertex behind B's
// representative and counts there; the map goes through both steps.
__global__ __launch_bounds__(kBlock) void clusters_merge_k(const int *__restrict__ rep_a, const int *__restrict__ map_a,
                                                           const int *__restrict__ owner, const int *__restrict__ map_b,
                                                           int *__restrict__ rep_out, int *__restrict__ map_out,
                                                           int64_t nv_a, int64_t nv_b)
{
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= nv_a) return;
    const int own = map_a[idx];
    map_out[idx] = (own >= 0 && own < nv_b) ? map_b[own] : -1;
    int64_t vi = idx;
    if (rep_a[idx] < 0) vi = -(int64_t)rep_a[idx];
    if (vi >= nv_a) return;
    const int vo = map_a[vi];
    if (vo < 0 || vo >= nv_b || owner[vo] >= 0) return;
    const int64_t vb = -(int64_t)owner[vo];
    if (vb >= nv_b) return;
    const int target = owner[vb];
    if (target < 0 || target >= nv_a) return;
    rep_out[idx] = -target;
    atomicAdd(&rep_out[target], 1);
}

}  // namespace pmesh

using namespace pmesh;

extern "C" size_t pmesh_vertex_csr_workspace_bytes(int64_t n_facets, int64_t n_rows)
{
    return csr_workspace(3 * n_facets, n_rows);
}

extern "C" int pmesh_build_vertex_csr(const int32_t *face, const int32_t *vt_map, int64_t n_facets,
                                      int64_t n_vt_map, int64_t n_rows, int32_t *rowptr, int32_t *colidx,
                                      void *workspace, size_t workspace_bytes, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_facets >= 0 && n_rows >= 0 && n_vt_map >= 0, "build_vertex_csr: negative size");
    PM_REQUIRE(n_facets <= INT32_MAX / 3 && n_rows < INT32_MAX, "build_vertex_csr: sizes exceed int32 indexing");
    PM_REQUIRE(rowptr, "build_vertex_csr: null rowptr");
    hipStream_t st = (hipStream_t)stream;
    const int64_t n = 3 * n_facets;
    if (n == 0) {
        fill_int_k<<<dim3((unsigned)ceil_div(n_rows + 1, kBlock)), dim3(kBlock), 0, st>>>(rowptr, n_rows + 1, 0);
        PM_LAUNCHED("build_vertex_csr(fill)");
        return 0;
    }
    PM_REQUIRE(face && colidx && workspace, "build_vertex_csr: null pointer");
    PM_REQUIRE(workspace_bytes >= 3 * align_up((size_t)n * 4), "build_vertex_csr: workspace too small");
    char *base = (char *)workspace;
    const size_t slot = align_up((size_t)n * 4);
    vertex_keys_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(
        face, vt_map, n, n_vt_map, n_rows, (unsigned *)base, (int *)(base + 2 * slot));
    PM_LAUNCHED("build_vertex_csr(keys)");
    return sort_and_rowptr("build_vertex_csr", n, n_rows, rowptr, colidx, workspace, workspace_bytes, st);
}

extern "C" size_t pmesh_index_csr_workspace_bytes(int64_t n, int64_t n_rows) { return csr_workspace(n, n_rows); }

extern "C" int pmesh_build_index_csr(const int32_t *keys, int key_stride, int64_t n, int64_t n_rows, int32_t *rowptr,
                                     int32_t *order, void *workspace, size_t workspace_bytes, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n >= 0 && n_rows >= 0 && key_stride > 0, "build_index_csr: bad sizes");
    PM_REQUIRE(n < INT32_MAX && n_rows < INT32_MAX, "build_index_csr: sizes exceed int32 indexing");
    PM_REQUIRE(rowptr, "build_index_csr: null rowptr");
    hipStream_t st = (hipStream_t)stream;
    if (n == 0) {
        fill_int_k<<<dim3((unsigned)ceil_div(n_rows + 1, kBlock)), dim3(kBlock), 0, st>>>(rowptr, n_rows + 1, 0);
        PM_LAUNCHED("build_index_csr(fill)");
        return 0;
    }
    PM_REQUIRE(keys && order && workspace, "build_index_csr: null pointer");
    PM_REQUIRE(workspace_bytes >= 3 * align_up((size_t)n * 4), "build_index_csr: workspace too small");
    char *base = (char *)workspace;
    const size_t slot = align_up((size_t)n * 4);
    index_keys_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(keys, key_stride, n, n_rows, (unsigned *)base,
                                                                               (int *)(base + 2 * slot));
    PM_LAUNCHED("build_index_csr(keys)");
    return sort_and_rowptr("build_index_csr", n, n_rows, rowptr, order, workspace, workspace_bytes, st);
}

extern "C" size_t pmesh_cluster_csr_workspace_bytes(int64_t n_fine, int64_t n_coarse)
{
    return csr_workspace(n_fine, n_coarse);
}

extern "C" int pmesh_build_cluster_csr(const int32_t *vt_replace, const int32_t *vt_map, int64_t n_fine,
                                       int64_t n_coarse, int32_t *rowptr, int32_t *members, void *workspace,
                                       size_t workspace_bytes, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_fine >= 0 && n_coarse >= 0, "build_cluster_csr: negative size");
    PM_REQUIRE(n_fine < INT32_MAX && n_coarse < INT32_MAX, "build_cluster_csr: sizes exceed int32 indexing");
    PM_REQUIRE(rowptr, "build_cluster_csr: null rowptr");
    hipStream_t st = (hipStream_t)stream;
    if (n_fine == 0) {
        fill_int_k<<<dim3((unsigned)ceil_div(n_coarse + 1, kBlock)), dim3(kBlock), 0, st>>>(rowptr, n_coarse + 1, 0);
        PM_LAUNCHED("build_cluster_csr(fill)");
        return 0;
    }
    PM_REQUIRE(vt_replace && vt_map && members && workspace, "build_cluster_csr: null pointer");
    PM_REQUIRE(workspace_bytes >= 3 * align_up((size_t)n_fine * 4), "build_cluster_csr: workspace too small");
    char *base = (char *)workspace;
    const size_t slot = align_up((size_t)n_fine * 4);
    cluster_keys_k<<<dim3((unsigned)ceil_div(n_fine, kBlock)), dim3(kBlock), 0, st>>>(
        vt_replace, vt_map, n_fine, n_coarse, (unsigned *)base, (int *)(base + 2 * slot));
    PM_LAUNCHED("build_cluster_csr(keys)");
    return sort_and_rowptr("build_cluster_csr", n_fine, n_coarse, rowptr, members, workspace, workspace_bytes, st);
}

extern "C" size_t pmesh_facet_order_workspace_bytes(int64_t n_facets)
{
    return 3 * align_up((size_t)n_facets * 4) + align_up(sort_temp_bytes(n_facets, 4)) + 256;
}

extern "C" int pmesh_build_facet_order(const int32_t *cum_texture, int64_t n_facets, int64_t n_points, int32_t *order,
                                       void *workspace, size_t workspace_bytes, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(n_facets >= 0 && n_facets < INT32_MAX && n_points >= 0 && n_points <= INT32_MAX,
               "build_facet_order: bad sizes");
    if (n_facets == 0) return 0;
    PM_REQUIRE(cum_texture && order && workspace, "build_facet_order: null pointer");
    hipStream_t st = (hipStream_t)stream;
    char *base = (char *)workspace;
    const size_t slot = align_up((size_t)n_facets * 4);
    size_t temp_bytes = sort_temp_bytes(n_facets, 4);
    PM_REQUIRE(3 * slot + temp_bytes <= workspace_bytes, "build_facet_order: workspace too small (%zu bytes)",
               workspace_bytes);
    unsigned *keys_in = (unsigned *)base, *keys_out = (unsigned *)(base + slot);
    int *vals_in = (int *)(base + 2 * slot);
    facet_keys_k<<<dim3((unsigned)ceil_div(n_facets, kBlock)), dim3(kBlock), 0, st>>>(cum_texture, n_facets,
                                                                                       (int)n_points, keys_in, vals_in);
    PM_LAUNCHED("build_facet_order(keys)");
    hipError_t e = rocprim::radix_sort_pairs(base + 3 * slot, temp_bytes, keys_in, keys_out, vals_in, order,
                                             (size_t)n_facets, 0, 4, st);
    PM_REQUIRE(e == hipSuccess, "build_facet_order: radix sort failed: %s", hipGetErrorString(e));
    return 0;
}

extern "C" int pmesh_combine_clusters(const int32_t *rep_a, const int32_t *map_a, const int32_t *rep_b,
                                      const int32_t *map_b, int32_t *rep_out, int32_t *map_out, int32_t *scratch,
                                      int64_t nv_a, int64_t nv_b, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(nv_a >= 0 && nv_b >= 0 && nv_a < INT32_MAX && nv_b < INT32_MAX, "combine_clusters: bad sizes");
    if (nv_a == 0) return 0;
    PM_REQUIRE(rep_a && map_a && rep_out && map_out, "combine_clusters: null pointer");
    PM_REQUIRE(nv_b == 0 || (rep_b && map_b && scratch), "combine_clusters: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int64_t n = nv_a > nv_b ? nv_a : nv_b;
    const dim3 grid_n((unsigned)ceil_div(n, kBlock)), grid_a((unsigned)ceil_div(nv_a, kBlock)), block(kBlock);
    clusters_copy_k<<<grid_n, block, 0, st>>>(rep_a, rep_b, rep_out, scratch, nv_a, nv_b);
    PM_LAUNCHED("combine_clusters(copy)");
    clusters_owner_k<<<grid_a, block, 0, st>>>(map_a, rep_b, scratch, nv_a, nv_b);
    PM_LAUNCHED("combine_clusters(owner)");
    clusters_merge_k<<<grid_a, block, 0, st>>>(rep_a, map_a, scratch, map_b, rep_out, map_out, nv_a, nv_b);
    PM_LAUNCHED("combine_clusters(merge)");
    return 0;
}
