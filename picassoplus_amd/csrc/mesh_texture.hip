// Texture points of the facets from vertex features (gfx950, wave64).
//
//   forward   tex[k, c] = sum_j bary[k, j] * in[face[f, j], c]   for the rows k of facet f's segment
//             [cum[f-1], cum[f]) -- the grouping facet2facet expects (picasso/mesh/layers.py:57) --
//             and, in the same pass, coeff[k, :] = spherical-harmonic basis at bary[k, :]
//             (what picasso/networks/scene_seg.py:150 computes with a chain of elementwise kernels);
//   backward  gin[v, c] = sum over the (facet, corner) pairs at v, over the facet's rows k, of
//             bary[k, corner] * gtex[k, c], a segmented sum over the sorted vertex adjacency (no atomics,
//             fixed order).
//
// Both are bound by HBM.  A group of lanes owns one facet (forward) or one vertex (backward) and spans the
// channels with 16-byte items; the three corner rows of a facet are fetched once and stay in registers for all of
// the facet's points, whose rows leave as one contiguous run.
#include "common.h"
#include "sph_internal.h"
#include "../../include/picasso_mesh.h"

namespace pmesh {

constexpr int kTexBatch = 4;   // texture points in flight per lane group

template <int V, int LC>   // LC: compile-time degree of the basis, -1 = read `L`
__global__ __launch_bounds__(kBlock) void texture_fwd_k(const float *__restrict__ in, const int *__restrict__ face,
                                                        const int *__restrict__ cum, const float *__restrict__ bary,
                                                        float *__restrict__ tex, float *__restrict__ coeff,
                                                        int64_t Nf, int64_t T, int C, int Q, int lpr_log2, int L)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int rpb = kBlock >> lpr_log2;
    const int64_t f = (int64_t)blockIdx.x * rpb + slot;
    int64_t k0 = 0, k1 = 0;
    if (f < Nf) {
        k0 = f ? cum[f - 1] : 0;
        k1 = cum[f];
        if (k0 < 0) k0 = 0;
        if (k1 > T) k1 = T;
    }
    if (k0 < k1) {
        const int64_t v0 = face[3 * f], v1 = face[3 * f + 1], v2 = face[3 * f + 2];
        for (int q = lane; q < Q; q += lpr) {
            const int c = q * V;
            const Pack<V> a0 = ldp<V>(in + v0 * C + c), a1 = ldp<V>(in + v1 * C + c), a2 = ldp<V>(in + v2 * C + c);
            for (int64_t kb = k0; kb < k1; kb += kTexBatch) {
                float b[kTexBatch][3];
#pragma unroll
                for (int i = 0; i < kTexBatch; ++i)
#pragma unroll
                    for (int j = 0; j < 3; ++j) b[i][j] = (kb + i < k1) ? bary[3 * (kb + i) + j] : 0.f;
#pragma unroll
                for (int i = 0; i < kTexBatch; ++i) {
                    if (kb + i >= k1) break;
                    Pack<V> o;
#pragma unroll
                    for (int u = 0; u < V; ++u) o.v[u] = fmaf(b[i][2], a2.v[u], fmaf(b[i][1], a1.v[u], b[i][0] * a0.v[u]));
                    stp<V>(tex + (kb + i) * C + c, o);
                }
            }
        }
    }
    if (!coeff) return;
    // The points of the workgroup's facets are one contiguous run of rows: its lanes take them one each, so
    // the coordinates come in and the basis values leave as contiguous pieces.
    const int64_t fa = (int64_t)blockIdx.x * rpb;
    int64_t fb = fa + rpb;
    if (fb > Nf) fb = Nf;
    int64_t ka = fa ? cum[fa - 1] : 0, kz = cum[fb - 1];
    if (ka < 0) ka = 0;
    if (kz > T) kz = T;
    const int Lv = LC >= 0 ? LC : L;
    const int B = (Lv + 1) * (Lv + 1);
    for (int64_t k = ka + threadIdx.x; k < kz; k += kBlock) {
        float v[36];
        sph_harm_at(bary[3 * k], bary[3 * k + 1], bary[3 * k + 2], Lv, v);
        float *o = coeff + k * B;
        if constexpr (LC == 3) {
#pragma unroll
            for (int i = 0; i < 16; i += 4) *reinterpret_cast<float4 *>(o + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
        } else {
            sph_store(o, v, Lv);
        }
    }
}

template <int V>
__global__ __launch_bounds__(kBlock) void texture_bwd_k(const float *__restrict__ gtex, const float *__restrict__ bary,
                                                        const int *__restrict__ cum, const int *__restrict__ rowptr,
                                                        const int *__restrict__ colidx, float *__restrict__ gin,
                                                        int64_t Nv, int64_t Nf, int64_t T, int C, int Q, int lpr_log2)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= Nv) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    constexpr int EB = 4;
    for (int q = lane; q < Q; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int eb = e0; eb < e1; eb += EB) {
            // the adjacency entries of a vertex four at a time: all segment bounds requested before any is used
            int ent[EB], corner[EB];
            int64_t s0[EB], s1[EB];
#pragma unroll
            for (int i = 0; i < EB; ++i) ent[i] = (eb + i < e1) ? colidx[eb + i] : -1;
#pragma unroll
            for (int i = 0; i < EB; ++i) {
                const int64_t f = ent[i] / 3;
                corner[i] = ent[i] - 3 * (int)f;
                const bool ok = ent[i] >= 0 && f < Nf;
                s0[i] = (ok && f > 0) ? cum[f - 1] : 0;
                s1[i] = ok ? cum[f] : 0;
            }
#pragma unroll
            for (int i = 0; i < EB; ++i) {
                if (s0[i] < 0) s0[i] = 0;
                if (s1[i] > T) s1[i] = T;
            }
#pragma unroll
            for (int i = 0; i < EB; ++i) {
                for (int64_t kb = s0[i]; kb < s1[i]; kb += kTexBatch) {
                    float w[kTexBatch];
                    Pack<V> g[kTexBatch];
#pragma unroll
                    for (int p = 0; p < kTexBatch; ++p) {
                        const bool in = kb + p < s1[i];
                        w[p] = in ? bary[3 * (kb + p) + corner[i]] : 0.f;
                        g[p] = in ? ldp<V>(gtex + (kb + p) * C + c) : zero_pack<V>();
                    }
#pragma unroll
                    for (int p = 0; p < kTexBatch; ++p)
#pragma unroll
                        for (int u = 0; u < V; ++u) acc.v[u] = fmaf(w[p], g[p].v[u], acc.v[u]);
                }
            }
        }
        stp<V>(gin + row * C + c, acc);
    }
}

// The same sum for rows of at most 64 lanes per vertex and at least 8, with a shorter dependent chain per vertex:
// row bounds -> eight adjacency entries -> their segment bounds -> the points of all eight facets as ONE flat
// sequence, eight rows requested at a time.  Lane s of the group locates flat point t + s (a facet's points follow
// its predecessor's, so the order of the sum is the one of texture_bwd_k and the results are identical); the lanes
// pick the eight locations up with cross-lane reads.  Workgroups go round-robin to the eight accelerator dies, each
// with an L2 of its own: die x takes the x-th contiguous eighth of the row blocks (the grid is 8 * ceil(blocks / 8)),
// so that the three vertices that read a facet's rows mostly meet in one L2.
template <int V>
__global__ __launch_bounds__(kBlock) void texture_bwd_flat_k(const float *__restrict__ gtex, const float *__restrict__ bary,
                                                             const int *__restrict__ cum, const int *__restrict__ rowptr,
                                                             const int *__restrict__ colidx, float *__restrict__ gin,
                                                             int64_t Nv, int64_t Nf, int T, int C, int Q, int lpr_log2)
{
    constexpr int EB = 8, PB = 8;
    const int lpr = 1 << lpr_log2, rpb = kBlock >> lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int gbase = (threadIdx.x & 63) & ~(lpr - 1);          // first lane of my group within the wavefront
    const int64_t nblk = (Nv + rpb - 1) / rpb, per_die = (nblk + 7) >> 3;
    const int64_t blk = (int64_t)(blockIdx.x & 7) * per_die + (blockIdx.x >> 3);
    const int64_t row = blk * rpb + slot;
    if ((int64_t)(blockIdx.x >> 3) >= per_die || row >= Nv) return;      // whole groups leave together
    const bool active = lane < Q;
    // byte offsets into grad_texture and bary fit 32 bits (checked by the caller): the vector ALU is this kernel's
    // busiest unit, so a point's location is turned into its two offsets once, by the lane that locates it
    const unsigned row_bytes = (unsigned)C * 4u, col_bytes = active ? (unsigned)(lane * V) * 4u : 0u;   // idle lanes read column 0
    const char *gbytes = reinterpret_cast<const char *>(gtex), *bbytes = reinterpret_cast<const char *>(bary);
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    Pack<V> acc = zero_pack<V>();
    for (int eb = e0; eb < e1; eb += EB) {
        // every load below is unconditional (indices clamped into the row, results masked afterwards): a conditional
        // load costs a branch of its own
        int ent[EB], pre[EB + 1], key[EB];
#pragma unroll
        for (int i = 0; i < EB; ++i) {
            const int idx = eb + i < e1 ? eb + i : e1 - 1;
            ent[i] = colidx[idx];
        }
#pragma unroll
        for (int i = 0; i < EB; ++i) ent[i] = (eb + i < e1) ? ent[i] : -1;
        int a[EB], b[EB];
#pragma unroll
        for (int i = 0; i < EB; ++i) {
            const int f = ent[i] / 3;
            int fc = f < 0 ? 0 : f;
            fc = fc < (int)Nf ? fc : (int)Nf - 1;
            a[i] = cum[fc > 0 ? fc - 1 : 0];
            b[i] = cum[fc];
        }
        pre[0] = 0;
#pragma unroll
        for (int i = 0; i < EB; ++i) {
            const int f = ent[i] / 3;
            const bool ok = ent[i] >= 0 && f < Nf;
            int lo = (ok && f > 0) ? a[i] : 0, hi = ok ? b[i] : 0;
            lo = lo < 0 ? 0 : lo;
            hi = hi > T ? T : hi;
            pre[i + 1] = pre[i] + (hi > lo ? hi - lo : 0);
            // flat point u of entry i is row lo + (u - pre[i]) with corner ent % 3: 4 * row + corner = 4 * u + key
            key[i] = 4 * (lo - pre[i]) + (ent[i] - 3 * f);
        }
        const int P = pre[EB];
        for (int t = 0; t < P; t += PB) {
            // slots past the end repeat the step's first point with weight zero
            const int ur = t + (lane & (PB - 1));
            const bool mine = ur < P;
            const int u = mine ? ur : t;
            int kq = key[0];
#pragma unroll
            for (int j = 1; j < EB; ++j) kq = u >= pre[j] ? key[j] : kq;
            kq += 4 * u;                                          // 4 * row + corner of my point
            const unsigned my_g = (unsigned)(kq >> 2) * row_bytes;
            const unsigned my_b = ((unsigned)(kq >> 2) * 12u + (unsigned)(kq & 3) * 4u) | (mine ? 0u : 1u);
            float w[PB];
            Pack<V> g[PB];
#pragma unroll
            for (int s = 0; s < PB; ++s) {
                const unsigned og = (unsigned)__shfl((int)my_g, gbase + s, 64);
                const unsigned ob = (unsigned)__shfl((int)my_b, gbase + s, 64);
                const float wr = *reinterpret_cast<const float *>(bbytes + (ob & ~1u));
                w[s] = (ob & 1u) ? 0.f : wr;
                g[s] = ldp<V>(reinterpret_cast<const float *>(gbytes + (og + col_bytes)));
            }
#pragma unroll
            for (int s = 0; s < PB; ++s)
#pragma unroll
                for (int x = 0; x < V; ++x) acc.v[x] = fmaf(w[s], g[s].v[x], acc.v[x]);
        }
    }
    if (active) stp<V>(gin + row * C + lane * V, acc);
}

// Per-level producer of the facet2vertex coefficients in one pass: triangle geometry (unit normal, plane offset,
// area: picasso/mesh/pi_modules/decimate.py:70-85), the normal turned towards the origin as the viewpoint
// (picasso/networks/scene_seg.py:117-124: flipped when -centre . normal < 0), and the spherical-harmonic basis at the
// oriented normal (scene_seg.py:149,164).  Any of the three outputs may be absent.
__global__ __launch_bounds__(kBlock) void facet_frame_k(const float *__restrict__ vertex, const int *__restrict__ face,
                                                       float *__restrict__ geometry, float *__restrict__ normal,
                                                       float *__restrict__ coeff, int64_t Nf, int vstride, int L)
{
    const int64_t f = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (f >= Nf) return;
    const float *a = vertex + (int64_t)face[3 * f] * vstride;
    const float *b = vertex + (int64_t)face[3 * f + 1] * vstride;
    const float *c = vertex + (int64_t)face[3 * f + 2] * vstride;
    const float ax = a[0], ay = a[1], az = a[2], bx = b[0], by = b[1], bz = b[2], cx = c[0], cy = c[1], cz = c[2];
    const float ux = bx - ax, uy = by - ay, uz = bz - az;
    const float vx = cx - ax, vy = cy - ay, vz = cz - az;
    float nx = uy * vz - uz * vy, ny = uz * vx - ux * vz, nz = ux * vy - uy * vx;
    const float len = sqrtf(nx * nx + ny * ny + nz * nz);
    const float inv = 1.0f / (len + 1e-10f);
    nx *= inv; ny *= inv; nz *= inv;
    if (geometry) {
        float *g = geometry + 5 * f;
        g[0] = nx; g[1] = ny; g[2] = nz;
        g[3] = -(nx * ax + ny * ay + nz * az);
        g[4] = 0.5f * len;
    }
    // sign(-centre . n), with 0 counted as +1
    const float mx = (ax + bx + cx) / 3.0f, my = (ay + by + cy) / 3.0f, mz = (az + bz + cz) / 3.0f;
    const float towards = -(mx * nx + my * ny + mz * nz);
    if (towards < 0.f) { nx = -nx; ny = -ny; nz = -nz; }
    if (normal) {
        normal[3 * f] = nx; normal[3 * f + 1] = ny; normal[3 * f + 2] = nz;
    }
    if (coeff) {
        const int B = (L + 1) * (L + 1);
        float v[36];
        sph_harm_at(nx, ny, nz, L, v);
        sph_store(coeff + f * B, v, L);
    }
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace pmesh

using namespace pmesh;

extern "C" int pmesh_texture_fwd(const float *input, const int32_t *face, const float *bary, const int32_t *cum_texture,
                                 float *texture, float *bary_coeff, int64_t Nv, int64_t Nf, int64_t T, int C, int L,
                                 pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nf >= 0 && T >= 0 && C >= 0, "texture_fwd: negative size");
    PM_REQUIRE(!bary_coeff || (L >= 0 && L <= 5), "texture_fwd: basis degree %d outside 0..5", L);
    PM_REQUIRE(T < (int64_t(1) << 31), "texture_fwd: more than 2^31 texture points");
    if (T == 0 || Nf == 0) return 0;
    PM_REQUIRE(face && bary && cum_texture, "texture_fwd: null pointer");
    PM_REQUIRE(C == 0 || (input && texture && Nv > 0), "texture_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = C % 4 == 0 && aligned16(input) && aligned16(texture);
    const RowShape rs = row_shape(C == 0 ? 1 : vec ? C / 4 : C);
    const int Q = C == 0 ? 0 : rs.items;
    const int64_t blocks = ceil_div(Nf, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "texture_fwd: grid too large");
    const dim3 grid((unsigned)blocks), block(kBlock);
    const bool l3 = bary_coeff && L == 3 && aligned16(bary_coeff);
    if (vec) {
        if (l3) texture_fwd_k<4, 3><<<grid, block, 0, st>>>(input, face, cum_texture, bary, texture, bary_coeff, Nf, T, C, Q, rs.lpr_log2, L);
        else texture_fwd_k<4, -1><<<grid, block, 0, st>>>(input, face, cum_texture, bary, texture, bary_coeff, Nf, T, C, Q, rs.lpr_log2, L);
    } else {
        if (l3) texture_fwd_k<1, 3><<<grid, block, 0, st>>>(input, face, cum_texture, bary, texture, bary_coeff, Nf, T, C, Q, rs.lpr_log2, L);
        else texture_fwd_k<1, -1><<<grid, block, 0, st>>>(input, face, cum_texture, bary, texture, bary_coeff, Nf, T, C, Q, rs.lpr_log2, L);
    }
    PM_LAUNCHED("texture_fwd");
    return 0;
}

extern "C" int pmesh_texture_bwd(const float *grad_texture, const float *bary, const int32_t *cum_texture,
                                 const int32_t *rowptr, const int32_t *colidx, float *grad_input, int64_t Nv,
                                 int64_t Nf, int64_t T, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nf >= 0 && T >= 0 && C >= 0, "texture_bwd: negative size");
    PM_REQUIRE(T < (int64_t(1) << 31), "texture_bwd: more than 2^31 texture points");
    if (Nv == 0 || C == 0) return 0;
    PM_REQUIRE(grad_input && rowptr, "texture_bwd: null pointer");
    PM_REQUIRE(Nf == 0 || (colidx && cum_texture), "texture_bwd: null pointer");
    PM_REQUIRE(T == 0 || (grad_texture && bary), "texture_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = C % 4 == 0 && aligned16(grad_input) && aligned16(grad_texture);
    const RowShape rs = row_shape(vec ? C / 4 : C);
    const int64_t blocks = ceil_div(Nv, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "texture_bwd: grid too large");
    // rows of 8 to 64 lanes take the flat kernel (a point's location travels as 32-bit byte offsets)
    const bool flat = rs.lpr >= 8 && rs.lpr <= 64 && rs.items <= rs.lpr && T < (int64_t(1) << 28) &&
                      T * C * 4 < (int64_t(1) << 32) - 4096;
    const int64_t fblocks = 8 * ceil_div(blocks, 8);
    PM_REQUIRE(grid_ok(fblocks), "texture_bwd: grid too large");
    if (vec && flat)
        texture_bwd_flat_k<4><<<dim3((unsigned)fblocks), dim3(kBlock), 0, st>>>(grad_texture, bary, cum_texture, rowptr, colidx, grad_input, Nv, Nf, (int)T, C, rs.items, rs.lpr_log2);
    else if (flat)
        texture_bwd_flat_k<1><<<dim3((unsigned)fblocks), dim3(kBlock), 0, st>>>(grad_texture, bary, cum_texture, rowptr, colidx, grad_input, Nv, Nf, (int)T, C, rs.items, rs.lpr_log2);
    else if (vec)
        texture_bwd_k<4><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_texture, bary, cum_texture, rowptr, colidx, grad_input, Nv, Nf, T, C, rs.items, rs.lpr_log2);
    else
        texture_bwd_k<1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_texture, bary, cum_texture, rowptr, colidx, grad_input, Nv, Nf, T, C, rs.items, rs.lpr_log2);
    PM_LAUNCHED("texture_bwd");
    return 0;
}

extern "C" int pmesh_facet_frame(const float *vertex, const int32_t *face, float *geometry, float *normal, float *coeff,
                                 int64_t Nv, int64_t Nf, int vertex_stride, int L, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nf >= 0 && vertex_stride >= 3, "facet_frame: bad sizes");
    PM_REQUIRE(!coeff || (L >= 0 && L <= 5), "facet_frame: basis degree %d outside 0..5", L);
    if (Nf == 0 || !(geometry || normal || coeff)) return 0;
    PM_REQUIRE(vertex && face, "facet_frame: null pointer");
    PM_REQUIRE(Nv * vertex_stride < (int64_t(1) << 40) && grid_ok(ceil_div(Nf, kBlock)), "facet_frame: sizes too large");
    facet_frame_k<<<dim3((unsigned)ceil_div(Nf, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(vertex, face, geometry, normal, coeff, Nf, vertex_stride, L);
    PM_LAUNCHED("facet_frame");
    return 0;
}
