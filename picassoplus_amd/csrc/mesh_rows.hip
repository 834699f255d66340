// HBM-bound row kernels of the mesh-conv path: vertex2facet, facet2vertex, mesh pooling and
// unpooling, spherical-harmonic basis.  gfx950, wave64.
//
// Common shape: one feature row (C floats) is owned by a power-of-two group of lanes, each
// lane moving V consecutive channels per access (V = 4 -> 16-byte accesses, used whenever the
// depth multiplier r is 1 and C is a multiple of 4; V = 1 covers every other shape).
// Scatter-type ops of the reference (float atomicAdd / CAS atomicMax) are run here as
// gathers over sorted CSR adjacency, so every sum has a fixed order and no atomics exist.
// Filter gradients are reduced in two stages: per-workgroup partial sums written to a
// workspace, then a fixed-order reduction over workgroups.
#include "common.h"
#include "rows_internal.h"
#include "sph_internal.h"
#include <stdlib.h>
#include "../../include/picasso_mesh.h"
#include <cstdlib>
#include <mutex>

namespace pmesh {

// ----------------------------------------------------------------------------------------
// small device helpers
// ----------------------------------------------------------------------------------------
__device__ __forceinline__ void load_coeff16(const float *p, int kc, bool vec_ok, float (&cf)[16])
{
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        if (vec_ok && 4 * g + 4 <= kc) {
            const float4 t = *reinterpret_cast<const float4 *>(p + 4 * g);
            cf[4 * g] = t.x; cf[4 * g + 1] = t.y; cf[4 * g + 2] = t.z; cf[4 * g + 3] = t.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) cf[4 * g + i] = (4 * g + i < kc) ? p[4 * g + i] : 0.f;
        }
    }
}

// Sum `acc` over the row slots of a workgroup in slot order and let slot 0 store the result.
template <int V>
__device__ __forceinline__ void block_reduce_store(const Pack<V> &acc, float *red, float *dst,
                                                   bool active, int lane, int slot, int lpr, int rpb)
{
#pragma unroll
    for (int i = 0; i < V; ++i) red[threadIdx.x * V + i] = acc.v[i];
    __syncthreads();
    if (slot == 0 && active) {
        Pack<V> s = zero_pack<V>();
        for (int t = 0; t < rpb; ++t)
#pragma unroll
            for (int i = 0; i < V; ++i) s.v[i] += red[(t * lpr + lane) * V + i];
        stp<V>(dst, s);
    }
    __syncthreads();
}

// out[o] = sum_g partial[g*n + o]: 64 interleaved slices of g (ascending within a slice), then the
// slices in a fixed tree order.  One workgroup of 1024 threads covers 16 outputs, so that the few
// thousand outputs of a filter gradient still spread over the chip.
__global__ __launch_bounds__(1024) void reduce_partials_k(const float *__restrict__ partial,
                                                         float *__restrict__ out, int G, int n, size_t stride)
{
    __shared__ float red[64][16];
    const int j = threadIdx.x & 15, s = threadIdx.x >> 4;
    const int o = blockIdx.x * 16 + j;
    float sum = 0.f;
    if (o < n)
        for (int g = s; g < G; g += 64) sum += partial[(size_t)g * stride + o];
    red[s][j] = sum;
    __syncthreads();
#pragma unroll
    for (int half = 32; half > 0; half >>= 1) {
        if (s < half) red[s][j] += red[s + half][j];
        __syncthreads();
    }
    if (s == 0 && o < n) out[o] = red[0][j];
}

__global__ __launch_bounds__(kBlock) void fill_zero_k(float *__restrict__ p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

// ----------------------------------------------------------------------------------------
// vertex2facet forward:  out[f, c*r+m] = sum_k filt[k,c,m] * in[face[f,k], c]
// ----------------------------------------------------------------------------------------
// V consecutive output channels of a lane read V / R consecutive input channels (R = depth multiplier when the
// vector form handles it: 1, or 2 with V = 4), each used R times
template <int V, int R> __device__ __forceinline__ Pack<V> ld_in_wide(const float *p)
{
    if constexpr (R == 1) {
        return ldp<V>(p);
    } else {
        const float2 t = *reinterpret_cast<const float2 *>(p);
        Pack<V> o;
        o.v[0] = t.x; o.v[1] = t.x; o.v[2] = t.y; o.v[3] = t.y;
        return o;
    }
}

template <int V, int R>
__global__ __launch_bounds__(kBlock) void v2f_fwd_k(const float *__restrict__ in,
                                                    const float *__restrict__ filt,
                                                    const int *__restrict__ face,
                                                    float *__restrict__ out, int64_t Nf, int C, int r,
                                                    int Q, int lpr_log2)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t f = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (f >= Nf) return;
    const int Co = C * r;
    const int64_t v0 = face[3 * f], v1 = face[3 * f + 1], v2 = face[3 * f + 2];
    for (int q = lane; q < Q; q += lpr) {
        const int co = q * V;
        const int c = (V == 4) ? co / R : co / r;
        const Pack<V> a0 = ld_in_wide<V, R>(in + v0 * C + c), a1 = ld_in_wide<V, R>(in + v1 * C + c),
                      a2 = ld_in_wide<V, R>(in + v2 * C + c);
        const Pack<V> f0 = ldp<V>(filt + co), f1 = ldp<V>(filt + Co + co), f2 = ldp<V>(filt + 2 * Co + co);
        Pack<V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) o.v[i] = fmaf(f2.v[i], a2.v[i], fmaf(f1.v[i], a1.v[i], f0.v[i] * a0.v[i]));
        stp<V>(out + f * Co + co, o);
    }
}

// ----------------------------------------------------------------------------------------
// vertex2facet backward, one pass over the vertex -> (facet, corner) adjacency:
//   gin[v,c]     = sum_{(f,k) at v} sum_m gout[f,c*r+m] * filt[k,c,m]
//   gfilt[k,c,m] = sum_v in[v,c] * sum_{(f,k) at v} gout[f,c*r+m]        (per-workgroup partials)
// Lanes own V output channels.  V = 1: any depth multiplier, as an outer loop.  V = 4: r = R = 1 (four input
// channels), or r = R = 2 (two input channels, each the sum over its two outputs: both sit in the lane).
// ----------------------------------------------------------------------------------------
template <int V, int R>
__global__ __launch_bounds__(kBlock) void v2f_bwd_k(const float *__restrict__ gout,
                                                    const float *__restrict__ in,
                                                    const float *__restrict__ filt,
                                                    const int *__restrict__ rowptr,
                                                    const int *__restrict__ colidx,
                                                    float *__restrict__ gin, float *__restrict__ partial,
                                                    int64_t Nv, int C, int r, int Q, int lpr_log2,
                                                    int64_t rows_per_block)
{
    __shared__ float red[kBlock * V];
    const int lpr = 1 << lpr_log2, rpb = kBlock >> lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int Co = C * r;
    const int64_t rbeg = (int64_t)blockIdx.x * rows_per_block;
    const int64_t rend = (rbeg + rows_per_block < Nv) ? rbeg + rows_per_block : Nv;
    for (int m = 0; m < (V == 4 ? 1 : r); ++m)
        for (int q0 = 0; q0 < Q; q0 += lpr) {
            const int q = q0 + lane;
            const bool active = q < Q;
            const int c = (V == 4) ? q * V / R : q;
            const int co = (V == 4) ? q * V : c * r + m;
            Pack<V> fk[3], acc[3];
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                fk[k] = active ? ldp<V>(filt + k * Co + co) : zero_pack<V>();
                acc[k] = zero_pack<V>();
            }
            if (active) {
                // entries of a vertex are taken eight at a time, all their gathers issued before any use;
                // the bounds of the next row are requested while this one is summed
                constexpr int EB = 8;
                int64_t row = rbeg + slot;
                int e0 = 0, e1 = 0;
                if (row < rend) { e0 = rowptr[row]; e1 = rowptr[row + 1]; }
                for (; row < rend; row += rpb) {
                    int ne0 = 0, ne1 = 0;
                    if (row + rpb < rend) { ne0 = rowptr[row + rpb]; ne1 = rowptr[row + rpb + 1]; }
                    const Pack<V> x = ld_in_wide<V, R>(in + row * C + c);
                    Pack<V> g = zero_pack<V>(), s[3];
#pragma unroll
                    for (int k = 0; k < 3; ++k) s[k] = zero_pack<V>();
                    for (int eb = e0; eb < e1; eb += EB) {
                        int ent[EB];
#pragma unroll
                        for (int i = 0; i < EB; ++i) ent[i] = (eb + i < e1) ? colidx[eb + i] : -1;
                        Pack<V> go[EB];
#pragma unroll
                        for (int i = 0; i < EB; ++i)
                            go[i] = (ent[i] >= 0) ? ldp<V>(gout + (int64_t)(ent[i] / 3) * Co + co) : zero_pack<V>();
#pragma unroll
                        for (int i = 0; i < EB; ++i) {
                            const int k = ent[i] - 3 * (ent[i] / 3);          // corner; masked entries carry zeros
#pragma unroll
                            for (int u = 0; u < V; ++u) {
                                const float w = (k == 0) ? fk[0].v[u] : (k == 1) ? fk[1].v[u] : fk[2].v[u];
                                g.v[u] = fmaf(go[i].v[u], w, g.v[u]);
                                s[0].v[u] += (k == 0) ? go[i].v[u] : 0.f;
                                s[1].v[u] += (k == 1) ? go[i].v[u] : 0.f;
                                s[2].v[u] += (k == 2) ? go[i].v[u] : 0.f;
                            }
                        }
                    }
#pragma unroll
                    for (int k = 0; k < 3; ++k)
#pragma unroll
                        for (int u = 0; u < V; ++u) acc[k].v[u] = fmaf(s[k].v[u], x.v[u], acc[k].v[u]);
                    float *gp = gin + row * C + c;
                    if constexpr (V == 4 && R == 2) {
                        *reinterpret_cast<float2 *>(gp) = make_float2(g.v[0] + g.v[1], g.v[2] + g.v[3]);
                    } else if (m == 0) {
                        stp<V>(gp, g);
                    } else {
#pragma unroll
                        for (int u = 0; u < V; ++u) gp[u] += g.v[u];
                    }
                    e0 = ne0;
                    e1 = ne1;
                }
            }
#pragma unroll
            for (int k = 0; k < 3; ++k)
                block_reduce_store<V>(acc[k], red, partial + ((size_t)blockIdx.x * 3 + k) * Co + co, active,
                                      lane, slot, lpr, rpb);
        }
}

// ----------------------------------------------------------------------------------------
// facet2vertex forward over the output-vertex -> facet adjacency:
//   out[vo,co] = (1/nf[vo]) * sum_{f at vo} in[f,c] * sum_k coeff[f,k] * filt[k,co]
// ----------------------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void f2v_fwd_k(const float *__restrict__ in,
                                                    const float *__restrict__ filt,
                                                    const float *__restrict__ coeff,
                                                    const int *__restrict__ nfcount,
                                                    const int *__restrict__ rowptr,
                                                    const int *__restrict__ colidx,
                                                    float *__restrict__ out, int64_t NvOut, int C, int r,
                                                    int K, int Q, int lpr_log2, int coeff_vec)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= NvOut) return;
    const int Co = C * r;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    const float inv = (e1 > e0) ? 1.0f / (float)nfcount[row] : 0.f;
    for (int q = lane; q < Q; q += lpr) {
        const int co = q * V;
        const int c = (V == 4) ? co : co / r;
        Pack<V> acc = zero_pack<V>();
        for (int k0 = 0; k0 < K; k0 += 16) {
            const int kc = (K - k0 < 16) ? K - k0 : 16;
            Pack<V> fl[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) fl[k] = (k < kc) ? ldp<V>(filt + (size_t)(k0 + k) * Co + co) : zero_pack<V>();
            for (int e = e0; e < e1; ++e) {
                const int64_t f = colidx[e] / 3;
                const Pack<V> x = ldp<V>(in + f * C + c);
                float cf[16];
                load_coeff16(coeff + f * K + k0, kc, coeff_vec != 0, cf);
                Pack<V> w = zero_pack<V>();
#pragma unroll
                for (int k = 0; k < 16; ++k)
#pragma unroll
                    for (int i = 0; i < V; ++i) w.v[i] = fmaf(cf[k], fl[k].v[i], w.v[i]);
#pragma unroll
                for (int i = 0; i < V; ++i) acc.v[i] = fmaf(w.v[i], x.v[i], acc.v[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < V; ++i) acc.v[i] *= inv;
        stp<V>(out + row * Co + co, acc);
    }
}

// Lane (l & 15) of every 16-lane row holds one of 16 filter coefficients of an entry; FMAs read
// them through DPP row broadcasts, so an entry in flight costs one register instead of sixteen.
// PM_FMAC4_BCAST: acc[u] += bcast_k(cf) * m[u], u = 0..3, with the broadcast as the DPP operand of the
// FMA itself (no separate move).  A DPP read of a register that a vector ALU instruction wrote needs two
// wait states, which the compiler does not insert for inline assembly: the group for coefficient 0
// starts with them and is declared to rewrite `cf`, so every other group of a sequence is ordered after it.
#define PM_SRC_0 "5"
#define PM_SRC_1 "6"
#define PM_SRC_2 "7"
#define PM_SRC_3 "8"
#define PM_FMAC_DPP(Kk, N) "v_fmac_f32_dpp %" #N ", %4, %" PM_SRC_##N " row_newbcast:" #Kk " row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
#define PM_FMAC4_BCAST0(CF, M, A)                                                               \
    asm("s_nop 1\n" PM_FMAC_DPP(0, 0) PM_FMAC_DPP(0, 1) PM_FMAC_DPP(0, 2) PM_FMAC_DPP(0, 3)      \
        : "+v"((A).v[0]), "+v"((A).v[1]), "+v"((A).v[2]), "+v"((A).v[3]), "+v"(CF)              \
        : "v"((M).v[0]), "v"((M).v[1]), "v"((M).v[2]), "v"((M).v[3]))
#define PM_FMAC4_BCAST(Kk, CF, M, A)                                                            \
    asm(PM_FMAC_DPP(Kk, 0) PM_FMAC_DPP(Kk, 1) PM_FMAC_DPP(Kk, 2) PM_FMAC_DPP(Kk, 3)             \
        : "+v"((A).v[0]), "+v"((A).v[1]), "+v"((A).v[2]), "+v"((A).v[3])                        \
        : "v"(CF), "v"((M).v[0]), "v"((M).v[1]), "v"((M).v[2]), "v"((M).v[3]))

__device__ __forceinline__ void fma_bcast16(float cf, const Pack<4> (&fl)[16], Pack<4> &w)
{
    PM_FMAC4_BCAST0(cf, fl[0], w);
    PM_FMAC4_BCAST(1, cf, fl[1], w);   PM_FMAC4_BCAST(2, cf, fl[2], w);   PM_FMAC4_BCAST(3, cf, fl[3], w);
    PM_FMAC4_BCAST(4, cf, fl[4], w);   PM_FMAC4_BCAST(5, cf, fl[5], w);   PM_FMAC4_BCAST(6, cf, fl[6], w);
    PM_FMAC4_BCAST(7, cf, fl[7], w);   PM_FMAC4_BCAST(8, cf, fl[8], w);   PM_FMAC4_BCAST(9, cf, fl[9], w);
    PM_FMAC4_BCAST(10, cf, fl[10], w); PM_FMAC4_BCAST(11, cf, fl[11], w); PM_FMAC4_BCAST(12, cf, fl[12], w);
    PM_FMAC4_BCAST(13, cf, fl[13], w); PM_FMAC4_BCAST(14, cf, fl[14], w); PM_FMAC4_BCAST(15, cf, fl[15], w);
}

// The four output channels co .. co+3 of a lane read the input channels co/R .. : for R = 1 four
// distinct ones, for R = 2 two, each used twice (out[., c*R + m]).  InRow keeps the loaded words as they
// come (expanding them right after a conditional load would make that load wait on the spot and undo
// the batching of the gathers); channel u of the four reads v[u / R].
template <int R> struct InRow { float v[4 / R]; };
template <int R> __device__ __forceinline__ InRow<R> zero_in()
{
    InRow<R> o;
#pragma unroll
    for (int i = 0; i < 4 / R; ++i) o.v[i] = 0.f;
    return o;
}
template <int R> __device__ __forceinline__ InRow<R> ld_in(const float *p)
{
    InRow<R> o;
    if constexpr (R == 1) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        o.v[0] = t.x; o.v[1] = t.y; o.v[2] = t.z; o.v[3] = t.w;
    } else {
        const float2 t = *reinterpret_cast<const float2 *>(p);
        o.v[0] = t.x; o.v[1] = t.y;
    }
    return o;
}

// facet2vertex forward for depth multiplier R = 1 or 2, Co = C*R a multiple of 4 and >= 64 (a 16-lane DPP row
// then lies inside one vertex's row group; lanes past Co/4 are masked), K <= 16.
// Persistent row groups: the filter stays in registers for all the vertices a group visits, and three
// stages of gathers are in flight at once -- the row bounds of the vertex after next, the entry list of
// the next vertex, and the facet rows / coefficients of the current one (eight entries at a time).
template <int R>
__global__ __launch_bounds__(kBlock) void f2v_fwd_fast_k(const float *__restrict__ in, const float *__restrict__ filt,
                                                         const float *__restrict__ coeff,
                                                         const int *__restrict__ nfcount,
                                                         const int *__restrict__ rowptr,
                                                         const int *__restrict__ colidx, float *__restrict__ out,
                                                         int64_t NvOut, int C, int K, int lpr_log2)
{
    constexpr int EB = 8;
    const int lpr = 1 << lpr_log2, rpb = kBlock >> lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2, l16 = threadIdx.x & 15;
    const int Co = C * R;
    const int c = lane * 4;                       // my four output channels; input channels c / R ..
    const bool on = c < Co;
    const bool kok = l16 < K;
    Pack<4> fl[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) fl[k] = (k < K && on) ? ldp<4>(filt + (size_t)k * Co + c) : zero_pack<4>();

    // Workgroups go round-robin to the eight accelerator dies, each with an L2 of its own: die x takes the
    // x-th contiguous eighth of the vertices, so that the vertices sharing a facet row mostly meet in one L2.
    const int64_t groups = (NvOut + rpb - 1) / rpb, gx = (groups + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int64_t stride = (int64_t)(gridDim.x >> 3) * rpb;
    const int64_t xend = (xcd + 1) * gx * rpb;
    const int64_t NvEnd = xend < NvOut ? xend : NvOut;
    int64_t row = (xcd * gx + (blockIdx.x >> 3)) * rpb + slot;
    // stage 1 (row bounds) of rows `row` and `row + stride`, stage 2 (entries) of `row`
    int e0 = 0, e1 = 0, ne0 = 0, ne1 = 0;
    if (row < NvEnd) { e0 = rowptr[row]; e1 = rowptr[row + 1]; }
    if (row + stride < NvEnd) { ne0 = rowptr[row + stride]; ne1 = rowptr[row + stride + 1]; }
    int f[EB];
#pragma unroll
    for (int i = 0; i < EB; ++i) f[i] = (e0 + i < e1) ? colidx[e0 + i] / 3 : -1;

    for (; row < NvEnd; row += stride) {
        // row bounds two rows ahead, entry list one row ahead
        int me0 = 0, me1 = 0;
        if (row + 2 * stride < NvEnd) { me0 = rowptr[row + 2 * stride]; me1 = rowptr[row + 2 * stride + 1]; }
        int nf[EB];
#pragma unroll
        for (int i = 0; i < EB; ++i) nf[i] = (ne0 + i < ne1) ? colidx[ne0 + i] / 3 : -1;
        const float inv = (e1 > e0) ? 1.0f / (float)nfcount[row] : 0.f;

        Pack<4> acc = zero_pack<4>();
        for (int eb = e0; eb < e1; eb += EB) {
            if (eb > e0) {                                   // vertices with more than eight entries
#pragma unroll
                for (int i = 0; i < EB; ++i) f[i] = (eb + i < e1) ? colidx[eb + i] / 3 : -1;
            }
            InRow<R> x[EB];
            float cf[EB];
#pragma unroll
            for (int i = 0; i < EB; ++i) {
                x[i] = (f[i] >= 0 && on) ? ld_in<R>(in + (int64_t)f[i] * C + c / R) : zero_in<R>();
                cf[i] = (f[i] >= 0 && kok) ? coeff[(int64_t)f[i] * K + l16] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < EB; ++i) {
                if (eb + i < e1) {
                    Pack<4> w = zero_pack<4>();
                    fma_bcast16(cf[i], fl, w);
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc.v[u] = fmaf(w.v[u], x[i].v[u / R], acc.v[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) acc.v[u] *= inv;
        if (on) stp<4>(out + row * Co + c, acc);
        e0 = ne0; e1 = ne1; ne0 = me0; ne1 = me1;
#pragma unroll
        for (int i = 0; i < EB; ++i) f[i] = nf[i];
    }
}

// ----------------------------------------------------------------------------------------
// facet2vertex backward, one pass over the facets:
//   s[f,co]      = sum_{corner j, vo_j >= 0} gout[vo_j,co] / nf[vo_j]
//   gin[f,c]     = sum_m s[f,co] * w[f,co],   w = sum_k coeff[f,k] * filt[k,co]
//   gfilt[k,co]  = sum_f coeff[f,k] * in[f,c] * s[f,co]                (per-workgroup partials)
// ----------------------------------------------------------------------------------------
template <int V>
__global__ __launch_bounds__(kBlock) void f2v_bwd_k(const float *__restrict__ gout,
                                                    const float *__restrict__ in,
                                                    const float *__restrict__ filt,
                                                    const float *__restrict__ coeff,
                                                    const int *__restrict__ face,
                                                    const int *__restrict__ nfcount,
                                                    const int *__restrict__ vtmap,
                                                    float *__restrict__ gin, float *__restrict__ partial,
                                                    int64_t Nf, int64_t NvOut, int C, int r, int K, int Q,
                                                    int lpr_log2, int coeff_vec, int64_t rows_per_block)
{
    __shared__ float red[kBlock * V];
    const int lpr = 1 << lpr_log2, rpb = kBlock >> lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int Co = C * r;
    const int64_t fbeg = (int64_t)blockIdx.x * rows_per_block;
    const int64_t fend = (fbeg + rows_per_block < Nf) ? fbeg + rows_per_block : Nf;
    for (int m = 0; m < r; ++m)
        for (int q0 = 0; q0 < Q; q0 += lpr) {
            const int q = q0 + lane;
            const bool active = q < Q;
            const int c = q * V;
            const int co = (V == 4) ? c : c * r + m;
            for (int k0 = 0; k0 < K; k0 += 16) {
                const int kc = (K - k0 < 16) ? K - k0 : 16;
                const bool first = (m == 0 && k0 == 0);
                Pack<V> fl[16], acc[16];
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    fl[k] = (active && k < kc) ? ldp<V>(filt + (size_t)(k0 + k) * Co + co) : zero_pack<V>();
                    acc[k] = zero_pack<V>();
                }
                if (active)
                    for (int64_t f = fbeg + slot; f < fend; f += rpb) {
                        Pack<V> s = zero_pack<V>();
#pragma unroll
                        for (int j = 0; j < 3; ++j) {
                            const int vo = vtmap[face[3 * f + j]];
                            if (vo >= 0 && vo < NvOut) {
                                const float inv = 1.0f / (float)nfcount[vo];
                                const Pack<V> g = ldp<V>(gout + (int64_t)vo * Co + co);
#pragma unroll
                                for (int i = 0; i < V; ++i) s.v[i] = fmaf(g.v[i], inv, s.v[i]);
                            }
                        }
                        const Pack<V> x = ldp<V>(in + f * C + c);
                        float cf[16];
                        load_coeff16(coeff + f * K + k0, kc, coeff_vec != 0, cf);
                        Pack<V> w = zero_pack<V>(), t;
#pragma unroll
                        for (int k = 0; k < 16; ++k)
#pragma unroll
                            for (int i = 0; i < V; ++i) w.v[i] = fmaf(cf[k], fl[k].v[i], w.v[i]);
#pragma unroll
                        for (int i = 0; i < V; ++i) t.v[i] = x.v[i] * s.v[i];
#pragma unroll
                        for (int k = 0; k < 16; ++k)
#pragma unroll
                            for (int i = 0; i < V; ++i) acc[k].v[i] = fmaf(cf[k], t.v[i], acc[k].v[i]);
                        float *gp = gin + f * C + c;
                        if (first) {
                            Pack<V> gi;
#pragma unroll
                            for (int i = 0; i < V; ++i) gi.v[i] = s.v[i] * w.v[i];
                            stp<V>(gp, gi);
                        } else {
#pragma unroll
                            for (int i = 0; i < V; ++i) gp[i] = fmaf(s.v[i], w.v[i], gp[i]);
                        }
                    }
#pragma unroll
                for (int k = 0; k < 16; ++k)
                    if (k < kc)
                        block_reduce_store<V>(acc[k], red,
                                              partial + ((size_t)blockIdx.x * K + k0 + k) * Co + co, active,
                                              lane, slot, lpr, rpb);
            }
        }
}

// facet2vertex backward for r = 1, C % 64 == 0, K <= 16: same arithmetic as f2v_bwd_k with the
// coefficient row spread over the 16 lanes of a DPP row, and the index chain
// face -> vt_map -> (nf_count, gout rows) of the NEXT facet resolved while the current one is computed.
template <int R>
__global__ __launch_bounds__(kBlock) void f2v_bwd_fast_k(const float *__restrict__ gout, const float *__restrict__ in,
                                                         const float *__restrict__ filt,
                                                         const float *__restrict__ coeff,
                                                         const int *__restrict__ face,
                                                         const int *__restrict__ nfcount,
                                                         const int *__restrict__ vtmap, float *__restrict__ gin,
                                                         float *__restrict__ partial, int64_t Nf, int64_t NvOut, int C,
                                                         int K, int lpr_log2, int64_t rows_per_block)
{
    __shared__ float red[kBlock * 4];
    const int lpr = 1 << lpr_log2, rpb = kBlock >> lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2, l16 = threadIdx.x & 15;
    const int64_t fbeg = (int64_t)blockIdx.x * rows_per_block;
    const int64_t fend = (fbeg + rows_per_block < Nf) ? fbeg + rows_per_block : Nf;
    const int Co = C * R;
    const int c = lane * 4;                       // my four output channels; input channels c / R ..
    const bool on = c < Co;
    Pack<4> fl[16], acc[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        fl[k] = (k < K && on) ? ldp<4>(filt + (size_t)k * Co + c) : zero_pack<4>();
        acc[k] = zero_pack<4>();
    }
    // software pipeline over this slot's facets: indices two facets ahead, output rows one ahead
    int64_t f = fbeg + slot;
    int va[3] = {0, 0, 0}, vo[3] = {-1, -1, -1};
    if (f < fend) {
#pragma unroll
        for (int j = 0; j < 3; ++j) va[j] = face[3 * f + j];
#pragma unroll
        for (int j = 0; j < 3; ++j) vo[j] = vtmap[va[j]];
    }
    if (f + rpb < fend) {
#pragma unroll
        for (int j = 0; j < 3; ++j) va[j] = face[3 * (f + rpb) + j];
    }
    for (; f < fend; f += rpb) {
        // data of facet f (its output rows are known), indices of the following two
        int von[3] = {-1, -1, -1};
        if (f + rpb < fend) {
#pragma unroll
            for (int j = 0; j < 3; ++j) von[j] = vtmap[va[j]];
        }
        if (f + 2 * rpb < fend) {
#pragma unroll
            for (int j = 0; j < 3; ++j) va[j] = face[3 * (f + 2 * rpb) + j];
        }
        Pack<4> g[3];
        float nf[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const bool ok = vo[j] >= 0 && vo[j] < NvOut;
            g[j] = (ok && on) ? ldp<4>(gout + (int64_t)vo[j] * Co + c) : zero_pack<4>();
            nf[j] = ok ? (float)nfcount[vo[j]] : 1.f;
        }
        const InRow<R> x = on ? ld_in<R>(in + f * C + c / R) : zero_in<R>();
        float cf = (l16 < K) ? coeff[f * K + l16] : 0.f;
        Pack<4> s = zero_pack<4>(), w = zero_pack<4>(), t;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const float inv = 1.0f / nf[j];
#pragma unroll
            for (int u = 0; u < 4; ++u) s.v[u] = fmaf(g[j].v[u], inv, s.v[u]);
        }
        fma_bcast16(cf, fl, w);
#pragma unroll
        for (int u = 0; u < 4; ++u) t.v[u] = x.v[u / R] * s.v[u];
        PM_FMAC4_BCAST0(cf, t, acc[0]);
        PM_FMAC4_BCAST(1, cf, t, acc[1]);   PM_FMAC4_BCAST(2, cf, t, acc[2]);   PM_FMAC4_BCAST(3, cf, t, acc[3]);
        PM_FMAC4_BCAST(4, cf, t, acc[4]);   PM_FMAC4_BCAST(5, cf, t, acc[5]);   PM_FMAC4_BCAST(6, cf, t, acc[6]);
        PM_FMAC4_BCAST(7, cf, t, acc[7]);   PM_FMAC4_BCAST(8, cf, t, acc[8]);   PM_FMAC4_BCAST(9, cf, t, acc[9]);
        PM_FMAC4_BCAST(10, cf, t, acc[10]); PM_FMAC4_BCAST(11, cf, t, acc[11]); PM_FMAC4_BCAST(12, cf, t, acc[12]);
        PM_FMAC4_BCAST(13, cf, t, acc[13]); PM_FMAC4_BCAST(14, cf, t, acc[14]); PM_FMAC4_BCAST(15, cf, t, acc[15]);
        if (on) {
            if constexpr (R == 1) {
                Pack<4> gi;
#pragma unroll
                for (int u = 0; u < 4; ++u) gi.v[u] = s.v[u] * w.v[u];
                stp<4>(gin + f * C + c, gi);
            } else {                                  // two input channels, each the sum over its two outputs
                *reinterpret_cast<float2 *>(gin + f * C + c / R) =
                    make_float2(fmaf(s.v[1], w.v[1], s.v[0] * w.v[0]), fmaf(s.v[3], w.v[3], s.v[2] * w.v[2]));
            }
        }
#pragma unroll
        for (int j = 0; j < 3; ++j) vo[j] = von[j];
    }
#pragma unroll
    for (int k = 0; k < 16; ++k)
        if (k < K)
            block_reduce_store<4>(acc[k], red, partial + ((size_t)blockIdx.x * K + k) * Co + c, on, lane, slot, lpr, rpb);
}

// ----------------------------------------------------------------------------------------
// pooling / unpooling over decimation clusters
//   rep(v) = vt_replace[v] < 0 ? -vt_replace[v] : v ;  vo(v) = vt_map[rep(v)] ;
//   cnt(v) = vt_replace[rep(v)] + 1
// ----------------------------------------------------------------------------------------
__device__ __forceinline__ int cluster_of(const int *__restrict__ vtrep, const int *__restrict__ vtmap,
                                          int64_t v, int64_t n_fine, int64_t n_coarse, int *cnt)
{
    const int rp = vtrep[v];
    const int64_t rep = rp < 0 ? -(int64_t)rp : v;
    if (rep >= n_fine) return -1;
    const int vo = vtmap[rep];
    if (vo < 0 || vo >= n_coarse) return -1;
    if (cnt) *cnt = vtrep[rep] + 1;
    return vo;
}

// max pooling forward over the coarse-vertex -> members adjacency (members ascending):
// running maximum that ignores NaN, first (smallest) member attaining it is the arg-max.
template <int V>
__global__ __launch_bounds__(kBlock) void pool_max_fwd_k(const float *__restrict__ in,
                                                         const int *__restrict__ rowptr,
                                                         const int *__restrict__ members,
                                                         float *__restrict__ out, int *__restrict__ maxidx,
                                                         int64_t NvOut, int C, int Q, int lpr_log2)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= NvOut) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    for (int q = lane; q < Q; q += lpr) {
        const int c = q * V;
        Pack<V> best = zero_pack<V>();
        int idx[V];
#pragma unroll
        for (int i = 0; i < V; ++i) idx[i] = 0;
        // members four at a time: their rows are all requested before the first comparison
        constexpr int EB = 4;
        for (int eb = e0; eb < e1; eb += EB) {
            int v[EB];
#pragma unroll
            for (int j = 0; j < EB; ++j) v[j] = (eb + j < e1) ? members[eb + j] : -1;
            Pack<V> x[EB];
#pragma unroll
            for (int j = 0; j < EB; ++j) x[j] = (v[j] >= 0) ? ldp<V>(in + (int64_t)v[j] * C + c) : zero_pack<V>();
#pragma unroll
            for (int j = 0; j < EB; ++j) {
                if (eb + j < e1) {
#pragma unroll
                    for (int i = 0; i < V; ++i) {
                        const float b = best.v[i], y = x[j].v[i];
                        const bool take = (eb + j == e0) || (y > b) || (b != b && y == y);
                        best.v[i] = take ? y : b;
                        idx[i] = take ? ((y == y) ? v[j] : 0) : idx[i];
                    }
                }
            }
        }
        stp<V>(out + row * C + c, best);
        if constexpr (V == 4) {
            *reinterpret_cast<int4 *>(maxidx + row * C + c) = make_int4(idx[0], idx[1], idx[2], idx[3]);
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) maxidx[row * C + c + i] = idx[i];
        }
    }
}

// segmented sum over cluster members: AVG weights each member by 1/cnt(member) (avg pool
// forward), otherwise plain sum (unpool backward).
template <int V, bool AVG>
__global__ __launch_bounds__(kBlock) void cluster_sum_k(const float *__restrict__ in,
                                                        const int *__restrict__ vtrep,
                                                        const int *__restrict__ rowptr,
                                                        const int *__restrict__ members,
                                                        float *__restrict__ out, int64_t NvFine,
                                                        int64_t NvOut, int C, int Q, int lpr_log2)
{
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= NvOut) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    for (int q = lane; q < Q; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        // members four at a time: indices, then all rows (and the cluster size), then the sums in member order
        constexpr int EB = 4;
        for (int eb = e0; eb < e1; eb += EB) {
            int64_t v[EB];
#pragma unroll
            for (int j = 0; j < EB; ++j) v[j] = (eb + j < e1) ? members[eb + j] : -1;
            Pack<V> x[EB];
            float wgt[EB];
            int rp[EB], cnt[EB];
#pragma unroll
            for (int j = 0; j < EB; ++j) {
                x[j] = (v[j] >= 0) ? ldp<V>(in + v[j] * C + c) : zero_pack<V>();
                rp[j] = (AVG && v[j] >= 0) ? vtrep[v[j]] : 0;
            }
#pragma unroll
            for (int j = 0; j < EB; ++j) {                 // cluster size, stored at the representative
                const int64_t rep = rp[j] < 0 ? -(int64_t)rp[j] : v[j];
                cnt[j] = (AVG && v[j] >= 0) ? vtrep[rep < NvFine ? rep : v[j]] : 0;
            }
#pragma unroll
            for (int j = 0; j < EB; ++j) wgt[j] = AVG ? 1.0f / (float)(cnt[j] + 1) : 1.f;
#pragma unroll
            for (int j = 0; j < EB; ++j)
                if (eb + j < e1) {
#pragma unroll
                    for (int i = 0; i < V; ++i) acc.v[i] = AVG ? fmaf(x[j].v[i], wgt[j], acc.v[i]) : acc.v[i] + x[j].v[i];
                }
        }
        stp<V>(out + row * C + c, acc);
    }
}

// per-fine-vertex gathers from the cluster's coarse row.
enum FineMode { kUnpoolFwd = 0, kAvgBwd = 1, kMaxBwdGather = 2 };

// A row group takes kFineBatch consecutive fine vertices and walks the index chain
// vt_replace -> vt_map (-> cluster size) -> coarse row for all of them in step, so that the three
// dependent round trips are paid once per batch.
constexpr int kFineBatch = 4;

template <int V, int MODE>
__global__ __launch_bounds__(kBlock) void fine_gather_k(const float *__restrict__ coarse,
                                                        const int *__restrict__ maxidx,
                                                        const int *__restrict__ vtrep,
                                                        const int *__restrict__ vtmap,
                                                        float *__restrict__ fine, int64_t NvFine,
                                                        int64_t NvCoarse, int C, int Q, int lpr_log2)
{
    constexpr int NB = kFineBatch;
    const int lpr = 1 << lpr_log2;
    const int lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t v0 = ((int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot) * NB;
    if (v0 >= NvFine) return;
    int rp[NB], vo[NB], cnt[NB];
    int64_t rep[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) rp[j] = (v0 + j < NvFine) ? vtrep[v0 + j] : 0;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        rep[j] = rp[j] < 0 ? -(int64_t)rp[j] : v0 + j;
        const bool ok = v0 + j < NvFine && rep[j] < NvFine;
        vo[j] = ok ? vtmap[rep[j]] : -1;
        cnt[j] = (ok && MODE == kAvgBwd) ? vtrep[rep[j]] + 1 : 1;
        if (vo[j] >= NvCoarse) vo[j] = -1;
    }
    for (int q = lane; q < Q; q += lpr) {
        const int c = q * V;
        Pack<V> g[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j) g[j] = (vo[j] >= 0) ? ldp<V>(coarse + (int64_t)vo[j] * C + c) : zero_pack<V>();
        if constexpr (MODE == kMaxBwdGather) {
            int mi[NB][V];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                if constexpr (V == 4) {
                    const int4 m4 = (vo[j] >= 0) ? *reinterpret_cast<const int4 *>(maxidx + (int64_t)vo[j] * C + c)
                                                 : make_int4(-1, -1, -1, -1);
                    mi[j][0] = m4.x; mi[j][1] = m4.y; mi[j][2] = m4.z; mi[j][3] = m4.w;
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) mi[j][i] = (vo[j] >= 0) ? maxidx[(int64_t)vo[j] * C + c + i] : -1;
                }
            }
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int i = 0; i < V; ++i) g[j].v[i] = (mi[j][i] == (int)(v0 + j)) ? g[j].v[i] : 0.f;
        } else if constexpr (MODE == kAvgBwd) {
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const float d = (float)cnt[j];
#pragma unroll
                for (int i = 0; i < V; ++i) g[j].v[i] = g[j].v[i] / d;
            }
        }
#pragma unroll
        for (int j = 0; j < NB; ++j)
            if (v0 + j < NvFine) stp<V>(fine + (v0 + j) * C + c, g[j]);
    }
}

// reference form of max-pool backward: scatter by max_index into a cleared gradient.
__global__ __launch_bounds__(kBlock) void pool_max_bwd_scatter_k(const float *__restrict__ gout,
                                                                 const int *__restrict__ maxidx,
                                                                 float *__restrict__ gin, int64_t n,
                                                                 int C, int64_t NvIn)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int ch = (int)(i % C);
    const int64_t v = maxidx[i];
    if (v >= 0 && v < NvIn) gin[v * C + ch] = gout[i];
}

// ----------------------------------------------------------------------------------------
// real spherical-harmonic basis, degree <= 5, cartesian closed forms on the unit direction
// ----------------------------------------------------------------------------------------
// (the degree is a compile-time constant so that a row stays in registers)
template <int L>
__global__ __launch_bounds__(kBlock) void sph_harm_k(const float *__restrict__ xyz, float *__restrict__ out, int64_t N)
{
    const int64_t n = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (n >= N) return;
    constexpr int B = (L + 1) * (L + 1);
    float v[B];
    sph_harm_at(xyz[3 * n], xyz[3 * n + 1], xyz[3 * n + 2], L, v);
    float *o = out + n * B;
    if constexpr (B % 4 == 0) {
        // (rows of 16 or 64 bytes times a multiple: aligned whenever the array is)
        if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
#pragma unroll
            for (int i = 0; i < B; i += 4) *reinterpret_cast<float4 *>(o + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) o[i] = v[i];
}

// ----------------------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------------------
static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// vertex2facet: V = 4 also with depth multiplier 2 (two input channels per lane) when C is even
static inline int pick_v2f(int C, int r, std::initializer_list<const void *> ptrs)
{
    if (!((r == 1 && !(C & 3)) || (r == 2 && !(C & 1)))) return 1;
    for (const void *p : ptrs)
        if ((reinterpret_cast<uintptr_t>(p) & 15u) != 0) return 1;
    return 4;
}

// V = 4 needs r == 1, C % 4 == 0 and 16-byte aligned feature arrays.
static inline int pick_v(int C, int r, std::initializer_list<const void *> ptrs)
{
    if (r != 1 || (C & 3)) return 1;
    for (const void *p : ptrs)
        if (!aligned16(p)) return 1;
    return 4;
}

// ----------------------------------------------------------------------------------------
// per-level producers of the convolution inputs
// ----------------------------------------------------------------------------------------
// nf_count[v] = number of (facet, corner) entries landing on output vertex v = its CSR row length
__global__ __launch_bounds__(kBlock) void row_length_k(const int *__restrict__ rowptr, int *__restrict__ out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = rowptr[i + 1] - rowptr[i];
}

// geometry[f] = (unit normal (3), plane offset d = -n.v0, area) of triangle f; vertex rows have
// `vstride` floats of which the first three are the position
__global__ __launch_bounds__(kBlock) void triangle_geometry_k(const float *__restrict__ vertex, const int *__restrict__ face,
                                                             float *__restrict__ geometry, int64_t Nf, int vstride)
{
    const int64_t f = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (f >= Nf) return;
    const float *a = vertex + (int64_t)face[3 * f] * vstride;
    const float *b = vertex + (int64_t)face[3 * f + 1] * vstride;
    const float *c = vertex + (int64_t)face[3 * f + 2] * vstride;
    const float ax = a[0], ay = a[1], az = a[2];
    const float ux = b[0] - ax, uy = b[1] - ay, uz = b[2] - az;
    const float vx = c[0] - ax, vy = c[1] - ay, vz = c[2] - az;
    const float nx = uy * vz - uz * vy, ny = uz * vx - ux * vz, nz = ux * vy - uy * vx;
    const float len = sqrtf(nx * nx + ny * ny + nz * nz);
    const float inv = 1.0f / (len + 1e-10f);
    float *g = geometry + 5 * f;
    g[0] = nx * inv; g[1] = ny * inv; g[2] = nz * inv;
    g[3] = -(g[0] * ax + g[1] * ay + g[2] * az);
    g[4] = 0.5f * len;
}

// The fast facet2vertex kernels: depth multiplier 1 or 2, Co = C*r a multiple of 4 in [64, 1024] (row groups
// of at least one 16-lane DPP row), at most 16 coefficients, 16-byte aligned rows.
static bool f2v_fast_ok(int C, int r, int K, std::initializer_list<const void *> ptrs)
{
    const int Co = C * r;
    if (!(r == 1 || r == 2) || (Co & 3) || Co < 64 || Co > 1024 || K > 16) return false;
    for (const void *p : ptrs)
        if (!aligned16(p)) return false;
    return true;
}

// the vector-ALU kernels on request (tests compare the two paths)
static bool force_valu() { return options().f2v_valu; }

int reduce_partials(const float *partial, float *out, int G, int n, hipStream_t st, size_t stride)
{
    reduce_partials_k<<<dim3((unsigned)ceil_div(n, 16)), dim3(1024), 0, st>>>(partial, out, G, n, stride ? stride : (size_t)n);
    PM_LAUNCHED("reduce_partials");
    return 0;
}

}  // namespace pmesh

using namespace pmesh;

#define PM_DIMS(name)                                                                     \
    PM_REQUIRE(C > 0 && r > 0 && (int64_t)C * r <= (1 << 20), name ": bad channel counts C=%d r=%d", C, r)

extern "C" int pmesh_v2f_fwd(const float *input, const float *filter, const int32_t *face, float *output,
                             int64_t Nv, int64_t Nf, int C, int r, pmesh_stream_t stream)
{
    clear_error();
    PM_DIMS("v2f_fwd");
    PM_REQUIRE(Nv >= 0 && Nf >= 0, "v2f_fwd: negative size");
    if (Nf == 0) return 0;
    PM_REQUIRE(input && filter && face && output, "v2f_fwd: null pointer");
    PM_REQUIRE(Nv > 0, "v2f_fwd: facets given but no input vertices");
    PM_REQUIRE(Nv <= INT32_MAX && Nf <= INT32_MAX / 3, "v2f_fwd: sizes exceed int32 indexing");
    hipStream_t st = (hipStream_t)stream;
    const int V = pick_v2f(C, r, {input, filter, output});
    const RowShape rs = row_shape(C * r / V);
    const int64_t blocks = ceil_div(Nf, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "v2f_fwd: grid too large");
    if (V == 4 && r == 2)
        v2f_fwd_k<4, 2><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, face, output, Nf, C, r, rs.items, rs.lpr_log2);
    else if (V == 4)
        v2f_fwd_k<4, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, face, output, Nf, C, r, rs.items, rs.lpr_log2);
    else
        v2f_fwd_k<1, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, face, output, Nf, C, r, rs.items, rs.lpr_log2);
    PM_LAUNCHED("v2f_fwd");
    return 0;
}

// workspace = per-workgroup partial filter gradients, worst case 1024 workgroups
extern "C" size_t pmesh_v2f_bwd_workspace_bytes(int C, int r) { return (size_t)1024 * 3 * C * r * sizeof(float); }

extern "C" int pmesh_v2f_bwd(const float *grad_output, const float *input, const float *filter,
                             const int32_t *face, const int32_t *rowptr, const int32_t *colidx,
                             float *grad_input, float *grad_filter, void *workspace, size_t workspace_bytes,
                             int64_t Nv, int64_t Nf, int C, int r, pmesh_stream_t stream)
{
    clear_error();
    (void)face;
    PM_DIMS("v2f_bwd");
    PM_REQUIRE(Nv >= 0 && Nf >= 0, "v2f_bwd: negative size");
    PM_REQUIRE(grad_filter, "v2f_bwd: null grad_filter");
    PM_REQUIRE(Nv <= INT32_MAX && Nf <= INT32_MAX / 3, "v2f_bwd: sizes exceed int32 indexing");
    hipStream_t st = (hipStream_t)stream;
    const int Co = C * r;
    if (Nv == 0) {
        fill_zero_k<<<dim3((unsigned)ceil_div(3 * Co, kBlock)), dim3(kBlock), 0, st>>>(grad_filter, 3 * Co);
        PM_LAUNCHED("v2f_bwd(fill)");
        return 0;
    }
    PM_REQUIRE(grad_output && input && filter && rowptr && colidx && grad_input && workspace, "v2f_bwd: null pointer");
    const int V = pick_v2f(C, r, {grad_output, input, filter, grad_input, workspace});
    const RowShape rs = row_shape(V == 4 ? Co / 4 : C);
    const int G = persistent_blocks(Nv, rs.rpb);
    const int64_t rows_per_block = ceil_div(ceil_div(Nv, G), rs.rpb) * rs.rpb;
    PM_REQUIRE(workspace_bytes >= (size_t)G * 3 * Co * sizeof(float), "v2f_bwd: workspace too small (%zu bytes)", workspace_bytes);
    float *partial = (float *)workspace;
    if (V == 4 && r == 2)
        v2f_bwd_k<4, 2><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, rowptr, colidx, grad_input, partial, Nv, C, r, rs.items, rs.lpr_log2, rows_per_block);
    else if (V == 4)
        v2f_bwd_k<4, 1><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, rowptr, colidx, grad_input, partial, Nv, C, r, rs.items, rs.lpr_log2, rows_per_block);
    else
        v2f_bwd_k<1, 1><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, rowptr, colidx, grad_input, partial, Nv, C, r, rs.items, rs.lpr_log2, rows_per_block);
    PM_LAUNCHED("v2f_bwd");
    return reduce_partials(partial, grad_filter, G, 3 * Co, st);
}

extern "C" int pmesh_f2v_fwd(const float *input, const float *filter, const float *coeff,
                             const int32_t *nf_count, const int32_t *rowptr, const int32_t *colidx,
                             float *output, int64_t Nf, int64_t NvOut, int C, int r, int K,
                             pmesh_stream_t stream)
{
    clear_error();
    PM_DIMS("f2v_fwd");
    PM_REQUIRE(K > 0 && K <= 4096, "f2v_fwd: bad filter size K=%d", K);
    PM_REQUIRE(Nf >= 0 && NvOut >= 0, "f2v_fwd: negative size");
    if (NvOut == 0) return 0;
    PM_REQUIRE(input && filter && coeff && nf_count && rowptr && colidx && output, "f2v_fwd: null pointer");
    PM_REQUIRE(NvOut <= INT32_MAX && Nf <= INT32_MAX / 3, "f2v_fwd: sizes exceed int32 indexing");
    hipStream_t st = (hipStream_t)stream;
    const int V = pick_v(C, r, {input, filter, output});
    const RowShape rs = row_shape(C * r / V);
    const int64_t blocks = ceil_div(NvOut, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "f2v_fwd: grid too large");
    const int cvec = ((K & 3) == 0 && aligned16(coeff)) ? 1 : 0;
    if (!force_valu() && f2v_mfma_ok(Nf, C, r, K, coeff)) return f2v_fwd_mfma(input, filter, coeff, nf_count, rowptr, colidx, output, Nf, NvOut, C, r, st);
    if (f2v_fast_ok(C, r, K, {input, filter, output})) {
        // persistent: enough workgroups to fill the chip several times over, each visiting many vertices
        const RowShape fs = row_shape(C * r / 4);
        const int64_t fb = ceil_div(ceil_div(NvOut, fs.rpb), 8) * 8, pb = fb < 4096 ? fb : 4096;   // a multiple of 8
        if (r == 1)
            f2v_fwd_fast_k<1><<<dim3((unsigned)pb), dim3(kBlock), 0, st>>>(input, filter, coeff, nf_count, rowptr, colidx, output, NvOut, C, K, fs.lpr_log2);
        else
            f2v_fwd_fast_k<2><<<dim3((unsigned)pb), dim3(kBlock), 0, st>>>(input, filter, coeff, nf_count, rowptr, colidx, output, NvOut, C, K, fs.lpr_log2);
    }
    else if (V == 4)
        f2v_fwd_k<4><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, coeff, nf_count, rowptr, colidx, output, NvOut, C, r, K, rs.items, rs.lpr_log2, cvec);
    else
        f2v_fwd_k<1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, coeff, nf_count, rowptr, colidx, output, NvOut, C, r, K, rs.items, rs.lpr_log2, cvec);
    PM_LAUNCHED("f2v_fwd");
    return 0;
}

extern "C" int pmesh_f2v_dense_supported(int64_t Nf, int C, int r, int K, int Co, const float *coeff)
{
    return (!force_valu() && !options().f2v_fp32mfma && f2v_tail_ok(Nf, C, r, K, coeff, Co)) ? 1 : 0;
}

extern "C" size_t pmesh_f2v_dense_fwd_workspace_bytes(int C, int r, int Co)
{
    if (C <= 0 || r <= 0 || Co <= 0) return 256;
    return f2v_tail_workspace_bytes(((C * r + 31) / 32) * 32, ((Co + 15) / 16) * 16) + 256;
}

extern "C" int pmesh_f2v_dense_fwd(const float *input, const float *filter, const float *coeff,
                                   const int32_t *nf_count, const int32_t *rowptr, const int32_t *colidx,
                                   const float *weight, const float *bias, const float *scale, const float *shift,
                                   int relu, float *output, uint32_t *relu_bits, float *conv_rows, void *workspace,
                                   size_t workspace_bytes, int64_t Nf, int64_t NvOut, int C, int r, int K, int Co,
                                   pmesh_stream_t stream)
{
    clear_error();
    PM_DIMS("f2v_dense_fwd");
    PM_REQUIRE(Nf >= 0 && NvOut >= 0, "f2v_dense_fwd: negative size");
    if (NvOut == 0) return 0;
    PM_REQUIRE(input && filter && coeff && nf_count && rowptr && colidx && weight && output && workspace,
               "f2v_dense_fwd: null pointer");
    PM_REQUIRE(NvOut <= INT32_MAX && Nf <= INT32_MAX / 3, "f2v_dense_fwd: sizes exceed int32 indexing");
    PM_REQUIRE(pmesh_f2v_dense_supported(Nf, C, r, K, Co, coeff),
               "f2v_dense_fwd: takes 16 coefficients in 16-byte aligned rows, 32 or 64 convolution channels and 32, 64 or 128 "
               "output channels (K=%d C=%d r=%d Co=%d)", K, C, r, Co);
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0 && workspace_bytes >= f2v_tail_workspace_bytes(C * r, Co),
               "f2v_dense_fwd: workspace too small or misaligned (%zu bytes)", workspace_bytes);
    return f2v_fwd_tail(input, filter, coeff, nf_count, rowptr, colidx, conv_rows, weight, bias, scale, shift, relu, output,
                        relu_bits, workspace, Nf, NvOut, C, r, Co, (hipStream_t)stream);
}

extern "C" size_t pmesh_f2v_bwd_workspace_bytes(int C, int r, int K) { return (size_t)1024 * K * C * r * sizeof(float); }

extern "C" int pmesh_f2v_bwd(const float *grad_output, const float *input, const float *filter,
                             const float *coeff, const int32_t *face, const int32_t *nf_count,
                             const int32_t *vt_map, float *grad_input, float *grad_filter, void *workspace,
                             size_t workspace_bytes, int64_t Nf, int64_t NvIn, int64_t NvOut, int C, int r,
                             int K, pmesh_stream_t stream)
{
    clear_error();
    (void)NvIn;
    PM_DIMS("f2v_bwd");
    PM_REQUIRE(K > 0 && K <= 4096, "f2v_bwd: bad filter size K=%d", K);
    PM_REQUIRE(Nf >= 0 && NvOut >= 0, "f2v_bwd: negative size");
    PM_REQUIRE(grad_filter, "f2v_bwd: null grad_filter");
    PM_REQUIRE(NvOut <= INT32_MAX && Nf <= INT32_MAX / 3, "f2v_bwd: sizes exceed int32 indexing");
    hipStream_t st = (hipStream_t)stream;
    const int Co = C * r;
    if (Nf == 0) {
        fill_zero_k<<<dim3((unsigned)ceil_div((int64_t)K * Co, kBlock)), dim3(kBlock), 0, st>>>(grad_filter, (int64_t)K * Co);
        PM_LAUNCHED("f2v_bwd(fill)");
        return 0;
    }
    PM_REQUIRE(grad_output && input && filter && coeff && face && nf_count && vt_map && grad_input && workspace, "f2v_bwd: null pointer");
    const int V = pick_v(C, r, {grad_output, input, filter, grad_input, workspace});
    const RowShape rs = row_shape(C / V);
    const int G = persistent_blocks(Nf, rs.rpb);
    const int64_t rows_per_block = ceil_div(ceil_div(Nf, G), rs.rpb) * rs.rpb;
    PM_REQUIRE(workspace_bytes >= (size_t)G * K * Co * sizeof(float), "f2v_bwd: workspace too small (%zu bytes)", workspace_bytes);
    const int cvec = ((K & 3) == 0 && aligned16(coeff)) ? 1 : 0;
    float *partial = (float *)workspace;
    if (!force_valu() && (r == 1 || r == 2) && f2v_mfma_ok(Nf, C, r, K, coeff) && (NvOut + 1) * (int64_t)Co < (int64_t(1) << 30) && Nf < (int64_t(1) << 25)) {
        const int Gm = f2v_bwd_mfma_blocks(Nf);
        PM_REQUIRE(workspace_bytes >= (size_t)Gm * K * Co * sizeof(float), "f2v_bwd: workspace too small (%zu bytes)", workspace_bytes);
        if (int rc = f2v_bwd_mfma(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Gm, Nf, NvOut, C, r, st)) return rc;
        return reduce_partials(partial, grad_filter, Gm, K * Co, st);
    }
    if (f2v_fast_ok(C, r, K, {grad_output, input, filter, grad_input, workspace})) {
        const RowShape fs = row_shape(Co / 4);
        const int64_t frows = ceil_div(ceil_div(Nf, G), fs.rpb) * fs.rpb;
        if (r == 1)
            f2v_bwd_fast_k<1><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Nf, NvOut, C, K, fs.lpr_log2, frows);
        else
            f2v_bwd_fast_k<2><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Nf, NvOut, C, K, fs.lpr_log2, frows);
    } else if (V == 4)
        f2v_bwd_k<4><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Nf, NvOut, C, r, K, rs.items, rs.lpr_log2, cvec, rows_per_block);
    else
        f2v_bwd_k<1><<<dim3(G), dim3(kBlock), 0, st>>>(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Nf, NvOut, C, r, K, rs.items, rs.lpr_log2, cvec, rows_per_block);
    PM_LAUNCHED("f2v_bwd");
    return reduce_partials(partial, grad_filter, G, K * Co, st);
}

// ---- facet2vertex with the features in bf16 (the reduced-precision variant of the layer) ----------------------
// input, output, grad_output and grad_input rows are bf16; filter, coefficients and the filter gradient stay float.
// Only the shapes of the matrix-core kernels: 16 coefficients, at least 32 output channels, depth multiplier 1 or 2.
extern "C" int pmesh_f2v_fwd_bf16(const uint16_t *input, const float *filter, const float *coeff,
                                  const int32_t *nf_count, const int32_t *rowptr, const int32_t *colidx,
                                  uint16_t *output, int64_t Nf, int64_t NvOut, int C, int r, int K,
                                  pmesh_stream_t stream)
{
    clear_error();
    PM_DIMS("f2v_fwd_bf16");
    PM_REQUIRE(Nf >= 0 && NvOut >= 0, "f2v_fwd_bf16: negative size");
    if (NvOut == 0) return 0;
    PM_REQUIRE(input && filter && coeff && nf_count && rowptr && colidx && output, "f2v_fwd_bf16: null pointer");
    PM_REQUIRE(NvOut <= INT32_MAX && Nf <= INT32_MAX / 3, "f2v_fwd_bf16: sizes exceed int32 indexing");
    PM_REQUIRE(f2v_mfma_ok(Nf, C, r, K, coeff) && !(C & 1) && !((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(output)) & 3u),
               "f2v_fwd_bf16: bf16 features need 16 coefficients in 16-byte aligned rows, an even channel count and at least 32 output channels (K=%d C=%d r=%d)", K, C, r);
    return f2v_fwd_mfma(input, filter, coeff, nf_count, rowptr, colidx, output, Nf, NvOut, C, r, (hipStream_t)stream, true);
}

extern "C" int pmesh_f2v_bwd_bf16(const uint16_t *grad_output, const uint16_t *input, const float *filter,
                                  const float *coeff, const int32_t *face, const int32_t *nf_count,
                                  const int32_t *vt_map, uint16_t *grad_input, float *grad_filter, void *workspace,
                                  size_t workspace_bytes, int64_t Nf, int64_t NvIn, int64_t NvOut, int C, int r,
                                  int K, pmesh_stream_t stream)
{
    clear_error();
    (void)NvIn;
    PM_DIMS("f2v_bwd_bf16");
    PM_REQUIRE(Nf >= 0 && NvOut >= 0, "f2v_bwd_bf16: negative size");
    PM_REQUIRE(grad_filter, "f2v_bwd_bf16: null grad_filter");
    PM_REQUIRE(NvOut <= INT32_MAX && Nf <= INT32_MAX / 3, "f2v_bwd_bf16: sizes exceed int32 indexing");
    hipStream_t st = (hipStream_t)stream;
    const int Co = C * r;
    if (Nf == 0) {
        fill_zero_k<<<dim3((unsigned)ceil_div((int64_t)K * Co, kBlock)), dim3(kBlock), 0, st>>>(grad_filter, (int64_t)K * Co);
        PM_LAUNCHED("f2v_bwd_bf16(fill)");
        return 0;
    }
    PM_REQUIRE(grad_output && input && filter && coeff && face && nf_count && vt_map && grad_input && workspace, "f2v_bwd_bf16: null pointer");
    PM_REQUIRE((r == 1 || r == 2) && f2v_mfma_ok(Nf, C, r, K, coeff) && (NvOut + 1) * (int64_t)Co < (int64_t(1) << 30) && Nf < (int64_t(1) << 25) && !(C & 1) &&
                   !((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(grad_output) | reinterpret_cast<uintptr_t>(grad_input)) & 3u),
               "f2v_bwd_bf16: bf16 features need 16 coefficients in 16-byte aligned rows, an even channel count, at least 32 output channels and depth multiplier 1 or 2 (K=%d C=%d r=%d)", K, C, r);
    const int Gm = f2v_bwd_mfma_blocks(Nf);
    PM_REQUIRE(workspace_bytes >= (size_t)Gm * K * Co * sizeof(float), "f2v_bwd_bf16: workspace too small (%zu bytes)", workspace_bytes);
    float *partial = (float *)workspace;
    if (int rc = f2v_bwd_mfma(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, partial, Gm, Nf, NvOut, C, r, st, true)) return rc;
    return reduce_partials(partial, grad_filter, Gm, K * Co, st);
}

// ---- facet2vertex backward without a workspace argument -----------------------------------
// For callers that cannot allocate device memory (stream capture, serving loops, harnesses that forbid it): the
// partial filter gradients live in a file-scope device array instead of a caller's workspace.  Every GPU the library
// runs on holds its own copy of the array, at its own address, until the process ends; the address is looked up
// once per device and kept.  Calls on one GPU share the array: calls that overlap there race.
constexpr size_t kStaticScratchBytes = size_t(8) << 20;                   // K * C * r <= 2048 at 1024 partial slices
constexpr int kStaticScratchMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void *g_scratch_ptr[kStaticScratchMaxDevices];                     // device address of `scratch`, per device
static std::mutex g_scratch_lock;

// Device address of the current device's copy of `scratch` (the array's name itself is a host-side handle).
static int static_scratch(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail("f2v_bwd_static: hipGetDevice failed: %s", hipGetErrorString(e));
    PM_REQUIRE(dev >= 0 && dev < kStaticScratchMaxDevices, "f2v_bwd_static: device index %d not supported", dev);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail("f2v_bwd_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

extern "C" size_t pmesh_f2v_bwd_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int pmesh_f2v_bwd_static(const float *grad_output, const float *input, const float *filter,
                                    const float *coeff, const int32_t *face, const int32_t *nf_count,
                                    const int32_t *vt_map, float *grad_input, float *grad_filter, int64_t Nf,
                                    int64_t NvIn, int64_t NvOut, int C, int r, int K, pmesh_stream_t stream)
{
    clear_error();
    PM_DIMS("f2v_bwd_static");
    PM_REQUIRE(K > 0 && K <= 4096, "f2v_bwd_static: bad filter size K=%d", K);
    const size_t need = pmesh_f2v_bwd_workspace_bytes(C, r, K);
    PM_REQUIRE(need <= kStaticScratchBytes,
               "f2v_bwd_static: K*C*r = %lld needs %zu bytes of scratch, the static array holds %zu (K*C*r <= %zu); "
               "use pmesh_f2v_bwd with a workspace", (long long)K * C * r, need, kStaticScratchBytes,
               kStaticScratchBytes / (1024 * sizeof(float)));
    void *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    // every partial slice the reduction reads is written by the kernels of this call: nothing to clear
    return pmesh_f2v_bwd(grad_output, input, filter, coeff, face, nf_count, vt_map, grad_input, grad_filter, ws,
                         kStaticScratchBytes, Nf, NvIn, NvOut, C, r, K, stream);
}

// ---- pooling ---------------------------------------------------------------------------
#define PM_POOL_DIMS(name)                                                                      \
    PM_REQUIRE(C > 0 && C <= (1 << 20), name ": bad channel count C=%d", C);                   \
    PM_REQUIRE(NvIn >= 0 && NvOut >= 0 && NvIn <= INT32_MAX && NvOut <= INT32_MAX, name ": bad vertex counts")

extern "C" int pmesh_pool_max_fwd(const float *input, const int32_t *rowptr, const int32_t *members,
                                  float *output, int32_t *max_index, int64_t NvIn, int64_t NvOut, int C,
                                  pmesh_stream_t stream)
{
    clear_error();
    PM_POOL_DIMS("pool_max_fwd");
    if (NvOut == 0) return 0;
    PM_REQUIRE(input && rowptr && members && output && max_index, "pool_max_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int V = (pick_v(C, 1, {input, output, max_index}));
    const RowShape rs = row_shape(C / V);
    const int64_t blocks = ceil_div(NvOut, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "pool_max_fwd: grid too large");
    if (V == 4)
        pool_max_fwd_k<4><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, rowptr, members, output, max_index, NvOut, C, rs.items, rs.lpr_log2);
    else
        pool_max_fwd_k<1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, rowptr, members, output, max_index, NvOut, C, rs.items, rs.lpr_log2);
    PM_LAUNCHED("pool_max_fwd");
    return 0;
}

template <int MODE>
static int launch_fine_gather(const char *name, const float *coarse, const int32_t *maxidx,
                              const int32_t *vtrep, const int32_t *vtmap, float *fine, int64_t NvFine,
                              int64_t NvCoarse, int C, hipStream_t st)
{
    const int V = pick_v(C, 1, {coarse, fine, maxidx ? (const void *)maxidx : (const void *)coarse});
    const RowShape rs = row_shape(C / V);
    const int64_t blocks = ceil_div(NvFine, (int64_t)rs.rpb * kFineBatch);
    PM_REQUIRE(grid_ok(blocks), "%s: grid too large", name);
    if (V == 4)
        fine_gather_k<4, MODE><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(coarse, maxidx, vtrep, vtmap, fine, NvFine, NvCoarse, C, rs.items, rs.lpr_log2);
    else
        fine_gather_k<1, MODE><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(coarse, maxidx, vtrep, vtmap, fine, NvFine, NvCoarse, C, rs.items, rs.lpr_log2);
    PM_LAUNCHED(name);
    return 0;
}

extern "C" int pmesh_pool_max_bwd(const float *grad_output, const int32_t *max_index,
                                  const int32_t *vt_replace, const int32_t *vt_map, float *grad_input,
                                  int64_t NvIn, int64_t NvOut, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_POOL_DIMS("pool_max_bwd");
    if (NvIn == 0) return 0;
    PM_REQUIRE(grad_input, "pool_max_bwd: null pointer");
    PM_REQUIRE((vt_replace == nullptr) == (vt_map == nullptr), "pool_max_bwd: pass both cluster maps or neither");
    hipStream_t st = (hipStream_t)stream;
    if (vt_replace) {
        PM_REQUIRE(NvOut == 0 || (grad_output && max_index), "pool_max_bwd: null pointer");
        return launch_fine_gather<kMaxBwdGather>("pool_max_bwd", grad_output, max_index, vt_replace, vt_map,
                                                 grad_input, NvIn, NvOut, C, st);
    }
    const int64_t n_in = NvIn * C, n_out = NvOut * C;
    PM_REQUIRE(grid_ok(ceil_div(n_in, kBlock)), "pool_max_bwd: grid too large");
    fill_zero_k<<<dim3((unsigned)ceil_div(n_in, kBlock)), dim3(kBlock), 0, st>>>(grad_input, n_in);
    PM_LAUNCHED("pool_max_bwd(fill)");
    if (n_out == 0) return 0;
    PM_REQUIRE(grad_output && max_index, "pool_max_bwd: null pointer");
    pool_max_bwd_scatter_k<<<dim3((unsigned)ceil_div(n_out, kBlock)), dim3(kBlock), 0, st>>>(grad_output, max_index, grad_input, n_out, C, NvIn);
    PM_LAUNCHED("pool_max_bwd(scatter)");
    return 0;
}

template <bool AVG>
static int launch_cluster_sum(const char *name, const float *in, const int32_t *vtrep, const int32_t *rowptr,
                              const int32_t *members, float *out, int64_t NvFine, int64_t NvOut, int C,
                              hipStream_t st)
{
    const int V = pick_v(C, 1, {in, out});
    const RowShape rs = row_shape(C / V);
    const int64_t blocks = ceil_div(NvOut, rs.rpb);
    PM_REQUIRE(grid_ok(blocks), "%s: grid too large", name);
    if (V == 4)
        cluster_sum_k<4, AVG><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(in, vtrep, rowptr, members, out, NvFine, NvOut, C, rs.items, rs.lpr_log2);
    else
        cluster_sum_k<1, AVG><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(in, vtrep, rowptr, members, out, NvFine, NvOut, C, rs.items, rs.lpr_log2);
    PM_LAUNCHED(name);
    return 0;
}

extern "C" int pmesh_pool_avg_fwd(const float *input, const int32_t *vt_replace, const int32_t *rowptr,
                                  const int32_t *members, float *output, int64_t NvIn, int64_t NvOut, int C,
                                  pmesh_stream_t stream)
{
    clear_error();
    PM_POOL_DIMS("pool_avg_fwd");
    if (NvOut == 0) return 0;
    PM_REQUIRE(input && vt_replace && rowptr && members && output, "pool_avg_fwd: null pointer");
    return launch_cluster_sum<true>("pool_avg_fwd", input, vt_replace, rowptr, members, output, NvIn, NvOut, C, (hipStream_t)stream);
}

extern "C" int pmesh_pool_avg_bwd(const float *grad_output, const int32_t *vt_replace, const int32_t *vt_map,
                                  float *grad_input, int64_t NvIn, int64_t NvOut, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_POOL_DIMS("pool_avg_bwd");
    if (NvIn == 0) return 0;
    PM_REQUIRE(vt_replace && vt_map && grad_input && (NvOut == 0 || grad_output), "pool_avg_bwd: null pointer");
    return launch_fine_gather<kAvgBwd>("pool_avg_bwd", grad_output, nullptr, vt_replace, vt_map, grad_input, NvIn, NvOut, C, (hipStream_t)stream);
}

extern "C" int pmesh_unpool_fwd(const float *input, const int32_t *vt_replace, const int32_t *vt_map,
                                float *output, int64_t NvCoarse, int64_t NvFine, int C, pmesh_stream_t stream)
{
    clear_error();
    const int64_t NvIn = NvFine, NvOut = NvCoarse;
    PM_POOL_DIMS("unpool_fwd");
    if (NvFine == 0) return 0;
    PM_REQUIRE(vt_replace && vt_map && output && (NvCoarse == 0 || input), "unpool_fwd: null pointer");
    return launch_fine_gather<kUnpoolFwd>("unpool_fwd", input, nullptr, vt_replace, vt_map, output, NvFine, NvCoarse, C, (hipStream_t)stream);
}

extern "C" int pmesh_unpool_bwd(const float *grad_output, const int32_t *rowptr, const int32_t *members,
                                float *grad_input, int64_t NvCoarse, int64_t NvFine, int C, pmesh_stream_t stream)
{
    clear_error();
    const int64_t NvIn = NvFine, NvOut = NvCoarse;
    PM_POOL_DIMS("unpool_bwd");
    if (NvCoarse == 0) return 0;
    PM_REQUIRE(rowptr && members && grad_input && (NvFine == 0 || grad_output), "unpool_bwd: null pointer");
    return launch_cluster_sum<false>("unpool_bwd", grad_output, nullptr, rowptr, members, grad_input, NvFine, NvCoarse, C, (hipStream_t)stream);
}

extern "C" int pmesh_sph_harm(const float *xyz, float *out, int64_t N, int L, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(L >= 0 && L <= 5, "sph_harm: degree %d not supported (0..5)", L);
    PM_REQUIRE(N >= 0, "sph_harm: negative size");
    if (N == 0) return 0;
    PM_REQUIRE(xyz && out, "sph_harm: null pointer");
    PM_REQUIRE(grid_ok(ceil_div(N, kBlock)), "sph_harm: grid too large");
    const dim3 grid((unsigned)ceil_div(N, kBlock)), block(kBlock);
    hipStream_t st = (hipStream_t)stream;
    switch (L) {
    case 0: sph_harm_k<0><<<grid, block, 0, st>>>(xyz, out, N); break;
    case 1: sph_harm_k<1><<<grid, block, 0, st>>>(xyz, out, N); break;
    case 2: sph_harm_k<2><<<grid, block, 0, st>>>(xyz, out, N); break;
    case 3: sph_harm_k<3><<<grid, block, 0, st>>>(xyz, out, N); break;
    case 4: sph_harm_k<4><<<grid, block, 0, st>>>(xyz, out, N); break;
    default: sph_harm_k<5><<<grid, block, 0, st>>>(xyz, out, N); break;
    }
    PM_LAUNCHED("sph_harm");
    return 0;
}

extern "C" int pmesh_count_vertex_adjface(const int32_t *rowptr, int32_t *nf_count, int64_t NvOut, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(NvOut >= 0, "count_vertex_adjface: negative size");
    if (NvOut == 0) return 0;
    PM_REQUIRE(rowptr && nf_count, "count_vertex_adjface: null pointer");
    PM_REQUIRE(grid_ok(ceil_div(NvOut, kBlock)), "count_vertex_adjface: grid too large");
    row_length_k<<<dim3((unsigned)ceil_div(NvOut, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(rowptr, nf_count, NvOut);
    PM_LAUNCHED("count_vertex_adjface");
    return 0;
}

extern "C" int pmesh_triangle_geometry(const float *vertex, const int32_t *face, float *geometry, int64_t Nv,
                                       int64_t Nf, int vertex_stride, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nf >= 0 && vertex_stride >= 3, "triangle_geometry: bad sizes");
    if (Nf == 0) return 0;
    PM_REQUIRE(vertex && face && geometry, "triangle_geometry: null pointer");
    PM_REQUIRE(Nv * vertex_stride < (int64_t(1) << 40) && grid_ok(ceil_div(Nf, kBlock)), "triangle_geometry: sizes too large");
    triangle_geometry_k<<<dim3((unsigned)ceil_div(Nf, kBlock)), dim3(kBlock), 0, (hipStream_t)stream>>>(vertex, face, geometry, Nf, vertex_stride);
    PM_LAUNCHED("triangle_geometry");
    return 0;
}
