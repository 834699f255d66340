// Point-cloud branch, part 2: the (fuzzy) depthwise point convolution, point pooling and weighted unpooling
// (picasso/point/pi_modules/source/pcloud_conv3d_gpu.cu, pcloud_pool3d_gpu.cu, pcloud_unpool3d_gpu.cu).
//
// The reference runs one thread per (neighbour pair, channel) and adds into the output with float atomics.  Here
// every op is a segmented sum over a sorted adjacency of the pairs (pmesh_build_index_csr): by query for the forward
// ops, by database point for the input gradients, so each output row is written once, by one lane group, in a fixed
// order.  The filter gradient is summed per workgroup (one column per thread, pairs in ascending order; bins in
// registers up to 64 of them, in LDS beyond) and the workgroups' partial results are added in a fixed tree order.
// With at most 36 bins, depth multiplier 1 and at most 256 channels, forward and input gradient keep the filter in
// registers and read the pairs' coefficients from a dense per-pair table in LDS (instances for 16, 20, 32 and 36 bins:
// a kernel's cost follows the instance's bins, not the filter's).
//
//   w[p, co]        = sum_t coeff[p, t] * filter[bin[p, t], co]           (plain form: one bin, weight 1)
//   out[o, co]      = (1 / nn_count[o]) sum_{p = (o, i)} in[i, co / r] * w[p, co]
//   gin[i, c]       = sum_{p = (o, i)} (1 / nn_count[o]) sum_m gout[o, c r + m] * w[p, c r + m]
//   gfilt[f, co]    = sum_p sum_t [bin[p, t] = f] coeff[p, t] * gout[o, co] * in[i, co / r] / nn_count[o]
#include "common.h"
#include "rows_internal.h"
#include "../../include/picasso_mesh.h"

namespace pmesh {

struct PairGraph {
    const int *nn_index;      // (Nout, 2): query, database point
    const int *nn_count;      // (Mp) divisor per query
    const int *bin_index;     // (Nout, T)
    const float *bin_coeff;   // (Nout, T) or null
    int64_t Np, Mp, Nout;
    int T, F;
};

// weight of pair p for V output channels starting at co
template <int V> __device__ __forceinline__ Pack<V> pair_weight(const PairGraph &g, const float *__restrict__ filt, int64_t p, int CR, int co)
{
    Pack<V> w = zero_pack<V>();
    for (int t = 0; t < g.T; ++t) {
        const int b = g.bin_index[p * g.T + t];
        const float c = g.bin_coeff ? g.bin_coeff[p * g.T + t] : 1.f;
        if (b >= 0 && b < g.F) {
            const Pack<V> f = ldp<V>(filt + (int64_t)b * CR + co);
#pragma unroll
            for (int u = 0; u < V; ++u) w.v[u] = fmaf(c, f.v[u], w.v[u]);
        }
    }
    return w;
}

__device__ __forceinline__ float inv_count(const int *__restrict__ nn_count, int64_t o)
{
    const int c = nn_count[o];
    return c > 0 ? 1.0f / (float)c : 0.f;
}

// V = 4 needs depth multiplier 1 (output channel = input channel) and 16-byte aligned rows
template <int V>
__global__ __launch_bounds__(kBlock) void point_conv_fwd_k(const float *__restrict__ in, const float *__restrict__ filt, PairGraph g,
                                                           const int *__restrict__ rowptr, const int *__restrict__ order,
                                                           float *__restrict__ out, int C, int r, int items, int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= g.Mp) return;
    const int CR = C * r, e0 = rowptr[row], e1 = rowptr[row + 1];
    const float inv = inv_count(g.nn_count, row);
    for (int q = lane; q < items; q += lpr) {
        const int co = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int e = e0; e < e1; ++e) {
            const int64_t p = order[e];
            const int i = g.nn_index[p * 2 + 1];
            if (i < 0 || i >= g.Np) continue;
            const Pack<V> w = pair_weight<V>(g, filt, p, CR, co);
            Pack<V> x;
            if constexpr (V == 1) x.v[0] = in[(int64_t)i * C + co / r];
            else x = ldp<V>(in + (int64_t)i * C + co);
#pragma unroll
            for (int u = 0; u < V; ++u) acc.v[u] = fmaf(x.v[u], w.v[u], acc.v[u]);
        }
#pragma unroll
        for (int u = 0; u < V; ++u) acc.v[u] *= inv;
        stp<V>(out + row * CR + co, acc);
    }
}

// rows = database points; lanes own V input channels (V = 4: depth multiplier 1)
template <int V>
__global__ __launch_bounds__(kBlock) void point_conv_bwd_in_k(const float *__restrict__ gout, const float *__restrict__ filt, PairGraph g,
                                                              const int *__restrict__ rowptr, const int *__restrict__ order,
                                                              float *__restrict__ gin, int C, int r, int items, int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= g.Np) return;
    const int CR = C * r, e0 = rowptr[row], e1 = rowptr[row + 1];
    for (int q = lane; q < items; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int e = e0; e < e1; ++e) {
            const int64_t p = order[e];
            const int o = g.nn_index[p * 2];
            if (o < 0 || o >= g.Mp) continue;
            const float inv = inv_count(g.nn_count, o);
            if constexpr (V == 1) {
                float s = 0.f;
                for (int m = 0; m < r; ++m) {
                    const Pack<1> w = pair_weight<1>(g, filt, p, CR, c * r + m);
                    s = fmaf(gout[(int64_t)o * CR + c * r + m], w.v[0], s);
                }
                acc.v[0] = fmaf(s, inv, acc.v[0]);
            } else {
                const Pack<V> w = pair_weight<V>(g, filt, p, CR, c), go = ldp<V>(gout + (int64_t)o * CR + c);
#pragma unroll
                for (int u = 0; u < V; ++u) acc.v[u] = fmaf(go.v[u] * w.v[u], inv, acc.v[u]);
            }
        }
        stp<V>(gin + row * C + c, acc);
    }
}

// Adds the coefficients of pair p's T entries to its row of a dense table cm[bin] in LDS (entries in ascending order).
// The entries are fetched eight at a time before the first of them is added: one thread walks a pair, and a fetch per
// step of the walk would leave it waiting T times in a row.
__device__ __forceinline__ void pair_row_to_table(const PairGraph &g, int64_t p, float *row)
{
    const int T = g.T;
    const int *bi = g.bin_index + p * T;
    const float *bc = g.bin_coeff ? g.bin_coeff + p * T : nullptr;
    for (int t0 = 0; t0 < T; t0 += 8) {
        int b[8];
        float cf[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = t0 + u < T ? t0 + u : T - 1;          // (no branch around a fetch; the surplus is dropped below)
            b[u] = bi[t];
            cf[u] = bc ? bc[t] : 1.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (t0 + u < T && b[u] >= 0 && b[u] < g.F) row[b[u]] += cf[u];
    }
}

// Forward (MODE 0: rows = queries, the other end of a pair is a database row of `src` = in) and input gradient (MODE 1:
// rows = database points, the other end a query row of `src` = gout, weighted by 1 / nn_count of that query) for at most
// FB bins, depth multiplier 1 and rows of at most 256 channels in four-channel pieces: a lane keeps its four columns of
// the filter in registers, and the workgroup turns the pairs of its rows, 128 at a time, into a dense table
// cm[pair][bin] in LDS (one thread per pair), together with the pair's other end and weight.  The weight of a pair for
// a lane's channels is then FB x 4 FMAs on table rows that all lanes of a row read at the same address, instead of T
// dependent fetches of filter rows per pair and lane.
template <int FB, int MODE>
__global__ __launch_bounds__(kBlock) void point_conv_rows_dense_k(const float *__restrict__ src, const float *__restrict__ filt,
                                                                  PairGraph g, const int *__restrict__ rowptr,
                                                                  const int *__restrict__ order, float *__restrict__ out, int C,
                                                                  int lpr_log2)
{
    constexpr int NP = 128;
    __shared__ __attribute__((aligned(16))) float s_cm[NP][FB];
    __shared__ int s_other[NP];
    __shared__ float s_scale[NP];
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2, rpb = kBlock >> lpr_log2;
    const int64_t rows = MODE == 0 ? g.Mp : g.Np, nother = MODE == 0 ? g.Np : g.Mp;
    const int64_t row0 = (int64_t)blockIdx.x * rpb, row = row0 + slot;
    const int64_t rowl = row0 + rpb < rows ? row0 + rpb : rows;
    const int eb = rowptr[row0], ee = rowptr[rowl];                 // the workgroup's pairs, in row order
    const bool live = row < rows && 4 * lane < C;
    const int e0 = row < rows ? rowptr[row] : 0, e1 = row < rows ? rowptr[row + 1] : 0;
    const int c = 4 * lane;
    float fr[FB][4];
#pragma unroll
    for (int f = 0; f < FB; ++f) {
        const float4 v = (live && f < g.F) ? *reinterpret_cast<const float4 *>(filt + (int64_t)f * C + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        fr[f][0] = v.x; fr[f][1] = v.y; fr[f][2] = v.z; fr[f][3] = v.w;
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int cb = eb; cb < ee; cb += NP) {
        __syncthreads();                                          // the table's readers of the chunk before are done
        for (int e = threadIdx.x; e < NP * FB / 4; e += kBlock) reinterpret_cast<float4 *>(&s_cm[0][0])[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        __syncthreads();
        if (threadIdx.x < NP && cb + (int)threadIdx.x < ee) {
            const int64_t p = order[cb + threadIdx.x];
            const int o = g.nn_index[p * 2], i = g.nn_index[p * 2 + 1];
            const int other = MODE == 0 ? i : o;
            const bool ok = other >= 0 && other < nother;
            s_other[threadIdx.x] = ok ? other : -1;
            s_scale[threadIdx.x] = (MODE == 1 && ok) ? inv_count(g.nn_count, o) : 1.f;
            if (ok) pair_row_to_table(g, p, s_cm[threadIdx.x]);
        }
        __syncthreads();
        if (!live) continue;
        const int a = e0 > cb ? e0 : cb, b = e1 < cb + NP ? e1 : cb + NP;
        for (int e4 = a; e4 < b; e4 += 4) {
            // the rows of four pairs are asked for before the first weight is formed (the sums stay in pair order)
            float4 x[4];
            bool ok[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int other = e4 + k < b ? s_other[e4 + k - cb] : -1;
                ok[k] = other >= 0;
                x[k] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ok[k]) x[k] = *reinterpret_cast<const float4 *>(src + (int64_t)other * C + c);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (!ok[k]) continue;
                const int q = e4 + k - cb;
                float w[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int f4 = 0; f4 < FB; f4 += 4) {
                    const float4 m = *reinterpret_cast<const float4 *>(&s_cm[q][f4]);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        w[u] = fmaf(m.x, fr[f4][u], w[u]);
                        w[u] = fmaf(m.y, fr[f4 + 1][u], w[u]);
                        w[u] = fmaf(m.z, fr[f4 + 2][u], w[u]);
                        w[u] = fmaf(m.w, fr[f4 + 3][u], w[u]);
                    }
                }
                const float sc = s_scale[q];
                acc[0] = fmaf(x[k].x * w[0], sc, acc[0]);
                acc[1] = fmaf(x[k].y * w[1], sc, acc[1]);
                acc[2] = fmaf(x[k].z * w[2], sc, acc[2]);
                acc[3] = fmaf(x[k].w * w[3], sc, acc[3]);
            }
        }
    }
    if (live) {
        const float inv = MODE == 0 ? inv_count(g.nn_count, row) : 1.f;
        *reinterpret_cast<float4 *>(out + row * C + c) = make_float4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
    }
}

// Input gradient AND filter gradient from one walk over the pairs (at most FB <= 20 bins, depth multiplier 1, rows of at
// most 128 channels): gin[i][c] = sum over the pairs of point i of gout[o][c] * w(p)[c] / count[o] with
// w(p)[c] = sum_f cm[p][f] * filt[f][c], and gfilt[f][c] += cm[p][f] * (gout[o][c] * in[i][c] / count[o]).  A lane keeps
// two channels of the filter and of the filter gradient in registers, a wave the rows of 64 / lanes-per-row database
// points; it builds the dense table cm of its own pairs, 64 at a time, in its own piece of LDS and meets no other wave
// until the end.  Waves are persistent over the row groups (their number is a function of the problem only); at the
// end the lanes that hold the same channels add their accumulators in a fixed order: partial[workgroup][F][C].
template <int FB>
__global__ __launch_bounds__(kBlock, 3) void point_conv_bwd_fused_k(const float *__restrict__ gout, const float *__restrict__ in,
                                                                    const float *__restrict__ filt, PairGraph g,
                                                                    const int *__restrict__ rowptr, const int *__restrict__ order,
                                                                    float *__restrict__ gin, float *__restrict__ partial, int C,
                                                                    int lpr_log2)
{
    constexpr int NW = kBlock / 64;
    __shared__ __attribute__((aligned(16))) float s_cm[NW][64][FB];
    __shared__ int s_other[NW][64];
    __shared__ float s_scale[NW][64];
    static_assert(NW * 64 >= 128, "the table doubles as the buffer of the final sum (FB x 128 floats)");
    const int wave = threadIdx.x >> 6, wl = threadIdx.x & 63;
    const int lpr = 1 << lpr_log2, lane = wl & (lpr - 1), slot = wl >> lpr_log2, rpw = 64 >> lpr_log2;
    const int64_t rows = g.Np, nother = g.Mp;
    const bool chan = 2 * lane < C;
    const int c = 2 * lane;
    float fr[FB][2], ga[FB][2];
#pragma unroll
    for (int f = 0; f < FB; ++f) {
        const float2 v = (chan && f < g.F) ? *reinterpret_cast<const float2 *>(filt + (int64_t)f * C + c) : make_float2(0.f, 0.f);
        fr[f][0] = v.x; fr[f][1] = v.y;
        ga[f][0] = ga[f][1] = 0.f;
    }
    float(*cm)[FB] = s_cm[wave];
    int *other_of = s_other[wave];
    float *scale_of = s_scale[wave];
    const int64_t groups = (rows + rpw - 1) / rpw;
    for (int64_t wb = (int64_t)blockIdx.x * NW + wave; wb < groups; wb += (int64_t)gridDim.x * NW) {
        const int64_t row0 = wb * rpw, row = row0 + slot;
        const int64_t rowl = row0 + rpw < rows ? row0 + rpw : rows;
        const int eb = rowptr[row0], ee = rowptr[rowl];             // the wave's pairs, in row order
        const bool live = row < rows && chan;
        const int e0 = row < rows ? rowptr[row] : 0, e1 = row < rows ? rowptr[row + 1] : 0;
        const float2 xin = live ? *reinterpret_cast<const float2 *>(in + row * C + c) : make_float2(0.f, 0.f);
        float acc[2] = {0.f, 0.f};
        for (int cb = eb; cb < ee; cb += 64) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the table's readers of the chunk before are done
            __builtin_amdgcn_wave_barrier();
            {
                int o = -1;
                float sc = 1.f;
                int64_t p = 0;
                if (cb + wl < ee) {
                    p = order[cb + wl];
                    const int oo = g.nn_index[p * 2], i = g.nn_index[p * 2 + 1];
                    if (oo >= 0 && oo < nother && i >= 0 && i < rows) o = oo;
                }
                if (o >= 0) sc = inv_count(g.nn_count, o);
                other_of[wl] = o;
                scale_of[wl] = sc;
#pragma unroll
                for (int f4 = 0; f4 < FB; f4 += 4) *reinterpret_cast<float4 *>(&cm[wl][f4]) = make_float4(0.f, 0.f, 0.f, 0.f);
                if (o >= 0) pair_row_to_table(g, p, cm[wl]);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (!live) continue;
            const int a = e0 > cb ? e0 : cb, b = e1 < cb + 64 ? e1 : cb + 64;
            for (int e4 = a; e4 < b; e4 += 4) {
                float2 x[4];
                bool ok[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int other = e4 + k < b ? other_of[e4 + k - cb] : -1;
                    ok[k] = other >= 0;
                    x[k] = make_float2(0.f, 0.f);
                    if (ok[k]) x[k] = *reinterpret_cast<const float2 *>(gout + (int64_t)other * C + c);
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (!ok[k]) continue;
                    const int q = e4 + k - cb;
                    const float sc = scale_of[q];
                    const float du[2] = {x[k].x * xin.x * sc, x[k].y * xin.y * sc};
                    float w[2] = {0.f, 0.f};
#pragma unroll
                    for (int f4 = 0; f4 < FB; f4 += 4) {
                        const float4 m = *reinterpret_cast<const float4 *>(&cm[q][f4]);
#pragma unroll
                        for (int u = 0; u < 2; ++u) {
                            w[u] = fmaf(m.x, fr[f4][u], w[u]);
                            w[u] = fmaf(m.y, fr[f4 + 1][u], w[u]);
                            w[u] = fmaf(m.z, fr[f4 + 2][u], w[u]);
                            w[u] = fmaf(m.w, fr[f4 + 3][u], w[u]);
                            ga[f4][u] = fmaf(m.x, du[u], ga[f4][u]);
                            ga[f4 + 1][u] = fmaf(m.y, du[u], ga[f4 + 1][u]);
                            ga[f4 + 2][u] = fmaf(m.z, du[u], ga[f4 + 2][u]);
                            ga[f4 + 3][u] = fmaf(m.w, du[u], ga[f4 + 3][u]);
                        }
                    }
                    acc[0] = fmaf(x[k].x * w[0], sc, acc[0]);
                    acc[1] = fmaf(x[k].y * w[1], sc, acc[1]);
                }
            }
        }
        if (live) *reinterpret_cast<float2 *>(gin + row * C + c) = make_float2(acc[0], acc[1]);
    }
    // the row slots of a wave add up across its lanes, then the waves one after the other through LDS, wave 0 first
    for (int off = lpr; off < 64; off <<= 1) {
#pragma unroll
        for (int f = 0; f < FB; ++f) {
            ga[f][0] += __shfl_xor(ga[f][0], off, 64);
            ga[f][1] += __shfl_xor(ga[f][1], off, 64);
        }
    }
    float *red = &s_cm[0][0][0];                                  // FB x C floats
    for (int w = 0; w < NW; ++w) {
        __syncthreads();
        if (wave == w && wl < lpr && chan) {
#pragma unroll
            for (int f = 0; f < FB; ++f) {
                float2 *d = reinterpret_cast<float2 *>(red + f * C + c);
                *d = w ? make_float2(d->x + ga[f][0], d->y + ga[f][1]) : make_float2(ga[f][0], ga[f][1]);
            }
        }
    }
    __syncthreads();
    float *dst = partial + (int64_t)blockIdx.x * g.F * C;
    for (int e = threadIdx.x; e < g.F * C; e += kBlock) dst[e] = red[e];
}

// filter gradient: workgroup (x, y) sums pairs [x * per, (x + 1) * per) for columns y * cols .. into LDS, one column per
// thread, and leaves partial[x][F][CR]
__global__ void point_conv_bwd_filt_k(const float *__restrict__ gout, const float *__restrict__ in, PairGraph g,
                                      float *__restrict__ partial, int C, int r, int cols, int64_t per)
{
    extern __shared__ float s_acc[];          // [F][cols]
    const int CR = C * r, co = blockIdx.y * cols + threadIdx.x;
    for (int f = 0; f < g.F; ++f) s_acc[f * cols + threadIdx.x] = 0.f;
    const int64_t p0 = (int64_t)blockIdx.x * per, p1 = p0 + per < g.Nout ? p0 + per : g.Nout;
    if (co < CR) {
        for (int64_t p = p0; p < p1; ++p) {
            const int o = g.nn_index[p * 2], i = g.nn_index[p * 2 + 1];
            if (o < 0 || o >= g.Mp || i < 0 || i >= g.Np) continue;
            const float d = gout[(int64_t)o * CR + co] * in[(int64_t)i * C + co / r] * inv_count(g.nn_count, o);
            for (int t = 0; t < g.T; ++t) {
                const int b = g.bin_index[p * g.T + t];
                const float c = g.bin_coeff ? g.bin_coeff[p * g.T + t] : 1.f;
                if (b >= 0 && b < g.F) s_acc[b * cols + threadIdx.x] = fmaf(c, d, s_acc[b * cols + threadIdx.x]);
            }
        }
        float *dst = partial + (int64_t)blockIdx.x * g.F * CR;
        for (int f = 0; f < g.F; ++f) dst[(int64_t)f * CR + co] = s_acc[f * cols + threadIdx.x];
    }
}

// The same with at most FB bins, kept in registers: the workgroup turns 32 pairs at a time into a dense table
// cm[pair][bin] (the coefficients of a pair's T entries, summed per bin, by one thread per pair), then every thread
// multiplies its column's 32 products gout * in / count by the table rows, which all lanes read at the same address.
// Pairs in ascending order per workgroup, as above.
template <int FB>
__global__ __launch_bounds__(256) void point_conv_bwd_filt_dense_k(const float *__restrict__ gout, const float *__restrict__ in,
                                                                   PairGraph g, float *__restrict__ partial, int C, int r,
                                                                   int64_t per)
{
    constexpr int PB = 32;
    __shared__ __attribute__((aligned(16))) float s_cm[PB][FB];
    __shared__ int s_o[PB], s_i[PB];
    __shared__ float s_inv[PB];
    const int CR = C * r, co = blockIdx.y * blockDim.x + threadIdx.x;
    const bool mine = co < CR;
    float acc[FB];
#pragma unroll
    for (int f = 0; f < FB; ++f) acc[f] = 0.f;
    const int64_t p0 = (int64_t)blockIdx.x * per, p1 = p0 + per < g.Nout ? p0 + per : g.Nout;
    for (int64_t pb = p0; pb < p1; pb += PB) {
        __syncthreads();                                          // the table's readers of the block before are done
        for (int e = threadIdx.x; e < PB * FB; e += blockDim.x) (&s_cm[0][0])[e] = 0.f;
        __syncthreads();
        if (threadIdx.x < PB) {
            const int64_t p = pb + threadIdx.x;
            int o = -1, i = -1;
            if (p < p1) {
                o = g.nn_index[p * 2];
                i = g.nn_index[p * 2 + 1];
                if (o < 0 || o >= g.Mp || i < 0 || i >= g.Np) o = -1;
            }
            s_o[threadIdx.x] = o;
            s_i[threadIdx.x] = i;
            s_inv[threadIdx.x] = o >= 0 ? inv_count(g.nn_count, o) : 0.f;
            if (o >= 0) pair_row_to_table(g, p, s_cm[threadIdx.x]);
        }
        __syncthreads();
        if (!mine) continue;
#pragma unroll 1
        for (int q0 = 0; q0 < PB; q0 += 8) {
            float d[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {                         // eight pairs' operands in flight
                const int o = s_o[q0 + u], i = s_i[q0 + u];
                d[u] = o >= 0 ? gout[(int64_t)o * CR + co] * in[(int64_t)i * C + co / r] * s_inv[q0 + u] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int f4 = 0; f4 < FB; f4 += 4) {
                    const float4 c = *reinterpret_cast<const float4 *>(&s_cm[q0 + u][f4]);
                    acc[f4] = fmaf(c.x, d[u], acc[f4]);
                    acc[f4 + 1] = fmaf(c.y, d[u], acc[f4 + 1]);
                    acc[f4 + 2] = fmaf(c.z, d[u], acc[f4 + 2]);
                    acc[f4 + 3] = fmaf(c.w, d[u], acc[f4 + 3]);
                }
        }
    }
    if (mine) {
        float *dst = partial + (int64_t)blockIdx.x * g.F * CR;
#pragma unroll
        for (int f = 0; f < FB; ++f)
            if (f < g.F) dst[(int64_t)f * CR + co] = acc[f];
    }
}

// ------------------------------------------------------------------------------------------------ pooling
// MODE 0: max with arg-max (first pair among equals; -1 and 0 for a query without neighbours), 1: average
template <int V, int MODE>
__global__ __launch_bounds__(kBlock) void point_pool_fwd_k(const float *__restrict__ in, const int *__restrict__ nn_index,
                                                           const int *__restrict__ nn_count, const int *__restrict__ rowptr,
                                                           const int *__restrict__ order, float *__restrict__ out,
                                                           int *__restrict__ max_index, int64_t Np, int64_t Mp, int C, int items,
                                                           int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= Mp) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    const float inv = MODE == 1 ? inv_count(nn_count, row) : 0.f;
    for (int q = lane; q < items; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        int idx[V];
#pragma unroll
        for (int u = 0; u < V; ++u) idx[u] = -1;
        for (int e = e0; e < e1; ++e) {
            const int i = nn_index[(int64_t)order[e] * 2 + 1];
            if (i < 0 || i >= Np) continue;
            const Pack<V> x = ldp<V>(in + (int64_t)i * C + c);
#pragma unroll
            for (int u = 0; u < V; ++u) {
                if constexpr (MODE == 0) {
                    if (idx[u] < 0 || x.v[u] > acc.v[u]) { acc.v[u] = x.v[u]; idx[u] = i; }
                } else {
                    acc.v[u] += x.v[u];
                }
            }
        }
        if constexpr (MODE == 1) {
#pragma unroll
            for (int u = 0; u < V; ++u) acc.v[u] *= inv;
        }
        stp<V>(out + row * C + c, acc);
        if constexpr (MODE == 0) {
#pragma unroll
            for (int u = 0; u < V; ++u) max_index[row * C + c + u] = idx[u];
        }
    }
}

// rows = database points: the gradient of every query that took its maximum here (MODE 0) / of every query it is a
// neighbour of, divided by that query's count (MODE 1)
template <int V, int MODE>
__global__ __launch_bounds__(kBlock) void point_pool_bwd_k(const float *__restrict__ gout, const int *__restrict__ max_index,
                                                           const int *__restrict__ nn_index, const int *__restrict__ nn_count,
                                                           const int *__restrict__ rowptr, const int *__restrict__ order,
                                                           float *__restrict__ gin, int64_t Np, int64_t Mp, int C, int items,
                                                           int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= Np) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    for (int q = lane; q < items; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int e = e0; e < e1; ++e) {
            const int o = nn_index[(int64_t)order[e] * 2];
            if (o < 0 || o >= Mp) continue;
            const Pack<V> go = ldp<V>(gout + (int64_t)o * C + c);
            if constexpr (MODE == 0) {
#pragma unroll
                for (int u = 0; u < V; ++u) acc.v[u] += (max_index[(int64_t)o * C + c + u] == (int)row) ? go.v[u] : 0.f;
            } else {
                const float inv = inv_count(nn_count, o);
#pragma unroll
                for (int u = 0; u < V; ++u) acc.v[u] = fmaf(go.v[u], inv, acc.v[u]);
            }
        }
        stp<V>(gin + row * C + c, acc);
    }
}

// ------------------------------------------------------------------------------------------------ unpooling
template <int V>
__global__ __launch_bounds__(kBlock) void point_unpool_fwd_k(const float *__restrict__ in, const float *__restrict__ weight,
                                                             const int *__restrict__ nn_index, float *__restrict__ out, int64_t Nrows,
                                                             int64_t Nin, int C, int K, int items, int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= Nrows) return;
    for (int q = lane; q < items; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int k = 0; k < K; ++k) {
            const int i = nn_index[row * K + k];
            if (i < 0 || i >= Nin) continue;
            const float w = weight[row * K + k];
            const Pack<V> x = ldp<V>(in + (int64_t)i * C + c);
#pragma unroll
            for (int u = 0; u < V; ++u) acc.v[u] = fmaf(x.v[u], w, acc.v[u]);
        }
        stp<V>(out + row * C + c, acc);
    }
}

// rows = coarse points; entries e = o * K + k of the flattened index array that name the row
template <int V>
__global__ __launch_bounds__(kBlock) void point_unpool_bwd_k(const float *__restrict__ gout, const float *__restrict__ weight,
                                                             const int *__restrict__ rowptr, const int *__restrict__ order,
                                                             float *__restrict__ gin, int64_t Nin, int C, int K, int items,
                                                             int lpr_log2)
{
    const int lpr = 1 << lpr_log2, lane = threadIdx.x & (lpr - 1), slot = threadIdx.x >> lpr_log2;
    const int64_t row = (int64_t)blockIdx.x * (kBlock >> lpr_log2) + slot;
    if (row >= Nin) return;
    const int e0 = rowptr[row], e1 = rowptr[row + 1];
    for (int q = lane; q < items; q += lpr) {
        const int c = q * V;
        Pack<V> acc = zero_pack<V>();
        for (int e = e0; e < e1; ++e) {
            const int64_t ent = order[e];
            const float w = weight[ent];
            const Pack<V> go = ldp<V>(gout + (ent / K) * C + c);
#pragma unroll
            for (int u = 0; u < V; ++u) acc.v[u] = fmaf(go.v[u], w, acc.v[u]);
        }
        stp<V>(gin + row * C + c, acc);
    }
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// number of workgroups (pair ranges) of the filter gradient: a function of the problem only, capped so that the partial
// results stay below 64 MiB
static int filt_blocks(int64_t Nout, int F, int CR)
{
    int64_t G = ceil_div(Nout, 256);
    if (G < 1) G = 1;
    if (G > 4096) G = 4096;
    const int64_t per = (int64_t)F * CR * 4;
    while (G > 1 && G * per > (int64_t(64) << 20)) G /= 2;
    return (int)G;
}

}  // namespace pmesh

using namespace pmesh;

#define PM_POINT_DIMS(name)                                                                                          \
    PM_REQUIRE(Np >= 0 && Mp >= 0 && Nout >= 0 && Np <= INT32_MAX && Mp <= INT32_MAX && Nout < INT32_MAX, name ": bad sizes"); \
    PM_REQUIRE(C > 0 && C <= (1 << 20), name ": bad channel count C=%d", C)

#define PM_ROW_LAUNCH(kernel, rows, items_, ...)                                                                     \
    do {                                                                                                             \
        const RowShape rs = row_shape(items_);                                                                       \
        const int64_t blocks = ceil_div(rows, rs.rpb);                                                               \
        PM_REQUIRE(grid_ok(blocks), "grid too large");                                                               \
        kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(__VA_ARGS__, rs.items, rs.lpr_log2);                 \
    } while (0)

extern "C" int pmesh_point_conv_fwd(const float *input, const float *filter, const int32_t *nn_count, const int32_t *nn_index,
                                    const int32_t *bin_index, const float *bin_coeff, const int32_t *rowptr, const int32_t *order,
                                    float *output, int64_t Np, int64_t Mp, int64_t Nout, int F, int C, int r, int T,
                                    pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_conv_fwd");
    PM_REQUIRE(F > 0 && r > 0 && T > 0 && (int64_t)C * r <= (1 << 20), "point_conv_fwd: bad filter shape");
    if (Mp == 0) return 0;
    PM_REQUIRE(output && nn_count && rowptr && filter, "point_conv_fwd: null pointer");
    PM_REQUIRE(Nout == 0 || (input && nn_index && bin_index && order), "point_conv_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const PairGraph g = {nn_index, nn_count, bin_index, bin_coeff, Np, Mp, Nout, T, F};
    const int CR = C * r;
    if (r == 1 && C % 4 == 0 && C <= 256 && F <= 36 && aligned16(input) && aligned16(filter) && aligned16(output)) {
        const RowShape rs = row_shape(C / 4);
        const int64_t blocks = ceil_div(Mp, rs.rpb);
        PM_REQUIRE(grid_ok(blocks), "grid too large");
        if (F <= 16) point_conv_rows_dense_k<16, 0><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, g, rowptr, order, output, C, rs.lpr_log2);
        else if (F <= 20) point_conv_rows_dense_k<20, 0><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, g, rowptr, order, output, C, rs.lpr_log2);
        else if (F <= 32) point_conv_rows_dense_k<32, 0><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, g, rowptr, order, output, C, rs.lpr_log2);
        else point_conv_rows_dense_k<36, 0><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(input, filter, g, rowptr, order, output, C, rs.lpr_log2);
    } else if (r == 1 && C % 4 == 0 && aligned16(input) && aligned16(filter) && aligned16(output))
        PM_ROW_LAUNCH(point_conv_fwd_k<4>, Mp, CR / 4, input, filter, g, rowptr, order, output, C, r);
    else
        PM_ROW_LAUNCH(point_conv_fwd_k<1>, Mp, CR, input, filter, g, rowptr, order, output, C, r);
    PM_LAUNCHED("point_conv_fwd");
    return 0;
}

extern "C" size_t pmesh_point_conv_bwd_workspace_bytes(int64_t Nout, int F, int C, int r)
{
    if (Nout < 0 || F <= 0 || C <= 0 || r <= 0) return 0;
    return (size_t)filt_blocks(Nout, F, C * r) * F * C * r * sizeof(float);
}

extern "C" int pmesh_point_conv_bwd(const float *grad_output, const float *input, const float *filter, const int32_t *nn_count,
                                    const int32_t *nn_index, const int32_t *bin_index, const float *bin_coeff,
                                    const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, float *grad_filter,
                                    void *workspace, size_t workspace_bytes, int64_t Np, int64_t Mp, int64_t Nout, int F, int C,
                                    int r, int T, pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_conv_bwd");
    PM_REQUIRE(F > 0 && F <= 512 && r > 0 && T > 0 && (int64_t)C * r <= (1 << 20), "point_conv_bwd: bad filter shape (at most 512 bins)");
    PM_REQUIRE(grad_filter, "point_conv_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int CR = C * r;
    if (Nout == 0 || Mp == 0 || Np == 0) {
        if (grad_input && Np > 0)
            if (int rc = reduce_partials(nullptr, grad_input, 0, (int)(Np * C), st)) return rc;
        return reduce_partials(nullptr, grad_filter, 0, F * CR, st);
    }
    PM_REQUIRE(grad_output && input && filter && nn_count && nn_index && bin_index && workspace, "point_conv_bwd: null pointer");
    const PairGraph g = {nn_index, nn_count, bin_index, bin_coeff, Np, Mp, Nout, T, F};
    if (grad_input && r == 1 && C % 4 == 0 && C <= 128 && F <= 20 && aligned16(grad_output) && aligned16(filter) && aligned16(grad_input) &&
        aligned16(input) && !options().point_conv_two_passes) {
        // both gradients from one walk over the pairs in database-point order
        PM_REQUIRE(rowptr_in && order_in, "point_conv_bwd: the input gradient needs the pairs sorted by database point");
        const RowShape rs = row_shape(C / 2);                        // two channels per lane: at most 64 lanes per row
        const int64_t groups = ceil_div(Np, (int64_t)(64 >> rs.lpr_log2)), wgs = ceil_div(groups, (int64_t)(kBlock / 64));
        int G = filt_blocks(Nout, F, CR);                            // as many workgroups as the chip holds at once
        if (G > 768) G = 768;
        if (G > wgs) G = (int)(wgs > 0 ? wgs : 1);
        PM_REQUIRE(workspace_bytes >= (size_t)G * F * CR * sizeof(float), "point_conv_bwd: workspace too small (%zu bytes)", workspace_bytes);
        if (F <= 16) point_conv_bwd_fused_k<16><<<dim3((unsigned)G), dim3(kBlock), 0, st>>>(grad_output, input, filter, g, rowptr_in, order_in, grad_input, (float *)workspace, C, rs.lpr_log2);
        else point_conv_bwd_fused_k<20><<<dim3((unsigned)G), dim3(kBlock), 0, st>>>(grad_output, input, filter, g, rowptr_in, order_in, grad_input, (float *)workspace, C, rs.lpr_log2);
        PM_LAUNCHED("point_conv_bwd(fused)");
        return reduce_partials((const float *)workspace, grad_filter, G, F * CR, st);
    }
    if (grad_input) {
        PM_REQUIRE(rowptr_in && order_in, "point_conv_bwd: the input gradient needs the pairs sorted by database point");
        if (r == 1 && C % 4 == 0 && C <= 256 && F <= 36 && aligned16(grad_output) && aligned16(filter) && aligned16(grad_input)) {
            const RowShape rs = row_shape(C / 4);
            const int64_t blocks = ceil_div(Np, rs.rpb);
            PM_REQUIRE(grid_ok(blocks), "grid too large");
            if (F <= 16) point_conv_rows_dense_k<16, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_output, filter, g, rowptr_in, order_in, grad_input, C, rs.lpr_log2);
            else if (F <= 20) point_conv_rows_dense_k<20, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_output, filter, g, rowptr_in, order_in, grad_input, C, rs.lpr_log2);
            else if (F <= 32) point_conv_rows_dense_k<32, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_output, filter, g, rowptr_in, order_in, grad_input, C, rs.lpr_log2);
            else point_conv_rows_dense_k<36, 1><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(grad_output, filter, g, rowptr_in, order_in, grad_input, C, rs.lpr_log2);
        } else if (r == 1 && C % 4 == 0 && aligned16(grad_output) && aligned16(filter) && aligned16(grad_input))
            PM_ROW_LAUNCH(point_conv_bwd_in_k<4>, Np, C / 4, grad_output, filter, g, rowptr_in, order_in, grad_input, C, r);
        else
            PM_ROW_LAUNCH(point_conv_bwd_in_k<1>, Np, C, grad_output, filter, g, rowptr_in, order_in, grad_input, C, r);
        PM_LAUNCHED("point_conv_bwd(input)");
    }
    const int G = filt_blocks(Nout, F, CR);
    PM_REQUIRE(workspace_bytes >= (size_t)G * F * CR * sizeof(float), "point_conv_bwd: workspace too small (%zu bytes)", workspace_bytes);
    const int64_t per = ceil_div(Nout, G);
    if (F <= 64) {
        int threads = 256;
        while (threads > 64 && threads / 2 >= CR) threads /= 2;
        const dim3 grid((unsigned)G, (unsigned)ceil_div(CR, threads));
        if (F <= 20) point_conv_bwd_filt_dense_k<20><<<grid, dim3(threads), 0, st>>>(grad_output, input, g, (float *)workspace, C, r, per);
        else if (F <= 32) point_conv_bwd_filt_dense_k<32><<<grid, dim3(threads), 0, st>>>(grad_output, input, g, (float *)workspace, C, r, per);
        else if (F <= 36) point_conv_bwd_filt_dense_k<36><<<grid, dim3(threads), 0, st>>>(grad_output, input, g, (float *)workspace, C, r, per);
        else point_conv_bwd_filt_dense_k<64><<<grid, dim3(threads), 0, st>>>(grad_output, input, g, (float *)workspace, C, r, per);
        PM_LAUNCHED("point_conv_bwd(filter)");
        return reduce_partials((const float *)workspace, grad_filter, G, F * CR, st);
    }
    int cols = 256;
    while (cols > 32 && ((size_t)F * cols * 4 > 65536 || cols / 2 >= CR)) cols /= 2;
    PM_REQUIRE((size_t)F * cols * 4 <= 65536, "point_conv_bwd: too many bins");
    point_conv_bwd_filt_k<<<dim3((unsigned)G, (unsigned)ceil_div(CR, cols)), dim3(cols), (size_t)F * cols * 4, st>>>(
        grad_output, input, g, (float *)workspace, C, r, cols, per);
    PM_LAUNCHED("point_conv_bwd(filter)");
    return reduce_partials((const float *)workspace, grad_filter, G, F * CR, st);
}

extern "C" int pmesh_point_pool_max_fwd(const float *input, const int32_t *nn_index, const int32_t *rowptr, const int32_t *order,
                                        float *output, int32_t *max_index, int64_t Np, int64_t Mp, int64_t Nout, int C,
                                        pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_pool_max_fwd");
    if (Mp == 0) return 0;
    PM_REQUIRE(output && max_index && rowptr && (Nout == 0 || (input && nn_index && order)), "point_pool_max_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(input) && aligned16(output))
        PM_ROW_LAUNCH((point_pool_fwd_k<4, 0>), Mp, C / 4, input, nn_index, nullptr, rowptr, order, output, max_index, Np, Mp, C);
    else
        PM_ROW_LAUNCH((point_pool_fwd_k<1, 0>), Mp, C, input, nn_index, nullptr, rowptr, order, output, max_index, Np, Mp, C);
    PM_LAUNCHED("point_pool_max_fwd");
    return 0;
}

extern "C" int pmesh_point_pool_max_bwd(const float *grad_output, const int32_t *max_index, const int32_t *nn_index,
                                        const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, int64_t Np, int64_t Mp,
                                        int64_t Nout, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_pool_max_bwd");
    if (Np == 0) return 0;
    PM_REQUIRE(grad_input && rowptr_in && (Nout == 0 || (grad_output && max_index && nn_index && order_in)), "point_pool_max_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(grad_output) && aligned16(grad_input))
        PM_ROW_LAUNCH((point_pool_bwd_k<4, 0>), Np, C / 4, grad_output, max_index, nn_index, nullptr, rowptr_in, order_in, grad_input, Np, Mp, C);
    else
        PM_ROW_LAUNCH((point_pool_bwd_k<1, 0>), Np, C, grad_output, max_index, nn_index, nullptr, rowptr_in, order_in, grad_input, Np, Mp, C);
    PM_LAUNCHED("point_pool_max_bwd");
    return 0;
}

extern "C" int pmesh_point_pool_avg_fwd(const float *input, const int32_t *nn_count, const int32_t *nn_index, const int32_t *rowptr,
                                        const int32_t *order, float *output, int64_t Np, int64_t Mp, int64_t Nout, int C,
                                        pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_pool_avg_fwd");
    if (Mp == 0) return 0;
    PM_REQUIRE(output && nn_count && rowptr && (Nout == 0 || (input && nn_index && order)), "point_pool_avg_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(input) && aligned16(output))
        PM_ROW_LAUNCH((point_pool_fwd_k<4, 1>), Mp, C / 4, input, nn_index, nn_count, rowptr, order, output, nullptr, Np, Mp, C);
    else
        PM_ROW_LAUNCH((point_pool_fwd_k<1, 1>), Mp, C, input, nn_index, nn_count, rowptr, order, output, nullptr, Np, Mp, C);
    PM_LAUNCHED("point_pool_avg_fwd");
    return 0;
}

extern "C" int pmesh_point_pool_avg_bwd(const float *grad_output, const int32_t *nn_count, const int32_t *nn_index,
                                        const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, int64_t Np, int64_t Mp,
                                        int64_t Nout, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_POINT_DIMS("point_pool_avg_bwd");
    if (Np == 0) return 0;
    PM_REQUIRE(grad_input && rowptr_in && (Nout == 0 || (grad_output && nn_count && nn_index && order_in)), "point_pool_avg_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(grad_output) && aligned16(grad_input))
        PM_ROW_LAUNCH((point_pool_bwd_k<4, 1>), Np, C / 4, grad_output, nullptr, nn_index, nn_count, rowptr_in, order_in, grad_input, Np, Mp, C);
    else
        PM_ROW_LAUNCH((point_pool_bwd_k<1, 1>), Np, C, grad_output, nullptr, nn_index, nn_count, rowptr_in, order_in, grad_input, Np, Mp, C);
    PM_LAUNCHED("point_pool_avg_bwd");
    return 0;
}

extern "C" int pmesh_point_unpool_fwd(const float *input, const float *weight, const int32_t *nn_index, float *output, int64_t Nrows,
                                      int64_t Nin, int C, int K, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nrows >= 0 && Nin >= 0 && Nrows <= INT32_MAX && Nin <= INT32_MAX && C > 0 && C <= (1 << 20) && K > 0 && K <= 1024,
               "point_unpool_fwd: bad sizes");
    if (Nrows == 0) return 0;
    PM_REQUIRE(output && weight && nn_index && (Nin == 0 || input), "point_unpool_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(input) && aligned16(output))
        PM_ROW_LAUNCH(point_unpool_fwd_k<4>, Nrows, C / 4, input, weight, nn_index, output, Nrows, Nin, C, K);
    else
        PM_ROW_LAUNCH(point_unpool_fwd_k<1>, Nrows, C, input, weight, nn_index, output, Nrows, Nin, C, K);
    PM_LAUNCHED("point_unpool_fwd");
    return 0;
}

extern "C" int pmesh_point_unpool_bwd(const float *grad_output, const float *weight, const int32_t *rowptr_in, const int32_t *order_in,
                                      float *grad_input, int64_t Nrows, int64_t Nin, int C, int K, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nrows >= 0 && Nin >= 0 && Nrows <= INT32_MAX / (K > 0 ? K : 1) && Nin <= INT32_MAX && C > 0 && C <= (1 << 20) && K > 0 && K <= 1024,
               "point_unpool_bwd: bad sizes");
    if (Nin == 0) return 0;
    PM_REQUIRE(grad_input && rowptr_in && (Nrows == 0 || (grad_output && weight && order_in)), "point_unpool_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (C % 4 == 0 && aligned16(grad_output) && aligned16(grad_input))
        PM_ROW_LAUNCH(point_unpool_bwd_k<4>, Nin, C / 4, grad_output, weight, rowptr_in, order_in, grad_input, Nin, C, K);
    else
        PM_ROW_LAUNCH(point_unpool_bwd_k<1>, Nin, C, grad_output, weight, rowptr_in, order_in, grad_input, Nin, C, K);
    PM_LAUNCHED("point_unpool_bwd");
    return 0;
}
