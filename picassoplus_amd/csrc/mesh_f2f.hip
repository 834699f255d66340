// facet2facet convolution on the matrix cores (gfx950, v_mfma_f32_32x32x2_f32, fp32 accumulate).
//
// The reference evaluates, per facet f with texture points k in seg(f) (K_f of them),
//     out[f,co] = (1/K_f) sum_k sum_ci tex[k,ci] * sum_d sh[k,d] * W[co,ci,d]
// one thread per (f,co), recomputing the inner d-sum for every (k,ci,co).  Here the sum over
// texture points is taken first,
//     G[f,q] = (1/K_f) sum_k tex[k,ci] * sh[k,d],      q = ci*F + d   (W[co,q] is the filter
//                                                                        memory layout as is)
// which turns the three ops into dense contractions against a (Cout x Q) matrix, Q = Cin*F:
//     forward        out  = G    . W^T        (Nf x Q)(Q x Cout)
//     grad texture   H    = gout . W          (Nf x Cout)(Cout x Q), then
//                    gtex[k,ci] = (1/K_f) sum_d sh[k,d] * H[f,ci*F+d]
//     grad filter    gW   = gout^T . G        (Cout x Nf)(Nf x Q)
// G and H are never stored in HBM: tiles of them live in LDS, produced and consumed by the
// same workgroup.  The reduction index q is walked in chunks of whole input channels,
// CB = max(1, 64 / F) channels = QC = CB*F <= 64 columns (zero padded to 64), so that a chunk
// of H holds every d of its channels.
#include "common.h"
#include "f2f_internal.h"
#include "rows_internal.h"
#include "../../include/picasso_mesh.h"
#include <cstdlib>

namespace pmesh {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kTS = 68;  // LDS row stride in floats of the 64-wide tiles (16-byte aligned rows)

struct ChunkGeom {
    int F, CB, QC, n_chunks, tsteps;  // tsteps = ceil(QC / 8) groups of four MFMA k-steps
};

static inline ChunkGeom chunk_geom(int Cin, int F)
{
    ChunkGeom g;
    g.F = F;
    g.CB = 64 / F < 1 ? 1 : 64 / F;
    g.QC = g.CB * F;
    g.n_chunks = (Cin + g.CB - 1) / g.CB;
    g.tsteps = (g.QC + 7) / 8;
    return g;
}

// seg[i] = first texture row of facet f0+i (i in [0, n]); facets past Nf are empty.  Values are
// clamped to [0, T] so that a malformed running total can never address outside the texture rows.
__device__ __forceinline__ void load_segments(const int *__restrict__ cum, int64_t f0, int64_t Nf, int n,
                                              int T, int *seg)
{
    for (int i = threadIdx.x; i <= n; i += blockDim.x) {
        int64_t idx = f0 + i;
        if (idx > Nf) idx = Nf;
        int v = (idx == 0) ? 0 : cum[idx - 1];
        seg[i] = v < 0 ? 0 : (v > T ? T : v);
    }
}

// One wavefront fills rows [row0, row0+nrows) of a G tile for the channel chunk starting at c0.
// Lane ql owns column ql = cl*F + d of the chunk.  Loop trip counts are wave uniform.
__device__ __forceinline__ void build_g_rows(const float *__restrict__ tex, const float *__restrict__ sh,
                                             int Cin, int F, int ci, int d, bool valid, const int *seg,
                                             int row0, int nrows, float *Gs, int lane)
{
    for (int j = 0; j < nrows; ++j) {
        const int row = row0 + j;
        const int k0 = seg[row], k1 = seg[row + 1];
        float g = 0.f;
        if (valid) {
            int k = k0;
            for (; k + 1 < k1; k += 2) {
                const float t0 = tex[(int64_t)k * Cin + ci], s0 = sh[(int64_t)k * F + d];
                const float t1 = tex[(int64_t)(k + 1) * Cin + ci], s1 = sh[(int64_t)(k + 1) * F + d];
                g = fmaf(t0, s0, g);
                g = fmaf(t1, s1, g);
            }
            if (k < k1) g = fmaf(tex[(int64_t)k * Cin + ci], sh[(int64_t)k * F + d], g);
            g = (k1 > k0) ? g / (float)(k1 - k0) : 0.f;
        }
        Gs[row * kTS + lane] = g;
    }
}

// Ws[co][ql] = W[n0+co][c0*F + ql] for a 64 x 64 tile, zero outside the matrix / the chunk.
__device__ __forceinline__ void load_w_tile(const float *__restrict__ W, int Q, int Cout, int n0, int qbase,
                                            int qc_valid, float *Ws)
{
    const int ql = threadIdx.x & 63, r0 = threadIdx.x >> 6;
    const bool okq = ql < qc_valid && qbase + ql < Q;
#pragma unroll 4
    for (int co = r0; co < 64; co += 4)
        Ws[co * kTS + ql] = (okq && n0 + co < Cout) ? W[(int64_t)(n0 + co) * Q + qbase + ql] : 0.f;
}

// ----------------------------------------------------------------------------------------
// forward: 64 facets x 64 output channels per workgroup, 4 wavefronts, one 32x32 MFMA tile each
// ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void f2f_fwd_k(const float *__restrict__ tex, const float *__restrict__ W,
                                                 const float *__restrict__ sh, const int *__restrict__ cum,
                                                 float *__restrict__ out, int64_t Nf, int T, int Cin,
                                                 int Cout, ChunkGeom cg)
{
    __shared__ int seg[65];
    __shared__ __attribute__((aligned(16))) float Gs[64 * kTS];
    __shared__ __attribute__((aligned(16))) float Ws[64 * kTS];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int mt = w & 1, nt = w >> 1;
    const int64_t f0 = (int64_t)blockIdx.x * 64;
    const int n0 = blockIdx.y * 64;
    const int F = cg.F, Q = Cin * F;
    const int cl = lane / F, d = lane - cl * F;
    load_segments(cum, f0, Nf, 64, T, seg);
    __syncthreads();
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int j = 0; j < cg.n_chunks; ++j) {
        const int c0 = j * cg.CB;
        build_g_rows(tex, sh, Cin, F, c0 + cl, d, lane < cg.QC && c0 + cl < Cin, seg, w * 16, 16, Gs, lane);
        load_w_tile(W, Q, Cout, n0, c0 * F, cg.QC, Ws);
        __syncthreads();
        const float *ga = Gs + (mt * 32 + l32) * kTS + 4 * h;
        const float *wb = Ws + (nt * 32 + l32) * kTS + 4 * h;
        for (int t = 0; t < cg.tsteps; ++t) {
            const float4 a = *reinterpret_cast<const float4 *>(ga + 8 * t);
            const float4 b = *reinterpret_cast<const float4 *>(wb + 8 * t);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    const int co = n0 + nt * 32 + l32;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t f = f0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (f < Nf && co < Cout) out[f * Cout + co] = acc[i];
    }
}

// ----------------------------------------------------------------------------------------
// texture gradient: per workgroup 64 facets; for every channel chunk H = gout . W (64 x 64 tile
// in LDS), then gtex[k,ci] = (1/K_f) sum_d sh[k,d] * H[f, cl*F+d] for the facets' texture rows.
// ----------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void f2f_bwd_tex_k(const float *__restrict__ gout, const float *__restrict__ W,
                                                     const float *__restrict__ sh, const int *__restrict__ cum,
                                                     float *__restrict__ gtex, int64_t Nf, int T, int Cin,
                                                     int Cout, ChunkGeom cg, int sh_vec)
{
    __shared__ int seg[65];
    __shared__ __attribute__((aligned(16))) float gOs[64 * kTS];
    __shared__ __attribute__((aligned(16))) float Ws[64 * kTS];
    __shared__ __attribute__((aligned(16))) float Hs[64 * kTS];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int mt = w & 1, nt = w >> 1;
    const int64_t f0 = (int64_t)blockIdx.x * 64;
    const int F = cg.F, Q = Cin * F, CB = cg.CB;
    const int ncc = (Cout + 63) / 64;
    load_segments(cum, f0, Nf, 64, T, seg);
    for (int j = 0; j < cg.n_chunks; ++j) {
        const int c0 = j * CB;
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
        for (int cc = 0; cc < ncc; ++cc) {
            const int co0 = cc * 64;
            if (ncc > 1 || j == 0) {
                // gOs[fl][col] = gout[f0+fl][co0+col]
                for (int fl = w; fl < 64; fl += 4)
                    gOs[fl * kTS + lane] = (f0 + fl < Nf && co0 + lane < Cout) ? gout[(f0 + fl) * Cout + co0 + lane] : 0.f;
            }
            load_w_tile(W, Q, Cout, co0, c0 * F, cg.QC, Ws);
            __syncthreads();
            const float *ga = gOs + (mt * 32 + l32) * kTS + 4 * h;
            const float *wb = Ws + (4 * h) * kTS + nt * 32 + l32;
#pragma unroll 2
            for (int t = 0; t < 8; ++t) {
                const float4 a = *reinterpret_cast<const float4 *>(ga + 8 * t);
                const float *bp = wb + 8 * t * kTS;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bp[0], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bp[kTS], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, bp[2 * kTS], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, bp[3 * kTS], acc, 0, 0, 0);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
            Hs[(mt * 32 + 8 * (i / 4) + 4 * h + (i % 4)) * kTS + nt * 32 + l32] = acc[i];
        __syncthreads();
        // contraction with the SH values: this wavefront owns facets [w*16, w*16+16)
        const int kbeg = seg[w * 16], kend = seg[w * 16 + 16];
        const int nitems = (kend - kbeg) * CB;
        for (int it = lane; it < nitems; it += 64) {
            const int p = it / CB, cl = it - p * CB;
            const int k = kbeg + p, ci = c0 + cl;
            if (ci >= Cin) continue;
            int r = w * 16;
            while (r < w * 16 + 15 && seg[r + 1] <= k) ++r;
            const float *hp = Hs + r * kTS + cl * F;
            const float *sp = sh + (int64_t)k * F;
            float s = 0.f;
            if (sh_vec) {
                for (int d4 = 0; d4 < F; d4 += 4) {
                    const float4 sv = *reinterpret_cast<const float4 *>(sp + d4);
                    const float4 hv = *reinterpret_cast<const float4 *>(hp + d4);
                    s = fmaf(sv.x, hv.x, s); s = fmaf(sv.y, hv.y, s);
                    s = fmaf(sv.z, hv.z, s); s = fmaf(sv.w, hv.w, s);
                }
            } else {
                for (int dd = 0; dd < F; ++dd) s = fmaf(sp[dd], hp[dd], s);
            }
            gtex[(int64_t)k * Cin + ci] = s / (float)(seg[r + 1] - seg[r]);
        }
        __syncthreads();
    }
}

// ----------------------------------------------------------------------------------------
// filter gradient: split over facets.  A workgroup owns one 64-channel slab of Cout, up to 16
// channel chunks (one per wavefront, 64 x 64 accumulators = four MFMA tiles each) and a
// contiguous facet range; it stores its partial (Cout x Q) block for a fixed-order reduction.
// ----------------------------------------------------------------------------------------
constexpr int kFiltFB = 16;       // facets staged per iteration
constexpr int kFiltMaxWaves = 16;

__global__ __launch_bounds__(1024) void f2f_bwd_filt_k(const float *__restrict__ gout, const float *__restrict__ tex,
                                                       const float *__restrict__ sh, const int *__restrict__ cum,
                                                       float *__restrict__ partial, int64_t Nf, int T, int Cin,
                                                       int Cout, ChunkGeom cg, int64_t facets_per_split, int waves)
{
    __shared__ int seg[kFiltFB + 1];
    __shared__ float gOs[kFiltFB * kTS];
    __shared__ float Gs[kFiltMaxWaves * kFiltFB * kTS];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int F = cg.F, Q = Cin * F;
    const int chunk = blockIdx.y * waves + w;      // channel chunk of this wavefront
    const int n0 = blockIdx.z * 64;                // Cout slab
    const int c0 = chunk * cg.CB;
    const int cl = lane / F, d = lane - cl * F;
    const bool valid = chunk < cg.n_chunks && lane < cg.QC && c0 + cl < Cin;
    float *Gw = Gs + w * kFiltFB * kTS;
    f32x16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
    const int64_t fbeg = (int64_t)blockIdx.x * facets_per_split;
    const int64_t fend = (fbeg + facets_per_split < Nf) ? fbeg + facets_per_split : Nf;
    for (int64_t fb = fbeg; fb < fend; fb += kFiltFB) {
        load_segments(cum, fb, fend, kFiltFB, T, seg);
        for (int i = threadIdx.x; i < kFiltFB * 64; i += blockDim.x) {
            const int fl = i >> 6, col = i & 63;
            gOs[fl * kTS + col] = (fb + fl < fend && n0 + col < Cout) ? gout[(fb + fl) * Cout + n0 + col] : 0.f;
        }
        __syncthreads();
        build_g_rows(tex, sh, Cin, F, c0 + cl, d, valid, seg, 0, kFiltFB, Gw, lane);
        __syncthreads();
#pragma unroll 2
        for (int s = 0; s < kFiltFB / 2; ++s) {
            const float a0 = gOs[(2 * s + h) * kTS + l32], a1 = gOs[(2 * s + h) * kTS + 32 + l32];
            const float b0 = Gw[(2 * s + h) * kTS + l32], b1 = Gw[(2 * s + h) * kTS + 32 + l32];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[3], 0, 0, 0);
        }
        __syncthreads();
    }
    if (chunk >= cg.n_chunks) return;
    float *P = partial + (size_t)blockIdx.x * Cout * Q;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int ql = (t & 1) * 32 + l32;
        const int q = c0 * F + ql;
        if (ql >= cg.QC || q >= Q) continue;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int co = n0 + (t >> 1) * 32 + 8 * (i / 4) + 4 * h + (i % 4);
            if (co < Cout) P[(size_t)co * Q + q] = acc[t][i];
        }
    }
}

// out[o] = sum over splits, fixed order (same scheme as the row kernels' partial reduction)
__global__ __launch_bounds__(kBlock) void f2f_reduce_k(const float *__restrict__ partial, float *__restrict__ out,
                                                       int S, int64_t n)
{
    __shared__ float red[4][64];
    const int j = threadIdx.x & 63, s = threadIdx.x >> 6;
    const int64_t o = (int64_t)blockIdx.x * 64 + j;
    float sum = 0.f;
    if (o < n)
        for (int g = s; g < S; g += 4) sum += partial[(size_t)g * n + o];
    red[s][j] = sum;
    __syncthreads();
    if (s == 0 && o < n) out[o] = ((red[0][j] + red[1][j]) + red[2][j]) + red[3][j];
}

__global__ __launch_bounds__(kBlock) void f2f_fill_zero_k(float *__restrict__ p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

// rows of grad_texture past the last facet's segment belong to no facet: clear them
template <typename TIO>
__global__ __launch_bounds__(kBlock) void f2f_zero_tail_k(TIO *__restrict__ gtex, const int *__restrict__ cum,
                                                          int64_t Nf, int T, int Cin)
{
    int last = cum[Nf - 1];
    last = last < 0 ? 0 : (last > T ? T : last);
    const int64_t n = (int64_t)(T - last) * Cin;
    TIO *p = gtex + (int64_t)last * Cin;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) p[i] = TIO(0);
}

constexpr int kFiltMaxSplits = 256;

static inline int filt_splits(int64_t Nf)
{
    int64_t s = ceil_div(Nf, (int64_t)kFiltFB * 16);
    if (s < 1) s = 1;
    if (s > kFiltMaxSplits) s = kFiltMaxSplits;
    return (int)s;
}

static inline bool force_generic() { return options().f2f_generic; }

}  // namespace pmesh

using namespace pmesh;

#define PM_F2F_DIMS(name)                                                                         \
    PM_REQUIRE(Cin > 0 && Cout > 0 && F > 0, name ": bad dims Cin=%d Cout=%d F=%d", Cin, Cout, F); \
    PM_REQUIRE(F <= 50, name ": a maximum of 50 filters is supported (F=%d)", F);                 \
    PM_REQUIRE((int64_t)Cin * F <= (1 << 24) && Cout <= (1 << 20), name ": dims too large");     \
    PM_REQUIRE(T >= 0 && Nf >= 0 && T <= INT32_MAX && Nf <= INT32_MAX, name ": bad sizes")

static inline bool force_bf16x3() { return options().f2f_bf16x3; }
static inline bool want_half() { return options().f2f_half; }

extern "C" size_t pmesh_f2f_fwd_workspace_bytes(int Cin, int Cout, int F)
{
    return F == 16 ? f2f16x3_fwd_workspace_bytes(Cin, Cout) : 0;
}

// *fused (may be null) <- true when the kernel that ran applied `tail` itself
static int f2f_fwd_any(const float *texture, const float *filter, const float *bary_coeff,
                       const int32_t *cum_texture, const int32_t *facet_order, float *output,
                       void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                       int F, pmesh_stream_t stream, const F2FTail *tail, bool *fused)
{
    if (fused) *fused = false;
    PM_F2F_DIMS("f2f_fwd");
    if (Nf == 0) return 0;
    PM_REQUIRE(filter && cum_texture && output && (T == 0 || (texture && bary_coeff)), "f2f_fwd: null pointer");
    // the split-bf16 forward addresses texture elements with 32-bit offsets
    if (!force_generic() && !force_bf16x3() && f2f_fwd_narrow_usable(Cin, F, bary_coeff))
        return f2f_fwd_narrow(texture, filter, bary_coeff, cum_texture, output, T, Nf, Cin, Cout, (hipStream_t)stream);
    if (!force_generic() && !force_bf16x3() && f2f16x3_usable(filter, bary_coeff, F) &&
        T * Cin < (int64_t(1) << 31)) {
        const bool fuse = tail && (!tail->bits || Cout % 32 == 0);
        if (fused) *fused = fuse;
        return f2f16h2_fwd(texture, filter, bary_coeff, cum_texture, facet_order, output, workspace, workspace_bytes,
                           T, Nf, Cin, Cout, (hipStream_t)stream, want_half(), false, fuse ? tail : nullptr);
    }
    if (!force_generic() && f2f16x3_usable(filter, bary_coeff, F) &&
        T * Cin < (int64_t(1) << 31))
        return f2f16x3_fwd(texture, filter, bary_coeff, cum_texture, facet_order, output, workspace, workspace_bytes,
                           T, Nf, Cin, Cout, (hipStream_t)stream);
    const ChunkGeom cg = chunk_geom(Cin, F);
    const int64_t gx = ceil_div(Nf, 64), gy = ceil_div(Cout, 64);
    PM_REQUIRE(grid_ok(gx) && gy <= 65535, "f2f_fwd: grid too large");
    f2f_fwd_k<<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, (hipStream_t)stream>>>(
        texture, filter, bary_coeff, cum_texture, output, Nf, (int)T, Cin, Cout, cg);
    PM_LAUNCHED("f2f_fwd");
    return 0;
}

extern "C" int pmesh_f2f_fwd(const float *texture, const float *filter, const float *bary_coeff,
                             const int32_t *cum_texture, const int32_t *facet_order, float *output,
                             void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                             int F, pmesh_stream_t stream)
{
    clear_error();
    return f2f_fwd_any(texture, filter, bary_coeff, cum_texture, facet_order, output, workspace, workspace_bytes, T, Nf,
                       Cin, Cout, F, stream, nullptr, nullptr);
}

extern "C" int pmesh_f2f_fwd_act(const float *texture, const float *filter, const float *bary_coeff,
                                 const int32_t *cum_texture, const int32_t *facet_order, const float *bias,
                                 const float *scale, const float *shift, int relu, float *output, uint32_t *relu_bits,
                                 void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                                 int F, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(!relu_bits || (Cout % 32 == 0 && !(reinterpret_cast<uintptr_t>(output) & 15u)),
               "f2f_fwd_act: the bit mask needs a multiple of 32 output channels and 16-byte aligned rows");
    const F2FTail tail = {bias, scale, shift, relu_bits, relu ? 1 : 0};
    bool fused = false;
    if (int rc = f2f_fwd_any(texture, filter, bary_coeff, cum_texture, facet_order, output, workspace, workspace_bytes, T,
                             Nf, Cin, Cout, F, stream, &tail, &fused))
        return rc;
    if (fused || Nf == 0) return 0;
    // kernels without the epilogue: the tail as a pass of its own over the result, in place
    return pmesh_bias_act_fwd(output, bias, scale, shift, relu, output, relu_bits, Nf, Cout, stream);
}

// the two halves run one after the other on a stream and share the workspace: partial filter gradients (as many
// slices as this facet count makes), then 256 bytes for the overflow flag of the fp16 filter gradient
static size_t f2f_bwd_ws(int64_t slices, int Cin, int Cout, int F)
{
    const size_t filt = (size_t)slices * Cout * Cin * F * sizeof(float) + 256;
    const size_t tex = F == 16 ? f2f16x3_bwd_texture_workspace_bytes(Cin, Cout) : 0;
    return filt > tex ? filt : tex;
}

extern "C" size_t pmesh_f2f_bwd_workspace_bytes(int Cin, int Cout, int F)
{
    // (a narrow shape too large for the narrow kernel's 32-bit offsets takes the general kernels: room for either)
    return f2f_bwd_ws(f2f_narrow_usable(Cin, F) && kNarrowMaxBlocks > kFiltMaxSplits ? kNarrowMaxBlocks : kFiltMaxSplits, Cin, Cout, F);
}

extern "C" size_t pmesh_f2f_bwd_workspace_bytes_for(int64_t Nf, int Cin, int Cout, int F)
{
    if (Nf < 0) Nf = 0;
    const int general = filt_splits(Nf), narrow = f2f_narrow_usable(Cin, F) ? f2f_narrow_blocks(Nf) : 0;
    return f2f_bwd_ws(narrow > general ? narrow : general, Cin, Cout, F);
}

extern "C" int pmesh_f2f_bwd_texture(const float *grad_output, const float *filter, const float *bary_coeff,
                                     const int32_t *cum_texture, const int32_t *facet_order, float *grad_texture,
                                     void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                                     int Cout, int F, pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_DIMS("f2f_bwd_texture");
    if (Nf == 0 || T == 0) return 0;
    PM_REQUIRE(grad_output && filter && bary_coeff && cum_texture && grad_texture, "f2f_bwd_texture: null pointer");
    f2f_zero_tail_k<float><<<dim3(64), dim3(kBlock), 0, (hipStream_t)stream>>>(grad_texture, cum_texture, Nf, (int)T, Cin);
    PM_LAUNCHED("f2f_bwd_texture(tail)");
    if (!force_generic() && !force_bf16x3() && f2f16x3_usable(filter, bary_coeff, F) &&
        f2f16x3_bwd_texture_usable(grad_output, Cout))
        return f2f16h2_bwd_texture(grad_output, filter, bary_coeff, cum_texture, facet_order, grad_texture, workspace,
                                   workspace_bytes, T, Nf, Cin, Cout, (hipStream_t)stream, want_half());
    if (!force_generic() && f2f16x3_usable(filter, bary_coeff, F) &&
        f2f16x3_bwd_texture_usable(grad_output, Cout))
        return f2f16x3_bwd_texture(grad_output, filter, bary_coeff, cum_texture, facet_order, grad_texture, workspace,
                                   workspace_bytes, T, Nf, Cin, Cout, (hipStream_t)stream);
    const ChunkGeom cg = chunk_geom(Cin, F);
    const int64_t gx = ceil_div(Nf, 64);
    PM_REQUIRE(grid_ok(gx), "f2f_bwd_texture: grid too large");
    const int sh_vec = ((F & 3) == 0 && (reinterpret_cast<uintptr_t>(bary_coeff) & 15u) == 0) ? 1 : 0;
    f2f_bwd_tex_k<<<dim3((unsigned)gx), dim3(256), 0, (hipStream_t)stream>>>(
        grad_output, filter, bary_coeff, cum_texture, grad_texture, Nf, (int)T, Cin, Cout, cg, sh_vec);
    PM_LAUNCHED("f2f_bwd_texture");
    return 0;
}

extern "C" int pmesh_f2f_bwd_texture_onto_supported(const float *grad_output, const float *filter, const float *bary_coeff,
                                                   int Cout, int F)
{
    return (!force_generic() && !force_bf16x3() && f2f16x3_usable(filter, bary_coeff, F) &&
            f2f16x3_bwd_texture_usable(grad_output, Cout)) ? 1 : 0;
}

extern "C" int pmesh_f2f_bwd_texture_onto(const float *grad_output, const float *filter, const float *bary_coeff,
                                          const int32_t *cum_texture, const int32_t *facet_order, float *grad_texture,
                                          void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                                          int Cout, int F, pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_DIMS("f2f_bwd_texture_onto");
    if (Nf == 0 || T == 0) return 0;
    PM_REQUIRE(grad_output && filter && bary_coeff && cum_texture && grad_texture, "f2f_bwd_texture_onto: null pointer");
    PM_REQUIRE(pmesh_f2f_bwd_texture_onto_supported(grad_output, filter, bary_coeff, Cout, F),
               "f2f_bwd_texture_onto: takes 16 coefficients, a multiple of 8 output channels and 16-byte aligned arrays (F=%d Cout=%d)", F, Cout);
    return f2f16h2_bwd_texture(grad_output, filter, bary_coeff, cum_texture, facet_order, grad_texture, workspace,
                               workspace_bytes, T, Nf, Cin, Cout, (hipStream_t)stream, want_half(), false, true);
}

extern "C" int pmesh_f2f_bwd_filter(const float *grad_output, const float *texture, const float *bary_coeff,
                                    const int32_t *cum_texture, const int32_t *facet_order, float *grad_filter, void *workspace,
                                    size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, int F,
                                    pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_DIMS("f2f_bwd_filter");
    PM_REQUIRE(grad_filter, "f2f_bwd_filter: null grad_filter");
    hipStream_t st = (hipStream_t)stream;
    const int64_t nW = (int64_t)Cout * Cin * F;
    if (Nf == 0 || T == 0) {
        f2f_fill_zero_k<<<dim3((unsigned)ceil_div(nW, kBlock)), dim3(kBlock), 0, st>>>(grad_filter, nW);
        PM_LAUNCHED("f2f_bwd_filter(fill)");
        return 0;
    }
    PM_REQUIRE(grad_output && texture && bary_coeff && cum_texture && workspace, "f2f_bwd_filter: null pointer");
    if (!force_generic() && f2f_narrow_bwd_usable(Cin, F, Nf, Cout) && !(reinterpret_cast<uintptr_t>(bary_coeff) & 15u)) {
        const int nb = f2f_narrow_blocks(Nf);
        PM_REQUIRE(workspace_bytes >= (size_t)nb * nW * sizeof(float), "f2f_bwd_filter: workspace too small (%zu bytes)",
                   workspace_bytes);
        if (int rc = f2f_bwd_filter_narrow_partials(grad_output, texture, bary_coeff, cum_texture, (float *)workspace, nb, T,
                                                    Nf, Cin, Cout, st))
            return rc;
        return reduce_partials((const float *)workspace, grad_filter, nb, (int)nW, st);
    }
    const ChunkGeom cg = chunk_geom(Cin, F);
    const int S = filt_splits(Nf);
    PM_REQUIRE(workspace_bytes >= (size_t)S * nW * sizeof(float), "f2f_bwd_filter: workspace too small (%zu bytes)",
               workspace_bytes);
    const bool x3 = !force_generic() && f2f16x3_usable(bary_coeff, bary_coeff, F);
    if (x3) {
        PM_REQUIRE(workspace_bytes >= (size_t)S * nW * sizeof(float) + 256, "f2f_bwd_filter: workspace too small (%zu bytes)",
                   workspace_bytes);
        if (!force_bf16x3()) {
            // fp16 kernel first; if its scales did not hold, the guarded bf16 launch after it does the work again
            int *overflow = reinterpret_cast<int *>((float *)workspace + (size_t)S * nW);
            f2f_fill_zero_k<<<dim3(1), dim3(kBlock), 0, st>>>(reinterpret_cast<float *>(overflow), 1);
            PM_LAUNCHED("f2f_bwd_filter(flag)");
            if (int rc = f2f16h2_bwd_filter_partials(grad_output, texture, bary_coeff, cum_texture, facet_order,
                                                     (float *)workspace, overflow, S, T, Nf, Cin, Cout, st, want_half()))
                return rc;
            if (int rc = f2f16x3_bwd_filter_partials(grad_output, texture, bary_coeff, cum_texture, facet_order,
                                                     (float *)workspace, S, T, Nf, Cin, Cout, st, overflow))
                return rc;
        } else if (int rc = f2f16x3_bwd_filter_partials(grad_output, texture, bary_coeff, cum_texture, facet_order,
                                                        (float *)workspace, S, T, Nf, Cin, Cout, st)) {
            return rc;
        }
        f2f_reduce_k<<<dim3((unsigned)ceil_div(nW, 64)), dim3(kBlock), 0, st>>>((const float *)workspace, grad_filter, S, nW);
        PM_LAUNCHED("f2f_bwd_filter(reduce)");
        return 0;
    }
    const int waves = cg.n_chunks < kFiltMaxWaves ? cg.n_chunks : kFiltMaxWaves;
    const int64_t gy = ceil_div(cg.n_chunks, waves), gz = ceil_div(Cout, 64);
    PM_REQUIRE(gy <= 65535 && gz <= 65535, "f2f_bwd_filter: grid too large");
    const int64_t fps = ceil_div(ceil_div(Nf, S), kFiltFB) * kFiltFB;
    f2f_bwd_filt_k<<<dim3((unsigned)S, (unsigned)gy, (unsigned)gz), dim3(64 * waves), 0, st>>>(
        grad_output, texture, bary_coeff, cum_texture, (float *)workspace, Nf, (int)T, Cin, Cout, cg, fps, waves);
    PM_LAUNCHED("f2f_bwd_filter");
    f2f_reduce_k<<<dim3((unsigned)ceil_div(nW, 64)), dim3(kBlock), 0, st>>>((const float *)workspace, grad_filter, S, nW);
    PM_LAUNCHED("f2f_bwd_filter(reduce)");
    return 0;
}

extern "C" int pmesh_f2f_bwd(const float *grad_output, const float *texture, const float *filter,
                             const float *bary_coeff, const int32_t *cum_texture, const int32_t *facet_order,
                             float *grad_texture, float *grad_filter, void *workspace, size_t workspace_bytes,
                             int64_t T, int64_t Nf, int Cin, int Cout, int F, pmesh_stream_t stream)
{
    int rc = pmesh_f2f_bwd_texture(grad_output, filter, bary_coeff, cum_texture, facet_order, grad_texture, workspace,
                                   workspace_bytes, T, Nf, Cin, Cout, F, stream);
    if (rc) return rc;
    return pmesh_f2f_bwd_filter(grad_output, texture, bary_coeff, cum_texture, facet_order, grad_filter, workspace,
                                workspace_bytes, T, Nf, Cin, Cout, F, stream);
}

// ---- features in bf16 (the reduced-precision variant): 16 coefficients only, one fp16 product per element
#define PM_F2F_BF16(name)                                                                                          \
    PM_F2F_DIMS(name);                                                                                             \
    PM_REQUIRE(F == 16, name ": bf16 features are implemented for 16 coefficients (SH degree 3), got F=%d", F);    \
    PM_REQUIRE(!(Cin & 3) && !(Cout & 7), name ": bf16 features need Cin %% 4 == 0 and Cout %% 8 == 0 (Cin=%d Cout=%d)", Cin, Cout)

extern "C" size_t pmesh_f2f_bwd_bf16_workspace_bytes(int64_t T, int64_t Nf, int Cin, int Cout, int F)
{
    if (T < 0) T = 0;
    const size_t filt = pmesh_f2f_bwd_workspace_bytes_for(Nf, Cin, Cout, F);
    const size_t tex = f2f16h2_bwd_texture_bf16_workspace_bytes(T, Cin, Cout);
    return filt > tex ? filt : tex;
}

extern "C" int pmesh_f2f_fwd_bf16(const uint16_t *texture, const float *filter, const float *bary_coeff,
                                  const int32_t *cum_texture, const int32_t *facet_order, uint16_t *output,
                                  void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                                  int F, pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_BF16("f2f_fwd_bf16");
    if (Nf == 0) return 0;
    PM_REQUIRE(filter && cum_texture && output && (T == 0 || (texture && bary_coeff)), "f2f_fwd_bf16: null pointer");
    PM_REQUIRE(f2f16x3_usable(filter, bary_coeff, F), "f2f_fwd_bf16: filter and bary_coeff must be 16-byte aligned");
    return f2f16h2_fwd(texture, filter, bary_coeff, cum_texture, facet_order, output, workspace, workspace_bytes, T, Nf,
                       Cin, Cout, (hipStream_t)stream, true, true);
}

extern "C" int pmesh_f2f_bwd_texture_bf16(const uint16_t *grad_output, const float *filter, const float *bary_coeff,
                                          const int32_t *cum_texture, const int32_t *facet_order,
                                          uint16_t *grad_texture, void *workspace, size_t workspace_bytes, int64_t T,
                                          int64_t Nf, int Cin, int Cout, int F, pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_BF16("f2f_bwd_texture_bf16");
    if (Nf == 0 || T == 0) return 0;
    PM_REQUIRE(grad_output && filter && bary_coeff && cum_texture && grad_texture, "f2f_bwd_texture_bf16: null pointer");
    PM_REQUIRE(f2f16x3_usable(filter, bary_coeff, F), "f2f_bwd_texture_bf16: filter and bary_coeff must be 16-byte aligned");
    f2f_zero_tail_k<uint16_t><<<dim3(64), dim3(kBlock), 0, (hipStream_t)stream>>>(grad_texture, cum_texture, Nf, (int)T, Cin);
    PM_LAUNCHED("f2f_bwd_texture_bf16(tail)");
    return f2f16h2_bwd_texture(grad_output, filter, bary_coeff, cum_texture, facet_order, grad_texture, workspace,
                               workspace_bytes, T, Nf, Cin, Cout, (hipStream_t)stream, true, true);
}

extern "C" int pmesh_f2f_bwd_filter_bf16(const uint16_t *grad_output, const uint16_t *texture, const float *bary_coeff,
                                         const int32_t *cum_texture, const int32_t *facet_order, float *grad_filter,
                                         void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                                         int Cout, int F, pmesh_stream_t stream)
{
    clear_error();
    PM_F2F_BF16("f2f_bwd_filter_bf16");
    PM_REQUIRE(grad_filter, "f2f_bwd_filter_bf16: null grad_filter");
    hipStream_t st = (hipStream_t)stream;
    const int64_t nW = (int64_t)Cout * Cin * F;
    if (Nf == 0 || T == 0) {
        f2f_fill_zero_k<<<dim3((unsigned)ceil_div(nW, kBlock)), dim3(kBlock), 0, st>>>(grad_filter, nW);
        PM_LAUNCHED("f2f_bwd_filter_bf16(fill)");
        return 0;
    }
    PM_REQUIRE(grad_output && texture && bary_coeff && cum_texture && workspace, "f2f_bwd_filter_bf16: null pointer");
    PM_REQUIRE(!(reinterpret_cast<uintptr_t>(bary_coeff) & 15u), "f2f_bwd_filter_bf16: bary_coeff must be 16-byte aligned");
    const int S = filt_splits(Nf);
    PM_REQUIRE(workspace_bytes >= (size_t)S * nW * sizeof(float) + 256, "f2f_bwd_filter_bf16: workspace too small (%zu bytes)",
               workspace_bytes);
    // as in pmesh_f2f_bwd_filter: the fp16 kernel, then the guarded bf16-product launch if its scales did not hold
    int *overflow = reinterpret_cast<int *>((float *)workspace + (size_t)S * nW);
    f2f_fill_zero_k<<<dim3(1), dim3(kBlock), 0, st>>>(reinterpret_cast<float *>(overflow), 1);
    PM_LAUNCHED("f2f_bwd_filter_bf16(flag)");
    if (int rc = f2f16h2_bwd_filter_partials(grad_output, texture, bary_coeff, cum_texture, facet_order, (float *)workspace,
                                             overflow, S, T, Nf, Cin, Cout, st, true, true))
        return rc;
    if (int rc = f2f16x3_bwd_filter_partials(grad_output, texture, bary_coeff, cum_texture, facet_order, (float *)workspace,
                                             S, T, Nf, Cin, Cout, st, overflow, true))
        return rc;
    f2f_reduce_k<<<dim3((unsigned)ceil_div(nW, 64)), dim3(kBlock), 0, st>>>((const float *)workspace, grad_filter, S, nW);
    PM_LAUNCHED("f2f_bwd_filter_bf16(reduce)");
    return 0;
}
