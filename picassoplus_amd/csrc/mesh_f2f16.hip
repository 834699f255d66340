// facet2facet, fast path for 16 spherical-harmonic coefficients (degree 3) and Cin % 4 == 0.
//
// Same contraction as mesh_f2f.hip (out = G . W^T with G[f, ci*16+d] = mean_k tex[k,ci]*sh[k,d]),
// but the G operand never touches memory at all: each lane owns one facet (and one half of the 16
// d's), keeps the SH values of that facet's texture points in registers and forms the eight G
// values of an input channel with a handful of FMAs right before the MFMAs that consume them.
//   wavefront: 32 facets x 64 output channels (two 32x32 accumulator tiles)
//   workgroup: 4 wavefronts = 128 facets sharing the filter stream
//   filter:    W[:, 4 channels, :] (16 KiB) per step, double buffered in LDS, prefetched through
//              registers while the matrix cores work on the previous step
//   texture:   one 16-byte load per texture point per step, prefetched one step ahead
// MFMA k-step s of channel ci pairs lane-half h with d = 8h + s on both operands.
#include "f2f_internal.h"

namespace pmesh {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kKB = 9;      // texture points of a facet covered by one sweep over the channels
constexpr int kWRow = 20;   // LDS stride (floats) of one 16-float filter row: b128 reads conflict free
constexpr int kWBuf = 4 * 64 * kWRow;

__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }

__device__ __forceinline__ int wave_max(int v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int t = __shfl_xor(v, o, 64);
        v = t > v ? t : v;
    }
    return __builtin_amdgcn_readfirstlane(v);
}

// filter rows of channels [c0, c0+4) x output channels [n0, n0+64): 1024 float4, 4 per thread
__device__ __forceinline__ void w_fetch(const float *__restrict__ W, int Q, int Cout, int n0, int c0,
                                        float4 (&r)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = threadIdx.x + 256 * i;
        const int co = e >> 4, ci_l = (e >> 2) & 3, d4 = e & 3;
        r[i] = (n0 + co < Cout) ? ld4(W + (int64_t)(n0 + co) * Q + (c0 + ci_l) * 16 + d4 * 4)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

__device__ __forceinline__ void w_publish(float *Ws, const float4 (&r)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = threadIdx.x + 256 * i;
        const int co = e >> 4, ci_l = (e >> 2) & 3, d4 = e & 3;
        *reinterpret_cast<float4 *>(Ws + (ci_l * 64 + co) * kWRow + d4 * 4) = r[i];
    }
}

__global__ __launch_bounds__(256, 2) void f2f16_fwd_k(const float *__restrict__ tex, const float *__restrict__ W,
                                                      const float *__restrict__ sh, const int *__restrict__ cum,
                                                      float *__restrict__ out, int64_t Nf, int T, int Cin,
                                                      int Cout)
{
    __shared__ __attribute__((aligned(16))) float Ws[2 * kWBuf];
    __shared__ int s_kmax;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int64_t f0 = (int64_t)blockIdx.x * 128;
    const int n0 = blockIdx.y * 64;
    const int Q = Cin * 16, nblk = Cin >> 2;
    const int64_t f = f0 + w * 32 + l32;

    int k0 = 0, K = 0;
    if (f < Nf) {
        int a = f ? cum[f - 1] : 0, b = cum[f];
        a = a < 0 ? 0 : (a > T ? T : a);
        b = b < 0 ? 0 : (b > T ? T : b);
        k0 = a;
        K = b > a ? b - a : 0;
    }
    const float invK = K > 0 ? 1.0f / (float)K : 0.f;
    if (threadIdx.x == 0) s_kmax = 0;
    __syncthreads();
    atomicMax(&s_kmax, K);
    __syncthreads();
    const int nsweeps = (s_kmax + kKB - 1) / kKB;

    f32x16 acc0, acc1;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc0[i] = acc1[i] = 0.f;

    for (int sw = 0; sw < nsweeps; ++sw) {
        const int kbase = k0 + sw * kKB;
        int Ks = K - sw * kKB;
        Ks = Ks < 0 ? 0 : (Ks > kKB ? kKB : Ks);
        const int Kw = wave_max(Ks);

        float shr[kKB][8];
#pragma unroll
        for (int kk = 0; kk < kKB; ++kk) {
            float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
            if (kk < Ks) {
                const float *p = sh + (int64_t)(kbase + kk) * 16 + 8 * h;
                u = ld4(p);
                v = ld4(p + 4);
            }
            shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
            shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
        }

        float4 tc[kKB], tn[kKB], wn[4];
#pragma unroll
        for (int kk = 0; kk < kKB; ++kk)
            tc[kk] = (kk < Ks) ? ld4(tex + (int64_t)(kbase + kk) * Cin) : make_float4(0.f, 0.f, 0.f, 0.f);
        w_fetch(W, Q, Cout, n0, 0, wn);
        w_publish(Ws, wn);
        __syncthreads();

        for (int j = 0; j < nblk; ++j) {
            const float *Wc = Ws + (j & 1) * kWBuf;
            const bool more = j + 1 < nblk;
            if (more) {
                w_fetch(W, Q, Cout, n0, 4 * (j + 1), wn);
#pragma unroll
                for (int kk = 0; kk < kKB; ++kk)
                    tn[kk] = (kk < Ks) ? ld4(tex + (int64_t)(kbase + kk) * Cin + 4 * (j + 1))
                                       : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int ci_l = 0; ci_l < 4; ++ci_l) {
                float a[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) a[s] = 0.f;
#pragma unroll
                for (int kk = 0; kk < kKB; ++kk) {
                    if (kk < Kw) {
                        const float t = ci_l == 0 ? tc[kk].x : ci_l == 1 ? tc[kk].y : ci_l == 2 ? tc[kk].z : tc[kk].w;
#pragma unroll
                        for (int s = 0; s < 8; ++s) a[s] = fmaf(t, shr[kk][s], a[s]);
                    }
                }
                const float *b0p = Wc + (ci_l * 64 + l32) * kWRow + 8 * h;
                const float *b1p = b0p + 32 * kWRow;
                const float4 b00 = ld4(b0p), b01 = ld4(b0p + 4), b10 = ld4(b1p), b11 = ld4(b1p + 4);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b00.x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b10.x, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b00.y, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b10.y, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b00.z, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b10.z, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b00.w, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b10.w, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4], b01.x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[4], b11.x, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[5], b01.y, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[5], b11.y, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[6], b01.z, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[6], b11.z, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[7], b01.w, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[7], b11.w, acc1, 0, 0, 0);
            }
            if (more) {
                w_publish(Ws + ((j + 1) & 1) * kWBuf, wn);
#pragma unroll
                for (int kk = 0; kk < kKB; ++kk) tc[kk] = tn[kk];
            }
            __syncthreads();
        }
    }

    const int co0 = n0 + l32, co1 = co0 + 32;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t fr = f0 + w * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (fr < Nf) {
            if (co0 < Cout) out[fr * Cout + co0] = acc0[i];
            if (co1 < Cout) out[fr * Cout + co1] = acc1[i];
        }
    }
}


// ----------------------------------------------------------------------------------------
// texture gradient.  H = gout . W is produced transposed, D[row = (ci_l, d)][col = facet], 32 rows =
// two input channels per MFMA tile, so that a lane (facet, half h) ends up holding, for both
// channels, the eight d's {4h..4h+3, 8+4h..8+4h+3} of ITS facet in its accumulator registers.
// The contraction with the facet's SH values (kept in registers, like in the forward kernel) is
// then eight FMAs per texture point and channel plus one exchange between the two lane halves.
//   A operand: filter rows W[co][c0*16 + row] from LDS (transposed while staging), k = co
//   B operand: the facet's own gout row, 32 values per lane-half held in registers
// ----------------------------------------------------------------------------------------
constexpr int kTRow = 68;            // LDS stride of one (ci_l, d) row holding 64 output channels
constexpr int kTBuf = 64 * kTRow;    // four input channels per step

// stage W[co0 .. co0+64)[c0*16 .. c0*16+64) transposed: Wt[row][co]
__device__ __forceinline__ void wt_fetch(const float *__restrict__ W, int Q, int Cout, int co0, int c0,
                                         float4 (&r)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = threadIdx.x + 256 * i;
        const int co = e >> 4, r4 = e & 15;
        r[i] = (co0 + co < Cout) ? ld4(W + (int64_t)(co0 + co) * Q + c0 * 16 + r4 * 4)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

__device__ __forceinline__ void wt_publish(float *Wt, const float4 (&r)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = threadIdx.x + 256 * i;
        const int co = e >> 4, r4 = e & 15;
        float *p = Wt + (r4 * 4) * kTRow + co;
        p[0] = r[i].x; p[kTRow] = r[i].y; p[2 * kTRow] = r[i].z; p[3 * kTRow] = r[i].w;
    }
}

__device__ __forceinline__ void load_gout_half(const float *__restrict__ gout, int64_t f, int64_t Nf, int Cout,
                                               int co_lo, float (&g)[32])
{
    const bool vec = (Cout & 3) == 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int co = co_lo + 4 * i;
        if (f < Nf && vec && co + 3 < Cout) {
            const float4 t = ld4(gout + f * Cout + co);
            g[4 * i] = t.x; g[4 * i + 1] = t.y; g[4 * i + 2] = t.z; g[4 * i + 3] = t.w;
        } else {
#pragma unroll
            for (int u = 0; u < 4; ++u) g[4 * i + u] = (f < Nf && co + u < Cout) ? gout[f * Cout + co + u] : 0.f;
        }
    }
}

// one texture point: contract both accumulator tiles with the point's SH values; returns the
// four channel gradients (c0 .. c0+3) summed over both lane halves
__device__ __forceinline__ float4 contract_point(const f32x16 &a0, const f32x16 &a1, const float (&s)[8])
{
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        p0 = fmaf(s[i], a0[i], p0);
        p1 = fmaf(s[i], a0[8 + i], p1);
        p2 = fmaf(s[i], a1[i], p2);
        p3 = fmaf(s[i], a1[8 + i], p3);
    }
    p0 += __shfl_xor(p0, 32, 64);
    p1 += __shfl_xor(p1, 32, 64);
    p2 += __shfl_xor(p2, 32, 64);
    p3 += __shfl_xor(p3, 32, 64);
    return make_float4(p0, p1, p2, p3);
}

__global__ __launch_bounds__(256, 2) void f2f16_bwd_tex_k(const float *__restrict__ gout, const float *__restrict__ W,
                                                          const float *__restrict__ sh, const int *__restrict__ cum,
                                                          float *__restrict__ gtex, int64_t Nf, int T, int Cin,
                                                          int Cout)
{
    __shared__ __attribute__((aligned(16))) float Wt[2 * kTBuf];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int64_t f = (int64_t)blockIdx.x * 128 + w * 32 + l32;
    const int Q = Cin * 16, nblk = Cin >> 2, ncc = (Cout + 63) >> 6;

    int k0 = 0, K = 0;
    if (f < Nf) {
        int a = f ? cum[f - 1] : 0, b = cum[f];
        a = a < 0 ? 0 : (a > T ? T : a);
        b = b < 0 ? 0 : (b > T ? T : b);
        k0 = a;
        K = b > a ? b - a : 0;
    }
    const float invK = K > 0 ? 1.0f / (float)K : 0.f;
    const int Kw = wave_max(K < kKB ? K : kKB);      // points served from registers
    const int Kx = wave_max(K);                      // longest facet of the wavefront

    // SH values of my facet's points, my half's eight d's: {4h..4h+3, 8+4h..8+4h+3}, pre-scaled by 1/K
    float shr[kKB][8];
#pragma unroll
    for (int kk = 0; kk < kKB; ++kk) {
        float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
        if (kk < K) {
            const float *p = sh + (int64_t)(k0 + kk) * 16 + 4 * h;
            u = ld4(p);
            v = ld4(p + 8);
        }
        shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
        shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
    }

    float g[32];
    load_gout_half(gout, f, Nf, Cout, 32 * h, g);
    float4 wn[4];
    wt_fetch(W, Q, Cout, 0, 0, wn);
    wt_publish(Wt, wn);
    __syncthreads();

    const int nsteps = nblk * ncc;
    for (int j = 0; j < nblk; ++j) {
        f32x16 acc0, acc1;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc0[i] = acc1[i] = 0.f;
        for (int cc = 0; cc < ncc; ++cc) {
            const int it = j * ncc + cc;
            const float *Wc = Wt + (it & 1) * kTBuf;
            const bool more = it + 1 < nsteps;
            if (more) {
                const int jn = (cc + 1 < ncc) ? j : j + 1, ccn = (cc + 1 < ncc) ? cc + 1 : 0;
                wt_fetch(W, Q, Cout, 64 * ccn, 4 * jn, wn);
            }
            if (ncc > 1) load_gout_half(gout, f, Nf, Cout, 64 * cc + 32 * h, g);
            const float *a0p = Wc + l32 * kTRow + 32 * h;
            const float *a1p = a0p + 32 * kTRow;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float4 x = ld4(a0p + 4 * i), y = ld4(a1p + 4 * i);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, g[4 * i], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.x, g[4 * i], acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, g[4 * i + 1], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.y, g[4 * i + 1], acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, g[4 * i + 2], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.z, g[4 * i + 2], acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, g[4 * i + 3], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.w, g[4 * i + 3], acc1, 0, 0, 0);
            }
            if (more) wt_publish(Wt + ((it + 1) & 1) * kTBuf, wn);
            __syncthreads();
        }
        // acc0: channels 4j, 4j+1; acc1: channels 4j+2, 4j+3
        float *dst = gtex + (int64_t)k0 * Cin + 4 * j;
#pragma unroll
        for (int kk = 0; kk < kKB; ++kk) {
            if (kk < Kw) {
                const float4 p = contract_point(acc0, acc1, shr[kk]);
                if (kk < K && (kk & 1) == h) *reinterpret_cast<float4 *>(dst + (int64_t)kk * Cin) = p;
            }
        }
        for (int kk = kKB; kk < Kx; ++kk) {           // facets with more than kKB points: SH from memory
            float s8[8];
            float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
            if (kk < K) {
                const float *p = sh + (int64_t)(k0 + kk) * 16 + 4 * h;
                u = ld4(p);
                v = ld4(p + 8);
            }
            s8[0] = u.x * invK; s8[1] = u.y * invK; s8[2] = u.z * invK; s8[3] = u.w * invK;
            s8[4] = v.x * invK; s8[5] = v.y * invK; s8[6] = v.z * invK; s8[7] = v.w * invK;
            const float4 p = contract_point(acc0, acc1, s8);
            if (kk < K && (kk & 1) == h) *reinterpret_cast<float4 *>(dst + (int64_t)kk * Cin) = p;
        }
    }
}

// ----------------------------------------------------------------------------------------
// filter gradient gW = gout^T . G, split over facets.  A workgroup of 8 wavefronts owns a 64-channel
// slab of Cout and 64 input channels (8 per wavefront = four MFMA column tiles of two channels) and
// walks a contiguous facet range in slabs of up to 16 facets / kPS texture points.  A slab's
// texture, SH and gout rows are fetched with bulk 16-byte loads one slab ahead (held in registers
// while the previous slab is processed), published to LDS, and each lane-half forms the G values
// of its eight facets in registers -- they are the MFMA B operand as they stand.
// ----------------------------------------------------------------------------------------
constexpr int kFB = 16;        // facets per slab (one MFMA k-step pair per two facets)
constexpr int kPS = 160;       // texture points per slab
constexpr int kSRow = 68;      // LDS stride of a staged texture row (64 channels)

struct Slab {
    int fa, n, pa, pb, flush;
};

__device__ __forceinline__ int seg_start(const int *__restrict__ cum, int64_t f, int T)
{
    const int v = f ? cum[f - 1] : 0;
    return v < 0 ? 0 : (v > T ? T : v);
}

__device__ __forceinline__ int seg_end(const int *__restrict__ cum, int64_t f, int T)
{
    const int s = seg_start(cum, f, T);
    int e = cum[f];
    e = e < 0 ? 0 : (e > T ? T : e);
    return e > s ? e : s;
}

// next slab starting at facet fa; pa_cont >= 0 continues a facet that has more than kPS points.
// Evaluated by every wavefront on its own (lanes 0..16 fetch the 17 segment bounds in one go, so
// the descriptor costs one memory round trip instead of a chain of dependent loads).
__device__ __forceinline__ Slab make_slab(const int *__restrict__ cum, int64_t fa, int64_t fend, int T, int pa_cont,
                                          int lane)
{
    Slab S;
    S.fa = (int)fa; S.n = 0; S.pa = 0; S.pb = 0; S.flush = 1;
    if (fa >= fend) return S;
    const int64_t fi = fa + lane;                       // lane i: start row of facet fa + i
    int c = T;
    if (lane <= kFB && fi <= fend) c = seg_start(cum, fi, T);
    const int s0 = __builtin_amdgcn_readfirstlane(c);
    const int cn = __shfl_down(c, 1, 64);
    const int e = cn > c ? cn : c;                      // end row of facet fa + lane
    const int e0 = __builtin_amdgcn_readfirstlane(e);
    const bool ok = lane < kFB && fi < fend && e - s0 <= kPS;
    const unsigned long long mask = __ballot(ok);
    const int n = __builtin_ctzll(~mask);               // leading facets that fit together
    if (pa_cont >= 0 || n == 0) {
        S.n = 1;
        S.pa = pa_cont >= 0 ? pa_cont : s0;
        S.pb = (S.pa + kPS < e0) ? S.pa + kPS : e0;
        S.flush = S.pb >= e0;
        return S;
    }
    int pb = lane < n ? e : s0;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
        const int t = __shfl_xor(pb, o, 64);
        pb = t > pb ? t : pb;
    }
    S.n = n; S.pa = s0; S.pb = __builtin_amdgcn_readfirstlane(pb);
    return S;
}

__global__ __launch_bounds__(512, 2) void f2f16_bwd_filt_k(const float *__restrict__ gout, const float *__restrict__ tex,
                                                           const float *__restrict__ sh, const int *__restrict__ cum,
                                                           float *__restrict__ partial, int64_t Nf, int T, int Cin,
                                                           int Cout, int64_t facets_per_split)
{
    __shared__ __attribute__((aligned(16))) float tex_s[kPS * kSRow];
    __shared__ __attribute__((aligned(16))) float sh_s[kPS * 16];
    __shared__ __attribute__((aligned(16))) float go_s[kFB * 64];
    __shared__ int seg_s[2 * kFB];                   // start row and point count of the slab's facets
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int cbase = blockIdx.y * 64, n0 = blockIdx.z * 64;
    const int Q = Cin * 16;
    const int sel = l32 >> 4, d = l32 & 15;
    const int64_t fbeg = (int64_t)blockIdx.x * facets_per_split;
    const int64_t fend = (fbeg + facets_per_split < Nf) ? fbeg + facets_per_split : Nf;

    f32x16 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
    float g[8][4];
#pragma unroll
    for (int jj = 0; jj < 8; ++jj)
#pragma unroll
        for (int t = 0; t < 4; ++t) g[jj][t] = 0.f;

    float4 rt[5], rs[2], rg;
    int rseg0 = 0, rseg1 = 0;
    auto fetch = [&](const Slab &S) {
        const int np = S.pb - S.pa;
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const int e = threadIdx.x + 512 * i, p = e >> 4, c4 = e & 15;
            rt[i] = (p < np && cbase + 4 * c4 < Cin) ? ld4(tex + (int64_t)(S.pa + p) * Cin + cbase + 4 * c4)
                                                    : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int e = threadIdx.x + 512 * i, p = e >> 2, d4 = e & 3;
            rs[i] = (p < np) ? ld4(sh + (int64_t)(S.pa + p) * 16 + 4 * d4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        rg = make_float4(0.f, 0.f, 0.f, 0.f);
        if (threadIdx.x < 256) {
            const int fl = threadIdx.x >> 4, c4 = threadIdx.x & 15;
            if (fl < S.n) {
                const float *gp = gout + (int64_t)(S.fa + fl) * Cout + n0 + 4 * c4;
                if ((Cout & 3) == 0 && n0 + 4 * c4 + 3 < Cout) rg = ld4(gp);
                else {
                    rg.x = (n0 + 4 * c4 < Cout) ? gp[0] : 0.f;
                    rg.y = (n0 + 4 * c4 + 1 < Cout) ? gp[1] : 0.f;
                    rg.z = (n0 + 4 * c4 + 2 < Cout) ? gp[2] : 0.f;
                    rg.w = (n0 + 4 * c4 + 3 < Cout) ? gp[3] : 0.f;
                }
            }
        }
        if (threadIdx.x < kFB) {
            const bool on = threadIdx.x < S.n;
            rseg0 = on ? seg_start(cum, S.fa + threadIdx.x, T) : 0;
            rseg1 = on ? seg_end(cum, S.fa + threadIdx.x, T) - rseg0 : 0;
        }
    };
    auto publish = [&]() {
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const int e = threadIdx.x + 512 * i, p = e >> 4, c4 = e & 15;
            if (p < kPS) *reinterpret_cast<float4 *>(tex_s + p * kSRow + 4 * c4) = rt[i];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int e = threadIdx.x + 512 * i;
            if (e < kPS * 4) *reinterpret_cast<float4 *>(sh_s + 4 * e) = rs[i];
        }
        if (threadIdx.x < 256) *reinterpret_cast<float4 *>(go_s + 4 * threadIdx.x) = rg;
        if (threadIdx.x < kFB) {
            seg_s[threadIdx.x] = rseg0;
            seg_s[kFB + threadIdx.x] = rseg1;
        }
    };

    Slab cur = make_slab(cum, fbeg, fend, T, -1, lane);
    if (cur.n > 0) fetch(cur);
    publish();
    __syncthreads();
    while (cur.n > 0) {
        const Slab nxt = cur.flush ? make_slab(cum, cur.fa + cur.n, fend, T, -1, lane)
                                   : make_slab(cum, cur.fa, fend, T, cur.pb, lane);
        if (nxt.n > 0) fetch(nxt);

        // G values of my half's facets (slab facet 2*jj + h), channels 8w + 2t + sel, SH index d
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
            const int fl = 2 * jj + h;
            if (fl < cur.n) {
                const int s = seg_s[fl], Kf = seg_s[kFB + fl];
                const float inv = Kf > 0 ? 1.0f / (float)Kf : 0.f;
                int r0 = s > cur.pa ? s : cur.pa, r1 = s + Kf < cur.pb ? s + Kf : cur.pb;
                for (int r = r0; r < r1; ++r) {
                    const int p = r - cur.pa;
                    const float4 v0 = ld4(tex_s + p * kSRow + 8 * w), v1 = ld4(tex_s + p * kSRow + 8 * w + 4);
                    const float sv = sh_s[p * 16 + d] * inv;
                    g[jj][0] = fmaf(sel ? v0.y : v0.x, sv, g[jj][0]);
                    g[jj][1] = fmaf(sel ? v0.w : v0.z, sv, g[jj][1]);
                    g[jj][2] = fmaf(sel ? v1.y : v1.x, sv, g[jj][2]);
                    g[jj][3] = fmaf(sel ? v1.w : v1.z, sv, g[jj][3]);
                }
            }
        }
        if (cur.flush) {
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const float a0 = go_s[(2 * s + h) * 64 + l32], a1 = go_s[(2 * s + h) * 64 + 32 + l32];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, g[s][t], acc[t], 0, 0, 0);
                    acc[4 + t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, g[s][t], acc[4 + t], 0, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) g[s][t] = 0.f;
            }
        }
        __syncthreads();
        publish();
        __syncthreads();
        cur = nxt;
    }

    float *P = partial + (size_t)blockIdx.x * Cout * Q;
    const int cw = cbase + 8 * w;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (cw + 2 * t >= Cin) continue;
        const int q = (cw + 2 * t) * 16 + l32;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int co = n0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
                if (co < Cout) P[(size_t)co * Q + q] = acc[mt * 4 + t][i];
            }
    }
}

bool f2f16_usable(const void *tex, const void *W, const void *sh, int Cin, int F)
{
    auto al = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    return F == 16 && (Cin & 3) == 0 && al(tex) && al(W) && al(sh);
}

int f2f16_fwd(const float *tex, const float *W, const float *sh, const int *cum, float *out, int64_t T,
              int64_t Nf, int Cin, int Cout, hipStream_t st)
{
    const int64_t gx = ceil_div(Nf, 128), gy = ceil_div(Cout, 64);
    PM_REQUIRE(grid_ok(gx) && gy <= 65535, "f2f_fwd: grid too large");
    f2f16_fwd_k<<<dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st>>>(tex, W, sh, cum, out, Nf, (int)T, Cin, Cout);
    PM_LAUNCHED("f2f_fwd");
    return 0;
}

int f2f16_bwd_texture(const float *gout, const float *W, const float *sh, const int *cum, float *gtex, int64_t T,
                      int64_t Nf, int Cin, int Cout, hipStream_t st)
{
    const int64_t gx = ceil_div(Nf, 128);
    PM_REQUIRE(grid_ok(gx), "f2f_bwd_texture: grid too large");
    f2f16_bwd_tex_k<<<dim3((unsigned)gx), dim3(256), 0, st>>>(gout, W, sh, cum, gtex, Nf, (int)T, Cin, Cout);
    PM_LAUNCHED("f2f_bwd_texture");
    return 0;
}

int f2f16_bwd_filter_partials(const float *gout, const float *tex, const float *sh, const int *cum, float *partial,
                              int splits, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st)
{
    const int64_t gy = ceil_div(Cin, 64), gz = ceil_div(Cout, 64);
    PM_REQUIRE(gy <= 65535 && gz <= 65535, "f2f_bwd_filter: grid too large");
    const int64_t fps = ceil_div(Nf, splits);
    f2f16_bwd_filt_k<<<dim3((unsigned)splits, (unsigned)gy, (unsigned)gz), dim3(512), 0, st>>>(
        gout, tex, sh, cum, partial, Nf, (int)T, Cin, Cout, fps);
    PM_LAUNCHED("f2f_bwd_filter");
    return 0;
}

}  // namespace pmesh
