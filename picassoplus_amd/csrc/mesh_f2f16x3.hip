// facet2facet for 16 SH coefficients (forward, texture gradient, filter gradient) on the bf16 matrix
// cores with fp32-level accuracy.
//
// v_mfma_f32_32x32x16_bf16 sustains ~14x the rate of v_mfma_f32_32x32x2_f32 on gfx950.  Both
// operands of out = G . W^T are therefore split exactly into three bf16 pieces each,
//     x = x1 + x2 + x3,  x1 = top 8 mantissa bits of x, x2 = top 8 bits of (x - x1), x3 = the rest
// (truncation, so every piece is exactly representable and the sum is exact), and the product is
// accumulated in fp32 from the six piece products of order <= 2^-16:
//     G.W ~ G1W1 + G1W2 + G2W1 + G1W3 + G2W2 + G3W1          (dropped terms are < 2^-23 relative)
// Six bf16 MFMAs replace eight fp32 MFMAs per 16 reduction steps at 1/14 of the cost each.
//
// Work decomposition of the forward (two wavefronts per SIMD, 256 registers per lane):
//   workgroup  256 facets (taken from a list sorted by number of texture points) x 64 output channels
//   wavefront  32 facets x 64 output channels = two 32x32 accumulator tiles
//   lane       (l32, h): facet slot l32 of the wavefront, SH indices d = 8h..8h+7
//   filter     pre-split and pre-arranged per lane by f2f16x3_pack_filter_k; the 24 KiB of four
//              input channels are copied to LDS two chunks ahead (three buffers)
//   G operand  formed in registers: for the next input channel, 8 values per facet from the
//              facet's texture points (SH values held in registers), then split and packed,
//              interleaved with the current channel's 12 MFMAs
#include "f2f_internal.h"

namespace pmesh {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kXKB = 4;                       // texture points per facet covered by one sweep (register budget)
constexpr int kXChunk = 4 * 2 * 3 * 64;       // uint4 per LDS buffer: 4 channels x 2 tiles x 3 pieces x 64 lanes

__device__ __forceinline__ float4 xld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
// four consecutive channels of a texture row of which `n` (may be <= 0 or > 4) exist; VEC: the rows are
// 16-byte aligned and the channel count is a multiple of 4 (compile time, so that the common case keeps
// its straight 16-byte loads)
template <bool VEC> __device__ __forceinline__ float4 xld4_row(const float *p, int n)
{
    if constexpr (VEC) return n > 0 ? xld4(p) : make_float4(0.f, 0.f, 0.f, 0.f);
    float4 r;
    r.x = n > 0 ? p[0] : 0.f;
    r.y = n > 1 ? p[1] : 0.f;
    r.z = n > 2 ? p[2] : 0.f;
    r.w = n > 3 ? p[3] : 0.f;
    return r;
}
// bf16 feature rows (the filter gradient also serves the reduced-precision variant as its guarded second launch)
typedef unsigned short bf16_t;
__device__ __forceinline__ float xbf(unsigned short v) { return __builtin_bit_cast(float, (unsigned)v << 16); }
template <bool VEC> __device__ __forceinline__ float4 xld4_row(const bf16_t *p, int n)
{
    if constexpr (VEC) {
        if (n <= 0) return make_float4(0.f, 0.f, 0.f, 0.f);
        const uint2 u = *reinterpret_cast<const uint2 *>(p);
        return make_float4(__builtin_bit_cast(float, u.x << 16), __builtin_bit_cast(float, u.x & 0xFFFF0000u),
                           __builtin_bit_cast(float, u.y << 16), __builtin_bit_cast(float, u.y & 0xFFFF0000u));
    }
    float4 r;
    r.x = n > 0 ? xbf(p[0]) : 0.f;
    r.y = n > 1 ? xbf(p[1]) : 0.f;
    r.z = n > 2 ? xbf(p[2]) : 0.f;
    r.w = n > 3 ? xbf(p[3]) : 0.f;
    return r;
}
__device__ __forceinline__ float xld1(const float *p) { return *p; }
__device__ __forceinline__ float xld1(const bf16_t *p) { return xbf(*p); }
__device__ __forceinline__ unsigned fbits(float x) { return __builtin_bit_cast(unsigned, x); }
__device__ __forceinline__ float bitsf(unsigned u) { return __builtin_bit_cast(float, u); }
// {hi16(b), hi16(a)}: two truncated bf16 values in one register, a in the low half
__device__ __forceinline__ unsigned pack_hi(float a, float b)
{
    return __builtin_amdgcn_perm(fbits(b), fbits(a), 0x07060302u);
}
__device__ __forceinline__ float trunc_bf16(float x) { return bitsf(fbits(x) & 0xFFFF0000u); }

// split eight fp32 values into three packed bf16x8 pieces (truncation; measured no slower than the
// v_cvt_pk_bf16_f32 / v_dot2c_f32_bf16 route, which needs 28 instead of 44 instructions but slower ones)
__device__ __forceinline__ void split8(const float (&x)[8], u32x4 &p1, u32x4 &p2, u32x4 &p3)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = x[2 * j], b = x[2 * j + 1];
        p1[j] = pack_hi(a, b);
        const float ra = a - trunc_bf16(a), rb = b - trunc_bf16(b);
        p2[j] = pack_hi(ra, rb);
        p3[j] = pack_hi(ra - trunc_bf16(ra), rb - trunc_bf16(rb));
    }
}

__device__ __forceinline__ f32x16 mfma_bf16(const u32x4 &a, const u32x4 &b, const f32x16 &c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                    0, 0, 0);
}

__device__ __forceinline__ int xwave_max(int v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int t = __shfl_xor(v, o, 64);
        v = t > v ? t : v;
    }
    return __builtin_amdgcn_readfirstlane(v);
}

// Filter (Cout, Cin, 16) -> per-lane MFMA B operands: Wp[((ci*NT + nt)*3 + piece)*64 + lane] holds the
// eight bf16 pieces of W[nt*32 + l32][ci][8h .. 8h+7], lane = 32h + l32.  NT = even number of
// 32-channel tiles covering Cout (zero padded).
__global__ __launch_bounds__(kBlock) void f2f16x3_pack_filter_k(const float *__restrict__ W, u32x4 *__restrict__ Wp,
                                                                int Cin, int CinPad, int Cout, int NT)
{
    const int idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= CinPad * NT * 64) return;
    const int lane = idx & 63, nt = (idx >> 6) % NT, ci = (idx >> 6) / NT;
    const int co = nt * 32 + (lane & 31), h = lane >> 5;
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = 0.f;
    if (co < Cout && ci < Cin) {                      // channels Cin .. CinPad-1 are zero rows
        const float *p = W + ((int64_t)co * Cin + ci) * 16 + 8 * h;
        const float4 u = xld4(p), v = xld4(p + 4);
        x[0] = u.x; x[1] = u.y; x[2] = u.z; x[3] = u.w; x[4] = v.x; x[5] = v.y; x[6] = v.z; x[7] = v.w;
    }
    u32x4 p1, p2, p3;
    split8(x, p1, p2, p3);
    u32x4 *dst = Wp + ((size_t)(ci * NT + nt) * 3) * 64 + lane;
    dst[0] = p1; dst[64] = p2; dst[128] = p3;
}

// Forward work decomposition: a workgroup of kFW wavefronts owns 256 facets x 64 output channels,
// each wavefront kFR 32-facet row tiles.  With one row tile per wavefront two wavefronts fit a SIMD
// (256 registers each), so the FMAs / conversions of one overlap the MFMAs of the other.
constexpr int kFR = 1;                          // row tiles (facets per lane) of a wavefront
constexpr int kFW = 8 / kFR;                    // wavefronts per workgroup
constexpr int kFThreads = 64 * kFW;
constexpr int kFWn = 1536 / kFThreads;          // uint4 of a filter chunk fetched per thread
constexpr int kXSlab = kXKB * 8 * 32 * kFR;     // floats per slab buffer: points x 8 channels x facet slots

__device__ __forceinline__ void w_chunk_fetch(const u32x4 *__restrict__ Wp, int c0, int NT, int nt0, u32x4 (&wn)[kFWn])
{
    // channel c of the chunk: 2 tiles x 3 pieces x 64 lanes = 384 consecutive uint4
#pragma unroll
    for (int i = 0; i < kFWn; ++i) {
        const int e = threadIdx.x + kFThreads * i, c = e / 384, o = e - c * 384;
        wn[i] = Wp[((size_t)(c0 + c) * NT + nt0) * 192 + o];
    }
}

// One pass over all input channels for up to KW texture points per facet (compile-time, so the
// operand generation is a straight line of FMAs).
//   texture values: the wavefront's 32*kFR x KW texture rows are fetched 8 channels at a time with
//     16-byte loads (two lanes per row), a group ahead, and parked in a wavefront-private LDS slab
//     from which every lane picks its own facets' values;
//   filter: chunks of four channels copied to LDS two chunks ahead (shared by the workgroup).
// Both are published right before the workgroup barrier that ends a chunk.
template <int KW, bool TVEC>
__device__ __forceinline__ void x3_sweep(const float *__restrict__ tex, const u32x4 *__restrict__ Wp,
                                         const float *__restrict__ sh, u32x4 *Ws, float *slab, f32x16 (&acc)[kFR][2],
                                         const int (&kbase)[kFR], const int (&Ks)[kFR], const float (&invK)[kFR],
                                         const int *s_k0, const int *s_K, int sweep, int Cin, int NT, int nt0,
                                         int nblk, int w, int lane, int h)
{
    constexpr int NL = kFR * KW;                 // slab loads per lane and group
    const int l32 = lane & 31;
    // SH values of my facets' points, my half's eight d's, pre-scaled by 1/K
    float shr[kFR][KW][8];
#pragma unroll
    for (int r = 0; r < kFR; ++r)
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) {
            float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
            if (kk < Ks[r]) {
                const float *p = sh + (int64_t)(kbase[r] + kk) * 16 + 8 * h;
                u = xld4(p);
                v = xld4(p + 4);
            }
            const float s = invK[r];
            shr[r][kk][0] = u.x * s; shr[r][kk][1] = u.y * s; shr[r][kk][2] = u.z * s; shr[r][kk][3] = u.w * s;
            shr[r][kk][4] = v.x * s; shr[r][kk][5] = v.y * s; shr[r][kk][6] = v.z * s; shr[r][kk][7] = v.w * s;
        }
    // rows this lane fetches for the slab: load i covers point kk = i / kFR of facet slot
    // (lane/2) + 32*(i % kFR), channels 4*(lane%2) .. +3 of the group
    const int cg4 = 4 * (lane & 1);
    unsigned ldoff[NL];
    bool ldok[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int slot = w * 32 * kFR + (lane >> 1) + 32 * (i % kFR), kk = sweep * kXKB + i / kFR;
        ldok[i] = kk < s_K[slot];
        ldoff[i] = (unsigned)(s_k0[slot] + (ldok[i] ? kk : 0)) * (unsigned)Cin + cg4;
    }
    float4 pf[NL];
    auto fetch_group = [&](int g) {
#pragma unroll
        for (int i = 0; i < NL; ++i)
            pf[i] = ldok[i] ? xld4_row<TVEC>(tex + (ldoff[i] + 8 * g), Cin - (8 * g + cg4)) : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    auto publish_group = [&](float *dst) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            float *q = dst + ((i / kFR) * 8 + cg4) * (32 * kFR) + (lane >> 1) + 32 * (i % kFR);
            q[0] = pf[i].x; q[32 * kFR] = pf[i].y; q[64 * kFR] = pf[i].z; q[96 * kFR] = pf[i].w;
        }
    };
    // filter chunks sit in three LDS buffers and are published two chunks ahead, so that the chunk
    // after the current one is always complete and operand reads may run ahead across chunk ends
    u32x4 wn[kFWn];
    fetch_group(0);
    publish_group(slab);
    w_chunk_fetch(Wp, 0, NT, nt0, wn);
#pragma unroll
    for (int i = 0; i < kFWn; ++i) Ws[threadIdx.x + kFThreads * i] = wn[i];
    if (nblk > 1) {
        w_chunk_fetch(Wp, 4, NT, nt0, wn);
#pragma unroll
        for (int i = 0; i < kFWn; ++i) Ws[kXChunk + threadIdx.x + kFThreads * i] = wn[i];
    }
    __syncthreads();

    auto read_b = [&](u32x4 (&b)[2][3], int c) {          // filter pieces of channel c (c < Cin)
        const u32x4 *Wc = Ws + ((c >> 2) % 3) * kXChunk + (c & 3) * 384 + lane;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int p = 0; p < 3; ++p) b[t][p] = Wc[(t * 3 + p) * 64];
    };
    auto read_tv = [&](float (&tv)[kFR][KW], int c) {     // my facets' texture values of channel c
        const float *sl = slab + ((c >> 3) & 1) * kXSlab + (c & 7) * (32 * kFR) + l32;
#pragma unroll
        for (int r = 0; r < kFR; ++r)
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) tv[r][kk] = sl[kk * 8 * (32 * kFR) + r * 32];
    };
    auto gen = [&](float (&a)[kFR][8], const float (&tv)[kFR][KW]) {
#pragma unroll
        for (int r = 0; r < kFR; ++r)
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                float v = 0.f;
#pragma unroll
                for (int kk = 0; kk < KW; ++kk) v = fmaf(tv[r][kk], shr[r][kk][s], v);
                a[r][s] = v;
            }
    };

    // software pipeline over channels: while channel c is multiplied, the G values of c+1 are
    // generated and split, and the LDS reads for c+1 (filter) and c+2 (texture) are in flight
    u32x4 pa[kFR][3], b[2][3];
    float tvn[kFR][KW];
    {
        float tv0[kFR][KW], a[kFR][8];
        read_tv(tv0, 0);
        read_tv(tvn, 1);
        read_b(b, 0);
        gen(a, tv0);
#pragma unroll
        for (int r = 0; r < kFR; ++r) split8(a[r], pa[r][0], pa[r][1], pa[r][2]);
    }

    for (int j = 0; j < nblk; ++j) {
        const int g = j >> 1;
        const bool wmore = j + 2 < nblk;
        const bool stage = !(j & 1) && 8 * (g + 1) < Cin;       // even chunk: bring in the next 8-channel group
        if (wmore) w_chunk_fetch(Wp, 4 * (j + 2), NT, nt0, wn);
        if (stage) fetch_group(g + 1);
#pragma unroll
        for (int ci_l = 0; ci_l < 4; ++ci_l) {
            const int c = 4 * j + ci_l;
            u32x4 bn[2][3];
            float tvnn[kFR][KW];
            // c+1 == Cin reads a chunk buffer / slab row that exists but is not used
            read_b(bn, c + 1 < 4 * nblk ? c + 1 : c);
            read_tv(tvnn, c + 2);

            float an[kFR][8];
            gen(an, tvn);
            u32x4 pn[kFR][3];
#pragma unroll
            for (int r = 0; r < kFR; ++r) split8(an[r], pn[r][0], pn[r][1], pn[r][2]);

            // six piece products per accumulator tile, smallest first
#pragma unroll
            for (int term = 0; term < 6; ++term) {
                const int ga = term == 0 ? 2 : term == 1 ? 1 : term == 2 ? 0 : term == 3 ? 1 : 0;
                const int wb = term == 0 ? 0 : term == 1 ? 1 : term == 2 ? 2 : term == 3 ? 0 : term == 4 ? 1 : 0;
#pragma unroll
                for (int r = 0; r < kFR; ++r)
#pragma unroll
                    for (int t = 0; t < 2; ++t) acc[r][t] = mfma_bf16(pa[r][ga], b[t][wb], acc[r][t]);
            }
#pragma unroll
            for (int r = 0; r < kFR; ++r) {
#pragma unroll
                for (int p = 0; p < 3; ++p) pa[r][p] = pn[r][p];
#pragma unroll
                for (int kk = 0; kk < KW; ++kk) tvn[r][kk] = tvnn[r][kk];
            }
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int p = 0; p < 3; ++p) b[t][p] = bn[t][p];
        }
        if (wmore) {
#pragma unroll
            for (int i = 0; i < kFWn; ++i) Ws[((j + 2) % 3) * kXChunk + threadIdx.x + kFThreads * i] = wn[i];
        }
        if (stage) publish_group(slab + ((g + 1) & 1) * kXSlab);
        __syncthreads();
    }
}

// `order` (may be null) lists the facets sorted by their number of texture points, so that the 256
// facets of a workgroup -- and the 32*kFR of a wavefront -- have (nearly) equal counts: the work per
// sweep is set by the longest facet, and facets with more than kXKB points need further sweeps.
template <bool TVEC>
__global__ __launch_bounds__(kFThreads, 2 / kFR) void f2f16x3_fwd_k(const float *__restrict__ tex,
                                                                   const u32x4 *__restrict__ Wp,
                                                                   const float *__restrict__ sh,
                                                                   const int *__restrict__ cum,
                                                                   const int *__restrict__ order,
                                                                   float *__restrict__ out, int64_t Nf, int T, int Cin,
                                                                   int Cout, int NT)
{
    __shared__ u32x4 Ws[3 * kXChunk];
    __shared__ __attribute__((aligned(16))) float s_slab[kFW * 2 * kXSlab];      // per wavefront: two buffers
    __shared__ int s_f[256], s_k0[256], s_K[256], s_kmax;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int64_t s0 = (int64_t)blockIdx.x * 256;
    const int nt0 = blockIdx.y * 2, n0 = blockIdx.y * 64;
    const int nblk = (Cin + 3) >> 2;

    if (threadIdx.x == 0) s_kmax = 0;
    for (int i = threadIdx.x; i < 256; i += kFThreads) {
        const int64_t slot = s0 + i;
        const int f = slot < Nf ? (order ? order[slot] : (int)slot) : -1;
        int a = 0, b = 0;
        if (f >= 0 && f < Nf) {
            a = f ? cum[f - 1] : 0;
            b = cum[f];
            a = a < 0 ? 0 : (a > T ? T : a);
            b = b < 0 ? 0 : (b > T ? T : b);
        }
        s_f[i] = f;
        s_k0[i] = a;
        s_K[i] = b > a ? b - a : 0;
    }
    __syncthreads();
    int k0[kFR], K[kFR], kmax = 0;
    float invK[kFR];
#pragma unroll
    for (int r = 0; r < kFR; ++r) {
        k0[r] = s_k0[w * 32 * kFR + r * 32 + l32];
        K[r] = s_K[w * 32 * kFR + r * 32 + l32];
        invK[r] = K[r] > 0 ? 1.0f / (float)K[r] : 0.f;
        kmax = K[r] > kmax ? K[r] : kmax;
    }
    {
        const int km = xwave_max(kmax);
        if (lane == 0) atomicMax(&s_kmax, km);
    }
    __syncthreads();
    const int nsweeps = (s_kmax + kXKB - 1) / kXKB;

    f32x16 acc[kFR][2];
#pragma unroll
    for (int r = 0; r < kFR; ++r)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[r][t][i] = 0.f;

    for (int sw = 0; sw < nsweeps; ++sw) {
        int kbase[kFR], Ks[kFR], kw = 0;
#pragma unroll
        for (int r = 0; r < kFR; ++r) {
            kbase[r] = k0[r] + sw * kXKB;
            const int rem = K[r] - sw * kXKB;
            Ks[r] = rem < 0 ? 0 : (rem > kXKB ? kXKB : rem);
            kw = Ks[r] > kw ? Ks[r] : kw;
        }
        // every variant runs the same barriers, so wavefronts of a workgroup may pick different ones
        kw = xwave_max(kw);
#define PM_X3(N) x3_sweep<N, TVEC>(tex, Wp, sh, Ws, s_slab + w * 2 * kXSlab, acc, kbase, Ks, invK, s_k0, s_K, sw, Cin, NT, nt0, nblk, w, lane, h)
        if (kw <= 1) PM_X3(1);
        else if (kw == 2) PM_X3(2);
        else if (kw == 3) PM_X3(3);
        else PM_X3(4);
#undef PM_X3
    }

#pragma unroll
    for (int r = 0; r < kFR; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int fr = s_f[w * 32 * kFR + r * 32 + 8 * (i / 4) + 4 * h + (i % 4)];
            if (fr >= 0 && fr < Nf) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int co = n0 + t * 32 + l32;
                    if (co < Cout) out[(int64_t)fr * Cout + co] = acc[r][t][i];
                }
            }
        }
}

// ----------------------------------------------------------------------------------------
// texture gradient on the bf16 matrix cores:
//     H[f, ci, d] = sum_co gout[f, co] W[co, ci, d]          (split-bf16 MFMAs, k = co)
//     gtex[t, ci] = (1/K_f) sum_d sh[t, d] H[f, ci, d]       (FMAs on the accumulator registers)
// The product is taken transposed, D[(ci,d)][f] = W^T . gout^T.  A tile tt = 4g + q holds the two input
// channels 8g + q ("a") and 8g + 4 + q ("b"); its 32 rows are ordered so that a lane (facet l32,
// half h) finds in its 16 accumulator registers eight d's of BOTH channels:
//     register i  <->  channel (i/4)%2,  d = 8(i/8) + 4h + i%4.
// Each lane contracts its eight d's with the SH values of ALL the facet's points (8 instead of 16 SH
// values per point in registers), and one v_permlane32_swap per point exchanges the partial sums so
// that half 0 ends up with channel a and half 1 with channel b.  After the four tiles of a group a
// lane owns four consecutive channels of each point.  The contraction of a tile runs while the MFMAs
// of the next tile are in flight.
//   workgroup  256 facets from the sorted list, 8 wavefronts x 32 facets, two wavefronts per SIMD
//   gout       a lane's facet row, split once into bf16 pieces (B operand, registers)
//   filter     pre-split / pre-arranged W^T tiles (f2f16x3_pack_filter_t_k), two tiles per LDS chunk,
//              three chunk buffers published two chunks ahead
//   points     sweeps of up to four texture points per facet (their SH rows in registers)
constexpr int kTKS = 4;                          // k-steps of 16 output channels (Cout <= 64)
constexpr int kTChunkMax = 2 * kTKS * 3 * 64;    // uint4 per chunk buffer: 2 tiles x k-steps x 3 pieces x 64 lanes

// W (Cout, Cin, 16) -> A operands of the transposed product:
// WpT[((tt*NKS + ks)*3 + piece)*64 + lane] = pieces of W[co0 + 16ks + 8h .. +7][ci(tt, r)][d(r)], r = lane % 32
__global__ __launch_bounds__(kBlock) void f2f16x3_pack_filter_t_k(const float *__restrict__ W, u32x4 *__restrict__ WpT,
                                                                  int Cin, int Cout, int NTt, int NKS, int co0)
{
    const int idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= NTt * NKS * 64) return;
    const int lane = idx & 63, ks = (idx >> 6) % NKS, tt = (idx >> 6) / NKS;
    const int r = lane & 31, h = lane >> 5;
    // row r = 8q + 4h' + j of the tile (h' = accumulator half, register 4q + j): channel q%2, d = 8(q/2) + 4h' + j
    const int ci = 8 * (tt >> 2) + 4 * ((r >> 3) & 1) + (tt & 3), d = 8 * (r >> 4) + 4 * ((r >> 2) & 1) + (r & 3);
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int co = co0 + 16 * ks + 8 * h + j;             // this launch covers channels co0 .. co0 + 16 NKS - 1
        x[j] = (ci < Cin && co < Cout) ? W[((int64_t)co * Cin + ci) * 16 + d] : 0.f;
    }
    u32x4 p1, p2, p3;
    split8(x, p1, p2, p3);
    u32x4 *dst = WpT + ((size_t)(tt * NKS + ks) * 3) * 64 + lane;
    dst[0] = p1; dst[64] = p2; dst[128] = p3;
}

template <int KW, int NKS, bool GVEC>
__device__ __forceinline__ void x3_tex_sweep(const u32x4 *__restrict__ WpT, const float *__restrict__ sh,
                                             float *__restrict__ gtex, u32x4 *Ws, float *stage, const int *w_k0,
                                             const int *w_K, const u32x4 (&bp)[NKS][3], int kbase, int Ks, float invK,
                                             int sweep, int Cin, int NG, bool add, int lane, int h)
{
    // SH values of my facet's points for my half's eight d's (4h..4h+3, 8+4h..8+4h+3), pre-scaled by 1/K
    float shr[KW][8];
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) {
        float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
        if (kk < Ks) {
            const float *p = sh + (int64_t)(kbase + kk) * 16 + 4 * h;
            u = xld4(p);
            v = xld4(p + 8);
        }
        shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
        shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
    }
    constexpr int chunk = 2 * NKS * 192;         // uint4 per chunk of two tiles
    const int nchunks = 2 * NG;
    auto chunk_fetch = [&](u32x4 (&wn)[3], int c) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int e = threadIdx.x + 512 * i;
            if (e < chunk) wn[i] = WpT[(size_t)c * chunk + e];
        }
    };
    auto chunk_publish = [&](const u32x4 (&wn)[3], int c) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int e = threadIdx.x + 512 * i;
            if (e < chunk) Ws[(c % 3) * kTChunkMax + e] = wn[i];
        }
    };
    u32x4 wn[3];
    chunk_fetch(wn, 0);
    chunk_publish(wn, 0);
    chunk_fetch(wn, 1);
    chunk_publish(wn, 1);
    __syncthreads();

    // 16-channel block gp of the stage -> global memory
    auto flush = [&](int gp) {
        const int ci = 16 * gp + 4 * (lane & 3);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int slot = 16 * i + (lane >> 2);
            const int k0s = w_k0[slot] + sweep * kXKB, Kss = w_K[slot] - sweep * kXKB;
#pragma unroll
            for (int kk = 0; kk < KW; ++kk)
                if (kk < Kss && ci < Cin) {
                    const float4 v = *reinterpret_cast<const float4 *>(stage + (kk * 32 + slot) * 16 + 4 * (lane & 3));
                    float *dst = gtex + (int64_t)(k0s + kk) * Cin + ci;
                    // `add`: a later block of 64 output channels accumulates onto what the earlier ones wrote
                    if constexpr (GVEC) {
                        float4 o = v;
                        if (add) {
                            const float4 p = *reinterpret_cast<const float4 *>(dst);
                            o = make_float4(p.x + v.x, p.y + v.y, p.z + v.z, p.w + v.w);
                        }
                        *reinterpret_cast<float4 *>(dst) = o;
                    } else {                               // channel count not a multiple of 4 / unaligned rows
                        dst[0] = add ? dst[0] + v.x : v.x;
                        if (ci + 1 < Cin) dst[1] = add ? dst[1] + v.y : v.y;
                        if (ci + 2 < Cin) dst[2] = add ? dst[2] + v.z : v.z;
                        if (ci + 3 < Cin) dst[3] = add ? dst[3] + v.w : v.w;
                    }
                }
        }
    };
    // Results go out 64 bytes at a time: two groups (16 channels) of every point are collected in
    // the wavefront's LDS stage [point][facet slot][16 channels], then four lanes write one
    // 64-byte piece of a row (32-byte pieces cost almost twice the HBM write traffic).
    float gacc[KW][4];
    auto finish_group = [&](int g) {
#pragma unroll
        for (int kk = 0; kk < KW; ++kk)
            *reinterpret_cast<float4 *>(stage + (kk * 32 + (lane & 31)) * 16 + (g & 1) * 8 + 4 * h) =
                make_float4(gacc[kk][0], gacc[kk][1], gacc[kk][2], gacc[kk][3]);
        if ((g & 1) || g == NG - 1) flush(g >> 1);
    };
    // contraction of a finished tile (accumulator accp) into channel slot q of the group
    f32x16 accp;
#pragma unroll
    for (int i = 0; i < 16; ++i) accp[i] = 0.f;
    auto contract = [&](int q) {
        float xa[KW], xb[KW];
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) {
            float va = 0.f, vb = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                va = fmaf(shr[kk][j], accp[8 * (j >> 2) + (j & 3)], va);          // channel a: registers 0-3, 8-11
                vb = fmaf(shr[kk][j], accp[8 * (j >> 2) + 4 + (j & 3)], vb);      // channel b: registers 4-7, 12-15
            }
            xa[kk] = va;
            xb[kk] = vb;
        }
        // xa: half 0 keeps its own, receives half 0's xb into half 1; xb: half 0 receives half 1's xa.
        // Afterwards xa + xb is the full sum over d of channel a in half 0 and of channel b in half 1.
        // (The s_nop cover the wait states between vector ALU writes / reads and the swap.)
#pragma unroll
        for (int kk = 0; kk < KW; ++kk)
            asm volatile("s_nop 3\n v_permlane32_swap_b32 %0, %1\n s_nop 3" : "+v"(xa[kk]), "+v"(xb[kk]));
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) gacc[kk][q] = xa[kk] + xb[kk];
    };

    for (int g = 0; g < NG; ++g) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int c = 2 * g + cc;
            const bool more = c + 2 < nchunks;
            if (more) chunk_fetch(wn, c + 2);
            const u32x4 *Wc = Ws + (c % 3) * kTChunkMax + lane;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                // H tile of two input channels: rows (d half, channel, d), columns = my wavefront's facets
                f32x16 acc0;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc0[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    u32x4 a[3];
#pragma unroll
                    for (int p = 0; p < 3; ++p) a[p] = Wc[((u * NKS + ks) * 3 + p) * 64];
                    // six piece products, smallest first
                    acc0 = mfma_bf16(a[2], bp[ks][0], acc0);
                    acc0 = mfma_bf16(a[1], bp[ks][1], acc0);
                    acc0 = mfma_bf16(a[0], bp[ks][2], acc0);
                    acc0 = mfma_bf16(a[1], bp[ks][0], acc0);
                    acc0 = mfma_bf16(a[0], bp[ks][1], acc0);
                    acc0 = mfma_bf16(a[0], bp[ks][0], acc0);
                }
                // meanwhile: the previous tile (the last one of the previous group when cc = u = 0)
                contract((2 * cc + u + 3) & 3);
                if (cc == 0 && u == 0 && g > 0) finish_group(g - 1);
                accp = acc0;
            }
            if (more) chunk_publish(wn, c + 2);
            __syncthreads();
        }
    }
    contract(3);
    finish_group(NG - 1);
}

// NKS = k-steps of 16 output channels (compile time, so that a tile's MFMAs and the previous tile's
// contraction share one basic block and get interleaved): 2 for Cout <= 32, else 4; the packed filter
// is zero padded to that many.
template <int NKS, bool GVEC>
__global__ __launch_bounds__(512, 2) void f2f16x3_bwd_tex_k(const float *__restrict__ gout,
                                                            const u32x4 *__restrict__ WpT,
                                                            const float *__restrict__ sh,
                                                            const int *__restrict__ cum,
                                                            const int *__restrict__ order, float *__restrict__ gtex,
                                                            int64_t Nf, int T, int Cin, int Cout, int NG, int co0)
{
    __shared__ u32x4 Ws[3 * kTChunkMax];
    __shared__ __attribute__((aligned(16))) float s_stage[8][kXKB * 32 * 16];
    __shared__ int s_k0[8][32], s_K[8][32], s_kmax;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    if (threadIdx.x == 0) s_kmax = 0;
    __syncthreads();

    const int64_t slot = (int64_t)blockIdx.x * 256 + w * 32 + l32;
    const int f = slot < Nf ? (order ? order[slot] : (int)slot) : -1;
    int k0 = 0, K = 0;
    if (f >= 0 && f < Nf) {
        int a = f ? cum[f - 1] : 0, b = cum[f];
        a = a < 0 ? 0 : (a > T ? T : a);
        b = b < 0 ? 0 : (b > T ? T : b);
        k0 = a;
        K = b > a ? b - a : 0;
    }
    const float invK = K > 0 ? 1.0f / (float)K : 0.f;
    if (h == 0) {
        s_k0[w][l32] = k0;
        s_K[w][l32] = K;
    }
    {
        const int km = xwave_max(K);
        if (lane == 0) atomicMax(&s_kmax, km);
    }
    // my facet's gout row as B operand pieces: k-step ks, half h <-> channels 16ks + 8h .. + 7
    u32x4 bp[NKS][3];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = 0.f;
        const int co = co0 + 16 * ks + 8 * h;
        if (K > 0 && co < Cout) {
            const float *p = gout + (int64_t)f * Cout + co;
            const float4 u = xld4(p), v = xld4(p + 4);
            x[0] = u.x; x[1] = u.y; x[2] = u.z; x[3] = u.w; x[4] = v.x; x[5] = v.y; x[6] = v.z; x[7] = v.w;
        }
        split8(x, bp[ks][0], bp[ks][1], bp[ks][2]);
    }
    __syncthreads();
    const int nsweeps = (s_kmax + kXKB - 1) / kXKB;
    for (int sw = 0; sw < nsweeps; ++sw) {
        const int rem = K - sw * kXKB;
        const int Ks = rem < 0 ? 0 : (rem > kXKB ? kXKB : rem);
        const int kw = xwave_max(Ks);
        const int kbase = k0 + sw * kXKB;
        // every variant runs the same barriers, so wavefronts of a workgroup may pick different ones
#define PM_X3T(N) x3_tex_sweep<N, NKS, GVEC>(WpT, sh, gtex, Ws, s_stage[w], s_k0[w], s_K[w], bp, kbase, Ks, invK, sw, Cin, NG, co0 > 0, lane, h)
        if (kw <= 1) PM_X3T(1);
        else if (kw == 2) PM_X3T(2);
        else if (kw == 3) PM_X3T(3);
        else PM_X3T(4);
#undef PM_X3T
    }
}

// ----------------------------------------------------------------------------------------
// filter gradient gW = gout^T . G on the bf16 matrix cores: G is formed exactly as in the forward (lane = facet, eight
// d's in registers, SH rows of the facet's points in registers), split into bf16 pieces, and each
// piece is TRANSPOSED BY THE MATRIX CORE ITSELF: D = piece . E with a 0/1 selection matrix E is exact
// and leaves, in the accumulator layout, lane = column (channel, d) and registers = facets -- the
// layout of an MFMA operand whose reduction index is the facet.  Two input channels share one
// transposition tile (columns 0..15 / 16..31).  The facet order inside a reduction step is the
// accumulator's row order; the gout operand is built with the same order.
//   workgroup  4 wavefronts (one per SIMD, accumulators in up to 256 registers), 64 input x 64 output
//              channels, a strided subset of the 32-facet tiles of the sorted facet list
//   wavefront  16 input channels = 8 channel pairs x 2 output tiles of gW^T[(ci,d)][co]; filters with
//              fewer than 64 input channels give every wavefront 1, 2 or 4 pairs instead (NCP)
//   gout^T     per facet tile split and laid out per lane in LDS by the whole workgroup

// One pass = up to KW texture points per facet (missing points contribute zeros), straight-line code.
// shr: SH values of my facet's points (my half's eight d's, scaled by 1/K); slab: the wavefront's
// texture values [point][16-byte piece][facet slot]; go: the tile's gout^T operand.
template <int KW, int NCP>
__device__ __forceinline__ void x3_filt_pass(const float (&shr)[KW][8], const float4 *slab, const u32x4 *go,
                                             f32x16 (&acc)[NCP][2], const u32x4 &ea, const u32x4 &eb, int lane)
{
    const int l32 = lane & 31;
    // G of channels cbase + 2cp (a) and + 1 (b), eight d's of my half for my facet, as bf16 pieces
    auto gen = [&](u32x4 (&pa)[3], u32x4 (&pb)[3], int cp) {
        float aa[8], ab[8];
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) {
            const float4 t4 = slab[(kk * 4 + (cp >> 1)) * 32 + l32];
            const float ta = (cp & 1) ? t4.z : t4.x, tb = (cp & 1) ? t4.w : t4.y;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                aa[q] = kk ? fmaf(ta, shr[kk][q], aa[q]) : ta * shr[kk][q];
                ab[q] = kk ? fmaf(tb, shr[kk][q], ab[q]) : tb * shr[kk][q];
            }
        }
        split8(aa, pa[0], pa[1], pa[2]);
        split8(ab, pb[0], pb[1], pb[2]);
    };
    // transposed pieces as operands of the two reduction steps (16 facets each); the three
    // transpositions are independent, so their MFMAs run back to back
    // The six MFMAs are written as one asm block with VGPR destinations: in a kernel whose accumulators
    // live in AGPRs the compiler gives every MFMA an AGPR destination, and the 48 results would have
    // to be copied out one by one before the packing.  The trailing s_nop cover the wait states a
    // vector ALU read of an MFMA result needs (the compiler cannot see into the block).
    auto transpose = [&](u32x4 (&o)[3][2], const u32x4 (&pa)[3], const u32x4 (&pb)[3]) {
        f32x16 d0, d1, d2;
        asm volatile("s_nop 3\n"
                     "v_mfma_f32_32x32x16_bf16 %0, %3, %9, 0\n"
                     "v_mfma_f32_32x32x16_bf16 %1, %4, %9, 0\n"
                     "v_mfma_f32_32x32x16_bf16 %2, %5, %9, 0\n"
                     "v_mfma_f32_32x32x16_bf16 %0, %6, %10, %0\n"
                     "v_mfma_f32_32x32x16_bf16 %1, %7, %10, %1\n"
                     "v_mfma_f32_32x32x16_bf16 %2, %8, %10, %2\n"
                     "s_nop 15\n"
                     "s_nop 7\n"
                     : "=&v"(d0), "=&v"(d1), "=&v"(d2)
                     : "v"(pa[0]), "v"(pa[1]), "v"(pa[2]), "v"(pb[0]), "v"(pb[1]), "v"(pb[2]), "v"(ea), "v"(eb));
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                o[0][st][jj] = pack_hi(d0[8 * st + 2 * jj], d0[8 * st + 2 * jj + 1]);
                o[1][st][jj] = pack_hi(d1[8 * st + 2 * jj], d1[8 * st + 2 * jj + 1]);
                o[2][st][jj] = pack_hi(d2[8 * st + 2 * jj], d2[8 * st + 2 * jj + 1]);
            }
    };

    // the gout^T operand stays in registers for the whole pass (it serves all eight channel pairs)
    u32x4 g[2][2][3];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int p = 0; p < 3; ++p) g[st][t][p] = go[((st * 2 + t) * 3 + p) * 64 + lane];

    // software pipeline over the channel pairs: the G values of pair cp+1 are generated and split
    // (vector ALU) while the products of pair cp run on the matrix core
    u32x4 o[3][2];
    {
        u32x4 pa[3], pb[3];
        gen(pa, pb, 0);
        transpose(o, pa, pb);
    }
#pragma unroll
    for (int cp = 0; cp < NCP; ++cp) {
        u32x4 pa[3], pb[3];
        if (cp + 1 < NCP) gen(pa, pb, cp + 1);
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            // six piece products, smallest first; the two output tiles alternate so that no MFMA
            // waits for the one issued right before it
#pragma unroll
            for (int term = 0; term < 6; ++term) {
                const int ga = term == 0 ? 2 : term == 1 ? 1 : term == 2 ? 0 : term == 3 ? 1 : 0;
                const int wb = term == 0 ? 0 : term == 1 ? 1 : term == 2 ? 2 : term == 3 ? 0 : term == 4 ? 1 : 0;
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[cp][t] = mfma_bf16(o[ga][st], g[st][t][wb], acc[cp][t]);
            }
        }
        if (cp + 1 < NCP) transpose(o, pa, pb);
    }
}

// slot descriptors of a 32-facet tile: facet id (-1: none), first texture point, number of points
struct XTile {
    int f, k0, K;
};
__device__ __forceinline__ XTile xtile_load(const int *__restrict__ cum, const int *__restrict__ order, int64_t tile,
                                            int64_t ntiles, int64_t Nf, int T, int i)
{
    XTile d = {-1, 0, 0};
    const int64_t slot = tile * 32 + i;
    if (tile < ntiles && slot < Nf) {
        const int f = order ? order[slot] : (int)slot;
        if (f >= 0 && f < Nf) {
            int a = f ? cum[f - 1] : 0, b = cum[f];
            a = a < 0 ? 0 : (a > T ? T : a);
            b = b < 0 ? 0 : (b > T ? T : b);
            if (b > a) d = {f, a, b - a};
        }
    }
    return d;
}

// The inputs of a tile's first pass are fetched by the whole workgroup while the previous tile is
// being multiplied (held in registers, written to the other LDS buffer afterwards):
//   gout     thread (co, step, half): its eight facets in accumulator-row order
//   SH rows  32 facets x 4 points x 64 bytes, two 16-byte pieces per thread
// (each wavefront fetches the texture rows of its own 16 channels at the start of a pass)
struct XPre {
    float g[8];
    float4 shv[2];
};
template <typename TIO>
__device__ __forceinline__ void xpre_issue(XPre &P, const TIO *__restrict__ gout, const TIO *__restrict__ tex,
                                           const float *__restrict__ sh, const int *sf, const int *sk0, const int *sK,
                                           int Cin, int Cout, int c0, int n0)
{
    const int co = threadIdx.x & 63, st = (threadIdx.x >> 6) & 1, hh = threadIdx.x >> 7;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int f = sf[16 * st + 8 * (j >> 2) + 4 * hh + (j & 3)];
        P.g[j] = (f >= 0 && n0 + co < Cout) ? xld1(gout + ((int64_t)f * Cout + n0 + co)) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = threadIdx.x + 256 * i, row = e >> 2, kk = row >> 5, slot = row & 31;
        P.shv[i] = kk < sK[slot] ? xld4(sh + (int64_t)(sk0[slot] + kk) * 16 + 4 * (e & 3)) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}
__device__ __forceinline__ void xpre_commit(const XPre &P, u32x4 *go, float *shs)
{
    const int co = threadIdx.x & 63, st = (threadIdx.x >> 6) & 1, hh = threadIdx.x >> 7;
    u32x4 p1, p2, p3;
    split8(P.g, p1, p2, p3);
    u32x4 *dst = go + ((st * 2 + (co >> 5)) * 3) * 64 + 32 * hh + (co & 31);
    dst[0] = p1; dst[64] = p2; dst[128] = p3;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int e = threadIdx.x + 256 * i;
        *reinterpret_cast<float4 *>(shs + 4 * e) = P.shv[i];             // [point*32 + slot][16]
    }
}

// texture rows of one pass (KW points per facet) for my wavefront's 16 channels: 64 bytes per row,
// four lanes per row
template <int KW, bool TVEC, int NCP, typename TIO>
__device__ __forceinline__ void xtex_issue(float4 (&pf)[2 * kXKB], const TIO *__restrict__ tex, const int *sk0,
                                           const int *sK, int sweep, int cw, int Cin, int lane)
{
    const int piece = lane & 3;
#pragma unroll
    for (int i = 0; i < 2 * KW; ++i) {
        const int rr = i * 16 + (lane >> 2), kk = rr >> 5, slot = rr & 31;
        const bool ok = sweep * kXKB + kk < sK[slot] && 4 * piece < 2 * NCP;
        pf[i] = ok ? xld4_row<TVEC>(tex + (int64_t)(sk0[slot] + sweep * kXKB + kk) * Cin + cw + 4 * piece,
                                    Cin - (cw + 4 * piece))
                   : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

__device__ __forceinline__ int xtile_kmax(const int *sK, int lane) { return xwave_max(sK[lane & 31]); }

// One tile of 32 facets whose inputs are in LDS buffer it % 2 (descriptors in it % 3): start the
// fetches for the next tile, run the passes, publish the next tile's inputs.
template <int KW, bool TVEC, int NCP, typename TIO>
__device__ __forceinline__ void x3_filt_tile(const TIO *__restrict__ gout, const TIO *__restrict__ tex,
                                             const float *__restrict__ sh, const int *__restrict__ cum,
                                             const int *__restrict__ order, u32x4 (*go_s)[2 * 2 * 3 * 64], float4 *slab,
                                             float (*sh_s)[kXKB * 32 * 16], int (*s_f)[32], int (*s_k0)[32],
                                             int (*s_K)[32], f32x16 (&acc)[NCP][2], const u32x4 &ea, const u32x4 &eb,
                                             int it, int64_t tile, int64_t stride, int64_t ntiles, int64_t Nf, int T,
                                             int Cin, int Cout, int c0, int n0, int lane, int w)
{
    const int l32 = lane & 31, h = lane >> 5;
    const int buf = it & 1, sb = it % 3, sb1 = (it + 1) % 3, sb2 = (it + 2) % 3;
    // in flight while this tile is multiplied: inputs of the next tile, descriptors of the one after
    XPre P;
    xpre_issue(P, gout, tex, sh, s_f[sb1], s_k0[sb1], s_K[sb1], Cin, Cout, c0, n0);
    XTile dn = {-1, 0, 0};
    if (threadIdx.x < 32) dn = xtile_load(cum, order, tile + 2 * stride, ntiles, Nf, T, threadIdx.x);

    const int k0 = s_k0[sb][l32], K = s_K[sb][l32];
    const float invK = K > 0 ? 1.0f / (float)K : 0.f;
    const int nsweeps = KW < kXKB ? 1 : (xwave_max(K) + kXKB - 1) / kXKB;
    const int cw = c0 + 2 * NCP * w;                     // my wavefront's first input channel
    const bool idle = cw >= Cin;                         // narrow filters leave wavefronts without channels
    for (int sw = 0; sw < nsweeps && !idle; ++sw) {
        const int rem = K - sw * kXKB;
        const int Ks = rem < 0 ? 0 : (rem > KW ? KW : rem);
        float shr[KW][8];
        if (sw == 0) {
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) {
                const float *p = sh_s[buf] + (kk * 32 + l32) * 16 + 8 * h;
                const float4 u = xld4(p), v = xld4(p + 4);
                shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
                shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
            }
        } else {
            // further points of long facets: fetched directly
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) {
                float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
                if (kk < Ks) {
                    const float *p = sh + (int64_t)(k0 + sw * kXKB + kk) * 16 + 8 * h;
                    u = xld4(p);
                    v = xld4(p + 4);
                }
                shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
                shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
            }
        }
        {
            // my wavefront's texture rows of this pass -> slab
            float4 pf[2 * kXKB];
            xtex_issue<KW, TVEC, NCP, TIO>(pf, tex, s_k0[sb], s_K[sb], sw, cw, Cin, lane);
            const int piece = lane & 3;
#pragma unroll
            for (int i = 0; i < 2 * KW; ++i) {
                const int rr = i * 16 + (lane >> 2), kk = rr >> 5, slot = rr & 31;
                slab[(kk * 4 + piece) * 32 + slot] = pf[i];
            }
        }
        x3_filt_pass<KW, NCP>(shr, slab, go_s[buf], acc, ea, eb, lane);
    }

    xpre_commit(P, go_s[buf ^ 1], sh_s[buf ^ 1]);
    if (threadIdx.x < 32) {
        s_f[sb2][threadIdx.x] = dn.f; s_k0[sb2][threadIdx.x] = dn.k0; s_K[sb2][threadIdx.x] = dn.K;
    }
    __syncthreads();
}

// NCP = channel pairs of a wavefront (8 for 64 or more input channels; fewer for narrow filters, so that
// the four wavefronts share what channels there are)
template <bool TVEC, int NCP, typename TIO>
__global__ __launch_bounds__(256, 1) void f2f16x3_bwd_filt_k(const TIO *__restrict__ gout,
                                                              const TIO *__restrict__ tex,
                                                              const float *__restrict__ sh,
                                                              const int *__restrict__ cum,
                                                              const int *__restrict__ order,
                                                              float *__restrict__ partial, int64_t Nf, int T, int Cin,
                                                              int Cout, int64_t ntiles, const int *__restrict__ only_if)
{
    if (only_if && *only_if == 0) return;          // guarded launch: nothing asked for
    __shared__ u32x4 go_s[2][2 * 2 * 3 * 64];
    __shared__ float4 slab_s[4 * kXKB * 4 * 32];
    __shared__ __attribute__((aligned(16))) float sh_s[2][kXKB * 32 * 16];
    __shared__ int s_f[3][32], s_k0[3][32], s_K[3][32];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int c0 = blockIdx.y * (8 * NCP), n0 = blockIdx.z * 64;

    // selection operands of the transposition: column n < 16 takes d = n of channel a, n >= 16 takes d = n - 16 of b
    u32x4 ea, eb;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        unsigned va = 0, vb = 0;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int d = 8 * h + 2 * jj + u;
            if (l32 < 16 && d == l32) va |= 0x3F80u << (16 * u);
            if (l32 >= 16 && d == l32 - 16) vb |= 0x3F80u << (16 * u);
        }
        ea[jj] = va;
        eb[jj] = vb;
    }

    f32x16 acc[NCP][2];
#pragma unroll
    for (int cp = 0; cp < NCP; ++cp)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[cp][t][i] = 0.f;

    // prologue: descriptors of my first two tiles, inputs of the first
    const int64_t stride = gridDim.x;
    int64_t tile = blockIdx.x;
    if (threadIdx.x < 64) {
        const int q = threadIdx.x >> 5;
        const XTile d = xtile_load(cum, order, tile + q * stride, ntiles, Nf, T, threadIdx.x & 31);
        s_f[q][threadIdx.x & 31] = d.f; s_k0[q][threadIdx.x & 31] = d.k0; s_K[q][threadIdx.x & 31] = d.K;
    }
    __syncthreads();
    {
        XPre P;
        xpre_issue(P, gout, tex, sh, s_f[0], s_k0[0], s_K[0], Cin, Cout, c0, n0);
        xpre_commit(P, go_s[0], sh_s[0]);
    }
    __syncthreads();

    // The sorted facet list makes the point counts of my tiles non-decreasing: four loops in sequence,
    // each with the pass specialised for its number of points (the last one takes everything left,
    // long facets in several sweeps).  The bound is uniform over the workgroup.
    int it = 0;
#define PM_PHASE(N)                                                                                                  \
    for (; tile < ntiles && (N == kXKB || xtile_kmax(s_K[it % 3], lane) <= N); ++it, tile += stride)                 \
        x3_filt_tile<N, TVEC, NCP, TIO>(gout, tex, sh, cum, order, go_s, slab_s + w * (kXKB * 4 * 32), sh_s, s_f, s_k0, s_K, acc, ea, eb,  \
                        it, tile, stride, ntiles, Nf, T, Cin, Cout, c0, n0, lane, w)
    PM_PHASE(1);
    PM_PHASE(2);
    PM_PHASE(3);
    PM_PHASE(4);
#undef PM_PHASE

    // accumulator (cp, t): lane (co = 32t + l32, half h), register i <-> row m = 8(i/4) + 4h + i%4
    // = (channel c0 + 16w + 2cp + m/16, d = m%16); four consecutive d's per group of four registers
    float *dst = partial + (int64_t)blockIdx.x * Cout * Cin * 16;
#pragma unroll
    for (int cp = 0; cp < NCP; ++cp)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int co = n0 + 32 * t + l32;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int ci = c0 + 2 * NCP * w + 2 * cp + (q >> 1);
                if (co < Cout && ci < Cin)
                    *reinterpret_cast<float4 *>(dst + ((int64_t)co * Cin + ci) * 16 + 8 * (q & 1) + 4 * h) =
                        make_float4(acc[cp][t][4 * q], acc[cp][t][4 * q + 1], acc[cp][t][4 * q + 2], acc[cp][t][4 * q + 3]);
            }
        }
}

int f2f16x3_bwd_filter_partials(const void *gout_, const void *tex_, const float *sh, const int *cum, const int *order,
                                 float *partial, int splits, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st,
                                 const int *only_if, bool bf16)
{
    // channel pairs per wavefront: the four wavefronts of a workgroup share up to 32 pairs
    const int pairs = (Cin + 1) / 2;
    const int ncp = pairs >= 32 ? 8 : pairs > 8 ? 4 : pairs > 4 ? 2 : 1;
    const int64_t gy = ceil_div(Cin, 8 * ncp), gz = ceil_div(Cout, 64);
    PM_REQUIRE(gy <= 65535 && gz <= 65535, "f2f_bwd_filter: grid too large");
    const int64_t ntiles = ceil_div(Nf, 32);
    const bool tvec = !(Cin & 3) && !(reinterpret_cast<uintptr_t>(tex_) & (bf16 ? 7u : 15u));
    PM_REQUIRE(!bf16 || tvec, "f2f_bwd_filter: bf16 features need a multiple of 4 input channels and 8-byte aligned rows");
    const dim3 grid((unsigned)splits, (unsigned)gy, (unsigned)gz);
#define PM_FILT(V, N, TIO) f2f16x3_bwd_filt_k<V, N, TIO><<<grid, dim3(256), 0, st>>>((const TIO *)gout_, (const TIO *)tex_, sh, cum, order, partial, Nf, (int)T, Cin, Cout, ntiles, only_if)
#define PM_FILT_N(V, TIO)                                                                     \
    do {                                                                                      \
        if (ncp == 8) PM_FILT(V, 8, TIO); else if (ncp == 4) PM_FILT(V, 4, TIO);              \
        else if (ncp == 2) PM_FILT(V, 2, TIO); else PM_FILT(V, 1, TIO);                       \
    } while (0)
    if (bf16) PM_FILT_N(true, bf16_t);
    else if (tvec) PM_FILT_N(true, float);
    else PM_FILT_N(false, float);
#undef PM_FILT_N
#undef PM_FILT
    PM_LAUNCHED("f2f_bwd_filter");
    return 0;
}

bool f2f16x3_usable(const void *W, const void *sh, int F)
{
    return F == 16 && !(reinterpret_cast<uintptr_t>(W) & 15u) && !(reinterpret_cast<uintptr_t>(sh) & 15u);
}

size_t f2f16x3_fwd_workspace_bytes(int Cin, int Cout)
{
    const int NT = 2 * ((Cout + 63) / 64), CinPad = (Cin + 3) & ~3;
    return (size_t)CinPad * NT * 3 * 64 * sizeof(u32x4);
}

int f2f16x3_fwd(const float *tex, const float *W, const float *sh, const int *cum, const int *order, float *out,
                void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st)
{
    const int NT = 2 * ((Cout + 63) / 64);
    PM_REQUIRE(T * Cin < (int64_t(1) << 31), "f2f_fwd: texture array too large for 32-bit offsets");
    PM_REQUIRE(workspace && workspace_bytes >= f2f16x3_fwd_workspace_bytes(Cin, Cout),
               "f2f_fwd: workspace too small (%zu bytes)", workspace_bytes);
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0, "f2f_fwd: workspace must be 16-byte aligned");
    u32x4 *Wp = (u32x4 *)workspace;
    const int CinPad = (Cin + 3) & ~3, n = CinPad * NT * 64;
    f2f16x3_pack_filter_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(W, Wp, Cin, CinPad, Cout, NT);
    PM_LAUNCHED("f2f_fwd(pack)");
    const int64_t gx = ceil_div(Nf, 256), gy = NT / 2;
    PM_REQUIRE(grid_ok(gx) && gy <= 65535, "f2f_fwd: grid too large");
    if (!(Cin & 3) && !(reinterpret_cast<uintptr_t>(tex) & 15u))
        f2f16x3_fwd_k<true><<<dim3((unsigned)gx, (unsigned)gy), dim3(kFThreads), 0, st>>>(tex, Wp, sh, cum, order, out, Nf, (int)T, Cin, Cout, NT);
    else
        f2f16x3_fwd_k<false><<<dim3((unsigned)gx, (unsigned)gy), dim3(kFThreads), 0, st>>>(tex, Wp, sh, cum, order, out, Nf, (int)T, Cin, Cout, NT);
    PM_LAUNCHED("f2f_fwd");
    return 0;
}

size_t f2f16x3_bwd_texture_workspace_bytes(int Cin, int Cout)
{
    const int NG = (Cin + 7) / 8, NKS = Cout <= 32 ? 2 : 4;       // one block of at most 64 output channels at a time
    return (size_t)NG * 4 * NKS * 3 * 64 * sizeof(u32x4);
}

bool f2f16x3_bwd_texture_usable(const void *gout, int Cout) { return (Cout & 7) == 0 && (reinterpret_cast<uintptr_t>(gout) & 15u) == 0; }

int f2f16x3_bwd_texture(const float *gout, const float *W, const float *sh, const int *cum, const int *order,
                        float *gtex, void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                        int Cout, hipStream_t st)
{
    const int NG = (Cin + 7) / 8;
    PM_REQUIRE(workspace && workspace_bytes >= f2f16x3_bwd_texture_workspace_bytes(Cin, Cout),
               "f2f_bwd_texture: workspace too small (%zu bytes)", workspace_bytes);
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0, "f2f_bwd_texture: workspace must be 16-byte aligned");
    u32x4 *WpT = (u32x4 *)workspace;
    const int64_t gx = ceil_div(Nf, 256);
    PM_REQUIRE(grid_ok(gx), "f2f_bwd_texture: grid too large");
    const bool gvec = !(Cin & 3) && !(reinterpret_cast<uintptr_t>(gtex) & 15u);
    // output channels go 64 at a time; the first block writes grad_texture, the others add to it
    // (launches on one stream run in order, so the packed filter buffer is reused)
    for (int co0 = 0; co0 < Cout; co0 += 64) {
        const int NKS = Cout - co0 <= 32 ? 2 : 4;
        const int n = NG * 4 * NKS * 64;
        f2f16x3_pack_filter_t_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(W, WpT, Cin, Cout, NG * 4, NKS, co0);
        PM_LAUNCHED("f2f_bwd_texture(pack)");
#define PM_TEX(N, G) f2f16x3_bwd_tex_k<N, G><<<dim3((unsigned)gx), dim3(512), 0, st>>>(gout, WpT, sh, cum, order, gtex, Nf, (int)T, Cin, Cout, NG, co0)
        if (NKS == 2 && gvec) PM_TEX(2, true);
        else if (NKS == 2) PM_TEX(2, false);
        else if (gvec) PM_TEX(4, true);
        else PM_TEX(4, false);
#undef PM_TEX
        PM_LAUNCHED("f2f_bwd_texture");
    }
    return 0;
}

}  // namespace pmesh
