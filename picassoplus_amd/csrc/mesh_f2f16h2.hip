// facet2facet forward for 16 SH coefficients on the fp16 matrix cores with fp32-level accuracy.
//
// Both operands of out = G . W^T are split into TWO fp16 pieces each,
//     x = x1 + x2 + e,   x1 = x rounded to 11 significant bits,  x2 = (x - x1) rounded to 11 bits,  |e| <= 2^-23 |x|
// and the product is accumulated in fp32 from three piece products,
//     G.W ~ G2W1 + G1W2 + G1W1                        (the dropped G2W2 is <= 2^-22 relative),
// three v_mfma_f32_32x32x16_f16 where the three-piece bf16 split needs six, and 16 instead of 44 vector
// instructions per eight values split.  fp16 has a narrow exponent range, so both operands are brought
// to a fixed magnitude by exact power-of-two scales that are taken out of the accumulator at the end:
//     W' = beta * W        beta from max|W| (one scalar per filter, computed by filter_scale)
//     G'_f = alpha_f * G_f alpha_f from a bound on max|G_f| = max|tex rows of f| * max|SH rows of f|,
//                          taken from the first fetches of the facet's first sweep with head room (every later
//                          value is checked against it; a workgroup whose bound did not hold starts over with
//                          the exact maxima); it rides on the SH values in registers
// so that |W'|, |G'| < 2^14.  Elements far below their row's maximum (by more than 2^17) fall into fp16's
// subnormal range and keep an ABSOLUTE error of 2^-25 in scaled units, i.e. below 2^-39 of the row maximum.
//
// Work decomposition of the forward: workgroup = 128 facets from the list sorted by point count x 64 output
// channels, 4 wavefronts x 32 facets; two workgroups share a CU (two wavefronts per SIMD) and run out of
// phase, so the prologue, barriers and stores of one overlap the channel loop of the other.  Filter chunks
// of four channels alternate between two LDS buffers and arrive there straight from global memory, requested one
// chunk ahead; texture rows go through a wavefront-private LDS slab.
#include <type_traits>
#include "f2f_internal.h"
#include "fp16_split.h"

namespace pmesh {

constexpr int kHKB = 9;                       // texture points per facet covered by one pass of the filter gradient (one wavefront per SIMD: 512 registers)
constexpr int kHFKB = 5;                      // the same per sweep of the forward (two wavefronts per SIMD: 256 registers)
constexpr int kHTKB = 6;                      // and in the texture gradient (bounded by its LDS stage)
constexpr int kHChunk = 4 * 2 * 2 * 64;       // uint4 per LDS buffer: 4 channels x 2 tiles x 2 pieces x 64 lanes
constexpr int kHW = 4;                        // wavefronts per workgroup of the forward: two workgroups share a CU
constexpr int kHFacets = 32 * kHW;            // facets per workgroup
constexpr int kHThreads = 64 * kHW;
constexpr int kHWn = kHChunk / kHThreads;     // uint4 of a filter chunk per thread
constexpr int kHSlab = kHFKB * 8 * 32;         // floats per slab buffer: points x 8 channels x facet slots

__device__ __forceinline__ float4 hld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
template <bool VEC> __device__ __forceinline__ float4 hld4_row(const float *p, int n)
{
    if constexpr (VEC) return n > 0 ? hld4(p) : make_float4(0.f, 0.f, 0.f, 0.f);
    float4 r;
    r.x = n > 0 ? p[0] : 0.f;
    r.y = n > 1 ? p[1] : 0.f;
    r.z = n > 2 ? p[2] : 0.f;
    r.w = n > 3 ? p[3] : 0.f;
    return r;
}
// Features kept in bf16 in HBM (the reduced-precision variant): rows of bf16 values, converted on load and
// rounded to nearest even on store; the arithmetic in between is the one-product fp16 path with fp32 accumulation.
typedef unsigned short bf16_t;
__device__ __forceinline__ float bf16_lo(unsigned u) { return __builtin_bit_cast(float, u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned u) { return __builtin_bit_cast(float, u & 0xFFFF0000u); }
__device__ __forceinline__ unsigned pack2_bf16(float a, float b)              // a in the low half
{
    unsigned r;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float4 hld4(const bf16_t *p)
{
    const uint2 u = *reinterpret_cast<const uint2 *>(p);
    return make_float4(bf16_lo(u.x), bf16_hi(u.x), bf16_lo(u.y), bf16_hi(u.y));
}
template <bool VEC> __device__ __forceinline__ float4 hld4_row(const bf16_t *p, int n)
{
    if constexpr (VEC) return n > 0 ? hld4(p) : make_float4(0.f, 0.f, 0.f, 0.f);
    float4 r;
    r.x = n > 0 ? bf16_lo(p[0]) : 0.f;
    r.y = n > 1 ? bf16_lo(p[1]) : 0.f;
    r.z = n > 2 ? bf16_lo(p[2]) : 0.f;
    r.w = n > 3 ? bf16_lo(p[3]) : 0.f;
    return r;
}
// eight consecutive values of a row (16-byte aligned for bf16, two 16-byte loads for float)
__device__ __forceinline__ void hld8(const float *p, float4 &u, float4 &v) { u = hld4(p); v = hld4(p + 4); }
__device__ __forceinline__ void hld8(const bf16_t *p, float4 &u, float4 &v)
{
    const uint4 w = *reinterpret_cast<const uint4 *>(p);
    u = make_float4(bf16_lo(w.x), bf16_hi(w.x), bf16_lo(w.y), bf16_hi(w.y));
    v = make_float4(bf16_lo(w.z), bf16_hi(w.z), bf16_lo(w.w), bf16_hi(w.w));
}
__device__ __forceinline__ float hld1(const float *p) { return *p; }
// two-byte accesses are slow on this memory path: a single bf16 value is read as the aligned 4 bytes that hold it
// (rows have an even number of values, neighbouring lanes share the word) ...
__device__ __forceinline__ float hld1(const bf16_t *p) { return bf16_lo(*p); }
// element `idx` of an array (even row lengths, 4-byte aligned base), in two steps: the fetch of the word that holds
// it, and its conversion once all fetches of a batch are out (arithmetic right behind a conditional fetch makes the
// wavefront wait for that fetch on the spot)
__device__ __forceinline__ unsigned hld_raw(const float *base, int64_t idx) { return reinterpret_cast<const unsigned *>(base)[idx]; }
__device__ __forceinline__ unsigned hld_raw(const bf16_t *base, int64_t idx) { return reinterpret_cast<const unsigned *>(base)[idx >> 1]; }
__device__ __forceinline__ float hcvt_raw(unsigned w, int, float) { return __builtin_bit_cast(float, w); }
__device__ __forceinline__ float hcvt_raw(unsigned w, int odd, bf16_t) { return odd ? bf16_hi(w) : bf16_lo(w); }
__device__ __forceinline__ void hst1(float *p, float v) { *p = v; }
__device__ __forceinline__ void hst1(bf16_t *p, float v) { *p = (bf16_t)(pack2_bf16(v, 0.f) & 0xFFFFu); }
// ... and neighbouring lanes that hold neighbouring values p[0], p[1] (the even lane the first) write them as one
// 4-byte store.  Every lane calls this; `ok` says whether the pair is stored.
__device__ __forceinline__ void hst1_pair(float *p, float v, bool ok, int lane)
{
    (void)lane;
    if (ok) *p = v;
}
__device__ __forceinline__ void hst1_pair(bf16_t *p, float v, bool ok, int lane)
{
    const float nb = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    if (ok && !(lane & 1)) *reinterpret_cast<unsigned *>(p) = pack2_bf16(v, nb);
}
__device__ __forceinline__ void hst4(float *p, const float4 &v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ void hst4(bf16_t *p, const float4 &v)
{
    *reinterpret_cast<uint2 *>(p) = make_uint2(pack2_bf16(v.x, v.y), pack2_bf16(v.z, v.w));
}

// What a conditional fetch of four consecutive channels leaves in registers, and its conversion to four floats.  The
// two are separate because arithmetic right behind a conditional fetch makes the wavefront wait for that fetch on the
// spot: all fetches of a batch go out first, the conversions follow.
template <typename TIO> struct HRaw4;
template <> struct HRaw4<float> { float4 v; };
template <> struct HRaw4<bf16_t> { uint2 v; };
template <bool VEC> __device__ __forceinline__ HRaw4<float> hld4_raw(const float *p, int n)
{
    HRaw4<float> r;
    r.v = hld4_row<VEC>(p, n);
    return r;
}
template <bool VEC> __device__ __forceinline__ HRaw4<bf16_t> hld4_raw(const bf16_t *p, int n)
{
    HRaw4<bf16_t> r;
    if constexpr (VEC) {
        r.v = n > 0 ? *reinterpret_cast<const uint2 *>(p) : make_uint2(0u, 0u);
    } else {
        r.v.x = (n > 0 ? (unsigned)p[0] : 0u) | (n > 1 ? (unsigned)p[1] << 16 : 0u);
        r.v.y = (n > 2 ? (unsigned)p[2] : 0u) | (n > 3 ? (unsigned)p[3] << 16 : 0u);
    }
    return r;
}
__device__ __forceinline__ HRaw4<float> hraw_zero(float)
{
    HRaw4<float> r;
    r.v = make_float4(0.f, 0.f, 0.f, 0.f);
    return r;
}
__device__ __forceinline__ HRaw4<bf16_t> hraw_zero(bf16_t)
{
    HRaw4<bf16_t> r;
    r.v = make_uint2(0u, 0u);
    return r;
}
__device__ __forceinline__ float4 hcvt4(const HRaw4<float> &r) { return r.v; }
__device__ __forceinline__ float4 hcvt4(const HRaw4<bf16_t> &r)
{
    return make_float4(bf16_lo(r.v.x), bf16_hi(r.v.x), bf16_lo(r.v.y), bf16_hi(r.v.y));
}

__device__ __forceinline__ float absmax4(const float4 &v, float m)
{
    return fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), m));
}

// Eight fp32 values -> one packed fp16x8 piece, rounded to nearest (the first piece of split8h): the operand of the
// half-precision variant, whose products keep fp16's 11 significant bits and accumulate in fp32.
__device__ __forceinline__ void cvt8h(const float (&x)[8], u32x4 &p1)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        unsigned hi;
        asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(hi) : "v"(x[2 * j]), "v"(x[2 * j + 1]));
        p1[j] = hi;
    }
}

// header of the packed filter: {beta, 1/beta}, from max|W| in two steps: up to 256 workgroups leave one maximum
// each in `partial` (the start of the packed-filter area, which the pack kernel overwrites afterwards), one
// workgroup combines them.  A maximum does not depend on the order, so the header is the same from run to run.
__global__ __launch_bounds__(256) void f2f16h2_absmax_k(const float *__restrict__ W, float *__restrict__ partial, int64_t n)
{
    __shared__ float red[4];
    float m = 0.f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) m = fmaxf(m, fabsf(W[i]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__global__ __launch_bounds__(256) void f2f16h2_scale_filter_k(const float *__restrict__ partial, int G, float *__restrict__ hdr)
{
    __shared__ float red[4];
    float m = (int)threadIdx.x < G ? partial[threadIdx.x] : 0.f;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        float inv;
        const float beta = pow2_scale(m, &inv);
        hdr[0] = beta;
        hdr[1] = inv;
    }
}

// hdr <- scale of the n filter values; `scratch` = at least 256 floats that the caller overwrites afterwards
static void filter_scale(const float *W, float *hdr, float *scratch, int64_t n, hipStream_t st)
{
    int G = (int)((n + 4095) / 4096);
    if (G < 1) G = 1;
    if (G > 256) G = 256;
    f2f16h2_absmax_k<<<dim3(G), dim3(256), 0, st>>>(W, scratch, n);
    f2f16h2_scale_filter_k<<<dim3(1), dim3(256), 0, st>>>(scratch, G, hdr);
}

// Filter (Cout, Cin, 16) -> per-lane MFMA B operands: Wp[((ci*NT + nt)*2 + piece)*64 + lane] holds the
// eight fp16 pieces of beta * W[nt*32 + l32][ci][8h .. 8h+7], lane = 32h + l32.  NT = even number of
// 32-channel tiles covering Cout; channels Cin .. CinPad-1 and output channels past Cout are zero.
__global__ __launch_bounds__(kBlock) void f2f16h2_pack_filter_k(const float *__restrict__ W, const float *__restrict__ hdr,
                                                                u32x4 *__restrict__ Wp, int Cin, int CinPad, int Cout, int NT)
{
    const int idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= CinPad * NT * 64) return;
    const int lane = idx & 63, nt = (idx >> 6) % NT, ci = (idx >> 6) / NT;
    const int co = nt * 32 + (lane & 31), h = lane >> 5;
    const float beta = hdr[0];
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = 0.f;
    if (co < Cout && ci < Cin) {
        const float *p = W + ((int64_t)co * Cin + ci) * 16 + 8 * h;
        const float4 u = hld4(p), v = hld4(p + 4);
        x[0] = u.x * beta; x[1] = u.y * beta; x[2] = u.z * beta; x[3] = u.w * beta;
        x[4] = v.x * beta; x[5] = v.y * beta; x[6] = v.z * beta; x[7] = v.w * beta;
    }
    u32x4 p1, p2;
    split8h(x, p1, p2);
    u32x4 *dst = Wp + ((size_t)(ci * NT + nt) * 2) * 64 + lane;
    dst[0] = p1; dst[64] = p2;
}

// A filter chunk (four channels; channel c of the chunk = 2 tiles x 2 pieces x 64 lanes = 256 consecutive uint4)
// straight from global memory into an LDS buffer (no registers in between, so the request can leave a whole chunk
// ahead): lane L of wavefront w delivers element 256 i + 64 w + L of the chunk, the wavefront's 64
// elements land side by side from the wavefront-uniform base in M0.  The data is there after vmcnt has drained.
__device__ __forceinline__ void hw_chunk_to_lds(const u32x4 *__restrict__ Wp, int c0, int NT, int nt0, u32x4 *Wbuf, int wave)
{
#pragma unroll
    for (int i = 0; i < kHWn; ++i) {
        const int e = kHThreads * i + threadIdx.x, c = e >> 8, o = e & 255;
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(Wp + ((size_t)(c0 + c) * NT + nt0) * 128 + o),
            (__attribute__((address_space(3))) void *)(Wbuf + kHThreads * i + 64 * wave), 16, 0, 0);
    }
}

// One pass over all input channels for up to KW texture points per facet.  shs = alpha_f / K_f, the factor on
// the SH values of my facet; slim / tlim = largest |SH value| of my facet / |texture value| of the rows I fetch
// that the scale allows for.  FIRST (the first sweep of the first try) chooses them itself from what it fetches
// anyway -- the SH rows of its points and the first eight channels of their texture rows, with 2^7 of head room --
// and leaves 1 / alpha_f in s_inv; the later sweeps take them from there.  Nothing of that leaves the wavefront.
template <int KW, bool TVEC, bool HALF, bool FIRST, typename TIO>
__device__ __forceinline__ void h2_sweep(const TIO *__restrict__ tex, const u32x4 *__restrict__ Wp,
                                         const float *__restrict__ sh, u32x4 *Ws, float *slab, f32x16 (&acc)[2],
                                         int kbase, int Ks, int K, float &shs, float &slim, float &tlim, bool &viol,
                                         const int *s_k0, const int *s_K, float *s_tl, float *s_inv, int sweep, int Cin,
                                         int NT, int nt0, int nblk, int w, int lane, int h
                                         )
{
    const int l32 = lane & 31;
    // rows this lane fetches for the slab: load i covers point i of facet slot lane/2, channels 4*(lane%2) .. +3 of the group
    const int cg4 = 4 * (lane & 1);
    unsigned ldoff[KW];
    bool ldok[KW];
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        const int slot = w * 32 + (lane >> 1), kk = sweep * kHFKB + i;
        ldok[i] = kk < s_K[slot];
        ldoff[i] = (unsigned)(s_k0[slot] + (ldok[i] ? kk : 0)) * (unsigned)Cin + cg4;
    }
    HRaw4<TIO> pf[KW];
    auto fetch_group = [&](int g) {
#pragma unroll
        for (int i = 0; i < KW; ++i)
            pf[i] = ldok[i] ? hld4_raw<TVEC>(tex + (ldoff[i] + 8 * g), Cin - (8 * g + cg4)) : hraw_zero(TIO());
    };
    auto publish_group = [&](float *dst) {
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < KW; ++i) {
            float *q = dst + (i * 8 + cg4) * 32 + (lane >> 1);
            const float4 pv = hcvt4(pf[i]);
            q[0] = pv.x; q[32] = pv.y; q[64] = pv.z; q[96] = pv.w;
            m = absmax4(pv, m);
        }
        viol |= m > tlim;
    };
    const int wave_u = __builtin_amdgcn_readfirstlane(w);
    // All requests of the set-up leave before any of them is waited for: the first filter chunk straight into its
    // buffer (free since the barrier that ended the sweep before), the first texture group and the SH rows through
    // registers.
    hw_chunk_to_lds(Wp, 0, NT, nt0, Ws, wave_u);
    fetch_group(0);
    float4 su[KW], sv[KW];
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) {
        su[kk] = make_float4(0.f, 0.f, 0.f, 0.f);
        sv[kk] = su[kk];
        if (kk < Ks) {
            const float *p = sh + (int64_t)(kbase + kk) * 16 + 8 * h;
            su[kk] = hld4(p);
            sv[kk] = hld4(p + 4);
        }
    }
    float smx = 0.f;
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) smx = absmax4(su[kk], absmax4(sv[kk], smx));
    if constexpr (FIRST) {
        float tm = 0.f;
#pragma unroll
        for (int i = 0; i < KW; ++i) tm = absmax4(hcvt4(pf[i]), tm);
        tm = fmaxf(tm, __builtin_bit_cast(float, hdpp<0xB1>(__builtin_bit_cast(int, tm))));      // the lane pair of a slot
        float sm = fmaxf(smx, __shfl_xor(smx, 32, 64));                                         // both halves of a facet
        tm *= 8.0f;
        sm *= 16.0f;
        slim = sm;
        tlim = tm;
        if (!(lane & 1)) s_tl[w * 32 + (lane >> 1)] = tm;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float inv;
        const float al = pow2_scale(s_tl[w * 32 + l32] * sm, &inv);
        if (h == 0) s_inv[w * 32 + l32] = inv;
        shs = K > 0 ? al / (float)K : 0.f;
    }
    // values past the limits the facet's scale was chosen for are recorded, not acted on here
    viol |= smx > slim;
    float shr[KW][8];
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) {
        shr[kk][0] = su[kk].x * shs; shr[kk][1] = su[kk].y * shs; shr[kk][2] = su[kk].z * shs; shr[kk][3] = su[kk].w * shs;
        shr[kk][4] = sv[kk].x * shs; shr[kk][5] = sv[kk].y * shs; shr[kk][6] = sv[kk].z * shs; shr[kk][7] = sv[kk].w * shs;
    }
    publish_group(slab);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    auto read_b = [&](u32x4 (&b)[2][2], int buf, int cl) { // filter pieces of channel cl of the chunk in buffer buf
        const u32x4 *Wc = Ws + buf * kHChunk + cl * 256 + lane;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int p = 0; p < 2; ++p) b[t][p] = Wc[(t * 2 + p) * 64];
    };
    auto read_tv = [&](float (&tv)[KW], int c) {          // my facet's texture values of channel c
        const float *sl = slab + ((c >> 3) & 1) * kHSlab + (c & 7) * 32 + l32;
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) tv[kk] = sl[kk * 8 * 32];
    };
    auto gen = [&](float (&a)[8], const float (&tv)[KW]) {
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            float v = 0.f;
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) v = fmaf(tv[kk], shr[kk][s], v);
            a[s] = v;
        }
    };

    // software pipeline over channels: while channel c is multiplied, the G values of c+1 are generated and
    // split, and the LDS reads for c+1 (filter) and c+2 (texture) are in flight
    u32x4 pa[2], b[2][2];
    float tvn[KW];
    {
        float tv0[KW], a[8];
        read_tv(tv0, 0);
        read_tv(tvn, 1);
        read_b(b, 0, 0);
        gen(a, tv0);
        if constexpr (HALF) cvt8h(a, pa[0]);
        else split8h(a, pa[0], pa[1]);
    }
    // filter chunks alternate between two LDS buffers: chunk j+1 is requested at the start of chunk j and has landed
    // at its end; the first channel of a chunk reads its pieces right after the barrier, under the generation
    // and split of the channel after it
    for (int j = 0; j < nblk; ++j) {
        const int g = j >> 1, wb = j & 1;
        const bool wmore = j + 1 < nblk;
        const bool stage = !(j & 1) && 8 * (g + 1) < Cin;       // even chunk: bring in the next 8-channel group
        if (wmore) hw_chunk_to_lds(Wp, 4 * (j + 1), NT, nt0, Ws + (wb ^ 1) * kHChunk, wave_u);   // nobody reads that buffer during this chunk
        if (stage) fetch_group(g + 1);
#pragma unroll
        for (int ci_l = 0; ci_l < 4; ++ci_l) {
            const int c = 4 * j + ci_l;
            u32x4 bn[2][2];
            float tvnn[KW];
            if (ci_l < 3) read_b(bn, wb, ci_l + 1);
            read_tv(tvnn, c + 2);

            float an[8];
            gen(an, tvn);
            u32x4 pn[2];
            if constexpr (HALF) {
                cvt8h(an, pn[0]);
                pn[1] = pn[0];
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_f16(pa[0], b[t][0], acc[t]);
            } else {
                split8h(an, pn[0], pn[1]);
                // three piece products per accumulator tile, smallest first
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_f16(pa[1], b[t][0], acc[t]);
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_f16(pa[0], b[t][1], acc[t]);
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_f16(pa[0], b[t][0], acc[t]);
                // order asked of the scheduler for this channel: each of the six products followed by six vector
                // instructions and an LDS read (left to itself it bunches the products: 2 % slower)
#pragma unroll
                for (int q = 0; q < 6; ++q) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            }

            pa[0] = pn[0]; pa[1] = pn[1];
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) tvn[kk] = tvnn[kk];
            if (ci_l < 3) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int p = 0; p < 2; ++p) b[t][p] = bn[t][p];
            }
        }
        if (wmore) __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): the next chunk has landed in its buffer
        if (stage) publish_group(slab + ((g + 1) & 1) * kHSlab);
        __syncthreads();
        if (wmore) read_b(b, wb ^ 1, 0);
    }
}

template <bool TVEC, bool HALF, typename TIO>
__global__ __launch_bounds__(kHThreads, 2) void f2f16h2_fwd_k(const TIO *__restrict__ tex, const float *__restrict__ hdr,
                                                              const u32x4 *__restrict__ Wp, const float *__restrict__ sh,
                                                              const int *__restrict__ cum, const int *__restrict__ order,
                                                              TIO *__restrict__ out, int64_t Nf, int T, int Cin,
                                                              int Cout, int NT, F2FTail tail)
{
    __shared__ u32x4 Ws[2 * kHChunk];
    __shared__ __attribute__((aligned(16))) float s_slab[kHW * 2 * kHSlab];      // per wavefront: two buffers
    __shared__ int s_f[kHFacets], s_k0[kHFacets], s_K[kHFacets], s_kmax[kHFacets / 64];
    __shared__ float s_inv[kHFacets], s_tl[kHFacets];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int64_t s0 = (int64_t)blockIdx.x * kHFacets;
    const int nt0 = blockIdx.y * 2, n0 = blockIdx.y * 64;
    const int nblk = (Cin + 3) >> 2;
    const float ibeta = hdr[1];                      // (needed by the stores at the end: asked for here, not there)

    static_assert(kHFacets <= kHThreads && kHFacets % 64 == 0, "one descriptor per thread of the first wavefronts");
    if (threadIdx.x < kHFacets) {
        const int i = threadIdx.x;
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
        const int km = hwave_max(b > a ? b - a : 0);            // (whole wavefronts are in here)
        if (lane == 0) s_kmax[w] = km;
    }
    __syncthreads();
    const int k0 = s_k0[w * 32 + l32], K = s_K[w * 32 + l32];
    int kmax_wg = 0;
#pragma unroll
    for (int i = 0; i < kHFacets / 64; ++i) kmax_wg = max(kmax_wg, s_kmax[i]);

    // Scale of each facet's G.  First try: a bound from the first eight channels of the points of the first sweep
    // (which that sweep works out itself from its first fetches), with 2^7 of head room; the sweeps check every
    // value they fetch against it.  If any facet of the workgroup exceeds its bound, everything is done again
    // with the exact maxima from a scan of all rows (which costs a second pass over the texture rows).
    f32x16 acc[2];
    for (int attempt = 0;; ++attempt) {
        const bool full = attempt > 0;
        float slim = 0.f, tlim = 0.f, shs = 0.f;
        if (full) {
            const int slot = w * 32 + (lane >> 1), cg4 = 4 * (lane & 1);
            const int rk0 = s_k0[slot], rK = s_K[slot];
            // all loads of a batch are issued before the first comparison
            const int rKmax = hwave_max(rK), Kmax = hwave_max(K);
            float sm = 0.f, tm = 0.f;
            for (int kb = 0; kb < Kmax; kb += 4) {
                float4 u[4][2];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float *p = sh + (int64_t)(k0 + kb + i) * 16 + 8 * h;
                    const bool ok = kb + i < K;
                    u[i][0] = ok ? hld4(p) : make_float4(0.f, 0.f, 0.f, 0.f);
                    u[i][1] = ok ? hld4(p + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) sm = absmax4(u[i][0], absmax4(u[i][1], sm));
            }
            for (int kb = 0; kb < rKmax; kb += 4)
                for (int cb = 0; cb < Cin; cb += 32) {
                    HRaw4<TIO> v[4][4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int c = cb + 8 * g + cg4;
                            v[i][g] = (kb + i < rK && c < Cin) ? hld4_raw<TVEC>(tex + (int64_t)(rk0 + kb + i) * Cin + c, Cin - c)
                                                              : hraw_zero(TIO());
                        }
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int g = 0; g < 4; ++g) tm = absmax4(hcvt4(v[i][g]), tm);
                }
            tm = fmaxf(tm, __shfl_xor(tm, 1, 64));
            sm = fmaxf(sm, __shfl_xor(sm, 32, 64));
            slim = sm;
            tlim = tm;
            if (!(lane & 1)) s_tl[slot] = tm;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            float inv;
            const float al = pow2_scale(s_tl[w * 32 + l32] * sm, &inv);
            if (h == 0) s_inv[w * 32 + l32] = inv;
            shs = K > 0 ? al / (float)K : 0.f;
        }
        const int nsweeps = (kmax_wg + kHFKB - 1) / kHFKB;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
        bool viol = false;
        for (int sw = 0; sw < nsweeps; ++sw) {
            const int kbase = k0 + sw * kHFKB;
            const int rem = K - sw * kHFKB;
            const int Ks = rem < 0 ? 0 : (rem > kHFKB ? kHFKB : rem);
            // every variant runs the same barriers, so wavefronts of a workgroup may pick different ones
            const int kw = hwave_max(Ks);
#define PM_H2(N, FIRST) h2_sweep<N, TVEC, HALF, FIRST, TIO>(tex, Wp, sh, Ws, s_slab + w * 2 * kHSlab, acc, kbase, Ks, K, shs, slim, tlim, viol, s_k0, s_K, s_tl, s_inv, sw, Cin, NT, nt0, nblk, w, lane, h)
            if (!full && sw == 0) {
                if (kw <= 1) PM_H2(1, true);
                else if (kw == 2) PM_H2(2, true);
                else if (kw == 3) PM_H2(3, true);
                else if (kw == 4) PM_H2(4, true);
                else PM_H2(5, true);
            } else {
                if (kw <= 1) PM_H2(1, false);
                else if (kw == 2) PM_H2(2, false);
                else if (kw == 3) PM_H2(3, false);
                else if (kw == 4) PM_H2(4, false);
                else PM_H2(5, false);
            }
#undef PM_H2
        }
        if (full || !__syncthreads_or(viol ? 1 : 0)) break;
    }

    // what rides on the store: bias, ReLU (and its mask as bits), a per-channel scale and shift
    float tb[2], tsc[2], tsf[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int co = n0 + t * 32 + l32;
        const bool cok = co < Cout;
        tb[t] = (tail.bias && cok) ? tail.bias[co] : 0.f;
        tsc[t] = (tail.scale && cok) ? tail.scale[co] : 1.f;
        tsf[t] = (tail.shift && cok) ? tail.shift[co] : 0.f;
    }
    const bool plain = !tail.bias && !tail.scale && !tail.shift && !tail.relu;
    // facets and scales of my 16 rows (four runs of four slots), read before the first store goes out
    int frow[16];
    float urow[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int slot = w * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        frow[i] = s_f[slot];
        urow[i] = s_inv[slot];
    }
    // the common case without any condition on a store: float rows, nothing riding on them, all of the wavefront's
    // rows and columns present
    if constexpr (std::is_same<TIO, float>::value) {
        bool mine = true;
#pragma unroll
        for (int i = 0; i < 16; ++i) mine = mine && frow[i] >= 0 && frow[i] < Nf;
        if (plain && n0 + 64 <= Cout && __builtin_amdgcn_ballot_w64(mine) == ~0ull) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float *rowp = out + ((int64_t)frow[i] * Cout + n0 + l32);
                const float us = urow[i] * ibeta;
                rowp[0] = acc[0][i] * us;
                rowp[32] = acc[1][i] * us;
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int fr = frow[i];
        const bool rok = fr >= 0 && fr < Nf;
        const float us = urow[i] * ibeta;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int co = n0 + t * 32 + l32;
            float v = acc[t][i] * us;
            if (!plain) {
                v += tb[t];
                if (tail.relu) v = fmaxf(v, 0.f);
                if (tail.bits) {
                    // the 32 lanes of a half are the 32 channels of one mask word of its facet
                    const unsigned long long m = __builtin_amdgcn_ballot_w64(v > 0.f && co < Cout);
                    if (l32 == 0 && rok && n0 + 32 * t < Cout) tail.bits[(int64_t)fr * (Cout >> 5) + ((n0 >> 5) + t)] = (unsigned)(m >> (32 * h));
                }
                v = v * tsc[t] + tsf[t];
            }
            hst1_pair(out + ((int64_t)(rok ? fr : 0) * Cout + co), v, rok && co < Cout, l32);
        }
    }
}

// workspace: 16-byte header {beta, 1/beta, -, -}, then the packed filter
size_t f2f16h2_fwd_workspace_bytes(int Cin, int Cout)
{
    const int NT = 2 * ((Cout + 63) / 64), CinPad = (Cin + 3) & ~3;
    return 16 + (size_t)CinPad * NT * 2 * 64 * sizeof(u32x4);
}

int f2f16h2_fwd(const void *tex_, const float *W, const float *sh, const int *cum, const int *order, void *out_,
                void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st, bool half,
                bool bf16, const F2FTail *tail)
{
    const int NT = 2 * ((Cout + 63) / 64);
    const F2FTail tl = tail ? *tail : F2FTail{nullptr, nullptr, nullptr, nullptr, 0};
    PM_REQUIRE(!tl.bits || (!bf16 && Cout % 32 == 0), "f2f_fwd: the bit mask needs float features and a multiple of 32 output channels");
    PM_REQUIRE(T * Cin < (int64_t(1) << 31), "f2f_fwd: texture array too large for 32-bit offsets");
    PM_REQUIRE(workspace && workspace_bytes >= f2f16h2_fwd_workspace_bytes(Cin, Cout),
               "f2f_fwd: workspace too small (%zu bytes)", workspace_bytes);
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0, "f2f_fwd: workspace must be 16-byte aligned");
    float *hdr = (float *)workspace;
    u32x4 *Wp = (u32x4 *)workspace + 1;
    filter_scale(W, hdr, (float *)Wp, (int64_t)Cout * Cin * 16, st);
    PM_LAUNCHED("f2f_fwd(scale)");
    const int CinPad = (Cin + 3) & ~3, n = CinPad * NT * 64;
    f2f16h2_pack_filter_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(W, hdr, Wp, Cin, CinPad, Cout, NT);
    PM_LAUNCHED("f2f_fwd(pack)");
    const int64_t gx = ceil_div(Nf, kHFacets), gy = NT / 2;
    PM_REQUIRE(grid_ok(gx) && gy <= 65535, "f2f_fwd: grid too large");
#define PM_FWD(V, H, TIO) f2f16h2_fwd_k<V, H, TIO><<<dim3((unsigned)gx, (unsigned)gy), dim3(kHThreads), 0, st>>>((const TIO *)tex_, hdr, Wp, sh, cum, order, (TIO *)out_, Nf, (int)T, Cin, Cout, NT, tl)
    if (bf16) {
        // bf16 features: the one-product kernels, rows read eight bytes at a time
        PM_REQUIRE(!(Cin & 3) && !(Cout & 1) && !(reinterpret_cast<uintptr_t>(tex_) & 7u) && !(reinterpret_cast<uintptr_t>(out_) & 3u),
                   "f2f_fwd: bf16 features need a multiple of 4 input channels, an even number of output channels and aligned rows");
        PM_FWD(true, true, bf16_t);
    } else {
        const bool tvec = !(Cin & 3) && !(reinterpret_cast<uintptr_t>(tex_) & 15u);
        if (tvec && half) PM_FWD(true, true, float);
        else if (tvec) PM_FWD(true, false, float);
        else if (half) PM_FWD(false, true, float);
        else PM_FWD(false, false, float);
    }
#undef PM_FWD
    PM_LAUNCHED("f2f_fwd");
    return 0;
}

// ----------------------------------------------------------------------------------------
// texture gradient on the fp16 matrix cores, same decomposition as the three-piece bf16 kernel:
//     H[f, ci, d] = sum_co gout[f, co] W[co, ci, d]          (two-piece fp16 MFMAs, k = co)
//     gtex[t, ci] = (1/K_f) sum_d sh[t, d] H[f, ci, d]       (FMAs on the accumulator registers)
// The product is taken transposed, D[(ci,d)][f] = (beta W)^T . (gamma_f gout_f)^T with gamma_f from the
// exact maximum of the facet's gout row (the lane holds it); 1 / (beta gamma_f K_f) rides on the SH values
// of the contraction.  A tile tt = 4g + q holds the two input channels 8g + q ("a") and 8g + 4 + q ("b");
// register i of a lane (facet l32, half h)  <->  channel (i/4)%2,  d = 8(i/8) + 4h + i%4.
constexpr int kHTChunkMax = 2 * 4 * 2 * 64;      // uint4 per chunk buffer: 2 tiles x 4 k-steps x 2 pieces x 64 lanes

// W (Cout, Cin, 16) -> A operands of the transposed product:
// WpT[((tt*NKS + ks)*2 + piece)*64 + lane] = pieces of beta * W[co0 + 16ks + 8h .. +7][ci(tt, r)][d(r)], r = lane % 32
__global__ __launch_bounds__(kBlock) void f2f16h2_pack_filter_t_k(const float *__restrict__ W, const float *__restrict__ hdr,
                                                                  u32x4 *__restrict__ WpT, int Cin, int Cout, int NTt,
                                                                  int NKS, int co0)
{
    const int idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= NTt * NKS * 64) return;
    const int lane = idx & 63, ks = (idx >> 6) % NKS, tt = (idx >> 6) / NKS;
    const int r = lane & 31, h = lane >> 5;
    // row r = 8q + 4h' + j of the tile (h' = accumulator half, register 4q + j): channel q%2, d = 8(q/2) + 4h' + j
    const int ci = 8 * (tt >> 2) + 4 * ((r >> 3) & 1) + (tt & 3), d = 8 * (r >> 4) + 4 * ((r >> 2) & 1) + (r & 3);
    const float beta = hdr[0];
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int co = co0 + 16 * ks + 8 * h + j;             // this launch covers channels co0 .. co0 + 16 NKS - 1
        x[j] = (ci < Cin && co < Cout) ? beta * W[((int64_t)co * Cin + ci) * 16 + d] : 0.f;
    }
    u32x4 p1, p2;
    split8h(x, p1, p2);
    u32x4 *dst = WpT + ((size_t)(tt * NKS + ks) * 2) * 64 + lane;
    dst[0] = p1; dst[64] = p2;
}

// FIRST (the first sweep) also turns the facet's gout row x, which the kernel has asked for, into the operand
// pieces bp and the factor shs -- after its own requests have left, so that the two round trips overlap.
template <int KW, int NKS, bool GVEC, bool HALF, bool FIRST, typename TIO>
__device__ __forceinline__ void h2_tex_sweep(const u32x4 *__restrict__ WpT, const float *__restrict__ sh,
                                             TIO *__restrict__ gtex, u32x4 *Ws, float *stage, const int *w_k0,
                                             const int *w_K, float (*x)[8], u32x4 (&bp)[NKS][2], int kbase, int Ks,
                                             int K, float ibeta, float &shs, int sweep, int Cin, int NG, bool add, int lane,
                                             int h
                                             )
{
    constexpr int chunk = 2 * NKS * 128;         // uint4 per chunk of two tiles
    constexpr int NWF = (chunk + 511) / 512;     // uint4 fetched per thread
    const int nchunks = 2 * NG;
    auto chunk_fetch = [&](u32x4 (&wn)[NWF], int c) {
#pragma unroll
        for (int i = 0; i < NWF; ++i) {
            const int e = threadIdx.x + 512 * i;
            if (e < chunk) wn[i] = WpT[(size_t)c * chunk + e];
        }
    };
    auto chunk_publish = [&](const u32x4 (&wn)[NWF], int c) {
#pragma unroll
        for (int i = 0; i < NWF; ++i) {
            const int e = threadIdx.x + 512 * i;
            if (e < chunk) Ws[(c % 3) * kHTChunkMax + e] = wn[i];
        }
    };
    // All requests of the set-up leave before any of them is waited for: the first two filter chunks and the SH rows.
    u32x4 wn[NWF], wn1[NWF];
    chunk_fetch(wn, 0);
    chunk_fetch(wn1, 1);
    // SH values of my facet's points for my half's eight d's (4h..4h+3, 8+4h..8+4h+3), times shs = 1 / (K gamma beta):
    // the scales of the two operands leave with the contraction
    float4 su[KW], sv[KW];
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) {
        su[kk] = make_float4(0.f, 0.f, 0.f, 0.f);
        sv[kk] = su[kk];
        if (kk < Ks) {
            const float *p = sh + (int64_t)(kbase + kk) * 16 + 4 * h;
            su[kk] = hld4(p);
            sv[kk] = hld4(p + 8);
        }
    }
    if constexpr (FIRST) {
        // my facet's gout row, scaled by gamma_f = a power of two that brings its largest element below 2^14, as B
        // operand pieces: k-step ks, half h <-> channels 16ks + 8h .. + 7
        float gm = 0.f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) gm = fmaxf(gm, fabsf(x[ks][j]));
        gm = fmaxf(gm, __shfl_xor(gm, 32, 64));
        float igamma;
        const float gamma = pow2_scale(gm, &igamma);
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
            for (int j = 0; j < 8; ++j) x[ks][j] *= gamma;
            float xs[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) xs[j] = x[ks][j];
            split8h(xs, bp[ks][0], bp[ks][1]);
        }
        shs = K > 0 ? igamma * ibeta / (float)K : 0.f;
    }
    float shr[KW][8];
#pragma unroll
    for (int kk = 0; kk < KW; ++kk) {
        shr[kk][0] = su[kk].x * shs; shr[kk][1] = su[kk].y * shs; shr[kk][2] = su[kk].z * shs; shr[kk][3] = su[kk].w * shs;
        shr[kk][4] = sv[kk].x * shs; shr[kk][5] = sv[kk].y * shs; shr[kk][6] = sv[kk].z * shs; shr[kk][7] = sv[kk].w * shs;
    }
    chunk_publish(wn, 0);
    chunk_publish(wn1, 1);
    __syncthreads();

    // 16-channel block gp of the stage -> global memory
    auto flush = [&](int gp) {
        const int ci = 16 * gp + 4 * (lane & 3);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int slot = 16 * i + (lane >> 2);
            const int k0s = w_k0[slot] + sweep * kHTKB, Kss = w_K[slot] - sweep * kHTKB;
#pragma unroll
            for (int kk = 0; kk < KW; ++kk)
                if (kk < Kss && ci < Cin) {
                    const float4 v = *reinterpret_cast<const float4 *>(stage + (kk * 32 + slot) * 16 + 4 * (lane & 3));
                    TIO *dst = gtex + (int64_t)(k0s + kk) * Cin + ci;
                    // `add`: a later block of 64 output channels accumulates onto what the earlier ones wrote
                    if constexpr (GVEC) {
                        float4 o = v;
                        if (add) {
                            const float4 p = hld4(dst);
                            o = make_float4(p.x + v.x, p.y + v.y, p.z + v.z, p.w + v.w);
                        }
                        hst4(dst, o);
                    } else {                               // channel count not a multiple of 4 / unaligned rows
                        hst1(dst, add ? hld1(dst) + v.x : v.x);
                        if (ci + 1 < Cin) hst1(dst + 1, add ? hld1(dst + 1) + v.y : v.y);
                        if (ci + 2 < Cin) hst1(dst + 2, add ? hld1(dst + 2) + v.z : v.z);
                        if (ci + 3 < Cin) hst1(dst + 3, add ? hld1(dst + 3) + v.w : v.w);
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
            const u32x4 *Wc = Ws + (c % 3) * kHTChunkMax + lane;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                // H tile of two input channels: rows (d half, channel, d), columns = my wavefront's facets
                f32x16 acc0;
#pragma unroll
                for (int i = 0; i < 16; ++i) acc0[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    u32x4 a[2];
#pragma unroll
                    for (int p = 0; p < 2; ++p) a[p] = Wc[((u * NKS + ks) * 2 + p) * 64];
                    // three piece products, smallest first (half-precision variant: the product of the first pieces)
                    if constexpr (!HALF) {
                        acc0 = mfma_f16(a[1], bp[ks][0], acc0);
                        acc0 = mfma_f16(a[0], bp[ks][1], acc0);
                    }
                    acc0 = mfma_f16(a[0], bp[ks][0], acc0);
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
template <int NKS, bool GVEC, bool HALF, typename TIN, typename TIO>
__global__ __launch_bounds__(512, 1) void f2f16h2_bwd_tex_k(const TIN *__restrict__ gout,
                                                            const float *__restrict__ hdr,
                                                            const u32x4 *__restrict__ WpT,
                                                            const float *__restrict__ sh,
                                                            const int *__restrict__ cum,
                                                            const int *__restrict__ order, TIO *__restrict__ gtex,
                                                            int64_t Nf, int T, int Cin, int Cout, int NG, int co0,
                                                            int onto)
{
    __shared__ u32x4 Ws[3 * kHTChunkMax];
    __shared__ __attribute__((aligned(16))) float s_stage[8][kHTKB * 32 * 16];
    __shared__ int s_k0[8][32], s_K[8][32], s_kmax[8];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const float ibeta = hdr[1];                      // (used after the first fetches have come back)

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
    if (h == 0) {
        s_k0[w][l32] = k0;
        s_K[w][l32] = K;
    }
    {
        const int km = hwave_max(K);
        if (lane == 0) s_kmax[w] = km;
    }
    // my facet's gout row (the 16 NKS channels of this launch): asked for here, used by the first sweep
    float x[NKS][8];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[ks][j] = 0.f;
        const int co = co0 + 16 * ks + 8 * h;
        if (K > 0 && co < Cout) {
            float4 u, v;
            hld8(gout + ((int64_t)f * Cout + co), u, v);
            x[ks][0] = u.x; x[ks][1] = u.y; x[ks][2] = u.z; x[ks][3] = u.w;
            x[ks][4] = v.x; x[ks][5] = v.y; x[ks][6] = v.z; x[ks][7] = v.w;
        }
    }
    u32x4 bp[NKS][2];
    float shs = 0.f;
    // The first sweep starts without a barrier in front (which would wait for the gout rows): every workgroup runs
    // it, and the barrier of its set-up is the one that makes the wavefronts' point counts visible to all.
#define PM_H2T(N, FIRST, X) h2_tex_sweep<N, NKS, GVEC, HALF, FIRST, TIO>(WpT, sh, gtex, Ws, s_stage[w], s_k0[w], s_K[w], X, bp, kbase, Ks, K, ibeta, shs, sw, Cin, NG, co0 > 0 || onto, lane, h)
    {
        const int sw = 0, kbase = k0;
        const int Ks = K > kHTKB ? kHTKB : K;
        const int kw = hwave_max(Ks);
        // every variant runs the same barriers, so wavefronts of a workgroup may pick different ones
        if (kw <= 1) PM_H2T(1, true, x);
        else if (kw == 2) PM_H2T(2, true, x);
        else if (kw == 3) PM_H2T(3, true, x);
        else if (kw == 4) PM_H2T(4, true, x);
        else if (kw == 5) PM_H2T(5, true, x);
        else PM_H2T(6, true, x);
    }
    int kmax_wg = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) kmax_wg = max(kmax_wg, s_kmax[i]);
    const int nsweeps = (kmax_wg + kHTKB - 1) / kHTKB;
    for (int sw = 1; sw < nsweeps; ++sw) {
        const int rem = K - sw * kHTKB;
        const int Ks = rem < 0 ? 0 : (rem > kHTKB ? kHTKB : rem);
        const int kw = hwave_max(Ks);
        const int kbase = k0 + sw * kHTKB;
        float (*none)[8] = nullptr;
        if (kw <= 1) PM_H2T(1, false, none);
        else if (kw == 2) PM_H2T(2, false, none);
        else if (kw == 3) PM_H2T(3, false, none);
        else if (kw == 4) PM_H2T(4, false, none);
        else if (kw == 5) PM_H2T(5, false, none);
        else PM_H2T(6, false, none);
    }
#undef PM_H2T
}


// workspace: 16-byte header {beta, 1/beta, -, -}, then the packed W^T of one block of at most 64 output channels
size_t f2f16h2_bwd_texture_workspace_bytes(int Cin, int Cout)
{
    const int NG = (Cin + 7) / 8, NKS = Cout <= 32 ? 2 : 4;
    return 16 + (size_t)NG * 4 * NKS * 2 * 64 * sizeof(u32x4);
}

// bf16 features and more than 64 output channels: the blocks of 64 output channels accumulate in a float32 copy of
// grad_texture behind the packed filter (a bf16 running sum would be rounded once per block), converted at the end
size_t f2f16h2_bwd_texture_bf16_workspace_bytes(int64_t T, int Cin, int Cout)
{
    const size_t base = (f2f16h2_bwd_texture_workspace_bytes(Cin, Cout) + 255) & ~(size_t)255;
    return Cout > 64 ? base + (size_t)T * Cin * sizeof(float) : base;
}

__global__ __launch_bounds__(kBlock) void f2f16h2_rows_to_bf16_k(const float *__restrict__ src, bf16_t *__restrict__ dst,
                                                                 const int *__restrict__ cum, int64_t Nf, int T, int Cin)
{
    int last = cum[Nf - 1];
    last = last < 0 ? 0 : (last > T ? T : last);
    const int64_t n4 = (int64_t)last * Cin / 4;                   // Cin is a multiple of 4
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += (int64_t)gridDim.x * kBlock)
        hst4(dst + 4 * i, hld4(src + 4 * i));
}

int f2f16h2_bwd_texture(const void *gout_, const float *W, const float *sh, const int *cum, const int *order,
                        void *gtex_, void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                        int Cout, hipStream_t st, bool half, bool bf16, bool onto)
{
    // onto: the result is added to what grad_texture holds (every block of output channels then adds, the first too)
    const int NG = (Cin + 7) / 8;
    PM_REQUIRE(workspace && workspace_bytes >= f2f16h2_bwd_texture_workspace_bytes(Cin, Cout),
               "f2f_bwd_texture: workspace too small (%zu bytes)", workspace_bytes);
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0, "f2f_bwd_texture: workspace must be 16-byte aligned");
    float *hdr = (float *)workspace;
    u32x4 *WpT = (u32x4 *)workspace + 1;
    filter_scale(W, hdr, (float *)WpT, (int64_t)Cout * Cin * 16, st);
    PM_LAUNCHED("f2f_bwd_texture(scale)");
    const int64_t gx = ceil_div(Nf, 256);
    PM_REQUIRE(grid_ok(gx), "f2f_bwd_texture: grid too large");
    const bool gvec = !(Cin & 3) && !(reinterpret_cast<uintptr_t>(gtex_) & (bf16 ? 7u : 15u));
    PM_REQUIRE(!bf16 || (gvec && !(Cout & 7) && !(reinterpret_cast<uintptr_t>(gout_) & 15u)),
               "f2f_bwd_texture: bf16 features need Cin %% 4 == 0, Cout %% 8 == 0 and 16-byte aligned rows");
    float *gtex32 = nullptr;
    if (bf16 && Cout > 64) {
        PM_REQUIRE(workspace_bytes >= f2f16h2_bwd_texture_bf16_workspace_bytes(T, Cin, Cout),
                   "f2f_bwd_texture: workspace too small (%zu bytes) for bf16 features and more than 64 output channels", workspace_bytes);
        gtex32 = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) +
                                           ((f2f16h2_bwd_texture_workspace_bytes(Cin, Cout) + 255) & ~(size_t)255));
    }
    // output channels go 64 at a time; the first block writes grad_texture, the others add to it
    // (launches on one stream run in order, so the packed filter buffer is reused)
    for (int co0 = 0; co0 < Cout; co0 += 64) {
        const int NKS = Cout - co0 <= 32 ? 2 : 4;
        const int n = NG * 4 * NKS * 64;
        f2f16h2_pack_filter_t_k<<<dim3((unsigned)ceil_div(n, kBlock)), dim3(kBlock), 0, st>>>(W, hdr, WpT, Cin, Cout, NG * 4, NKS, co0);
        PM_LAUNCHED("f2f_bwd_texture(pack)");
#define PM_TEX(N, G, H, TIN, TIO, DST) f2f16h2_bwd_tex_k<N, G, H, TIN, TIO><<<dim3((unsigned)gx), dim3(512), 0, st>>>((const TIN *)gout_, hdr, WpT, sh, cum, order, (TIO *)(DST), Nf, (int)T, Cin, Cout, NG, co0, onto ? 1 : 0)
        if (bf16 && gtex32) {
            if (NKS == 2) PM_TEX(2, true, true, bf16_t, float, gtex32);
            else PM_TEX(4, true, true, bf16_t, float, gtex32);
        } else if (bf16) {
            if (NKS == 2) PM_TEX(2, true, true, bf16_t, bf16_t, gtex_);
            else PM_TEX(4, true, true, bf16_t, bf16_t, gtex_);
        } else if (half) {
            if (NKS == 2 && gvec) PM_TEX(2, true, true, float, float, gtex_);
            else if (NKS == 2) PM_TEX(2, false, true, float, float, gtex_);
            else if (gvec) PM_TEX(4, true, true, float, float, gtex_);
            else PM_TEX(4, false, true, float, float, gtex_);
        } else {
            if (NKS == 2 && gvec) PM_TEX(2, true, false, float, float, gtex_);
            else if (NKS == 2) PM_TEX(2, false, false, float, float, gtex_);
            else if (gvec) PM_TEX(4, true, false, float, float, gtex_);
            else PM_TEX(4, false, false, float, float, gtex_);
        }
#undef PM_TEX
        PM_LAUNCHED("f2f_bwd_texture");
    }
    if (gtex32) {
        f2f16h2_rows_to_bf16_k<<<dim3(1024), dim3(kBlock), 0, st>>>(gtex32, (bf16_t *)gtex_, cum, Nf, (int)T, Cin);
        PM_LAUNCHED("f2f_bwd_texture(convert)");
    }
    return 0;
}

// ----------------------------------------------------------------------------------------
// filter gradient gW = gout^T . G on the fp16 matrix cores, same decomposition as the three-piece bf16
// kernel: G is formed as in the forward (lane = facet, eight d's in registers), split into two fp16 pieces,
// and each piece is transposed by the matrix core itself (D = piece . E with a 0/1 selection matrix is
// exact), which leaves lane = column (channel, d) and registers = facets -- the layout of an operand whose
// reduction index is the facet.  Two input channels share one transposition tile.
//
// The reduction runs over facets, so the power-of-two scales of the two operands cannot differ from facet
// to facet inside a sum.  They are uniform per pass instead, and the accumulators carry a scale of their own:
//     gamma   one per 32-facet tile and workgroup, on the gout^T operand that the workgroup prepares in LDS.
//             The operand of the next tile is split with the scale of the tiles before it (with 2^3 of
//             head room) while its own maximum is collected; in the rare case that this maximum would
//             overflow fp16 or leave fewer than 2^5 above the smallest normal step, the tile is fetched
//             and split again with a scale of its own.
//     alpha   one per pass and wavefront, on G.  A wavefront's accumulators keep one scale S = alpha * gamma,
//             fixed by its first pass (with 2^9 of head room below the overflow bound from the largest
//             texture value it just fetched and the largest SH value of its facets), so alpha = S / gamma
//             afterwards; 1 / S is taken out when the partial result is written.  Small operands cost
//             nothing (their error is absolute, far below the accumulated sum).  Operands that outgrow the
//             head room along the facet list raise *overflow: the result of this kernel is then void and
//             the caller's guarded launch of the three-piece bf16 kernel, which needs no scales, replaces it.
//   workgroup  4 wavefronts (one per SIMD), 64 input x 64 output channels, a strided subset of the tiles
//   wavefront  16 input channels = 8 channel pairs x 2 output tiles of gW^T[(ci,d)][co]; narrower filters give
//              every wavefront 1, 2 or 4 pairs instead (NCP)
template <int KW, int NCP, bool HALF, bool PRE>
__device__ __forceinline__ void h2_filt_pass(const float (&shr)[KW][8], const float4 *slab, const u32x4 *go,
                                             f32x16 (&acc)[NCP][2], const u32x4 &ea, const u32x4 &eb, int lane)
{
    const int l32 = lane & 31;
    // G of channels cbase + 2cp (a) and + 1 (b), eight d's of my half for my facet, as fp16 pieces
    // texture values of my facet's points for four channels (two pairs).  With few points per facet they are read a
    // pair of channel pairs ahead, into the registers the wider phases need for their SH values: the blocks of matrix
    // instructions between the generations are fixed points of the instruction order, and a read issued behind one
    // would be waited for right there.
    constexpr bool RP = KW <= 6;
    float4 tq[RP ? KW : 1];
    auto slab_at = [&](int kk, int q) -> float4 {
        return PRE ? slab[(kk * 32 + l32) * 4 + (q ^ ((l32 >> 2) & 3))] : slab[(kk * 4 + q) * 32 + l32];
    };
    auto read_q = [&](int q) {
        if constexpr (RP) {
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) tq[kk] = slab_at(kk, q);
        }
    };
    auto gen = [&](u32x4 (&pa)[2], u32x4 (&pb)[2], int cp) {
        float aa[8], ab[8];
#pragma unroll
        for (int kk = 0; kk < KW; ++kk) {
            float4 t4;
            if constexpr (RP) t4 = tq[kk];
            else t4 = slab_at(kk, cp >> 1);
            const float ta = (cp & 1) ? t4.z : t4.x, tb = (cp & 1) ? t4.w : t4.y;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                aa[q] = kk ? fmaf(ta, shr[kk][q], aa[q]) : ta * shr[kk][q];
                ab[q] = kk ? fmaf(tb, shr[kk][q], ab[q]) : tb * shr[kk][q];
            }
        }
        if constexpr (HALF) {
            cvt8h(aa, pa[0]);
            cvt8h(ab, pb[0]);
            pa[1] = pa[0]; pb[1] = pb[0];
        } else {
            split8h(aa, pa[0], pa[1]);
            split8h(ab, pb[0], pb[1]);
        }
    };
    // The four transposition MFMAs are one asm block with VGPR destinations: in a kernel whose accumulators
    // live in AGPRs the compiler gives every MFMA an AGPR destination, and the results would have to be
    // copied out one by one before the packing.  The compiler cannot see into the block: the s_nop in the middle
    // keep the second product of a chain behind the first one's write of its accumulator (only one other MFMA
    // lies between them), the trailing ones cover the wait states a vector ALU read of an MFMA result needs.
    auto transpose = [&](u32x4 (&o)[2][2], const u32x4 (&pa)[2], const u32x4 (&pb)[2]) {
        if constexpr (HALF) {
            // one piece per operand: the chain of two products with the wait states of the block below
            f32x16 d;
            asm volatile("s_nop 3\n"
                         "v_mfma_f32_32x32x16_f16 %0, %1, %3, 0\n"
                         "s_nop 7\n"
                         "s_nop 7\n"
                         "s_nop 7\n"
                         "v_mfma_f32_32x32x16_f16 %0, %2, %4, %0\n"
                         "s_nop 15\n"
                         "s_nop 7\n"
                         : "=&v"(d)
                         : "v"(pa[0]), "v"(pb[0]), "v"(ea), "v"(eb));
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    o[0][st][jj] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(d[8 * st + 2 * jj], d[8 * st + 2 * jj + 1]));
                    o[1][st][jj] = o[0][st][jj];
                }
            return;
        }
        f32x16 d0, d1;
        asm volatile("s_nop 3\n"
                     "v_mfma_f32_32x32x16_f16 %0, %2, %6, 0\n"
                     "v_mfma_f32_32x32x16_f16 %1, %3, %6, 0\n"
                     "s_nop 7\n"
                     "s_nop 7\n"
                     "v_mfma_f32_32x32x16_f16 %0, %4, %7, %0\n"
                     "v_mfma_f32_32x32x16_f16 %1, %5, %7, %1\n"
                     "s_nop 15\n"
                     "s_nop 7\n"
                     : "=&v"(d0), "=&v"(d1)
                     : "v"(pa[0]), "v"(pa[1]), "v"(pb[0]), "v"(pb[1]), "v"(ea), "v"(eb));
        // every result is one fp16 value, so the conversion back is exact
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                o[0][st][jj] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(d0[8 * st + 2 * jj], d0[8 * st + 2 * jj + 1]));
                o[1][st][jj] = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(d1[8 * st + 2 * jj], d1[8 * st + 2 * jj + 1]));
            }
    };

    // the gout^T operand stays in registers for the whole pass (it serves all channel pairs)
    u32x4 g[2][2][2];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int p = 0; p < 2; ++p) g[st][t][p] = go[((st * 2 + t) * 2 + p) * 64 + lane];

    // software pipeline over the channel pairs: the G values of pair cp+1 are generated and split
    // (vector ALU) while the products of pair cp run on the matrix core
    u32x4 o[2][2];
    read_q(0);
    {
        u32x4 pa[2], pb[2];
        gen(pa, pb, 0);
        transpose(o, pa, pb);
    }
#pragma unroll
    for (int cp = 0; cp < NCP; ++cp) {
        u32x4 pa[2], pb[2];
        if (cp + 1 < NCP) gen(pa, pb, cp + 1);
        if (!(cp & 1) && cp + 2 < NCP) read_q((cp + 2) >> 1);      // (pair cp + 1 was the last reader of the registers)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            // three piece products, smallest first; the two output tiles alternate
            if constexpr (!HALF) {
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[cp][t] = mfma_f16(o[1][st], g[st][t][0], acc[cp][t]);
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[cp][t] = mfma_f16(o[0][st], g[st][t][1], acc[cp][t]);
            }
#pragma unroll
            for (int t = 0; t < 2; ++t) acc[cp][t] = mfma_f16(o[0][st], g[st][t][0], acc[cp][t]);
        }
        if (cp + 1 < NCP) transpose(o, pa, pb);
    }
}

// 256 zero bytes in global memory: what a fetch without a row reads instead, so that no fetch of the prefetch stage
// sits behind a branch (a branch per fetch also puts a wait for LDS in front of every single one)
__device__ __attribute__((aligned(256))) unsigned h2_zero_row[64];

// slot descriptors of a 32-facet tile: facet id (-1: none), first texture point, number of points.  They come in
// two dependent fetches (facet order, then the running totals of that facet), issued in two different tiles (by lanes
// i < 32 of two wavefronts, the facet passing through LDS), so that neither waits for the other: the results stay as
// fetched until the end of the tile.
struct HTile {
    int f, k0, K;
};
__device__ __forceinline__ int htile_facet(const int *__restrict__ order, int64_t tile, int64_t ntiles, int64_t Nf, int i)
{
    const int64_t slot = tile * 32 + i;
    const bool ok = tile < ntiles && slot < Nf;
    return order ? order[ok ? slot : 0] : (int)slot;            // (a valid slot's value is used only)
}
struct HTileRaw {
    int f, a, b;                                               // facet or -1, cum[f - 1] (cum[0] for f = 0), cum[f]
};
__device__ __forceinline__ HTileRaw htile_totals(const int *__restrict__ cum, int f, int64_t tile, int64_t ntiles, int64_t Nf, int i)
{
    const int64_t slot = tile * 32 + i;
    const bool ok = tile < ntiles && slot < Nf && f >= 0 && f < Nf;
    const int fi = ok ? f : 0;
    HTileRaw r;
    r.f = ok ? f : -1;
    r.a = cum[fi ? fi - 1 : 0];
    r.b = cum[fi];
    return r;
}
__device__ __forceinline__ HTile htile_finish(const HTileRaw &r, int T)
{
    HTile d = {-1, 0, 0};
    int a = r.f > 0 ? r.a : 0, b = r.b;
    a = a < 0 ? 0 : (a > T ? T : a);
    b = b < 0 ? 0 : (b > T ? T : b);
    if (r.f >= 0 && b > a) d = {r.f, a, b - a};
    return d;
}

// The inputs of a tile's first pass are fetched by the whole workgroup while the previous tile is
// being multiplied (held in registers, written to the other LDS buffer afterwards):
//   gout     thread (co, step, half): its eight facets in accumulator-row order
//   SH rows  32 facets x kHKB points x 64 bytes, kHShv 16-byte pieces per thread
constexpr int kHShv = (kHKB * 32 * 4 + 255) / 256;      // 16-byte pieces of the tile's SH rows per thread
struct HPre {
    float g[8];
    float4 shv[kHShv];
};
__device__ __forceinline__ unsigned hld_raw_or_zero(const float *base, int64_t idx, bool ok)
{
    return *(ok ? reinterpret_cast<const unsigned *>(base) + idx : h2_zero_row);
}
__device__ __forceinline__ unsigned hld_raw_or_zero(const bf16_t *base, int64_t idx, bool ok)
{
    return *(ok ? reinterpret_cast<const unsigned *>(base) + (idx >> 1) : h2_zero_row);
}
template <typename TIO>
__device__ __forceinline__ void hpre_issue(HPre &P, const TIO *__restrict__ gout, const float *__restrict__ sh,
                                           const int *sf, const int *sk0, const int *sK, int Cout, int n0)
{
    const int co = threadIdx.x & 63, st = (threadIdx.x >> 6) & 1, hh = threadIdx.x >> 7;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int f = sf[16 * st + 8 * (j >> 2) + 4 * hh + (j & 3)];
        // (kept as raw bits until the fetches are out; Cout is even for bf16 rows, so the half is the column's parity)
        P.g[j] = __builtin_bit_cast(float, hld_raw_or_zero(gout, (int64_t)f * Cout + n0 + co, f >= 0 && n0 + co < Cout));
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) P.g[j] = hcvt_raw(__builtin_bit_cast(unsigned, P.g[j]), (n0 + co) & 1, TIO());
    // piece threadIdx.x + 256 i of the SH rows: slot (threadIdx.x / 4) % 32 for every i, point threadIdx.x / 128 + 2 i
    const int slot = (threadIdx.x >> 2) & 31, K = sK[slot];
    const float *row0 = sh + ((int64_t)sk0[slot] + (threadIdx.x >> 7)) * 16 + 4 * (threadIdx.x & 3);
#pragma unroll
    for (int i = 0; i < kHShv; ++i) {
        const int kk = (threadIdx.x >> 7) + 2 * i;
        const bool ok = kk < kHKB && kk < K;
        P.shv[i] = hld4(ok ? row0 + 32 * i : reinterpret_cast<const float *>(h2_zero_row));
    }
}
__device__ __forceinline__ float hpre_gmax(const HPre &P)
{
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(P.g[j]));
    return hwave_fmax(m);
}
// gamma: scale of the gout operand
__device__ __forceinline__ void hpre_commit(const HPre &P, u32x4 *go, float *shs, float gamma, bool with_sh)
{
    const int co = threadIdx.x & 63, st = (threadIdx.x >> 6) & 1, hh = threadIdx.x >> 7;
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = P.g[j] * gamma;
    u32x4 p1, p2;
    split8h(x, p1, p2);
    u32x4 *dst = go + ((st * 2 + (co >> 5)) * 2) * 64 + 32 * hh + (co & 31);
    dst[0] = p1; dst[64] = p2;
    if (with_sh) {
#pragma unroll
        for (int i = 0; i < kHShv; ++i) {
            const int e = threadIdx.x + 256 * i;
            if (e < kHKB * 32 * 4) *reinterpret_cast<float4 *>(shs + 4 * e) = P.shv[i];      // [point*32 + slot][16]
        }
    }
}

// does the scale s put a maximum m (> 0) into the band the pieces keep their accuracy in?
__device__ __forceinline__ bool scale_fits(float s, float m) { return s * m < 32768.0f && s * m >= 32.0f; }

// texture rows of one pass (KW points per facet) for my wavefront's channels: 64 bytes per row, four lanes per row
template <int KW, bool TVEC, int NCP, typename TIO>
__device__ __forceinline__ void htex_issue(HRaw4<TIO> (&pf)[2 * kHKB], const TIO *__restrict__ tex, const int *sk0,
                                           const int *sK, int sweep, int cw, int Cin, int lane)
{
    const int piece = lane & 3;
#pragma unroll
    for (int i = 0; i < 2 * KW; ++i) {
        const int rr = i * 16 + (lane >> 2), kk = rr >> 5, slot = rr & 31;
        const bool ok = sweep * kHKB + kk < sK[slot] && 4 * piece < 2 * NCP;
        pf[i] = ok ? hld4_raw<TVEC>(tex + (int64_t)(sk0[slot] + sweep * kHKB + kk) * Cin + cw + 4 * piece,
                                    Cin - (cw + 4 * piece))
                   : hraw_zero(TIO());
    }
}

// The same rows straight into a slab buffer of the wavefront (fp32 rows, four or eight channel pairs per wavefront, at most kHPre points
// per facet), a whole tile ahead: no register holds them on the way, so the request can leave before the tile in
// front is multiplied.  Row-major slab, 64 bytes per (point, facet slot); lane L of instruction j delivers the
// 16 bytes at position 64 j + L, and fetches the piece (L & 3) ^ (slot / 4 & 3) of its row there, which spreads the
// 16-byte reads of 16 consecutive slots over all banks.  Entries without a row receive zeros from h2_zero_row.
// The data is there after vmcnt has drained.
// The requests are written as instructions: the compiler puts a wait for all outstanding fetches in front of the
// next LDS access it cannot tell apart from the landing zone of such a request, which would end the prefetch right
// where it starts.  It counts its own fetches only; the ones here are older than any fetch it waits for later in the
// tile and return in order, so its waits hold.  The readers of the slab wait themselves (hwait_vm0).
constexpr int kHPre = 6;
constexpr int kHSlabW = 2 * kHPre * 128;              // float4 of a wavefront's slab: two buffers of kHPre points (>= one of kHKB)
static_assert(kHSlabW >= kHKB * 128, "slab");
__device__ __forceinline__ void hdma16(const float *src, unsigned lds_base)
{
    unsigned keep;                                      // (M0 is handed back as it was found: the compiler may hold a value of its own there)
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "v"(src), "s"(lds_base)
                 : "memory");
}
template <int KW, int NCP>
__device__ __forceinline__ void htex_dma(const float *__restrict__ tex, const int *sk0, const int *sK, float4 *buf, int cw,
                                         int Cin, int lane)
{
    // row 16 j + lane / 4 of the tile's (point, slot) rows: point j / 2, slot lane / 4 or 16 + lane / 4
    const int r = lane >> 2;
    const int k0a = sk0[r], Ka = sK[r], k0b = sk0[16 + r], Kb = sK[16 + r];
    const unsigned base = (unsigned)(size_t)(__attribute__((address_space(3))) void *)buf;
    // (one address per slot in front of the selections: a product inside a selected operand turns it into a branch)
    const int pa = (lane & 3) ^ ((r >> 2) & 3), pb = (lane & 3) ^ (((16 + r) >> 2) & 3);
    const float *rowa = tex + (int64_t)k0a * Cin + cw + 4 * pa, *rowb = tex + (int64_t)k0b * Cin + cw + 4 * pb;
    // (a wavefront with four channel pairs owns the first 32 bytes of its 64-byte slab rows; the rest reads zeros)
    const bool cola = cw + 4 * pa < Cin && 4 * pa < 2 * NCP, colb = cw + 4 * pb < Cin && 4 * pb < 2 * NCP;
#pragma unroll
    for (int j = 0; j < 2 * KW; ++j) {
        const int kk = j >> 1;
        const bool ok = (j & 1) ? (kk < Kb && colb) : (kk < Ka && cola);
        const float *row = ((j & 1) ? rowb : rowa) + (int64_t)kk * Cin;
        hdma16(ok ? row : reinterpret_cast<const float *>(h2_zero_row), base + 1024u * j);
    }
}
// every outstanding fetch has arrived (an instruction the compiler keeps count with, and a fence for its LDS reads)
__device__ __forceinline__ void hwait_vm0()
{
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}


// State of the scales: gam_cur (workgroup-uniform) = scale the next operand is split with; S
// (wavefront-uniform) = scale of the accumulators, fixed by the wavefront's first pass.
struct HScales {
    float gam_cur, S;
};

// One tile of 32 facets whose inputs are in LDS buffer it % 2 (descriptors in it % 3): start the
// fetches for the next tile, run the passes, publish the next tile's inputs.
template <int KW, bool TVEC, int NCP, bool HALF, bool PRE, typename TIO>
__device__ __forceinline__ void h2_filt_tile(const TIO *__restrict__ gout, const TIO *__restrict__ tex,
                                             const float *__restrict__ sh, const int *__restrict__ cum,
                                             const int *__restrict__ order, u32x4 (*go_s)[2 * 2 * 2 * 64], float4 *slab,
                                             float (*sh_s)[kHKB * 32 * 16], int (*s_f)[32], int (*s_k0)[32],
                                             int (*s_K)[32], int *s_kmax, int (*s_fn)[32], float *s_gamma, unsigned *s_gm, f32x16 (&acc)[NCP][2],
                                             HScales &sc, int *overflow, const u32x4 &ea, const u32x4 &eb, int it, int64_t tile,
                                             int64_t stride, int64_t ntiles, int64_t Nf, int T, int Cin, int Cout, int c0,
                                             int n0, int lane, int w)
{
    const int l32 = lane & 31, h = lane >> 5;
    const int buf = it & 1, sb = it % 3, sb1 = (it + 1) % 3, sb2 = (it + 2) % 3;
    const int cw = c0 + 2 * NCP * w;                     // my wavefront's first input channel
    const bool idle = cw >= Cin;                         // narrow filters leave wavefronts without channels
    if constexpr (PRE) {
        // my texture rows of this tile were requested a tile ago (or at the start of the phase); nothing else is
        // outstanding here, the end of the tile before consumed all of its fetches
        hwait_vm0();
        if (!idle)
            if constexpr (std::is_same<TIO, float>::value)
                htex_dma<KW, NCP>(tex, s_k0[sb1], s_K[sb1], slab + ((it + 1) & 1) * (KW * 128), cw, Cin, lane);
        slab += (it & 1) * (KW * 128);
    }
    // in flight while this tile is multiplied: inputs of the next tile, descriptors of the one after
    HPre P;
    hpre_issue(P, gout, sh, s_f[sb1], s_k0[sb1], s_K[sb1], Cout, n0);
    // descriptors: running totals of the tile after the next (its facets came in during the tile before), facets
    // of the one after that
    HTileRaw dr = {-1, 0, 0};
    int fn3 = -1;
    if (w == 1 && lane < 32) dr = htile_totals(cum, s_fn[it & 1][lane], tile + 2 * stride, ntiles, Nf, lane);
    if (w == 2 && lane < 32) fn3 = htile_facet(order, tile + 3 * stride, ntiles, Nf, lane);
    // maxima of the gout operands: slot (it + 1) % 3 collects the next tile's at the commit below; the slot of
    // the tile after that is cleared here (its last readers passed the barrier that ended the previous tile)
    const int gs = (it + 1) % 3;
    if (threadIdx.x == 0) s_gm[(it + 2) % 3] = 0u;

    const float gamma = s_gamma[buf];
    const int k0 = s_k0[sb][l32], K = s_K[sb][l32];
    const float invK = K > 0 ? 1.0f / (float)K : 0.f;
    const int nsweeps = KW < kHKB ? 1 : (__builtin_amdgcn_readfirstlane(s_kmax[sb]) + kHKB - 1) / kHKB;
    for (int sw = 0; sw < nsweeps && !idle; ++sw) {
        const int rem = K - sw * kHKB;
        const int Ks = rem < 0 ? 0 : (rem > KW ? KW : rem);
        float shr[KW][8];
        if (sw == 0) {
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) {
                const float *p = sh_s[buf] + (kk * 32 + l32) * 16 + 8 * h;
                const float4 u = hld4(p), v = hld4(p + 4);
                shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
                shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
            }
        } else {
            // further points of long facets: fetched directly
#pragma unroll
            for (int kk = 0; kk < KW; ++kk) {
                float4 u = make_float4(0.f, 0.f, 0.f, 0.f), v = u;
                if (kk < Ks) {
                    const float *p = sh + (int64_t)(k0 + sw * kHKB + kk) * 16 + 8 * h;
                    u = hld4(p);
                    v = hld4(p + 4);
                }
                shr[kk][0] = u.x * invK; shr[kk][1] = u.y * invK; shr[kk][2] = u.z * invK; shr[kk][3] = u.w * invK;
                shr[kk][4] = v.x * invK; shr[kk][5] = v.y * invK; shr[kk][6] = v.z * invK; shr[kk][7] = v.w * invK;
            }
        }
        float tmax = 0.f;
        if constexpr (PRE) {
#pragma unroll
            for (int i = 0; i < 2 * KW; ++i) tmax = absmax4(slab[64 * i + lane], tmax);
        } else {
            // my wavefront's texture rows of this pass -> slab
            HRaw4<TIO> pf[2 * kHKB];
            htex_issue<KW, TVEC, NCP, TIO>(pf, tex, s_k0[sb], s_K[sb], sw, cw, Cin, lane);
            const int piece = lane & 3;
#pragma unroll
            for (int i = 0; i < 2 * KW; ++i) {
                const int rr = i * 16 + (lane >> 2), kk = rr >> 5, slot = rr & 31;
                const float4 pv = hcvt4(pf[i]);
                slab[(kk * 4 + piece) * 32 + slot] = pv;
                tmax = absmax4(pv, tmax);
            }
        }
        // scale of G for this pass: |G| <= KW * max|tex| * max|sh / K|
        float smax = 0.f;
#pragma unroll
        for (int kk = 0; kk < KW; ++kk)
#pragma unroll
            for (int q = 0; q < 8; ++q) smax = fmaxf(smax, fabsf(shr[kk][q]));
        const float bound = hwave_fmax(tmax) * hwave_fmax(smax) * (float)KW;
        if (bound > 0.f) {
            float inv;
            const float need = pow2_scale(bound, &inv);          // need * bound < 2^14
            // The accumulators keep the scale S of the wavefront's first pass (2^9 below its overflow bound), so
            // alpha follows gamma: alpha = S / gamma.  Smaller operands later on cost nothing (their error is
            // absolute, far below the sum).  Operands that have grown past the head room cannot be taken in
            // at this scale: the wavefront raises the overflow flag -- the caller's next launch, the
            // three-piece bf16 kernel, then computes the whole gradient again -- and carries on with a
            // scale that is safe to execute.
            if (sc.S == 0.f) sc.S = need * (1.0f / 512.0f) * gamma;
            float al = sc.S / gamma;
            if (al > need) {
                if (lane == 0) *overflow = 1;
                al = need;
            }
#pragma unroll
            for (int kk = 0; kk < KW; ++kk)
#pragma unroll
                for (int q = 0; q < 8; ++q) shr[kk][q] *= al;
            h2_filt_pass<KW, NCP, HALF, PRE>(shr, slab, go_s[buf], acc, ea, eb, lane);
        }
    }

    // next tile's operand: split with the running scale, its own maximum collected on the side
    {
        const float m = hpre_gmax(P);
        if (lane == 0) atomicMax(&s_gm[gs], __builtin_bit_cast(unsigned, m));
    }
    hpre_commit(P, go_s[buf ^ 1], sh_s[buf ^ 1], sc.gam_cur, true);
    if (threadIdx.x == 0) s_gamma[buf ^ 1] = sc.gam_cur;
    if (w == 1) {
        const HTile dn = htile_finish(dr, T);            // (lanes 32..63: no facet)
        if (lane < 32) {
            s_f[sb2][lane] = dn.f; s_k0[sb2][lane] = dn.k0; s_K[sb2][lane] = dn.K;
        }
        const int km = hwave_max(dn.K);
        if (lane == 0) s_kmax[sb2] = km;
    }
    if (w == 2 && lane < 32) s_fn[(it + 1) & 1][lane] = fn3;       // (read at the start of the next tile)
    __syncthreads();
    const float gm = __builtin_bit_cast(float, s_gm[gs]);
    if (gm > 0.f && !scale_fits(sc.gam_cur, gm)) {           // workgroup-uniform: fetch and split that tile again
        float inv;
        sc.gam_cur = pow2_scale(gm, &inv) * 0.125f;          // gam * gm in [2^10, 2^11)
        hpre_issue(P, gout, sh, s_f[sb1], s_k0[sb1], s_K[sb1], Cout, n0);
        hpre_commit(P, go_s[buf ^ 1], sh_s[buf ^ 1], sc.gam_cur, false);
        if (threadIdx.x == 0) s_gamma[buf ^ 1] = sc.gam_cur;
        __syncthreads();
    }
}

// NCP = channel pairs of a wavefront (8 for 64 or more input channels; fewer for narrow filters, so that
// the four wavefronts share what channels there are)
template <bool TVEC, int NCP, bool HALF, typename TIO>
__global__ __launch_bounds__(256, 1) void f2f16h2_bwd_filt_k(const TIO *__restrict__ gout,
                                                              const TIO *__restrict__ tex,
                                                              const float *__restrict__ sh,
                                                              const int *__restrict__ cum,
                                                              const int *__restrict__ order,
                                                              float *__restrict__ partial, int *__restrict__ overflow,
                                                              int64_t Nf, int T, int Cin, int Cout, int64_t ntiles)
{
    __shared__ u32x4 go_s[2][2 * 2 * 2 * 64];
    __shared__ float4 slab_s[4 * kHSlabW];
    __shared__ __attribute__((aligned(16))) float sh_s[2][kHKB * 32 * 16];
    __shared__ int s_f[3][32], s_k0[3][32], s_K[3][32], s_kmax[3], s_fn[2][32];
    __shared__ float s_gamma[2];
    __shared__ unsigned s_gm[3];
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int c0 = blockIdx.y * (8 * NCP), n0 = blockIdx.z * 64;
    // phases of at most kHPre points request their texture rows a tile ahead, into the two halves of the slab
    constexpr bool kPre = TVEC && NCP >= 4 && std::is_same<TIO, float>::value;

    // selection operands of the transposition: column n < 16 takes d = n of channel a, n >= 16 takes d = n - 16 of b
    u32x4 ea, eb;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        unsigned va = 0, vb = 0;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int d = 8 * h + 2 * jj + u;
            if (l32 < 16 && d == l32) va |= 0x3C00u << (16 * u);            // fp16 1.0
            if (l32 >= 16 && d == l32 - 16) vb |= 0x3C00u << (16 * u);
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
    HScales sc = {1.0f, 0.f};

    // prologue: descriptors of my first two tiles, inputs of the first (its gout maximum first, then the split)
    const int64_t stride = gridDim.x;
    int64_t tile = blockIdx.x;
    if (w == 0) {
        const int q = lane >> 5;
        const int64_t tq = tile + q * stride;
        const HTile d = htile_finish(htile_totals(cum, htile_facet(order, tq, ntiles, Nf, l32), tq, ntiles, Nf, l32), T);
        s_f[q][l32] = d.f; s_k0[q][l32] = d.k0; s_K[q][l32] = d.K;
        const int km = hrow_max(d.K);                   // rows of 16 lanes
        const int k0m = max(__builtin_amdgcn_readlane(km, 0), __builtin_amdgcn_readlane(km, 16));
        const int k1m = max(__builtin_amdgcn_readlane(km, 32), __builtin_amdgcn_readlane(km, 48));
        if (lane == 0) { s_kmax[0] = k0m; s_kmax[1] = k1m; }
        if (lane < 32) s_fn[0][lane] = htile_facet(order, tile + 2 * stride, ntiles, Nf, lane);
    }
    if (threadIdx.x < 3) s_gm[threadIdx.x] = 0u;
    __syncthreads();
    {
        HPre P;
        hpre_issue(P, gout, sh, s_f[0], s_k0[0], s_K[0], Cout, n0);
        const float m = hpre_gmax(P);
        if (lane == 0) atomicMax(&s_gm[0], __builtin_bit_cast(unsigned, m));
        __syncthreads();
        const float gm = __builtin_bit_cast(float, s_gm[0]);
        if (gm > 0.f) {
            float inv;
            sc.gam_cur = pow2_scale(gm, &inv) * 0.125f;
        }
        hpre_commit(P, go_s[0], sh_s[0], sc.gam_cur, true);
        if (threadIdx.x == 0) s_gamma[0] = sc.gam_cur;
    }
    __syncthreads();

    // The sorted facet list makes the point counts of my tiles non-decreasing: one loop per point count in sequence,
    // each with the pass specialised for its number of points (the last one takes everything left,
    // long facets in several sweeps).  The bound is uniform over the workgroup.
    int it = 0;
#define PM_PHASE(N)                                                                                                  \
    if (tile < ntiles && (N == kHKB || __builtin_amdgcn_readfirstlane(s_kmax[it % 3]) <= N)) {                                        \
        if constexpr (kPre && N <= kHPre) {                                                                          \
            /* rows of the phase's first tile; requests of the phase before (same slab, other plane count) land first */ \
            hwait_vm0();                                                                                             \
            if (c0 + 2 * NCP * w < Cin)                                                                              \
                if constexpr (std::is_same<TIO, float>::value)                                                       \
                    htex_dma<N, NCP>(tex, s_k0[it % 3], s_K[it % 3], slab_s + w * kHSlabW + (it & 1) * (N * 128), \
                                c0 + 2 * NCP * w, Cin, lane);                                                        \
        }                                                                                                            \
        for (; tile < ntiles && (N == kHKB || __builtin_amdgcn_readfirstlane(s_kmax[it % 3]) <= N); ++it, tile += stride)             \
            h2_filt_tile<N, TVEC, NCP, HALF, (kPre && N <= kHPre), TIO>(                                             \
                gout, tex, sh, cum, order, go_s, slab_s + w * kHSlabW, sh_s, s_f, s_k0, s_K, s_kmax, s_fn, s_gamma, s_gm, acc, sc, \
                overflow, ea, eb, it, tile, stride, ntiles, Nf, T, Cin, Cout, c0, n0, lane, w);                      \
    }
    PM_PHASE(1);
    PM_PHASE(2);
    PM_PHASE(3);
    PM_PHASE(4);
    PM_PHASE(5);
    PM_PHASE(6);
    PM_PHASE(7);
    PM_PHASE(8);
    PM_PHASE(9);
#undef PM_PHASE

    // accumulator (cp, t): lane (co = 32t + l32, half h), register i <-> row m = 8(i/4) + 4h + i%4
    // = (channel c0 + 2 NCP w + 2cp + m/16, d = m%16); four consecutive d's per group of four registers
    const float unscale = sc.S != 0.f ? 1.0f / sc.S : 0.f;
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
                        make_float4(acc[cp][t][4 * q] * unscale, acc[cp][t][4 * q + 1] * unscale,
                                    acc[cp][t][4 * q + 2] * unscale, acc[cp][t][4 * q + 3] * unscale);
            }
        }
}

int f2f16h2_bwd_filter_partials(const void *gout_, const void *tex_, const float *sh, const int *cum, const int *order,
                                 float *partial, int *overflow, int splits, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st,
                                 bool half, bool bf16)
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
#define PM_FILT(V, N, H, TIO) f2f16h2_bwd_filt_k<V, N, H, TIO><<<grid, dim3(256), 0, st>>>((const TIO *)gout_, (const TIO *)tex_, sh, cum, order, partial, overflow, Nf, (int)T, Cin, Cout, ntiles)
#define PM_FILT_N(V, H, TIO)                                                                              \
    do {                                                                                                  \
        if (ncp == 8) PM_FILT(V, 8, H, TIO); else if (ncp == 4) PM_FILT(V, 4, H, TIO);                    \
        else if (ncp == 2) PM_FILT(V, 2, H, TIO); else PM_FILT(V, 1, H, TIO);                             \
    } while (0)
    if (bf16) PM_FILT_N(true, true, bf16_t);
    else if (tvec && half) PM_FILT_N(true, true, float);
    else if (tvec) PM_FILT_N(true, false, float);
    else if (half) PM_FILT_N(false, true, float);
    else PM_FILT_N(false, false, float);
#undef PM_FILT_N
#undef PM_FILT
    PM_LAUNCHED("f2f_bwd_filter");
    return 0;
}

}  // namespace pmesh
