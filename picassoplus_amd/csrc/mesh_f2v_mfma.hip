// facet2vertex with the filter combination on the matrix cores, 16 SH coefficients: two-piece fp16 products
// (three v_mfma_f32_32x32x16_f16 per block) by default, the fp32 instruction (eight v_mfma_f32_32x32x2_f32) behind a switch.
//
//   w[e,co]   = sum_k coeff[f_e,k] * filt[k,co]        one 32 x 16 x 32 product per 32 entries and 32 channels
//   out[v,co] = (1/nf[v]) * sum_{e of v} w[e,co] * in[f_e, co/r]
//
// A wavefront takes four output vertices at a time and eight adjacency entries of each: the 32 entries
// are the rows of the product, 32 output channels its columns.  The product comes out with
// lane = channel and registers = entries, so the facet rows are gathered one float per lane (128
// contiguous bytes per entry) and the weighted sum over a vertex's entries stays inside a lane:
//     register i of lane (col, h)  <->  vertex i/4 of the four, entry slot 4h + i%4 of its eight.
// One cross-half exchange per vertex pair and channel block finishes the sum.
// Against the vector-ALU version this replaces 64 FMAs per entry and four channels by 1/4 of an MFMA.
#include <type_traits>
#include "common.h"
#include "fp16_split.h"
#include "rows_internal.h"

namespace pmesh {

// vdst lanes 32..63 <-> vsrc lanes 0..31; the s_nop cover the wait states around the swap.
__device__ __forceinline__ void half_swap(float &a, float &b)
{
    asm volatile("s_nop 3\n v_permlane32_swap_b32 %0, %1\n s_nop 3" : "+v"(a), "+v"(b));
}

template <typename TIO> __device__ __forceinline__ const TIO *at_bytes(const TIO *base, unsigned byte_offset)
{
    return reinterpret_cast<const TIO *>(reinterpret_cast<const char *>(base) + byte_offset);
}

// Features kept in bf16 in HBM (the reduced-precision variant of the layer): converted on load, rounded to nearest
// even on store; all sums stay in fp32.
typedef unsigned short bf16_t;
// Value at `byte_offset` from `base`, in two steps: ld_raw fetches the 4 bytes that hold it (a conditional fetch must
// not be followed by arithmetic inside its branch, or the wavefront waits for every fetch on the spot and the gathers
// no longer overlap), cvt_raw turns them into the value once all fetches of a batch are out.  A bf16 value is read
// as the aligned word that holds it (rows have an even number of values, so neighbouring lanes share the word) and
// written as one 4-byte store per lane pair: 2-byte accesses are slow on this memory path.
__device__ __forceinline__ unsigned ld_raw(const float *base, unsigned byte_offset)
{
    return *reinterpret_cast<const unsigned *>(reinterpret_cast<const char *>(base) + byte_offset);
}
__device__ __forceinline__ unsigned ld_raw(const bf16_t *base, unsigned byte_offset)
{
    return *reinterpret_cast<const unsigned *>(reinterpret_cast<const char *>(base) + (byte_offset & ~3u));
}
// The same fetch through a buffer descriptor (base, size in bytes): an offset at or past the size reads zero, so a
// gather over slots that may be empty needs neither a branch around each fetch nor a zero beforehand -- an empty slot
// carries the array's size as its offset.
typedef __amdgpu_buffer_rsrc_t buffer_t;
__device__ __forceinline__ buffer_t buffer_of(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ unsigned ld_buf(buffer_t b, unsigned byte_offset, float)
{
    return __builtin_amdgcn_raw_buffer_load_b32(b, (int)byte_offset, 0, 0);
}
__device__ __forceinline__ unsigned ld_buf(buffer_t b, unsigned byte_offset, bf16_t)
{
    return __builtin_amdgcn_raw_buffer_load_b32(b, (int)(byte_offset & ~3u), 0, 0);
}
__device__ __forceinline__ float cvt_raw(unsigned w, unsigned, float) { return __builtin_bit_cast(float, w); }
// (the half of the word that holds a bf16 value depends on its column only: `half_sel` is computed once per lane and
// channel block, the conversion is then one byte permutation: the value's two bytes on top of two zero bytes)
__device__ __forceinline__ unsigned half_sel(unsigned byte_offset) { return (byte_offset & 2u) ? 0x03020C0Cu : 0x01000C0Cu; }
__device__ __forceinline__ float cvt_raw(unsigned w, unsigned sel, bf16_t)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_perm(w, w, sel));
}
// Lanes l and l ^ STEP hold neighbouring values p[0], p[1] (the lane with (lane & STEP) == 0 the first): every lane
// calls this, `ok` says whether the pair is stored.  STEP = 1: neighbouring lanes; 2: lanes two apart.
template <int STEP> __device__ __forceinline__ void st1_pair(float *p, float v, bool ok, int lane)
{
    (void)lane;
    if (ok) *p = v;
}
template <int STEP> __device__ __forceinline__ void st1_pair(bf16_t *p, float v, bool ok, int lane)
{
    // quad_perm [1,0,3,2] swaps neighbours, [2,3,0,1] swaps lanes two apart
    const float nb = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), STEP == 1 ? 0xB1 : 0x4E, 0xF, 0xF, true));
    if (ok && !(lane & STEP)) {
        unsigned r;
        asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(v), "v"(nb));
        *reinterpret_cast<unsigned *>(p) = r;
    }
}

// Forward.  NCB = 32-channel blocks per workgroup column (blockIdx.y selects a chunk of 32*NCB channels).
// Requires K == 16, 16-byte aligned coefficient rows, Nf * C * 4 < 2^32.  Workgroups are persistent; the
// eight dies take contiguous eighths of the vertices (blockIdx.x & 7 = die).
// H2: the product on the fp16 matrix instruction, both operands split into two fp16 pieces (three piece products of
// 32 cycles where the fp32 instruction takes eight of 64, and matrix work that runs beside the vector ALU instead of
// in its place): every filter column is scaled by its own power of two and split once per wavefront, the coefficients
// of a pass's 32 entries are brought below 2^14 by one power of two for the wavefront, and both leave the sum again on
// the way into the vertex sums.
template <int NCB, typename TIO, bool H2>
__global__ __launch_bounds__(kBlock, (H2 && NCB <= 2 && sizeof(TIO) == 4) ? 4 : 1) void f2v_fwd_mfma_k(const TIO *__restrict__ in, const float *__restrict__ filt,
                                                         const float *__restrict__ coeff,
                                                         const int *__restrict__ nfcount,
                                                         const int *__restrict__ rowptr,
                                                         const int *__restrict__ colidx, TIO *__restrict__ out,
                                                         int64_t NvOut, int C, int r, int Co, unsigned in_bytes)
{
    const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = l & 31, h = l >> 5, j = col >> 3, s = col & 7;
    const buffer_t in_buf = buffer_of(in, in_bytes);
    const int co0 = blockIdx.y * (32 * NCB);
    const unsigned row_bytes = (unsigned)C * (unsigned)sizeof(TIO);

    // B operands: step kk of half h is coefficient 8h + kk (the A operand uses the same assignment)
    float wb[NCB][8];
    unsigned chb[NCB], xsel[NCB];
    bool con[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int co = co0 + 32 * cb + col;
        con[cb] = co < Co;
        chb[cb] = con[cb] ? (unsigned)(co / r) * (unsigned)sizeof(TIO) : 0u;
        xsel[cb] = half_sel(chb[cb]);
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) wb[cb][kk] = con[cb] ? filt[(size_t)(8 * h + kk) * Co + co] : 0.f;
    }

    // (H2) every filter column under its own power-of-two scale: a column of small weights keeps its accuracy beside a large one
    u32x4 bh[NCB], bl[NCB];
    float inv_beta[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        inv_beta[cb] = 1.f;
        if constexpr (H2) {
            float m = 0.f;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(wb[cb][kk]));
            m = fmaxf(m, __shfl_xor(m, 32, 64));                       // the column's other eight coefficients
            const float beta = pow2_scale(m, &inv_beta[cb]);
            float t[8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) t[kk] = wb[cb][kk] * beta;
            split8h(t, bh[cb], bl[cb]);
        }
    }

    const int64_t groups = (NvOut + 3) >> 2, gx = (groups + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int64_t gstride = (int64_t)(gridDim.x >> 3) * 4;
    const int64_t gend = ((xcd + 1) * gx < groups) ? (xcd + 1) * gx : groups;
    int64_t g = xcd * gx + (int64_t)(blockIdx.x >> 3) * 4 + wave;

    auto bounds = [&](int64_t gg, int &a, int &b) {
        a = 0; b = 0;
        const int64_t v = 4 * gg + j;
        if (gg < gend && v < NvOut) { a = rowptr[v]; b = rowptr[v + 1]; }
    };
    int e0, e1, ne0, ne1;
    bounds(g, e0, e1);
    bounds(g + gstride, ne0, ne1);
    int f = (e0 + s < e1) ? colidx[e0 + s] / 3 : -1;

    for (; g < gend; g += gstride) {
        // row bounds two groups ahead, first entries one group ahead
        int me0, me1;
        bounds(g + 2 * gstride, me0, me1);
        const int nf = (ne0 + s < ne1) ? colidx[ne0 + s] / 3 : -1;
        // this half stores vertices 4g + 2h and 4g + 2h + 1
        const int64_t vs = 4 * g + 2 * h;
        const int cnt0 = (vs < NvOut) ? nfcount[vs] : 1, cnt1 = (vs + 1 < NvOut) ? nfcount[vs + 1] : 1;
        const unsigned long long has = __builtin_amdgcn_ballot_w64(e1 > e0);      // bit 8j: vertex j has entries

        float acc[NCB][4];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[cb][q] = 0.f;

        for (int p = 0;; ++p) {
            if (p > 0) f = (e0 + 8 * p + s < e1) ? colidx[e0 + 8 * p + s] / 3 : -1;
            // A operand: coefficients 8h .. 8h+7 of my entry (zero rows for empty slots)
            float a[8];
            {
                float4 t0 = make_float4(0.f, 0.f, 0.f, 0.f), t1 = t0;
                if (f >= 0) {
                    const float4 *cp = reinterpret_cast<const float4 *>(coeff + (int64_t)f * 16 + 8 * h);
                    t0 = cp[0]; t1 = cp[1];
                }
                a[0] = t0.x; a[1] = t0.y; a[2] = t0.z; a[3] = t0.w;
                a[4] = t1.x; a[5] = t1.y; a[6] = t1.z; a[7] = t1.w;
            }
            // byte offsets of the facet rows my registers pair with (an empty slot: past the end, reads zero)
            const unsigned boff = (f >= 0) ? (unsigned)f * row_bytes : in_bytes;
            unsigned b[16];
#pragma unroll
            for (int i = 0; i < 16; ++i)
                b[i] = (unsigned)__builtin_amdgcn_ds_bpermute((8 * (i >> 2) + 4 * h + (i & 3)) * 4, (int)boff);
            unsigned xr[NCB][16];
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int i = 0; i < 16; ++i) xr[cb][i] = ld_buf(in_buf, b[i] + chb[cb], TIO());
            float x[NCB][16];
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int i = 0; i < 16; ++i) x[cb][i] = cvt_raw(xr[cb][i], xsel[cb], TIO());
            if constexpr (H2) {
                float m = 0.f;
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(a[kk]));
                float inv_alpha;
                const float alpha = pow2_scale(hwave_fmax(m), &inv_alpha);       // (every lane of the wavefront is here)
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) a[kk] *= alpha;
                u32x4 ah, al;
                split8h(a, ah, al);
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    const float unscale = inv_alpha * inv_beta[cb];
                    f32x16 d;
#pragma unroll
                    for (int i = 0; i < 16; ++i) d[i] = 0.f;
                    // three piece products, smallest first
                    d = mfma_f16(al, bh[cb], d);
                    d = mfma_f16(ah, bl[cb], d);
                    d = mfma_f16(ah, bh[cb], d);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        float t = 0.f;
#pragma unroll
                        for (int i = 4 * q; i < 4 * q + 4; ++i) t = fmaf(d[i], x[cb][i], t);
                        acc[cb][q] = fmaf(t, unscale, acc[cb][q]);
                    }
                }
            } else {
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    f32x16 d;
#pragma unroll
                    for (int i = 0; i < 16; ++i) d[i] = 0.f;
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) d = __builtin_amdgcn_mfma_f32_32x32x2f32(a[kk], wb[cb][kk], d, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[cb][i >> 2] = fmaf(d[i], x[cb][i], acc[cb][i >> 2]);
                }
            }
            if (!__builtin_amdgcn_ballot_w64(e0 + 8 * (p + 1) < e1)) break;
        }

        const float inv0 = ((has >> (8 * (2 * h))) & 1ull) ? 1.0f / (float)cnt0 : 0.f;
        const float inv1 = ((has >> (8 * (2 * h + 1))) & 1ull) ? 1.0f / (float)cnt1 : 0.f;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            // (acc0, acc2) and (acc1, acc3): after the swap the sums are vertex 0/1 in half 0, 2/3 in half 1
            half_swap(acc[cb][0], acc[cb][2]);
            half_swap(acc[cb][1], acc[cb][3]);
            const float o0 = (acc[cb][0] + acc[cb][2]) * inv0, o1 = (acc[cb][1] + acc[cb][3]) * inv1;
            const int co = co0 + 32 * cb + col;
            st1_pair<1>(out + (vs * Co + co), o0, con[cb] && vs < NvOut, col);
            st1_pair<1>(out + ((vs + 1) * Co + co), o1, con[cb] && vs + 1 < NvOut, col);
        }
        e0 = ne0; e1 = ne1; ne0 = me0; ne1 = me1;
        f = nf;
    }
}


// ----------------------------------------------------------------------------------------
// Forward with the pointwise tail of the convolution module on its store (picasso/mesh/layers.py:163-174 runs
// the tail as a matmul with depth_weights, + biases, the activation and batch norm after the native op):
//     out2[v, n] = max(sum_c conv[v, c] * Wd[c, n] + bias[n], floor) * scale[n] + shift[n]
// The kernel above is kept as it is; a wavefront additionally parks the four vertex rows of every pass over its
// groups in a private LDS tile and, every four passes, multiplies the 16 rows by the weights: two-piece fp16
// products on v_mfma_f32_16x16x32_f16 (three piece products per 16 x 16 x 32 block), the rows under one power-of-two
// scale per tile, every weight column under its own (taken out again with the bias).  The weights sit in LDS in
// operand layout, packed once per call by f2v_tail_pack_k:
//     Wp[((s * NTD + nt) * 2 + piece) * 64 + lane] = pieces of beta_n * Wd[32 s + 8 (lane / 16) .. + 7][16 nt + lane % 16]
//     meta[4 n .. 4 n + 3] = 1 / beta_n, bias_n, scale_n, shift_n
// A / B operand of the instruction: lane l holds row / column l % 16, reduction indices 8 (l / 16) .. + 7;
// result: lane l holds column l % 16, rows 4 (l / 16) .. + 3.  NCB = 32-channel blocks of the convolution's
// rows (its Co = 32 NCB is the product's reduction length), NTD = 16-column tiles of the tail's output.
typedef float f32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4v mfma16_f16(const u32x4 &a, const u32x4 &b, const f32x4v &c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__global__ __launch_bounds__(kBlock) void f2v_tail_pack_k(const float *__restrict__ Wd, const float *__restrict__ bias,
                                                          const float *__restrict__ scale, const float *__restrict__ shift,
                                                          u32x4 *__restrict__ Wp, float *__restrict__ meta, int Kc, int Cd,
                                                          int NS, int NTD)
{
    const int idx = blockIdx.x * kBlock + threadIdx.x;
    if (idx >= NS * NTD * 64) return;
    const int lane = idx & 63, nt = (idx >> 6) % NTD, s = (idx >> 6) / NTD;
    const int n = 16 * nt + (lane & 15), kg = lane >> 4;
    // the column's largest weight: Kc is 32 or 64, all requests of a batch of 32 leave together
    float m = 0.f;
    for (int k0 = 0; k0 < Kc; k0 += 32) {
        float wv[32];
#pragma unroll
        for (int k = 0; k < 32; ++k) wv[k] = Wd[(size_t)(k0 + k) * Cd + n];      // (Kc is a multiple of 32)
#pragma unroll
        for (int k = 0; k < 32; ++k) m = fmaxf(m, fabsf(wv[k]));
    }
    float inv;
    const float beta = pow2_scale(m, &inv);
    float t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int k = 32 * s + 8 * kg + j;
        t[j] = Wd[(size_t)k * Cd + n] * beta;
    }
    u32x4 hi, lo;
    split8h(t, hi, lo);
    Wp[((size_t)(s * NTD + nt) * 2 + 0) * 64 + lane] = hi;
    Wp[((size_t)(s * NTD + nt) * 2 + 1) * 64 + lane] = lo;
    if (s == 0 && kg == 0) {
        meta[4 * n] = inv;
        meta[4 * n + 1] = bias ? bias[n] : 0.f;
        meta[4 * n + 2] = scale ? scale[n] : 1.f;
        meta[4 * n + 3] = shift ? shift[n] : 0.f;
    }
}

constexpr int kTailPad = 4;         // floats between staged rows: 16-byte reads of 16 rows spread over the banks

#ifndef PM_TAIL_OCC
#define PM_TAIL_OCC 4
#endif
template <int NCB, int NTD>
__global__ __launch_bounds__(kBlock, NTD <= 4 ? PM_TAIL_OCC : 2) void f2v_fwd_tail_k(const float *__restrict__ in, const float *__restrict__ filt,
                                                         const float *__restrict__ coeff,
                                                         const int *__restrict__ nfcount,
                                                         const int *__restrict__ rowptr,
                                                         const int *__restrict__ colidx, float *__restrict__ conv_out,
                                                         const u32x4 *__restrict__ Wp, const float *__restrict__ meta,
                                                         float *__restrict__ out2, unsigned *__restrict__ bits, int relu,
                                                         int64_t NvOut, int C, int r, unsigned in_bytes)
{
    constexpr int Co = 32 * NCB, Cd = 16 * NTD, kRow = Co + kTailPad;
    __shared__ u32x4 s_W[NCB * NTD * 2 * 64];
    __shared__ __attribute__((aligned(16))) float s_meta[4 * Cd];
    __shared__ __attribute__((aligned(16))) float s_stage[kBlock / 64][16 * kRow];
    const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = l & 31, h = l >> 5, j = col >> 3, s = col & 7;
    const buffer_t in_buf = buffer_of(in, in_bytes);
    const unsigned row_bytes = (unsigned)C * 4u;

    for (int i = threadIdx.x; i < NCB * NTD * 2 * 64; i += kBlock) s_W[i] = Wp[i];
    for (int i = threadIdx.x; i < 4 * Cd; i += kBlock) s_meta[i] = meta[i];

    float wb[NCB][8];
    unsigned chb[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int co = 32 * cb + col;
        chb[cb] = (unsigned)(co / r) * 4u;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) wb[cb][kk] = filt[(size_t)(8 * h + kk) * Co + co];
    }
    u32x4 bh[NCB], bl[NCB];
    float inv_beta[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        float m = 0.f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(wb[cb][kk]));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        const float beta = pow2_scale(m, &inv_beta[cb]);
        float t[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) t[kk] = wb[cb][kk] * beta;
        split8h(t, bh[cb], bl[cb]);
    }
    __syncthreads();

    const int64_t groups = (NvOut + 3) >> 2, gx = (groups + 7) >> 3;
    const int xcd = blockIdx.x & 7;
    const int64_t gstride = (int64_t)(gridDim.x >> 3) * 4;
    const int64_t gend = ((xcd + 1) * gx < groups) ? (xcd + 1) * gx : groups;
    int64_t g = xcd * gx + (int64_t)(blockIdx.x >> 3) * 4 + wave;
    float *stage = s_stage[wave];
    const float floor_v = relu ? 0.f : -__builtin_inff();

    // the tile's rows (cnt passes of four vertices, the last one at group g_last) times the weights, and the store.
    // FULL: four passes, every vertex of them inside the array -- no condition on a row.
    auto flush = [&](auto full_tag, int64_t g_last, int cnt) {
        constexpr bool FULL = decltype(full_tag)::value;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int r16 = l & 15, kg = l >> 4;
        const bool rvalid = FULL || (r16 >> 2) < cnt;          // rows of passes that did not happen hold old values
        float a[NCB][8];
        float m = 0.f;
#pragma unroll
        for (int ks = 0; ks < NCB; ++ks) {
            const float4 *sp = reinterpret_cast<const float4 *>(stage + r16 * kRow + 32 * ks + 8 * kg);
            const float4 u = sp[0], v = sp[1];
            a[ks][0] = rvalid ? u.x : 0.f; a[ks][1] = rvalid ? u.y : 0.f; a[ks][2] = rvalid ? u.z : 0.f; a[ks][3] = rvalid ? u.w : 0.f;
            a[ks][4] = rvalid ? v.x : 0.f; a[ks][5] = rvalid ? v.y : 0.f; a[ks][6] = rvalid ? v.z : 0.f; a[ks][7] = rvalid ? v.w : 0.f;
#pragma unroll
            for (int q = 0; q < 8; ++q) m = fmaxf(m, fabsf(a[ks][q]));
        }
        float inv_alpha;
        const float alpha = pow2_scale(hwave_fmax(m), &inv_alpha);
        u32x4 ah[NCB], al[NCB];
#pragma unroll
        for (int ks = 0; ks < NCB; ++ks) {
#pragma unroll
            for (int q = 0; q < 8; ++q) a[ks][q] *= alpha;
            split8h(a[ks], ah[ks], al[ks]);
        }
        // my four rows of the result: pass kg of the tile, vertices 4 g_kg .. + 3
        const int64_t v0 = 4 * (g_last - (int64_t)((FULL ? 4 : cnt) - 1 - kg) * gstride);
        const bool qok = FULL || kg < cnt;
        float *orow = out2 + v0 * Cd + r16;
        unsigned mine = 0u;                                     // the mask word of row r16 / 2, columns 32 (r16 % 2) .. + 31
#pragma unroll
        for (int np = 0; np < NTD / 2; ++np) {
            f32x4v d[2];
            float4 mt[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int nt = 2 * np + e;
                d[e] = f32x4v{0.f, 0.f, 0.f, 0.f};
                mt[e] = reinterpret_cast<const float4 *>(s_meta)[16 * nt + r16];
            }
#pragma unroll
            for (int ks = 0; ks < NCB; ++ks)
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const u32x4 *wp = s_W + ((ks * NTD + 2 * np + e) * 2) * 64 + l;
                    const u32x4 wh = wp[0], wl = wp[64];
                    d[e] = mfma16_f16(al[ks], wh, d[e]);
                    d[e] = mfma16_f16(ah[ks], wl, d[e]);
                    d[e] = mfma16_f16(ah[ks], wh, d[e]);
                }
            unsigned long long pos[2][4];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const float us = inv_alpha * mt[e].x;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float v = fmaxf(fmaf(d[e][i], us, mt[e].y), floor_v);
                    const bool ok = FULL || (qok && v0 + i < NvOut);
                    if (ok) orow[(int64_t)i * Cd + 16 * (2 * np + e)] = fmaf(v, mt[e].z, mt[e].w);
                    pos[e][i] = __builtin_amdgcn_ballot_w64(ok && v > 0.f);
                }
            }
            if (bits) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const unsigned word = (unsigned)((pos[0][i] >> (16 * kg)) & 0xFFFFull) |
                                          ((unsigned)((pos[1][i] >> (16 * kg)) & 0xFFFFull) << 16);
                    mine = (r16 == (NTD / 2) * i + np) ? word : mine;
                }
            }
        }
        // lanes 0 .. 2 NTD - 1 of a group of 16 hold the words of its four rows, in the order they lie in memory
        if (bits && r16 < 2 * NTD) {
            const int i = r16 / (NTD / 2);
            if (FULL || (qok && v0 + i < NvOut)) bits[v0 * (Cd / 32) + r16] = mine;
        }
        // (the next pass writes the tile again: its reads above are complete, the values sit in registers)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    auto bounds = [&](int64_t gg, int &a, int &b) {
        a = 0; b = 0;
        const int64_t v = 4 * gg + j;
        if (gg < gend && v < NvOut) { a = rowptr[v]; b = rowptr[v + 1]; }
    };
    int e0, e1, ne0, ne1;
    bounds(g, e0, e1);
    bounds(g + gstride, ne0, ne1);
    int f = (e0 + s < e1) ? colidx[e0 + s] / 3 : -1;
    int q4 = 0;                                                 // passes parked in the tile

    for (; g < gend; g += gstride) {
        int me0, me1;
        bounds(g + 2 * gstride, me0, me1);
        const int nf = (ne0 + s < ne1) ? colidx[ne0 + s] / 3 : -1;
        const int64_t vs = 4 * g + 2 * h;
        const int cnt0 = (vs < NvOut) ? nfcount[vs] : 1, cnt1 = (vs + 1 < NvOut) ? nfcount[vs + 1] : 1;
        const unsigned long long has = __builtin_amdgcn_ballot_w64(e1 > e0);

        float acc[NCB][4];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[cb][q] = 0.f;

        for (int p = 0;; ++p) {
            if (p > 0) f = (e0 + 8 * p + s < e1) ? colidx[e0 + 8 * p + s] / 3 : -1;
            float a[8];
            {
                float4 t0 = make_float4(0.f, 0.f, 0.f, 0.f), t1 = t0;
                if (f >= 0) {
                    const float4 *cp = reinterpret_cast<const float4 *>(coeff + (int64_t)f * 16 + 8 * h);
                    t0 = cp[0]; t1 = cp[1];
                }
                a[0] = t0.x; a[1] = t0.y; a[2] = t0.z; a[3] = t0.w;
                a[4] = t1.x; a[5] = t1.y; a[6] = t1.z; a[7] = t1.w;
            }
            const unsigned boff = (f >= 0) ? (unsigned)f * row_bytes : in_bytes;
            unsigned b[16];
#pragma unroll
            for (int i = 0; i < 16; ++i)
                b[i] = (unsigned)__builtin_amdgcn_ds_bpermute((8 * (i >> 2) + 4 * h + (i & 3)) * 4, (int)boff);
            unsigned xr[NCB][16];
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int i = 0; i < 16; ++i) xr[cb][i] = ld_buf(in_buf, b[i] + chb[cb], float());
            float m = 0.f;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(a[kk]));
            float inv_alpha;
            const float alpha = pow2_scale(hwave_fmax(m), &inv_alpha);
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) a[kk] *= alpha;
            u32x4 ah, al;
            split8h(a, ah, al);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const float unscale = inv_alpha * inv_beta[cb];
                f32x16 d;
#pragma unroll
                for (int i = 0; i < 16; ++i) d[i] = 0.f;
                d = mfma_f16(al, bh[cb], d);
                d = mfma_f16(ah, bl[cb], d);
                d = mfma_f16(ah, bh[cb], d);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float t = 0.f;
#pragma unroll
                    for (int i = 4 * q; i < 4 * q + 4; ++i) t = fmaf(d[i], __builtin_bit_cast(float, xr[cb][i]), t);
                    acc[cb][q] = fmaf(t, unscale, acc[cb][q]);
                }
            }
            if (!__builtin_amdgcn_ballot_w64(e0 + 8 * (p + 1) < e1)) break;
        }

        const float inv0 = ((has >> (8 * (2 * h))) & 1ull) ? 1.0f / (float)cnt0 : 0.f;
        const float inv1 = ((has >> (8 * (2 * h + 1))) & 1ull) ? 1.0f / (float)cnt1 : 0.f;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            half_swap(acc[cb][0], acc[cb][2]);
            half_swap(acc[cb][1], acc[cb][3]);
            const float o0 = (acc[cb][0] + acc[cb][2]) * inv0, o1 = (acc[cb][1] + acc[cb][3]) * inv1;
            const int co = 32 * cb + col;
            if (conv_out) {
                if (vs < NvOut) conv_out[vs * Co + co] = o0;
                if (vs + 1 < NvOut) conv_out[(vs + 1) * Co + co] = o1;
            }
            stage[(4 * q4 + 2 * h) * kRow + co] = o0;
            stage[(4 * q4 + 2 * h + 1) * kRow + co] = o1;
        }
        if (++q4 == 4) {
            if (4 * g + 3 < NvOut) flush(std::true_type(), g, 4);
            else flush(std::false_type(), g, 4);
            q4 = 0;
        }
        e0 = ne0; e1 = ne1; ne0 = me0; ne1 = me1;
        f = nf;
    }
    if (q4) flush(std::false_type(), g - gstride, q4);
}


// ----------------------------------------------------------------------------------------
// Backward.  A wavefront takes 32 consecutive facets (rows); per 32-channel block
//     w  = coeff_tile (32 x 16) * filt (16 x 32)                      8 MFMAs, as in the forward
//     s  = sum over the three corners of gout[vo, co] / nf[vo]         gathered, lane = channel
//     gin[f, co/R] = sum over the R outputs of a channel of s * w
//     gfilt[k, co] += coeff_tile^T (16 x 32) * (in * s) (32 x 32)      16 MFMAs, two facets each; rows
//                                                                      16..31 of the product are unused
// Register i of lane (col, h) is facet 8(i/4) + 4h + i%4 of the tile in every one of these.  The
// per-facet corner data (byte offset of the gout row, 1 / nf) go through a small LDS table that each
// wavefront writes for its own tile; the index chain face -> vt_map -> nf_count runs three tiles ahead.
// Workgroups own contiguous facet ranges (fixed by the problem size only) and leave one partial filter
// gradient each, summed by reduce_partials in a fixed order.
// H2: both products as two-piece fp16 products (3 + 6 instructions of 32 cycles per tile and channel block instead of
// 8 + 16 of 64): the tile's coefficients share one power-of-two scale in both of their layouts, every filter column
// and every channel of in * s has its own, and the second product of a tile is taken out of its scales before it
// joins the running filter gradient.
template <int NCB, int R, typename TIO, bool H2>
__global__ __launch_bounds__(kBlock, 2) void f2v_bwd_mfma_k(const TIO *__restrict__ gout, const TIO *__restrict__ in,
                                                         const float *__restrict__ filt,
                                                         const float *__restrict__ coeff,
                                                         const int *__restrict__ face,
                                                         const int *__restrict__ nfcount,
                                                         const int *__restrict__ vtmap, TIO *__restrict__ gin,
                                                         float *__restrict__ partial, int64_t Nf, int64_t NvOut, int C,
                                                         int Co, int64_t rows_per_block)
{
    __shared__ uint4 meta[4][32][2];
    __shared__ float red[4][NCB * 8][64];
    const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = l & 31, h = l >> 5;
    const int co0 = blockIdx.y * (32 * NCB);
    const int G = gridDim.x;
    // contiguous ranges per die (workgroups go round-robin over the eight dies)
    const int64_t rb = (G & 7) ? blockIdx.x : (int64_t)(blockIdx.x & 7) * (G >> 3) + (blockIdx.x >> 3);
    const int64_t fbeg = rb * rows_per_block;
    const int64_t fend = (fbeg + rows_per_block < Nf) ? fbeg + rows_per_block : Nf;
    const unsigned in_row = (unsigned)C * (unsigned)sizeof(TIO), out_row = (unsigned)Co * (unsigned)sizeof(TIO);
    // Gathers go through buffer descriptors: an offset at or past a descriptor's size reads zero, so neither the rows
    // beyond this workgroup's range (the feature and coefficient descriptors end at its last facet) nor the corners
    // without an output vertex (offset = the size of gout) need a branch, a compare or a zero per fetch.
    const unsigned gout_bytes = (unsigned)NvOut * out_row;
    const buffer_t gout_buf = buffer_of(gout, gout_bytes);
    const buffer_t in_buf = buffer_of(in, (unsigned)(fend > 0 ? fend : 0) * in_row);
    const buffer_t coeff_buf = buffer_of(coeff, (unsigned)(fend > 0 ? fend : 0) * 64u);

    float wb[NCB][8];
    unsigned chb[NCB], cob[NCB], xsel[NCB], gsel[NCB];
    bool con[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int co = co0 + 32 * cb + col;
        con[cb] = co < Co;
        chb[cb] = con[cb] ? (unsigned)(co / R) * (unsigned)sizeof(TIO) : 0u;
        cob[cb] = con[cb] ? (unsigned)co * (unsigned)sizeof(TIO) : 0u;
        xsel[cb] = half_sel(chb[cb]);
        gsel[cb] = half_sel(cob[cb]);
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) wb[cb][kk] = con[cb] ? filt[(size_t)(8 * h + kk) * Co + co] : 0.f;
    }
    f32x16 d2[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) d2[cb][i] = 0.f;
    // (H2) every filter column under its own power-of-two scale: a column of small weights keeps its accuracy beside a large one
    u32x4 bh[NCB], bl[NCB];
    float inv_beta[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        inv_beta[cb] = 1.f;
        if constexpr (H2) {
            float m = 0.f;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(wb[cb][kk]));
            m = fmaxf(m, __shfl_xor(m, 32, 64));                       // the column's other eight coefficients
            const float beta = pow2_scale(m, &inv_beta[cb]);
            float t[8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) t[kk] = wb[cb][kk] * beta;
            split8h(t, bh[cb], bl[cb]);
        }
    }

    auto ld_face = [&](int64_t f0, int (&va)[3]) {
        const int64_t f = f0 + col;
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) va[jj] = (f < fend) ? face[3 * f + jj] : -1;
    };
    auto ld_vo = [&](const int (&va)[3], int (&vo)[3]) {
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) {
            const int t = (va[jj] >= 0) ? vtmap[va[jj]] : -1;
            vo[jj] = (t >= 0 && t < NvOut) ? t : -1;
        }
    };
    auto ld_cnt = [&](const int (&vo)[3], int (&cnt)[3]) {
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) cnt[jj] = (vo[jj] >= 0) ? nfcount[vo[jj]] : 1;
    };

    constexpr int kStep = 4 * 32;                       // facets per workgroup step
    int64_t f0 = fbeg + 32 * wave;
    int vo_c[3], cnt_c[3], vo_n[3], va_nn[3];
    {
        int va[3];
        ld_face(f0, va); ld_vo(va, vo_c); ld_cnt(vo_c, cnt_c);
        ld_face(f0 + kStep, va); ld_vo(va, vo_n);
        ld_face(f0 + 2 * kStep, va_nn);
    }
    for (; f0 < fend; f0 += kStep) {
        int cnt_n[3], vo_nn[3], va_3[3];
        ld_cnt(vo_n, cnt_n);
        ld_vo(va_nn, vo_nn);
        ld_face(f0 + 3 * kStep, va_3);

        // corner table of my tile
        if (h == 0) {
            uint4 m0, m1;
            m0.x = (vo_c[0] >= 0) ? (unsigned)vo_c[0] * out_row : gout_bytes;
            m0.y = (vo_c[1] >= 0) ? (unsigned)vo_c[1] * out_row : gout_bytes;
            m0.z = (vo_c[2] >= 0) ? (unsigned)vo_c[2] * out_row : gout_bytes;
            m0.w = 0u;
            m1.x = __float_as_uint((vo_c[0] >= 0) ? 1.0f / (float)cnt_c[0] : 0.f);
            m1.y = __float_as_uint((vo_c[1] >= 0) ? 1.0f / (float)cnt_c[1] : 0.f);
            m1.z = __float_as_uint((vo_c[2] >= 0) ? 1.0f / (float)cnt_c[2] : 0.f);
            m1.w = 0u;
            meta[wave][col][0] = m0;
            meta[wave][col][1] = m1;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // A operands: my row's coefficients 8h .. 8h+7 (first product); coefficient `col` of the facets my
        // registers pair with (second product, lanes col < 16)
        const bool rok = f0 + col < fend;
        float a1[8], a2[16];
        {
            float4 t0 = make_float4(0.f, 0.f, 0.f, 0.f), t1 = t0;
            if (rok) {
                const float4 *cp = reinterpret_cast<const float4 *>(coeff + (f0 + col) * 16 + 8 * h);
                t0 = cp[0]; t1 = cp[1];
            }
            a1[0] = t0.x; a1[1] = t0.y; a1[2] = t0.z; a1[3] = t0.w;
            a1[4] = t1.x; a1[5] = t1.y; a1[6] = t1.z; a1[7] = t1.w;
        }
        {
            // (lanes col >= 16 hold no coefficient: an offset that stays past the end with the row steps added)
            const unsigned cbase = col < 16 ? (unsigned)(f0 + 4 * h) * 64u + 4u * col : 0x80000000u;
#pragma unroll
            for (int i = 0; i < 16; ++i)
                a2[i] = __builtin_bit_cast(float, ld_buf(coeff_buf, cbase + (8 * (i >> 2) + (i & 3)) * 64u, float()));
        }

        float sv[NCB][16], xv[NCB][16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int ri = 8 * (i >> 2) + 4 * h + (i & 3);
            const uint4 m0 = meta[wave][ri][0], m1 = meta[wave][ri][1];
            const unsigned xoff = (unsigned)(f0 + ri) * in_row;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const unsigned r0 = ld_buf(gout_buf, m0.x + cob[cb], TIO()), r1 = ld_buf(gout_buf, m0.y + cob[cb], TIO());
                const unsigned r2 = ld_buf(gout_buf, m0.z + cob[cb], TIO()), rx = ld_buf(in_buf, xoff + chb[cb], TIO());
                // (row offsets are multiples of 4 bytes: the half of the word depends on the column only)
                const float g0 = cvt_raw(r0, gsel[cb], TIO()), g1 = cvt_raw(r1, gsel[cb], TIO()), g2 = cvt_raw(r2, gsel[cb], TIO());
                sv[cb][i] = fmaf(g2, __uint_as_float(m1.z), fmaf(g1, __uint_as_float(m1.y), g0 * __uint_as_float(m1.x)));
                xv[cb][i] = cvt_raw(rx, xsel[cb], TIO());
            }
        }
        // (H2) the tile's coefficients, in both layouts, under one scale
        u32x4 a1h, a1l, a2h[2], a2l[2];
        float inv_alpha = 1.f;
        if constexpr (H2) {
            float m = 0.f;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) m = fmaxf(m, fabsf(a1[kk]));
            const float alpha = pow2_scale(hwave_fmax(m), &inv_alpha);      // (every lane of the wavefront is here)
            float t[8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) t[kk] = a1[kk] * alpha;
            split8h(t, a1h, a1l);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) t[kk] = a2[8 * g + kk] * alpha;
                split8h(t, a2h[g], a2l[g]);
            }
        }
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            f32x16 d;
#pragma unroll
            for (int i = 0; i < 16; ++i) d[i] = 0.f;
            if constexpr (H2) {
                d = mfma_f16(a1l, bh[cb], d);
                d = mfma_f16(a1h, bl[cb], d);
                d = mfma_f16(a1h, bh[cb], d);
                const float unscale = inv_alpha * inv_beta[cb];
#pragma unroll
                for (int i = 0; i < 16; ++i) d[i] *= unscale;
            } else {
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) d = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[kk], wb[cb][kk], d, 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int ri = 8 * (i >> 2) + 4 * h + (i & 3);
                float gi = sv[cb][i] * d[i];
                if constexpr (R == 2)          // the two outputs of an input channel sit in neighbouring lanes
                    gi += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, gi), 0xB1, 0xF, 0xF, true));
                // R == 2: the even lanes hold the channels, neighbouring channels sit two lanes apart
                st1_pair<R>(const_cast<TIO *>(at_bytes(gin, (unsigned)(f0 + ri) * in_row + chb[cb])), gi,
                            f0 + ri < fend && con[cb] && (R == 1 || !(col & 1)), col);
            }
            if constexpr (H2) {
                float D[16], m = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    D[i] = xv[cb][i] * sv[cb][i];
                    m = fmaxf(m, fabsf(D[i]));
                }
                m = fmaxf(m, __shfl_xor(m, 32, 64));                     // my channel's other sixteen facets
                float inv_delta;
                const float delta = pow2_scale(m, &inv_delta);            // one scale per channel
                f32x16 t2;
#pragma unroll
                for (int i = 0; i < 16; ++i) t2[i] = 0.f;
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    float t[8];
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) t[kk] = D[8 * g + kk] * delta;
                    u32x4 Dh, Dl;
                    split8h(t, Dh, Dl);
                    t2 = mfma_f16(a2l[g], Dh, t2);
                    t2 = mfma_f16(a2h[g], Dl, t2);
                    t2 = mfma_f16(a2h[g], Dh, t2);
                }
                const float unscale2 = inv_alpha * inv_delta;
#pragma unroll
                for (int q = 0; q < 8; ++q) d2[cb][q] = fmaf(t2[q], unscale2, d2[cb][q]);      // (rows 0..15: the coefficients)
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    d2[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a2[i], xv[cb][i] * sv[cb][i], d2[cb], 0, 0, 0);
            }
        }
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) { vo_c[jj] = vo_n[jj]; cnt_c[jj] = cnt_n[jj]; vo_n[jj] = vo_nn[jj]; va_nn[jj] = va_3[jj]; }
    }

    // sum the four wavefronts' products; rows 0..15 (registers 0..7) are the 16 coefficients
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int q = 0; q < 8; ++q) red[wave][cb * 8 + q][l] = d2[cb][q];
    __syncthreads();
    for (int idx = threadIdx.x; idx < NCB * 8 * 64; idx += kBlock) {
        const int ll = idx & 63, cq = idx >> 6, cb = cq >> 3, q = cq & 7;
        const int k = 8 * (q >> 2) + 4 * (ll >> 5) + (q & 3), co = co0 + 32 * cb + (ll & 31);
        const float v = (red[0][cq][ll] + red[1][cq][ll]) + (red[2][cq][ll] + red[3][cq][ll]);
        if (co < Co) partial[((size_t)blockIdx.x * 16 + k) * Co + co] = v;
    }
}

bool f2v_mfma_ok(int64_t Nf, int C, int r, int K, const void *coeff)
{
    // (32-bit byte offsets into the feature array, with room for one row past the end)
    return K == 16 && C * r >= 32 && (reinterpret_cast<uintptr_t>(coeff) & 15) == 0 && (Nf + 1) * (int64_t)C < (int64_t(1) << 30);
}

template <typename TIO>
static void f2v_fwd_launch(const TIO *in, const float *filt, const float *coeff, const int *nfcount, const int *rowptr,
                           const int *colidx, TIO *out, int64_t Nf, int64_t NvOut, int C, int r, hipStream_t st)
{
    const int Co = C * r;
    const unsigned in_bytes = (unsigned)(Nf * C * (int64_t)sizeof(TIO));
    const int ncb = Co <= 32 ? 1 : Co <= 64 ? 2 : Co <= 96 ? 3 : 2;      // wider rows: chunks of 64 channels (more wavefronts in flight)
    const unsigned gy = (unsigned)ceil_div(Co, 32 * ncb);
    const int64_t want = ceil_div(ceil_div(NvOut, 16), 8) * 8;            // 16 vertices per workgroup sweep
    const unsigned gxn = (unsigned)(want < 4096 ? want : 4096);
    const dim3 grid(gxn, gy), block(kBlock);
#define PM_F2V_FWD(N, H) f2v_fwd_mfma_k<N, TIO, H><<<grid, block, 0, st>>>(in, filt, coeff, nfcount, rowptr, colidx, out, NvOut, C, r, Co, in_bytes)
    if (options().f2v_fp32mfma) {
        switch (ncb) {
        case 1: PM_F2V_FWD(1, false); break;
        case 2: PM_F2V_FWD(2, false); break;
        default: PM_F2V_FWD(3, false); break;
        }
    } else {
        switch (ncb) {
        case 1: PM_F2V_FWD(1, true); break;
        case 2: PM_F2V_FWD(2, true); break;
        default: PM_F2V_FWD(3, true); break;
        }
    }
#undef PM_F2V_FWD
}

int f2v_fwd_mfma(const void *in, const float *filt, const float *coeff, const int *nfcount, const int *rowptr,
                 const int *colidx, void *out, int64_t Nf, int64_t NvOut, int C, int r, hipStream_t st, bool bf16)
{
    if (bf16) f2v_fwd_launch((const bf16_t *)in, filt, coeff, nfcount, rowptr, colidx, (bf16_t *)out, Nf, NvOut, C, r, st);
    else f2v_fwd_launch((const float *)in, filt, coeff, nfcount, rowptr, colidx, (float *)out, Nf, NvOut, C, r, st);
    PM_LAUNCHED("f2v_fwd(mfma)");
    return 0;
}


bool f2v_tail_ok(int64_t Nf, int C, int r, int K, const void *coeff, int Cd)
{
    const int Co = C * r;
    return f2v_mfma_ok(Nf, C, r, K, coeff) && (Co == 32 || Co == 64) && (Cd == 32 || Cd == 64 || Cd == 128);
}

size_t f2v_tail_workspace_bytes(int Co, int Cd) { return (size_t)(Co / 32) * (Cd / 16) * 2 * 64 * sizeof(u32x4) + (size_t)4 * Cd * sizeof(float); }

int f2v_fwd_tail(const float *in, const float *filt, const float *coeff, const int *nfcount, const int *rowptr,
                 const int *colidx, float *conv_out, const float *Wd, const float *bias, const float *scale, const float *shift,
                 int relu, float *out2, unsigned *bits, void *workspace, int64_t Nf, int64_t NvOut, int C, int r, int Cd,
                 hipStream_t st)
{
    const int Co = C * r, ncb = Co / 32, ntd = Cd / 16;
    u32x4 *Wp = (u32x4 *)workspace;
    float *meta = (float *)(Wp + (size_t)ncb * ntd * 2 * 64);
    f2v_tail_pack_k<<<dim3((unsigned)ceil_div(ncb * ntd * 64, kBlock)), dim3(kBlock), 0, st>>>(Wd, bias, scale, shift, Wp, meta, Co, Cd, ncb, ntd);
    PM_LAUNCHED("f2v_dense_fwd(pack)");
    const unsigned in_bytes = (unsigned)(Nf * C * (int64_t)sizeof(float));
    const int64_t want = ceil_div(ceil_div(NvOut, 16), 8) * 8;
    const unsigned gxn = (unsigned)(want < 4096 ? want : 4096);
    const dim3 grid(gxn), block(kBlock);
#define PM_F2V_TAIL(N, T) f2v_fwd_tail_k<N, T><<<grid, block, 0, st>>>(in, filt, coeff, nfcount, rowptr, colidx, conv_out, Wp, meta, out2, bits, relu, NvOut, C, r, in_bytes)
    if (ncb == 1) {
        if (ntd == 2) PM_F2V_TAIL(1, 2); else if (ntd == 4) PM_F2V_TAIL(1, 4); else PM_F2V_TAIL(1, 8);
    } else {
        if (ntd == 2) PM_F2V_TAIL(2, 2); else if (ntd == 4) PM_F2V_TAIL(2, 4); else PM_F2V_TAIL(2, 8);
    }
#undef PM_F2V_TAIL
    PM_LAUNCHED("f2v_dense_fwd");
    return 0;
}


// rows_per_block and the workgroup count depend on the problem size only (fixed summation order).
int f2v_bwd_mfma_blocks(int64_t Nf) { return persistent_blocks(Nf, 128); }

template <typename TIO>
static void f2v_bwd_launch(const TIO *gout, const TIO *in, const float *filt, const float *coeff, const int *face,
                           const int *nfcount, const int *vtmap, TIO *gin, float *partial, int G, int64_t Nf, int64_t NvOut,
                           int C, int r, hipStream_t st)
{
    const int Co = C * r;
    // one 32-channel block per workgroup column: two wavefronts per SIMD fit, which beats sharing the
    // index chain between two blocks at one wavefront per SIMD
    const unsigned gy = (unsigned)ceil_div(Co, 32);
    const int64_t rows_per_block = ceil_div(ceil_div(Nf, G), 128) * 128;
    const dim3 grid((unsigned)G, gy), block(kBlock);
#define PM_F2V_BWD(RR, H) f2v_bwd_mfma_k<1, RR, TIO, H><<<grid, block, 0, st>>>(gout, in, filt, coeff, face, nfcount, vtmap, gin, partial, Nf, NvOut, C, Co, rows_per_block)
    if (options().f2v_fp32mfma) {
        if (r == 1) PM_F2V_BWD(1, false);
        else PM_F2V_BWD(2, false);
    } else {
        if (r == 1) PM_F2V_BWD(1, true);
        else PM_F2V_BWD(2, true);
    }
#undef PM_F2V_BWD
}

int f2v_bwd_mfma(const void *gout, const void *in, const float *filt, const float *coeff, const int *face,
                 const int *nfcount, const int *vtmap, void *gin, float *partial, int G, int64_t Nf, int64_t NvOut,
                 int C, int r, hipStream_t st, bool bf16)
{
    if (bf16)
        f2v_bwd_launch((const bf16_t *)gout, (const bf16_t *)in, filt, coeff, face, nfcount, vtmap, (bf16_t *)gin, partial, G, Nf, NvOut, C, r, st);
    else
        f2v_bwd_launch((const float *)gout, (const float *)in, filt, coeff, face, nfcount, vtmap, (float *)gin, partial, G, Nf, NvOut, C, r, st);
    PM_LAUNCHED("f2v_bwd(mfma)");
    return 0;
}

}  // namespace pmesh
