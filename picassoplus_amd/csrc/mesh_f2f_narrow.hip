// facet2facet for narrow inputs (at most four input channels, 16 SH coefficients) -- the colour input of a network's
// first block: G[f,ci,d] = (1/K_f) sum_k tex[k,ci] * sh[k,d] has only Cin * 16 <= 64 columns per facet, so both kernels
// are streams over the SH rows, the texture rows and gout / out, with the products on the fp16 matrix instruction.
#include "common.h"
#include "f2f_internal.h"
#include "fp16_split.h"

namespace pmesh {

// Filter gradient gW[co][ci][d] = sum_f gout[f,co] * G[f,ci,d] with the facet as the reduction index of the fp16 matrix
// instruction (16 facets per step), both operands split into two fp16 pieces:
//   wavefront  a contiguous run of 32-facet tiles.  Lane (facet m, half h) forms the 32 G values of its facet and half
//              (columns (ci = c, d = 8h + q), as the forward does: 32 bytes of each SH row, the point's texture
//              values, five points in flight), scaled by one power of two for the tile, into the wavefront's LDS
//              stage [facet][column]
//   product    gW^T tile (32 columns x 32 output channels) += G^T (32 columns x 16 facets) . gout (16 facets x 32):
//              A = the stage read by columns (lane = column, conflict-free), B = gout rows fetched through a buffer
//              descriptor that ends at the wavefront's last facet (lane = output channel, one power of two per
//              channel and tile); 2 column tiles x 2 facet steps x 3 piece products per tile; the tile's product is
//              taken out of its scales as it joins the running sums
//   workgroup  4 wavefronts, summed through LDS into one partial gradient per workgroup
typedef __amdgpu_buffer_rsrc_t narrow_buffer_t;
constexpr int kNarrowPitch = 68;      // floats per stage row: 64 columns + 4 (the rows of 16 lanes fall on different banks)

template <int NT>
__global__ __launch_bounds__(kBlock) void f2f_bwd_filt_narrow_h2_k(const float *__restrict__ gout, const float *__restrict__ tex,
                                                                   const float *__restrict__ sh, const int *__restrict__ cum,
                                                                   float *__restrict__ partial, int64_t Nf, int T, int Cin,
                                                                   int Cout, int64_t tiles_per_wave)
{
    constexpr int KU = 5;
    __shared__ __attribute__((aligned(16))) float stage[4][32 * kNarrowPitch];
    const int l = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // (a scalar: the descriptor below is built from it)
    const int m = l & 31, h = l >> 5;
    const int n0 = blockIdx.y * (32 * NT);
    const int64_t ntiles = (Nf + 31) >> 5;
    const int64_t tbeg = ((int64_t)blockIdx.x * 4 + wave) * tiles_per_wave;
    const int64_t tend = (tbeg + tiles_per_wave < ntiles) ? tbeg + tiles_per_wave : ntiles;
    const int64_t fend = tend * 32 < Nf ? tend * 32 : Nf;           // my wavefront's facets end here
    const int MT = Cin > 2 ? 2 : 1;                                 // column tiles in use (ci = 2 mt, 2 mt + 1)
    float *st = stage[wave];
    // gout through a descriptor that ends at my last facet: rows beyond read zero; lanes without a channel too
    const unsigned row_bytes = (unsigned)Cout * 4u;
    const narrow_buffer_t gbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(gout), 0,
                                                                   (int)((unsigned)(fend > 0 ? fend : 0) * row_bytes), 0x00020000);
    unsigned cob[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) cob[nt] = (n0 + 32 * nt + m < Cout) ? (unsigned)(n0 + 32 * nt + m) * 4u : 0x80000000u;

    f32x16 acc[2][NT];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

    auto bounds = [&](int64_t tile, int &a, int &b) {
        const int64_t f = tile * 32 + m;
        a = 0; b = 0;
        if (tile < tend && f < Nf) {
            a = f ? cum[f - 1] : 0;
            b = cum[f];
        }
        a = a < 0 ? 0 : (a > T ? T : a);
        b = b < a ? a : (b > T ? T : b);
    };
    int k0, k1;
    bounds(tbeg, k0, k1);
    for (int64_t tile = tbeg; tile < tend; ++tile) {
        int nk0, nk1;
        bounds(tile + 1, nk0, nk1);
        // B operands: gout of the facets 16 ks + 8h + j of the tile, my channel(s)
        float gv[NT][2][8];
        {
            const unsigned base = (unsigned)(tile * 32 + 8 * h) * row_bytes;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        gv[nt][ks][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                            gbuf, (int)(base + (unsigned)(16 * ks + j) * row_bytes + cob[nt]), 0, 0));
        }
        const int K = k1 - k0;
        float G[4][8];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int q = 0; q < 8; ++q) G[c][q] = 0.f;
        for (int kb = 0; kb == 0 || __builtin_amdgcn_ballot_w64(kb < K) != 0ull; kb += KU) {
            float4 su[KU], sv[KU];
            float tv[KU][4];
#pragma unroll
            for (int u = 0; u < KU; ++u) {
                const bool on = kb + u < K;
                const int64_t pt = k0 + kb + u;
                su[u] = on ? *reinterpret_cast<const float4 *>(sh + pt * 16 + 8 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
                sv[u] = on ? *reinterpret_cast<const float4 *>(sh + pt * 16 + 8 * h + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int c = 0; c < 4; ++c) tv[u][c] = (on && c < Cin) ? tex[pt * Cin + c] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < KU; ++u)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    G[c][0] = fmaf(tv[u][c], su[u].x, G[c][0]); G[c][1] = fmaf(tv[u][c], su[u].y, G[c][1]);
                    G[c][2] = fmaf(tv[u][c], su[u].z, G[c][2]); G[c][3] = fmaf(tv[u][c], su[u].w, G[c][3]);
                    G[c][4] = fmaf(tv[u][c], sv[u].x, G[c][4]); G[c][5] = fmaf(tv[u][c], sv[u].y, G[c][5]);
                    G[c][6] = fmaf(tv[u][c], sv[u].z, G[c][6]); G[c][7] = fmaf(tv[u][c], sv[u].w, G[c][7]);
                }
        }
        const float invK = K > 0 ? 1.0f / (float)K : 0.f;
        float gm = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                G[c][q] *= invK;
                gm = fmaxf(gm, fabsf(G[c][q]));
            }
        float inv_alpha;
        const float alpha = pow2_scale(hwave_fmax(gm), &inv_alpha);          // (every lane of the wavefront is here)
        // the scaled G values into the stage: row = my facet, columns 16c + 8h + q
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");              // the readers of the tile before are done
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float *d = st + m * kNarrowPitch + 16 * c + 8 * h;
            *reinterpret_cast<float4 *>(d) = make_float4(G[c][0] * alpha, G[c][1] * alpha, G[c][2] * alpha, G[c][3] * alpha);
            *reinterpret_cast<float4 *>(d + 4) = make_float4(G[c][4] * alpha, G[c][5] * alpha, G[c][6] * alpha, G[c][7] * alpha);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // B pieces: one scale per output channel and tile
        u32x4 gh[NT][2], gl[NT][2];
        float unscale[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float mx = 0.f;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int j = 0; j < 8; ++j) mx = fmaxf(mx, fabsf(gv[nt][ks][j]));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            float inv_delta;
            const float delta = pow2_scale(mx, &inv_delta);
            unscale[nt] = inv_alpha * inv_delta;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float t[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) t[j] = gv[nt][ks][j] * delta;
                split8h(t, gh[nt][ks], gl[nt][ks]);
            }
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            if (mt >= MT) break;
            u32x4 ah[2], al[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                float t[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) t[j] = st[(16 * ks + 8 * h + j) * kNarrowPitch + 32 * mt + m];
                split8h(t, ah[ks], al[ks]);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                f32x16 t2;
#pragma unroll
                for (int i = 0; i < 16; ++i) t2[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    t2 = mfma_f16(al[ks], gh[nt][ks], t2);
                    t2 = mfma_f16(ah[ks], gl[nt][ks], t2);
                    t2 = mfma_f16(ah[ks], gh[nt][ks], t2);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[mt][nt][i] = fmaf(t2[i], unscale[nt], acc[mt][nt][i]);
            }
        }
        k0 = nk0; k1 = nk1;
    }

    // accumulator (mt, nt): lane (co = n0 + 32nt + m, half h), register i <-> column 32 mt + 8(i/4) + 4h + i%4 = 16 ci + d
    float *dst = partial + (size_t)blockIdx.x * Cout * Cin * 16;
    float *red = &stage[0][0];                                          // 4 x 16 x 64 floats
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 16; ++i) red[(wave * 16 + i) * 64 + l] = acc[mt][nt][i];
            __syncthreads();
            for (int idx = threadIdx.x; idx < 16 * 64; idx += kBlock) {
                const int ll = idx & 63, i = idx >> 6;
                const int col = 32 * mt + 8 * (i >> 2) + 4 * (ll >> 5) + (i & 3);
                const int cc = col >> 4, dd = col & 15, co = n0 + 32 * nt + (ll & 31);
                const float v = (red[(0 * 16 + i) * 64 + ll] + red[(1 * 16 + i) * 64 + ll]) + (red[(2 * 16 + i) * 64 + ll] + red[(3 * 16 + i) * 64 + ll]);
                if (cc < Cin && co < Cout) dst[((size_t)co * Cin + cc) * 16 + dd] = v;
            }
        }
}

bool f2f_narrow_usable(int Cin, int F) { return F == 16 && Cin <= 4; }       // plus 16-byte aligned SH rows, checked by the caller
// the filter gradient addresses gout with 32-bit byte offsets (and one that marks a lane without a channel)
bool f2f_narrow_bwd_usable(int Cin, int F, int64_t Nf, int Cout) { return f2f_narrow_usable(Cin, F) && Nf * (int64_t)Cout < (int64_t(1) << 29); }

// Workgroup count: a function of the facet count only (fixed summation order on any device).
int f2f_narrow_blocks(int64_t Nf)
{
    int64_t b = ceil_div(Nf, 512);
    if (b < 1) b = 1;
    if (b > kNarrowMaxBlocks) b = kNarrowMaxBlocks;
    return (int)b;
}

int f2f_bwd_filter_narrow_partials(const float *gout, const float *tex, const float *sh, const int *cum, float *partial,
                                   int blocks, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st)
{
    const int nt = Cout <= 32 ? 1 : 2;
    const int64_t gy = ceil_div(Cout, 32 * nt);
    PM_REQUIRE(gy <= 65535, "f2f_bwd_filter: grid too large");
    const dim3 grid((unsigned)blocks, (unsigned)gy);
    const int64_t tpw = ceil_div(ceil_div(Nf, 32), (int64_t)blocks * 4);
    if (nt == 1)
        f2f_bwd_filt_narrow_h2_k<1><<<grid, dim3(kBlock), 0, st>>>(gout, tex, sh, cum, partial, Nf, (int)T, Cin, Cout, tpw);
    else
        f2f_bwd_filt_narrow_h2_k<2><<<grid, dim3(kBlock), 0, st>>>(gout, tex, sh, cum, partial, Nf, (int)T, Cin, Cout, tpw);
    PM_LAUNCHED("f2f_bwd_filter(narrow)");
    return 0;
}


// ----------------------------------------------------------------------------------------
// Forward for the same narrow inputs: out[f, co] = sum_(ci,d) G[f,ci,d] * W[co,ci,d] on the fp16 matrix instruction
// with both operands split into two fp16 pieces (three piece products), the reduction index running over the (at most)
// 64 columns (ci, d):
//   product    out tile (32 facets x 32 output channels) += G (32 facets x 16 columns) . W^T (16 columns x 32), one
//              step per input channel: step c, half h, element q <-> column (ci = c, d = 8h + q).  Every output
//              channel's weights carry their own power-of-two scale (set once), the G values of a tile one for the
//              wavefront; both leave the sums on the way out
//   lane       (facet l%32 of the tile, half h): forms the 32 G values of its half from the facet's points
//              (32 bytes of each SH row and the point's texture values); as B operand it holds W of output
//              channel l%32 for the same columns (registers, loaded once)
//   wavefront  a contiguous run of 32-facet tiles in natural order (sequential reads and writes), five points
//              per facet and round with all loads of a round in flight together
template <int NT>
__global__ __launch_bounds__(kBlock) void f2f_fwd_narrow_k(const float *__restrict__ tex, const float *__restrict__ W,
                                                           const float *__restrict__ sh, const int *__restrict__ cum,
                                                           float *__restrict__ out, int64_t Nf, int T, int Cin, int Cout,
                                                           int64_t tiles_per_wave)
{
    constexpr int KU = 5;
    const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = l & 31, h = l >> 5;
    const int n0 = blockIdx.y * (32 * NT);
    // B operands: pieces of beta * W[n0 + 32nt + m][c][8h .. 8h + 7] for the four steps c
    u32x4 bh[NT][4], bl[NT][4];
    float inv_beta[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int co = n0 + 32 * nt + m;
        float wv[4][8], mx = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                wv[c][q] = (co < Cout && c < Cin) ? W[((int64_t)co * Cin + c) * 16 + 8 * h + q] : 0.f;
                mx = fmaxf(mx, fabsf(wv[c][q]));
            }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                      // the channel's other half of the columns
        const float beta = pow2_scale(mx, &inv_beta[nt]);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int q = 0; q < 8; ++q) wv[c][q] *= beta;
            split8h(wv[c], bh[nt][c], bl[nt][c]);
        }
    }
    const int64_t ntiles = (Nf + 31) >> 5;
    const int64_t tbeg = ((int64_t)blockIdx.x * 4 + wave) * tiles_per_wave;
    const int64_t tend = (tbeg + tiles_per_wave < ntiles) ? tbeg + tiles_per_wave : ntiles;

    auto bounds = [&](int64_t tile, int &a, int &b) {
        const int64_t f = tile * 32 + m;
        a = 0; b = 0;
        if (tile < tend && f < Nf) {
            a = f ? cum[f - 1] : 0;
            b = cum[f];
        }
        a = a < 0 ? 0 : (a > T ? T : a);
        b = b < a ? a : (b > T ? T : b);
    };
    int k0, k1;
    bounds(tbeg, k0, k1);
    for (int64_t tile = tbeg; tile < tend; ++tile) {
        int nk0, nk1;
        bounds(tile + 1, nk0, nk1);
        const int K = k1 - k0;
        float G[4][8];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int q = 0; q < 8; ++q) G[c][q] = 0.f;
        for (int kb = 0; kb == 0 || __builtin_amdgcn_ballot_w64(kb < K) != 0ull; kb += KU) {
            float4 su[KU], sv[KU];
            float tv[KU][4];
#pragma unroll
            for (int u = 0; u < KU; ++u) {
                const bool on = kb + u < K;
                const int64_t pt = k0 + kb + u;
                su[u] = on ? *reinterpret_cast<const float4 *>(sh + pt * 16 + 8 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
                sv[u] = on ? *reinterpret_cast<const float4 *>(sh + pt * 16 + 8 * h + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int c = 0; c < 4; ++c) tv[u][c] = (on && c < Cin) ? tex[pt * Cin + c] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < KU; ++u)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    G[c][0] = fmaf(tv[u][c], su[u].x, G[c][0]); G[c][1] = fmaf(tv[u][c], su[u].y, G[c][1]);
                    G[c][2] = fmaf(tv[u][c], su[u].z, G[c][2]); G[c][3] = fmaf(tv[u][c], su[u].w, G[c][3]);
                    G[c][4] = fmaf(tv[u][c], sv[u].x, G[c][4]); G[c][5] = fmaf(tv[u][c], sv[u].y, G[c][5]);
                    G[c][6] = fmaf(tv[u][c], sv[u].z, G[c][6]); G[c][7] = fmaf(tv[u][c], sv[u].w, G[c][7]);
                }
        }
        const float invK = K > 0 ? 1.0f / (float)K : 0.f;
        float gm = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                G[c][q] *= invK;
                gm = fmaxf(gm, fabsf(G[c][q]));
            }
        float inv_alpha;
        const float alpha = pow2_scale(hwave_fmax(gm), &inv_alpha);      // (every lane of the wavefront is here)
        f32x16 acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nt][i] = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float t[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) t[q] = G[c][q] * alpha;
            u32x4 ah, al;
            split8h(t, ah, al);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                acc[nt] = mfma_f16(al, bh[nt][c], acc[nt]);
                acc[nt] = mfma_f16(ah, bl[nt][c], acc[nt]);
                acc[nt] = mfma_f16(ah, bh[nt][c], acc[nt]);
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const float unscale = inv_alpha * inv_beta[nt];
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nt][i] *= unscale;
        }
        // accumulator: lane (co = n0 + 32nt + m, half h), register i <-> facet 8(i/4) + 4h + i%4 of the tile
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int co = n0 + 32 * nt + m;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int64_t f = tile * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (f < Nf && co < Cout) out[f * Cout + co] = acc[nt][i];
            }
        }
        k0 = nk0; k1 = nk1;
    }
}

bool f2f_fwd_narrow_usable(int Cin, int F, const void *sh) { return F == 16 && Cin <= 4 && !(reinterpret_cast<uintptr_t>(sh) & 15u); }

int f2f_fwd_narrow(const float *tex, const float *W, const float *sh, const int *cum, float *out, int64_t T, int64_t Nf,
                   int Cin, int Cout, hipStream_t st)
{
    const int nt = Cout <= 32 ? 1 : 2;
    const int64_t gy = ceil_div(Cout, 32 * nt);
    PM_REQUIRE(gy <= 65535, "f2f_fwd: grid too large");
    const int64_t ntiles = ceil_div(Nf, 32);
    int64_t blocks = ceil_div(ntiles, 4 * 4);                 // at least four tiles per wavefront
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
    const int64_t tpw = ceil_div(ntiles, blocks * 4);
    const dim3 grid((unsigned)blocks, (unsigned)gy);
    if (nt == 1)
        f2f_fwd_narrow_k<1><<<grid, dim3(kBlock), 0, st>>>(tex, W, sh, cum, out, Nf, (int)T, Cin, Cout, tpw);
    else
        f2f_fwd_narrow_k<2><<<grid, dim3(kBlock), 0, st>>>(tex, W, sh, cum, out, Nf, (int)T, Cin, Cout, tpw);
    PM_LAUNCHED("f2f_fwd(narrow)");
    return 0;
}

}  // namespace pmesh
