// The pointwise tail of the mesh convolutions on the matrix cores (gfx950; v_mfma_f32_32x32x16_bf16 with both
// operands split exactly into three bf16 pieces, or v_mfma_f32_32x32x2_f32 behind a switch; fp32
// accumulators): out = act(rows . W + bias) [* scale + shift], and its gradients.  The
// reference runs this tail as separate PyTorch ops after every convolution (picasso/mesh/layers.py:114-119,
// 169-174, 232-238: matmul with depth_weights, + biases, activation, batch norm); here the bias, the ReLU and
// an inference-mode batch norm ride in the epilogue of the product, and the ReLU mask of the backward pass
// rides in the operand loads -- as one bit per entry that the forward's epilogue leaves behind, or read off
// the forward's output -- so every pass touches each feature row once.
#include "common.h"
#include "rows_internal.h"
#include "../../include/picasso_mesh.h"
#include <stdlib.h>

namespace pmesh {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Exact split of eight fp32 values into three bf16 pieces each (8 + 8 + 8 mantissa bits, by truncation), packed
// in the k order of v_mfma_f32_32x32x16_bf16.  Six piece products a1b1 + a1b2 + a2b1 + a1b3 + a2b2 + a3b1,
// accumulated in fp32, give the fp32 product to 2^-24: the matrix cores run them at a sixth of the bf16 rate,
// still 2.6 times the rate of the fp32 matrix instruction.
__device__ __forceinline__ unsigned dense_pack_hi(float a, float b)
{
    return __builtin_amdgcn_perm(__builtin_bit_cast(unsigned, b), __builtin_bit_cast(unsigned, a), 0x07060302u);
}
__device__ __forceinline__ float dense_trunc(float x)
{
    return __builtin_bit_cast(float, __builtin_bit_cast(unsigned, x) & 0xFFFF0000u);
}
__device__ __forceinline__ void dense_split8(const float (&x)[8], u32x4 &p1, u32x4 &p2, u32x4 &p3)
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float a = x[2 * j], b = x[2 * j + 1];
        p1[j] = dense_pack_hi(a, b);
        const float ra = a - dense_trunc(a), rb = b - dense_trunc(b);
        p2[j] = dense_pack_hi(ra, rb);
        p3[j] = dense_pack_hi(ra - dense_trunc(ra), rb - dense_trunc(rb));
    }
}
__device__ __forceinline__ f32x16 dense_mfma_bf16(const u32x4 &a, const u32x4 &b, const f32x16 &c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

constexpr int kDenseChunk = 64;            // reduction entries per register chunk (32 per lane half)
constexpr int kDenseSlabBytes = 48 * 1024;      // preferred weight slab of a four-wavefront workgroup in LDS
constexpr int kDenseSlabWideBytes = 88 * 1024;  // of an eight-wavefront workgroup
constexpr int kDenseSlabSixBytes = 104 * 1024;  // of a six-wavefront workgroup (split-bf16 products only)
constexpr size_t kDenseLdsMax = 160 * 1024;
constexpr int kDenseMaxK = 896;            // a 32-column slab of that length is 112 KiB, beside 34 KiB of row stages

// rows (N x K, row stride K) times Wm (K x C, element (k, c) at w[k * wk + c * wc]) for the NT * 32 columns
// of this workgroup's column block.  A wavefront owns 32 rows at a time.  It fetches a 32 x 64 block of them with
// fully coalesced loads (a 16-lane group per row), one block ahead of the arithmetic, and turns it into the
// operand layout of the matrix instruction (lane = row) through a private LDS stage: lane (r, h) reads entries
// h*32 .. h*32+31 of row r (the order of the reduction index is free as long as both operands agree).  The
// weight slab sits in LDS as [k/4][column][k%4], one 16-byte read feeds four matrix instructions.  MASK: the
// row operand is a[r][k] where mask[r][k] > 0, else 0 (the ReLU backward).
constexpr int kStageStride = 68;                       // floats per staged row: 16-byte reads of 32 rows hit all banks
constexpr int kStageWave = 32 * kStageStride;          // per wavefront

// MASK: 0 = rows as they are, 1 = a float array of the rows' shape decides (entries > 0 pass),
// 2 = one bit per entry decides (32-bit words, W per row, bit c % 32 of word c / 32),
// 3 = the rows are vertex2facet rows formed while they are loaded (the convolution in front of the tail never
//     leaves its result in memory unless asked to): row f, column c = sum_j vfilt[j][c] * a[face[f][j]][c].
template <bool VEC, int MASK> struct RowBlock {
    float v[32];
    float m[MASK == 1 ? 32 : 1];
    unsigned w[MASK == 2 ? (VEC ? 8 : 32) : 1];
    float g[MASK == 3 ? 64 : 1];              // the rows of the second and third corner
};

// What mode 3 reads besides the vertex rows `a` (Nv x K): facets (N x 3), the per-corner channel weights (3 x K),
// and where the formed rows go as well when the caller keeps them for the backward pass (N x K, or null).
struct RowGather {
    const int *face;
    const float *vfilt;
    float *keep;
};

// The 96 corner indices of a 32-facet tile, spread over the wavefront: lane l holds entries l and 64 + l.
struct TileCorners {
    int lo, hi;
};
__device__ __forceinline__ TileCorners corners_issue(const int *__restrict__ face, int64_t tile, int64_t N, int lane)
{
    TileCorners c;
    const int64_t base = tile * 96, end = 3 * N;
    c.lo = base + lane < end ? face[base + lane] : 0;
    c.hi = (lane < 32 && base + 64 + lane < end) ? face[base + 64 + lane] : 0;
    return c;
}
// corner j of row r of the tile, read from the lane that holds it
__device__ __forceinline__ int corner_of(const TileCorners &c, int r, int j)
{
    const int e = 3 * r + j;
    const int a = __builtin_amdgcn_ds_bpermute((e & 63) * 4, c.lo), b = __builtin_amdgcn_ds_bpermute((e & 63) * 4, c.hi);
    return e < 64 ? a : b;
}

// Mode 3, the fetches of a 32 x 64 block: three gathered 16-byte pieces per row and 16-lane group.
__device__ __forceinline__ void rows_issue_gather(RowBlock<true, 3> &b, const float *__restrict__ a, const TileCorners &tc,
                                                  int64_t tile, int q, int64_t N, int K, int lane)
{
    const int col = q + 4 * (lane & 15), sub = lane >> 4;
    const int64_t left = N - tile * 32;
    // 32-bit byte offsets from the scalar base (the launcher checks that the vertex array stays below 4 GiB)
    const unsigned row_bytes = (unsigned)K * 4u, col_bytes = (unsigned)col * 4u;
    const char *base = reinterpret_cast<const char *>(a);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 4 * i + sub;
        const int v0 = corner_of(tc, r, 0), v1 = corner_of(tc, r, 1), v2 = corner_of(tc, r, 2);
        float4 t0 = make_float4(0.f, 0.f, 0.f, 0.f), t1 = t0, t2 = t0;
        if (r < left && col < K) {
            t0 = *reinterpret_cast<const float4 *>(base + ((unsigned)v0 * row_bytes + col_bytes));
            t1 = *reinterpret_cast<const float4 *>(base + ((unsigned)v1 * row_bytes + col_bytes));
            t2 = *reinterpret_cast<const float4 *>(base + ((unsigned)v2 * row_bytes + col_bytes));
        }
        b.v[4 * i] = t0.x; b.v[4 * i + 1] = t0.y; b.v[4 * i + 2] = t0.z; b.v[4 * i + 3] = t0.w;
        b.g[4 * i] = t1.x; b.g[4 * i + 1] = t1.y; b.g[4 * i + 2] = t1.z; b.g[4 * i + 3] = t1.w;
        b.g[32 + 4 * i] = t2.x; b.g[32 + 4 * i + 1] = t2.y; b.g[32 + 4 * i + 2] = t2.z; b.g[32 + 4 * i + 3] = t2.w;
    }
}

// Mode 3, the block into the stage: the three corners' pieces weighted per channel (corner 0 first, as the
// reference sums them, mesh_conv3d_gpu.cu:176-195), and into `keep` for the first column block's workgroups.
__device__ __forceinline__ void rows_commit_gather(const RowBlock<true, 3> &b, float *stage, const float *__restrict__ vfilt,
                                                   float *__restrict__ keep, int64_t tile, int q, int64_t N, int K, int lane)
{
    const int col = q + 4 * (lane & 15), sub = lane >> 4;
    float4 f0 = make_float4(0.f, 0.f, 0.f, 0.f), f1 = f0, f2 = f0;
    if (col < K) {
        f0 = *reinterpret_cast<const float4 *>(vfilt + col);
        f1 = *reinterpret_cast<const float4 *>(vfilt + K + col);
        f2 = *reinterpret_cast<const float4 *>(vfilt + 2 * K + col);
    }
    const int64_t left = N - tile * 32;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float4 t;
        t.x = fmaf(f2.x, b.g[32 + 4 * i], fmaf(f1.x, b.g[4 * i], f0.x * b.v[4 * i]));
        t.y = fmaf(f2.y, b.g[32 + 4 * i + 1], fmaf(f1.y, b.g[4 * i + 1], f0.y * b.v[4 * i + 1]));
        t.z = fmaf(f2.z, b.g[32 + 4 * i + 2], fmaf(f1.z, b.g[4 * i + 2], f0.z * b.v[4 * i + 2]));
        t.w = fmaf(f2.w, b.g[32 + 4 * i + 3], fmaf(f1.w, b.g[4 * i + 3], f0.w * b.v[4 * i + 3]));
        *reinterpret_cast<float4 *>(stage + (4 * i + sub) * kStageStride + 4 * (lane & 15)) = t;
        if (keep && 4 * i + sub < left && col < K)
            *reinterpret_cast<float4 *>(keep + (tile * 32 + 4 * i + sub) * K + col) = t;
    }
}

template <bool VEC, int MASK>
__device__ __forceinline__ void rows_issue(RowBlock<VEC, MASK> &b, const float *__restrict__ a,
                                           const float *__restrict__ mask, const unsigned *__restrict__ bits, int W,
                                           int64_t tile, int q, int64_t N, int K, int lane)
{
    if constexpr (VEC) {
        // tile and q are uniform: a scalar base per group of four rows plus one lane offset
        const int col = q + 4 * (lane & 15), sub = lane >> 4;
        const int lane_off = sub * K + col, lane_word = sub * W + (col >> 5);
        const int64_t left = N - tile * 32;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int64_t row0 = tile * 32 + 4 * i;
            float4 t = make_float4(0.f, 0.f, 0.f, 0.f), mm = make_float4(1.f, 1.f, 1.f, 1.f);
            if constexpr (MASK == 2) b.w[i] = 0u;
            if (4 * i + sub < left && col < K) {
                t = *reinterpret_cast<const float4 *>(a + row0 * K + lane_off);
                if constexpr (MASK == 1) mm = *reinterpret_cast<const float4 *>(mask + row0 * K + lane_off);
                if constexpr (MASK == 2) b.w[i] = bits[row0 * W + lane_word];
            }
            b.v[4 * i] = t.x; b.v[4 * i + 1] = t.y; b.v[4 * i + 2] = t.z; b.v[4 * i + 3] = t.w;
            if constexpr (MASK == 1) { b.m[4 * i] = mm.x; b.m[4 * i + 1] = mm.y; b.m[4 * i + 2] = mm.z; b.m[4 * i + 3] = mm.w; }
        }
    } else {
        const int col = q + lane;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int64_t row = tile * 32 + i;
            const bool ok = row < N && col < K;
            b.v[i] = ok ? a[row * K + col] : 0.f;
            if constexpr (MASK == 1) b.m[i] = ok ? mask[row * K + col] : 1.f;
            if constexpr (MASK == 2) b.w[i] = ok ? bits[row * W + (col >> 5)] : 0u;
        }
    }
}

template <bool VEC, int MASK>
__device__ __forceinline__ void rows_commit(const RowBlock<VEC, MASK> &b, float *stage, int lane)
{
    if constexpr (VEC) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float4 t = make_float4(b.v[4 * i], b.v[4 * i + 1], b.v[4 * i + 2], b.v[4 * i + 3]);
            if constexpr (MASK == 1) {
                t.x = b.m[4 * i] > 0.f ? t.x : 0.f; t.y = b.m[4 * i + 1] > 0.f ? t.y : 0.f;
                t.z = b.m[4 * i + 2] > 0.f ? t.z : 0.f; t.w = b.m[4 * i + 3] > 0.f ? t.w : 0.f;
            }
            if constexpr (MASK == 2) {
                const unsigned nib = b.w[i] >> ((4 * (lane & 15)) & 31);      // chunks start at multiples of 64 columns
                t.x = (nib & 1u) ? t.x : 0.f; t.y = (nib & 2u) ? t.y : 0.f;
                t.z = (nib & 4u) ? t.z : 0.f; t.w = (nib & 8u) ? t.w : 0.f;
            }
            *reinterpret_cast<float4 *>(stage + (4 * i + (lane >> 4)) * kStageStride + 4 * (lane & 15)) = t;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            float t = b.v[i];
            if constexpr (MASK == 1) t = b.m[i] > 0.f ? t : 0.f;
            if constexpr (MASK == 2) t = ((b.w[i] >> (lane & 31)) & 1u) ? t : 0.f;
            stage[i * kStageStride + lane] = t;
        }
    }
}

// Epilogue of one 32-row tile: out = max(acc + bias, floor) * scale + shift, lane (n, h) holds column n of every
// 32-column block and rows 8(i/4) + 4h + i%4.  BITS: one ballot per register gives the 32 mask bits of a row of
// either lane half; lane i keeps the word of its row and the sixteen rows of a half leave in one store.
// FULL: the tile lies inside the matrix, no bounds.  Clears the accumulators.
template <int NT, bool BITS, bool FULL>
__device__ __forceinline__ void rows_store(f32x16 (&acc)[NT], const float (&bia)[NT], const float (&scl)[NT],
                                           const float (&shf)[NT], float floor_v, float *__restrict__ tile_out,
                                           unsigned *__restrict__ tile_bits, int C, int Wout, int col0, int n, int h,
                                           int64_t left)
{
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int c = col0 + j * 32 + n;
        const bool col_ok = FULL || c < C;
        float *lane_out = tile_out + 4 * h * C + c;
        unsigned word = 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int ri = 8 * (i / 4) + (i % 4);                      // row of lane half 0; half 1 is four rows on
            const float v = fmaxf(acc[j][i] + bia[j], floor_v);
            if (FULL || (col_ok && ri + 4 * h < left)) lane_out[(int64_t)ri * C] = v * scl[j] + shf[j];
            if constexpr (BITS) {
                const unsigned long long pos = __builtin_amdgcn_ballot_w64(col_ok && v > 0.f);
                const unsigned mine = h ? (unsigned)(pos >> 32) : (unsigned)pos;
                word = (n == i) ? mine : word;
            }
            acc[j][i] = 0.f;
        }
        if constexpr (BITS) {
            const int rn = 8 * (n / 4) + 4 * h + (n % 4);
            if (n < 16 && (FULL || (rn < left && (col0 >> 5) + j < Wout))) tile_bits[(int64_t)rn * Wout + j] = word;
        }
    }
}

// X3: the product runs on the bf16 matrix instruction with both operands split in three (the slab then holds
// [k/8][column][piece] blocks of eight bf16, 6 bytes per weight); otherwise on the fp32 matrix instruction.
template <int NT, int NW, bool VEC, int MASK, bool X3>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void dense_rows_k(const float *__restrict__ a, const float *__restrict__ mask,
                                                       const unsigned *__restrict__ bits_in,
                                                       unsigned *__restrict__ bits_out,
                                                       const float *__restrict__ w, int64_t wk, int64_t wc,
                                                       const float *__restrict__ bias,
                                                       const float *__restrict__ scale,
                                                       const float *__restrict__ shift, int relu,
                                                       float *__restrict__ out, int64_t N, int K, int Kpad, int C,
                                                       RowGather gat)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int NC = NT * 32;
    // the wavefront index as a scalar: tile numbers and with them every row base stay in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int n = lane & 31, h = lane >> 5;
    // the column blocks of the same rows are neighbouring workgroups: they run together and share the rows' HBM reads
    const int ncb = (C + NC - 1) / NC;
    const int col0 = (int)(blockIdx.x % ncb) * NC;
    const int64_t row_block = blockIdx.x / ncb, row_blocks = gridDim.x / ncb;
    float *slab = lds + NW * kStageWave;
    float *stage = lds + wave * kStageWave;
    if constexpr (X3) {
        u32x4 *slab3 = reinterpret_cast<u32x4 *>(slab);
        for (int idx = threadIdx.x; idx < (Kpad >> 3) * NC; idx += NW * 64) {
            const int kb = idx / NC, c = idx - kb * NC;
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int k = 8 * kb + e;
                v[e] = (k < K && col0 + c < C) ? w[(int64_t)k * wk + (int64_t)(col0 + c) * wc] : 0.f;
            }
            u32x4 p1, p2, p3;
            dense_split8(v, p1, p2, p3);
            slab3[(size_t)idx * 3] = p1; slab3[(size_t)idx * 3 + 1] = p2; slab3[(size_t)idx * 3 + 2] = p3;
        }
    } else {
        for (int idx = threadIdx.x; idx < Kpad * NC; idx += NW * 64) {
            const int k = idx / NC, c = idx - k * NC;
            const float v = (k < K && col0 + c < C) ? w[(int64_t)k * wk + (int64_t)(col0 + c) * wc] : 0.f;
            slab[((k >> 2) * NC + c) * 4 + (k & 3)] = v;
        }
    }
    __syncthreads();
    float bia[NT], scl[NT], shf[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int c = col0 + j * 32 + n;
        bia[j] = (bias && c < C) ? bias[c] : 0.f;
        scl[j] = (scale && c < C) ? scale[c] : 1.f;
        shf[j] = (shift && c < C) ? shift[c] : 0.f;
    }
    const float floor_v = relu ? 0.f : -__builtin_inff();      // max(v, floor_v) is the ReLU or the identity
    const int64_t ntiles = (N + 31) / 32, stride = row_blocks * NW;
    int64_t tile = row_block * NW + wave;
    int q = 0;
    bool have = tile < ntiles;
    RowBlock<VEC, MASK> blk;
    const int Win = (K + 31) >> 5, Wout = (C + 31) >> 5;
    // mode 3: the corner indices of a tile are fetched one tile ahead of its rows
    TileCorners tc = {0, 0}, tc_next = {0, 0};
    float *keep = nullptr;
    if constexpr (MASK == 3) {
        static_assert(MASK != 3 || VEC, "rows formed on load come in 16-byte pieces");
        keep = col0 == 0 ? gat.keep : nullptr;
        // The gathered rows of a block are fetched when the block is due, not a block ahead: three corners are 96
        // registers in flight, which do not fit beside the product's; the other wavefronts of the CU cover the wait.
        if (have) {
            tc = corners_issue(gat.face, tile, N, lane);
            tc_next = corners_issue(gat.face, tile + stride, N, lane);
        }
    } else {
        if (have) rows_issue<VEC, MASK>(blk, a, mask, bits_in, Win, tile, 0, N, K, lane);
    }
    f32x16 acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    while (have) {
        if constexpr (MASK == 3) {
            rows_issue_gather(blk, a, tc, tile, q, N, K, lane);
            rows_commit_gather(blk, stage, gat.vfilt, keep, tile, q, N, K, lane);
        } else {
            rows_commit<VEC, MASK>(blk, stage, lane);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int64_t ntile = tile;
        int nq = q + kDenseChunk;
        if (nq >= Kpad) { nq = 0; ntile += stride; }
        const bool nhave = ntile < ntiles;
        if constexpr (MASK == 3) {
            if (nhave && nq == 0) {
                tc = tc_next;
                tc_next = corners_issue(gat.face, ntile + stride, N, lane);
            }
        } else {
            if (nhave) rows_issue<VEC, MASK>(blk, a, mask, bits_in, Win, ntile, nq, N, K, lane);
        }
        const float *xs = stage + n * kStageStride + h * 32;
        if constexpr (X3) {
            // lane (r, h) owns reduction entries q + 32h + 8t + e of row r in step t, the slab block (q + 32h)/8 + t
            u32x4 pa[4][3];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float4 lo = *reinterpret_cast<const float4 *>(xs + 8 * t);
                const float4 hi = *reinterpret_cast<const float4 *>(xs + 8 * t + 4);
                const float xv[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                dense_split8(xv, pa[t][0], pa[t][1], pa[t][2]);
            }
            const u32x4 *sl = reinterpret_cast<const u32x4 *>(slab) + ((size_t)((q + h * 32) >> 3) * NC + n) * 3;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const u32x4 *bp = sl + ((size_t)t * NC + j * 32) * 3;
                    const u32x4 b1 = bp[0], b2 = bp[1], b3 = bp[2];
                    acc[j] = dense_mfma_bf16(pa[t][2], b1, acc[j]);
                    acc[j] = dense_mfma_bf16(pa[t][1], b2, acc[j]);
                    acc[j] = dense_mfma_bf16(pa[t][0], b3, acc[j]);
                    acc[j] = dense_mfma_bf16(pa[t][1], b1, acc[j]);
                    acc[j] = dense_mfma_bf16(pa[t][0], b2, acc[j]);
                    acc[j] = dense_mfma_bf16(pa[t][0], b1, acc[j]);
                }
            }
        } else {
            const float *sl = slab + ((size_t)((q + h * 32) >> 2) * NC + n) * 4;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                const float4 x4 = *reinterpret_cast<const float4 *>(xs + 4 * g);
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const float4 b = *reinterpret_cast<const float4 *>(sl + ((size_t)g * NC + j * 32) * 4);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(x4.x, b.x, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(x4.y, b.y, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(x4.z, b.z, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(x4.w, b.w, acc[j], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (q + kDenseChunk >= Kpad) {
            const int64_t left = N - tile * 32;
            const bool full = left >= 32 && col0 + NC <= C;            // uniform: no bounds inside the tile
            float *tile_out = out + tile * 32 * C;
            unsigned *tile_bits = bits_out ? bits_out + tile * 32 * Wout + (col0 >> 5) : nullptr;
            if (tile_bits) {
                if (full) rows_store<NT, true, true>(acc, bia, scl, shf, floor_v, tile_out, tile_bits, C, Wout, col0, n, h, left);
                else rows_store<NT, true, false>(acc, bia, scl, shf, floor_v, tile_out, tile_bits, C, Wout, col0, n, h, left);
            } else {
                if (full) rows_store<NT, false, true>(acc, bia, scl, shf, floor_v, tile_out, tile_bits, C, Wout, col0, n, h, left);
                else rows_store<NT, false, false>(acc, bia, scl, shf, floor_v, tile_out, tile_bits, C, Wout, col0, n, h, left);
            }
        }
        tile = ntile; q = nq; have = nhave;
    }
}

// U row pairs of the weight-gradient kernel in registers: lane half h holds row base + 2u + h.
template <int TA, int TB, int U, int MASK> struct PairBlock {
    Pack<TA> xa[U];
    Pack<TB> gz[U];
    Pack<MASK == 1 ? TB : 1> yy[U];
    unsigned yw[MASK == 2 ? U : 1];
};

// `base` is uniform over the wavefront, so every row pair costs one scalar base per array and the lanes share
// one 32-bit offset; FULL skips the row bound.
template <int TA, int TB, int U, bool VEC, int MASK, bool FULL>
__device__ __forceinline__ void pairs_issue(PairBlock<TA, TB, U, MASK> &blk, const float *__restrict__ x,
                                            const float *__restrict__ g, const float *__restrict__ y,
                                            const unsigned *__restrict__ bits, int64_t base, int64_t r1, int h, int Ci,
                                            int Co, int ci0, int co0)
{
    const int xo = h * Ci + ci0, go = h * Co + co0, W = (Co + 31) >> 5, wo = h * W + (co0 >> 5);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const float *xu = x + (base + 2 * u) * Ci;
        const float *gu = g + (base + 2 * u) * Co;
        const float *yu = MASK == 1 ? y + (base + 2 * u) * Co : nullptr;
        const bool live = FULL || base + 2 * u + h < r1;
        blk.xa[u] = zero_pack<TA>();
        blk.gz[u] = zero_pack<TB>();
        blk.yy[u] = zero_pack<MASK == 1 ? TB : 1>();
        if constexpr (MASK == 2) blk.yw[u] = (live && co0 < Co) ? bits[(base + 2 * u) * W + wo] : 0u;
        if constexpr (VEC) {
            if (live && ci0 < Ci) blk.xa[u] = ldp<TA>(xu + xo);
            if (live && co0 < Co) {
                blk.gz[u] = ldp<TB>(gu + go);
                if constexpr (MASK == 1) blk.yy[u] = ldp<TB>(yu + go);
            }
        } else {
#pragma unroll
            for (int ja = 0; ja < TA; ++ja)
                if (live && ci0 + ja < Ci) blk.xa[u].v[ja] = xu[xo + ja];
#pragma unroll
            for (int jb = 0; jb < TB; ++jb)
                if (live && co0 + jb < Co) {
                    blk.gz[u].v[jb] = gu[go + jb];
                    if constexpr (MASK == 1) blk.yy[u].v[jb] = yu[go + jb];
                }
        }
    }
}

// Weight and bias gradient: gW[ci][co] = sum_rows x[row][ci] * gz[row][co], gb[co] = sum_rows gz[row][co] with
// gz = g where y > 0 (MASK) or g.  The rows are the reduction index: one matrix instruction consumes two rows
// (lane half h takes row 2t + h), lane (m, h) supplies TA input channels and TB output channels that lie
// contiguously in its rows, and a wavefront keeps TA x TB tiles of 32 x 32 sums.  Every workgroup leaves one
// partial of (Ci + 1) * Co floats (row Ci = bias gradient).  The channel chunks of one row range are neighbouring
// workgroups (chunk = blockIdx.x % chunks), so they run at the same time and the rows they share come from HBM once.
// X3: the sixteen rows of a block are one reduction step of the bf16 matrix instruction (lane half h holds the
// eight rows base + 2u + h), both operands split in three pieces, six piece products per tile.
template <int TA, int TB, bool VEC, int MASK, bool X3>
__global__ __launch_bounds__(256, 2) void dense_wgrad_k(const float *__restrict__ x, const float *__restrict__ g,
                                                        const float *__restrict__ y,
                                                        const unsigned *__restrict__ bits, float *__restrict__ partial,
                                                        int64_t N, int Ci, int Co, int nA, int64_t rows_per_wave)
{
    __shared__ float red[TA * TB * 16 * 64];
    __shared__ float bred[4][2][32 * TB];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 31, h = lane >> 5;
    const int nchunks = nA * ((Co + TB * 32 - 1) / (TB * 32));
    const int chunk = (int)(blockIdx.x % nchunks), range = (int)(blockIdx.x / nchunks);
    const int chunkA = chunk % nA, chunkB = chunk / nA;
    const int ci0 = chunkA * TA * 32 + m * TA, co0 = chunkB * TB * 32 + m * TB;
    f32x16 acc[TA][TB];
#pragma unroll
    for (int ja = 0; ja < TA; ++ja)
#pragma unroll
        for (int jb = 0; jb < TB; ++jb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[ja][jb][i] = 0.f;
    float gb[TB];
#pragma unroll
    for (int jb = 0; jb < TB; ++jb) gb[jb] = 0.f;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int64_t r0 = ((int64_t)range * 4 + wave_u) * rows_per_wave;
    int64_t r1 = r0 + rows_per_wave;
    if (r1 > N) r1 = N;
    constexpr int U = 8;
    PairBlock<TA, TB, U, MASK> blk;
    for (int64_t base = r0; base < r1; base += 2 * U) {
        if (base + 2 * U <= r1) pairs_issue<TA, TB, U, VEC, MASK, true>(blk, x, g, y, bits, base, r1, h, Ci, Co, ci0, co0);
        else pairs_issue<TA, TB, U, VEC, MASK, false>(blk, x, g, y, bits, base, r1, h, Ci, Co, ci0, co0);
        if constexpr (X3) {
            u32x4 pb[TB][3];
#pragma unroll
            for (int jb = 0; jb < TB; ++jb) {
                float gzv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    gzv[u] = blk.gz[u].v[jb];
                    if constexpr (MASK == 1) gzv[u] = blk.yy[u].v[jb] > 0.f ? gzv[u] : 0.f;
                    if constexpr (MASK == 2) gzv[u] = ((blk.yw[u] >> ((co0 & 31) + jb)) & 1u) ? gzv[u] : 0.f;
                    gb[jb] += gzv[u];
                }
                dense_split8(gzv, pb[jb][0], pb[jb][1], pb[jb][2]);
            }
#pragma unroll
            for (int ja = 0; ja < TA; ++ja) {
                float xv[U];
#pragma unroll
                for (int u = 0; u < U; ++u) xv[u] = blk.xa[u].v[ja];
                u32x4 pa[3];
                dense_split8(xv, pa[0], pa[1], pa[2]);
#pragma unroll
                for (int jb = 0; jb < TB; ++jb) {
                    acc[ja][jb] = dense_mfma_bf16(pa[2], pb[jb][0], acc[ja][jb]);
                    acc[ja][jb] = dense_mfma_bf16(pa[1], pb[jb][1], acc[ja][jb]);
                    acc[ja][jb] = dense_mfma_bf16(pa[0], pb[jb][2], acc[ja][jb]);
                    acc[ja][jb] = dense_mfma_bf16(pa[1], pb[jb][0], acc[ja][jb]);
                    acc[ja][jb] = dense_mfma_bf16(pa[0], pb[jb][1], acc[ja][jb]);
                    acc[ja][jb] = dense_mfma_bf16(pa[0], pb[jb][0], acc[ja][jb]);
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float gzv[TB];
#pragma unroll
                for (int jb = 0; jb < TB; ++jb) {
                    gzv[jb] = blk.gz[u].v[jb];
                    if constexpr (MASK == 1) gzv[jb] = blk.yy[u].v[jb] > 0.f ? gzv[jb] : 0.f;
                    if constexpr (MASK == 2) gzv[jb] = ((blk.yw[u] >> ((co0 & 31) + jb)) & 1u) ? gzv[jb] : 0.f;
                    gb[jb] += gzv[jb];
                }
#pragma unroll
                for (int ja = 0; ja < TA; ++ja)
#pragma unroll
                    for (int jb = 0; jb < TB; ++jb)
                        acc[ja][jb] = __builtin_amdgcn_mfma_f32_32x32x2f32(blk.xa[u].v[ja], gzv[jb], acc[ja][jb], 0, 0, 0);
            }
        }
    }
    // the four wavefronts add up in wavefront order
    for (int wv = 0; wv < 4; ++wv) {
        if (wave == wv) {
#pragma unroll
            for (int ja = 0; ja < TA; ++ja)
#pragma unroll
                for (int jb = 0; jb < TB; ++jb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        float *p = red + ((ja * TB + jb) * 16 + i) * 64 + lane;
                        *p = wv == 0 ? acc[ja][jb][i] : *p + acc[ja][jb][i];
                    }
        }
        __syncthreads();
    }
#pragma unroll
    for (int jb = 0; jb < TB; ++jb) bred[wave][h][m * TB + jb] = gb[jb];
    __syncthreads();
    float *dst = partial + (size_t)range * (size_t)(Ci + 1) * Co;
    for (int idx = threadIdx.x; idx < TA * TB * 16 * 64; idx += 256) {
        const int ln = idx & 63, i = (idx >> 6) & 15, t = idx >> 10;
        const int ja = t / TB, jb = t - ja * TB;
        const int mm = 8 * (i / 4) + 4 * (ln >> 5) + (i % 4), nn = ln & 31;
        const int ci = chunkA * TA * 32 + mm * TA + ja, co = chunkB * TB * 32 + nn * TB + jb;
        if (ci < Ci && co < Co) dst[(size_t)ci * Co + co] = red[idx];
    }
    if (chunkA == 0 && threadIdx.x < 32 * TB) {
        const int co = chunkB * TB * 32 + threadIdx.x;
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < 4; ++wv) s += bred[wv][0][threadIdx.x] + bred[wv][1][threadIdx.x];
        if (co < Co) dst[(size_t)Ci * Co + co] = s;
    }
}

// The same tail without a product, for convolutions that mix channels themselves (facet2facet):
// out = act(x + bias) * scale + shift, V floats per thread.
template <int V>
__global__ __launch_bounds__(256) void bias_act_fwd_k(const float *__restrict__ x, const float *__restrict__ bias,
                                                      const float *__restrict__ scale,
                                                      const float *__restrict__ shift, int relu,
                                                      float *__restrict__ out, unsigned *__restrict__ bits_out,
                                                      int64_t n_items, int items)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = i < n_items;
    unsigned nib = 0u;
    if (live) {
        const int c = (int)(i % items) * V;
        Pack<V> v = ldp<V>(x + i * V);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float t = v.v[j] + (bias ? bias[c + j] : 0.f);
            if (relu) t = fmaxf(t, 0.f);
            nib |= (t > 0.f ? 1u : 0u) << j;
            v.v[j] = t * (scale ? scale[c + j] : 1.f) + (shift ? shift[c + j] : 0.f);
        }
        stp<V>(out + i * V, v);
    }
    if constexpr (V == 4) {
        // eight neighbouring lanes hold the 32 columns of one mask word (rows are multiples of 32 columns here)
        if (bits_out) {
            unsigned word = nib << (4 * (threadIdx.x & 7));
            word |= __shfl_xor(word, 1);
            word |= __shfl_xor(word, 2);
            word |= __shfl_xor(word, 4);
            if (live && (threadIdx.x & 7) == 0) bits_out[i >> 3] = word;
        }
    }
}

// Its gradient: gin = g where y > 0 (MASK; skipped when gin is null), partial[block][c] = the block's column sums
// of the masked g.  A group of `lpr` lanes walks a row (looping when the row has more than lpr items, at most
// kBiasLoops times), 256 / lpr rows in flight; the row slots add up in slot order.
constexpr int kBiasLoops = 4;

template <int V, int MASK>
__global__ __launch_bounds__(256) void bias_act_bwd_k(const float *__restrict__ g, const float *__restrict__ y,
                                                      const unsigned *__restrict__ bits, float *__restrict__ gin,
                                                      float *__restrict__ partial,
                                                      int64_t N, int C, int lpr, int64_t rows_per_block)
{
    __shared__ float red[256 * kBiasLoops * V];
    const int lane = threadIdx.x % lpr, slot = threadIdx.x / lpr, rpb = 256 / lpr, items = C / V;
    Pack<V> acc[kBiasLoops];
#pragma unroll
    for (int k = 0; k < kBiasLoops; ++k) acc[k] = zero_pack<V>();
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
    int64_t r1 = r0 + rows_per_block;
    if (r1 > N) r1 = N;
    for (int64_t row = r0 + slot; row < r1; row += rpb) {
#pragma unroll
        for (int k = 0; k < kBiasLoops; ++k) {
            const int cv = lane + k * lpr;
            if (cv < items) {
                const int64_t o = row * C + (int64_t)cv * V;
                Pack<V> gz = ldp<V>(g + o);
                if constexpr (MASK == 1) {
                    const Pack<V> yy = ldp<V>(y + o);
#pragma unroll
                    for (int j = 0; j < V; ++j) gz.v[j] = yy.v[j] > 0.f ? gz.v[j] : 0.f;
                    if (gin) stp<V>(gin + o, gz);
                }
                if constexpr (MASK == 2) {
                    // V == 4 and C % 32 == 0: word cv / 8 of the row, nibble cv % 8
                    const unsigned nib = bits[row * (C >> 5) + (cv >> 3)] >> (4 * (cv & 7));
#pragma unroll
                    for (int j = 0; j < V; ++j) gz.v[j] = ((nib >> j) & 1u) ? gz.v[j] : 0.f;
                    if (gin) stp<V>(gin + o, gz);
                }
#pragma unroll
                for (int j = 0; j < V; ++j) acc[k].v[j] += gz.v[j];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < kBiasLoops; ++k)
#pragma unroll
        for (int j = 0; j < V; ++j) red[(threadIdx.x * kBiasLoops + k) * V + j] = acc[k].v[j];
    __syncthreads();
    if (slot == 0) {
#pragma unroll
        for (int k = 0; k < kBiasLoops; ++k) {
            const int cv = lane + k * lpr;
            if (cv >= items) continue;
            Pack<V> sum = zero_pack<V>();
            for (int t = 0; t < rpb; ++t)
#pragma unroll
                for (int j = 0; j < V; ++j) sum.v[j] += red[((t * lpr + lane) * kBiasLoops + k) * V + j];
#pragma unroll
            for (int j = 0; j < V; ++j) partial[(size_t)blockIdx.x * C + cv * V + j] = sum.v[j];
        }
    }
}

struct BiasPlan {
    int V, lpr, G;
    int64_t rows_per_block;
};

static BiasPlan bias_plan(int64_t N, int C, bool aligned)
{
    BiasPlan p;
    p.V = (aligned && C % 4 == 0) ? 4 : 1;
    const RowShape rs = row_shape(C / p.V);
    p.lpr = rs.lpr;
    p.G = persistent_blocks(N, rs.rpb);
    p.rows_per_block = ceil_div(ceil_div(N, p.G), rs.rpb) * rs.rpb;
    return p;
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Column tiles per workgroup of dense_rows_k: as many as the preferred slab size and 4 accumulator tiles allow.
static int rows_tiles(int Kpad, int C, int slab_weights)
{
    int nt = 4;
    while (nt > 1 && (Kpad * nt * 32 > slab_weights || (nt / 2) * 32 >= C)) nt >>= 1;
    return nt;
}

// the fp32 matrix instruction on request (tests compare the two paths)
static bool force_fp32_mfma() { return options().dense_fp32mfma; }

// Launch with as many workgroups as are resident at once (every tile is independent, so the count only
// balances the load): a grid that needs a second round of workgroups would run that round at low occupancy.
struct RowsArgs {
    const float *a, *mask;
    const unsigned *bits_in;
    unsigned *bits_out;
    const float *w;
    int64_t wk, wc;
    const float *bias, *scale, *shift;
    int relu;
    float *out;
    int64_t N;
    int K, Kpad, C;
    RowGather gat;
};

template <int NT, int NW, bool VEC, int MASK, bool X3>
static void launch_rows_nt(int64_t ntiles, unsigned gy, size_t lds, hipStream_t st, const RowsArgs &p)
{
    const void *fn = reinterpret_cast<const void *>(dense_rows_k<NT, NW, VEC, MASK, X3>);
    if (lds > 65536) (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    int per_cu = 0, dev = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, NW * 64, lds) != hipSuccess || per_cu < 1) per_cu = 1;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
        cus = 256;
    int64_t gx = (int64_t)per_cu * cus / gy;
    const int64_t wanted = ceil_div(ntiles, NW);
    if (gx < 1) gx = 1;
    if (gx > wanted) gx = wanted;
    dense_rows_k<NT, NW, VEC, MASK, X3><<<dim3((unsigned)(gx * gy)), dim3(NW * 64), lds, st>>>(
        p.a, p.mask, p.bits_in, p.bits_out, p.w, p.wk, p.wc, p.bias, p.scale, p.shift, p.relu, p.out, p.N, p.K, p.Kpad, p.C, p.gat);
}

template <bool VEC, int MASK, bool X3>
static void launch_rows(int NT, int NW, int64_t ntiles, unsigned gy, size_t lds, hipStream_t st, const RowsArgs &p)
{
#define PM_ROWS(T, W) launch_rows_nt<T, W, VEC, MASK, X3>(ntiles, gy, lds, st, p)
    if constexpr (X3) {
        if (NW == 6) {
            if (NT == 4) PM_ROWS(4, 6);
            else PM_ROWS(2, 6);
            return;
        }
    }
    if (NW == 8) {
        switch (NT) {
        case 4: PM_ROWS(4, 8); break;
        case 2: PM_ROWS(2, 8); break;
        default: PM_ROWS(1, 8); break;
        }
    } else {
        switch (NT) {
        case 4: PM_ROWS(4, 4); break;
        case 2: PM_ROWS(2, 4); break;
        default: PM_ROWS(1, 4); break;
        }
    }
#undef PM_ROWS
}

// out (N x C) = act(a' (N x K) . Wm + bias) * scale + shift; a' = a masked by mask > 0 (float array) or by
// bits_in (one bit per entry) when given; bits_out receives one bit per output entry, set where act(.) > 0.
static int dense_rows(const char *name, const float *a, const float *mask, const unsigned *bits_in, unsigned *bits_out,
                      const float *w, int64_t wk, int64_t wc, const float *bias, const float *scale, const float *shift,
                      int relu, float *out, int64_t N, int K, int C, hipStream_t st, const RowGather *gather = nullptr)
{
    PM_REQUIRE(K > 0 && C > 0 && K <= kDenseMaxK && C <= (1 << 20), "%s: channel counts out of range (%d, %d)", name, K, C);
    PM_REQUIRE(N * (int64_t)(K > C ? K : C) < (int64_t(1) << 40), "%s: sizes too large", name);
    const int Kpad = (int)ceil_div(K, kDenseChunk) * kDenseChunk;
    // Four wavefronts per workgroup and a slab of at most 48 KiB keep two workgroups on a CU.  When that slab
    // cannot hold all the columns (the rows would be fetched once per column block), or leaves room for one
    // workgroup only, eight wavefronts share a slab of up to 88 KiB instead.  The split-bf16 product needs
    // 6 bytes per weight; reductions too long for that slab stay on the fp32 matrix instruction.
    bool x3 = !force_fp32_mfma();
    int NT = 1, NW = 4;
    size_t lds = 0;
    for (;;) {
        const int wbytes = x3 ? 6 : 4;
        NT = rows_tiles(Kpad, C, kDenseSlabBytes / wbytes);
        NW = 4;
        lds = (size_t)Kpad * NT * 32 * wbytes + 4 * kStageWave * sizeof(float);
        const int nt8 = rows_tiles(Kpad, C, kDenseSlabWideBytes / wbytes);
        const size_t lds8 = (size_t)Kpad * nt8 * 32 * wbytes + 8 * kStageWave * sizeof(float);
        if (lds8 <= kDenseLdsMax && (nt8 > NT || lds > kDenseLdsMax / 2)) {
            NT = nt8; NW = 8; lds = lds8;
        }
        if (x3) {
            // six wavefronts leave 108 KiB for the slab: 128 columns of a 128-long reduction in split bf16
            const int nt6 = rows_tiles(Kpad, C, kDenseSlabSixBytes / wbytes);
            const size_t lds6 = (size_t)Kpad * nt6 * 32 * wbytes + 6 * kStageWave * sizeof(float);
            if (lds6 <= kDenseLdsMax && nt6 > NT) {
                NT = nt6; NW = 6; lds = lds6;
            }
        }
        if (lds <= kDenseLdsMax || !x3) break;
        x3 = false;
    }
    PM_REQUIRE(lds <= kDenseLdsMax, "%s: reduction length %d too large", name, K);
    if (gather && NT > 2) {
        // rows formed on load: 96 registers of gathered pieces beside at most two accumulator tiles
        NT = 2;
        lds = (size_t)Kpad * NT * 32 * (x3 ? 6 : 4) + (size_t)NW * kStageWave * sizeof(float);
    }
    const int64_t ntiles = ceil_div(N, 32);
    const unsigned gy = (unsigned)ceil_div(C, NT * 32);
    const bool vec = (K % 4 == 0) && aligned16(a) && (!mask || aligned16(mask));
    const RowsArgs p{a, mask, bits_in, bits_out, w, wk, wc, bias, scale, shift, relu, out, N, K, Kpad, C,
                     gather ? *gather : RowGather{nullptr, nullptr, nullptr}};
    const int mode = gather ? 3 : bits_in ? 2 : mask ? 1 : 0;
    PM_REQUIRE(mode != 3 || (vec && aligned16(gather->vfilt) && (!gather->keep || aligned16(gather->keep))),
               "%s: rows formed on load need a multiple of 4 channels and 16-byte aligned arrays", name);
#define PM_PICK(V, M)                                                          \
    do {                                                                       \
        if (x3) launch_rows<V, M, true>(NT, NW, ntiles, gy, lds, st, p);       \
        else launch_rows<V, M, false>(NT, NW, ntiles, gy, lds, st, p);         \
    } while (0)
    if (vec) {
        if (mode == 3) PM_PICK(true, 3);
        else if (mode == 2) PM_PICK(true, 2);
        else if (mode == 1) PM_PICK(true, 1);
        else PM_PICK(true, 0);
    } else {
        if (mode == 2) PM_PICK(false, 2);
        else if (mode == 1) PM_PICK(false, 1);
        else PM_PICK(false, 0);
    }
#undef PM_PICK
    PM_LAUNCHED(name);
    return 0;
}

struct WgradPlan {
    int ta, tb, nA, nB, G;
    int64_t rows_per_wave;
};

static int pick_tiles(int ch)
{
    return ch > 64 ? 4 : ch > 32 ? 2 : 1;
}

static WgradPlan wgrad_plan(int64_t N, int Ci, int Co)
{
    WgradPlan p;
    p.ta = pick_tiles(Ci);
    p.tb = pick_tiles(Co);
    if (p.ta * p.tb > 8) p.tb = 2;   // at most 8 accumulator tiles per wavefront
    p.nA = (int)ceil_div(Ci, p.ta * 32);
    p.nB = (int)ceil_div(Co, p.tb * 32);
    int64_t G = ceil_div(N, 4 * 256);   // at least 256 rows per wavefront
    if (G < 1) G = 1;
    if (G > 1024) G = 1024;
    // keep the partials of wide layers modest: G * (Ci + 1) * Co floats <= 8 Mi floats
    while (G > 1 && G * (int64_t)(Ci + 1) * Co > (int64_t(1) << 23)) G >>= 1;
    p.G = (int)G;
    p.rows_per_wave = ceil_div(ceil_div(N, G * 4), 2) * 2;
    return p;
}

template <int TA, int TB>
static void launch_wgrad(bool vec, int mode, dim3 grid, hipStream_t st, const float *x, const float *g, const float *y,
                         const unsigned *bits, float *partial, int64_t N, int Ci, int Co, int nA, int64_t rpw)
{
    const bool x3 = !force_fp32_mfma();
#define PM_WGK(V, M)                                                                                                        \
    do {                                                                                                                    \
        if (x3) dense_wgrad_k<TA, TB, V, M, true><<<grid, dim3(256), 0, st>>>(x, g, y, bits, partial, N, Ci, Co, nA, rpw);  \
        else dense_wgrad_k<TA, TB, V, M, false><<<grid, dim3(256), 0, st>>>(x, g, y, bits, partial, N, Ci, Co, nA, rpw);    \
    } while (0)
    if (vec) {
        if (mode == 2) PM_WGK(true, 2);
        else if (mode == 1) PM_WGK(true, 1);
        else PM_WGK(true, 0);
    } else {
        if (mode == 2) PM_WGK(false, 2);
        else if (mode == 1) PM_WGK(false, 1);
        else PM_WGK(false, 0);
    }
#undef PM_WGK
}

}  // namespace pmesh

using namespace pmesh;

extern "C" int pmesh_dense_fwd(const float *input, const float *weight, const float *bias, const float *scale,
                               const float *shift, int relu, float *output, uint32_t *relu_bits, int64_t N, int Ci,
                               int Co, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(N >= 0, "dense_fwd: negative size");
    if (N == 0) return 0;
    PM_REQUIRE(input && weight && output, "dense_fwd: null pointer");
    return dense_rows("dense_fwd", input, nullptr, nullptr, relu_bits, weight, Co, 1, bias, scale, shift, relu, output, N,
                      Ci, Co, (hipStream_t)stream);
}

extern "C" int pmesh_v2f_dense_fwd(const float *input, const float *filter, const int32_t *face, const float *weight,
                                   const float *bias, const float *scale, const float *shift, int relu, float *output,
                                   uint32_t *relu_bits, float *conv_rows, int64_t Nv, int64_t Nf, int C, int Co,
                                   pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(Nv >= 0 && Nf >= 0, "v2f_dense_fwd: negative size");
    if (Nf == 0) return 0;
    PM_REQUIRE(Nv > 0, "v2f_dense_fwd: facets without vertices");
    PM_REQUIRE(input && filter && face && weight && output, "v2f_dense_fwd: null pointer");
    PM_REQUIRE(Nv <= INT32_MAX && Nf <= INT32_MAX / 3, "v2f_dense_fwd: sizes exceed int32 indexing");
    PM_REQUIRE(C > 0 && C % 4 == 0, "v2f_dense_fwd: the channel count must be a multiple of 4 (got %d)", C);
    PM_REQUIRE(Nv * (int64_t)C * 4 < (int64_t(1) << 32), "v2f_dense_fwd: vertex array too large for 32-bit offsets");
    const RowGather gat{face, filter, conv_rows};
    return dense_rows("v2f_dense_fwd", input, nullptr, nullptr, relu_bits, weight, Co, 1, bias, scale, shift, relu, output, Nf,
                      C, Co, (hipStream_t)stream, &gat);
}

extern "C" size_t pmesh_dense_bwd_workspace_bytes(int64_t N, int Ci, int Co)
{
    if (N <= 0 || Ci <= 0 || Co <= 0) return 256;
    const WgradPlan p = wgrad_plan(N, Ci, Co);
    return (size_t)p.G * (size_t)(Ci + 1) * Co * sizeof(float) + 256;
}

extern "C" int pmesh_dense_bwd(const float *grad_output, const float *input, const float *weight, const float *output,
                               const uint32_t *relu_bits, float *grad_input, float *grad_weight, float *grad_bias,
                               void *workspace, size_t workspace_bytes, int64_t N, int Ci, int Co, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(N >= 0 && Ci > 0 && Co > 0, "dense_bwd: bad sizes");
    PM_REQUIRE(grad_weight && grad_bias, "dense_bwd: null gradient pointer");
    hipStream_t st = (hipStream_t)stream;
    if (N == 0) {
        const int rc = reduce_partials(nullptr, grad_weight, 0, Ci * Co, st);
        return rc ? rc : reduce_partials(nullptr, grad_bias, 0, Co, st);
    }
    PM_REQUIRE(grad_output && input && weight && workspace, "dense_bwd: null pointer");
    PM_REQUIRE((int64_t)Ci * Co <= (int64_t(1) << 24), "dense_bwd: weight too large");
    if (relu_bits) output = nullptr;          // the bits are the cheaper form of the same mask
    if (grad_input) {
        // grad_input (N x Ci) = gz (N x Co) . W^T: element (k = co, c = ci) of the matrix is weight[ci * Co + co]
        const int rc = dense_rows("dense_bwd(input)", grad_output, output, relu_bits, nullptr, weight, 1, Co, nullptr,
                                  nullptr, nullptr, 0, grad_input, N, Co, Ci, st);
        if (rc) return rc;
    }
    const WgradPlan p = wgrad_plan(N, Ci, Co);
    const size_t slice = (size_t)(Ci + 1) * Co;
    PM_REQUIRE(workspace_bytes >= (size_t)p.G * slice * sizeof(float), "dense_bwd: workspace too small (%zu bytes)",
               workspace_bytes);
    PM_REQUIRE(N * (int64_t)(Ci > Co ? Ci : Co) < (int64_t(1) << 40), "dense_bwd: sizes too large");
    float *partial = (float *)workspace;
    const bool vec = Ci % p.ta == 0 && Co % p.tb == 0 && aligned16(input) && aligned16(grad_output) &&
                     (!output || aligned16(output));
    const dim3 grid((unsigned)(p.G * p.nA * p.nB));
    const int mode = relu_bits ? 2 : output ? 1 : 0;
#define PM_WG(A, B) launch_wgrad<A, B>(vec, mode, grid, st, input, grad_output, output, relu_bits, partial, N, Ci, Co, p.nA, p.rows_per_wave)
    if (p.ta == 4 && p.tb == 2) PM_WG(4, 2);
    else if (p.ta == 4 && p.tb == 1) PM_WG(4, 1);
    else if (p.ta == 2 && p.tb == 4) PM_WG(2, 4);
    else if (p.ta == 2 && p.tb == 2) PM_WG(2, 2);
    else if (p.ta == 2 && p.tb == 1) PM_WG(2, 1);
    else if (p.ta == 1 && p.tb == 4) PM_WG(1, 4);
    else if (p.ta == 1 && p.tb == 2) PM_WG(1, 2);
    else PM_WG(1, 1);
#undef PM_WG
    PM_LAUNCHED("dense_bwd(weight)");
    int rc = reduce_partials(partial, grad_weight, p.G, Ci * Co, st, slice);
    if (rc) return rc;
    return reduce_partials(partial + (size_t)Ci * Co, grad_bias, p.G, Co, st, slice);
}

extern "C" int pmesh_bias_act_fwd(const float *input, const float *bias, const float *scale, const float *shift,
                                  int relu, float *output, uint32_t *relu_bits, int64_t N, int C, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(N >= 0 && C > 0, "bias_act_fwd: bad sizes");
    if (N == 0) return 0;
    PM_REQUIRE(input && output, "bias_act_fwd: null pointer");
    PM_REQUIRE(N * (int64_t)C < (int64_t(1) << 40), "bias_act_fwd: sizes too large");
    const bool v4 = C % 4 == 0 && aligned16(input) && aligned16(output);
    PM_REQUIRE(!relu_bits || (v4 && C % 32 == 0), "bias_act_fwd: the bit mask needs C %% 32 == 0 and 16-byte aligned rows");
    const int V = v4 ? 4 : 1;
    const int64_t n_items = N * C / V;
    const int64_t blocks = ceil_div(n_items, 256);
    PM_REQUIRE(grid_ok(blocks), "bias_act_fwd: grid too large");
    if (v4)
        bias_act_fwd_k<4><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(input, bias, scale, shift, relu,
                                                                                          output, relu_bits, n_items, C / 4);
    else
        bias_act_fwd_k<1><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(input, bias, scale, shift, relu,
                                                                                          output, nullptr, n_items, C);
    PM_LAUNCHED("bias_act_fwd");
    return 0;
}

extern "C" size_t pmesh_bias_act_bwd_workspace_bytes(int C)
{
    return (size_t)1024 * (size_t)(C > 0 ? C : 1) * sizeof(float);
}

extern "C" int pmesh_bias_act_bwd(const float *grad_output, const float *output, const uint32_t *relu_bits,
                                  float *grad_input, float *grad_bias, void *workspace, size_t workspace_bytes, int64_t N,
                                  int C, pmesh_stream_t stream)
{
    clear_error();
    PM_REQUIRE(N >= 0 && C > 0, "bias_act_bwd: bad sizes");
    PM_REQUIRE(grad_bias, "bias_act_bwd: null grad_bias");
    hipStream_t st = (hipStream_t)stream;
    if (N == 0) return reduce_partials(nullptr, grad_bias, 0, C, st);
    PM_REQUIRE(grad_output && workspace, "bias_act_bwd: null pointer");
    if (relu_bits) output = nullptr;
    PM_REQUIRE(!grad_input || output || relu_bits, "bias_act_bwd: grad_input is grad_output itself when there is no activation");
    PM_REQUIRE(N * (int64_t)C < (int64_t(1) << 40), "bias_act_bwd: sizes too large");
    const bool aligned = aligned16(grad_output) && (!output || aligned16(output)) && (!grad_input || aligned16(grad_input));
    const BiasPlan p = bias_plan(N, C, aligned);
    PM_REQUIRE(!relu_bits || (p.V == 4 && C % 32 == 0), "bias_act_bwd: the bit mask needs C %% 32 == 0 and 16-byte aligned rows");
    PM_REQUIRE(C / p.V <= 256 * kBiasLoops, "bias_act_bwd: more than %d channels", 256 * kBiasLoops * p.V);
    PM_REQUIRE(workspace_bytes >= (size_t)p.G * C * sizeof(float), "bias_act_bwd: workspace too small (%zu bytes)",
               workspace_bytes);
    float *partial = (float *)workspace;
    const dim3 grid((unsigned)p.G), block(256);
    if (p.V == 4) {
        if (relu_bits) bias_act_bwd_k<4, 2><<<grid, block, 0, st>>>(grad_output, output, relu_bits, grad_input, partial, N, C, p.lpr, p.rows_per_block);
        else if (output) bias_act_bwd_k<4, 1><<<grid, block, 0, st>>>(grad_output, output, relu_bits, grad_input, partial, N, C, p.lpr, p.rows_per_block);
        else bias_act_bwd_k<4, 0><<<grid, block, 0, st>>>(grad_output, output, relu_bits, grad_input, partial, N, C, p.lpr, p.rows_per_block);
    } else {
        if (output) bias_act_bwd_k<1, 1><<<grid, block, 0, st>>>(grad_output, output, relu_bits, grad_input, partial, N, C, p.lpr, p.rows_per_block);
        else bias_act_bwd_k<1, 0><<<grid, block, 0, st>>>(grad_output, output, relu_bits, grad_input, partial, N, C, p.lpr, p.rows_per_block);
    }
    PM_LAUNCHED("bias_act_bwd");
    return reduce_partials(partial, grad_bias, p.G, C, st);
}
