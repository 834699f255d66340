// Internal interface between the row kernels' entry points (mesh_rows.hip) and the matrix-core
// facet2vertex kernels (mesh_f2v_mfma.hip).
#pragma once
#include "common.h"

namespace pmesh {

// out[i] = sum over the G slices of partial[g*stride + i], in a fixed tree order (mesh_rows.hip); stride 0
// means densely packed slices of n floats.  G == 0 stores zeros.
int reduce_partials(const float *partial, float *out, int G, int n, hipStream_t st, size_t stride = 0);

// K == 16 coefficients in 16-byte aligned rows, at least 32 output channels, 32-bit byte offsets into `input`.
bool f2v_mfma_ok(int64_t Nf, int C, int r, int K, const void *coeff);

// bf16: feature rows (in, out) are bf16 (unsigned short) instead of float
int f2v_fwd_mfma(const void *in, const float *filt, const float *coeff, const int *nfcount, const int *rowptr,
                 const int *colidx, void *out, int64_t Nf, int64_t NvOut, int C, int r, hipStream_t st, bool bf16 = false);

// facet2vertex with the module's pointwise tail on its store (float rows, 32 or 64 convolution channels C * r,
// 32 / 64 / 128 tail outputs Cd, the conditions of f2v_mfma_ok): out2 = max(conv . Wd + bias, 0 or -inf) * scale + shift;
// conv_out (may be null) also receives the convolution's rows, bits (may be null) the mask of positive activations;
// workspace: f2v_tail_workspace_bytes, 16-byte aligned.
bool f2v_tail_ok(int64_t Nf, int C, int r, int K, const void *coeff, int Cd);
size_t f2v_tail_workspace_bytes(int Co, int Cd);
int f2v_fwd_tail(const float *in, const float *filt, const float *coeff, const int *nfcount, const int *rowptr,
                 const int *colidx, float *conv_out, const float *Wd, const float *bias, const float *scale, const float *shift,
                 int relu, float *out2, unsigned *bits, void *workspace, int64_t Nf, int64_t NvOut, int C, int r, int Cd,
                 hipStream_t st);

// Backward on the matrix cores: depth multiplier 1 or 2, additionally NvOut * C * r * 4 < 2^32.  G workgroups
// (f2v_bwd_mfma_blocks) leave G partial filter gradients of 16 * C * r floats in `partial`.
int f2v_bwd_mfma_blocks(int64_t Nf);
int f2v_bwd_mfma(const void *gout, const void *in, const float *filt, const float *coeff, const int *face,
                 const int *nfcount, const int *vtmap, void *gin, float *partial, int G, int64_t Nf, int64_t NvOut,
                 int C, int r, hipStream_t st, bool bf16 = false);

// Stable radix sort of (32-bit key, id) pairs on the low `bits` bits of the keys (mesh_csr.hip); `temp` holds
// sort_pairs_temp_bytes(n, bits) bytes.
size_t sort_pairs_temp_bytes(int64_t n, int bits);
hipError_t sort_pairs(void *temp, size_t temp_bytes, const unsigned *keys_in, unsigned *keys_out, const int *vals_in,
                      int *vals_out, int64_t n, int bits, hipStream_t st);

}  // namespace pmesh
