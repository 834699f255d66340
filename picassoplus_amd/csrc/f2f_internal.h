// Internal launchers of the F = 16 (spherical-harmonic degree 3) fast path of facet2facet.
#pragma once
#include "common.h"

namespace pmesh {

// The split-bf16 kernels (mesh_f2f16x3.hip) take any channel counts; they need F == 16 and 16-byte aligned
// filter and SH arrays.  Texture rows are read 16 bytes at a time when Cin % 4 == 0 and the array is aligned,
// element by element otherwise.
bool f2f16x3_usable(const void *W, const void *sh, int F);

// forward on the bf16 matrix cores with an exact three-way split of both operands (fp32-level accuracy)
size_t f2f16x3_fwd_workspace_bytes(int Cin, int Cout);
int f2f16x3_fwd(const float *tex, const float *W, const float *sh, const int *cum, const int *order, float *out,
                void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st);

// forward on the fp16 matrix cores with a two-way split and power-of-two scaling of both operands
// (mesh_f2f16h2.hip); same conditions as the bf16 kernels, workspace no larger than theirs
size_t f2f16h2_fwd_workspace_bytes(int Cin, int Cout);
// What the forward does to a value before it stores it: out = act(conv + bias) * scale + shift, every pointer optional
// (per output channel); bits (float features, Cout % 32 == 0): the ReLU mask, one word per facet and 32 channels.
struct F2FTail {
    const float *bias, *scale, *shift;
    unsigned *bits;
    int relu;
};
// bf16: texture and output rows are bf16 (unsigned short) instead of float; runs the one-product kernels
int f2f16h2_fwd(const void *tex, const float *W, const float *sh, const int *cum, const int *order, void *out,
                void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st, bool half = false,
                bool bf16 = false, const F2FTail *tail = nullptr);

// texture gradient on the fp16 matrix cores (conditions of the bf16 kernel, workspace no larger)
size_t f2f16h2_bwd_texture_workspace_bytes(int Cin, int Cout);
size_t f2f16h2_bwd_texture_bf16_workspace_bytes(int64_t T, int Cin, int Cout);
int f2f16h2_bwd_texture(const void *gout, const float *W, const float *sh, const int *cum, const int *order,
                        void *gtex, void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                        int Cout, hipStream_t st, bool half = false, bool bf16 = false, bool onto = false);

// texture gradient on the bf16 matrix cores (Cout % 8 == 0, 16-byte aligned grad_output; output channels are
// taken 64 at a time, later blocks accumulate onto grad_texture)
bool f2f16x3_bwd_texture_usable(const void *gout, int Cout);
size_t f2f16x3_bwd_texture_workspace_bytes(int Cin, int Cout);
int f2f16x3_bwd_texture(const float *gout, const float *W, const float *sh, const int *cum, const int *order,
                        float *gtex, void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                        int Cout, hipStream_t st);

// the same on the fp16 matrix cores (block-floating scales, see mesh_f2f16h2.hip).  *overflow (cleared by the
// caller) is set when the data outgrew the scales: the partials are then void and must be computed again by
// f2f16x3_bwd_filter_partials, whose `only_if` argument makes that launch a no-op otherwise.
int f2f16h2_bwd_filter_partials(const void *gout, const void *tex, const float *sh, const int *cum, const int *order,
                                 float *partial, int *overflow, int splits, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st,
                                 bool half = false, bool bf16 = false);

// `splits` workgroups each write one partial (Cout x Cin*16) block; every split gets a strided share of the 32-facet tiles
// only_if (may be null): device flag; the kernel returns at once when it reads 0
int f2f16x3_bwd_filter_partials(const void *gout, const void *tex, const float *sh, const int *cum, const int *order,
                                 float *partial, int splits, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st,
                                 const int *only_if = nullptr, bool bf16 = false);


// Narrow filter gradient (mesh_f2f_narrow.hip): at most four input channels, F == 16.  `blocks` partial
// gradients of Cout*Cin*16 floats are left in `partial` (blocks = f2f_narrow_blocks(Nf) <= kNarrowMaxBlocks).
constexpr int kNarrowMaxBlocks = 2048;
bool f2f_narrow_usable(int Cin, int F);
bool f2f_narrow_bwd_usable(int Cin, int F, int64_t Nf, int Cout);
int f2f_narrow_blocks(int64_t Nf);
int f2f_bwd_filter_narrow_partials(const float *gout, const float *tex, const float *sh, const int *cum, float *partial,
                                   int blocks, int64_t T, int64_t Nf, int Cin, int Cout, hipStream_t st);

// Narrow forward (same file): at most four input channels, F == 16, 16-byte aligned SH rows; no workspace.
bool f2f_fwd_narrow_usable(int Cin, int F, const void *sh);
int f2f_fwd_narrow(const float *tex, const float *W, const float *sh, const int *cum, float *out, int64_t T, int64_t Nf,
                   int Cin, int Cout, hipStream_t st);

}  // namespace pmesh
