/*
 * picasso_mesh.h -- C ABI of libpicasso_mesh.so (MI355X / gfx950).
 *
 * Replaces, for the mesh-convolution and mesh (un)pooling path, the three pybind11
 * torch extensions of EnyaHermite/PicassoPlus:
 *     mesh_conv3d   (picasso/mesh/pi_modules/source/mesh_conv3d.cpp:272-279)
 *     mesh_pool3d   (picasso/mesh/pi_modules/source/mesh_pool3d.cpp:151-157)
 *     mesh_unpool3d (picasso/mesh/pi_modules/source/mesh_unpool3d.cpp:81-85)
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller (PyTorch's allocator in the
 *     Python binding).  Features are float32, indices int32, all arrays row-major and
 *     densely packed, exactly what the reference's CHECK_INPUT macros enforce
 *     (mesh_conv3d.cpp:24-30).
 *   - Outputs and workspaces are allocated by the caller; the library never allocates
 *     device memory.  Outputs need no pre-clearing: every element is written.
 *   - `stream` is a hipStream_t passed as void*; work is enqueued there and the call
 *     returns without synchronising.
 *   - Return value 0 = success.  Non-zero = failure; pmesh_last_error() then returns a
 *     thread-local message.  Argument errors are detected before anything is launched.
 *   - Reductions run over sorted adjacency (CSR) in a fixed order: results are
 *     bit-reproducible from run to run, unlike the reference's float atomics.
 *   - Entry points are re-entrant; they keep no global mutable state (pmesh_f2v_bwd_static is the
 *     one exception, see there).
 *
 * Symbols: cout = c*r + m is the depth-multiplied output channel of the V2F / F2V
 * convolutions, (C, r) = filter.shape[1:].
 */
#ifndef PICASSO_MESH_H
#define PICASSO_MESH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *pmesh_stream_t;

/* ABI revision of this header; bumped on any signature change. */
int pmesh_abi_version(void);
/* Message of the last failing call on the calling thread ("" if none). */
const char *pmesh_last_error(void);
/* The library reads its switches from the environment once, at its first call: PMESH_F2F_GENERIC, PMESH_F2F_BF16X3,
 * PMESH_F2F_HALF, PMESH_F2V_VALU, PMESH_DENSE_FP32MFMA ("1" = set; they select other kernel families than the
 * default for comparison).  pmesh_reload_options() reads them again.  No counterpart in the reference. */
void pmesh_reload_options(void);

/* ------------------------------------------------------------------ adjacency (CSR)
 * The reference scatters with float atomics and therefore needs no adjacency.  Here the
 * scatter ops are segmented reductions over these arrays, built once per index tensor
 * and reused by every conv of a mesh level (forward and backward).
 */

/* Vertex -> incident (facet, corner) list.
 *   key(e) = vt_map ? vt_map[face[e]] : face[e]   for e = 3*f + corner, e in [0, 3*Nf)
 *   rowptr[v] .. rowptr[v+1]: slots of row v, v in [0, n_rows); colidx holds e, ascending
 *   within a row; entries with key < 0 are dropped (rowptr[n_rows] = number kept).
 *   rowptr: n_rows+1 ints, colidx: 3*Nf ints.
 * Serves facet2vertex forward (rows = output vertices, mesh_conv3d_gpu.cu:318-326) and
 * vertex2facet input-backward (rows = input vertices, vt_map = NULL, :213-216). */
size_t pmesh_vertex_csr_workspace_bytes(int64_t n_facets, int64_t n_rows);
int pmesh_build_vertex_csr(const int32_t *face, const int32_t *vt_map, int64_t n_facets,
                           int64_t n_vt_map, int64_t n_rows, int32_t *rowptr, int32_t *colidx,
                           void *workspace, size_t workspace_bytes, pmesh_stream_t stream);

/* Coarse vertex -> member list of a decimation cluster map.
 *   rep(v) = vt_replace[v] < 0 ? -vt_replace[v] : v ;  key(v) = vt_map[rep(v)]
 *   rowptr: n_coarse+1 ints; members: n_fine ints, ascending within a row.
 * Serves max/avg pool forward and unpool backward (mesh_pool3d_gpu.cu:39-58,109-129,
 * mesh_unpool3d_gpu.cu:27-46). */
size_t pmesh_cluster_csr_workspace_bytes(int64_t n_fine, int64_t n_coarse);
int pmesh_build_cluster_csr(const int32_t *vt_replace, const int32_t *vt_map, int64_t n_fine,
                            int64_t n_coarse, int32_t *rowptr, int32_t *members,
                            void *workspace, size_t workspace_bytes, pmesh_stream_t stream);

/* ------------------------------------------------------------------ vertex2facet
 * replaces vertex2facet_forward / vertex2facet_backward (mesh_conv3d.cpp:123-188)
 *   input (Nv,C)  filter (3,C,r)  face (Nf,3)  ->  output (Nf,C*r)
 */
int pmesh_v2f_fwd(const float *input, const float *filter, const int32_t *face, float *output,
                  int64_t Nv, int64_t Nf, int C, int r, pmesh_stream_t stream);

/* grad_input (Nv,C), grad_filter (3,C,r).  rowptr/colidx: vertex CSR with vt_map = NULL,
 * n_rows = Nv.  workspace: pmesh_v2f_bwd_workspace_bytes(C, r) bytes. */
size_t pmesh_v2f_bwd_workspace_bytes(int C, int r);
int pmesh_v2f_bwd(const float *grad_output, const float *input, const float *filter,
                  const int32_t *face, const int32_t *rowptr, const int32_t *colidx,
                  float *grad_input, float *grad_filter, void *workspace, size_t workspace_bytes,
                  int64_t Nv, int64_t Nf, int C, int r, pmesh_stream_t stream);

/* ------------------------------------------------------------------ facet2vertex
 * replaces facet2vertex_forward / facet2vertex_backward (mesh_conv3d.cpp:33-122)
 *   input (Nf,C)  filter (K,C,r)  coeff (Nf,K)  face (Nf,3)  nf_count (NvOut)  vt_map (NvIn)
 *   -> output (NvOut, C*r).  rowptr/colidx: vertex CSR with this vt_map, n_rows = NvOut.
 */
int pmesh_f2v_fwd(const float *input, const float *filter, const float *coeff,
                  const int32_t *nf_count, const int32_t *rowptr, const int32_t *colidx,
                  float *output, int64_t Nf, int64_t NvOut, int C, int r, int K,
                  pmesh_stream_t stream);

/* grad_input (Nf,C), grad_filter (K,C,r).  workspace: pmesh_f2v_bwd_workspace_bytes(C,r,K). */
size_t pmesh_f2v_bwd_workspace_bytes(int C, int r, int K);
int pmesh_f2v_bwd(const float *grad_output, const float *input, const float *filter,
                  const float *coeff, const int32_t *face, const int32_t *nf_count,
                  const int32_t *vt_map, float *grad_input, float *grad_filter, void *workspace,
                  size_t workspace_bytes, int64_t Nf, int64_t NvIn, int64_t NvOut, int C, int r,
                  int K, pmesh_stream_t stream);

/* pmesh_f2v_bwd for callers that cannot allocate device memory.  No counterpart in the reference (whose
 * extensions allocate their outputs and need no workspace): it is for code that runs under HIP graph capture,
 * tight serving loops and harnesses that forbid allocation.  Same arguments and results as pmesh_f2v_bwd without
 * the workspace: the partial filter gradients go to a device array of pmesh_f2v_bwd_static_max_bytes() (8 MiB)
 * that is part of the library image -- every GPU the library runs on holds its copy until the process ends.
 * Limit: pmesh_f2v_bwd_workspace_bytes(C, r, K) must fit, i.e. K * C * r <= 2048 (16 coefficients: C * r <= 128);
 * larger shapes fail with an error before anything is launched.  The call allocates and frees nothing.  All calls
 * on one GPU share the array, which keeps the last call's contents (nothing needs clearing: every slice read is
 * written first): calls that overlap on one GPU, on different streams or threads, race and must be serialised by
 * the caller.  Unlike every other entry point, this one keeps state in the library (the array's address per
 * device, looked up on the first call on that device). */
size_t pmesh_f2v_bwd_static_max_bytes(void);
int pmesh_f2v_bwd_static(const float *grad_output, const float *input, const float *filter,
                         const float *coeff, const int32_t *face, const int32_t *nf_count,
                         const int32_t *vt_map, float *grad_input, float *grad_filter, int64_t Nf,
                         int64_t NvIn, int64_t NvOut, int C, int r, int K, pmesh_stream_t stream);

/* ------------------------------------------------------------------ facet2facet
 * replaces facet2facet_forward / facet2facet_backward (mesh_conv3d.cpp:192-269)
 *   texture (T,Cin)  filter (Cout,Cin,F)  bary_coeff (T,F)  cum_texture (Nf, inclusive
 *   running total of texture points per facet, as layers.py:57 prepares it)
 *   -> output (Nf,Cout).   F <= 50 as in mesh_conv3d.cpp:211.
 * workspace: pmesh_f2f_fwd_workspace_bytes(Cin,Cout,F) bytes, 16-byte aligned (holds the filter
 * re-arranged for the matrix cores; may be 0 bytes for shapes that need none).
 * facet_order: NULL, or the permutation pmesh_build_facet_order made from this cum_texture.  It
 * only groups facets with equal numbers of texture points into the same workgroups (faster when
 * the counts vary).  With F = 16 the products run on fp16 matrix instructions with both operands
 * split in two and scaled by powers of two; a facet's scale may depend on its workgroup when one of
 * the workgroup's facets exceeds its first bound, so results with and without the order agree to
 * an ulp, and bit for bit otherwise.
 */
size_t pmesh_facet_order_workspace_bytes(int64_t n_facets);
int pmesh_build_facet_order(const int32_t *cum_texture, int64_t n_facets, int64_t n_points,
                            int32_t *order, void *workspace, size_t workspace_bytes,
                            pmesh_stream_t stream);

size_t pmesh_f2f_fwd_workspace_bytes(int Cin, int Cout, int F);
int pmesh_f2f_fwd(const float *texture, const float *filter, const float *bary_coeff,
                  const int32_t *cum_texture, const int32_t *facet_order, float *output, void *workspace,
                  size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, int F,
                  pmesh_stream_t stream);
/* The same with the module's tail on the store (picasso/mesh/layers.py:59-63: outputs + biases, activation_fn; the
 * per-channel scale and shift carry a batch norm that only applies its running statistics):
 *   output = act(conv + bias) * scale + shift      bias, scale, shift (Cout) each optional; relu: 0 / 1
 * relu_bits (NULL, or Nf * Cout/32 words when Cout % 32 == 0 and output is 16-byte aligned): bit c % 32 of word
 * [f][c / 32] is set where the ReLU let the value through, the form pmesh_bias_act_bwd takes.  The fp16 kernels for 16
 * coefficients apply the tail as they store; every other shape runs pmesh_f2f_fwd and then pmesh_bias_act_fwd in place. */
int pmesh_f2f_fwd_act(const float *texture, const float *filter, const float *bary_coeff,
                      const int32_t *cum_texture, const int32_t *facet_order, const float *bias,
                      const float *scale, const float *shift, int relu, float *output, uint32_t *relu_bits,
                      void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                      int F, pmesh_stream_t stream);

/* grad_texture (T,Cin), grad_filter (Cout,Cin,F).
 * workspace: pmesh_f2f_bwd_workspace_bytes(Cin,Cout,F), 16-byte aligned; the two halves may share
 * it when they run on the same stream.  facet_order: NULL or the permutation of
 * pmesh_build_facet_order, as for the forward (grad_texture is bit-identical with and without
 * it; grad_filter sums the facets in the order given, so its last bits depend on it, and on
 * nothing else).  With F = 16 the filter half runs an fp16 kernel whose block-floating scales hold
 * unless magnitudes grow by more than 2^9 along the facet list; it then flags the case on the
 * device and a second, guarded launch (three-piece bf16, no scales) computes the result again.  Every row of grad_texture is written
 * (rows past the last facet's segment are cleared) provided cum_texture is non-decreasing.
 * pmesh_f2f_bwd is the texture half followed by the filter half; each half can be called
 * alone when only one gradient is wanted (the reference always computes both,
 * mesh_conv3d_gpu.cu:144-168). */
size_t pmesh_f2f_bwd_workspace_bytes(int Cin, int Cout, int F);
/* The same for a given number of facets: the partial filter gradients take one slice per group of facets, so a
 * small mesh needs a fraction of the upper bound above (which holds for any Nf). */
size_t pmesh_f2f_bwd_workspace_bytes_for(int64_t Nf, int Cin, int Cout, int F);
int pmesh_f2f_bwd(const float *grad_output, const float *texture, const float *filter,
                  const float *bary_coeff, const int32_t *cum_texture, const int32_t *facet_order,
                  float *grad_texture, float *grad_filter, void *workspace, size_t workspace_bytes,
                  int64_t T, int64_t Nf, int Cin, int Cout, int F, pmesh_stream_t stream);
int pmesh_f2f_bwd_texture(const float *grad_output, const float *filter, const float *bary_coeff,
                          const int32_t *cum_texture, const int32_t *facet_order, float *grad_texture,
                          void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                          int Cout, int F, pmesh_stream_t stream);
/* pmesh_f2f_bwd_texture with the result ADDED to what grad_texture holds (rows that belong to no facet are left as
 * they are): a convolution with more than 16 coefficients runs as a sum over blocks of 16 (the texture gradient is
 * linear in the pair filter x coefficients), and the blocks after the first add onto the first one's result in
 * place instead of through a separate pass.  No counterpart in the reference.  Only where
 * pmesh_f2f_bwd_texture_onto_supported returns 1 (F == 16, Cout % 8 == 0, 16-byte aligned arrays). */
int pmesh_f2f_bwd_texture_onto_supported(const float *grad_output, const float *filter, const float *bary_coeff,
                                         int Cout, int F);
int pmesh_f2f_bwd_texture_onto(const float *grad_output, const float *filter, const float *bary_coeff,
                               const int32_t *cum_texture, const int32_t *facet_order, float *grad_texture,
                               void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                               int Cout, int F, pmesh_stream_t stream);
int pmesh_f2f_bwd_filter(const float *grad_output, const float *texture, const float *bary_coeff,
                         const int32_t *cum_texture, const int32_t *facet_order, float *grad_filter,
                         void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin,
                         int Cout, int F, pmesh_stream_t stream);

/* ------------------------------------------------------------------ features in bf16 (reduced-precision variant)
 * No counterpart in the reference, which computes in float32 throughout.  The convolutions of a layer with the
 * FEATURE tensors -- texture rows, layer inputs / outputs and their gradients -- kept in bf16 in HBM (uint16_t here:
 * the upper half of the float32 bit pattern, rounded to nearest even on store).  Filters, SH coefficients and filter
 * gradients stay float32; every sum is accumulated in float32; the facet2facet products take one fp16 piece per
 * operand (exact power-of-two scales as in the float32 path).  Results agree with the float64 evaluation of the same
 * bf16-rounded inputs within 1e-3 of the largest output before the final rounding to bf16.
 * Shapes: facet2facet F = 16, Cin % 4 == 0, Cout % 8 == 0; facet2vertex K = 16, C * r >= 32, r = 1 or 2.  Other
 * arguments, workspaces and the facet order are those of the float32 entry points of the same name, except the
 * backward workspace: pmesh_f2f_bwd_bf16_workspace_bytes (with more than 64 output channels the texture gradient
 * accumulates its blocks of 64 channels in a float32 copy of grad_texture inside the workspace). */
size_t pmesh_f2f_bwd_bf16_workspace_bytes(int64_t T, int64_t Nf, int Cin, int Cout, int F);
int pmesh_f2f_fwd_bf16(const uint16_t *texture, const float *filter, const float *bary_coeff,
                       const int32_t *cum_texture, const int32_t *facet_order, uint16_t *output, void *workspace,
                       size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout, int F,
                       pmesh_stream_t stream);
int pmesh_f2f_bwd_texture_bf16(const uint16_t *grad_output, const float *filter, const float *bary_coeff,
                               const int32_t *cum_texture, const int32_t *facet_order, uint16_t *grad_texture,
                               void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                               int F, pmesh_stream_t stream);
int pmesh_f2f_bwd_filter_bf16(const uint16_t *grad_output, const uint16_t *texture, const float *bary_coeff,
                              const int32_t *cum_texture, const int32_t *facet_order, float *grad_filter,
                              void *workspace, size_t workspace_bytes, int64_t T, int64_t Nf, int Cin, int Cout,
                              int F, pmesh_stream_t stream);
int pmesh_f2v_fwd_bf16(const uint16_t *input, const float *filter, const float *coeff, const int32_t *nf_count,
                       const int32_t *rowptr, const int32_t *colidx, uint16_t *output, int64_t Nf, int64_t NvOut,
                       int C, int r, int K, pmesh_stream_t stream);
int pmesh_f2v_bwd_bf16(const uint16_t *grad_output, const uint16_t *input, const float *filter, const float *coeff,
                       const int32_t *face, const int32_t *nf_count, const int32_t *vt_map, uint16_t *grad_input,
                       float *grad_filter, void *workspace, size_t workspace_bytes, int64_t Nf, int64_t NvIn,
                       int64_t NvOut, int C, int r, int K, pmesh_stream_t stream);

/* ------------------------------------------------------------------ mesh pooling
 * replaces max_forward / max_backward / avg_forward / avg_backward
 * (mesh_pool3d.cpp:29-148).  rowptr/members: cluster CSR of (vt_replace, vt_map).
 *   input (NvIn,C) -> output (NvOut,C) [, max_index (NvOut,C) int32]
 * Ties in the arg-max resolve to the smallest vertex index; rows without members get
 * value 0 and index 0, as the reference's zero-filled outputs do (mesh_pool3d.cpp:53-54).
 */
int pmesh_pool_max_fwd(const float *input, const int32_t *rowptr, const int32_t *members,
                       float *output, int32_t *max_index, int64_t NvIn, int64_t NvOut, int C,
                       pmesh_stream_t stream);
/* grad_input (NvIn,C).  With vt_replace/vt_map given, grad_input is produced by a gather
 * (row v takes grad_output where max_index names v) -- valid when max_index came from
 * pmesh_pool_max_fwd on the same maps.  With both NULL it is the reference's zero-fill
 * plus scatter by max_index (mesh_pool3d_gpu.cu:90-102). */
int pmesh_pool_max_bwd(const float *grad_output, const int32_t *max_index,
                       const int32_t *vt_replace, const int32_t *vt_map, float *grad_input,
                       int64_t NvIn, int64_t NvOut, int C, pmesh_stream_t stream);
int pmesh_pool_avg_fwd(const float *input, const int32_t *vt_replace, const int32_t *rowptr,
                       const int32_t *members, float *output, int64_t NvIn, int64_t NvOut, int C,
                       pmesh_stream_t stream);
int pmesh_pool_avg_bwd(const float *grad_output, const int32_t *vt_replace,
                       const int32_t *vt_map, float *grad_input, int64_t NvIn, int64_t NvOut,
                       int C, pmesh_stream_t stream);

/* ------------------------------------------------------------------ mesh unpooling
 * replaces forward / backward of mesh_unpool3d (mesh_unpool3d.cpp:20-78)
 *   input (NvCoarse,C) -> output (NvFine,C): every fine vertex copies its cluster's row.
 */
int pmesh_unpool_fwd(const float *input, const int32_t *vt_replace, const int32_t *vt_map,
                     float *output, int64_t NvCoarse, int64_t NvFine, int C,
                     pmesh_stream_t stream);
int pmesh_unpool_bwd(const float *grad_output, const int32_t *rowptr, const int32_t *members,
                     float *grad_input, int64_t NvCoarse, int64_t NvFine, int C,
                     pmesh_stream_t stream);

/* ------------------------------------------------------------------ spherical harmonics
 * replaces SphHarmCoeff.__call__ + torch_sph_harm_reorder (picasso/mesh/layers.py:348-356,
 * picasso/math_utils.py:10-62): real SH basis of degree <= L (L <= 5) at the directions
 * xyz (N,3) -> out (N,(L+1)^2); a zero vector evaluates at direction (1,0,0). */
int pmesh_sph_harm(const float *xyz, float *out, int64_t N, int L, pmesh_stream_t stream);

/* ------------------------------------------------------------------ texture points from vertex features
 * No counterpart among the reference's extensions: the reference reads the features of the texture
 * points from its dataset files (picasso/mesh/dataset_scene.py:29-33) and evaluates the basis of
 * their barycentric coordinates with SphHarmCoeff (picasso/networks/scene_seg.py:150).  An encoder
 * block that runs facet2facet on vertex features needs them interpolated:
 *   texture[k,c] = sum_j bary[k,j] * input[face[f,j], c]   for k in [cum_texture[f-1], cum_texture[f])
 *   bary_coeff[k,:] = SH basis of degree L at bary[k,:]     (as pmesh_sph_harm; NULL = not wanted)
 * in one pass: input (Nv,C), face (Nf,3), bary (T,3), cum_texture (Nf, inclusive running total as for
 * facet2facet) -> texture (T,C), bary_coeff (T,(L+1)^2).  Rows of texture / bary_coeff beyond
 * cum_texture[Nf-1] are not written.
 * Backward: grad_input (Nv,C) = transpose of the interpolation applied to grad_texture (T,C), summed in
 * adjacency order; rowptr/colidx: vertex CSR with vt_map = NULL, n_rows = Nv (the one
 * pmesh_v2f_bwd takes).  bary gets no gradient. */
int pmesh_texture_fwd(const float *input, const int32_t *face, const float *bary,
                      const int32_t *cum_texture, float *texture, float *bary_coeff, int64_t Nv,
                      int64_t Nf, int64_t T, int C, int L, pmesh_stream_t stream);
int pmesh_texture_bwd(const float *grad_texture, const float *bary, const int32_t *cum_texture,
                      const int32_t *rowptr, const int32_t *colidx, float *grad_input, int64_t Nv,
                      int64_t Nf, int64_t T, int C, pmesh_stream_t stream);

/* ------------------------------------------------------------------ per-level inputs of the convs
 * pmesh_count_vertex_adjface replaces count_vertex_adjface (decimate_gpu.cu:813-836,
 * decimate.py:88-93): the number of (facet, corner) entries per output vertex is the row length
 * of the facet2vertex CSR (pmesh_build_vertex_csr with that vt_map); nf_count (NvOut) int32.
 * pmesh_triangle_geometry replaces compute_triangle_geometry_ (decimate.py:70-85):
 * geometry (Nf,5) = unit normal, plane offset d = -n.v0, area; vertex rows have vertex_stride
 * floats (>= 3), position first.  normal = raw / (|raw| + 1e-10) as in the reference. */
int pmesh_count_vertex_adjface(const int32_t *rowptr, int32_t *nf_count, int64_t NvOut,
                               pmesh_stream_t stream);
int pmesh_triangle_geometry(const float *vertex, const int32_t *face, float *geometry, int64_t Nv,
                            int64_t Nf, int vertex_stride, pmesh_stream_t stream);

/* pmesh_facet_frame gives, in one pass over the facets, what a network computes per mesh level before its
 * facet2vertex convolutions: geometry (Nf,5) as pmesh_triangle_geometry; normal (Nf,3) = the unit normal turned
 * towards the origin as the viewpoint, i.e. negated when -centre . normal < 0 (get_oriented_normals,
 * picasso/networks/scene_seg.py:117-124); coeff (Nf,(L+1)^2) = SH basis at that normal (cal_sph_harm on the
 * oriented normals, scene_seg.py:149,164).  Any output pointer may be NULL. */
int pmesh_facet_frame(const float *vertex, const int32_t *face, float *geometry, float *normal, float *coeff,
                      int64_t Nv, int64_t Nf, int vertex_stride, int L, pmesh_stream_t stream);

/* pmesh_combine_clusters replaces combineClustersLauncher (decimate_gpu.cu:750-810, decimate.py:53-67): the
 * cluster maps of two consecutive decimation steps -- A over nv_a fine vertices, B over the nv_b vertices A
 * keeps -- become one pair (rep_out, map_out) over the fine vertices, the vt_replace / vt_map a pooling layer
 * over both steps takes.  rep: -r = contracted into vertex r, >= 0 = number of vertices contracted into this
 * one; map: row among the kept vertices or -1.  scratch: nv_b int32.  Counts are integer sums, so the result
 * does not depend on the order of execution. */
int pmesh_combine_clusters(const int32_t *rep_a, const int32_t *map_a, const int32_t *rep_b,
                           const int32_t *map_b, int32_t *rep_out, int32_t *map_out, int32_t *scratch,
                           int64_t nv_a, int64_t nv_b, pmesh_stream_t stream);

/* ------------------------------------------------------------------ mesh decimation (producer of the cluster maps)
 * The arithmetic of one decimation round, meshDecimationLauncher (decimate_gpu.cu:618-747), re-specified with fixed
 * summation orders and total orders so that vt_replace / vt_map are the same on every run (the reference's float
 * atomics, unstable sorts and tie handling make them vary).  The integer plumbing between these calls -- edge
 * extraction, sorting, unique, scans -- is the caller's (picassoplus_amd/mesh/pi_modules/decimate.py).
 *   pmesh_vertex_quadrics    quadric (Nv,10) of every vertex from its facets (initVertexQuadrics :220-247), summed
 *                            over the vertex CSR in ascending (facet, corner) order; geometry (Nf,5) as
 *                            pmesh_triangle_geometry; use_area weights a facet by area * 100 / 3, else by 1.
 *   pmesh_boundary_quadrics  rows (n_edges,10): weighted quadric of the plane through each boundary edge
 *                            perpendicular to its facet (addBoundaryQuadrics :304-362); the caller adds row i to both
 *                            end points, in ascending edge order.
 *   pmesh_edge_costs         contraction cost of each candidate edge (vi, vj) (computeEdgeCost :365-404, with the
 *                            3 x 3 solve and conditioning test of RrefDim3 :79-193).
 *   pmesh_cluster_vertices_host  the two greedy passes of clusterVertices (:561-614) over ONE sample's candidate
 *                            edges in contraction order.  HOST pointers, like the reference's host routine.  An edge
 *                            of the second pass joins its free end to the cluster of its covered end in either
 *                            position (the reference contracts a covered non-seed vertex into a free one when they
 *                            come in that order, which leaves chains the pooling ops cannot follow). */
/*   pmesh_edge_list_count / _fill  the unique edges (vi < vj) of the facets in ascending (vi, vj) order, replacing
 *                            the sort of all 3 Nf facet edges and the duplicate removal (:250-297): one thread per
 *                            vertex orders the higher corners of the facets in its row of the vertex CSR (rowptr,
 *                            colidx of pmesh_build_vertex_csr over `face`).  count: counts (2,Nv) <- per vertex the
 *                            number of edges it is the lower end of, and of those held by ONE facet side (boundary
 *                            edges).  fill: offsets (2,Nv) = exclusive running totals of each row of counts; writes the edges,
 *                            and the boundary edges with the facet that holds each.  spill: 12 Nf ints, touched by
 *                            rows of more than 16 entries only; with spill NULL such a row sets *need_spill (which
 *                            the caller zeroes beforehand) and counts nothing: call again with a spill area. */
int pmesh_edge_list_count(const int32_t *face, const int32_t *rowptr, const int32_t *colidx, int64_t Nv, int64_t Nf,
                          int32_t *counts, int32_t *spill, int32_t *need_spill, pmesh_stream_t stream);
int pmesh_edge_list_fill(const int32_t *face, const int32_t *rowptr, const int32_t *colidx, int64_t Nv, int64_t Nf,
                         const int32_t *offsets, int32_t *edge_vi, int32_t *edge_vj, int32_t *bnd_vi, int32_t *bnd_vj,
                         int32_t *bnd_face, int32_t *spill, pmesh_stream_t stream);
int pmesh_vertex_quadrics(const float *geometry, const int32_t *rowptr, const int32_t *colidx, float *quadric,
                          int64_t Nv, int use_area, pmesh_stream_t stream);
int pmesh_boundary_quadrics(const float *vertex, const float *geometry, const int32_t *edge_vi, const int32_t *edge_vj,
                            const int32_t *edge_face, float *rows, int64_t n_edges, int vertex_stride, int use_area,
                            float wgt_bnd, pmesh_stream_t stream);
int pmesh_edge_costs(const float *vertex, const float *quadric, const int32_t *edge_vi, const int32_t *edge_vj,
                     float *cost, int64_t n_edges, int vertex_stride, pmesh_stream_t stream);
/* Sort keys of the contraction order (the reference sorts (sample, cost) with thrust, decimate_gpu.cu:662-686; ties
 * are broken here by a 24-bit mix of the end points, then by (vi, vj) through a stable sort): keys[e] =
 * sample(vi) << 56 | cost as order-preserving 32-bit integer << 24 | mix(vi, vj), for B < 128 samples with the running
 * totals nv_cumsum of their vertex counts. */
int pmesh_contraction_keys(const float *cost, const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *nv_cumsum,
                           int64_t n_edges, int B, int64_t *keys, pmesh_stream_t stream);
int pmesh_cluster_vertices_host(const int32_t *edge_vi, const int32_t *edge_vj, int64_t n_edges, int32_t vt_start,
                                int32_t vt_num, int32_t n_remove, int32_t *vt_replace);

/* After the clustering (decimate_gpu.cu:487-549): pmesh_simplify_faces writes the facets over the clusters'
 * representatives (new_face (Nf,3)), which of them collapse (degenerate (Nf) bytes, alive = 1 - degenerate as int32
 * for the caller's running totals) and which vertices keep a facet (kept (Nv), cleared here first);
 * pmesh_simplify_renumber, given kept_total = inclusive running total of kept, the output numbering: vt_map (Nv)
 * = kept_total - 1 for kept vertices, -1 otherwise, and face_out (Nf,3) = vt_map of the new corners for live
 * facets (collapsed facets keep their unmapped corners, as in the reference). */
int pmesh_simplify_faces(const int32_t *face, const int32_t *vt_replace, int64_t Nf, int64_t Nv, int32_t *new_face,
                         uint8_t *degenerate, int32_t *alive, int32_t *kept, pmesh_stream_t stream);
int pmesh_simplify_renumber(const int32_t *new_face, const uint8_t *degenerate, const int32_t *kept,
                            const int32_t *kept_total, int64_t Nf, int64_t Nv, int32_t *vt_map, int32_t *face_out,
                            pmesh_stream_t stream);

/* The same two passes (clusterVertices, decimate_gpu.cu:561-614) for the whole batch on the DEVICE, in four steps
 * between which the chosen edges are cut by their rank within the sample (a running total of the caller's + pmesh_cluster_cut): the result is
 * that of pmesh_cluster_vertices_host sample by sample.  edge_vi / edge_vj: the candidate edges of all samples in
 * ascending (vi, vj) order (vi < vj, every edge inside one sample; neighbouring threads then touch neighbouring
 * vertices), edge_rank: each edge's position in the contraction order (distinct integers, ascending within a sample
 * in the order the serial routine would walk them).
 *   pmesh_cluster_match           `rounds` rounds of the first pass's fixed point (an edge is chosen when it is the
 *                                 lowest-ranked edge with two free ends at both of its ends).  state (Nv) and chosen
 *                                 (n_edges) are zero before the first call and carry over; best (Nv) is scratch.
 *                                 status[0] <- 1 while an edge with two free ends is left (call again), status[1]
 *                                 <- 1 if an edge is not (0 <= vi < vj < Nv) -- such an edge is left out.
 *   pmesh_cluster_ranks           edge_rank / edge_sample from the contraction order: order (n_edges) lists the edges
 *                                 in the order of contraction, order_sample their samples in that order.
 *   pmesh_cluster_flags_by_rank   by_rank[edge_rank[e]] = (flags[e] != 0): the chosen edges in contraction order, for
 *                                 the caller's running total `run` (inclusive, int32).
 *   pmesh_cluster_cut             keep[e] = flags[e] and the edge is among the first allowance[sample] flagged edges of
 *                                 its sample; first (B + 1): where each sample's edges begin in the contraction order.
 *                                 With sample_open / left (B, together or both null): whether the sample's flagged
 *                                 edges stayed below its allowance, and the allowance they leave.
 *   pmesh_cluster_contract_pairs  vt_replace[vi] = -vj, vt_replace[vj] = 1 for the edges with keep != 0 (the chosen
 *                                 edges whose rank among the sample's chosen edges is within its budget).
 *   pmesh_cluster_attach_propose  second pass, for the samples with sample_open != 0 (budget not exhausted by the
 *                                 first): first_edge (Nv) <- for every free vertex the rank of its first edge to a
 *                                 covered vertex whose cluster's representative is not vertex 0; attaches (n_edges)
 *                                 <- 1 for these edges.
 *   pmesh_cluster_attach          for the edges with keep != 0 among them: the free end joins the covered end's
 *                                 cluster; pairs = a copy of vt_replace as the first pass left it. */
int pmesh_cluster_match(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank, int64_t n_edges, int64_t Nv,
                        int32_t *state, int32_t *best, int32_t *chosen, int32_t *status, int rounds, pmesh_stream_t stream);
int pmesh_cluster_ranks(const int64_t *order, const int32_t *order_sample, int64_t n_edges, int32_t *edge_rank, int32_t *edge_sample,
                        pmesh_stream_t stream);
int pmesh_cluster_flags_by_rank(const int32_t *flags, const int32_t *edge_rank, int64_t n_edges, int32_t *by_rank, pmesh_stream_t stream);
int pmesh_cluster_cut(const int32_t *flags, const int32_t *edge_rank, const int32_t *edge_sample, const int32_t *run,
                      const int64_t *first, const int32_t *allowance, int64_t n_edges, int B, int32_t *keep, int32_t *sample_open,
                      int32_t *left, pmesh_stream_t stream);
int pmesh_cluster_contract_pairs(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *keep, int64_t n_edges,
                                 int32_t *vt_replace, pmesh_stream_t stream);
int pmesh_cluster_attach_propose(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank,
                                 const int32_t *edge_sample, const int32_t *sample_open, int64_t n_edges, int64_t Nv,
                                 const int32_t *vt_replace, int32_t *first_edge, int32_t *attaches, pmesh_stream_t stream);
int pmesh_cluster_attach(const int32_t *edge_vi, const int32_t *edge_vj, const int32_t *edge_rank, const int32_t *keep,
                         int64_t n_edges, const int32_t *first_edge, const int32_t *pairs, int32_t *vt_replace,
                         pmesh_stream_t stream);

/* ------------------------------------------------------------------ pointwise tail of the convs
 * replaces the PyTorch ops that follow every convolution (picasso/mesh/layers.py:114-119, 169-174,
 * 232-238: torch.matmul(outputs, depth_weights) + biases, activation_fn, BatchNorm) by one pass:
 *   output (N,Co) = act(input (N,Ci) . weight (Ci,Co) + bias (Co)) * scale (Co) + shift (Co)
 * relu != 0 selects max(.,0), else identity; bias, scale, shift may be NULL (0, 1, 0): scale/shift carry
 * an inference-mode batch norm (gamma/sqrt(var+eps), beta - mean*that).  Ci <= 896.
 * relu_bits (NULL or N * ceil(Co/32) uint32) receives one bit per output entry, set where the activated value
 * is > 0 (bit c % 32 of word c / 32 of the row): the ReLU mask for the backward pass at 1/32 of the output's size.
 * pmesh_dense_bwd is the gradient of the tail without scale/shift (training-mode batch norm stays
 * outside): gz = grad_output where the ReLU let the value through -- read from relu_bits when given, else
 * from output > 0 (output = the forward result); both NULL = no activation.
 * grad_input (N,Ci) = gz . weight^T (NULL skips it; needs Co <= 896), grad_weight (Ci,Co) = input^T . gz,
 * grad_bias (Co) = column sums of gz; both sums in a fixed order. */
int pmesh_dense_fwd(const float *input, const float *weight, const float *bias, const float *scale,
                    const float *shift, int relu, float *output, uint32_t *relu_bits, int64_t N, int Ci,
                    int Co, pmesh_stream_t stream);
size_t pmesh_dense_bwd_workspace_bytes(int64_t N, int Ci, int Co);
int pmesh_dense_bwd(const float *grad_output, const float *input, const float *weight,
                    const float *output, const uint32_t *relu_bits, float *grad_input,
                    float *grad_weight, float *grad_bias, void *workspace, size_t workspace_bytes,
                    int64_t N, int Ci, int Co, pmesh_stream_t stream);

/* vertex2facet (depth multiplier 1) and its tail as ONE pass: replaces mesh_conv3d.vertex2facet_forward
 * (mesh_conv3d.cpp:123-152, kernel mesh_conv3d_gpu.cu:176-195) followed by the PyTorch ops of V2FConv3d.forward
 * (picasso/mesh/layers.py:113-119):
 *   output (Nf,Co) = act((sum_j filter[j] * input[face[:,j]]) . weight (C,Co) + bias) * scale + shift
 * The facet rows of the convolution are formed in the loads of the product (three gathered vertex rows per facet,
 * weighted per channel) and never pass through memory -- unless conv_rows (Nf,C) is given, which receives them for
 * the backward pass (pmesh_dense_bwd takes them as its `input`, pmesh_v2f_bwd the gradient that comes out of it).
 * filter (3,C) = the (3,C,1) filter of pmesh_v2f_fwd; C % 4 == 0, C <= 896; every face index in [0, Nv) (the
 * caller's check, as for pmesh_v2f_fwd); bias, scale, shift, relu, relu_bits as in pmesh_dense_fwd. */
int pmesh_v2f_dense_fwd(const float *input, const float *filter, const int32_t *face, const float *weight,
                        const float *bias, const float *scale, const float *shift, int relu, float *output,
                        uint32_t *relu_bits, float *conv_rows, int64_t Nv, int64_t Nf, int C, int Co,
                        pmesh_stream_t stream);

/* facet2vertex and its tail as ONE pass: replaces mesh_conv3d.facet2vertex_forward (mesh_conv3d.cpp:258-291,
 * kernel mesh_conv3d_gpu.cu:299-330) followed by the PyTorch ops of F2VConv3d.forward
 * (picasso/mesh/layers.py:163-174):
 *   output (NvOut,Co) = act(facet2vertex(input, filter, coeff) (NvOut,C*r) . weight (C*r,Co) + bias) * scale + shift
 * A wavefront keeps the vertex rows of four passes of the convolution kernel in LDS and multiplies the 16 rows by the
 * weights on the matrix cores before they leave; conv_rows (NvOut,C*r), when given, also receives them for the
 * backward pass (pmesh_dense_bwd takes them as its `input`, pmesh_f2v_bwd the gradient that comes out of it).
 * Supported (pmesh_f2v_dense_supported returns 1): K == 16 with 16-byte aligned coeff rows, C*r == 32 or 64,
 * Co == 32, 64 or 128; other shapes run pmesh_f2v_fwd and pmesh_dense_fwd.  rowptr / colidx as in pmesh_f2v_fwd;
 * bias, scale, shift, relu, relu_bits as in pmesh_dense_fwd; workspace (16-byte aligned): the packed weights. */
int pmesh_f2v_dense_supported(int64_t Nf, int C, int r, int K, int Co, const float *coeff);
size_t pmesh_f2v_dense_fwd_workspace_bytes(int C, int r, int Co);
int pmesh_f2v_dense_fwd(const float *input, const float *filter, const float *coeff, const int32_t *nf_count,
                        const int32_t *rowptr, const int32_t *colidx, const float *weight, const float *bias,
                        const float *scale, const float *shift, int relu, float *output, uint32_t *relu_bits,
                        float *conv_rows, void *workspace, size_t workspace_bytes, int64_t Nf, int64_t NvOut, int C,
                        int r, int K, int Co, pmesh_stream_t stream);

/* The same tail for a convolution that mixes the channels itself (F2FConv3d, picasso/mesh/layers.py:60-64:
 * outputs + biases, activation_fn, BatchNorm): output (N,C) = act(input + bias) * scale + shift, one pass;
 * output may be input.  relu_bits as in pmesh_dense_fwd (NULL, or N * C/32 words when C % 32 == 0 and the rows
 * are 16-byte aligned).  pmesh_bias_act_bwd: grad_input = grad_output where the ReLU let the value through
 * (relu_bits, else output > 0; both NULL = no activation: then the gradient of the input is grad_output
 * itself and grad_input must be NULL), grad_bias (C) = column sums of that, in a fixed order.  The backward
 * takes C <= 1024, or <= 4096 when C % 4 == 0 and the pointers are 16-byte aligned. */
int pmesh_bias_act_fwd(const float *input, const float *bias, const float *scale, const float *shift,
                       int relu, float *output, uint32_t *relu_bits, int64_t N, int C,
                       pmesh_stream_t stream);
size_t pmesh_bias_act_bwd_workspace_bytes(int C);
int pmesh_bias_act_bwd(const float *grad_output, const float *output, const uint32_t *relu_bits,
                       float *grad_input, float *grad_bias, void *workspace, size_t workspace_bytes,
                       int64_t N, int C, pmesh_stream_t stream);

/* ------------------------------------------------------------------ point-cloud branch
 * replaces the reference's point_nnquery / point_sample / point_buildkernel / point_conv3d / point_pool3d /
 * point_unpool3d extensions (picasso/point/pi_modules/source/).  Points of a batch are concatenated;
 * nv_database / nv_query are INCLUSIVE running totals of the points per sample (B entries), as the reference's
 * wrappers pass them (picasso/point/pi_modules/nnquery.py:20-21).  Pairs are (query, database point) rows.
 *
 * Adjacency of an index column: row r -> ascending list of the entries i with keys[i * key_stride] == r (entries
 * outside [0, n_rows) belong to no row).  The point ops take it sorted by query for their forward, by database
 * point for their input gradients; pmesh_point_unpool_bwd takes it over the flattened (Nrows * K) index array. */
size_t pmesh_index_csr_workspace_bytes(int64_t n, int64_t n_rows);
int pmesh_build_index_csr(const int32_t *keys, int key_stride, int64_t n, int64_t n_rows, int32_t *rowptr,
                          int32_t *order, void *workspace, size_t workspace_bytes, pmesh_stream_t stream);

/* range search (nnquery.cpp:29-78 "range", nnquery_gpu.cu:20-126): database points of the query's sample closer than
 * radius, ascending, the first nn_sample of them.  Two steps, because the caller allocates the pair arrays between
 * them: count (Mp) <- neighbours per query; then, with cnt_info = inclusive running total of count (int64) and
 * Nout = its last entry, nn_index (Nout,2) and nn_dist (Nout) <- the pairs and their distances. */
int pmesh_point_range_count(const float *database, const float *query, const int32_t *nv_database,
                            const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float radius, int nn_sample,
                            int32_t *count, pmesh_stream_t stream);
int pmesh_point_range_fill(const float *database, const float *query, const int32_t *nv_database,
                           const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float radius, const int64_t *cnt_info,
                           int64_t Nout, int32_t *nn_index, float *nn_dist, pmesh_stream_t stream);
/* cube search (nnquery.cpp:81-129 "cube", nnquery_gpu.cu:134-250): neighbours inside the axis-aligned cube of edge
 * length; nn_index (Nout,3) = query, database point, cell of a grid_size^3 grid over the cube. */
int pmesh_point_cube_count(const float *database, const float *query, const int32_t *nv_database,
                           const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float length, int nn_sample,
                           int32_t *count, pmesh_stream_t stream);
int pmesh_point_cube_fill(const float *database, const float *query, const int32_t *nv_database,
                          const int32_t *nv_query, int B, int64_t Np, int64_t Mp, float length, int grid_size,
                          const int64_t *cnt_info, int64_t Nout, int32_t *nn_index, pmesh_stream_t stream);
/* The range and cube searches over a cell grid of the database points: the same outputs as the four functions above
 * (which scan a query's whole sample, as nnquery_gpu.cu:20-250 does), at a cost that grows with the neighbours
 * instead of the sample size.  pmesh_point_grid_build sorts the database points into cells at least `reach` wide
 * (the radius of the range searches, half the edge of the cube searches that will use the grid; a search that
 * reaches further still works, over more cells) and leaves the grid in `grid` (256-byte aligned,
 * pmesh_point_grid_workspace_bytes(Np) bytes; Np > 0, B <= 2^20).  The *_grid searches take the grid and otherwise
 * the arguments of their scanning counterparts. */
size_t pmesh_point_grid_workspace_bytes(int64_t Np);
int pmesh_point_grid_build(const float *database, const int32_t *nv_database, int B, int64_t Np, float reach,
                           void *grid, size_t grid_bytes, pmesh_stream_t stream);
int pmesh_point_range_count_grid(const void *grid, const float *database, const float *query,
                                 const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                 float radius, int nn_sample, int32_t *count, pmesh_stream_t stream);
int pmesh_point_range_fill_grid(const void *grid, const float *database, const float *query,
                                const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                float radius, const int64_t *cnt_info, int64_t Nout, int32_t *nn_index, float *nn_dist,
                                pmesh_stream_t stream);
int pmesh_point_cube_count_grid(const void *grid, const float *database, const float *query,
                                const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                                float length, int nn_sample, int32_t *count, pmesh_stream_t stream);
int pmesh_point_cube_fill_grid(const void *grid, const float *database, const float *query,
                               const int32_t *nv_database, const int32_t *nv_query, int B, int64_t Np, int64_t Mp,
                               float length, int grid_size, const int64_t *cnt_info, int64_t Nout, int32_t *nn_index,
                               pmesh_stream_t stream);
/* three nearest neighbours (nnquery.cpp:132-171 "knn3", nnquery_gpu.cu:262-330): nn_index, nn_dist (Mp,3). */
int pmesh_point_knn3(const float *database, const float *query, const int32_t *nv_database, const int32_t *nv_query,
                     int B, int64_t Np, int64_t Mp, int32_t *nn_index, float *nn_dist, pmesh_stream_t stream);
/* The same search over a cell grid (pmesh_point_grid_build with reach = -c: no radius to go by, about c cells per
 * database point of a sample), same nn_index and nn_dist bit for bit: the window of cells around a query grows
 * until its third nearest is closer than anything outside the window can be. */
int pmesh_point_knn3_grid(const void *grid, const float *database, const float *query, const int32_t *nv_database,
                          const int32_t *nv_query, int B, int64_t Np, int64_t Mp, int32_t *nn_index, float *nn_dist,
                          pmesh_stream_t stream);
/* farthest point sampling (sample.cpp:20-50 "fps", sample_gpu.cu:11-100): index_out (Mp) <- per sample its first
 * point, then repeatedly the point farthest from those chosen (lowest index among equals); temp: Np floats. */
int pmesh_point_fps(const float *xyz, const int32_t *nv_in, const int32_t *nv_out, int B, int64_t Np, int64_t Mp,
                    float *temp, int32_t *index_out, pmesh_stream_t stream);
/* kernel bins of neighbour pairs (buildkernel.cpp:22-117 "SPH3D", "fuzzySPH3D", buildkernel_gpu.cu:20-155): an
 * (n azimuth, p elevation, q radial) spherical kernel plus the centre bin 0.  filt_index (Nout); fuzzy form:
 * filt_index, filt_coeff (Nout,3): centre, own elevation bin, neighbouring elevation bin. */
int pmesh_point_sph3d_kernel(const float *database, const float *query, const int32_t *nn_index, const float *nn_dist,
                             int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q, float radius,
                             int32_t *filt_index, pmesh_stream_t stream);
int pmesh_point_fuzzy_sph3d_kernel(const float *database, const float *query, const int32_t *nn_index,
                                   const float *nn_dist, int64_t Nout, int64_t Np, int64_t Mp, int n, int p, int q,
                                   float radius, int32_t *filt_index, float *filt_coeff, pmesh_stream_t stream);

/* depthwise point convolution (pcloud_conv3d.cpp:29-213: SPH3D_forward/backward, fuzzySPH3D_forward/backward):
 *   input (Np,C), filter (F,C,r), nn_count (Mp), nn_index (Nout,2), bin_index (Nout,T), bin_coeff (Nout,T) or NULL
 *   (plain form: T = 1, weight 1) -> output (Mp,C*r); rowptr / order: the pairs sorted by query (key column 0).
 * backward: grad_input (Np,C) (NULL skips it; needs rowptr_in / order_in: the pairs sorted by database point, key
 * column 1), grad_filter (F,C,r); workspace pmesh_point_conv_bwd_workspace_bytes.  At most 512 bins. */
int pmesh_point_conv_fwd(const float *input, const float *filter, const int32_t *nn_count, const int32_t *nn_index,
                         const int32_t *bin_index, const float *bin_coeff, const int32_t *rowptr, const int32_t *order,
                         float *output, int64_t Np, int64_t Mp, int64_t Nout, int F, int C, int r, int T,
                         pmesh_stream_t stream);
size_t pmesh_point_conv_bwd_workspace_bytes(int64_t Nout, int F, int C, int r);
int pmesh_point_conv_bwd(const float *grad_output, const float *input, const float *filter, const int32_t *nn_count,
                         const int32_t *nn_index, const int32_t *bin_index, const float *bin_coeff,
                         const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, float *grad_filter,
                         void *workspace, size_t workspace_bytes, int64_t Np, int64_t Mp, int64_t Nout, int F, int C,
                         int r, int T, pmesh_stream_t stream);

/* point pooling (pcloud_pool3d.cpp:23-148): input (Np,C) -> output (Mp,C) over the pairs.  max: max_index (Mp,C) =
 * database point that holds the maximum (first pair among equals; -1 and output 0 for a query without pairs); its
 * backward gathers, per database point, the gradients of the queries whose maximum it holds. */
int pmesh_point_pool_max_fwd(const float *input, const int32_t *nn_index, const int32_t *rowptr, const int32_t *order,
                             float *output, int32_t *max_index, int64_t Np, int64_t Mp, int64_t Nout, int C,
                             pmesh_stream_t stream);
int pmesh_point_pool_max_bwd(const float *grad_output, const int32_t *max_index, const int32_t *nn_index,
                             const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, int64_t Np, int64_t Mp,
                             int64_t Nout, int C, pmesh_stream_t stream);
int pmesh_point_pool_avg_fwd(const float *input, const int32_t *nn_count, const int32_t *nn_index, const int32_t *rowptr,
                             const int32_t *order, float *output, int64_t Np, int64_t Mp, int64_t Nout, int C,
                             pmesh_stream_t stream);
int pmesh_point_pool_avg_bwd(const float *grad_output, const int32_t *nn_count, const int32_t *nn_index,
                             const int32_t *rowptr_in, const int32_t *order_in, float *grad_input, int64_t Np, int64_t Mp,
                             int64_t Nout, int C, pmesh_stream_t stream);

/* weighted unpooling (pcloud_unpool3d.cpp:20-83): output (Nrows,C) = sum_k input[nn_index[o,k]] * weight[o,k] with
 * nn_index, weight (Nrows,K), input (Nin,C); backward over the adjacency of the flattened index array. */
int pmesh_point_unpool_fwd(const float *input, const float *weight, const int32_t *nn_index, float *output, int64_t Nrows,
                           int64_t Nin, int C, int K, pmesh_stream_t stream);
int pmesh_point_unpool_bwd(const float *grad_output, const float *weight, const int32_t *rowptr_in, const int32_t *order_in,
                           float *grad_input, int64_t Nrows, int64_t Nin, int C, int K, pmesh_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PICASSO_MESH_H */
