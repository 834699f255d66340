"""Native mesh convolution ops: counterpart of the reference's ``mesh_conv3d`` extension.

Same six functions, argument order and result shapes as the pybind module defined in
picasso/mesh/pi_modules/source/mesh_conv3d.cpp:272-279; the arithmetic runs in
libpicasso_mesh.so (HIP, gfx950) through the C ABI of include/picasso_mesh.h.
"""
import os

import torch

from ... import _lib
from .. import topology
from ._check import BF16, F32, I32, check_input, feature_dtype, same_device, stream_of, workspace


# ---------------------------------------------------------------- vertex2facet
def _v2f_dims(input, filter, face):
    check_input(input, "input", 2, F32)
    check_input(filter, "filter", 3, F32)
    check_input(face, "face", 2, I32)
    C, r = input.shape[1], filter.shape[2]
    if filter.shape[0] != 3 or filter.shape[1] != C:
        raise RuntimeError("3 filters required, or input Channel size error of the filter")
    if face.shape[1] != 3:
        raise RuntimeError("face must have shape (NfIn, 3)")
    return input.shape[0], face.shape[0], C, r


def vertex2facet_forward(input, filter, face):
    """mesh_conv3d.cpp:123-152: (NvIn,C),(3,C,r),(NfIn,3) -> (NfIn,C*r)."""
    Nv, Nf, C, r = _v2f_dims(input, filter, face)
    dev = same_device(input, filter, face)
    if Nf:
        topology._check_range_cached(face, Nv)       # an empty input with facets raises: every index is out of range
    with torch.cuda.device(dev):
        out = torch.empty((Nf, C * r), dtype=F32, device=dev)
        _lib.call("pmesh_v2f_fwd", input.data_ptr(), filter.data_ptr(), face.data_ptr(), out.data_ptr(),
                  Nv, Nf, C, r, stream_of(input))
    return out


def vertex2facet_backward(grad_output, input, filter, face):
    """mesh_conv3d.cpp:153-188 -> [grad_input (NvIn,C), grad_filter (3,C,r)]."""
    Nv, Nf, C, r = _v2f_dims(input, filter, face)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (Nf, C * r):
        raise RuntimeError("grad_output must have shape (NfIn, C*r)")
    dev = same_device(grad_output, input, filter, face)
    rowptr, colidx = topology.vertex_csr(face, None, Nv)
    with torch.cuda.device(dev):
        gin = torch.empty((Nv, C), dtype=F32, device=dev)
        gfilt = torch.empty((3, C, r), dtype=F32, device=dev)
        nbytes = _lib.query("pmesh_v2f_bwd_workspace_bytes", C, r)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_v2f_bwd", grad_output.data_ptr(), input.data_ptr(), filter.data_ptr(), face.data_ptr(),
                  rowptr.data_ptr(), colidx.data_ptr(), gin.data_ptr(), gfilt.data_ptr(), ws.data_ptr(), nbytes,
                  Nv, Nf, C, r, stream_of(input))
    return [gin, gfilt]


# ---------------------------------------------------------------- facet2vertex
def _f2v_dims(input, filter, coeff, face, nf_count, vt_map):
    check_input(input, "input", 2, feature_dtype(input, "input"))
    check_input(filter, "filter", 3, F32)
    check_input(coeff, "coeff", 2, F32)
    check_input(face, "face", 2, I32)
    check_input(nf_count, "nf_count", 1, I32)
    check_input(vt_map, "vt_map", 1, I32)
    Nf, C = input.shape
    K, r = filter.shape[0], filter.shape[2]
    if filter.shape[1] != C:
        raise RuntimeError("Input Channel size error of the filter")
    if tuple(coeff.shape) != (Nf, K):
        raise RuntimeError("coeff must have shape (NfIn, filter_size)")
    if tuple(face.shape) != (Nf, 3):
        raise RuntimeError("face must have shape (NfIn, 3)")
    return Nf, C, K, r, nf_count.shape[0], vt_map.shape[0]


def _f2v_blocks_of_16(input, filter, coeff):
    """The matrix-core kernels of facet2vertex take 16 coefficients.  From 9 coefficients on, any other count runs as
    ceil(K / 16) such convolutions over zero-padded blocks (the output is linear in the pair filter x coefficients)
    instead of on the vector-ALU kernels, whose cost grows with K.  Returns [(filter block (16,C,r), coefficient block
    (Nf,16))], or None where the native call takes the operands as they are."""
    K, C, r = filter.shape
    if K == 16 or K < 9 or C * r < 32 or input.dtype != F32 or os.environ.get("PMESH_F2V_VALU") == "1":
        return None
    n = (K + 15) // 16
    pad = torch.nn.functional.pad
    cblocks = topology.coefficient_blocks(coeff)                      # (cut once per coefficient tensor, not per call)
    blocks = []
    for j in range(n):
        if 16 * j + 16 <= K:
            blocks.append((filter[16 * j:16 * j + 16].contiguous(), cblocks[j]))
        else:                                                        # (only the last block is padded)
            blocks.append((pad(filter[16 * j:], (0, 0, 0, 0, 0, 16 * j + 16 - K)), cblocks[j]))
    return blocks


def facet2vertex_forward(input, filter, coeff, face, nf_count, vt_map):
    """mesh_conv3d.cpp:33-74 -> (NvOut, C*r).  ``input`` may be bfloat16 (features in bf16 in HBM: the output is
    bfloat16 too, filter and coefficients stay float32)."""
    Nf, C, K, r, NvOut, NvIn = _f2v_dims(input, filter, coeff, face, nf_count, vt_map)
    dev = same_device(input, filter, coeff, face, nf_count, vt_map)
    blocks = _f2v_blocks_of_16(input, filter, coeff)
    if blocks is not None:
        out = None
        for fb, cb in blocks:
            part = facet2vertex_forward(input, fb, cb, face, nf_count, vt_map)
            out = part if out is None else out.add_(part)
        return out
    rowptr, colidx = topology.vertex_csr(face, vt_map, NvOut)
    with torch.cuda.device(dev):
        out = torch.empty((NvOut, C * r), dtype=input.dtype, device=dev)
        _lib.call("pmesh_f2v_fwd_bf16" if input.dtype == BF16 else "pmesh_f2v_fwd", input.data_ptr(), filter.data_ptr(),
                  coeff.data_ptr(), nf_count.data_ptr(), rowptr.data_ptr(), colidx.data_ptr(), out.data_ptr(), Nf, NvOut,
                  C, r, K, stream_of(input))
    return out


def facet2vertex_backward(grad_output, input, filter, coeff, face, nf_count, vt_map):
    """mesh_conv3d.cpp:75-122 -> [grad_input (NfIn,C), grad_filter (K,C,r)]; bfloat16 features give a bfloat16
    grad_input and a float32 grad_filter."""
    Nf, C, K, r, NvOut, NvIn = _f2v_dims(input, filter, coeff, face, nf_count, vt_map)
    check_input(grad_output, "grad_output", 2, input.dtype)
    if tuple(grad_output.shape) != (NvOut, C * r):
        raise RuntimeError("grad_output must have shape (NvOut, C*r)")
    dev = same_device(grad_output, input, filter, coeff, face, nf_count, vt_map)
    blocks = _f2v_blocks_of_16(input, filter, coeff)
    if blocks is not None:
        gin, parts = None, []
        for fb, cb in blocks:
            g_in, g_f = facet2vertex_backward(grad_output, input, fb, cb, face, nf_count, vt_map)
            gin = g_in if gin is None else gin.add_(g_in)
            parts.append(g_f)
        return [gin, torch.cat(parts, 0)[:K].contiguous()]
    if Nf:
        topology._check_range_cached(face, NvIn)
    with torch.cuda.device(dev):
        gin = torch.empty((Nf, C), dtype=input.dtype, device=dev)
        gfilt = torch.empty((K, C, r), dtype=F32, device=dev)
        nbytes = _lib.query("pmesh_f2v_bwd_workspace_bytes", C, r, K)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_f2v_bwd_bf16" if input.dtype == BF16 else "pmesh_f2v_bwd", grad_output.data_ptr(), input.data_ptr(),
                  filter.data_ptr(), coeff.data_ptr(), face.data_ptr(), nf_count.data_ptr(), vt_map.data_ptr(),
                  gin.data_ptr(), gfilt.data_ptr(), ws.data_ptr(), nbytes, Nf, NvIn, NvOut, C, r, K, stream_of(input))
    return [gin, gfilt]


# ---------------------------------------------------------------- facet2facet
def _f2f_dims(input, filter, bary_coeff, num_texture, forward):
    check_input(input, "input", 2, feature_dtype(input, "input"))
    check_input(filter, "filter", 3, F32)
    check_input(bary_coeff, "bary_coeff", 2, F32)
    check_input(num_texture, "num_texture", 1, I32)
    T, Cin = input.shape
    Cout, _, F = filter.shape
    if filter.shape[1] != Cin:
        raise RuntimeError("input Channel size error of the filter.")
    if F > 50:
        raise RuntimeError("A maximum of 50 filters are supported in face2face convolution.")
    if bary_coeff.shape[1] != F:
        raise RuntimeError("Dimension of bary_coeff mismatches number of filters.")
    if bary_coeff.shape[0] != T:
        raise RuntimeError("The shape of bary_coeff should be (NiK, Dim)).")
    return T, Cin, Cout, F, num_texture.shape[0]


def _blocks_of_16(input, filter, bary_coeff):
    """The matrix-core kernels take 16 coefficients (degree 3).  Any other count is run as ceil(F / 16) such
    convolutions: the filter and the coefficient rows are padded with zeros to a multiple of 16 and cut into blocks,
    and ``G . W^T`` is the sum over the blocks (the convolution is linear in the pair).  Returns the list of
    (filter block (Cout,Cin,16), coefficient block (T,16)), or None where the native call takes the operands as they are
    (16 coefficients; bfloat16 features, whose block sums would be rounded once more; the shape-generic kernels asked
    for by PMESH_F2F_GENERIC=1)."""
    F = filter.shape[2]
    if F == 16 or input.dtype != F32 or os.environ.get("PMESH_F2F_GENERIC") == "1":
        return None
    n = (F + 15) // 16
    pad = torch.nn.functional.pad
    cut = lambda t, j: (t[..., 16 * j:16 * j + 16].contiguous() if 16 * j + 16 <= F        # (only the last block is padded)
                        else pad(t[..., 16 * j:], (0, 16 * j + 16 - F)))
    cblocks = topology.coefficient_blocks(bary_coeff)                 # (cut once per coefficient tensor, not per call)
    return [(cut(filter, j), cblocks[j]) for j in range(n)]


def facet2facet_forward(input, filter, bary_coeff, num_texture):
    """mesh_conv3d.cpp:192-228; ``num_texture`` is the inclusive running total per facet.  ``input`` may be bfloat16
    (features in bf16 in HBM: bfloat16 output, float32 filter and coefficients, one fp16 product per element)."""
    T, Cin, Cout, F, Nf = _f2f_dims(input, filter, bary_coeff, num_texture, True)
    dev = same_device(input, filter, bary_coeff, num_texture)
    blocks = _blocks_of_16(input, filter, bary_coeff)
    if blocks is not None:
        out = None
        for fb, bb in blocks:
            part = facet2facet_forward(input, fb, bb, num_texture)
            out = part if out is None else out.add_(part)
        return out
    with torch.cuda.device(dev):
        out = torch.empty((Nf, Cout), dtype=input.dtype, device=dev)
        nbytes = _lib.query("pmesh_f2f_fwd_workspace_bytes", Cin, Cout, F)
        ws = workspace(nbytes, dev)
        order = topology.facet_order(num_texture, T) if Nf else None
        _lib.call("pmesh_f2f_fwd_bf16" if input.dtype == BF16 else "pmesh_f2f_fwd", input.data_ptr(), filter.data_ptr(),
                  bary_coeff.data_ptr(), num_texture.data_ptr(), order.data_ptr() if order is not None else None,
                  out.data_ptr(), ws.data_ptr(), nbytes, T, Nf, Cin, Cout, F, stream_of(input))
    return out


def facet2facet_forward_act(input, filter, bary_coeff, num_texture, bias=None, relu=True, scale=None, shift=None,
                            with_bits=False):
    """facet2facet_forward with the module's tail on the store (picasso/mesh/layers.py:59-63):
    act(conv + bias) * scale + shift, float32 features; ``bias`` / ``scale`` / ``shift`` (Cout,) float32 or None.
    ``with_bits`` (Cout % 32 == 0) also returns the ReLU mask as bits, int32 (Nf, Cout / 32)."""
    T, Cin, Cout, F, Nf = _f2f_dims(input, filter, bary_coeff, num_texture, True)
    if input.dtype != F32:
        raise RuntimeError("the fused tail takes float32 features")
    for name, t in (("bias", bias), ("scale", scale), ("shift", shift)):
        if t is not None:
            check_input(t, name, 1, F32)
            if t.shape[0] != Cout:
                raise RuntimeError("%s must have one entry per output channel" % name)
    if with_bits and Cout % 32:
        raise RuntimeError("the bit mask needs a multiple of 32 output channels")
    dev = same_device(input, filter, bary_coeff, num_texture, *[t for t in (bias, scale, shift) if t is not None])
    if _blocks_of_16(input, filter, bary_coeff) is not None:
        # other coefficient counts: the sum over the blocks of 16 first, the tail as one pass over it
        from . import dense
        conv = facet2facet_forward(input, filter, bary_coeff, num_texture)
        return dense.bias_act_forward(conv, bias, relu, scale, shift, with_bits=with_bits)
    with torch.cuda.device(dev):
        out = torch.empty((Nf, Cout), dtype=F32, device=dev)
        bits = torch.empty((Nf, Cout // 32), dtype=torch.int32, device=dev) if with_bits else None
        nbytes = _lib.query("pmesh_f2f_fwd_workspace_bytes", Cin, Cout, F)
        ws = workspace(nbytes, dev)
        order = topology.facet_order(num_texture, T) if Nf else None
        ptr = lambda t: t.data_ptr() if t is not None else None
        _lib.call("pmesh_f2f_fwd_act", input.data_ptr(), filter.data_ptr(), bary_coeff.data_ptr(), num_texture.data_ptr(),
                  ptr(order), ptr(bias), ptr(scale), ptr(shift), 1 if relu else 0, out.data_ptr(), ptr(bits), ws.data_ptr(),
                  nbytes, T, Nf, Cin, Cout, F, stream_of(input))
    return (out, bits) if with_bits else out


def facet2facet_backward(grad_output, input, filter, bary_coeff, num_texture):
    """mesh_conv3d.cpp:229-269 -> [grad_input (NiK,Cin), grad_filter (Cout,Cin,F)]."""
    return facet2facet_backward_selected(grad_output, input, filter, bary_coeff, num_texture, needs=(True, True))


def facet2facet_backward_selected(grad_output, input, filter, bary_coeff, num_texture, needs):
    """facet2facet_backward with ``needs`` = (texture gradient wanted, filter gradient wanted): an unwanted
    gradient is not computed and comes back as None (no counterpart in the reference, which always
    computes both)."""
    T, Cin, Cout, F, Nf = _f2f_dims(input, filter, bary_coeff, num_texture, False)
    check_input(grad_output, "grad_output", 2, input.dtype)
    if tuple(grad_output.shape) != (Nf, Cout):
        raise RuntimeError("grad_output must have shape (NfIn, Cout)")
    dev = same_device(grad_output, input, filter, bary_coeff, num_texture)
    blocks = _blocks_of_16(input, filter, bary_coeff)
    if blocks is not None:
        # the texture gradient is the sum over the blocks, the filter gradient their concatenation
        gin, parts = None, []
        for fb, bb in blocks:
            if needs[0] and gin is not None and _lib.query("pmesh_f2f_bwd_texture_onto_supported", grad_output.data_ptr(),
                                                           fb.data_ptr(), bb.data_ptr(), Cout, 16):
                # the later blocks add their texture gradient onto the first one's in place
                with torch.cuda.device(dev):
                    nbytes = _lib.query("pmesh_f2f_bwd_workspace_bytes_for", Nf, Cin, Cout, 16)
                    ws = workspace(nbytes, dev)
                    order = topology.facet_order(num_texture, T) if Nf else None
                    _lib.call("pmesh_f2f_bwd_texture_onto", grad_output.data_ptr(), fb.data_ptr(), bb.data_ptr(),
                              num_texture.data_ptr(), order.data_ptr() if order is not None else None, gin.data_ptr(),
                              ws.data_ptr(), nbytes, T, Nf, Cin, Cout, 16, stream_of(input))
                g_f = facet2facet_backward_selected(grad_output, input, fb, bb, num_texture, (False, needs[1]))[1]
            else:
                g_in, g_f = facet2facet_backward_selected(grad_output, input, fb, bb, num_texture, needs)
                if needs[0]:
                    gin = g_in if gin is None else gin.add_(g_in)
            parts.append(g_f)
        return [gin, torch.cat(parts, 2)[:, :, :F].contiguous() if needs[1] else None]
    sfx = "_bf16" if input.dtype == BF16 else ""
    with torch.cuda.device(dev):
        gin = torch.empty((T, Cin), dtype=input.dtype, device=dev) if needs[0] else None
        gfilt = torch.empty((Cout, Cin, F), dtype=F32, device=dev) if needs[1] else None
        nbytes = (_lib.query("pmesh_f2f_bwd_bf16_workspace_bytes", T, Nf, Cin, Cout, F) if sfx
                  else _lib.query("pmesh_f2f_bwd_workspace_bytes_for", Nf, Cin, Cout, F))
        ws = workspace(nbytes, dev)
        st = stream_of(input)
        order = topology.facet_order(num_texture, T) if Nf else None
        order_ptr = order.data_ptr() if order is not None else None
        if needs[0]:
            _lib.call("pmesh_f2f_bwd_texture" + sfx, grad_output.data_ptr(), filter.data_ptr(), bary_coeff.data_ptr(),
                      num_texture.data_ptr(), order_ptr, gin.data_ptr(), ws.data_ptr(), nbytes, T, Nf, Cin, Cout, F, st)
        if needs[1]:
            _lib.call("pmesh_f2f_bwd_filter" + sfx, grad_output.data_ptr(), input.data_ptr(), bary_coeff.data_ptr(),
                      num_texture.data_ptr(), order_ptr, gfilt.data_ptr(), ws.data_ptr(), nbytes, T, Nf, Cin, Cout, F, st)
    return [gin, gfilt]
