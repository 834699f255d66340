"""Native point convolutions: counterpart of the reference's ``point_conv3d`` extension
(pcloud_conv3d.cpp:220-223), same four functions.  The pairs' adjacency (sorted by query for the forward, by database
point for the input gradient) is built once per ``nn_index`` tensor and cached."""
import torch

from ... import _lib
from ...mesh import topology
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of, workspace


def _dims(input, filter, nn_count, nn_index, bin_index, bin_coeff):
    check_input(input, "input", 2, F32)
    check_input(filter, "filter", 3, F32)
    check_input(nn_count, "nn_count", 1, I32)
    check_input(nn_index, "nn_index", 2, I32)
    fuzzy = bin_coeff is not None
    check_input(bin_index, "bin_index", 2 if fuzzy else 1, I32)
    if fuzzy:
        check_input(bin_coeff, "bin_coeff", 2, F32)
        if tuple(bin_coeff.shape) != tuple(bin_index.shape):
            raise RuntimeError("bin_index and bin_coeff must have the same shape")
    Np, C = input.shape
    F, Cf, r = filter.shape
    if Cf != C:
        raise RuntimeError("Input Channel size error of the filter")
    if nn_index.shape[1] != 2:
        raise RuntimeError("nn_index must have shape (Nout, 2)")
    Nout = nn_index.shape[0]
    if bin_index.shape[0] != Nout:
        raise RuntimeError("bin_index must have one row per neighbour pair")
    T = bin_index.shape[1] if fuzzy else 1
    dev = same_device(input, filter, nn_count, nn_index, bin_index, *([bin_coeff] if fuzzy else []))
    return Np, nn_count.shape[0], Nout, F, C, r, T, dev


def _forward(input, filter, nn_count, nn_index, bin_index, bin_coeff):
    Np, Mp, Nout, F, C, r, T, dev = _dims(input, filter, nn_count, nn_index, bin_index, bin_coeff)
    rowptr, order = topology.index_csr(nn_index, 0, Mp)
    with torch.cuda.device(dev):
        out = torch.empty((Mp, C * r), dtype=F32, device=dev)
        _lib.call("pmesh_point_conv_fwd", input.data_ptr(), filter.data_ptr(), nn_count.data_ptr(), nn_index.data_ptr(),
                  bin_index.data_ptr(), bin_coeff.data_ptr() if bin_coeff is not None else None, rowptr.data_ptr(),
                  order.data_ptr(), out.data_ptr(), Np, Mp, Nout, F, C, r, T, stream_of(input))
    return out


def _backward(grad_output, input, filter, nn_count, nn_index, bin_index, bin_coeff):
    Np, Mp, Nout, F, C, r, T, dev = _dims(input, filter, nn_count, nn_index, bin_index, bin_coeff)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (Mp, C * r):
        raise RuntimeError("grad_output must have shape (Mp, C*r)")
    rowptr, order = topology.index_csr(nn_index, 1, Np)
    with torch.cuda.device(dev):
        gin = torch.empty((Np, C), dtype=F32, device=dev)
        gfilt = torch.empty((F, C, r), dtype=F32, device=dev)
        nbytes = _lib.query("pmesh_point_conv_bwd_workspace_bytes", Nout, F, C, r)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_point_conv_bwd", grad_output.data_ptr(), input.data_ptr(), filter.data_ptr(), nn_count.data_ptr(),
                  nn_index.data_ptr(), bin_index.data_ptr(), bin_coeff.data_ptr() if bin_coeff is not None else None,
                  rowptr.data_ptr(), order.data_ptr(), gin.data_ptr(), gfilt.data_ptr(), ws.data_ptr(), nbytes, Np, Mp, Nout,
                  F, C, r, T, stream_of(input))
    return [gin, gfilt]


def SPH3D_forward(input, filter, nn_count, nn_index, bin_index):
    """pcloud_conv3d.cpp:29-72 -> output (Mp, C*r)."""
    return _forward(input, filter, nn_count, nn_index, bin_index, None)


def SPH3D_backward(grad_output, input, filter, nn_count, nn_index, bin_index):
    """pcloud_conv3d.cpp:74-118 -> [grad_input (Np,C), grad_filter (F,C,r)]."""
    return _backward(grad_output, input, filter, nn_count, nn_index, bin_index, None)


def fuzzySPH3D_forward(input, filter, nn_count, nn_index, bin_index, bin_coeff):
    """pcloud_conv3d.cpp:120-167."""
    return _forward(input, filter, nn_count, nn_index, bin_index, bin_coeff)


def fuzzySPH3D_backward(grad_output, input, filter, nn_count, nn_index, bin_index, bin_coeff):
    """pcloud_conv3d.cpp:169-217."""
    return _backward(grad_output, input, filter, nn_count, nn_index, bin_index, bin_coeff)
