"""Native point pooling: counterpart of the reference's ``point_pool3d`` extension (pcloud_pool3d.cpp:154-157)."""
import torch

from ... import _lib
from ...mesh import topology
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of


def _dims(input, nn_count, nn_index):
    check_input(input, "input", 2, F32)
    check_input(nn_count, "nn_count", 1, I32)
    check_input(nn_index, "nn_index", 2, I32)
    if nn_index.shape[1] != 2:
        raise RuntimeError("Shape of nn_index should be (Nout,2).")
    return input.shape[0], nn_count.shape[0], nn_index.shape[0], input.shape[1], same_device(input, nn_count, nn_index)


def max_forward(input, nn_count, nn_index):
    """pcloud_pool3d.cpp:23-57 -> [output (Mp,C), max_index (Mp,C) int32]; among equal values the first pair wins, a
    query without neighbours gives 0 and index -1."""
    Np, Mp, Nout, C, dev = _dims(input, nn_count, nn_index)
    rowptr, order = topology.index_csr(nn_index, 0, Mp)
    with torch.cuda.device(dev):
        out = torch.empty((Mp, C), dtype=F32, device=dev)
        idx = torch.empty((Mp, C), dtype=I32, device=dev)
        _lib.call("pmesh_point_pool_max_fwd", input.data_ptr(), nn_index.data_ptr(), rowptr.data_ptr(), order.data_ptr(),
                  out.data_ptr(), idx.data_ptr(), Np, Mp, Nout, C, stream_of(input))
    return [out, idx]


def max_backward(grad_output, input, max_index, nn_index=None):
    """pcloud_pool3d.cpp:59-86 -> grad_input (Np,C).  The gradient is gathered per database point over the pairs
    that name it, so the pair list the forward ran on is needed as a fourth argument (the reference scatters by
    ``max_index`` with float atomics and takes three)."""
    if nn_index is None:
        raise RuntimeError("max_backward gathers over the neighbour pairs: pass the nn_index of the forward")
    check_input(input, "input", 2, F32)
    check_input(grad_output, "grad_output", 2, F32)
    check_input(max_index, "max_index", 2, I32)
    check_input(nn_index, "nn_index", 2, I32)
    Np, C = input.shape
    Mp = grad_output.shape[0]
    if grad_output.shape[1] != C or tuple(max_index.shape) != (Mp, C):
        raise RuntimeError("grad_output and max_index must have shape (Mp, C)")
    dev = same_device(grad_output, input, max_index, nn_index)
    rowptr, order = topology.index_csr(nn_index, 1, Np)
    with torch.cuda.device(dev):
        gin = torch.empty((Np, C), dtype=F32, device=dev)
        _lib.call("pmesh_point_pool_max_bwd", grad_output.data_ptr(), max_index.data_ptr(), nn_index.data_ptr(),
                  rowptr.data_ptr(), order.data_ptr(), gin.data_ptr(), Np, Mp, nn_index.shape[0], C, stream_of(input))
    return gin


def avg_forward(input, nn_count, nn_index):
    """pcloud_pool3d.cpp:88-119 -> output (Mp,C)."""
    Np, Mp, Nout, C, dev = _dims(input, nn_count, nn_index)
    rowptr, order = topology.index_csr(nn_index, 0, Mp)
    with torch.cuda.device(dev):
        out = torch.empty((Mp, C), dtype=F32, device=dev)
        _lib.call("pmesh_point_pool_avg_fwd", input.data_ptr(), nn_count.data_ptr(), nn_index.data_ptr(), rowptr.data_ptr(),
                  order.data_ptr(), out.data_ptr(), Np, Mp, Nout, C, stream_of(input))
    return out


def avg_backward(grad_output, input, nn_count, nn_index):
    """pcloud_pool3d.cpp:121-151 -> grad_input (Np,C)."""
    Np, Mp, Nout, C, dev = _dims(input, nn_count, nn_index)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (Mp, C):
        raise RuntimeError("grad_output must have shape (Mp, C)")
    rowptr, order = topology.index_csr(nn_index, 1, Np)
    with torch.cuda.device(dev):
        gin = torch.empty((Np, C), dtype=F32, device=dev)
        _lib.call("pmesh_point_pool_avg_bwd", grad_output.data_ptr(), nn_count.data_ptr(), nn_index.data_ptr(),
                  rowptr.data_ptr(), order.data_ptr(), gin.data_ptr(), Np, Mp, Nout, C, stream_of(input))
    return gin
