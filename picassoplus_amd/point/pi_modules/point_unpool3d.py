"""Native weighted unpooling: counterpart of the reference's ``point_unpool3d`` extension
(pcloud_unpool3d.cpp:87-88)."""
import torch

from ... import _lib
from ...mesh import topology
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of


def _dims(input, weight, nn_index):
    check_input(input, "input", 2, F32)
    check_input(weight, "weight", 2, F32)
    check_input(nn_index, "nn_index", 2, I32)
    if tuple(weight.shape) != tuple(nn_index.shape):
        raise RuntimeError("weight and nn_index must have the same shape (Nout, K)")
    return nn_index.shape[0], input.shape[0], input.shape[1], nn_index.shape[1], same_device(input, weight, nn_index)


def forward(input, weight, nn_index):
    """pcloud_unpool3d.cpp:20-52: input (Mp,C) coarse features, weight / nn_index (Np,K) -> output (Np,C)."""
    rows, n_in, C, K, dev = _dims(input, weight, nn_index)
    with torch.cuda.device(dev):
        out = torch.empty((rows, C), dtype=F32, device=dev)
        _lib.call("pmesh_point_unpool_fwd", input.data_ptr(), weight.data_ptr(), nn_index.data_ptr(), out.data_ptr(), rows,
                  n_in, C, K, stream_of(input))
    return out


def backward(grad_output, input, weight, nn_index):
    """pcloud_unpool3d.cpp:54-83 -> grad_input (Mp,C)."""
    rows, n_in, C, K, dev = _dims(input, weight, nn_index)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (rows, C):
        raise RuntimeError("grad_output must have shape (Np, C)")
    rowptr, order = topology.index_csr(nn_index, None, n_in)
    with torch.cuda.device(dev):
        gin = torch.empty((n_in, C), dtype=F32, device=dev)
        _lib.call("pmesh_point_unpool_bwd", grad_output.data_ptr(), weight.data_ptr(), rowptr.data_ptr(), order.data_ptr(),
                  gin.data_ptr(), rows, n_in, C, K, stream_of(input))
    return gin
