"""Native mesh pooling ops: counterpart of the reference's ``mesh_pool3d`` extension
(picasso/mesh/pi_modules/source/mesh_pool3d.cpp:151-157), same four functions."""
import torch

from ... import _lib
from .. import topology
from ._check import F32, I32, check_input, same_device, stream_of


def _pool_dims(input, vt_replace, vt_map, vt_out):
    check_input(input, "input", 2, F32)
    check_input(vt_replace, "vt_replace", 1, I32)
    check_input(vt_map, "vt_map", 1, I32)
    if vt_out is not None:
        if not isinstance(vt_out, torch.Tensor) or not vt_out.is_cuda:
            raise RuntimeError("vt_out must be a CUDA tensor")
        if not vt_out.is_contiguous():
            raise RuntimeError("vt_out must be contiguous")
        if vt_out.dim() != 2:
            raise RuntimeError("vt_out must have dimension of 2")
    if vt_replace.shape[0] != input.shape[0] or vt_map.shape[0] != input.shape[0]:
        raise RuntimeError("vt_replace and vt_map must have one entry per input vertex")
    return input.shape[0], input.shape[1]


def max_forward(input, vt_replace, vt_map, vt_out):
    """mesh_pool3d.cpp:29-60 -> [output (NvOut,C), max_index (NvOut,C) int32].
    ``vt_out`` only supplies the number of output vertices (mesh_pool3d.cpp:43)."""
    NvIn, C = _pool_dims(input, vt_replace, vt_map, vt_out)
    NvOut = vt_out.shape[0]
    dev = same_device(input, vt_replace, vt_map, vt_out)
    rowptr, members = topology.cluster_csr(vt_replace, vt_map, NvOut)
    with torch.cuda.device(dev):
        out = torch.empty((NvOut, C), dtype=F32, device=dev)
        idx = torch.empty((NvOut, C), dtype=I32, device=dev)
        _lib.call("pmesh_pool_max_fwd", input.data_ptr(), rowptr.data_ptr(), members.data_ptr(), out.data_ptr(),
                  idx.data_ptr(), NvIn, NvOut, C, stream_of(input))
    return [out, idx]


def max_backward(grad_output, input, max_index, vt_replace=None, vt_map=None):
    """mesh_pool3d.cpp:61-87 -> grad_input (NvIn,C).

    With the cluster maps supplied (and ``max_index`` produced by ``max_forward`` on them)
    the gradient is gathered per fine vertex in one pass; without them it is the reference's
    zero-fill plus scatter by ``max_index``."""
    check_input(input, "input", 2, F32)
    check_input(grad_output, "grad_output", 2, F32)
    check_input(max_index, "max_index", 2, I32)
    NvIn, C = input.shape
    NvOut = grad_output.shape[0]
    if grad_output.shape[1] != C or tuple(max_index.shape) != (NvOut, C):
        raise RuntimeError("grad_output and max_index must have shape (NvOut, C)")
    dev = same_device(grad_output, input, max_index)
    with torch.cuda.device(dev):
        gin = torch.empty((NvIn, C), dtype=F32, device=dev)
        _lib.call("pmesh_pool_max_bwd", grad_output.data_ptr(), max_index.data_ptr(),
                  vt_replace.data_ptr() if vt_replace is not None else None,
                  vt_map.data_ptr() if vt_map is not None else None,
                  gin.data_ptr(), NvIn, NvOut, C, stream_of(input))
    return gin


def avg_forward(input, vt_replace, vt_map, vt_out):
    """mesh_pool3d.cpp:89-118 -> output (NvOut,C)."""
    NvIn, C = _pool_dims(input, vt_replace, vt_map, vt_out)
    NvOut = vt_out.shape[0]
    dev = same_device(input, vt_replace, vt_map, vt_out)
    rowptr, members = topology.cluster_csr(vt_replace, vt_map, NvOut)
    with torch.cuda.device(dev):
        out = torch.empty((NvOut, C), dtype=F32, device=dev)
        _lib.call("pmesh_pool_avg_fwd", input.data_ptr(), vt_replace.data_ptr(), rowptr.data_ptr(),
                  members.data_ptr(), out.data_ptr(), NvIn, NvOut, C, stream_of(input))
    return out


def avg_backward(grad_output, input, vt_replace, vt_map):
    """mesh_pool3d.cpp:119-148 -> grad_input (NvIn,C)."""
    NvIn, C = _pool_dims(input, vt_replace, vt_map, None)
    check_input(grad_output, "grad_output", 2, F32)
    if grad_output.shape[1] != C:
        raise RuntimeError("grad_output must have C channels")
    NvOut = grad_output.shape[0]
    dev = same_device(grad_output, input, vt_replace, vt_map)
    topology._check_cluster_cached(vt_replace, vt_map)
    with torch.cuda.device(dev):
        gin = torch.empty((NvIn, C), dtype=F32, device=dev)
        _lib.call("pmesh_pool_avg_bwd", grad_output.data_ptr(), vt_replace.data_ptr(), vt_map.data_ptr(),
                  gin.data_ptr(), NvIn, NvOut, C, stream_of(input))
    return gin
