"""Native mesh unpooling ops: counterpart of the reference's ``mesh_unpool3d`` extension
(picasso/mesh/pi_modules/source/mesh_unpool3d.cpp:81-85), same two functions."""
import torch

from ... import _lib
from .. import topology
from ._check import F32, I32, check_input, same_device, stream_of


def _dims(input, vt_replace, vt_map):
    check_input(input, "input", 2, F32)
    check_input(vt_replace, "vt_replace", 1, I32)
    check_input(vt_map, "vt_map", 1, I32)
    if vt_replace.shape[0] != vt_map.shape[0]:
        raise RuntimeError("vt_replace and vt_map must have the same length")
    return input.shape[0], input.shape[1], vt_map.shape[0]


def forward(input, vt_replace, vt_map):
    """mesh_unpool3d.cpp:20-47: (NvCoarse,C) -> (NvFine,C), NvFine = len(vt_map)."""
    NvCoarse, C, NvFine = _dims(input, vt_replace, vt_map)
    dev = same_device(input, vt_replace, vt_map)
    topology._check_cluster_cached(vt_replace, vt_map)
    with torch.cuda.device(dev):
        out = torch.empty((NvFine, C), dtype=F32, device=dev)
        _lib.call("pmesh_unpool_fwd", input.data_ptr(), vt_replace.data_ptr(), vt_map.data_ptr(), out.data_ptr(),
                  NvCoarse, NvFine, C, stream_of(input))
    return out


def backward(grad_output, input, vt_replace, vt_map):
    """mesh_unpool3d.cpp:48-78 -> grad_input (NvCoarse,C)."""
    NvCoarse, C, NvFine = _dims(input, vt_replace, vt_map)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (NvFine, C):
        raise RuntimeError("grad_output must have shape (NvFine, C)")
    dev = same_device(grad_output, input, vt_replace, vt_map)
    rowptr, members = topology.cluster_csr(vt_replace, vt_map, NvCoarse)
    with torch.cuda.device(dev):
        gin = torch.empty((NvCoarse, C), dtype=F32, device=dev)
        _lib.call("pmesh_unpool_bwd", grad_output.data_ptr(), rowptr.data_ptr(), members.data_ptr(),
                  gin.data_ptr(), NvCoarse, NvFine, C, stream_of(input))
    return gin
