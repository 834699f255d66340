"""Native farthest point sampling: counterpart of the reference's ``point_sample`` extension (sample.cpp:53)."""
import torch

from ... import _lib
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of


def fps(xyz_in, nv_in, nv_out):
    """sample.cpp:20-50: ``nv_in`` / ``nv_out`` inclusive running totals per sample -> index_out (Mp) int32."""
    check_input(xyz_in, "xyz_in", 2, F32)
    check_input(nv_in, "nv_in", 1, I32)
    check_input(nv_out, "nv_out", 1, I32)
    if xyz_in.shape[1] != 3:
        raise RuntimeError("FarthestPointSample expects (Np,3) inp shape")
    if nv_in.shape[0] != nv_out.shape[0]:
        raise RuntimeError("nv_in and nv_out must have one entry per sample")
    dev = same_device(xyz_in, nv_in, nv_out)
    B, Np = nv_in.shape[0], xyz_in.shape[0]
    Mp = int(nv_out[-1]) if B else 0
    with torch.cuda.device(dev):
        temp = torch.empty(max(Np, 1), dtype=F32, device=dev)
        index_out = torch.zeros(Mp, dtype=I32, device=dev)
        _lib.call("pmesh_point_fps", xyz_in.data_ptr(), nv_in.data_ptr(), nv_out.data_ptr(), B, Np, Mp, temp.data_ptr(),
                  index_out.data_ptr(), stream_of(xyz_in))
    return index_out
