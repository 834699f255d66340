"""Native kernel-bin builders: counterpart of the reference's ``point_buildkernel`` extension
(buildkernel.cpp:120-121)."""
import torch

from ... import _lib
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of


def _dims(database, query, nn_index, nn_dist, radius, n_azim, p_elev, q_radi):
    check_input(database, "database", 2, F32)
    check_input(query, "query", 2, F32)
    check_input(nn_index, "nn_index", 2, I32)
    check_input(nn_dist, "nn_dist", 1, F32)
    if not radius > 0:
        raise RuntimeError("Range search requires radius>0")
    if not (n_azim > 2 and n_azim % 2 == 0):
        raise RuntimeError("Need n_azim>2 and n_azim%2==0")
    if not (p_elev > 0 and p_elev % 2 == 0):
        raise RuntimeError("Need p_elev>0 and p_elev%2==0")
    if not q_radi > 0:
        raise RuntimeError("Need q_radi>0")
    if database.shape[1] != 3 or query.shape[1] != 3:
        raise RuntimeError("Shape of database and query points requires to be (N, 3)")
    if nn_index.shape[1] != 2 or nn_dist.shape[0] != nn_index.shape[0]:
        raise RuntimeError("Shape of nn_index requires to be (Nout, 2), of nn_dist (Nout)")
    return same_device(database, query, nn_index, nn_dist)


def SPH3D(database, query, nn_index, nn_dist, radius, n_azim, p_elev, q_radi):
    """buildkernel.cpp:22-70 -> filt_index (Nout) int32."""
    dev = _dims(database, query, nn_index, nn_dist, radius, n_azim, p_elev, q_radi)
    with torch.cuda.device(dev):
        filt_index = torch.empty(nn_index.shape[0], dtype=I32, device=dev)
        _lib.call("pmesh_point_sph3d_kernel", database.data_ptr(), query.data_ptr(), nn_index.data_ptr(), nn_dist.data_ptr(),
                  nn_index.shape[0], database.shape[0], query.shape[0], int(n_azim), int(p_elev), int(q_radi), float(radius),
                  filt_index.data_ptr(), stream_of(database))
    return filt_index


def fuzzySPH3D(database, query, nn_index, nn_dist, radius, n_azim, p_elev, q_radi):
    """buildkernel.cpp:73-117 -> (filt_index (Nout,3) int32, filt_coeff (Nout,3))."""
    dev = _dims(database, query, nn_index, nn_dist, radius, n_azim, p_elev, q_radi)
    with torch.cuda.device(dev):
        filt_index = torch.empty((nn_index.shape[0], 3), dtype=I32, device=dev)
        filt_coeff = torch.empty((nn_index.shape[0], 3), dtype=F32, device=dev)
        _lib.call("pmesh_point_fuzzy_sph3d_kernel", database.data_ptr(), query.data_ptr(), nn_index.data_ptr(),
                  nn_dist.data_ptr(), nn_index.shape[0], database.shape[0], query.shape[0], int(n_azim), int(p_elev),
                  int(q_radi), float(radius), filt_index.data_ptr(), filt_coeff.data_ptr(), stream_of(database))
    return filt_index, filt_coeff
