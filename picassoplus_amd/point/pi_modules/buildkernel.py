"""Kernel bins of neighbour pairs: API of picasso/point/pi_modules/buildkernel.py (SPH3Dkernel_ :5,
fuzzySPH3Dkernel_ :27)."""
from . import point_buildkernel as module


def SPH3Dkernel_(database, query, nn_index, nn_dist, radius, kernel=[8, 2, 3]):
    """-> filt_index (Nout,) int32: bin of each pair in a spherical kernel of kernel = [azimuth, elevation, radial]
    divisions; bin 0 is the centre."""
    return module.SPH3D(database[:, :3].contiguous(), query[:, :3].contiguous(), nn_index, nn_dist, radius, *kernel)


def fuzzySPH3Dkernel_(database, query, nn_index, nn_dist, radius, kernel=[8, 4, 1]):
    """-> (filt_index (Nout,3) int32, filt_coeff (Nout,3) float32): centre bin, own bin and the neighbouring elevation
    bin with weights that sum to one; kernel size = prod(kernel) + 1."""
    return module.fuzzySPH3D(database[:, :3].contiguous(), query[:, :3].contiguous(), nn_index, nn_dist, radius, *kernel)
