"""Differentiable mesh unpooling: API of picasso/mesh/pi_modules/unpool3d.py (interpolate :21)."""
from . import mesh_unpool3d as module
from ._autograd import native_op

InterpolateFunction = native_op("InterpolateFunction", module.forward, module.backward, n_inputs=3, n_grads=1)


def interpolate(input, vt_replace, vt_map):
    """Fine-vertex features (NvFine, C) copied from the coarse row of each vertex's cluster.

    input (NvCoarse, C) float32;  vt_replace, vt_map (NvFine,) int32 decimation cluster maps
    """
    return InterpolateFunction.apply(input, vt_replace, vt_map)
