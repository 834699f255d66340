"""Differentiable mesh pooling: API of picasso/mesh/pi_modules/pool3d.py (maxPool :23, avgPool :43)."""
from . import mesh_pool3d as module
from ._autograd import native_op

# The reference keeps (input, max_index) for the max-pool backward (pool3d.py:13); the two cluster maps
# ride along so that backward can gather per fine vertex instead of zero-filling and scattering.
MaxPoolFunction = native_op("MaxPoolFunction", module.max_forward, module.max_backward, n_inputs=4, n_grads=1,
                            keep=lambda inputs, extras: (inputs[0], extras[0], inputs[1], inputs[2]))
AvgPoolFunction = native_op("AvgPoolFunction", module.avg_forward, module.avg_backward, n_inputs=4, n_grads=1,
                            keep=lambda inputs, extras: inputs[:3])


def maxPool(input, vt_replace, vt_map, vt_out):
    """Per-channel maximum over the fine vertices of every decimation cluster.

    input (NvFine, C) float32;  vt_replace, vt_map (NvFine,) int32;  vt_out (NvCoarse, .) gives the
    number of coarse vertices.  Returns (NvCoarse, C); ties keep the smallest vertex id.
    """
    return MaxPoolFunction.apply(input, vt_replace, vt_map, vt_out)


def avgPool(input, vt_replace, vt_map, vt_out):
    """Per-channel mean over the fine vertices of every decimation cluster; arguments as ``maxPool``."""
    return AvgPoolFunction.apply(input, vt_replace, vt_map, vt_out)
