"""Differentiable point pooling: API of picasso/point/pi_modules/pool3d.py (maxPool :24, avgPool :43)."""
from ...mesh.pi_modules._autograd import native_op
from . import point_pool3d as module

# The reference keeps (input, max_index) for the max-pool backward (pool3d.py:12); the pair list rides along so that
# backward can gather per database point.
MaxPoolFunction = native_op("MaxPoolFunction", module.max_forward, module.max_backward, n_inputs=3, n_grads=1,
                            keep=lambda inputs, extras: (inputs[0], extras[0], inputs[2]))
AvgPoolFunction = native_op("AvgPoolFunction", module.avg_forward, module.avg_backward, n_inputs=3, n_grads=1)


def maxPool(input, nn_count, nn_index):
    """Per-channel maximum of input (Np,C) over the neighbours of every query -> (Mp,C)."""
    return MaxPoolFunction.apply(input, nn_count, nn_index)


def avgPool(input, nn_count, nn_index):
    """Per-channel mean over the neighbours of every query."""
    return AvgPoolFunction.apply(input, nn_count, nn_index)
