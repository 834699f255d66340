"""Differentiable weighted unpooling: API of picasso/point/pi_modules/unpool3d.py (interpolate :21)."""
from ...mesh.pi_modules._autograd import native_op
from . import point_unpool3d as module

InterpolateFunction = native_op("InterpolateFunction", module.forward, module.backward, n_inputs=3, n_grads=1)


def interpolate(input, weight, nn_index):
    """input (Mp,C) coarse features, weight / nn_index (Np,K): out[o] = sum_k input[nn_index[o,k]] * weight[o,k]."""
    return InterpolateFunction.apply(input, weight, nn_index)
