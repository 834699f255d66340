"""Differentiable point convolutions: API of picasso/point/pi_modules/conv3d.py (conv3d :22, fuzzyconv3d :44).
Same arguments in the same order, the same tensors saved for backward, ``None`` gradients for the index and
coefficient inputs."""
from ...mesh.pi_modules._autograd import native_op
from . import point_conv3d as module

ConvFunction = native_op("ConvFunction", module.SPH3D_forward, module.SPH3D_backward, n_inputs=5, n_grads=2)
FuzzyConv3dFunction = native_op("FuzzyConv3dFunction", module.fuzzySPH3D_forward, module.fuzzySPH3D_backward, n_inputs=6,
                                n_grads=2)


def conv3d(input, filter, nn_count, nn_index, bin_index):
    """input (Np,C), filter (F,C,r), nn_count (Mp,) int32, nn_index (Nout,2) int32, bin_index (Nout,) int32
    -> (Mp, C*r): per query the mean over its neighbours of input * filter[bin of the pair]."""
    return ConvFunction.apply(input, filter, nn_count, nn_index, bin_index)


def fuzzyconv3d(input, filter, nn_count, nn_index, bin_index, bin_coeff):
    """As ``conv3d`` with T weighted bins per pair: bin_index (Nout,T) int32, bin_coeff (Nout,T) float32."""
    return FuzzyConv3dFunction.apply(input, filter, nn_count, nn_index, bin_index, bin_coeff)
