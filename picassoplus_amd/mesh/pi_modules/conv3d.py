"""Differentiable mesh convolutions: API of picasso/mesh/pi_modules/conv3d.py.

``vertex2facet``, ``facet2facet`` and ``facet2vertex`` take the same arguments in the same
order as the reference functions (conv3d.py:21,55,89), save the same tensors for backward
and return ``None`` gradients for index and coefficient inputs.  The feature and the filter
gradient of vertex2facet and facet2vertex come out of one native call, so both are always computed,
as in the reference; facet2facet has one native call per gradient and skips the one autograd does not
ask for (the texture gradient of a network's input colours, the largest single saving of a first block).
"""
import torch

from . import dense
from . import mesh_conv3d as module
from ._autograd import native_op

f2f_Function = native_op("f2f_Function", module.facet2facet_forward, module.facet2facet_backward_selected, n_inputs=4,
                         n_grads=2, selective=True)
v2f_Function = native_op("v2f_Function", module.vertex2facet_forward, module.vertex2facet_backward, n_inputs=3, n_grads=2)
f2v_Function = native_op("f2v_Function", module.facet2vertex_forward, module.facet2vertex_backward, n_inputs=6, n_grads=2)


def facet2facet(textureIn, filter, baryCoeff, numTexture):
    """Facet features from the features of texture points sampled inside each facet.

    textureIn  (T, Cin) float32, rows grouped by facet in facet order
    filter     (Cout, Cin, F) float32
    baryCoeff  (T, F) float32: spherical-harmonic values of each point's barycentric coordinates
    numTexture (Nf,) int32: inclusive running total of texture points per facet
    returns    (Nf, Cout) float32
    """
    return f2f_Function.apply(textureIn, filter, baryCoeff, numTexture)


def vertex2facet(input, filter, face):
    """Facet features as a filtered combination of the three corner features.

    input  (Nv, C) float32;  filter (3, C, r) float32;  face (Nf, 3) int32
    returns (Nf, C*r) float32
    """
    return v2f_Function.apply(input, filter, face)


def facet2vertex(input, filter, coeff, face, nfCount, vtMap):
    """Vertex features averaged over the incident facets, filtered per facet.

    input (Nf, C);  filter (K, C, r);  coeff (Nf, K);  face (Nf, 3) int32;
    nfCount (NvOut,) int32 divisor per output vertex;  vtMap (NvIn,) int32 input->output vertex
    returns (NvOut, C*r) float32
    """
    return f2v_Function.apply(input, filter, coeff, face, nfCount, vtMap)


class F2FBiasActFunction(torch.autograd.Function):
    """facet2facet followed by ``+ bias`` and a ReLU (or no activation), the first two steps of F2FConv3d's tail
    (picasso/mesh/layers.py:59-63), as ONE native forward: the convolution kernel applies them as it stores.  Backward:
    the masked gradient and the bias gradient in one pass, then the two facet2facet gradients autograd asks for."""

    @staticmethod
    def forward(ctx, textureIn, filter, bias, baryCoeff, numTexture, relu):
        for t in (baryCoeff, numTexture):
            if t.requires_grad:
                t.requires_grad = False
        bits = None
        if relu and filter.shape[0] % 32 == 0:
            out, bits = module.facet2facet_forward_act(textureIn, filter, baryCoeff, numTexture, bias, True, with_bits=True)
        else:
            out = module.facet2facet_forward_act(textureIn, filter, baryCoeff, numTexture, bias, relu)
        ctx.relu = relu
        ctx.save_for_backward(textureIn, filter, baryCoeff, numTexture, out if (relu and bits is None) else None, bits)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        textureIn, filter, baryCoeff, numTexture, out, bits = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if bits is not None and grad_output.data_ptr() % 16:
            grad_output = grad_output.clone()
        need_conv = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        gz, gb = dense.bias_act_backward(grad_output, out, need_input=need_conv, relu_bits=bits)
        gtex = gfilt = None
        if need_conv:
            gtex, gfilt = module.facet2facet_backward_selected(gz, textureIn, filter, baryCoeff, numTexture,
                                                               needs=tuple(ctx.needs_input_grad[:2]))
        return gtex, gfilt, gb if ctx.needs_input_grad[2] else None, None, None, None


def facet2facet_bias_act(textureIn, filter, bias, baryCoeff, numTexture, relu=True):
    """act(facet2facet(textureIn, filter, baryCoeff, numTexture) + bias) with gradients for the texture, the filter
    and the bias (Cout,); no counterpart function in the reference, whose module adds the bias and applies the
    activation as separate PyTorch ops (picasso/mesh/layers.py:59-63)."""
    return F2FBiasActFunction.apply(textureIn, filter, bias, baryCoeff, numTexture, relu)
