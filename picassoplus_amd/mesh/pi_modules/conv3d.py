"""Differentiable mesh convolutions: API of picasso/mesh/pi_modules/conv3d.py.

``vertex2facet``, ``facet2facet`` and ``facet2vertex`` take the same arguments in the same
order as the reference functions (conv3d.py:21,55,89), save the same tensors for backward
and return ``None`` gradients for index and coefficient inputs.  Backward only computes the
gradients autograd asks for through ``needs_input_grad``; both are produced by one native
call, so nothing is saved by skipping and both are always computed, as in the reference.
"""
import torch

from . import mesh_conv3d as module


def _no_grad_flags(*tensors):
    # the reference clears requires_grad on index / coefficient inputs in place (conv3d.py:8-9)
    for t in tensors:
        if t.requires_grad:
            t.requires_grad = False


class f2f_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, textureIn, filter, baryCoeff, numTexture):
        _no_grad_flags(baryCoeff, numTexture)
        output = module.facet2facet_forward(textureIn, filter, baryCoeff, numTexture)
        ctx.save_for_backward(textureIn, filter, baryCoeff, numTexture)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input, grad_filter = module.facet2facet_backward(grad_output.contiguous(), *ctx.saved_tensors)
        return grad_input, grad_filter, None, None


def facet2facet(textureIn, filter, baryCoeff, numTexture):
    """Facet features from the features of texture points sampled inside each facet.

    textureIn  (T, Cin) float32, rows grouped by facet in facet order
    filter     (Cout, Cin, F) float32
    baryCoeff  (T, F) float32: spherical-harmonic values of each point's barycentric coordinates
    numTexture (Nf,) int32: inclusive running total of texture points per facet
    returns    (Nf, Cout) float32
    """
    return f2f_Function.apply(textureIn, filter, baryCoeff, numTexture)


class v2f_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, filter, face):
        _no_grad_flags(face)
        output = module.vertex2facet_forward(input, filter, face)
        ctx.save_for_backward(input, filter, face)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input, grad_filter = module.vertex2facet_backward(grad_output.contiguous(), *ctx.saved_tensors)
        return grad_input, grad_filter, None


def vertex2facet(input, filter, face):
    """Facet features as a filtered combination of the three corner features.

    input  (Nv, C) float32;  filter (3, C, r) float32;  face (Nf, 3) int32
    returns (Nf, C*r) float32
    """
    return v2f_Function.apply(input, filter, face)


class f2v_Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, filter, coeff, face, nfCount, vtMap):
        _no_grad_flags(coeff, face, nfCount, vtMap)
        output = module.facet2vertex_forward(input, filter, coeff, face, nfCount, vtMap)
        ctx.save_for_backward(input, filter, coeff, face, nfCount, vtMap)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input, grad_filter = module.facet2vertex_backward(grad_output.contiguous(), *ctx.saved_tensors)
        return grad_input, grad_filter, None, None, None, None


def facet2vertex(input, filter, coeff, face, nfCount, vtMap):
    """Vertex features averaged over the incident facets, filtered per facet.

    input (Nf, C);  filter (K, C, r);  coeff (Nf, K);  face (Nf, 3) int32;
    nfCount (NvOut,) int32 divisor per output vertex;  vtMap (NvIn,) int32 input->output vertex
    returns (NvOut, C*r) float32
    """
    return f2v_Function.apply(input, filter, coeff, face, nfCount, vtMap)
