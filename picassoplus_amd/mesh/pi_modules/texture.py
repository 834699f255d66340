"""Texture points of the facets from vertex features, with the basis values of their barycentric coordinates.

The reference has no such routine: it loads the texture points' features from its dataset files
(picasso/mesh/dataset_scene.py:29-33) and evaluates the spherical-harmonic basis of their barycentric
coordinates in the network (picasso/networks/scene_seg.py:150).  A block that chains facet2facet after
vertex features (vertex2facet -> facet2facet -> facet2vertex) needs the features at the texture points:
``interpolate`` computes both inputs of ``conv3d.facet2facet`` in one native pass and is differentiable
with respect to the vertex features.
"""
import torch

from ... import _lib
from .. import topology
from ._check import F32, I32, check_input, same_device, stream_of


def _dims(input, face, baryCoord, numTexture):
    check_input(input, "input", 2, F32)
    check_input(face, "face", 2, I32)
    check_input(baryCoord, "baryCoord", 2, F32)
    check_input(numTexture, "numTexture", 1, I32)
    if face.shape[1] != 3:
        raise RuntimeError("face must have shape (NfIn, 3)")
    if baryCoord.shape[1] != 3:
        raise RuntimeError("baryCoord must have shape (NiK, 3)")
    if numTexture.shape[0] != face.shape[0]:
        raise RuntimeError("numTexture must hold one running total per facet")
    return input.shape[0], face.shape[0], baryCoord.shape[0], input.shape[1]


def _check_totals(numTexture, T):
    """One-off validation of the running totals (synchronises; only the first time a tensor is seen)."""
    def check():
        if numTexture.numel() and topology._checks_enabled():
            steps = torch.diff(numTexture, prepend=numTexture.new_zeros(1))
            if int(steps.min()) < 0 or int(numTexture[-1]) != T:
                raise RuntimeError("numTexture must be a non-decreasing running total that ends at the number of "
                                   "texture points (%d)" % T)
    topology.checked_once("rt", (numTexture,), (int(T),), check)


def texture_forward(input, face, baryCoord, numTexture, degree):
    """(Nv,C), (Nf,3), (T,3), (Nf,) -> [texture (T,C), baryCoeff (T,(degree+1)^2) or None if degree is None]."""
    Nv, Nf, T, C = _dims(input, face, baryCoord, numTexture)
    if degree is not None and (degree < 0 or degree > 5):
        raise NotImplementedError("spherical harmonics are implemented for degree 0..5")
    dev = same_device(input, face, baryCoord, numTexture)
    if Nf:
        topology._check_range_cached(face, Nv)       # an empty input with facets raises: every index is out of range
    _check_totals(numTexture, T)
    with torch.cuda.device(dev):
        tex = torch.empty((T, C), dtype=F32, device=dev)
        coeff = torch.empty((T, (degree + 1) ** 2), dtype=F32, device=dev) if degree is not None else None
        _lib.call("pmesh_texture_fwd", input.data_ptr(), face.data_ptr(), baryCoord.data_ptr(), numTexture.data_ptr(),
                  tex.data_ptr(), coeff.data_ptr() if coeff is not None else None, Nv, Nf, T, C,
                  int(degree) if degree is not None else 0, stream_of(input))
    return [tex, coeff]


def texture_backward(grad_texture, face, baryCoord, numTexture, n_vertices):
    """Transpose of the interpolation: (T,C) -> grad_input (Nv,C)."""
    check_input(grad_texture, "grad_texture", 2, F32)
    T, C = grad_texture.shape
    Nf = face.shape[0]
    if baryCoord.shape[0] != T:
        raise RuntimeError("grad_texture must have one row per texture point")
    dev = same_device(grad_texture, face, baryCoord, numTexture)
    rowptr, colidx = topology.vertex_csr(face, None, n_vertices)
    with torch.cuda.device(dev):
        gin = torch.empty((n_vertices, C), dtype=F32, device=dev)
        _lib.call("pmesh_texture_bwd", grad_texture.data_ptr(), baryCoord.data_ptr(), numTexture.data_ptr(),
                  rowptr.data_ptr(), colidx.data_ptr(), gin.data_ptr(), n_vertices, Nf, T, C, stream_of(grad_texture))
    return gin


class TextureFunction(torch.autograd.Function):
    """autograd Function of ``interpolate``: gradient for the vertex features only."""

    @staticmethod
    def forward(ctx, input, face, baryCoord, numTexture, degree):
        for t in (face, baryCoord, numTexture):
            if t.requires_grad:
                t.requires_grad = False
        tex, coeff = texture_forward(input, face, baryCoord, numTexture, degree)
        ctx.save_for_backward(face, baryCoord, numTexture)
        ctx.n_vertices = input.shape[0]
        if coeff is None:
            return tex
        ctx.mark_non_differentiable(coeff)
        return tex, coeff

    @staticmethod
    def backward(ctx, grad_texture, *unused):
        face, baryCoord, numTexture = ctx.saved_tensors
        gin = texture_backward(grad_texture.contiguous(), face, baryCoord, numTexture, ctx.n_vertices)
        return gin, None, None, None, None


def interpolate(input, face, baryCoord, numTexture, degree=3):
    """Features and basis values of the texture points, the first and third argument of ``conv3d.facet2facet``.

    input      (Nv, C) float32 vertex features
    face       (Nf, 3) int32
    baryCoord  (T, 3) float32 barycentric coordinates of the texture points, rows grouped by facet in facet order
    numTexture (Nf,) int32: inclusive running total of texture points per facet
    degree     degree of the spherical-harmonic basis (0..5), or None for the features alone
    returns    (texture (T, C), baryCoeff (T, (degree+1)^2)), or texture alone when degree is None
    """
    return TextureFunction.apply(input, face, baryCoord, numTexture, degree)
