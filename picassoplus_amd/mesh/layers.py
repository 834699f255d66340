"""Mesh convolution / pooling modules: module API of picasso/mesh/layers.py in the reference.

Class names, constructor and ``forward`` signatures, parameter names, shapes and initialisers
(and with them the state-dict keys a checkpoint carries) follow the reference so that a network
written against ``picasso.mesh.layers`` can switch its import.  The three convolutions and the
pool / unpool ops run in hand-written HIP kernels (``pi_modules``), and so does the tail after each
separable convolution and of ``PerItemConv3d`` -- channel-mixing matmul, bias and ReLU in one pass
(``pi_modules/dense.py``), in the reference's order: matmul, bias, activation, then
BatchNorm1d(eps=1e-3), which stays a PyTorch op while it trains.
"""
from typing import List

import torch
import torch.nn as nn

from .. import _lib
from . import topology
from .pi_modules import conv3d, dense, mesh_conv3d, pool3d, unpool3d
from .pi_modules._check import stream_of


def _filter_variable_(shape, stddev=1.0, use_xavier=True):
    """New parameter: Xavier-normal by default, truncated normal(std=stddev) otherwise
    (picasso/mesh/layers.py:10-15)."""
    weight = nn.Parameter(torch.empty(shape))
    if use_xavier:
        return nn.init.xavier_normal_(weight)
    return nn.init.trunc_normal_(weight, mean=0, std=stddev)


def sph_harm_values(cart_coords, degree):
    """Real spherical-harmonic basis (N, (degree+1)^2) at the directions of ``cart_coords``
    (N, 3), evaluated by the native kernel.  Zero vectors evaluate at direction (1, 0, 0).
    No gradient flows to the coordinates."""
    xyz = cart_coords.detach()
    if not xyz.is_cuda:
        raise RuntimeError("cart_coords must be a CUDA tensor")
    if xyz.dim() != 2 or xyz.shape[1] != 3:
        raise RuntimeError("cart_coords must have shape (N, 3)")
    if degree < 0 or degree > 5:
        raise NotImplementedError("spherical harmonics are implemented for degree 0..5")
    xyz = xyz.to(torch.float32).contiguous()
    with torch.cuda.device(xyz.device):
        out = torch.empty((xyz.shape[0], (degree + 1) ** 2), dtype=torch.float32, device=xyz.device)
        _lib.call("pmesh_sph_harm", xyz.data_ptr(), out.data_ptr(), xyz.shape[0], int(degree), stream_of(xyz))
    return out


class SphHarmCoeff(nn.Module):
    """Spherical-harmonic filter coefficients of directions (facet normals, triangle corners or
    barycentric coordinates), picasso/mesh/layers.py:331-356."""

    def __init__(self, l):
        super().__init__()
        self.l = l

    def __call__(self, cart_coords):
        return sph_harm_values(cart_coords, self.l)


class _ConvTail(nn.Module):
    """bias -> activation -> batch norm, shared by every convolution module."""

    def _init_tail(self, out_channels, activation_fn, with_bn, bn_momentum):
        self.with_bn = with_bn
        self.activation_fn = activation_fn
        if with_bn:
            self.BatchNorm = nn.BatchNorm1d(out_channels, eps=0.001, momentum=bn_momentum)

    def _tail(self, outputs):
        outputs = outputs + self.biases
        if self.activation_fn is not None:
            outputs = self.activation_fn(outputs)
        if self.with_bn:
            outputs = self.BatchNorm(outputs)
        return outputs

    def _frozen_norm(self):
        """(scale, shift) of the batch norm when it only applies its running statistics, else None."""
        bn = self.BatchNorm
        if bn.training or bn.running_mean is None:
            return None
        scale = torch.rsqrt(bn.running_var + bn.eps)
        if bn.weight is not None:
            scale = scale * bn.weight
        shift = -bn.running_mean * scale
        if bn.bias is not None:
            shift = shift + bn.bias
        return scale.contiguous(), shift.contiguous()

    def _bias_tail(self, outputs):
        """``_tail(outputs)`` with bias and ReLU (or no activation) in one native pass, and a batch norm that only
        applies its running statistics folded in when no gradients are recorded."""
        relu = isinstance(self.activation_fn, nn.ReLU)
        if not (relu or self.activation_fn is None):
            return self._tail(outputs)
        biases = self.biases.reshape(-1)
        if self.with_bn and not torch.is_grad_enabled():
            frozen = self._frozen_norm()
            if frozen is not None:
                return dense.bias_act_forward(outputs.contiguous(), biases.contiguous(), relu, frozen[0], frozen[1])
        outputs = dense.bias_act(outputs.contiguous(), biases, relu)
        return self.BatchNorm(outputs) if self.with_bn else outputs

    def _dense_tail(self, inputs, weights):
        """``_tail(inputs @ weights)`` with the product, the bias and a ReLU (or no activation) in one
        native pass; without gradients an inference-mode batch norm rides along as scale/shift.  Any
        other activation, and batch norm in training mode, run as PyTorch ops on the result.  Layers with more
        than ``dense.MAX_CHANNELS`` (896) input or output channels run the reference's PyTorch ops instead."""
        if max(weights.shape) > dense.MAX_CHANNELS:
            # wider than the native pass takes (its weight slab must fit LDS): the reference's own ops
            return self._tail(torch.matmul(inputs, weights))
        relu = isinstance(self.activation_fn, nn.ReLU)
        fused_act = relu or self.activation_fn is None
        biases = self.biases.reshape(-1)
        if fused_act and self.with_bn and not torch.is_grad_enabled():
            frozen = self._frozen_norm()
            if frozen is not None:
                return dense.dense_tail_forward(inputs.contiguous(), weights.contiguous(), biases.contiguous(), relu,
                                                frozen[0], frozen[1])
        outputs = dense.dense_tail(inputs.contiguous(), weights.contiguous(), biases, relu and fused_act)
        if not fused_act:
            outputs = self.activation_fn(outputs)
        if self.with_bn:
            outputs = self.BatchNorm(outputs)
        return outputs


class F2FConv3d(_ConvTail):
    """Convolution on facet textures (picasso/mesh/layers.py:18-64).

    forward(input_texture (T,Cin), bary_coeff (T,(L+1)^2), num_texture (Nf,) per-facet counts)
    """

    def __init__(self, in_channels, out_channels, spharm_L, use_xavier=True, stddev=1e-3,
                 activation_fn=nn.ReLU(), with_bn=True, bn_momentum=0.1):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.L = spharm_L
        self.num_basis = (spharm_L + 1) ** 2
        self.use_xavier = use_xavier
        self.stddev = stddev
        self._init_tail(out_channels, activation_fn, with_bn, bn_momentum)
        self.reset_parameters()

    def reset_parameters(self):
        self.weights = _filter_variable_([self.out_channels, self.in_channels, self.num_basis],
                                         stddev=self.stddev, use_xavier=self.use_xavier)
        self.biases = nn.Parameter(torch.zeros(1, self.out_channels))

    def forward(self, input_texture, bary_coeff, num_texture):
        assert self.in_channels == input_texture.shape[-1]
        assert self.num_basis == bary_coeff.shape[-1]
        running_total = topology.running_total(num_texture)
        relu = isinstance(self.activation_fn, nn.ReLU)
        if (relu or self.activation_fn is None) and input_texture.dtype == torch.float32:
            # bias and activation ride on the convolution's store; a batch norm that only applies its running
            # statistics rides along when no gradients are recorded
            biases = self.biases.reshape(-1)
            if self.with_bn and not torch.is_grad_enabled():
                frozen = self._frozen_norm()
                if frozen is not None:
                    return mesh_conv3d.facet2facet_forward_act(input_texture.contiguous(), self.weights, bary_coeff,
                                                               running_total, biases.contiguous(), relu, frozen[0], frozen[1])
            outputs = conv3d.facet2facet_bias_act(input_texture, self.weights, biases, bary_coeff, running_total, relu)
            return self.BatchNorm(outputs) if self.with_bn else outputs
        outputs = conv3d.facet2facet(input_texture, self.weights, bary_coeff, running_total)
        return self._bias_tail(outputs)


class _SeparableConv(_ConvTail):
    """Common constructor of the two separable convolutions (spatial filter + pointwise mix)."""

    def __init__(self, in_channels, out_channels, spharm_L, depth_multiplier=1, use_xavier=True,
                 stddev=1e-3, activation_fn=nn.ReLU(), with_bn=True, bn_momentum=0.1):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.L = spharm_L
        self.num_basis = (spharm_L + 1) ** 2
        self.multiplier = depth_multiplier
        self.use_xavier = use_xavier
        self.stddev = stddev
        self._init_tail(out_channels, activation_fn, with_bn, bn_momentum)
        self.reset_parameters()

    def _spatial_shape(self):
        raise NotImplementedError

    def reset_parameters(self):
        self.spatial_weights = _filter_variable_(self._spatial_shape(), stddev=self.stddev,
                                                 use_xavier=self.use_xavier)
        self.depth_weights = _filter_variable_([self.in_channels * self.multiplier, self.out_channels],
                                               stddev=self.stddev, use_xavier=self.use_xavier)
        self.biases = nn.Parameter(torch.zeros(1, self.out_channels))

    def _mix(self, outputs):
        return self._dense_tail(outputs, self.depth_weights)


class V2FConv3d(_SeparableConv):
    """Feature propagation from vertices to facets (picasso/mesh/layers.py:67-120).

    The 3 x C x r spatial filter is the SH basis at the three triangle corners (the unit
    vectors e1, e2, e3) times ``spatial_weights`` ((L+1)^2, C*r)."""

    _corner_basis = {}

    def _spatial_shape(self):
        return [self.num_basis, self.in_channels * self.multiplier]

    def _corners(self, device):
        key = (self.L, device)
        if key not in V2FConv3d._corner_basis:
            # an ordinary tensor also when the first call comes from inside torch.inference_mode(): an inference
            # tensor could not be saved for a later training step's backward
            with torch.inference_mode(False), torch.no_grad():
                V2FConv3d._corner_basis[key] = sph_harm_values(torch.eye(3, device=device), self.L)
        return V2FConv3d._corner_basis[key]

    def forward(self, inputs, face):
        spatial_filter = torch.matmul(self._corners(inputs.device), self.spatial_weights)
        spatial_filter = spatial_filter.reshape([3, self.in_channels, self.multiplier])
        relu = isinstance(self.activation_fn, nn.ReLU)
        weights = self.depth_weights
        if ((relu or self.activation_fn is None) and max(weights.shape) <= dense.MAX_CHANNELS
                and inputs.dim() == 2 and inputs.is_contiguous() and dense.v2f_dense_supported(inputs, spatial_filter, weights)):
            # the convolution, the pointwise product, the bias and the activation in one native pass: the facet rows
            # of the convolution are formed inside the product's loads (and kept only for a backward pass); a batch
            # norm that only applies its running statistics rides along when no gradients are recorded
            spatial_filter = spatial_filter.contiguous()
            biases = self.biases.reshape(-1)
            if self.with_bn and not torch.is_grad_enabled():
                frozen = self._frozen_norm()
                if frozen is not None:
                    return dense.v2f_dense_forward(inputs, spatial_filter, face, weights.contiguous(), biases.contiguous(),
                                                   relu, frozen[0], frozen[1])
            outputs = dense.v2f_dense(inputs, spatial_filter, face, weights.contiguous(), biases, relu)
            return self.BatchNorm(outputs) if self.with_bn else outputs
        outputs = conv3d.vertex2facet(inputs, spatial_filter, face)
        return self._mix(outputs)


class F2VConv3d(_SeparableConv):
    """Convolution gathering facet features at vertices (picasso/mesh/layers.py:123-175)."""

    def _spatial_shape(self):
        return [self.num_basis, self.in_channels, self.multiplier]

    def forward(self, inputs, face, nf_count, vt_map, filt_coeff):
        relu = isinstance(self.activation_fn, nn.ReLU)
        weights = self.depth_weights
        recording = torch.is_grad_enabled() and (inputs.requires_grad or self.spatial_weights.requires_grad
                                                 or weights.requires_grad or self.biases.requires_grad)
        if (not recording and (relu or self.activation_fn is None) and inputs.dim() == 2 and inputs.is_contiguous()
                and filt_coeff.is_contiguous() and self.spatial_weights.is_contiguous()
                and dense.f2v_dense_supported(inputs, self.spatial_weights, filt_coeff, weights)):
            # Without a backward pass to serve, the convolution, the pointwise product, the bias and the activation run
            # as one native pass: a wavefront multiplies the vertex rows of the convolution by the weights before they
            # leave, and a batch norm that only applies its running statistics rides along.  With gradients recorded
            # the rows have to be written for the weight gradient anyway, and the two passes are the faster form
            # (0.48 against 0.54-0.57 ms on a 1.2 M-vertex batch; 0.49-0.50 against 0.48 ms without).
            biases = self.biases.reshape(-1).contiguous()
            frozen = self._frozen_norm() if self.with_bn else None
            if not self.with_bn or frozen is not None:
                scale, shift = frozen if frozen is not None else (None, None)
                return dense.f2v_dense_forward(inputs, self.spatial_weights, filt_coeff, face, nf_count, vt_map,
                                               weights.contiguous(), biases, relu, scale, shift)
        outputs = conv3d.facet2vertex(inputs, self.spatial_weights, filt_coeff, face, nf_count, vt_map)
        return self._mix(outputs)


class V2VConv3d(nn.Module):
    """Vertex-to-vertex convolution: V2F followed by F2V (picasso/mesh/layers.py:178-195);
    ``dual_out_channels`` and ``dual_depth_multiplier`` hold one value per stage."""

    def __init__(self, in_channels, dual_out_channels, spharm_L, dual_depth_multiplier: List[int],
                 use_xavier=True, stddev=1e-3, activation_fn=nn.ReLU(), with_bn=True, bn_momentum=0.1):
        super().__init__()
        self.V2F_conv3d = V2FConv3d(in_channels, dual_out_channels[0], spharm_L, dual_depth_multiplier[0],
                                    use_xavier, stddev, activation_fn, with_bn, bn_momentum)
        self.F2V_conv3d = F2VConv3d(dual_out_channels[0], dual_out_channels[1], spharm_L,
                                    dual_depth_multiplier[1], use_xavier, stddev, activation_fn, with_bn,
                                    bn_momentum)

    def forward(self, inputs, face, nf_count, vt_map, filt_coeff):
        outputs = self.V2F_conv3d(inputs, face)
        return self.F2V_conv3d(outputs, face, nf_count, vt_map, filt_coeff)


class PerItemConv3d(_ConvTail):
    """Pointwise (per vertex / per facet) linear layer with the conv tail
    (picasso/mesh/layers.py:198-239)."""

    def __init__(self, in_channels, out_channels, use_xavier=True, stddev=1e-3,
                 activation_fn=nn.ReLU(), with_bn=True, bn_momentum=0.1):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.use_xavier = use_xavier
        self.stddev = stddev
        self._init_tail(out_channels, activation_fn, with_bn, bn_momentum)
        self.reset_parameters()

    def reset_parameters(self):
        self.weights = _filter_variable_([self.in_channels, self.out_channels], stddev=self.stddev,
                                         use_xavier=self.use_xavier)
        self.biases = nn.Parameter(torch.zeros(1, self.out_channels))

    def forward(self, inputs):
        return self._dense_tail(inputs, self.weights)


class GlobalPool3d(nn.Module):
    """Per-sample global pooling over the vertices of a concatenated batch
    (picasso/mesh/layers.py:242-260).  'max' returns (values, argmax) like the reference's
    scatter_max call does.  Plain PyTorch ops; not part of the native path."""

    def __init__(self, method='avg'):
        super().__init__()
        self.method = method

    def forward(self, inputs, nv_in):
        batch = nv_in.shape[0]
        sample = torch.repeat_interleave(torch.arange(batch, device=inputs.device), nv_in.to(torch.int64))
        index = sample[:, None].expand(-1, inputs.shape[1])
        if self.method == 'avg':
            total = torch.zeros(batch, inputs.shape[1], dtype=inputs.dtype, device=inputs.device)
            total = total.index_add(0, sample, inputs)
            return total / nv_in.to(inputs.dtype).clamp(min=1)[:, None]
        if self.method == 'max':
            values = torch.zeros(batch, inputs.shape[1], dtype=inputs.dtype, device=inputs.device)
            values = values.scatter_reduce(0, index, inputs, 'amax', include_self=False)
            rows = torch.arange(inputs.shape[0], device=inputs.device)[:, None].expand_as(inputs)
            cand = torch.where(inputs == values[sample], rows, torch.full_like(rows, inputs.shape[0]))
            arg = torch.full((batch, inputs.shape[1]), inputs.shape[0], dtype=torch.int64, device=inputs.device)
            arg = arg.scatter_reduce(0, index, cand, 'amin', include_self=True)
            return values, arg
        raise ValueError("Unknow pooling method %s." % self.method)


class Pool3d(nn.Module):
    """Mesh pooling over decimation clusters (picasso/mesh/layers.py:263-282)."""

    def __init__(self, method='max'):
        super().__init__()
        self.method = method

    def forward(self, inputs, vt_replace, vt_map, vt_out):
        if self.method == 'max':
            return pool3d.maxPool(inputs, vt_replace, vt_map, vt_out)
        if self.method == 'avg':
            return pool3d.avgPool(inputs, vt_replace, vt_map, vt_out)
        raise ValueError("Unknow pooling method %s." % self.method)


class Unpool3d(nn.Module):
    """Mesh unpooling: every fine vertex copies its cluster's coarse row
    (picasso/mesh/layers.py:285-296)."""

    def __init__(self):
        super().__init__()

    @staticmethod
    def forward(inputs, vt_replace, vt_map):
        return unpool3d.interpolate(inputs, vt_replace, vt_map)


class BuildF2VCoeff(nn.Module):
    """Soft assignment of facet normals to learnt unit centres, softmax(cos / tau)
    (picasso/mesh/layers.py:299-328).  Plain PyTorch ops."""

    def __init__(self, kernel_size, tau=0.1, dim=3, stddev=1.0):
        super().__init__()
        self.kernel_size = kernel_size
        self.tau = tau
        self.dim = dim
        self.stddev = stddev
        self.reset_parameters()

    def reset_parameters(self):
        self.centers = _filter_variable_([self.kernel_size, self.dim], stddev=self.stddev, use_xavier=False)

    def forward(self, face_normals):
        unit = self.centers / torch.sqrt(torch.sum(self.centers ** 2, dim=-1, keepdim=True))
        zeta = torch.matmul(face_normals, unit.to(face_normals.device).t()) / self.tau
        coeff = torch.exp(zeta)
        return coeff / torch.sum(coeff, dim=-1, keepdim=True)
