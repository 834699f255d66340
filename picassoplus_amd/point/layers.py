"""Point-cloud modules with the API of picasso/point/layers.py: same class names, constructor arguments, ``forward``
signatures and parameter names (``spatial_weights``, ``depth_weights``, ``biases``, ``BatchNorm.*``)."""
import torch
import torch.nn as nn

from ..mesh.layers import PerItemConv3d, _ConvTail, _filter_variable_, sph_harm_values  # noqa: F401 (PerItemConv3d: layers.py:78-119)
from .pi_modules import conv3d, pool3d, unpool3d


class PCloudConv3d(_ConvTail):
    """Separable point convolution (picasso/point/layers.py:19-75): depthwise (fuzzy) SPH3D convolution over the
    neighbour pairs, then the pointwise product, bias, activation and batch norm.

    forward(inputs (Np,Cin), nn_count, nn_index, filt_index, filt_coeff=None)"""

    def __init__(self, in_channels, out_channels, num_basis, depth_multiplier=1, use_xavier=True, stddev=1e-3,
                 activation_fn=nn.ReLU(), with_bn=True, bn_momentum=0.1):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.num_basis = num_basis
        self.multiplier = depth_multiplier
        self.use_xavier = use_xavier
        self.stddev = stddev
        self._init_tail(out_channels, activation_fn, with_bn, bn_momentum)
        self.reset_parameters()

    def reset_parameters(self):
        self.spatial_weights = _filter_variable_([self.num_basis, self.in_channels, self.multiplier],
                                                 use_xavier=self.use_xavier)
        self.depth_weights = _filter_variable_([self.in_channels * self.multiplier, self.out_channels],
                                               use_xavier=self.use_xavier)
        self.biases = nn.Parameter(torch.zeros(1, self.out_channels))

    def forward(self, inputs, nn_count, nn_index, filt_index, filt_coeff=None):
        if filt_coeff is None:
            outputs = conv3d.conv3d(inputs, self.spatial_weights, nn_count, nn_index, filt_index)
        else:
            outputs = conv3d.fuzzyconv3d(inputs, self.spatial_weights, nn_count, nn_index, filt_index, filt_coeff)
        return self._dense_tail(outputs, self.depth_weights)


class Pool3d(nn.Module):
    """Point pooling over neighbour pairs (picasso/point/layers.py:122-142): method 'max' or 'avg'."""

    def __init__(self, method='max'):
        super().__init__()
        self.method = method

    def forward(self, inputs, nn_count, nn_index):
        if self.method == 'max':
            return pool3d.maxPool(inputs, nn_count, nn_index)
        if self.method == 'avg':
            return pool3d.avgPool(inputs, nn_count, nn_index)
        raise ValueError("Unknow pooling method %s." % self.method)


class Unpool3d(nn.Module):
    """Weighted interpolation from a coarse point set (picasso/point/layers.py:145-155)."""

    def forward(self, inputs, weight, nn_index):
        return unpool3d.interpolate(inputs, weight, nn_index)


class BuildSpharmCoeff(nn.Module):
    """Spherical-harmonic values of the directions from every query to its neighbours
    (picasso/point/layers.py:158-185) -> (Nout, (l+1)^2)."""

    def __init__(self, l):
        super().__init__()
        self.l = l

    @staticmethod
    def proj_to_sphere(xyz):
        l2norm = torch.sqrt(torch.sum(xyz ** 2, dim=-1, keepdim=True))
        return xyz / (l2norm + 1e-10)

    def forward(self, xyz_data, xyz_query, nn_idx):
        nn_idx = nn_idx.to(torch.long)
        delta = xyz_data[nn_idx[:, 1], :3] - xyz_query[nn_idx[:, 0], :3]
        return sph_harm_values(delta, self.l)
