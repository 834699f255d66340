"""Ops of the point-cloud branch (same module and function names as picasso/point/pi_modules): ``nnquery``,
``sample``, ``buildkernel``, ``conv3d``, ``pool3d``, ``unpool3d``.  The ``point_*`` modules are the
native-extension-shaped layer underneath, implemented over the C ABI of libpicasso_mesh."""
from . import buildkernel, conv3d, nnquery, pool3d, sample, unpool3d

__all__ = ['buildkernel', 'conv3d', 'nnquery', 'pool3d', 'sample', 'unpool3d']
