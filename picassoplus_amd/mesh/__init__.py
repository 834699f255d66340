"""Mesh convolution / pooling modules with the API of ``picasso.mesh`` of the reference."""
from . import pi_modules  # noqa: F401
from .pi_modules import conv3d, pool3d, unpool3d  # noqa: F401
