from . import conv3d, geometry, pool3d, unpool3d

__all__ = ['conv3d', 'geometry', 'pool3d', 'unpool3d']
