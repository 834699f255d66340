from . import conv3d, pool3d, unpool3d

__all__ = ['conv3d', 'pool3d', 'unpool3d']
