"""Differentiable ops of the mesh layer (same module and function names as picasso/mesh/pi_modules):
``conv3d`` (vertex2facet, facet2facet, facet2vertex), ``pool3d`` (maxPool, avgPool), ``unpool3d``
(interpolate), plus ``geometry`` (adjacent-facet counts, triangle geometry) and ``texture`` (texture points of the
facets interpolated from vertex features).  The ``mesh_*`` modules
are the native-extension-shaped layer underneath, implemented over the C ABI of libpicasso_mesh."""
import importlib

__all__ = ["conv3d", "geometry", "pool3d", "texture", "unpool3d"]
for _name in __all__:
    globals()[_name] = importlib.import_module("." + _name, __name__)
del _name
