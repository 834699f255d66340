"""MI355X (gfx950) implementation of the PicassoPlus mesh convolution / pooling path:
``picassoplus_amd.mesh.layers`` (modules), ``picassoplus_amd.mesh.pi_modules`` (ops), over the C ABI of
``csrc/libpicasso_mesh.so`` (``python -m picassoplus_amd.build``)."""
