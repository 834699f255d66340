"""TEST INFRASTRUCTURE ONLY: numpy front end of the brute-force C loop oracle.

Loads ``oracle/libmesh_oracle.so`` (built from ``mesh_loops.c`` by the Makefile
beside it) and exposes every loop function on numpy arrays in float32 or
float64.  The product never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmesh_oracle.so")
_lib = None


def build(force=False):
    """Compile the loop oracle with gcc (a few hundred ms)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError("loop oracle supports float32 and float64 only")


def _f(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _call(name, dtype, *args):
    fn = getattr(_load(), "%s_%s" % (name, _suffix(dtype)))
    fn.restype = ctypes.c_int
    conv = []
    for a in args:
        conv.append(_p(a) if isinstance(a, np.ndarray) else ctypes.c_int(int(a)))
    return fn(*conv)


def v2f_fwd(x, filt, face, dtype=np.float64):
    x, filt, face = _f(x, dtype), _f(filt, dtype), _i(face)
    Nf, (C, r) = face.shape[0], filt.shape[1:]
    out = np.empty((Nf, C * r), dtype)
    _call("ref_v2f_fwd", dtype, Nf, C, r, face, x, filt, out)
    return out


def v2f_bwd(gout, x, filt, face, dtype=np.float64):
    gout, x, filt, face = _f(gout, dtype), _f(x, dtype), _f(filt, dtype), _i(face)
    Nf, Nv, (C, r) = face.shape[0], x.shape[0], filt.shape[1:]
    gin, gfilt = np.empty((Nv, C), dtype), np.empty((3, C, r), dtype)
    _call("ref_v2f_bwd", dtype, Nf, Nv, C, r, face, x, filt, gout, gin, gfilt)
    return gin, gfilt


def f2v_fwd(x, filt, coeff, face, nfcount, vtmap, dtype=np.float64):
    x, filt, coeff = _f(x, dtype), _f(filt, dtype), _f(coeff, dtype)
    face, nfcount, vtmap = _i(face), _i(nfcount), _i(vtmap)
    Nf, C = x.shape
    K, _, r = filt.shape
    NvOut = nfcount.shape[0]
    out = np.empty((NvOut, C * r), dtype)
    _call("ref_f2v_fwd", dtype, Nf, C, r, K, NvOut, vtmap, nfcount, face, coeff, x, filt, out)
    return out


def f2v_bwd(gout, x, filt, coeff, face, nfcount, vtmap, dtype=np.float64):
    gout, x, filt, coeff = _f(gout, dtype), _f(x, dtype), _f(filt, dtype), _f(coeff, dtype)
    face, nfcount, vtmap = _i(face), _i(nfcount), _i(vtmap)
    Nf, C = x.shape
    K, _, r = filt.shape
    gin, gfilt = np.empty((Nf, C), dtype), np.empty((K, C, r), dtype)
    _call("ref_f2v_bwd", dtype, Nf, C, r, K, nfcount.shape[0], vtmap, nfcount, face,
          coeff, x, filt, gout, gin, gfilt)
    return gin, gfilt


def f2f_fwd(tex, filt, bary, cum, dtype=np.float64):
    tex, filt, bary, cum = _f(tex, dtype), _f(filt, dtype), _f(bary, dtype), _i(cum)
    Cout, Cin, F = filt.shape
    Nf = cum.shape[0]
    out = np.empty((Nf, Cout), dtype)
    _call("ref_f2f_fwd", dtype, Nf, F, Cin, Cout, cum, bary, tex, filt, out)
    return out


def f2f_bwd(gout, tex, filt, bary, cum, dtype=np.float64):
    gout, tex, filt, bary = _f(gout, dtype), _f(tex, dtype), _f(filt, dtype), _f(bary, dtype)
    cum = _i(cum)
    Cout, Cin, F = filt.shape
    Nf, T = cum.shape[0], tex.shape[0]
    gin, gfilt = np.empty((T, Cin), dtype), np.empty((Cout, Cin, F), dtype)
    _call("ref_f2f_bwd", dtype, Nf, T, F, Cin, Cout, cum, bary, tex, filt, gout, gin, gfilt)
    return gin, gfilt


def maxpool_fwd(x, vt_replace, vt_map, nv_out, dtype=np.float64):
    x, vt_replace, vt_map = _f(x, dtype), _i(vt_replace), _i(vt_map)
    Nv, C = x.shape
    out, idx = np.empty((nv_out, C), dtype), np.empty((nv_out, C), np.int32)
    _call("ref_maxpool_fwd", dtype, Nv, C, nv_out, vt_replace, vt_map, x, out, idx)
    return out, idx


def maxpool_bwd(gout, nv_in, maxidx, dtype=np.float64):
    gout, maxidx = _f(gout, dtype), _i(maxidx)
    NvOut, C = gout.shape
    gin = np.empty((nv_in, C), dtype)
    _call("ref_maxpool_bwd", dtype, NvOut, C, nv_in, maxidx, gout, gin)
    return gin


def avgpool_fwd(x, vt_replace, vt_map, nv_out, dtype=np.float64):
    x, vt_replace, vt_map = _f(x, dtype), _i(vt_replace), _i(vt_map)
    Nv, C = x.shape
    out = np.empty((nv_out, C), dtype)
    _call("ref_avgpool_fwd", dtype, Nv, C, nv_out, vt_replace, vt_map, x, out)
    return out


def avgpool_bwd(gout, vt_replace, vt_map, dtype=np.float64):
    gout, vt_replace, vt_map = _f(gout, dtype), _i(vt_replace), _i(vt_map)
    Nv, C = vt_map.shape[0], gout.shape[1]
    gin = np.empty((Nv, C), dtype)
    _call("ref_avgpool_bwd", dtype, Nv, C, vt_replace, vt_map, gout, gin)
    return gin


def unpool_fwd(x, vt_replace, vt_map, dtype=np.float64):
    x, vt_replace, vt_map = _f(x, dtype), _i(vt_replace), _i(vt_map)
    Nv, C = vt_map.shape[0], x.shape[1]
    out = np.empty((Nv, C), dtype)
    _call("ref_unpool_fwd", dtype, Nv, C, vt_replace, vt_map, x, out)
    return out


def unpool_bwd(gout, nv_coarse, vt_replace, vt_map, dtype=np.float64):
    gout, vt_replace, vt_map = _f(gout, dtype), _i(vt_replace), _i(vt_map)
    Nv, C = gout.shape
    gin = np.empty((nv_coarse, C), dtype)
    _call("ref_unpool_bwd", dtype, Nv, C, nv_coarse, vt_replace, vt_map, gout, gin)
    return gin


def sph_harm(xyz, L, dtype=np.float64):
    xyz = _f(xyz, dtype).reshape(-1, 3)
    out = np.empty((xyz.shape[0], (L + 1) ** 2), dtype)
    if _call("ref_sph_harm", dtype, xyz.shape[0], L, xyz, out):
        raise NotImplementedError("spherical-harmonic degree must be 0..5")
    return out


def texture_fwd(x, face, bary, cum, dtype=np.float64):
    """Features of texture points by barycentric interpolation of the corner features: (T, C)."""
    x, bary, face, cum = _f(x, dtype), _f(bary, dtype), _i(face), _i(cum)
    T = int(cum[-1]) if cum.shape[0] else 0
    tex = np.empty((T, x.shape[1]), dtype)
    _call("ref_texture_fwd", dtype, cum.shape[0], x.shape[1], face, cum, bary, x, tex)
    return tex


def texture_bwd(gtex, nv, face, bary, cum, dtype=np.float64):
    gtex, bary, face, cum = _f(gtex, dtype), _f(bary, dtype), _i(face), _i(cum)
    gin = np.empty((nv, gtex.shape[1]), dtype)
    _call("ref_texture_bwd", dtype, cum.shape[0], nv, gtex.shape[1], face, cum, bary, gtex, gin)
    return gin
