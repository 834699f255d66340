"""Per-level producers of the convolution inputs: adjacent-facet counts of the output vertices,
triangle geometry, oriented normals with their basis coefficients, and the composition of two decimation steps' cluster maps, with the reference's function
names (picasso/mesh/pi_modules/decimate.py:53-93).  The decimation that produces the cluster maps is in decimate.py."""
import torch

from ... import _lib
from .. import topology
from ._check import F32, I32, check_input, same_device, stream_of


def count_vertex_adjface_(face, vtMap, vertexOut):
    """Number of adjacent (facet, corner) entries of every output vertex ``{vtMap[i] | vtMap[i] >= 0}``
    (decimate.py:88-93, decimate_gpu.cu:813-836) -> int32 (NvOut,).  It is the row length of the
    facet-to-vertex adjacency, which is built (and cached for the convolutions) here."""
    check_input(face, "face", 2, I32)
    check_input(vtMap, "vtMap", 1, I32)
    if not isinstance(vertexOut, torch.Tensor) or vertexOut.dim() != 2:
        raise RuntimeError("vertexOut must have dimension of 2")
    dev = same_device(face, vtMap)
    nv_out = vertexOut.shape[0]
    rowptr, _ = topology.vertex_csr(face, vtMap, nv_out)
    with torch.cuda.device(dev):
        out = torch.empty(nv_out, dtype=I32, device=dev)
        _lib.call("pmesh_count_vertex_adjface", rowptr.data_ptr(), out.data_ptr(), nv_out, stream_of(face))
    return out


def compute_triangle_geometry_(vertex, face):
    """(Nf, 5) = unit normal, plane offset d = -n.v0, area of every facet (decimate.py:70-85).
    ``vertex`` (Nv, >= 3) float32 with the position in the first three columns."""
    check_input(vertex, "vertex", 2, F32)
    check_input(face, "face", 2, I32)
    if vertex.shape[1] < 3 or face.shape[1] != 3:
        raise RuntimeError("vertex must have at least 3 columns and face exactly 3")
    dev = same_device(vertex, face)
    topology._check_range_cached(face, vertex.shape[0])
    with torch.cuda.device(dev):
        out = torch.empty((face.shape[0], 5), dtype=F32, device=dev)
        _lib.call("pmesh_triangle_geometry", vertex.data_ptr(), face.data_ptr(), out.data_ptr(), vertex.shape[0],
                  face.shape[0], vertex.shape[1], stream_of(vertex))
    return out


def facet_frame_(vertex, face, degree=3):
    """Triangle geometry, oriented normals and their spherical-harmonic coefficients in one native pass:
    what a network prepares per mesh level for its facet2vertex convolutions (picasso/networks/scene_seg.py:146-149,
    161-164: ``compute_triangle_geometry_`` -> ``get_oriented_normals`` -> ``cal_sph_harm``).

    returns (geometry (Nf, 5), face_normals (Nf, 3) turned towards the origin, filt_coeff (Nf, (degree+1)^2));
    ``degree`` None skips the coefficients (third result None)."""
    check_input(vertex, "vertex", 2, F32)
    check_input(face, "face", 2, I32)
    if vertex.shape[1] < 3 or face.shape[1] != 3:
        raise RuntimeError("vertex must have at least 3 columns and face exactly 3")
    if degree is not None and (degree < 0 or degree > 5):
        raise NotImplementedError("spherical harmonics are implemented for degree 0..5")
    dev = same_device(vertex, face)
    topology._check_range_cached(face, vertex.shape[0])
    nf = face.shape[0]
    with torch.cuda.device(dev):
        geo = torch.empty((nf, 5), dtype=F32, device=dev)
        nrm = torch.empty((nf, 3), dtype=F32, device=dev)
        coeff = torch.empty((nf, (degree + 1) ** 2), dtype=F32, device=dev) if degree is not None else None
        _lib.call("pmesh_facet_frame", vertex.data_ptr(), face.data_ptr(), geo.data_ptr(), nrm.data_ptr(),
                  coeff.data_ptr() if coeff is not None else None, vertex.shape[0], nf, vertex.shape[1],
                  int(degree) if degree is not None else 0, stream_of(vertex))
    return geo, nrm, coeff


def combine_clusters_(repA, mapA, repB, mapB):
    """Cluster maps of two consecutive decimation steps -> the maps of both steps together (decimate.py:53-67,
    decimate_gpu.cu:750-810).  ``repA``/``mapA`` (int32, fine vertices) describe the first step, ``repB``/``mapB``
    the second over the vertices the first keeps; returns (repComb, mapComb) over the fine vertices: the
    ``vt_replace`` / ``vt_map`` of a pooling layer across both steps."""
    for name, t in (("repA", repA), ("mapA", mapA), ("repB", repB), ("mapB", mapB)):
        check_input(t, name, 1, I32)
    if repA.shape != mapA.shape or repB.shape != mapB.shape:
        raise RuntimeError("rep and map of one step must have the same length")
    dev = same_device(repA, mapA, repB, mapB)
    nv_a, nv_b = repA.shape[0], repB.shape[0]
    topology._check_range("mapA", mapA, -1, nv_b)
    topology._check_range("repA", repA, -(nv_a - 1), max(nv_a, 1))
    topology._check_range("repB", repB, -(nv_b - 1), max(nv_b, 1))
    with torch.cuda.device(dev):
        rep_out = torch.empty_like(repA)
        map_out = torch.empty_like(mapA)
        scratch = torch.empty(max(nv_b, 1), dtype=I32, device=dev)
        _lib.call("pmesh_combine_clusters", repA.data_ptr(), mapA.data_ptr(), repB.data_ptr(), mapB.data_ptr(),
                  rep_out.data_ptr(), map_out.data_ptr(), scratch.data_ptr(), nv_a, nv_b, stream_of(repA))
    return rep_out, map_out
