"""Mesh preparation helpers with the names of picasso/mesh/utils.py: thin wrappers over the decimation module and
``MeshHierarchy``, the builder of the per-level meshes and cluster maps a network consumes
(picasso/mesh/utils.py:32-58; picasso/networks/scene_seg.py:131 calls it once per batch).  The reference's
``view_geometry`` (an open3d window) has no counterpart here."""
import torch

from .pi_modules.decimate import (combine_clusters_, compute_triangle_geometry_, count_vertex_adjface_,
                                  mesh_decimation_)


def mesh_decimation(vertexIn, faceIn, geometryIn, nvIn, mfIn, nvSample, useArea=True, wgtBnd=1.):
    """utils.py:8-12 -> (vertexOut, faceOut, geometryOut, nvOut, mfOut, repOut, mapOut)."""
    return mesh_decimation_(vertexIn, faceIn, geometryIn, nvIn, mfIn, nvSample, useArea=useArea, wgtBnd=wgtBnd)


def compute_triangle_geometry(vertex, face):
    """[unit normal, plane offset, area] of every facet (utils.py:16-18)."""
    return compute_triangle_geometry_(vertex, face)


def count_vertex_adjface(face, vtMap, vertexOut):
    """Number of adjacent facets of the output vertices ``vtMap[i] >= 0`` (utils.py:22-24)."""
    return count_vertex_adjface_(face, vtMap, vertexOut)


def combine_clusters(rep_highRes, map_highRes, rep_lowRes, map_lowRes):
    """utils.py:27-29."""
    return combine_clusters_(rep_highRes, map_highRes, rep_lowRes, map_lowRes)


class MeshHierarchy:
    """``MeshHierarchy(nv_samples, useArea, wgtBnd)``: level l is decimated to ``nv_samples[l]`` vertices per sample;
    ``MeshHierarchy(stride, min_nvOut, useArea, wgtBnd)``: to ``nv / stride[l]`` vertices, at least ``min_nvOut[l]``
    (utils.py:32-42).  Calling it returns the list of levels, each
    ``(vertex, face, geometry, nv, mf, vt_replace, vt_map)`` with the maps from the level above (None at level 0)."""

    def __init__(self, *params):
        self.num_params = len(params)
        if self.num_params == 3:
            self.nv_samples, self.useArea, self.wgtBnd = params
            self.Iters = len(self.nv_samples)
        elif self.num_params == 4:
            self.stride, self.min_nvOut, self.useArea, self.wgtBnd = params
            self.Iters = len(self.stride)
        else:
            raise TypeError("MeshHierarchy takes (nv_samples, useArea, wgtBnd) or (stride, min_nvOut, useArea, wgtBnd)")

    def __call__(self, vertex_in, face_in, nv_in, mf_in):
        geometry_in = compute_triangle_geometry(vertex_in, face_in)
        mesh_hierarchy = [(vertex_in, face_in, geometry_in, nv_in, mf_in, None, None)]
        for l in range(self.Iters):
            if self.num_params == 3:
                nv_out = self.nv_samples[l]
            else:
                nv_out = (nv_in.to(torch.float) / float(self.stride[l])).to(torch.int)
                nv_out = torch.clip(nv_out, min=self.min_nvOut[l])
            nv_out = nv_out.to(device=nv_in.device, dtype=torch.int32).contiguous()
            level = mesh_decimation(vertex_in, face_in, geometry_in, nv_in, mf_in, nv_out, self.useArea, self.wgtBnd)
            mesh_hierarchy.append(level)
            vertex_in, face_in, geometry_in, nv_in, mf_in = level[:5]
        return mesh_hierarchy
