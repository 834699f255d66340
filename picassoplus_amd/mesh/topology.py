"""Sorted adjacency (CSR) of index tensors, built on the GPU once and reused.

The reference passes raw index tensors (``face``, ``vt_map``, ``vt_replace``) to every op
and scatters with float atomics.  Here the scatter ops are segmented reductions, which need
the transposed adjacency.  A network reuses the same index tensors for every convolution of
a mesh level, forward and backward (picasso/networks/pi2_blocks.py:89-92 in the reference),
so the adjacency is cached per index tensor: the key is the tensor's storage address, shape
and in-place version counter, and the entry keeps the tensor alive so the address cannot be
recycled while cached.
"""
import os
import threading
from collections import OrderedDict

import torch

from .. import _lib

_LOCK = threading.Lock()
_CACHE = OrderedDict()
MAX_ENTRIES = 256


def clear_cache():
    with _LOCK:
        _CACHE.clear()


def _key(kind, *tensors_and_ints):
    parts = [kind]
    for t in tensors_and_ints:
        if isinstance(t, torch.Tensor):
            parts.append((t.data_ptr(), tuple(t.shape), t._version, t.device.index))
        else:
            parts.append(t)
    return tuple(parts)


def _lookup(key):
    with _LOCK:
        hit = _CACHE.get(key)
        if hit is not None:
            _CACHE.move_to_end(key)
        return hit


def _store(key, value):
    with _LOCK:
        _CACHE[key] = value
        while len(_CACHE) > MAX_ENTRIES:
            _CACHE.popitem(last=False)


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _checks_enabled():
    return os.environ.get("PICASSO_MESH_SKIP_CHECKS", "0") != "1"


def _check_range(name, t, lo, hi):
    """One-off validation of an index tensor (synchronises; only on a cache miss)."""
    if t.numel() == 0 or not _checks_enabled():
        return
    mn, mx = int(t.min()), int(t.max())
    if mn < lo or mx >= hi:
        raise RuntimeError("%s holds indices in [%d, %d], valid range is [%d, %d)" % (name, mn, mx, lo, hi))


def vertex_csr(face, vt_map, n_rows):
    """Row v -> ascending list of entries e = 3*facet + corner landing on v.

    ``vt_map`` None keys entries by ``face`` itself (rows = input vertices); otherwise by
    ``vt_map[face]`` with negative values dropped (rows = output vertices).
    Returns (rowptr int32 (n_rows+1), colidx int32 (3*Nf)).
    """
    key = _key("v", face, vt_map, int(n_rows))
    hit = _lookup(key)
    if hit is not None:
        return hit[0], hit[1]
    nf = face.shape[0]
    n_keys = vt_map.shape[0] if vt_map is not None else n_rows
    _check_range("face", face, 0, n_keys)
    with torch.cuda.device(face.device):
        rowptr = torch.empty(n_rows + 1, dtype=torch.int32, device=face.device)
        colidx = torch.empty(3 * nf, dtype=torch.int32, device=face.device)
        ws_bytes = _lib.query("pmesh_vertex_csr_workspace_bytes", nf, n_rows)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=face.device)
        _lib.call("pmesh_build_vertex_csr", face.data_ptr(), vt_map.data_ptr() if vt_map is not None else None,
                  nf, n_keys if vt_map is not None else 0, n_rows, rowptr.data_ptr(), colidx.data_ptr(),
                  ws.data_ptr(), ws_bytes, _stream(face))
    _store(key, (rowptr, colidx, face, vt_map))
    return rowptr, colidx


def cluster_csr(vt_replace, vt_map, n_coarse):
    """Coarse row -> ascending list of fine vertices of that decimation cluster.

    Returns (rowptr int32 (n_coarse+1), members int32 (n_fine)).
    """
    key = _key("c", vt_replace, vt_map, int(n_coarse))
    hit = _lookup(key)
    if hit is not None:
        return hit[0], hit[1]
    n_fine = vt_replace.shape[0]
    if vt_map.shape[0] != n_fine:
        raise RuntimeError("vt_replace and vt_map must have the same length")
    _check_range("vt_replace", vt_replace, -(n_fine - 1), max(n_fine, 1))
    with torch.cuda.device(vt_replace.device):
        rowptr = torch.empty(n_coarse + 1, dtype=torch.int32, device=vt_replace.device)
        members = torch.empty(n_fine, dtype=torch.int32, device=vt_replace.device)
        ws_bytes = _lib.query("pmesh_cluster_csr_workspace_bytes", n_fine, n_coarse)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=vt_replace.device)
        _lib.call("pmesh_build_cluster_csr", vt_replace.data_ptr(), vt_map.data_ptr(), n_fine, n_coarse,
                  rowptr.data_ptr(), members.data_ptr(), ws.data_ptr(), ws_bytes, _stream(vt_replace))
    _store(key, (rowptr, members, vt_replace, vt_map))
    return rowptr, members


def facet_order(cum_texture, n_points):
    """Permutation of the facets by their number of texture points (stable), from the running
    total ``cum_texture``; lets the facet2facet kernels give every wavefront facets of equal length."""
    key = _key("o", cum_texture, int(n_points))
    hit = _lookup(key)
    if hit is not None:
        return hit[0]
    nf = cum_texture.shape[0]
    with torch.cuda.device(cum_texture.device):
        order = torch.empty(nf, dtype=torch.int32, device=cum_texture.device)
        ws_bytes = _lib.query("pmesh_facet_order_workspace_bytes", nf)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=cum_texture.device)
        _lib.call("pmesh_build_facet_order", cum_texture.data_ptr(), nf, int(n_points), order.data_ptr(),
                  ws.data_ptr(), ws_bytes, _stream(cum_texture))
    _store(key, (order, cum_texture))
    return order


def running_total(num_texture):
    """Inclusive running total (int32) of the per-facet texture-point counts, the form facet2facet takes
    (picasso/mesh/layers.py:57 computes it in every forward); cached per counts tensor, so that the facet order
    built from it is found again too."""
    key = _key("c", num_texture)
    hit = _lookup(key)
    if hit is not None:
        return hit[0]
    total = torch.cumsum(num_texture, dim=0, dtype=torch.int)
    _store(key, (total, num_texture))
    return total


def _check_range_cached(face, n_vertices):
    """Validate a facet tensor against a vertex count once per tensor."""
    key = _key("rf", face, int(n_vertices))
    if _lookup(key) is None:
        _check_range("face", face, 0, n_vertices)
        _store(key, (True, face))


def _check_cluster_cached(vt_replace, vt_map):
    key = _key("rk", vt_replace, vt_map)
    if _lookup(key) is None:
        n_fine = vt_replace.shape[0]
        _check_range("vt_replace", vt_replace, -(n_fine - 1), max(n_fine, 1))
        _store(key, (True, vt_replace, vt_map))
