"""Quadric-error mesh decimation: API of picasso/mesh/pi_modules/decimate.py (``mesh_decimation_`` and the
``simplify`` round of the reference's ``mesh_decimation`` extension, decimate.cpp:21-89), deterministic.

One round (``simplify``) = vertex quadrics from the facets and the boundary edges -> cost of every candidate
edge -> greedy vertex clustering in cost order -> cluster maps, contracted vertices, remapped facets.  The
reference gets different ``vt_replace`` / ``vt_map`` from run to run (float atomics, unstable sorts, ties broken by
whatever order a sort leaves); here every sum has a fixed order and the candidate edges a total order
(sample, cost, mix(vi, vj), vi, vj), so the maps are a function of the input alone.  The arithmetic runs in native kernels
(``pmesh_vertex_quadrics``, ``pmesh_boundary_quadrics``, ``pmesh_edge_costs``), the greedy clustering on the device as a
fixed-point iteration with the serial routine's result (``cluster_vertices_device``; the reference's serial host
routine is ``pmesh_cluster_vertices_host``, kept as the checker and behind ``PMESH_DECIMATE_HOST_CLUSTERING=1``), the
contraction is the average pooling op over the new maps; sorting / unique / scans of integer keys between them are
PyTorch ops.
"""
import contextlib
import ctypes
import os
import threading

import numpy as np
import torch

from ... import _lib
from .. import topology
from . import mesh_pool3d
from ._check import F32, I32, check_input, same_device, stream_of
from .geometry import combine_clusters_, compute_triangle_geometry_, count_vertex_adjface_  # noqa: F401 (decimate.py:53-93)


def vertex_quadrics(vertexIn, faceIn, geometryIn, useArea=True, wgtBnd=5.0, own_face=False):
    """Quadric (Nv, 10) of every vertex and the candidate edges of the batch.

    returns (quadric, edge_vi, edge_vj): the unique edges (vi < vj, int32) in ascending (vi, vj) order.
    ``own_face``: the facets are an earlier round's output, their index range is not checked again."""
    check_input(vertexIn, "vertexIn", 2, F32)
    check_input(faceIn, "faceIn", 2, I32)
    check_input(geometryIn, "geometryIn", 2, F32)
    Nv, D = vertexIn.shape
    Nf = faceIn.shape[0]
    if D < 3:
        raise RuntimeError("The shape of input vertex should be (Nv, 3+)).")
    if faceIn.shape[1] != 3:
        raise RuntimeError("The shape of input face should be (Nf, 3)).")
    if tuple(geometryIn.shape) != (Nf, 5):
        raise RuntimeError("The shape of input face normals should be (Nf, 5)).")
    dev = same_device(vertexIn, faceIn, geometryIn)
    st = stream_of(vertexIn)
    rowptr, colidx = topology.vertex_csr(faceIn, None, Nv)
    with torch.cuda.device(dev):
        quadric = torch.empty((Nv, 10), dtype=F32, device=dev)
        _lib.call("pmesh_vertex_quadrics", geometryIn.data_ptr(), rowptr.data_ptr(), colidx.data_ptr(), quadric.data_ptr(),
                  Nv, 1 if useArea else 0, st)
        # the unique edges (vi < vj) in ascending order and the boundary edges among them, from the adjacency rows
        evi, evj, bvi, bvj, bface = edge_list(faceIn, rowptr, colidx, Nv)
        nb = bvi.shape[0]
        if wgtBnd > 0 and nb:
            rows = torch.empty((nb, 10), dtype=F32, device=dev)
            _lib.call("pmesh_boundary_quadrics", vertexIn.data_ptr(), geometryIn.data_ptr(), bvi.data_ptr(), bvj.data_ptr(),
                      bface.data_ptr(), rows.data_ptr(), nb, D, 1 if useArea else 0, float(wgtBnd), st)
            # every row goes to both end points: a segmented sum over the end points in ascending edge order
            by_end = torch.sort(torch.cat([bvi, bvj]), stable=True)
            ptr = torch.searchsorted(by_end.values, torch.arange(Nv + 1, dtype=I32, device=dev), out_int32=True)
            quadric = quadric + _segment_row_sum(torch.cat([rows, rows]), ptr, by_end.indices.to(I32), Nv)
    return quadric, evi, evj


def edge_list(faceIn, rowptr, colidx, Nv):
    """Unique edges of the facets from the vertex adjacency (``topology.vertex_csr(faceIn, None, Nv)``), without a sort
    of all facet edges: -> (edge_vi, edge_vj, bnd_vi, bnd_vj, bnd_face) int32; edges with vi < vj in ascending (vi, vj)
    order, the boundary edges (held by one facet side) among them in the same order with the facet that holds each."""
    dev = faceIn.device
    Nf = faceIn.shape[0]
    st = stream_of(faceIn)
    with torch.cuda.device(dev):
        counts = torch.empty((2, Nv), dtype=I32, device=dev)
        flag = torch.zeros(1, dtype=I32, device=dev)
        spill = None
        while True:
            _lib.call("pmesh_edge_list_count", faceIn.data_ptr(), rowptr.data_ptr(), colidx.data_ptr(), Nv, Nf, counts.data_ptr(),
                      spill.data_ptr() if spill is not None else None, flag.data_ptr(), st)
            # (row by row: a scan along the rows of a two-row tensor takes a slow path of the library)
            ends = torch.stack([torch.cumsum(counts[0], 0, dtype=I32), torch.cumsum(counts[1], 0, dtype=I32)])
            n_edges, n_bnd, need = torch.cat([ends[:, -1] if Nv else ends.new_zeros(2), flag]).tolist()
            if not need:
                break
            # some vertex has more than 16 adjacency entries: its candidates are ordered in memory
            spill = torch.empty(12 * Nf, dtype=I32, device=dev)
            flag.zero_()
        offsets = (ends - counts).contiguous()
        evi, evj = torch.empty(n_edges, dtype=I32, device=dev), torch.empty(n_edges, dtype=I32, device=dev)
        bvi, bvj, bface = (torch.empty(n_bnd, dtype=I32, device=dev) for _ in range(3))
        _lib.call("pmesh_edge_list_fill", faceIn.data_ptr(), rowptr.data_ptr(), colidx.data_ptr(), Nv, Nf, offsets.data_ptr(),
                  evi.data_ptr(), evj.data_ptr(), bvi.data_ptr(), bvj.data_ptr(), bface.data_ptr(),
                  spill.data_ptr() if spill is not None else None, st)
    return evi, evj, bvi, bvj, bface


def _segment_row_sum(rows, rowptr, members, n_out):
    """out[v] = sum of rows[members[rowptr[v] .. rowptr[v+1])] in that order (the segmented row sum of the unpooling
    gradient, used here for quadrics)."""
    out = torch.empty((n_out, rows.shape[1]), dtype=F32, device=rows.device)
    _lib.call("pmesh_unpool_bwd", rows.data_ptr(), rowptr.data_ptr(), members.data_ptr(), out.data_ptr(), n_out,
              rows.shape[0], rows.shape[1], stream_of(rows))
    return out


def edge_costs(vertexIn, quadric, edge_vi, edge_vj):
    """Contraction cost (float32) of every candidate edge."""
    check_input(quadric, "quadric", 2, F32)
    check_input(edge_vi, "edge_vi", 1, I32)
    check_input(edge_vj, "edge_vj", 1, I32)
    dev = same_device(vertexIn, quadric, edge_vi, edge_vj)
    with torch.cuda.device(dev):
        cost = torch.empty(edge_vi.shape[0], dtype=F32, device=dev)
        _lib.call("pmesh_edge_costs", vertexIn.data_ptr(), quadric.data_ptr(), edge_vi.data_ptr(), edge_vj.data_ptr(),
                  cost.data_ptr(), edge_vi.shape[0], vertexIn.shape[1], stream_of(vertexIn))
    return cost


def edge_mix(edge_vi, edge_vj):
    """24-bit mix of an edge's end points (int64 tensor): the criterion between candidate edges of EQUAL cost.  The
    flat parts of a scene give most of its edges the same (zero) cost; in (vi, vj) order the greedy clustering would
    sweep them one after the other along the vertex numbering (thousands of dependent steps), in the order of this mix
    the choices are local and the device's rounds settle in a few dozen."""
    m = 0xFFFFFFFF
    h = (((edge_vi.long() * 0x9E3779B1) & m) + ((edge_vj.long() * 0x85EBCA77) & m)) & m
    h = h ^ (h >> 15)
    h = (h * 0x2C1B3C6D) & m
    h = h ^ (h >> 12)
    h = (h * 0x297A2D39) & m
    return (h ^ (h >> 15)) >> 8


def contraction_order(cost, edge_vi, edge_vj, nvIn_cumsum):
    """Order of the candidate edges: by sample, then cost (NaN last), then ``edge_mix``, then (vi, vj) -- the edges come
    in (vi, vj) order, so three stable sorts do it.  returns (permutation, sample of each edge in that order)."""
    # one 64-bit key per edge: the sample number (when there are fewer than 256) on top, the cost as an integer that
    # orders like the float (NaN above everything, -0 = +0) below it, the 24-bit mix at the bottom; the sort is stable,
    # so equal keys stay in (vi, vj) order
    if cost.is_cuda and nvIn_cumsum.shape[0] < 128:
        # the keys in one native pass, the sample read back off the sorted keys
        E = cost.shape[0]
        with torch.cuda.device(cost.device):
            keys = torch.empty(E, dtype=torch.int64, device=cost.device)
            _lib.call("pmesh_contraction_keys", cost.contiguous().data_ptr(), edge_vi.contiguous().data_ptr(),
                      edge_vj.contiguous().data_ptr(), nvIn_cumsum.contiguous().data_ptr(), E, nvIn_cumsum.shape[0],
                      keys.data_ptr(), stream_of(cost))
            by_key = torch.sort(keys, stable=True)
        return by_key.indices, by_key.values >> 56
    bits = (cost + 0.0).view(torch.int32).long()
    ordered = torch.where(bits >= 0, bits, -(bits + 2147483648) - 1)               # negative floats: larger magnitude, lower
    ordered = torch.where(torch.isnan(cost), torch.full_like(ordered, 2147483647), ordered)
    key = ((ordered + 2147483648) << 24) | edge_mix(edge_vi, edge_vj)               # 32 + 24 bits, non-negative
    sample = torch.bucketize(edge_vi.long(), nvIn_cumsum.long(), right=True)
    if nvIn_cumsum.shape[0] < 128:
        perm = torch.sort((sample << 56) | key, stable=True).indices
        return perm, sample[perm]
    by_cost = torch.sort(key, stable=True).indices
    by_sample = torch.sort(sample[by_cost], stable=True)
    return by_cost[by_sample.indices], by_sample.values


_staging = threading.local()


def _pinned(name, n, dtype):
    """A page-locked host buffer of at least ``n`` elements, kept between calls (the edge lists of a scene-scale batch
    are tens of megabytes: through pageable memory their trip to the host costs more than the clustering itself).
    One set of buffers per calling thread: two threads that decimate at once never share one."""
    bufs = _staging.__dict__.setdefault("bufs", {})
    buf = bufs.get(name)
    if buf is None or buf.numel() < n or buf.dtype != dtype:
        buf = torch.empty(max(n, 1), dtype=dtype, pin_memory=True)
        bufs[name] = buf
    return buf[:n]


def cluster_vertices(edge_vi, edge_vj, sample, nvIn_cumsum, nv2Remove, Nv):
    """The two greedy passes per sample on the host (as the reference runs them): -> vt_replace int32 (Nv,) on the host."""
    n = edge_vi.shape[0]
    B = nvIn_cumsum.shape[0]
    # where each sample's edges begin: found on the device, so that the per-edge sample numbers stay there
    bounds_d = torch.searchsorted(sample.contiguous(), torch.arange(B + 1, device=sample.device, dtype=sample.dtype))
    if edge_vi.is_cuda:
        vi_h, vj_h = _pinned("vi", n, I32), _pinned("vj", n, I32)
        vi_h.copy_(edge_vi, non_blocking=True)
        vj_h.copy_(edge_vj, non_blocking=True)
        torch.cuda.current_stream(edge_vi.device).synchronize()
    else:
        vi_h, vj_h = edge_vi.contiguous(), edge_vj.contiguous()
    vi, vj = vi_h.numpy(), vj_h.numpy()
    bounds = bounds_d.cpu().numpy()
    ends = np.asarray(nvIn_cumsum.cpu().numpy(), dtype=np.int64)
    budget = np.asarray(nv2Remove.cpu().numpy(), dtype=np.int64)
    vt_replace = np.zeros(Nv, dtype=np.int32)               # (ordinary memory: the passes access it at random)
    P = ctypes.c_void_p
    jobs = []
    for b in range(len(ends)):
        e0, e1 = int(bounds[b]), int(bounds[b + 1])
        start = int(ends[b - 1]) if b else 0
        if e1 > e0 and budget[b] > 0:
            jobs.append((P(vi.ctypes.data + 4 * e0), P(vj.ctypes.data + 4 * e0), e1 - e0, start, int(ends[b]) - start,
                         int(budget[b]), P(vt_replace.ctypes.data)))
    # the samples are independent and write disjoint ranges of vt_replace: one host thread each
    _lib.call_many("pmesh_cluster_vertices_host", jobs)
    return vt_replace


def cluster_vertices_device(edge_vi, edge_vj, perm, sample, nvIn_cumsum, nv2Remove, Nv, rounds_per_check=8):
    """The same two greedy passes on the device, for all samples at once: -> vt_replace int32 (Nv,) on the device, equal
    to what ``cluster_vertices`` returns for ``edge_vi[perm], edge_vj[perm]``.  ``edge_vi`` / ``edge_vj``: the candidate
    edges in ascending (vi, vj) order, ``perm`` / ``sample``: their contraction order and the sample of each edge in
    that order (``contraction_order``).  Nothing but a status word per ``rounds_per_check`` rounds of the first pass
    crosses to the host.

    First pass: the serial choice "take an edge when both its ends are free" over a total order is the fixed point of
    "an edge that is the first edge with two free ends at BOTH of its ends is taken" (``pmesh_cluster_match``); the
    serial pass stops at its budget, i.e. keeps the lowest-ranked of these edges.  Second pass (only for a sample whose
    first pass left budget, i.e. ended with no edge between two free vertices): a free vertex joins the cluster behind
    its first edge to a covered vertex -- no vertex that joins can enable another one -- again cut by rank.  The kernels
    walk the edges in (vi, vj) order, where neighbouring threads touch neighbouring vertices, and carry each edge's
    rank along."""
    dev = edge_vi.device
    E, B = edge_vi.shape[0], nvIn_cumsum.shape[0]
    st = stream_of(edge_vi)
    with torch.cuda.device(dev):
        vt_replace = torch.zeros(Nv, dtype=I32, device=dev)
        if E == 0 or Nv == 0:
            return vt_replace
        edge_vi, edge_vj = edge_vi.contiguous(), edge_vj.contiguous()
        perm = perm.long().contiguous()
        sample = sample.to(I32).contiguous()                         # of the edges in contraction order
        rank = torch.empty(E, dtype=I32, device=dev)
        sample_e = torch.empty(E, dtype=I32, device=dev)
        _lib.call("pmesh_cluster_ranks", perm.data_ptr(), sample.data_ptr(), E, rank.data_ptr(), sample_e.data_ptr(), st)
        budget = nv2Remove.to(I32).clamp(min=0).contiguous()
        state = torch.zeros(Nv, dtype=I32, device=dev)
        best = torch.empty(Nv, dtype=I32, device=dev)
        chosen = torch.zeros(E, dtype=I32, device=dev)
        status = torch.zeros(4, dtype=I32, device=dev)
        while True:
            _lib.call("pmesh_cluster_match", edge_vi.data_ptr(), edge_vj.data_ptr(), rank.data_ptr(), E, Nv, state.data_ptr(),
                      best.data_ptr(), chosen.data_ptr(), status.data_ptr(), rounds_per_check, st)
            left, bad = status[:2].tolist()
            if bad:
                raise RuntimeError("cluster_vertices: a candidate edge is not (vi < vj) inside the vertex range")
            if not left:
                break
        # where each sample's edges begin in the contraction order
        first = torch.searchsorted(sample, torch.arange(B + 1, device=dev, dtype=I32)).contiguous()
        by_rank = torch.empty(E, dtype=I32, device=dev)

        def cut(flags_e, allowance, with_rest):
            # the flagged edges whose place among their sample's flagged edges (contraction order) is within its allowance
            _lib.call("pmesh_cluster_flags_by_rank", flags_e.data_ptr(), rank.data_ptr(), E, by_rank.data_ptr(), st)
            run = torch.cumsum(by_rank, 0, dtype=I32)
            keep = torch.empty(E, dtype=I32, device=dev)
            open_ = torch.empty(B, dtype=I32, device=dev) if with_rest else None
            rest = torch.empty(B, dtype=I32, device=dev) if with_rest else None
            _lib.call("pmesh_cluster_cut", flags_e.data_ptr(), rank.data_ptr(), sample_e.data_ptr(), run.data_ptr(), first.data_ptr(),
                      allowance.data_ptr(), E, B, keep.data_ptr(), open_.data_ptr() if with_rest else 0,
                      rest.data_ptr() if with_rest else 0, st)
            return keep, open_, rest

        keep, open_, rest = cut(chosen, budget, True)
        _lib.call("pmesh_cluster_contract_pairs", edge_vi.data_ptr(), edge_vj.data_ptr(), keep.data_ptr(), E, vt_replace.data_ptr(), st)
        # second pass where the first one left budget
        first_edge = best
        attaches = chosen
        _lib.call("pmesh_cluster_attach_propose", edge_vi.data_ptr(), edge_vj.data_ptr(), rank.data_ptr(), sample_e.data_ptr(),
                  open_.data_ptr(), E, Nv, vt_replace.data_ptr(), first_edge.data_ptr(), attaches.data_ptr(), st)
        keep2, _, _ = cut(attaches, rest, False)
        pairs = vt_replace.clone()
        _lib.call("pmesh_cluster_attach", edge_vi.data_ptr(), edge_vj.data_ptr(), rank.data_ptr(), keep2.data_ptr(), E,
                  first_edge.data_ptr(), pairs.data_ptr(), vt_replace.data_ptr(), st)
    return vt_replace


def simplify(vertexIn, faceIn, geometryIn, nvIn_cumsum, mfIn_cumsum, nv2Remove, useArea=True, wgtBnd=5.0, own_face=False):
    """One decimation round: the reference's ``mesh_decimation.simplify`` (decimate.cpp:21-89,
    decimate_gpu.cu:618-747).  ``nvIn_cumsum`` / ``mfIn_cumsum``: running totals of vertices / facets per sample.

    returns [vertexOut (Nv, D), faceOut (Nf, 3), isDegenerate (Nf,) bool, vtReplace (Nv,), vtMap (Nv,), nvOut (B,),
    mfOut (B,)]: contracted vertices in the rows of the surviving input vertices (filter with ``vtMap >= 0``), facets
    renumbered to the output vertices (filter with ``~isDegenerate``)."""
    for name, t in (("nvIn", nvIn_cumsum), ("mfIn", mfIn_cumsum), ("nv2Remove", nv2Remove)):
        check_input(t, name, 1, I32)
    useArea, wgtBnd = bool(useArea), float(wgtBnd)
    Nv, D = vertexIn.shape
    dev = vertexIn.device
    quadric, evi, evj = vertex_quadrics(vertexIn, faceIn, geometryIn, useArea, wgtBnd, own_face)
    cost = edge_costs(vertexIn, quadric, evi, evj)
    perm, sample = contraction_order(cost, evi, evj, nvIn_cumsum)
    if evi.is_cuda and os.environ.get("PMESH_DECIMATE_HOST_CLUSTERING") != "1":
        vt_replace = cluster_vertices_device(evi, evj, perm, sample, nvIn_cumsum, nv2Remove, Nv)
    else:
        vt_replace = torch.from_numpy(cluster_vertices(evi[perm], evj[perm], sample, nvIn_cumsum, nv2Remove, Nv)).to(dev)
    Nf = faceIn.shape[0]
    B = nvIn_cumsum.shape[0]
    st = stream_of(vertexIn)
    with torch.cuda.device(dev):
        # facets over the representatives, collapsed facets, vertices that keep a facet; then the output numbering from
        # the running totals: vertices that keep a facet are numbered in order, the others get -1
        new_face = torch.empty((Nf, 3), dtype=I32, device=dev)
        degenerate = torch.empty(Nf, dtype=torch.bool, device=dev)
        alive = torch.empty(Nf, dtype=I32, device=dev)
        kept = torch.empty(Nv, dtype=I32, device=dev)
        faceIn = faceIn.contiguous()
        _lib.call("pmesh_simplify_faces", faceIn.data_ptr(), vt_replace.data_ptr(), Nf, Nv, new_face.data_ptr(),
                  degenerate.data_ptr(), alive.data_ptr(), kept.data_ptr(), st)
        kept_total = torch.cumsum(kept, 0, dtype=I32)
        alive_total = torch.cumsum(alive, 0, dtype=I32)
        vt_map = torch.empty(Nv, dtype=I32, device=dev)
        face_out = torch.empty((Nf, 3), dtype=I32, device=dev)
        _lib.call("pmesh_simplify_renumber", new_face.data_ptr(), degenerate.data_ptr(), kept.data_ptr(), kept_total.data_ptr(),
                  Nf, Nv, vt_map.data_ptr(), face_out.data_ptr(), st)

        def per_sample(total, ends):
            # counts per sample from a running total read at the samples' ends
            at = torch.cat([total.new_zeros(1), total])[ends.long().clamp(0, total.shape[0])]
            return (at - torch.cat([at.new_zeros(1), at[:-1]])).to(I32)

        nv_out = per_sample(kept_total, nvIn_cumsum)
        mf_out = per_sample(alive_total, mfIn_cumsum)
        # contracted position = mean of the cluster's vertices (all D columns) in the row of its representative; rows of
        # contracted vertices stay zero (decimate_gpu.cu:401-441): the average pooling op over a map that sends every
        # representative to its own row
        own_row = torch.where(vt_replace >= 0, torch.arange(Nv, dtype=I32, device=dev), torch.full_like(vt_replace, -1))
        with topology.trusted_indices():                  # (maps made by the kernels above)
            vertex_out = (mesh_pool3d.avg_forward(vertexIn, vt_replace, own_row, torch.empty((Nv, 1), dtype=F32, device=dev))
                          if Nv else torch.zeros((0, D), dtype=F32, device=dev))
    return [vertex_out, face_out, degenerate, vt_replace, vt_map, nv_out, mf_out]


def mesh_decimation_(vertexIn, faceIn, geometryIn, nvIn, mfIn, nvOut, useArea=True, wgtBnd=5):
    """Decimate every sample of the batch to (about) ``nvOut`` vertices (decimate.py:5-52): rounds of ``simplify``
    until no sample has vertices left to remove, the rounds' cluster maps composed with ``combine_clusters_``.

    returns (vertexOut, faceOut, geometryOut, nvOut, mfOut, vtReplace, vtMap) with vtReplace / vtMap over the INPUT
    vertices: the index maps the pooling / unpooling ops and the strided facet2vertex take."""
    dev = vertexIn.device
    nv2Remove = (nvIn - nvOut).to(I32)
    repIn = torch.zeros(vertexIn.shape[0], dtype=I32, device=dev)
    mapIn = torch.arange(vertexIn.shape[0], dtype=I32, device=dev)
    left = int(nv2Remove.max()) if nv2Remove.numel() else 0
    rounds = 0
    while left > 0:
        nv_cum = torch.cumsum(nvIn, 0, dtype=I32)
        mf_cum = torch.cumsum(mfIn, 0, dtype=I32)
        # (from the second round on the facets are the round before's output: valid by construction, not checked again)
        vertexOut, faceOut, isDegenerate, repOut, mapOut, nvOut, mfOut = simplify(
            vertexIn, faceIn, geometryIn, nv_cum, mf_cum, nv2Remove.contiguous(), useArea, wgtBnd, own_face=rounds > 0)
        rounds += 1
        removed = nvIn - nvOut
        still = (nv2Remove - removed).to(I32)
        # what the host needs of this round, in one transfer: did it remove anything, the sizes of the next round's
        # arrays, and whether a sample still has vertices to remove
        most, nv_total, mf_total, left = torch.stack([removed.max(), nvOut.sum(), mfOut.sum(), still.max()]).tolist()
        if most <= 0:
            break                                     # nothing left that can be contracted (no candidate edges)
        faceIn = _rows_where(faceOut, ~isDegenerate, mf_total)
        vertexIn = _rows_where(vertexOut, mapOut >= 0, nv_total)
        with topology.trusted_indices():
            geometryIn = compute_triangle_geometry_(vertexIn, faceIn)
            repIn, mapIn = combine_clusters_(repIn, mapIn, repOut, mapOut)
        nv2Remove = still
        nvIn, mfIn = nvOut, mfOut
    return vertexIn, faceIn, geometryIn, nvIn, mfIn, repIn, mapIn


def _rows_where(rows, mask, count):
    """rows[mask] when the number of selected rows is known already (no second trip to the host for it)."""
    if hasattr(torch, "nonzero_static"):
        return rows.index_select(0, torch.nonzero_static(mask, size=int(count)).squeeze(1))
    return rows[mask].contiguous()
