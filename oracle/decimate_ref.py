"""TEST INFRASTRUCTURE ONLY: numpy restatement of one round of the reference's quadric-error mesh decimation
(picasso/mesh/pi_modules/source/decimate_gpu.cu, decimate.cpp:21-89) and of the loop around it
(picasso/mesh/pi_modules/decimate.py:5-52).  The product never imports this module.

The reference's result depends on the order of float atomics and on how unstable sorts leave ties, so "the
reference's output" is a set, not a value.  This restatement picks one member of that set by giving every step an
order (marked DETERMINISTIC below); the arithmetic follows the reference line by line and is dtype generic
(float64 as the parity answer, float32 to see what single precision costs).

What pins it (tests/test_oracle.py): ``rref_solve`` against numpy.linalg on well-conditioned systems and against
hand-made singular ones; vertex / boundary quadrics through the geometry they encode (zero error on the planes,
hand-counted weights); the clustering passes against hand cases and the invariants the pooling ops rely on; a
whole round on closed and open meshes through its counts and maps.  No fixture of the reference holds a decimation
output, so nothing here is pinned against recorded reference outputs: the choice among equal-cost edges is
this restatement's own and documented as such.

Paths cited are relative to picasso/mesh/pi_modules/source/ of the reference.
"""
import numpy as np

AREA_MAGNITUDE = 100.0                      # decimate_gpu.cu:16
RREF_EPS = 2.220446049250313e-16            # decimate_gpu.cu:13 (a float literal there: rounds to float32)
RCOND_EPS = 1e-6                            # decimate_gpu.cu:14


def plane_quadrics(normal, d):
    """(n, 10) entries q11 q12 q13 q22 q23 q33 q14 q24 q34 q44 of [n; d][n; d]^T (decimate_gpu.cu:204-212)."""
    n0, n1, n2 = normal[:, 0], normal[:, 1], normal[:, 2]
    return np.stack([n0 * n0, n0 * n1, n0 * n2, n1 * n1, n1 * n2, n2 * n2, n0 * d, n1 * d, n2 * d, d * d], 1)


def unique_edges(face, nv):
    """Edges of the facets as (lower, higher) vertex pairs (decimate_gpu.cu:250-297), unique, in ascending (vi, vj)
    order; for each the number of facets it belongs to and the first (lowest 3 f + slot) facet that holds it.
    DETERMINISTIC: the reference sorts with an unstable comparator and takes whichever duplicate comes first."""
    f = face.astype(np.int64)
    a = np.stack([f[:, 0], f[:, 0], f[:, 1]], 1).reshape(-1)
    b = np.stack([f[:, 1], f[:, 2], f[:, 2]], 1).reshape(-1)
    key = np.minimum(a, b) * nv + np.maximum(a, b)
    order = np.argsort(key, kind="stable")
    ukey, first, counts = np.unique(key[order], return_index=True, return_counts=True)
    return ukey // nv, ukey % nv, counts, order[first] // 3


def vertex_quadrics(vertex, face, geometry, use_area=True, wgt_bnd=5.0, dtype=np.float64):
    """Vertex quadrics from the facets (decimate_gpu.cu:220-247) plus the boundary-edge planes (:300-362).
    returns (quadric (Nv, 10), edge_vi, edge_vj): candidate edges vi < vj in ascending order.
    DETERMINISTIC: facet terms in ascending (facet, corner) order, then boundary terms in ascending edge order,
    first the edges a vertex starts, then those it ends."""
    vertex = np.asarray(vertex, dtype)
    geometry = np.asarray(geometry, dtype)
    nv = vertex.shape[0]
    Q = plane_quadrics(geometry[:, :3], geometry[:, 3])
    w = geometry[:, 4] * dtype(AREA_MAGNITUDE) / dtype(3) if use_area else np.ones(face.shape[0], dtype)
    quadric = np.zeros((nv, 10), dtype)
    np.add.at(quadric, face.reshape(-1).astype(np.int64), np.repeat(Q * w[:, None], 3, 0))
    vi, vj, counts, first_face = unique_edges(face, nv)
    ok = vi != vj
    if wgt_bnd > 0:
        bnd = (counts == 1) & ok
        bi, bj, bf = vi[bnd], vj[bnd], first_face[bnd]
        pi, pj, n = vertex[bi, :3], vertex[bj, :3], geometry[bf, :3]
        dx = pj - pi
        b = np.cross(n, dx).astype(dtype)                              # in the facet's plane, across the edge
        length = np.maximum(np.sqrt((b * b).sum(1)), dtype(1e-20))
        b = b / length[:, None]
        d = -(b * pi).sum(1)
        wb = (dx * dx).sum(1) * dtype(AREA_MAGNITUDE) * dtype(wgt_bnd) if use_area else np.full(len(bi), wgt_bnd, dtype)
        rows = plane_quadrics(b, d) * wb[:, None]
        extra = np.zeros_like(quadric)
        np.add.at(extra, bi, rows)
        np.add.at(extra, bj, rows)
        quadric = quadric + extra
    return quadric, vi[ok].astype(np.int32), vj[ok].astype(np.int32)


def rref_solve(A, b, dtype=np.float64):
    """RrefDim3 (decimate_gpu.cu:79-193) for a batch: reduced row echelon form of [A | b | I] with partial pivoting,
    columns whose pivot is <= eps * 7 * |A|_inf zeroed and skipped.  returns (x = -"A^-1 b", rcond)."""
    A = np.asarray(A, dtype)
    n = A.shape[0]
    M = np.zeros((n, 3, 7), dtype)
    M[:, :, :3] = A
    M[:, :, 3] = np.asarray(b, dtype)
    M[:, [0, 1, 2], [4, 5, 6]] = 1
    norm_a = np.abs(A).sum(2).max(1)
    tol = dtype(np.float32(RREF_EPS)) * dtype(7) * norm_a
    i = np.zeros(n, np.int64)
    rows = np.arange(3)[None, :]
    every = np.arange(n)
    for j in range(7):
        active = i < 3
        below = rows >= i[:, None]
        mag = np.where(below, np.abs(M[:, :, j]), -1)
        k = mag.argmax(1)                                             # first largest, as the strict "<" leaves it
        p = mag[every, k]
        skip = active & (p <= tol)
        use = active & (p > tol)
        M[:, :, j] = np.where(skip[:, None] & below, 0, M[:, :, j])
        if use.any():
            u = np.nonzero(use)[0]
            iu, ku = i[u], k[u]
            Mi, Mk = M[u, iu].copy(), M[u, ku].copy()                 # columns left of j are zero in both rows
            M[u, ku] = Mi
            M[u, iu] = Mk / Mk[:, j:j + 1]
            piv = M[u, iu]
            for r in range(3):
                other = u[iu != r]
                M[other, r] = M[other, r] - M[other, r, j:j + 1] * piv[iu != r]
            i[u] += 1
    x = -M[:, :, 3]
    norm_inv = np.abs(M[:, :, 4:]).sum(2).max(1)
    with np.errstate(divide="ignore"):
        rcond = dtype(1) / (norm_a * norm_inv)
    return x, rcond


def quadric_error(x, Q):
    """x^T A x + 2 b.x + c in the reference's association (decimate_gpu.cu:190-198)."""
    A = Q[:, [0, 1, 2, 1, 3, 4, 2, 4, 5]].reshape(-1, 3, 3)
    # every product and sum written out, left to right: in float32 the result is then a function of the inputs alone
    # (an einsum may fuse or reorder), which is what a device kernel can be compared with bit for bit
    x0, x1, x2 = x[:, 0], x[:, 1], x[:, 2]
    xa = [x0 * A[:, 0, c] + x1 * A[:, 1, c] + x2 * A[:, 2, c] for c in range(3)]
    return (xa[0] * x0 + xa[1] * x1 + xa[2] * x2) + (x0 * Q[:, 6] + x1 * Q[:, 7] + x2 * Q[:, 8]) * 2 + Q[:, 9]


def edge_costs(vertex, quadric, edge_vi, edge_vj, dtype=np.float64, return_rcond=False):
    """Cost of contracting every candidate edge (decimate_gpu.cu:365-404)."""
    vertex = np.asarray(vertex, dtype)
    Q = np.asarray(quadric, dtype)[edge_vi] + np.asarray(quadric, dtype)[edge_vj]
    A = Q[:, [0, 1, 2, 1, 3, 4, 2, 4, 5]].reshape(-1, 3, 3)
    x, rcond = rref_solve(A, Q[:, 6:9], dtype)
    at_opt = quadric_error(x, Q)
    at_end = np.minimum(quadric_error(vertex[edge_vi, :3], Q), quadric_error(vertex[edge_vj, :3], Q))
    cost = np.where(rcond > dtype(np.float32(RCOND_EPS)), at_opt, at_end)
    return (cost, rcond) if return_rcond else cost


def edge_mix(edge_vi, edge_vj):
    """24-bit mix of an edge's end points: what orders candidate edges of EQUAL cost.  Flat regions give thousands of
    edges the same (zero) cost; ordered by (vi, vj) the greedy clustering would sweep them one after the other along the
    vertex numbering, ordered by this mix their choices are local (and can be made in parallel rounds)."""
    m = 0xFFFFFFFF
    h = ((edge_vi.astype(np.int64) * 0x9E3779B1) & m) + ((edge_vj.astype(np.int64) * 0x85EBCA77) & m) & m
    h &= m
    h ^= h >> 15
    h = (h * 0x2C1B3C6D) & m
    h ^= h >> 12
    h = (h * 0x297A2D39) & m
    h ^= h >> 15
    return h >> 8                              # 24 bits: cost, mix and a sample number below 256 share one 64-bit key


def contraction_order(cost, edge_vi, edge_vj, nv_cumsum):
    """DETERMINISTIC: candidate edges by (sample, cost, mix(vi, vj), vi, vj), NaN costs last, -0 = +0; the reference
    sorts each sample's costs with thrust::sort_by_key and leaves ties to it (decimate_gpu.cu:682-705).  The edges come
    in ascending (vi, vj) order, so stable sorts keep that as the last criterion.  returns (perm, sample[perm])."""
    by_mix = np.argsort(edge_mix(edge_vi, edge_vj), kind="stable")
    by_cost = by_mix[np.argsort(np.asarray(cost)[by_mix], kind="stable")]
    sample = np.searchsorted(np.asarray(nv_cumsum, np.int64), edge_vi[by_cost].astype(np.int64), side="right")
    by_sample = np.argsort(sample, kind="stable")
    return by_cost[by_sample], sample[by_sample]


def cluster_vertices(edge_vi, edge_vj, vt_start, vt_num, n_remove, vt_replace):
    """clusterVertices (decimate_gpu.cu:561-614) over one sample's edges in contraction order, in place.

    Two departures, both needed for maps the pooling ops can follow: in the second pass an edge joins its free end
    to the cluster of its covered end whichever position the two are in (the reference swaps only for a seed vertex
    in second position and can otherwise contract a covered vertex a second time, which leaves a chain), and a
    vertex is never contracted into vertex 0 (its negative cannot be told from "not contracted")."""
    covered = np.zeros(vt_num, np.int8)
    removed = 0
    for vi, vj in zip(edge_vi.tolist(), edge_vj.tolist()):
        if removed >= n_remove:
            break
        if vi != vj and vj != 0 and not covered[vi - vt_start] and not covered[vj - vt_start]:
            vt_replace[vi] = -vj
            vt_replace[vj] += 1
            covered[vi - vt_start] = covered[vj - vt_start] = 1
            removed += 1
    for a, b in zip(edge_vi.tolist(), edge_vj.tolist()):
        if removed >= n_remove:
            break
        ca, cb = covered[a - vt_start] != 0, covered[b - vt_start] != 0
        if ca == cb or a == b:
            continue
        if cb:
            a, b = b, a
        if vt_replace[a] < 0:
            a = -int(vt_replace[a])
        if a == 0:
            continue
        vt_replace[b] = -a
        vt_replace[a] += 1
        covered[b - vt_start] = 2
        removed += 1
    return removed


def simplify(vertex, face, geometry, nv_cumsum, mf_cumsum, nv2remove, use_area=True, wgt_bnd=5.0, dtype=np.float64,
             cost=None):
    """One round (decimate.cpp:21-89, decimate_gpu.cu:618-747).  ``cost`` replaces the edge costs computed here (to
    check the integer stages against a device that computed its own in float32).
    returns (vertex_out, face_out, degenerate, vt_replace, vt_map, nv_out, mf_out)."""
    vertex = np.asarray(vertex, dtype)
    nv = vertex.shape[0]
    quadric, evi, evj = vertex_quadrics(vertex, face, geometry, use_area, wgt_bnd, dtype)
    if cost is None:
        cost = edge_costs(vertex, quadric, evi, evj, dtype)
    perm, sample = contraction_order(np.asarray(cost), evi, evj, nv_cumsum)
    vt_replace = np.zeros(nv, np.int32)
    bounds = np.searchsorted(sample, np.arange(len(nv_cumsum) + 1))
    for b in range(len(nv_cumsum)):
        start = int(nv_cumsum[b - 1]) if b else 0
        e = perm[bounds[b]:bounds[b + 1]]
        cluster_vertices(evi[e], evj[e], start, int(nv_cumsum[b]) - start, int(nv2remove[b]), vt_replace)
    ids = np.arange(nv)
    rep = np.where(vt_replace < 0, -vt_replace.astype(np.int64), ids)
    new_face = rep[face.astype(np.int64)]
    degenerate = (new_face[:, 0] == new_face[:, 1]) | (new_face[:, 0] == new_face[:, 2]) | (new_face[:, 1] == new_face[:, 2])
    kept = np.zeros(nv, np.int64)
    kept[new_face[~degenerate].reshape(-1)] = 1                        # decimate_gpu.cu:487-496
    vt_map = np.where(kept > 0, np.cumsum(kept) - 1, -1).astype(np.int32)   # :519-531
    face_out = np.where(degenerate[:, None], new_face, vt_map[new_face]).astype(np.int32)   # :533-549
    sample_v = np.searchsorted(np.asarray(nv_cumsum, np.int64), ids, side="right")
    sample_f = np.searchsorted(np.asarray(mf_cumsum, np.int64), np.arange(face.shape[0]), side="right")
    B = len(nv_cumsum)
    nv_out = np.bincount(sample_v[kept > 0], minlength=B)[:B].astype(np.int32)
    mf_out = np.bincount(sample_f[~degenerate], minlength=B)[:B].astype(np.int32)
    # mean of each cluster in the representative's row, zero rows for contracted vertices (:401-441)
    total = np.zeros_like(vertex)
    np.add.at(total, rep, vertex)
    vertex_out = np.where((vt_replace >= 0)[:, None], total / (np.maximum(vt_replace, 0) + 1)[:, None].astype(dtype), 0)
    return vertex_out, face_out, degenerate, vt_replace, vt_map, nv_out, mf_out


def triangle_geometry(vertex, face, dtype=np.float64):
    """(Nf, 5): unit normal, d = -n.v0, area (picasso/mesh/pi_modules/decimate.py:70-85)."""
    v = np.asarray(vertex, dtype)[:, :3]
    f = face.astype(np.int64)
    raw = np.cross(v[f[:, 1]] - v[f[:, 0]], v[f[:, 2]] - v[f[:, 0]])
    length = np.sqrt((raw * raw).sum(1, keepdims=True))
    n = raw / (length + dtype(1e-10))
    d = -(n * v[f[:, 0]]).sum(1, keepdims=True)
    return np.concatenate([n, d, length / 2], 1)


def combine_clusters(rep_a, map_a, rep_b, map_b):
    """decimate_gpu.cu:750-810: the restatement in torch_ref.py over numpy arrays."""
    import torch
    from . import torch_ref
    out = torch_ref.combine_clusters(*(torch.from_numpy(np.ascontiguousarray(a, np.int32)) for a in (rep_a, map_a, rep_b, map_b)))
    return out[0].numpy(), out[1].numpy()


def mesh_decimation(vertex, face, geometry, nv_in, mf_in, nv_out, use_area=True, wgt_bnd=5.0, dtype=np.float64):
    """The loop of picasso/mesh/pi_modules/decimate.py:5-52."""
    vertex = np.asarray(vertex, dtype)
    nv2remove = (np.asarray(nv_in) - np.asarray(nv_out)).astype(np.int64)
    rep_in = np.zeros(vertex.shape[0], np.int32)
    map_in = np.arange(vertex.shape[0], dtype=np.int32)
    nv_in, mf_in = np.asarray(nv_in), np.asarray(mf_in)
    while (nv2remove > 0).any():
        out = simplify(vertex, face, geometry, np.cumsum(nv_in), np.cumsum(mf_in), nv2remove, use_area, wgt_bnd, dtype)
        vertex_out, face_out, degenerate, rep_out, map_out, nv_o, mf_o = out
        removed = nv_in - nv_o
        if not (removed > 0).any():
            break
        face = face_out[~degenerate]
        vertex = vertex_out[map_out >= 0]
        geometry = triangle_geometry(vertex, face, dtype)
        nv2remove = nv2remove - removed
        rep_in, map_in = combine_clusters(rep_in, map_in, rep_out, map_out)
        nv_in, mf_in = nv_o, mf_o
    return vertex, face, geometry, nv_in, mf_in, rep_in, map_in
