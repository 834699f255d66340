"""Pins oracle/decimate_ref.py without a GPU.

The reference holds no decimation fixture, so each function is pinned by what the geometry and the algebra fix:
the 3 x 3 solver against numpy.linalg and hand-made singular systems, quadrics through the planes they encode and
hand-counted weights, the clustering against hand cases, a brute-force statement of its two passes and the
invariants the pooling ops rely on, a whole round through counts, maps and the surviving facets.
"""
import numpy as np
import pytest

from oracle import decimate_ref as D
from util import mesh_case


def case(name, seed=0):
    v, f = mesh_case(name, seed)
    v = np.asarray(v, np.float64)[:, :3]
    return v, f, D.triangle_geometry(v, f)


# ------------------------------------------------------------------ solver
def test_rref_solve_matches_linalg_on_regular_systems():
    rng = np.random.default_rng(0)
    B = rng.normal(size=(400, 3, 3))
    A = B @ B.transpose(0, 2, 1) + 0.05 * np.eye(3)                    # symmetric positive definite, as quadrics are
    b = rng.normal(size=(400, 3))
    x, rcond = D.rref_solve(A, b)
    want = -np.linalg.solve(A, b[:, :, None])[:, :, 0]
    assert np.abs(x - want).max() < 1e-9 * np.abs(want).max()
    inv = np.linalg.inv(A)
    want_rcond = 1 / (np.abs(A).sum(2).max(1) * np.abs(inv).sum(2).max(1))
    assert np.allclose(rcond, want_rcond, rtol=1e-9)
    # needs pivoting: zero on the diagonal
    P = np.array([[[0., 2, 0], [1, 0, 0], [0, 0, 4]]])
    x, rcond = D.rref_solve(P, np.array([[2., 3, 4]]))
    assert np.allclose(x, [[-3, -1, -1]])
    assert np.isclose(rcond[0], 1 / (4 * 1))


def test_rref_solve_singular_systems():
    # one plane z = 0 (rank 1): the only pivot is the third column; rows of the inverse block do not form an inverse,
    # and the reciprocal condition number says so for a rank-2 matrix with a tiny third direction
    A = np.array([np.diag([0., 0, 1]), np.diag([1., 1, 1e-9])])
    x, rcond = D.rref_solve(A, np.array([[0., 0, 0.5], [1., 2, 0]]))
    assert np.allclose(x[0], [-0.5, 0, 0])          # the pivot row moved to the top: x is not a solution in this case
    assert rcond[1] < 1e-8 and np.allclose(x[1], [-1, -2, 0])
    # all-zero matrix: every column skipped, no division by zero, rcond not finite or zero
    x, rcond = D.rref_solve(np.zeros((1, 3, 3)), np.zeros((1, 3)))
    assert np.all(x == 0) and not (rcond[0] > D.RCOND_EPS and np.isfinite(rcond[0]))
    # float32 mode keeps float32 throughout
    x32, r32 = D.rref_solve(np.eye(3, dtype=np.float32)[None], np.ones((1, 3), np.float32), np.float32)
    assert x32.dtype == np.float32 and r32.dtype == np.float32 and np.allclose(x32, -1)


# ------------------------------------------------------------------ quadrics
def test_vertex_quadrics_hand_case_single_triangle():
    # the triangle (0,0,1) (2,0,1) (0,2,1): plane z = 1, area 2 -> weight 2 * 100 / 3 per corner; three boundary edges
    v = np.array([[0., 0, 1], [2, 0, 1], [0, 2, 1]])
    f = np.array([[0, 1, 2]], np.int32)
    g = D.triangle_geometry(v, f)
    assert np.allclose(g, [[0, 0, 1, -1, 2]])
    q, vi, vj = D.vertex_quadrics(v, f, g, use_area=True, wgt_bnd=0)
    w = 200 / 3
    want = np.zeros(10)
    want[[5, 8, 9]] = [w, -w, w]                                       # n = (0,0,1), d = -1: q33, q34, q44
    assert np.allclose(q, want[None].repeat(3, 0))
    assert (vi.tolist(), vj.tolist()) == ([0, 0, 1], [1, 2, 2])
    q1, _, _ = D.vertex_quadrics(v, f, g, use_area=False, wgt_bnd=0)
    assert np.allclose(q1[0], [0, 0, 0, 0, 0, 1, 0, 0, -1, 1])
    # boundary planes, unit weights times 5: edge (0,1) lies on y = 0, edge (0,2) on x = 0, edge (1,2) on x + y = 2
    qb, _, _ = D.vertex_quadrics(v, f, g, use_area=False, wgt_bnd=5.0)
    extra = qb - q1
    assert np.allclose(extra[0], [5, 0, 0, 5, 0, 0, 0, 0, 0, 0])                         # x^2 + y^2
    assert np.allclose(extra[1], [2.5, 2.5, 0, 5 + 2.5, 0, 0, -5, -5, 0, 10])            # y^2 + (x + y - 2)^2 / 2
    # with areas the boundary weight is |edge|^2 * 100 * wgt
    qa, _, _ = D.vertex_quadrics(v, f, g, use_area=True, wgt_bnd=5.0)
    assert np.isclose((qa - q)[0][0], 4 * 100 * 5) and np.isclose((qa - q)[0][3], 4 * 100 * 5)


@pytest.mark.parametrize("name", ["tetra", "octa", "sphere2", "torus", "room_small"])
def test_vertex_quadric_vanishes_on_its_own_vertex(name):
    """Every plane in a vertex's quadric passes through that vertex: facets it belongs to and the perpendicular planes
    through boundary edges it ends."""
    v, f, g = case(name)
    q, vi, vj = D.vertex_quadrics(v, f, g, True, 5.0)
    err = D.quadric_error(v, q)
    scale = np.abs(q).sum(1) * (1 + (v * v).sum(1))
    assert np.all(np.abs(err) <= 1e-12 * np.maximum(scale, 1e-30))
    assert np.all(vi < vj)
    key = vi.astype(np.int64) * len(v) + vj
    assert np.all(np.diff(key) > 0)                                    # unique and ascending
    want = {tuple(sorted(e)) for t in f.tolist() for e in ((t[0], t[1]), (t[0], t[2]), (t[1], t[2])) if e[0] != e[1]}
    assert set(zip(vi.tolist(), vj.tolist())) == want


def test_closed_mesh_has_no_boundary_terms_and_open_mesh_has():
    v, f, g = case("sphere1")
    assert np.array_equal(D.vertex_quadrics(v, f, g, True, 5.0)[0], D.vertex_quadrics(v, f, g, True, 0.0)[0])
    v, f, g = case("grid2")
    a, b = D.vertex_quadrics(v, f, g, True, 5.0)[0], D.vertex_quadrics(v, f, g, True, 0.0)[0]
    interior = 4                                                       # centre of the 3 x 3 vertex grid
    changed = np.abs(a - b).sum(1) > 0
    assert not changed[interior] and changed.sum() == 8
    # the boundary planes are perpendicular to the patch, so points of the patch's plane on the boundary line stay free
    _, vi, vj, = D.vertex_quadrics(v, f, g, True, 5.0)
    extra = a - b
    assert np.all(np.abs(D.quadric_error(v, extra)) < 1e-9)


# ------------------------------------------------------------------ edge costs
def test_edge_costs_closed_forms():
    # a flat patch through the origin: every quadric is the same plane with d = 0, so b = 0, c = 0 and any x costs 0
    gx, gy = np.meshgrid(np.arange(3.0), np.arange(3.0), indexing="ij")
    v = np.stack([gx.ravel(), gy.ravel(), np.zeros(9)], 1)
    cell = lambda i, j: [[3 * i + j, 3 * i + j + 3, 3 * i + j + 1], [3 * i + j + 1, 3 * i + j + 3, 3 * i + j + 4]]
    f = np.array([t for i in range(2) for j in range(2) for t in cell(i, j)], np.int32)
    g = D.triangle_geometry(v, f)
    assert np.allclose(g[:, :4], [0, 0, 1, 0])
    q, vi, vj = D.vertex_quadrics(v, f, g, True, 0.0)
    cost, rcond = D.edge_costs(v, q, vi, vj, return_rcond=True)
    assert np.all(np.abs(cost) < 1e-12)
    # The same patch lifted to z = 2.  The routine skips the two empty columns and moves the only pivot row to the top,
    # then finds its other two pivots in the identity block: the "inverse" block ends as rows (0, 0, 1/w), (1, 0, 0),
    # (0, 1, 0), the reciprocal condition number comes out as 1 / (w * max(1, 1/w)), far above the 1e-6 threshold,
    # and the z-solution lands in x's FIRST slot: x = (2, 0, 0), whose error is w * 2^2 and not 0.  This is what the
    # reference's RrefDim3 does with a rank-deficient quadric (decimate_gpu.cu:116-171); restated, not repaired.
    v2 = v + np.array([0, 0, 2.0])
    g2 = D.triangle_geometry(v2, f)
    q2, _, _ = D.vertex_quadrics(v2, f, g2, True, 0.0)
    cost2, rcond2 = D.edge_costs(v2, q2, vi, vj, return_rcond=True)
    w = (q2[vi] + q2[vj])[:, 5]
    assert np.allclose(rcond2, 1 / np.maximum(w, 1)) and np.allclose(cost2, 4 * w)
    # regular quadrics: cost = c - b^T A^-1 b
    v, f, g = case("sphere2")
    q, vi, vj = D.vertex_quadrics(v, f, g, True, 5.0)
    cost, rcond = D.edge_costs(v, q, vi, vj, return_rcond=True)
    Q = q[vi] + q[vj]
    A = Q[:, [0, 1, 2, 1, 3, 4, 2, 4, 5]].reshape(-1, 3, 3)
    want = Q[:, 9] - np.einsum("ni,ni->n", Q[:, 6:9], np.linalg.solve(A, Q[:, 6:9, None])[:, :, 0])
    assert np.all(rcond > D.RCOND_EPS)
    assert np.abs(cost - want).max() < 1e-9 * np.abs(Q[:, 9]).max()
    assert np.all(cost > -1e-9) and cost.max() > 1e-6                  # a sum of squared distances, curved surface
    # the minimiser beats both end points
    ends = np.minimum(D.quadric_error(v[vi], Q), D.quadric_error(v[vj], Q))
    assert np.all(cost <= ends + 1e-9)


def test_edge_costs_float32_mode_is_close():
    v, f, g = case("room_small")
    q, vi, vj = D.vertex_quadrics(v, f, g, True, 5.0)
    c64, r64 = D.edge_costs(v, q, vi, vj, return_rcond=True)
    q32, _, _ = D.vertex_quadrics(v, f, g, True, 5.0, np.float32)
    assert q32.dtype == np.float32 and np.abs(q32 - q).max() <= 1e-5 * np.abs(q).max()
    c32 = D.edge_costs(v, q32, vi, vj, np.float32)
    clear = (r64 > 10 * D.RCOND_EPS) | (r64 < 0.1 * D.RCOND_EPS)
    Q = q[vi] + q[vj]
    scale = np.abs(Q).sum(1) * (1 + np.maximum((v[vi] ** 2).sum(1), (v[vj] ** 2).sum(1)))
    assert clear.sum() > 0.5 * len(clear)
    assert np.all(np.abs(c32 - c64)[clear] <= 1e-3 * scale[clear])


# ------------------------------------------------------------------ order and clustering
def _mix_by_hand(a, b):
    """edge_mix with Python integers and explicit 32-bit masks."""
    m = (1 << 32) - 1
    h = (a * 0x9E3779B1 + b * 0x85EBCA77) & m
    h ^= h >> 15
    h = (h * 0x2C1B3C6D) & m
    h ^= h >> 12
    h = (h * 0x297A2D39) & m
    return (h ^ (h >> 15)) >> 8


def test_contraction_order_is_total():
    """(sample, cost, mix, vi, vj): samples apart, costs ascending with NaN last and -0 = +0, equal costs by the mix of
    their end points (checked against integer arithmetic by hand), equal mixes by (vi, vj)."""
    rng = np.random.default_rng(4)
    n = 400
    vi = np.sort(rng.integers(0, 8, n)).astype(np.int32)                # samples: vertices 0-3, 4-7
    vj = (vi + rng.integers(1, 2 ** 30, n)).astype(np.int32)
    key = np.argsort(vi.astype(np.int64) * 2 ** 31 + vj, kind="stable")  # the callers' ascending (vi, vj) order
    vi, vj = vi[key], vj[key]
    cost = rng.choice([0.0, -0.0, 0.25, 0.25, 1e-9, np.nan, 3.0], n)
    perm, sample = D.contraction_order(cost, vi, vj, np.array([4, 8]))
    assert sorted(perm.tolist()) == list(range(n))
    assert np.array_equal(sample, (vi[perm] >= 4).astype(int)) and np.all(np.diff(sample) >= 0)
    mix = [_mix_by_hand(int(a), int(b)) for a, b in zip(vi, vj)]
    assert np.array_equal(D.edge_mix(vi, vj), np.array(mix, np.int64))
    assert len(set(mix)) > 0.95 * len(set(zip(vi.tolist(), vj.tolist()))) and max(mix) < 2 ** 24     # it does spread the pairs
    for x, y in zip(perm[:-1].tolist(), perm[1:].tolist()):
        if (vi[x] >= 4) != (vi[y] >= 4):
            continue
        cx, cy = cost[x], cost[y]
        if np.isnan(cx):
            assert np.isnan(cy)
        elif not np.isnan(cy) and cx != cy:
            assert cx < cy
        elif not np.isnan(cy):
            assert (mix[x], vi[x], vj[x]) < (mix[y], vi[y], vj[y])
    # a case small enough to read: costs decide, then the mix (edge (2, 3) before (1, 2) because its mix is smaller)
    vi3, vj3 = np.array([0, 1, 2], np.int32), np.array([1, 2, 3], np.int32)
    order3, _ = D.contraction_order(np.array([0.5, 0.1, 0.1]), vi3, vj3, np.array([4]))
    first, second = ((1, 2), (2, 3)) if _mix_by_hand(1, 2) < _mix_by_hand(2, 3) else ((2, 3), (1, 2))
    assert [(int(vi3[i]), int(vj3[i])) for i in order3] == [first, second, (0, 1)]


def brute_force_clusters(edges, start, num, budget):
    """The two passes stated over sets: seeds pair up along the first edges that touch no seed yet; then free vertices
    join the cluster behind the first edge that links them to a covered vertex."""
    head, members = {}, {}
    removed = 0
    for a, b in edges:
        if removed == budget:
            break
        if a != b and b != 0 and a not in head and b not in head:
            head[a] = head[b] = b
            members[b] = {a, b}
            removed += 1
    for a, b in edges:
        if removed == budget:
            break
        if a == b or (a in head) == (b in head):
            continue
        free, cov = (a, b) if b in head else (b, a)
        if head[cov] == 0:
            continue
        head[free] = head[cov]
        members[head[cov]].add(free)
        removed += 1
    rep = np.zeros(num + start, np.int32)
    for h, ms in members.items():
        rep[h] = len(ms) - 1
        for m in ms - {h}:
            rep[m] = -h
    return rep, removed


def test_cluster_vertices_hand_cases():
    # path 1-2-3-4-5 with the middle edges cheapest: pairs (2,3) then (4,5); then 1 joins 2's cluster, whose head is 3
    ei, ej = np.array([2, 4, 1, 3]), np.array([3, 5, 2, 4])
    rep = np.zeros(6, np.int32)
    assert D.cluster_vertices(ei, ej, 0, 6, 10, rep) == 3
    assert rep.tolist() == [0, -3, -3, 2, -5, 1]
    # budget 1: only the first pair
    rep = np.zeros(6, np.int32)
    assert D.cluster_vertices(ei, ej, 0, 6, 1, rep) == 1 and rep.tolist() == [0, 0, -3, 1, 0, 0]
    # the free end in FIRST position joins as well (the reference would contract the covered vertex 3 a second time)
    rep = np.zeros(6, np.int32)
    D.cluster_vertices(np.array([3, 3]), np.array([4, 5]), 0, 6, 10, rep)
    assert rep.tolist() == [0, 0, 0, -4, 2, -4]
    # nothing is ever contracted into vertex 0; a second sample starts at its own offset
    rep = np.zeros(8, np.int32)
    D.cluster_vertices(np.array([5, 4]), np.array([6, 5]), 4, 4, 10, rep)
    assert rep.tolist() == [0, 0, 0, 0, -6, -6, 2, 0]


@pytest.mark.parametrize("seed", range(6))
def test_cluster_vertices_matches_set_statement_and_invariants(seed):
    rng = np.random.default_rng(seed)
    num, start = 40, (0 if seed % 2 else 7)
    pairs = {tuple(sorted(p)) for p in rng.integers(start, start + num, (90, 2)).tolist() if p[0] != p[1]}
    edges = [list(p) for p in pairs]
    rng.shuffle(edges)
    budget = [3, 12, 100][seed % 3]
    rep = np.zeros(start + num, np.int32)
    removed = D.cluster_vertices(np.array([e[0] for e in edges]), np.array([e[1] for e in edges]), start, num, budget, rep)
    want, want_removed = brute_force_clusters(edges, start, num, budget)
    assert removed == want_removed and np.array_equal(rep, want)
    assert removed <= budget and (rep < 0).sum() == removed
    heads = -rep[rep < 0]
    assert np.all(rep[heads] > 0)                                      # no chains: a head is never contracted itself
    assert np.array_equal(np.bincount(heads, minlength=len(rep)) * (rep >= 0), rep * (rep >= 0))


# ------------------------------------------------------------------ a whole round
@pytest.mark.parametrize("name,frac", [("sphere2", 0.5), ("torus", 0.3), ("room_small", 0.5), ("shapes_small", 0.4)])
def test_simplify_round_invariants(name, frac):
    v, f, g = case(name)
    nv, nf = len(v), len(f)
    cum_v, cum_f = np.array([nv]), np.array([nf])
    n_remove = np.array([int(nv * frac)])
    vo, fo, deg, rep, vmap, nv_out, mf_out = D.simplify(v, f, g, cum_v, cum_f, n_remove)
    removed = (rep < 0).sum()
    assert 0 < removed <= n_remove[0]
    kept = vmap >= 0
    assert nv_out.sum() == kept.sum() and mf_out.sum() == (~deg).sum()
    assert np.array_equal(vmap[kept], np.arange(kept.sum()))           # ascending numbering of the survivors
    assert not np.any(kept & (rep < 0))                                # a contracted vertex is never an output vertex
    live = fo[~deg]
    assert live.min() >= 0 and live.max() < kept.sum()
    assert np.all((live[:, 0] != live[:, 1]) & (live[:, 0] != live[:, 2]) & (live[:, 1] != live[:, 2]))
    assert set(np.unique(live)) == set(range(kept.sum()))              # every output vertex keeps a facet
    # a facet dies exactly when two of its corners share a cluster
    head = np.where(rep < 0, -rep, np.arange(nv))
    hf = head[f]
    assert np.array_equal(deg, (hf[:, 0] == hf[:, 1]) | (hf[:, 0] == hf[:, 2]) | (hf[:, 1] == hf[:, 2]))
    # contracted positions: the centroid of each cluster
    for h in np.nonzero(rep > 0)[0][:20]:
        members = np.nonzero(head == h)[0]
        assert len(members) == rep[h] + 1 and np.allclose(vo[h], v[members].mean(0))
    assert np.array_equal(vo[rep == 0], v[rep == 0]) and np.all(vo[rep < 0] == 0)
    # contraction merges only vertices joined by a path of edges inside the cluster (here: an edge to the head's pair)
    edges = {tuple(sorted(e)) for t in f.tolist() for e in ((t[0], t[1]), (t[0], t[2]), (t[1], t[2]))}
    adj = {}
    for a, b in edges:
        adj.setdefault(a, set()).add(b)
        adj.setdefault(b, set()).add(a)
    for m in np.nonzero(rep < 0)[0][:200]:
        cluster = set(np.nonzero(head == head[m])[0].tolist())
        assert adj[m] & cluster


def test_simplify_two_samples_stay_apart_and_cheap_edges_go_first():
    va, fa, _ = case("sphere2")
    vb, fb, _ = case("torus")
    v = np.concatenate([va, vb + 5.0])
    f = np.concatenate([fa, fb + len(va)]).astype(np.int32)
    g = D.triangle_geometry(v, f)
    cum_v, cum_f = np.array([len(va), len(v)]), np.array([len(fa), len(f)])
    out = D.simplify(v, f, g, cum_v, cum_f, np.array([20, 0]))
    rep, nv_out = out[3], out[5]
    assert (rep[:len(va)] < 0).sum() == 20 and not np.any(rep[len(va):] != 0)
    assert nv_out.tolist() == [len(va) - 20, len(vb)]
    # with a budget of one, the single cheapest edge of the sample is the one contracted
    q, vi, vj = D.vertex_quadrics(v, f, g)
    cost = D.edge_costs(v, q, vi, vj)
    mine = np.nonzero(vi < len(va))[0]
    first = mine[np.lexsort((vj[mine], vi[mine], cost[mine]))[0]]
    rep1 = D.simplify(v, f, g, cum_v, cum_f, np.array([1, 0]))[3]
    assert rep1[vi[first]] == -vj[first] and (rep1 < 0).sum() == 1


def test_mesh_decimation_reaches_the_target_and_maps_compose():
    v, f, g = case("sphere3")
    nv_in, mf_in = np.array([len(v)]), np.array([len(f)])
    target = np.array([len(v) // 4])
    vo, fo, go, nv_o, mf_o, rep, vmap = D.mesh_decimation(v, f, g, nv_in, mf_in, target)
    assert nv_o[0] == target[0] == len(vo) and mf_o[0] == len(fo)       # closed surface: Euler keeps facets in step
    assert len(fo) == 2 * len(vo) - 4
    assert fo.max() == len(vo) - 1
    kept = vmap >= 0
    assert kept.sum() == len(vo) and np.array_equal(np.sort(vmap[kept]), np.arange(len(vo)))
    head = np.where(rep < 0, -rep, np.arange(len(v)))
    assert np.all(rep[head] >= 0) and np.all(vmap[head] >= 0)           # every input vertex lands on an output vertex
    assert np.array_equal(np.bincount(head, minlength=len(v))[kept] - 1, rep[kept])
    # the decimated surface stays near the unit sphere
    assert np.abs(np.linalg.norm(vo, axis=1) - 1).max() < 0.2
