"""Mesh decimation on the GPU against oracle/decimate_ref.py.

Floating-point stages (vertex quadrics, edge costs, contracted positions) within a tolerance of the float64 oracle;
integer stages (candidate edges, cluster maps, facets, counts) bit-exact against the oracle run on the SAME costs
(the device computes them in float32, so the order of near-equal costs is the device's; everything after the costs
is a function of their order alone).  The whole loop through the properties its callers rely on."""
import sys

import numpy as np
import pytest
import torch

from oracle import decimate_ref as D
from oracle import torch_ref
from picassoplus_amd.mesh.pi_modules import decimate, pool3d
from picassoplus_amd.mesh.pi_modules.geometry import compute_triangle_geometry_
from util import dev, mesh_case

pytestmark = pytest.mark.gpu
I32 = torch.int32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def batch(names, seed=0):
    vs, fs, nv, mf, off = [], [], [], [], 0
    for k, name in enumerate(names):
        v, f = mesh_case(name, seed + k)
        v = np.asarray(v, np.float32)[:, :3] + np.float32(3.0 * k)
        vs.append(v)
        fs.append(f.astype(np.int32) + off)
        nv.append(len(v))
        mf.append(len(f))
        off += len(v)
    return np.concatenate(vs), np.concatenate(fs), np.array(nv, np.int32), np.array(mf, np.int32)


CASES = [("tetra",), ("grid2",), ("sphere2",), ("torus", "sphere3"), ("room_small",), ("shapes_small", "fans")]


@pytest.mark.parametrize("names", CASES, ids=lambda n: "+".join(n))
@pytest.mark.parametrize("use_area,wgt_bnd", [(True, 5.0), (False, 5.0), (True, 0.0)])
def test_quadrics_and_costs_match_oracle(cuda, names, use_area, wgt_bnd):
    say("case decimate quadrics", names, use_area, wgt_bnd)
    v, f, nv, mf = batch(names)
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    g = geo.cpu().numpy()
    q, evi, evj = decimate.vertex_quadrics(vx, fc, geo, use_area, wgt_bnd)
    wq, wi, wj = D.vertex_quadrics(v, f, g, use_area, wgt_bnd)
    assert np.array_equal(evi.cpu().numpy(), wi) and np.array_equal(evj.cpu().numpy(), wj)
    qn = q.cpu().numpy()
    row = np.abs(wq).max(1, keepdims=True)
    assert np.all(np.abs(qn - wq) <= 2e-6 * np.maximum(row, 1e-30)), "vertex quadrics"
    cost = decimate.edge_costs(vx, q, evi, evj).cpu().numpy()
    want, rcond = D.edge_costs(v, qn, wi, wj, return_rcond=True)           # float64 arithmetic on the device's quadrics
    Q = qn[wi].astype(np.float64) + qn[wj]
    reach = 1 + np.maximum((v[wi].astype(np.float64) ** 2).sum(1), (v[wj].astype(np.float64) ** 2).sum(1))
    scale = np.abs(Q).sum(1) * reach
    # the branch is taken on a float32 reciprocal condition number: compare where the float64 one is clear of the
    # threshold; at a well-conditioned minimiser float32 elimination loses about 1 / rcond ulps
    clear = (rcond > 4 * D.RCOND_EPS) | (rcond < 0.25 * D.RCOND_EPS)
    loss = np.where(rcond > D.RCOND_EPS, 1 / np.maximum(rcond, 1e-30), 1.0)
    tol = 4e-7 * scale * np.maximum(loss, 8.0)
    bad = clear & ~(np.abs(cost - want) <= tol)
    assert not bad.any(), "edge costs: %d of %d off, worst %g" % (bad.sum(), len(bad), np.abs(cost - want)[bad].max())
    assert clear.mean() > 0.9


def _ulps(a, b):
    """Distance of two float32 arrays in units of the last place (0 where both are NaN or bit-equal)."""
    ia = np.ascontiguousarray(a, np.float32).view(np.int32).astype(np.int64)
    ib = np.ascontiguousarray(b, np.float32).view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    return np.where(np.isnan(a) & np.isnan(b), 0, d)


@pytest.mark.parametrize("names", CASES, ids=lambda n: "+".join(n))
@pytest.mark.parametrize("use_area,wgt_bnd", [(True, 5.0), (False, 5.0), (True, 0.0)])
def test_quadrics_and_costs_equal_the_float32_oracle(cuda, names, use_area, wgt_bnd):
    """EVERY candidate edge (no conditioning mask): the kernels round each product and sum on its own, so their
    float32 quadrics and costs are the float32 oracle's bit for bit -- including which branch an edge near the
    condition-number threshold takes."""
    say("case decimate float32 identity", names, use_area, wgt_bnd)
    v, f, nv, mf = batch(names)
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    g = geo.cpu().numpy()
    q, evi, evj = decimate.vertex_quadrics(vx, fc, geo, use_area, wgt_bnd)
    wq, wi, wj = D.vertex_quadrics(v, f, g, use_area, wgt_bnd, dtype=np.float32)
    assert wq.dtype == np.float32
    qn = q.cpu().numpy()
    dq = _ulps(qn, wq)
    assert dq.max() == 0, "vertex quadrics: %d of %d entries differ from the float32 oracle, worst %d ulp" % ((dq > 0).sum(), dq.size, dq.max())
    cost = decimate.edge_costs(vx, q, evi, evj).cpu().numpy()
    want = D.edge_costs(v, qn, wi, wj, dtype=np.float32)
    assert want.dtype == np.float32
    dc = _ulps(cost, want)
    assert dc.max() == 0, "edge costs: %d of %d differ from the float32 oracle, worst %d ulp" % ((dc > 0).sum(), dc.size, dc.max())


@pytest.mark.parametrize("names,frac", [(("sphere2",), 0.5), (("torus", "sphere3"), 0.3), (("room_small",), 0.5),
                                        (("shapes_small", "fans"), 0.45)],
                         ids=lambda n: "+".join(n) if isinstance(n, tuple) else str(n))
def test_simplify_round_equals_the_float32_oracle_from_the_mesh_alone(cuda, names, frac):
    """The oracle runs the whole round from (vertex, face, geometry) in float32 -- its own quadrics, its own costs, its
    own contraction order -- and every integer output of the device's round equals it."""
    say("case decimate simplify from the mesh alone", names, frac)
    v, f, nv, mf = batch(names)
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    nv_cum, mf_cum = np.cumsum(nv).astype(np.int32), np.cumsum(mf).astype(np.int32)
    n_remove = (nv * frac).astype(np.int32)
    out = decimate.simplify(vx, fc, geo, dev(nv_cum, cuda), dev(mf_cum, cuda), dev(n_remove, cuda), True, 5.0)
    want = D.simplify(v, f, geo.cpu().numpy(), nv_cum, mf_cum, n_remove, True, 5.0, dtype=np.float32)
    vo, fo, deg, rep, vmap, nv_o, mf_o = (t.cpu().numpy() for t in out)
    same = (rep == want[3]) & (vmap == want[4])
    assert same.all(), "maps differ from the float32 oracle's on %d of %d vertices" % ((~same).sum(), len(same))
    assert np.array_equal(deg, want[2]) and np.array_equal(fo, want[1]), "facets"
    assert np.array_equal(nv_o, want[5]) and np.array_equal(mf_o, want[6]), "counts"
    assert np.abs(vo - want[0]).max() <= 1e-6 * max(np.abs(v).max(), 1.0), "contracted positions"


@pytest.mark.parametrize("names,frac", [(("tetra",), 0.5), (("grid2",), 0.4), (("sphere2",), 0.5), (("torus", "sphere3"), 0.3),
                                        (("room_small",), 0.5), (("shapes_small", "fans"), 0.45), (("sphere3", "torus"), 0.0)],
                         ids=lambda n: "+".join(n) if isinstance(n, tuple) else str(n))
def test_simplify_round_is_exact_given_the_costs(cuda, names, frac):
    say("case decimate simplify", names, frac)
    v, f, nv, mf = batch(names)
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    nv_cum, mf_cum = np.cumsum(nv).astype(np.int32), np.cumsum(mf).astype(np.int32)
    n_remove = (nv * frac).astype(np.int32)
    out = decimate.simplify(vx, fc, geo, dev(nv_cum, cuda), dev(mf_cum, cuda), dev(n_remove, cuda), True, 5.0)
    again = decimate.simplify(vx.clone(), fc.clone(), geo.clone(), dev(nv_cum, cuda), dev(mf_cum, cuda), dev(n_remove, cuda), True, 5.0)
    for a, b in zip(out, again):
        assert torch.equal(a, b), "two runs differ"
    q, evi, evj = decimate.vertex_quadrics(vx, fc, geo, True, 5.0)
    cost = decimate.edge_costs(vx, q, evi, evj).cpu().numpy()
    want = D.simplify(v, f, geo.cpu().numpy(), nv_cum, mf_cum, n_remove, True, 5.0, cost=cost)
    vo, fo, deg, rep, vmap, nv_o, mf_o = (t.cpu().numpy() for t in out)
    assert np.array_equal(rep, want[3]), "vt_replace"
    assert np.array_equal(vmap, want[4]), "vt_map"
    assert np.array_equal(deg, want[2]) and np.array_equal(fo, want[1]), "facets"
    assert np.array_equal(nv_o, want[5]) and np.array_equal(mf_o, want[6]), "counts"
    assert np.abs(vo - want[0]).max() <= 1e-6 * max(np.abs(v).max(), 1.0), "contracted positions"
    assert (rep < 0).sum() <= n_remove.sum()
    if frac == 0.0:
        assert not rep.any() and np.array_equal(vmap, np.arange(len(v))) and not deg.any()


def test_decimation_loop_feeds_the_pooling_ops(cuda):
    say("case decimate loop")
    v, f, nv, mf = batch(("sphere3", "torus", "room_small"))
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    target = (nv // 3).astype(np.int32)
    res = decimate.mesh_decimation_(vx, fc, geo, dev(nv, cuda), dev(mf, cuda), dev(target, cuda))
    res2 = decimate.mesh_decimation_(vx, fc, geo, dev(nv, cuda), dev(mf, cuda), dev(target, cuda))
    for a, b in zip(res, res2):
        assert torch.equal(a, b), "two runs differ"
    vo, fo, go, nv_o, mf_o, rep, vmap = res
    nv_o, mf_o = nv_o.cpu().numpy(), mf_o.cpu().numpy()
    say("  vertices", nv.tolist(), "->", nv_o.tolist(), "facets", mf.tolist(), "->", mf_o.tolist())
    # closed surfaces reach their target exactly; the open room may lose vertices whose facets all collapse
    assert nv_o[0] == target[0] and nv_o[1] == target[1] and nv_o[2] <= target[2]
    assert mf_o[0] == 2 * nv_o[0] - 4 and mf_o[1] == 2 * nv_o[1]           # Euler: sphere, torus
    assert vo.shape[0] == nv_o.sum() and fo.shape[0] == mf_o.sum() and go.shape == (fo.shape[0], 5)
    fo_n = fo.cpu().numpy()
    cum = np.concatenate([[0], np.cumsum(nv_o)])
    fcum = np.concatenate([[0], np.cumsum(mf_o)])
    for b in range(3):                                                      # facets stay inside their own sample
        part = fo_n[fcum[b]:fcum[b + 1]]
        assert part.min() >= cum[b] and part.max() < cum[b + 1]
    assert torch.equal(go, compute_triangle_geometry_(vo, fo))
    # the maps over the input vertices are what pooling takes
    rep_n, map_n = rep.cpu().numpy(), vmap.cpu().numpy()
    head = np.where(rep_n < 0, -rep_n, np.arange(len(v)))
    assert np.all(rep_n[head] >= 0)
    x = np.random.default_rng(0).normal(size=(len(v), 8)).astype(np.float32)
    T = torch.from_numpy
    pooled = pool3d.maxPool(dev(x, cuda), rep, vmap, vo)
    want, _ = torch_ref.maxpool_fwd(T(x), T(rep_n), T(map_n), vo.shape[0])
    assert np.array_equal(pooled.cpu().numpy(), want.numpy())
    # positions are means over clusters of means: the pooled input positions stay close to them
    centre = pool3d.avgPool(vx, rep, vmap, vo).cpu().numpy()
    used = np.bincount(map_n[head][map_n[head] >= 0], minlength=vo.shape[0]) > 0
    assert used.all()
    assert np.abs(centre - vo.cpu().numpy()).max() < 0.35


def test_decimate_argument_errors(cuda):
    say("case decimate errors")
    v, f, nv, mf = batch(("sphere1",))
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    args = [dev(np.cumsum(nv).astype(np.int32), cuda), dev(np.cumsum(mf).astype(np.int32), cuda), dev((nv // 2).astype(np.int32), cuda)]
    with pytest.raises(RuntimeError):
        decimate.simplify(vx.cpu(), fc, geo, *args)
    with pytest.raises(RuntimeError):
        decimate.simplify(vx, fc.long(), geo, *args)
    with pytest.raises(RuntimeError):
        decimate.simplify(vx, fc, geo[:, :4].contiguous(), *args)
    with pytest.raises(RuntimeError):
        decimate.simplify(vx[:, :2].contiguous(), fc, geo, *args)
    with pytest.raises(RuntimeError):
        decimate.simplify(vx, fc, geo, args[0].long(), args[1], args[2])


def test_mesh_hierarchy_levels_feed_a_network_block(cuda):
    """MeshHierarchy (picasso/mesh/utils.py:32-58) in both constructor forms: every level is a valid mesh, the maps of
    a level pool the features of the level above, and the strided form honours the floor on the vertex count."""
    say("case decimate hierarchy")
    from picassoplus_amd.mesh.utils import MeshHierarchy, count_vertex_adjface
    v, f, nv, mf = batch(("sphere3", "torus"))
    vx, fc = dev(v, cuda), dev(f, cuda)
    levels = MeshHierarchy([2, 3], [100, 150], True, 1.0)(vx, fc, dev(nv, cuda), dev(mf, cuda))
    assert len(levels) == 3 and levels[0][5] is None and levels[0][6] is None
    n_prev = nv
    for lvl, (vl, fl, gl, nvl, mfl, rep, vmap) in enumerate(levels):
        nvl_n, mfl_n = nvl.cpu().numpy(), mfl.cpu().numpy()
        assert vl.shape[0] == nvl_n.sum() and fl.shape[0] == mfl_n.sum() and gl.shape == (fl.shape[0], 5)
        assert int(fl.max()) < vl.shape[0] and int(fl.min()) >= 0
        if lvl:
            want = np.maximum(n_prev // [2, 3][lvl - 1], [100, 150][lvl - 1])
            assert np.array_equal(nvl_n, want), (nvl_n, want)          # closed surfaces reach the target exactly
            above = levels[lvl - 1][0]
            assert rep.shape[0] == above.shape[0] and vmap.shape[0] == above.shape[0]
            pooled = pool3d.avgPool(above, rep, vmap, vl)
            assert pooled.shape == vl.shape and bool(torch.isfinite(pooled).all())
            nf_count = count_vertex_adjface(fl, torch.arange(vl.shape[0], dtype=I32, device=cuda), vl)
            assert int(nf_count.min()) >= 1 and int(nf_count.sum()) == 3 * fl.shape[0]
        n_prev = nvl_n
    fixed = MeshHierarchy([dev(np.array([300, 200], np.int32), cuda)], True, 1.0)(vx, fc, dev(nv, cuda), dev(mf, cuda))
    assert fixed[1][3].cpu().tolist() == [300, 200]


@pytest.mark.parametrize("seed", range(10))
def test_device_clustering_equals_the_serial_host_routine(cuda, seed):
    """cluster_vertices_device (fixed-point rounds of the first pass, one-step second pass, both cut by rank) against
    pmesh_cluster_vertices_host and the oracle's statement of the two serial passes, on random graphs of several samples
    with budgets from nothing to everything -- including chains of ascending ranks, the slowest case for the rounds."""
    say("case device clustering", seed)
    rng = np.random.default_rng(100 + seed)
    samples = 1 + seed % 4
    num = [int(n) for n in rng.integers(2, 400, samples)]
    starts = np.concatenate([[0], np.cumsum(num)])
    vi_l, vj_l, smp = [], [], []
    for b in range(samples):
        lo, n = int(starts[b]), num[b]
        pairs = {tuple(sorted(p)) for p in rng.integers(lo, lo + n, (int(rng.integers(1, 5)) * n, 2)).tolist() if p[0] != p[1]}
        if seed % 3 == 0:                                   # a path in ascending order of rank: one choice per round
            pairs |= {(lo + i, lo + i + 1) for i in range(min(n - 1, 40))}
        pairs = sorted(pairs)
        order = np.arange(len(pairs)) if seed % 3 == 0 else rng.permutation(len(pairs))
        vi_l.append(np.array(pairs, np.int32).reshape(-1, 2)[order, 0])
        vj_l.append(np.array(pairs, np.int32).reshape(-1, 2)[order, 1])
        smp.append(np.full(len(pairs), b, np.int64))
    vi, vj, sample = np.concatenate(vi_l), np.concatenate(vj_l), np.concatenate(smp)
    nv_cum = torch.from_numpy(starts[1:].astype(np.int32))
    Nv = int(starts[-1])
    for frac in (0.0, 0.1, 0.45, 0.8, 1.0):
        budget = np.array([int(n * frac) for n in num], np.int32)
        want = np.zeros(Nv, np.int32)
        for b in range(samples):
            m = sample == b
            D.cluster_vertices(vi[m], vj[m], int(starts[b]), num[b], int(budget[b]), want)
        host = decimate.cluster_vertices(torch.from_numpy(vi), torch.from_numpy(vj), torch.from_numpy(sample), nv_cum,
                                         torch.from_numpy(budget), Nv)
        assert np.array_equal(host, want)
        # the device routine takes the edges in ascending (vi, vj) order plus their contraction order
        by_pair = np.lexsort((vj, vi))
        perm = np.argsort(by_pair, kind="stable")               # position of contraction-order edge k in the (vi, vj) list
        got = decimate.cluster_vertices_device(dev(vi[by_pair], cuda), dev(vj[by_pair], cuda), dev(perm, cuda), dev(sample, cuda),
                                               nv_cum.to(cuda), dev(budget, cuda), Nv, rounds_per_check=1 + seed % 3)
        assert np.array_equal(got.cpu().numpy(), want), "budget fraction %g: %d vertices differ" % (frac, (got.cpu().numpy() != want).sum())
    with pytest.raises(RuntimeError):
        decimate.cluster_vertices_device(dev(vj, cuda), dev(vi, cuda), dev(np.arange(len(vi)), cuda), dev(sample, cuda), nv_cum.to(cuda),
                                         dev(budget, cuda), Nv)


def test_contraction_order_on_the_device_is_the_oracles(cuda):
    """The native sort keys (few samples) and the two-sort path (many samples) order the candidate edges exactly as the
    oracle's lexicographic statement, for costs that are negative, signed zeros, denormal, infinite, NaN or an ulp
    apart; the samples read off the keys are the oracle's."""
    rng = np.random.default_rng(0)
    n = 20000
    vi = rng.integers(0, 300, n)
    vj = vi + rng.integers(1, 50, n)
    k = np.argsort(vi.astype(np.int64) * 1000 + vj, kind="stable")
    vi, vj = vi[k].astype(np.int32), vj[k].astype(np.int32)
    special = np.array([0.0, -0.0, 1e-45, -1e-45, 1e-30, -1e-30, -2.5, 2.5, np.nan, np.inf, -np.inf, 1.0, 1.0000001, -1.0], np.float32)
    cost = rng.choice(special, n)
    cost[::7] = rng.normal(size=len(cost[::7])).astype(np.float32)
    for cum in (np.array([300]), np.array([100, 100, 200, 300]), np.arange(3, 384, 3)[:127], np.arange(2, 302, 2)):
        cum = cum.astype(np.int32)
        want_perm, want_sample = D.contraction_order(cost, vi, vj, cum)
        perm, sample = decimate.contraction_order(dev(cost, cuda), dev(vi, cuda), dev(vj, cuda), dev(cum, cuda))
        assert np.array_equal(perm.cpu().numpy(), want_perm), len(cum)
        assert np.array_equal(sample.cpu().numpy(), want_sample), len(cum)
    perm, sample = decimate.contraction_order(dev(cost[:0], cuda), dev(vi[:0], cuda), dev(vj[:0], cuda), dev(np.array([5], np.int32), cuda))
    assert perm.shape[0] == 0 and sample.shape[0] == 0


def test_simplify_is_the_same_with_host_clustering(cuda, monkeypatch):
    v, f, nv, mf = batch(("sphere3", "room_small", "torus"))
    vx, fc = dev(v, cuda), dev(f, cuda)
    geo = compute_triangle_geometry_(vx, fc)
    args = (vx, fc, geo, dev(np.cumsum(nv).astype(np.int32), cuda), dev(np.cumsum(mf).astype(np.int32), cuda))
    for frac in (0.3, 0.7):
        n_remove = dev((nv * frac).astype(np.int32), cuda)
        monkeypatch.delenv("PMESH_DECIMATE_HOST_CLUSTERING", raising=False)
        a = decimate.simplify(*args, n_remove, True, 5.0)
        monkeypatch.setenv("PMESH_DECIMATE_HOST_CLUSTERING", "1")
        b = decimate.simplify(*args, n_remove, True, 5.0)
        for x, y in zip(a, b):
            assert torch.equal(x, y)


@pytest.mark.parametrize("case", ["fans", "hub60", "sphere3+torus", "degenerate"])
def test_edge_list_from_the_adjacency_equals_the_sorted_edge_list(cuda, case):
    """decimate.edge_list (one thread per vertex over its adjacency row) against the oracle's sort of all facet edges:
    the same unique edges in the same order, the same boundary edges with the same facets -- including a vertex whose
    row is too long for the kernel's private memory and facets with a repeated vertex."""
    from picassoplus_amd.mesh import topology
    say("case edge list", case)
    if case == "hub60":
        n = 60
        rim = 1 + np.arange(n)
        f = np.stack([np.zeros(n, np.int64), rim, np.roll(rim, -1)], 1)[:-7].astype(np.int32)      # an open fan
        f = np.concatenate([f, f[:5, [0, 2, 1]]]).astype(np.int32)                                  # some sides held twice
        nv = n + 1
    elif case == "degenerate":
        f = np.array([[0, 1, 2], [2, 2, 3], [3, 4, 4], [5, 5, 5], [1, 2, 3], [6, 0, 6]], np.int32)
        nv = 7
    elif case == "fans":
        v, f = mesh_case("fans")
        nv = v.shape[0]
    else:
        v, f, _, _ = batch(("sphere3", "torus"))
        nv = v.shape[0]
    fc = dev(f, cuda)
    rowptr, colidx = topology.vertex_csr(fc, None, nv)
    evi, evj, bvi, bvj, bface = decimate.edge_list(fc, rowptr, colidx, nv)
    wi, wj, counts, first_face = D.unique_edges(f, nv)
    ok = wi != wj
    assert np.array_equal(evi.cpu().numpy(), wi[ok]) and np.array_equal(evj.cpu().numpy(), wj[ok])
    bnd = (counts == 1) & ok
    assert np.array_equal(bvi.cpu().numpy(), wi[bnd]) and np.array_equal(bvj.cpu().numpy(), wj[bnd])
    assert np.array_equal(bface.cpu().numpy(), first_face[bnd])


def test_round_on_degenerate_batches(cuda):
    """A sample without facets beside a regular one, a mesh whose facets are all collapsed, and a round with nothing to
    remove: the round's outputs keep their shapes and meanings (no candidate edges -> nothing contracted)."""
    v, f = mesh_case("octa")
    v = np.asarray(v, np.float32)
    lone = np.zeros((3, 3), np.float32)                                  # three vertices, no facet
    vs = np.concatenate([v, lone])
    nv_cum = np.array([len(v), len(vs)], np.int32)
    mf_cum = np.array([len(f), len(f)], np.int32)
    vx, fc = dev(vs, cuda), dev(f.astype(np.int32), cuda)
    geo = compute_triangle_geometry_(vx, fc)
    out = decimate.simplify(vx, fc, geo, dev(nv_cum, cuda), dev(mf_cum, cuda), dev(np.array([3, 2], np.int32), cuda), True, 5.0)
    want = D.simplify(vs, f.astype(np.int32), geo.cpu().numpy(), nv_cum, mf_cum, np.array([3, 2], np.int32), True, 5.0, dtype=np.float32)
    for got, ref in zip(out[1:], want[1:]):
        assert np.array_equal(got.cpu().numpy(), ref)
    assert not out[3][len(v):].any()                                     # nothing to contract in the facet-less sample
    # every facet collapsed: no edges at all
    flat = dev(np.array([[0, 0, 0], [2, 2, 2]], np.int32), cuda)
    vx2 = dev(v[:3], cuda)
    geo2 = compute_triangle_geometry_(vx2, flat)
    one = torch.tensor([3], dtype=I32, device=cuda)
    out2 = decimate.simplify(vx2, flat, geo2, one, torch.tensor([2], dtype=I32, device=cuda), torch.tensor([2], dtype=I32, device=cuda))
    assert not out2[3].any() and bool(out2[2].all()) and out2[5].tolist() == [0] and out2[6].tolist() == [0]
    res = decimate.mesh_decimation_(vx2, flat, geo2, one, torch.tensor([2], dtype=I32, device=cuda), torch.tensor([1], dtype=I32, device=cuda))
    # vertices left without a live facet leave the mesh (as in the reference); the loop ends, sizes agree
    assert res[0].shape[0] == int(res[3].sum()) == 0 and res[1].shape[0] == int(res[4].sum()) == 0
