"""Pins the CPU oracle (oracle/) without a GPU.

The reference ships no tests, fixtures or golden vectors for this path, so each oracle function
is pinned by checks that do not retype its formula: an independent pure-Python statement of the
op on tiny meshes, closed forms and invariants of the mathematics, a library routine (scipy's
spherical harmonics), autograd of the forward restatement for every explicit backward, and the
agreement of the two independently written restatements (C loops vs vectorised torch).
"""
import math

import numpy as np
import pytest
import scipy.special
import torch

from oracle import loops, torch_ref
from picassoplus_amd import synthetic as S
from util import mesh_case, rel_err, strided_vt_map, texture_case, tiny_meshes

T = torch.from_numpy
EPS = 1e-12


# ------------------------------------------------------------------ spherical harmonics
def scipy_basis(xyz, L):
    """Per degree l: Re Y_l^{-m} for m = l..0, then -Im Y_l^{-m} for m = l..1 (complex Y, no sqrt 2)."""
    u = xyz / np.linalg.norm(xyz, axis=1, keepdims=True)
    polar = np.arccos(np.clip(u[:, 2], -1, 1))
    azim = np.arctan2(u[:, 1], u[:, 0])
    cols = []
    for l in range(L + 1):
        ys = {m: scipy.special.sph_harm_y(l, -m, polar, azim) for m in range(l + 1)}
        cols += [ys[m].real for m in range(l, -1, -1)] + [-ys[m].imag for m in range(l, 0, -1)]
    return np.stack(cols, 1)


@pytest.mark.parametrize("L", range(6))
def test_sph_harm_matches_scipy(L):
    xyz = np.random.default_rng(L).normal(size=(500, 3))
    ref = scipy_basis(xyz, L)
    assert rel_err(loops.sph_harm(xyz, L), ref) < 1e-12
    assert rel_err(torch_ref.sph_harm(T(xyz), L).numpy(), ref) < 1e-12


def test_sph_harm_sum_rule_and_scale_invariance():
    xyz = np.random.default_rng(1).normal(size=(200, 3))
    c = loops.sph_harm(xyz, 5)
    off = 0
    for l in range(6):
        blk = c[:, off:off + 2 * l + 1]
        total = 2 * (blk ** 2).sum(1) - blk[:, l] ** 2       # the m = 0 term sits in the middle
        assert np.allclose(total, (2 * l + 1) / (4 * math.pi), atol=1e-12)
        off += 2 * l + 1
    assert rel_err(loops.sph_harm(xyz * 37.5, 5), c) < 1e-12


def test_sph_harm_hand_values_and_zero_vector():
    c = loops.sph_harm(np.eye(3), 3)
    p = math.pi
    assert np.allclose(c[:, 0], 0.5 * math.sqrt(1 / p))
    assert np.allclose(c[0, 1:4], [0.5 * math.sqrt(1.5 / p), 0, 0], atol=1e-15)           # +x
    assert np.allclose(c[1, 1:4], [0, 0, 0.5 * math.sqrt(1.5 / p)], atol=1e-15)           # +y
    assert np.allclose(c[2, 1:4], [0, 0.5 * math.sqrt(3 / p), 0], atol=1e-15)             # +z
    assert np.isclose(c[2, 6], 0.25 * math.sqrt(5 / p) * 2) and np.isclose(c[2, 12], 0.25 * math.sqrt(7 / p) * 2)
    assert np.isclose(c[0, 9], 0.125 * math.sqrt(35 / p)) and np.isclose(c[1, 13], -0.125 * math.sqrt(35 / p))
    zero = loops.sph_harm(np.zeros((1, 3)), 3)
    assert np.allclose(zero, c[0:1], atol=1e-15)                                           # evaluates at (1,0,0)
    with pytest.raises(NotImplementedError):
        loops.sph_harm(np.eye(3), 6)
    with pytest.raises(NotImplementedError):
        torch_ref.sph_harm(torch.eye(3), 6)


# ------------------------------------------------------------------ independent tiny-mesh statements
def py_v2f(x, filt, face):
    nf, (_, C, r) = face.shape[0], filt.shape
    out = np.zeros((nf, C * r))
    for f in range(nf):
        for c in range(C):
            for m in range(r):
                out[f, c * r + m] = sum(filt[k, c, m] * x[face[f, k], c] for k in range(3))
    return out


def py_f2v(x, filt, coeff, face, nfc, vt_map):
    nf, C = x.shape
    K, _, r = filt.shape
    out = np.zeros((nfc.shape[0], C * r))
    for f in range(nf):
        for c in range(C):
            for m in range(r):
                w = sum(coeff[f, k] * filt[k, c, m] for k in range(K))
                for j in range(3):
                    vo = vt_map[face[f, j]]
                    if vo >= 0:
                        out[vo, c * r + m] += w * x[f, c] / nfc[vo]
    return out


def py_f2f(tex, filt, sh, counts):
    Cout, Cin, F = filt.shape
    out = np.zeros((counts.shape[0], Cout))
    k0 = 0
    for f, K in enumerate(counts):
        for co in range(Cout):
            s = 0.0
            for k in range(k0, k0 + K):
                for ci in range(Cin):
                    s += tex[k, ci] * float(np.dot(sh[k], filt[co, ci]))
            out[f, co] = s / K if K else 0.0
        k0 += K
    return out


@pytest.mark.parametrize("name", ["tetra", "octa", "grid2"])
def test_loops_match_independent_python(name):
    v, f = tiny_meshes()[name]
    rng = np.random.default_rng(3)
    nv, nf, C, r, K = v.shape[0], f.shape[0], 3, 2, 4
    x, filt = rng.normal(size=(nv, C)), rng.normal(size=(3, C, r))
    assert rel_err(loops.v2f_fwd(x, filt, f), py_v2f(x, filt, f)) < EPS
    vt_map, nvo = strided_vt_map(rng, nv, keep=0.7)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nvo), 1)
    xf, fl, cf = rng.normal(size=(nf, C)), rng.normal(size=(K, C, r)), rng.normal(size=(nf, K))
    assert rel_err(loops.f2v_fwd(xf, fl, cf, f, nfc, vt_map), py_f2v(xf, fl, cf, f, nfc, vt_map)) < EPS
    counts = rng.integers(0, 4, nf).astype(np.int32)
    Tn = int(counts.sum())
    tex, sh, W = rng.normal(size=(Tn, C)), rng.normal(size=(Tn, K)), rng.normal(size=(5, C, K))
    assert rel_err(loops.f2f_fwd(tex, W, sh, np.cumsum(counts)), py_f2f(tex, W, sh, counts)) < EPS


# ------------------------------------------------------------------ closed forms
def test_v2f_constant_input_closed_form():
    v, f = mesh_case("sphere2")
    rng = np.random.default_rng(4)
    C, r = 5, 2
    xc = rng.normal(size=C)
    filt = rng.normal(size=(3, C, r))
    out = loops.v2f_fwd(np.tile(xc, (v.shape[0], 1)), filt, f)
    expect = (xc[:, None] * filt.sum(0)).reshape(-1)
    assert np.allclose(out, expect[None, :], atol=1e-13)


def test_f2v_closed_forms():
    v, f = mesh_case("sphere2")                       # closed mesh: every vertex has its full fan
    rng = np.random.default_rng(5)
    nv, nf, C, K = v.shape[0], f.shape[0], 4, 16
    ident = np.arange(nv, dtype=np.int32)
    valence = S.vertex_facet_count(f, ident, nv)
    # one-hot coeff and unit nf_count: plain scatter-add of filt[k0] * x
    x, filt = rng.normal(size=(nf, C)), rng.normal(size=(K, C, 1))
    onehot = np.zeros((nf, K)); onehot[:, 5] = 1
    ref = np.zeros((nv, C)); np.add.at(ref, f.reshape(-1), np.repeat(x * filt[5, :, 0], 3, axis=0))
    assert rel_err(loops.f2v_fwd(x, filt, onehot, f, np.ones(nv, np.int32), ident), ref) < EPS
    # constant input, constant coeff, nf_count = valence: every vertex gets x * (coeff . filt)
    xc, cc = rng.normal(size=C), rng.normal(size=K)
    out = loops.f2v_fwd(np.tile(xc, (nf, 1)), filt, np.tile(cc, (nf, 1)), f, valence, ident)
    assert np.allclose(out, (xc * (cc @ filt[:, :, 0]))[None, :], atol=1e-13)
    # dropped vertices contribute nothing and receive nothing
    vt_map, nvo = strided_vt_map(rng, nv)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nvo), 1)
    coeff = rng.normal(size=(nf, K))
    full = loops.f2v_fwd(x, filt, coeff, f, np.ones(nv, np.int32), ident)
    part = loops.f2v_fwd(x, filt, coeff, f, np.ones(nvo, np.int32), vt_map)
    assert rel_err(part, full[vt_map >= 0]) < EPS
    assert part.shape[0] == nvo and nfc.min() >= 1


def test_f2f_closed_forms():
    rng = np.random.default_rng(6)
    nf, Cin, Cout, F = 40, 6, 5, 16
    W = rng.normal(size=(Cout, Cin, F))
    # one texture point per facet and a one-hot SH row: a plain matrix product with W[:, :, d0]
    tex = rng.normal(size=(nf, Cin))
    sh = np.zeros((nf, F)); sh[:, 7] = 1
    out = loops.f2f_fwd(tex, W, sh, np.arange(1, nf + 1))
    assert rel_err(out, tex @ W[:, :, 7].T) < EPS
    # facets without texture points give zero rows; the factored form equals the naive loops
    counts, bary, _ = texture_case(rng, nf, 4, empty_frac=0.3)
    Tn, cum = int(counts.sum()), np.cumsum(counts).astype(np.int32)
    tex, sh = rng.normal(size=(Tn, Cin)), rng.normal(size=(Tn, F))
    naive = loops.f2f_fwd(tex, W, sh, cum)
    assert np.all(naive[counts == 0] == 0) and (counts == 0).any()
    assert rel_err(torch_ref.f2f_fwd(T(tex), T(W), T(sh), T(cum)).numpy(), naive) < EPS
    # dense special case against einsum: K points per facet, G = mean of outer products
    K = 3
    tex, sh = rng.normal(size=(nf * K, Cin)), rng.normal(size=(nf * K, F))
    G = np.einsum("fkc,fkd->fcd", tex.reshape(nf, K, Cin), sh.reshape(nf, K, F)) / K
    assert rel_err(loops.f2f_fwd(tex, W, sh, np.arange(1, nf + 1) * K), np.einsum("fcd,ocd->fo", G, W)) < EPS


# ------------------------------------------------------------------ backward = derivative of forward
def _vjp(fn, args, wrt, g):
    leaves = [a.clone().requires_grad_(i in wrt) if a.is_floating_point() else a for i, a in enumerate(args)]
    out = fn(*leaves)
    return torch.autograd.grad(out, [leaves[i] for i in wrt], g)


def test_explicit_backwards_match_autograd_and_loops():
    v, f = mesh_case("sphere2")
    rng = np.random.default_rng(7)
    nv, nf, C, r, K = v.shape[0], f.shape[0], 4, 2, 9
    x, filt, g = rng.normal(size=(nv, C)), rng.normal(size=(3, C, r)), rng.normal(size=(nf, C * r))
    auto = _vjp(torch_ref.v2f_fwd, [T(x), T(filt), T(f)], [0, 1], T(g))
    expl = torch_ref.v2f_bwd(T(g), T(x), T(filt), T(f))
    lp = loops.v2f_bwd(g, x, filt, f)
    for a, e, l in zip(auto, expl, lp):
        assert rel_err(e.numpy(), a.numpy()) < EPS and rel_err(l, a.numpy()) < EPS

    vt_map, nvo = strided_vt_map(rng, nv)
    nfc = np.maximum(S.vertex_facet_count(f, vt_map, nvo), 1)
    xf, fl, cf, go = rng.normal(size=(nf, C)), rng.normal(size=(K, C, r)), rng.normal(size=(nf, K)), rng.normal(size=(nvo, C * r))
    args = [T(xf), T(fl), T(cf), T(f), T(nfc), T(vt_map)]
    auto = _vjp(torch_ref.f2v_fwd, args, [0, 1], T(go))
    expl = torch_ref.f2v_bwd(T(go), *args)
    lp = loops.f2v_bwd(go, xf, fl, cf, f, nfc, vt_map)
    for a, e, l in zip(auto, expl, lp):
        assert rel_err(e.numpy(), a.numpy()) < EPS and rel_err(l, a.numpy()) < EPS

    counts, _, _ = texture_case(rng, 60, 4)
    Tn, cum = int(counts.sum()), np.cumsum(counts).astype(np.int32)
    tex, sh, W, go = rng.normal(size=(Tn, C)), rng.normal(size=(Tn, K)), rng.normal(size=(6, C, K)), rng.normal(size=(60, 6))
    args = [T(tex), T(W), T(sh), T(cum)]
    auto = _vjp(torch_ref.f2f_fwd, args, [0, 1], T(go))
    expl = torch_ref.f2f_bwd(T(go), *args)
    lp = loops.f2f_bwd(go, tex, W, sh, cum)
    for a, e, l in zip(auto, expl, lp):
        assert rel_err(e.numpy(), a.numpy()) < EPS and rel_err(l, a.numpy()) < EPS
    # the point-wise form of the filter gradient (blocks of points, no per-facet moments) is the same sum:
    # against autograd of the forward and the loops, with blocks that cut facets in two
    pw = torch_ref.f2f_bwd_filter_pointwise(T(go), T(tex), T(sh), T(cum), block=7)
    assert rel_err(pw.numpy(), auto[1].numpy()) < EPS and rel_err(pw.numpy(), lp[1]) < EPS
    # nf_count as produced by count_vertex_adjface: the number of (facet, corner) pairs per kept vertex, counted by hand
    cnt = np.zeros(nvo, np.int64)
    for fc in f:
        for vtx in fc:
            if vt_map[vtx] >= 0:
                cnt[vt_map[vtx]] += 1
    assert np.array_equal(torch_ref.count_vertex_adjface(T(f), T(vt_map), nvo).numpy(), cnt)
    assert np.array_equal(S.vertex_facet_count(f, vt_map, nvo), cnt)


def test_adjoint_identities():
    """<op(x), g> == <x, op_bwd_input(g)> for the three linear convolutions (loop oracle)."""
    v, f = mesh_case("octa")
    rng = np.random.default_rng(8)
    nv, nf, C, K = v.shape[0], f.shape[0], 3, 4
    x, filt, g = rng.normal(size=(nv, C)), rng.normal(size=(3, C, 1)), rng.normal(size=(nf, C))
    assert np.isclose((loops.v2f_fwd(x, filt, f) * g).sum(), (x * loops.v2f_bwd(g, x, filt, f)[0]).sum())
    ident = np.arange(nv, dtype=np.int32)
    nfc = S.vertex_facet_count(f, ident, nv)
    xf, fl, cf, go = rng.normal(size=(nf, C)), rng.normal(size=(K, C, 1)), rng.normal(size=(nf, K)), rng.normal(size=(nv, C))
    assert np.isclose((loops.f2v_fwd(xf, fl, cf, f, nfc, ident) * go).sum(),
                      (xf * loops.f2v_bwd(go, xf, fl, cf, f, nfc, ident)[0]).sum())


# ------------------------------------------------------------------ pooling
def brute_clusters(vt_replace, vt_map):
    members = {}
    for v in range(len(vt_replace)):
        rep = -vt_replace[v] if vt_replace[v] < 0 else v
        if vt_map[rep] >= 0:
            members.setdefault(int(vt_map[rep]), []).append(v)
    return members


@pytest.mark.parametrize("spatial,orphans", [(True, 0.0), (False, 0.1)])
def test_pool_unpool_against_brute_force(spatial, orphans):
    rng = np.random.default_rng(9)
    nv, C = 400, 3
    vt_replace, vt_map, nvo = S.cluster_maps(rng, nv, spatial=spatial, orphan_frac=orphans)
    x = rng.normal(size=(nv, C))
    x[rng.integers(0, nv, 50)] = x[rng.integers(0, nv, 50)]          # plant some ties
    mem = brute_clusters(vt_replace, vt_map)
    mx, idx = loops.maxpool_fwd(x, vt_replace, vt_map, nvo)
    av = loops.avgpool_fwd(x, vt_replace, vt_map, nvo)
    for o in range(nvo):
        rows = mem[o]
        assert np.array_equal(mx[o], x[rows].max(0))
        assert np.array_equal(idx[o], [rows[int(np.argmax(x[rows][:, c]))] for c in range(C)])   # first max = smallest id
        assert np.allclose(av[o], x[rows].mean(0), atol=1e-13)
        assert vt_replace[rows].max() + 1 == len(rows)                # the divisor the op uses
    mx_t, idx_t = torch_ref.maxpool_fwd(T(x), T(vt_replace), T(vt_map), nvo)
    assert np.array_equal(mx_t.numpy(), mx) and np.array_equal(idx_t.numpy(), idx)
    assert rel_err(torch_ref.avgpool_fwd(T(x), T(vt_replace), T(vt_map), nvo).numpy(), av) < EPS

    g = rng.normal(size=(nvo, C))
    gmax = loops.maxpool_bwd(g, nv, idx)
    assert np.allclose(gmax.sum(0), g.sum(0)) and np.count_nonzero(gmax) == g.size
    assert np.array_equal(torch_ref.maxpool_bwd(T(g), nv, idx_t).numpy(), gmax)
    up = loops.unpool_fwd(g, vt_replace, vt_map)
    for o, rows in mem.items():
        assert np.array_equal(up[rows], np.tile(g[o], (len(rows), 1)))
    dropped = np.setdiff1d(np.arange(nv), np.concatenate(list(mem.values())))
    assert np.all(up[dropped] == 0)
    assert rel_err(loops.avgpool_fwd(up, vt_replace, vt_map, nvo), g) < EPS        # avg(unpool(y)) = y
    _, cnt = torch_ref.cluster_maps(T(vt_replace), T(vt_map))
    gavg = loops.avgpool_bwd(g, vt_replace, vt_map)
    assert np.allclose(gavg, up / np.maximum(cnt.numpy(), 1)[:, None])            # avg bwd = unpool / count
    gf = rng.normal(size=(nv, C))
    gun = loops.unpool_bwd(gf, nvo, vt_replace, vt_map)
    for o, rows in mem.items():
        assert np.allclose(gun[o], gf[rows].sum(0))
    for a, b in [(torch_ref.avgpool_bwd(T(g), T(vt_replace), T(vt_map)), gavg),
                 (torch_ref.unpool_fwd(T(g), T(vt_replace), T(vt_map)), up),
                 (torch_ref.unpool_bwd(T(gf), nvo, T(vt_replace), T(vt_map)), gun)]:
        assert rel_err(a.numpy(), b) < EPS


def test_avg_pool_of_constant_is_constant():
    rng = np.random.default_rng(10)
    vt_replace, vt_map, nvo = S.cluster_maps(rng, 300)
    out = loops.avgpool_fwd(np.full((300, 2), 3.25), vt_replace, vt_map, nvo)
    assert np.allclose(out, 3.25)


def test_float32_loops_close_to_float64():
    """The reference-precision build of the loops stays within 1e-5 of the float64 answer."""
    v, f = mesh_case("sphere3")
    rng = np.random.default_rng(11)
    nv, nf, C, K = v.shape[0], f.shape[0], 16, 16
    ident = np.arange(nv, dtype=np.int32)
    nfc = S.vertex_facet_count(f, ident, nv)
    xf, fl, cf = rng.normal(size=(nf, C)), rng.normal(size=(K, C, 1)), rng.normal(size=(nf, K))
    a = loops.f2v_fwd(xf, fl, cf, f, nfc, ident, dtype=np.float32)
    assert a.dtype == np.float32 and rel_err(a, loops.f2v_fwd(xf, fl, cf, f, nfc, ident)) < 1e-5


def test_dense_tail_matches_torch_layers_and_hand_values():
    """The tail restatement against nn.Linear + ReLU + BatchNorm1d in eval mode (an independent spelling of
    layers.py:114-119 with torch's own modules), its explicit gradients against autograd, and a case worked by
    hand."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(37, 5, dtype=torch.float64, generator=g)
    lin = torch.nn.Linear(5, 7).double()
    bn = torch.nn.BatchNorm1d(7, eps=1e-3).double()
    with torch.no_grad():
        bn.running_mean.copy_(torch.randn(7, dtype=torch.float64, generator=g))
        bn.running_var.copy_(torch.rand(7, dtype=torch.float64, generator=g) + 0.5)
        bn.weight.copy_(torch.randn(7, dtype=torch.float64, generator=g))
        bn.bias.copy_(torch.randn(7, dtype=torch.float64, generator=g))
    bn.eval()
    w, b = lin.weight.detach().t().contiguous(), lin.bias.detach()
    scale = bn.weight.detach() / torch.sqrt(bn.running_var + bn.eps)
    shift = bn.bias.detach() - bn.running_mean * scale
    want = bn(torch.relu(lin(x))).detach()
    assert rel_err(torch_ref.dense_tail_fwd(x, w, b, True, scale, shift).numpy(), want.numpy()) < 1e-13
    assert rel_err(torch_ref.dense_tail_fwd(x, w, b, False).numpy(), lin(x).detach().numpy()) < 1e-13
    for relu in (True, False):
        xg = x.clone().requires_grad_(True)
        lin.zero_grad()
        y = torch.relu(lin(xg)) if relu else lin(xg)
        go = torch.randn(y.shape, dtype=torch.float64, generator=g)
        y.backward(go)
        gx, gw, gb = torch_ref.dense_tail_bwd(go, x, w, y.detach() if relu else None)
        assert rel_err(gx.numpy(), xg.grad.numpy()) < 1e-13
        assert rel_err(gw.numpy(), lin.weight.grad.t().numpy()) < 1e-13
        assert rel_err(gb.numpy(), lin.bias.grad.numpy()) < 1e-13
    x2 = torch.tensor([[1.0, 2.0], [-1.0, 0.5]], dtype=torch.float64)
    w2 = torch.tensor([[1.0, -1.0, 0.0], [0.5, 1.0, 2.0]], dtype=torch.float64)
    b2 = torch.tensor([0.0, -2.0, 1.0], dtype=torch.float64)
    assert torch_ref.dense_tail_fwd(x2, w2, b2, True).tolist() == [[2.0, 0.0, 5.0], [0.0, 0.0, 2.0]]
    go2 = torch.ones(2, 3, dtype=torch.float64)
    gx2, gw2, gb2 = torch_ref.dense_tail_bwd(go2, x2, w2, torch_ref.dense_tail_fwd(x2, w2, b2, True))
    assert gx2.tolist() == [[1.0, 2.5], [0.0, 2.0]]
    assert gw2.tolist() == [[1.0, 0.0, 0.0], [2.0, 0.0, 2.5]]
    assert gb2.tolist() == [1.0, 0.0, 2.0]


def test_bias_act_matches_autograd_and_hand_values():
    g = torch.Generator().manual_seed(12)
    x = torch.randn(29, 6, dtype=torch.float64, generator=g)
    b = torch.randn(6, dtype=torch.float64, generator=g)
    go = torch.randn(29, 6, dtype=torch.float64, generator=g)
    for relu in (True, False):
        xg, bg = x.clone().requires_grad_(True), b.clone().requires_grad_(True)
        y = torch.nn.functional.relu(xg + bg) if relu else xg + bg
        y.backward(go)
        assert rel_err(torch_ref.bias_act_fwd(x, b, relu).numpy(), y.detach().numpy()) < 1e-15
        gx, gb = torch_ref.bias_act_bwd(go, y.detach() if relu else None)
        assert rel_err(gx.numpy(), xg.grad.numpy()) < 1e-15 and rel_err(gb.numpy(), bg.grad.numpy()) < 1e-14
    x2 = torch.tensor([[1.0, -3.0], [0.5, 2.0]], dtype=torch.float64)
    b2 = torch.tensor([-1.0, 1.5], dtype=torch.float64)
    s2, t2 = torch.tensor([2.0, -1.0], dtype=torch.float64), torch.tensor([0.25, 0.5], dtype=torch.float64)
    assert torch_ref.bias_act_fwd(x2, b2, True, s2, t2).tolist() == [[0.25, 0.5], [0.25, -3.0]]
    gx2, gb2 = torch_ref.bias_act_bwd(torch.ones(2, 2, dtype=torch.float64), torch_ref.bias_act_fwd(x2, b2, True))
    assert gx2.tolist() == [[0.0, 0.0], [0.0, 1.0]] and gb2.tolist() == [0.0, 1.0]


def _roots(rep):
    idx = np.arange(rep.shape[0])
    return np.where(rep < 0, -rep, idx)


@pytest.mark.parametrize("spatial,orphans", [(True, 0.0), (False, 0.0), (False, 0.1)])
def test_combine_clusters_composes_the_two_steps(spatial, orphans):
    """What the combined maps must mean, stated without the reference's three passes: a fine vertex lands on
    the coarse row that step B gives to the middle vertex step A gave it, every cluster points at one member
    that survives both steps, and that member counts the others."""
    rng = np.random.default_rng(31)
    nv = 5000
    ra, ma, nmid = S.cluster_maps(rng, nv, spatial=spatial, orphan_frac=orphans)
    rb, mb, ncoarse = S.cluster_maps(rng, nmid, spatial=spatial, orphan_frac=orphans)
    rc, mc = (t.numpy() for t in torch_ref.combine_clusters(*(T(a) for a in (ra, ma, rb, mb))))
    mid = ma[_roots(ra)]                                   # middle vertex of every fine vertex, -1 if dropped
    want = np.where(mid >= 0, mb[_roots(rb)[np.maximum(mid, 0)]], -1)
    root_c = _roots(rc)
    assert np.array_equal(rc[root_c] >= 0, np.ones(nv, bool))              # roots are representatives
    live = want >= 0
    assert np.array_equal(mc[root_c][live], want[live])                    # same coarse row as the two steps
    members = np.bincount(root_c, minlength=nv)
    reps = np.nonzero((rc >= 0) & (mid >= 0) & live)[0]
    assert np.array_equal(rc[reps], members[reps] - 1)                     # the representative counts the rest
    assert np.array_equal(mc, np.where(ma >= 0, mb[np.maximum(ma, 0)], -1))


def test_combine_clusters_hand_case_and_identity():
    # fine 0..5; step A: {0}, {1,2 -> 2}, {3}, {4,5 -> 4}; middle rows 0:0, 1:2, 2:3, 3:4
    ra = np.array([0, -2, 1, 0, 1, -4], np.int32)
    ma = np.array([0, -1, 1, 2, 3, -1], np.int32)
    # step B over middle 0..3: {0}, {1,2 -> 2}, {3}; coarse rows 0:0, 1:2, 2:3
    rb = np.array([0, -2, 1, 0], np.int32)
    mb = np.array([0, -1, 1, 2], np.int32)
    rc, mc = torch_ref.combine_clusters(T(ra), T(ma), T(rb), T(mb))
    # middle 1 (fine 2, with member 1) is contracted into middle 2 (fine 3): fine 1, 2 now point at 3, which counts 2
    assert rc.tolist() == [0, -3, -3, 2, 1, -4]
    assert mc.tolist() == [0, -1, -1, 1, 2, -1]
    ident_r, ident_m = np.zeros(4, np.int32), np.arange(4, dtype=np.int32)
    rc, mc = torch_ref.combine_clusters(T(ident_r), T(ident_m), T(rb), T(mb))
    assert rc.tolist() == rb.tolist() and mc.tolist() == mb.tolist()


# ------------------------------------------------------------------ texture points from vertex features
def test_texture_interpolation_pins():
    """Hand values on one triangle, the invariants barycentric weights fix, autograd of the forward for the
    explicit backward, the adjoint identity, and agreement of the two restatements."""
    # one triangle, four points: the three corners and the centroid
    x = np.array([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]])
    face = np.array([[2, 0, 1]], np.int32)                       # corner order differs from vertex order on purpose
    bary = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1 / 3, 1 / 3, 1 / 3]])
    cum = np.array([4], np.int32)
    tex = loops.texture_fwd(x, face, bary, cum)
    assert np.allclose(tex, [[4, 40], [1, 10], [2, 20], [7 / 3, 70 / 3]], atol=EPS)
    g = np.array([[1.0, 0.0], [0.0, 1.0], [2.0, 2.0], [3.0, 6.0]])
    gin = loops.texture_bwd(g, 3, face, bary, cum)
    # vertex 0 is corner 1, vertex 1 is corner 2, vertex 2 is corner 0
    assert np.allclose(gin, [[0 + 1, 1 + 2], [2 + 1, 2 + 2], [1 + 1, 0 + 2]], atol=EPS)

    rng = np.random.default_rng(11)
    v, f = mesh_case("sphere2")
    nv, nf, C = v.shape[0], f.shape[0], 7
    counts, bary, owner = texture_case(rng, nf)                  # includes facets without points
    cum = np.cumsum(counts).astype(np.int32)
    x = rng.normal(size=(nv, C))
    tex = loops.texture_fwd(x, f, bary, cum)
    # independent statement through the owner list the generator returns
    ref = np.einsum("kj,kjc->kc", bary, x[f[owner].astype(np.int64)])
    assert rel_err(tex, ref) < EPS
    # weights sum to one: constant features stay constant, affine functions of position are reproduced
    assert np.allclose(loops.texture_fwd(np.full((nv, 2), 3.5), f, bary, cum), 3.5, atol=EPS)
    pos = loops.texture_fwd(v, f, bary, cum)
    assert rel_err(pos, np.einsum("kj,kjc->kc", bary, v[f[owner].astype(np.int64)])) < EPS
    # the torch restatement agrees, forward and backward; its backward is autograd of its forward
    xt = T(x).requires_grad_(True)
    tt = torch_ref.texture_fwd(xt, T(f), T(bary), T(cum))
    assert rel_err(tt.detach().numpy(), tex) < EPS
    g = rng.normal(size=tex.shape)
    (ga,) = torch.autograd.grad(tt, xt, T(g))
    gl = loops.texture_bwd(g, nv, f, bary, cum)
    gt = torch_ref.texture_bwd(T(g), nv, T(f), T(bary), T(cum)).numpy()
    assert rel_err(gl, ga.numpy()) < EPS and rel_err(gt, ga.numpy()) < EPS
    assert abs((tex * g).sum() - (x * gl).sum()) < 1e-9 * abs((tex * g).sum())
    # float32 loops stay close to float64
    assert rel_err(loops.texture_fwd(x, f, bary, cum, np.float32), tex) < 1e-6


def test_oriented_normals_pins():
    """Hand case, an element-by-element restatement, and what orientation towards the origin means."""
    v = T(np.array([[1.0, 0, 2], [0, 1, 2], [0, 0, 2], [1, 0, -3], [0, 1, -3], [0, 0, -3]]))
    f = T(np.array([[0, 1, 2], [3, 4, 5], [2, 1, 0]], np.int32))
    n = torch_ref.face_normals(v, f)
    assert np.allclose(n.numpy(), [[0, 0, 1], [0, 0, 1], [0, 0, -1]], atol=EPS)
    o = torch_ref.oriented_normals(n, v, f).numpy()
    # facets above the origin look down, the one below looks up, whatever the winding
    assert np.allclose(o, [[0, 0, -1], [0, 0, 1], [0, 0, -1]], atol=EPS)
    # a plane through the origin (-centre . n = 0) keeps its normal
    v0 = T(np.array([[1.0, 0, 0], [0, 1, 0], [-1, -1, 0]]))
    f0 = T(np.array([[0, 1, 2]], np.int32))
    n0 = torch_ref.face_normals(v0, f0)
    assert np.array_equal(torch_ref.oriented_normals(n0, v0, f0).numpy(), n0.numpy())
    rng = np.random.default_rng(31)
    vv, ff = mesh_case("room_small")
    vv = vv + rng.normal(0, 1, 3)                                   # origin somewhere inside the scene
    n = torch_ref.face_normals(T(vv), T(ff))
    o = torch_ref.oriented_normals(n, T(vv), T(ff)).numpy()
    centre = vv[ff.astype(np.int64)].mean(1)
    for i in range(0, ff.shape[0], 7):                             # the reference's rule, one facet at a time
        s = np.sign(-(centre[i] * n[i].numpy()).sum())
        assert np.array_equal(o[i], n[i].numpy() * (s if s == -1 else 1.0))
    assert ((centre * o).sum(1) <= 1e-12).all()                     # every normal faces the origin
    assert np.allclose(np.abs(o), np.abs(n.numpy()))
    assert np.array_equal(torch_ref.oriented_normals(T(o), T(vv), T(ff)).numpy(), o)    # idempotent
    assert (o != n.numpy()).any() and (o == n.numpy()).all(1).any()
