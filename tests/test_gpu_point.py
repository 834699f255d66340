"""The point-cloud branch on the GPU against oracle/point_ref.py, through the reference-shaped API.

Searches, sampling and arg-max indices bit-exact (the device compares the same float32 distances, each operation
rounded on its own); kernel bins exact away from bin borders, fuzzy weights within 1e-5; convolution, pooling and
unpooling outputs and gradients within 1e-5 of the float64 oracle."""
import sys

import numpy as np
import pytest
import torch

from oracle import point_ref as P
from picassoplus_amd import _lib
from picassoplus_amd.point import layers as point_layers
from picassoplus_amd.point import utils as point_utils
from picassoplus_amd.point.pi_modules import (buildkernel, conv3d, nnquery, point_nnquery, point_pool3d, pool3d, sample,
                                               unpool3d)
from test_oracle_point import cloud, subsample
from util import assert_close, dev

pytestmark = pytest.mark.gpu
I32, F32 = torch.int32, torch.float32


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def n(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("sizes,frac,radius,limit", [([300, 1, 120], 0.4, 0.2, None), ([2000, 1500], 1.0, 0.12, None),
                                                     ([500], 0.5, 0.3, 7), ([64, 64, 64, 64, 64], 1.0, 0.5, 1),
                                                     ([4000], 0.25, 0.05, None)])
@pytest.mark.parametrize("grid", [False, True])
def test_range_cube_knn_bit_exact(cuda, monkeypatch, sizes, frac, radius, limit, grid):
    say("case point search", sizes, frac, radius, limit, "grid" if grid else "scan")
    monkeypatch.setattr(point_nnquery, "GRID_MIN_POINTS", 0 if grid else 1 << 40)
    db, nvd = cloud(21, sizes)
    q, nvq = (db, nvd) if frac == 1.0 else subsample(22, db, nvd, frac)
    D, Q, ND, NQ = dev(db, cuda), dev(q, cuda), dev(nvd, cuda), dev(nvq, cuda)
    cnt_info, nn_count, nn_index, nn_dist = nnquery.range_search_(D, Q, ND, NQ, radius=radius, nnsample=limit)
    w = P.range_search(db, q, np.cumsum(nvd), np.cumsum(nvq), radius, 2147483647 if limit is None else limit)
    assert cnt_info.dtype == torch.int64 and nn_count.dtype == I32 and nn_index.dtype == I32
    assert np.array_equal(n(cnt_info), w[0]) and np.array_equal(n(nn_count), w[1])
    assert np.array_equal(n(nn_index), w[2]) and np.array_equal(n(nn_dist), w[3])
    cnt_info, nn_count, nn_index = nnquery.cube_search_(D, Q, ND, NQ, length=2 * radius, nnsample=limit, gridsize=3)
    w = P.cube_search(db, q, np.cumsum(nvd), np.cumsum(nvq), 2 * radius, 2147483647 if limit is None else limit, 3)
    assert np.array_equal(n(cnt_info), w[0]) and np.array_equal(n(nn_count), w[1]) and np.array_equal(n(nn_index), w[2])
    nn3, d3 = nnquery.knn3_search_(D, Q, ND, NQ)
    w = P.knn3_search(db, q, np.cumsum(nvd), np.cumsum(nvq))
    assert np.array_equal(n(nn3), w[0]) and np.array_equal(n(d3), w[1])
    # extra feature columns of the point arrays are ignored
    wide = torch.cat([D, torch.ones_like(D)], 1)
    again = nnquery.range_search_(wide, Q, ND, NQ, radius=radius, nnsample=limit)
    assert torch.equal(again[2], nnquery.range_search_(D, Q, ND, NQ, radius=radius, nnsample=limit)[2])


def _searches(D, Q, ND, NQ, radius, limit):
    a = nnquery.range_search_(D, Q, ND, NQ, radius=radius, nnsample=limit)
    b = nnquery.cube_search_(D, Q, ND, NQ, length=2 * radius, nnsample=limit, gridsize=4)
    c = nnquery.knn3_search_(D, Q, ND, NQ)
    return [n(t) for t in a + b + c]


@pytest.mark.parametrize("shape", ["plane", "far", "same", "spread", "nonfinite", "outside", "dense", "dense_all"])
def test_grid_search_matches_scan(cuda, monkeypatch, shape):
    """The cell-grid searches return what the scans return (which the test above holds against the oracle), also where
    the grid degenerates: no extent on an axis, coordinates far from the origin (coarse float spacing), all points
    equal, an extent so large that the cells grow, coordinates that are not finite, queries outside the database's
    bounding box, more neighbours than the limit keeps (the lowest indices must survive, in order), and more neighbours
    per query than the search kernel buffers, all of them kept."""
    say("case grid search", shape)
    rng = np.random.default_rng(77)
    sizes, radius, limit = ([500, 300] if shape == "dense_all" else [1500, 900]), 0.15, None
    db, nvd = cloud(31, sizes)
    q, nvq = subsample(32, db, nvd, 0.5)
    if shape == "plane":
        db[:, 2] = 0.25
        q[:, 2] = 0.25
    elif shape == "far":
        db += np.float32(4096.0)
        q += np.float32(4096.0)
    elif shape == "same":
        db[:] = db[0]
        q[:] = db[0]
        limit = 40
    elif shape == "spread":
        db[::50] *= np.float32(3.0e6)
    elif shape == "nonfinite":
        db[5] = np.nan
        db[17, 1] = np.inf
        db[400, 0] = -np.inf
        q[3] = np.nan
        q[9, 2] = np.inf
    elif shape == "outside":
        q = (q + rng.uniform(-2.0, 2.0, q.shape)).astype(np.float32)
    elif shape == "dense":
        radius, limit = 0.6, 9
    elif shape == "dense_all":
        radius = 0.6
    D, Q, ND, NQ = dev(db, cuda), dev(q, cuda), dev(nvd, cuda), dev(nvq, cuda)
    monkeypatch.setattr(point_nnquery, "GRID_MIN_POINTS", 1 << 40)
    want = _searches(D, Q, ND, NQ, radius, limit)
    monkeypatch.setattr(point_nnquery, "GRID_MIN_POINTS", 0)
    got = _searches(D, Q, ND, NQ, radius, limit)
    assert want[0][-1] > 0 or shape == "nonfinite"
    for a, b in zip(want, got):
        assert a.dtype == b.dtype and np.array_equal(a, b, equal_nan=True)


@pytest.mark.parametrize("limit", [None, 300, 20])
def test_grid_search_with_more_neighbours_than_any_buffer(cuda, monkeypatch, limit):
    """4500 database points inside the reach of three queries: more than the per-query buffers of the fill kernels
    hold (128 and 258 places in the first, 4096 in the one for long segments), kept all, cut to a long segment, cut
    to a short one."""
    say("case grid search crowd", limit)
    rng = np.random.default_rng(5)
    db = (0.5 + 0.01 * rng.standard_normal((4500, 3))).astype(np.float32)
    db = np.concatenate([db, cloud(6, [600])[0]])
    q = np.array([[0.5, 0.5, 0.5], [0.51, 0.5, 0.49], [0.9, 0.1, 0.2]], np.float32)
    nvd, nvq = np.array([db.shape[0]], np.int32), np.array([3], np.int32)
    D, Q, ND, NQ = dev(db, cuda), dev(q, cuda), dev(nvd, cuda), dev(nvq, cuda)
    monkeypatch.setattr(point_nnquery, "GRID_MIN_POINTS", 1 << 40)
    want = _searches(D, Q, ND, NQ, 0.2, limit)
    monkeypatch.setattr(point_nnquery, "GRID_MIN_POINTS", 0)
    got = _searches(D, Q, ND, NQ, 0.2, limit)
    assert want[1].max() > 4096 or limit is not None
    for a, b in zip(want, got):
        assert a.dtype == b.dtype and np.array_equal(a, b)


def test_grid_search_beyond_the_reach_it_was_built_for(cuda):
    """A search that reaches further than the cells are wide looks at more cells: through the C-ABI, a grid built for a
    tenth of the radius."""
    from picassoplus_amd import _lib
    db, nvd = cloud(41, [1200])
    D, ND = dev(db, cuda), dev(np.cumsum(nvd).astype(np.int32), cuda)
    Np, radius = db.shape[0], 0.2
    ws = torch.empty(_lib.query("pmesh_point_grid_workspace_bytes", Np), dtype=torch.uint8, device=cuda)
    _lib.call("pmesh_point_grid_build", D.data_ptr(), ND.data_ptr(), 1, Np, radius / 10, ws.data_ptr(), ws.numel(), None)
    count = torch.zeros(Np, dtype=I32, device=cuda)
    _lib.call("pmesh_point_range_count_grid", ws.data_ptr(), D.data_ptr(), D.data_ptr(), ND.data_ptr(), ND.data_ptr(), 1, Np, Np,
              radius, 2147483647, count.data_ptr(), None)
    w = P.range_search(db, db, np.cumsum(nvd), np.cumsum(nvd), radius, 2147483647)
    assert np.array_equal(n(count), w[1])
    cnt_info = torch.cumsum(count, 0, dtype=torch.int64)
    n_out = int(cnt_info[-1])
    nn_index = torch.empty((n_out, 2), dtype=I32, device=cuda)
    nn_dist = torch.empty(n_out, dtype=F32, device=cuda)
    _lib.call("pmesh_point_range_fill_grid", ws.data_ptr(), D.data_ptr(), D.data_ptr(), ND.data_ptr(), ND.data_ptr(), 1, Np, Np,
              radius, cnt_info.data_ptr(), n_out, nn_index.data_ptr(), nn_dist.data_ptr(), None)
    assert np.array_equal(n(nn_index), w[2]) and np.array_equal(n(nn_dist), w[3])


@pytest.mark.parametrize("sizes,keep", [([120, 60], [15, 60]), ([3000], [700]), ([1, 5, 2048], [1, 3, 256]),
                                        # a sample beyond the 16 384 points that the kernel holds in registers
                                        ([17000, 300], [40, 20])])
def test_fps_bit_exact(cuda, sizes, keep):
    say("case point fps", sizes, keep)
    xyz, nv = cloud(23, sizes)
    m = np.array(keep, np.int32)
    got = sample.fps_(dev(xyz, cuda), dev(nv, cuda), dev(m, cuda))
    assert got.dtype == I32 and np.array_equal(n(got), P.fps(xyz, np.cumsum(nv), np.cumsum(m)))


@pytest.mark.parametrize("kernel", [(8, 2, 3), (8, 4, 1), (4, 2, 2)])
def test_kernel_bins(cuda, kernel):
    say("case point bins", kernel)
    db, nvd = cloud(24, [1500, 900])
    q, nvq = subsample(25, db, nvd, 0.3)
    radius = 0.25
    _, _, nn_index, nn_dist = P.range_search(db, q, np.cumsum(nvd), np.cumsum(nvq), radius)
    D, Q, NI, ND = dev(db, cuda), dev(q, cuda), dev(nn_index, cuda), dev(nn_dist, cuda)
    got = n(buildkernel.SPH3Dkernel_(D, Q, NI, ND, radius, kernel=list(kernel)))
    want, (al, be, ga) = P.sph3d_kernel(db, q, nn_index, nn_dist, radius, kernel)
    # a pair within 1e-4 of a bin border (or of the centre radius) may fall on either side of it
    frac = lambda v: np.abs(v - np.round(v))
    away = (frac(al) > 1e-4) & (frac(be) > 1e-4) & (frac(ga) > 1e-4)
    centre = nn_dist < 0.3 * radius - 1e-6                            # bin 0 whatever the direction (a point paired with itself too)
    clear = centre | (away & (nn_dist > 0.3 * radius + 1e-6))
    assert clear.mean() > 0.99 and np.array_equal(got[clear], want[clear])
    assert got.min() >= 0 and got.max() <= kernel[0] * kernel[1] * kernel[2]
    fi, fc = buildkernel.fuzzySPH3Dkernel_(D, Q, NI, ND, radius, kernel=list(kernel))
    wi, wc, _ = P.fuzzy_sph3d_kernel(db, q, nn_index, nn_dist, radius, kernel)
    clear = away & (nn_dist > 0) & (np.abs(frac(be) - 0.5) > 1e-4)     # also clear of the side the pair leans to
    assert clear.mean() > 0.97
    assert np.abs(n(fc) - wc).max() < 1e-5 or np.abs(n(fc)[clear] - wc[clear]).max() < 1e-5
    assert np.array_equal(n(fi)[clear], wi[clear]) and np.abs(n(fc)[clear] - wc[clear]).max() < 1e-5
    assert np.allclose(n(fc).sum(1), 1, atol=1e-5)


def point_graph(cuda, seed, sizes, radius, T, F, limit=None):
    rng = np.random.default_rng(seed)
    db, nvd = cloud(seed, sizes)
    q, nvq = subsample(seed + 1, db, nvd, 0.5)
    _, count, nn_index, nn_dist = P.range_search(db, q, np.cumsum(nvd), np.cumsum(nvq), radius, 2147483647 if limit is None else limit)
    if T is None:
        bins, coeff = rng.integers(0, F, len(nn_index)).astype(np.int32), None
    else:
        bins = rng.integers(0, F, (len(nn_index), T)).astype(np.int32)
        coeff = rng.uniform(0, 1, (len(nn_index), T)).astype(np.float32)
    return db, q, count, nn_index, nn_dist, bins, coeff


@pytest.mark.parametrize("sizes,radius,C,r,F,T", [([60], 0.45, 5, 1, 7, None), ([60], 0.45, 5, 2, 7, 3), ([800, 500], 0.2, 64, 1, 17, 17),
                                                  ([2000], 0.15, 32, 2, 33, 3), ([300], 0.3, 130, 1, 49, None),
                                                  ([500], 0.25, 16, 1, 125, 1), ([400], 0.25, 8, 3, 300, 2),
                                                  # filter in registers: 16 / 20 / 32 / 36 bins, several table chunks per workgroup
                                                  ([700], 0.25, 64, 1, 33, 3), ([500], 0.3, 128, 1, 20, 6), ([400], 0.3, 12, 1, 36, None),
                                                  ([1500], 0.3, 256, 1, 26, 5), ([900, 40], 0.2, 128, 1, 10, 4),
                                                  ([700], 0.25, 32, 1, 8, None), ([600], 0.3, 36, 1, 32, 2)])
def test_conv_parity(cuda, sizes, radius, C, r, F, T):
    say("case point conv", sizes, radius, C, r, F, T)
    db, q, count, nn_index, _, bins, coeff = point_graph(cuda, 31, sizes, radius, T, F)
    rng = np.random.default_rng(32)
    x, filt = rng.normal(size=(len(db), C)), rng.normal(0, 0.3, (F, C, r))
    g = rng.normal(size=(len(q), C * r))
    out_ref = P.conv_fwd(x, filt, count, nn_index, bins, coeff)
    gin_ref, gfilt_ref = P.conv_bwd(g, x, filt, count, nn_index, bins, coeff)
    xt, ft = dev(x, cuda, F32).requires_grad_(True), dev(filt, cuda, F32).requires_grad_(True)
    args = (dev(count, cuda), dev(nn_index, cuda), dev(bins, cuda))
    out = conv3d.conv3d(xt, ft, *args) if coeff is None else conv3d.fuzzyconv3d(xt, ft, *args, dev(coeff, cuda))
    out.backward(dev(g, cuda, F32))
    torch.cuda.synchronize()
    assert_close(out, out_ref, "point conv out")
    assert_close(xt.grad, gin_ref, "point conv grad_input")
    assert_close(ft.grad, gfilt_ref, "point conv grad_filter")
    # same bits on a second run
    xt2, ft2 = xt.detach().clone().requires_grad_(True), ft.detach().clone().requires_grad_(True)
    out2 = conv3d.conv3d(xt2, ft2, *args) if coeff is None else conv3d.fuzzyconv3d(xt2, ft2, *args, dev(coeff, cuda))
    out2.backward(dev(g, cuda, F32))
    assert torch.equal(out, out2) and torch.equal(xt.grad, xt2.grad) and torch.equal(ft.grad, ft2.grad)


@pytest.mark.parametrize("sizes,radius,C,F,T", [([800, 500], 0.2, 64, 17, 17), ([500], 0.3, 128, 20, 6), ([900, 40], 0.2, 128, 10, 4),
                                                ([700], 0.25, 32, 8, None), ([400], 0.25, 8, 12, 2), ([300, 1, 90], 0.3, 4, 16, 3),
                                                ([3000], 0.12, 20, 5, 2)])
def test_conv_backward_in_one_pass_and_in_two(cuda, native_options, sizes, radius, C, F, T):
    """Shapes the one-pass backward takes (depth multiplier 1, at most 20 bins and 128 channels, from one row per
    wavefront to 32): both gradients against the oracle, and against the separate input- and filter-gradient passes."""
    say("case point conv backward", sizes, radius, C, F, T)
    db, q, count, nn_index, _, bins, coeff = point_graph(cuda, 41, sizes, radius, T, F)
    rng = np.random.default_rng(42)
    x, filt = rng.normal(size=(len(db), C)), rng.normal(0, 0.3, (F, C, 1))
    g = rng.normal(size=(len(q), C))
    gin_ref, gfilt_ref = P.conv_bwd(g, x, filt, count, nn_index, bins, coeff)
    args = (dev(count, cuda), dev(nn_index, cuda), dev(bins, cuda))
    grads = {}
    for two in (False, True):
        if two:
            native_options(PMESH_POINT_CONV_TWO_PASSES="1")
        seen = []
        _lib.set_call_hook(lambda name, phase: seen.append(name))
        xt, ft = dev(x, cuda, F32).requires_grad_(True), dev(filt, cuda, F32).requires_grad_(True)
        out = conv3d.conv3d(xt, ft, *args) if coeff is None else conv3d.fuzzyconv3d(xt, ft, *args, dev(coeff, cuda))
        out.backward(dev(g, cuda, F32))
        torch.cuda.synchronize()
        _lib.set_call_hook(None)
        assert "pmesh_point_conv_bwd" in seen
        label = "two passes" if two else "one pass"
        assert_close(xt.grad, gin_ref, "point conv grad_input [%s]" % label)
        assert_close(ft.grad, gfilt_ref, "point conv grad_filter [%s]" % label)
        grads[two] = (xt.grad, ft.grad)
    assert_close(grads[False][0], grads[True][0].double().cpu().numpy(), "point conv grad_input one pass vs two")
    assert_close(grads[False][1], grads[True][1].double().cpu().numpy(), "point conv grad_filter one pass vs two")


@pytest.mark.parametrize("sizes,radius,C", [([60], 0.45, 4), ([1500, 700], 0.2, 64), ([900], 0.25, 37)])
def test_pool_and_unpool_parity(cuda, sizes, radius, C):
    say("case point pool", sizes, radius, C)
    db, q, count, nn_index, nn_dist, _, _ = point_graph(cuda, 41, sizes, radius, None, 3)
    rng = np.random.default_rng(42)
    x = rng.normal(size=(len(db), C)).astype(np.float32)
    x[5] = x[9]
    g = rng.normal(size=(len(q), C)).astype(np.float32)
    CT, NI = dev(count, cuda), dev(nn_index, cuda)
    xt = dev(x, cuda).requires_grad_(True)
    mx = pool3d.maxPool(xt, CT, NI)
    mx.backward(dev(g, cuda))
    w_mx, w_idx = P.pool_max_fwd(x, count, nn_index)
    out, idx = point_pool3d.max_forward(xt.detach(), CT, NI)
    assert np.array_equal(n(mx), w_mx) and np.array_equal(n(idx), w_idx) and torch.equal(out, mx.detach())
    assert_close(xt.grad, P.pool_max_bwd(g.astype(np.float64), len(db), w_idx), "point max pool grad")
    xt.grad = None
    av = pool3d.avgPool(xt, CT, NI)
    av.backward(dev(g, cuda))
    assert_close(av, P.pool_avg_fwd(x, count, nn_index), "point avg pool")
    assert_close(xt.grad, P.pool_avg_bwd(g, len(db), count, nn_index), "point avg pool grad")
    with pytest.raises(RuntimeError):
        point_pool3d.max_backward(dev(g, cuda), xt.detach(), idx)       # the gather form needs the pairs
    # unpooling from the queries back to the database points
    nn3, d3 = P.knn3_search(q, db, np.cumsum([max(1, int(s * 0.5)) for s in sizes]), np.cumsum(sizes))
    w = (1 / (d3 + 1e-8)).astype(np.float32)
    w = w / w.sum(1, keepdims=True)
    y = rng.normal(size=(len(q), C)).astype(np.float32)
    yt = dev(y, cuda).requires_grad_(True)
    up = unpool3d.interpolate(yt, dev(w, cuda), dev(nn3, cuda))
    gu = rng.normal(size=(len(db), C)).astype(np.float32)
    up.backward(dev(gu, cuda))
    assert_close(up, P.unpool_fwd(y, w, nn3), "point unpool")
    assert_close(yt.grad, P.unpool_bwd(gu, len(q), w, nn3), "point unpool grad")


def test_dual_block_graph_and_module(cuda):
    """What DualBlock does with the point branch (picasso/networks/pi2_blocks.py:43-62): the spherical-harmonic graph
    of a vertex set on itself, then PCloudConv3d on it, against the oracle composition."""
    say("case point module")
    xyz, nv = cloud(51, [700, 400], scale=1.0)
    L, radius, limit = 3, 0.2, 20
    X, NV = dev(xyz, cuda), dev(nv, cuda)
    nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff = point_utils.build_sphere_harmonics(X, X, NV, NV, radius, L=L, nn_uplimit=limit)
    w = P.range_search(xyz, xyz, np.cumsum(nv), np.cumsum(nv), radius, limit)
    assert np.array_equal(n(nn_cnt), w[1]) and np.array_equal(n(nn_idx), w[2]) and np.array_equal(n(nn_dst), w[3])
    assert int(nn_cnt.max()) <= limit and int(nn_cnt.min()) >= 1      # every point finds itself
    K = (L + 1) ** 2 + 1
    assert tuple(filt_idx.shape) == (len(w[2]), K) and filt_idx.dtype == I32 and torch.equal(filt_idx[0], torch.arange(K, dtype=I32, device=cuda))
    from oracle import loops
    delta = xyz[w[2][:, 1]].astype(np.float64) - xyz[w[2][:, 0]].astype(np.float64)
    gamma = np.clip(w[3].astype(np.float64) / radius, 0, 1)[:, None]
    # a pair of a point with itself has no direction: the basis is evaluated at (1, 0, 0), as atan2(0, 0) = 0 makes the reference do
    sh = loops.sph_harm(np.where((np.abs(delta).sum(1) == 0)[:, None], [[1.0, 0, 0]], delta), L)
    coeff_ref = np.concatenate([1 - gamma, gamma * sh], 1)
    assert np.abs(n(filt_coeff) - coeff_ref).max() < 2e-6
    torch.manual_seed(0)
    conv = point_layers.PCloudConv3d(24, 40, K, with_bn=False).to(cuda)
    feat = torch.randn(len(xyz), 24, device=cuda, requires_grad=True)
    out = conv(feat, nn_cnt, nn_idx, filt_idx, filt_coeff)
    g = torch.randn_like(out)
    out.backward(g)
    f64 = lambda t: n(t).astype(np.float64)
    mid = P.conv_fwd(f64(feat), f64(conv.spatial_weights), w[1], w[2], n(filt_idx), f64(filt_coeff))
    z = mid @ f64(conv.depth_weights) + f64(conv.biases)
    assert_close(out, np.maximum(z, 0), "PCloudConv3d out")
    gz = f64(g) * (z > 0)
    gmid = gz @ f64(conv.depth_weights).T
    gin, gfilt = P.conv_bwd(gmid, f64(feat), f64(conv.spatial_weights), w[1], w[2], n(filt_idx), f64(filt_coeff))
    assert_close(feat.grad, gin, "PCloudConv3d grad input")
    assert_close(conv.spatial_weights.grad, gfilt, "PCloudConv3d grad spatial")
    assert_close(conv.depth_weights.grad, mid.T @ gz, "PCloudConv3d grad depth")
    # the other two graph builders
    g_rng = point_utils.build_range_graph(X, X, NV, NV, radius, nn_uplimit=limit, kernel_shape=[8, 4, 1], fuzzy=True)
    assert tuple(g_rng[3].shape) == (len(w[2]), 3) and torch.equal(g_rng[1], nn_idx)
    g_cube = point_utils.build_cube_graph(X, X, NV, NV, radius, nn_uplimit=limit, grid_size=3)
    assert g_cube[1].shape[1] == 2 and g_cube[3].dim() == 1 and int(g_cube[3].max()) < 27
    plain = point_layers.PCloudConv3d(24, 8, 27, with_bn=True).to(cuda)
    y = plain(feat.detach(), g_cube[0], g_cube[1], g_cube[3])
    assert tuple(y.shape) == (len(xyz), 8) and bool(torch.isfinite(y).all())


def test_point_block_step_replays_from_a_hip_graph(cuda):
    """Forward and backward of the point branch of a dual block (fuzzy convolution with its tail, max pooling to a
    sampled set, interpolation back; the graphs built beforehand) recorded once as a HIP graph: every replay equals the
    eager step on the inputs then in the static buffers, with eager steps between the replays."""
    say("case point graph replay")
    xyz, nv = cloud(61, [900, 500], scale=1.0)
    L, radius, C = 3, 0.2, 32
    X, NV = dev(xyz, cuda), dev(nv, cuda)
    nn_cnt, nn_idx, _, filt_idx, filt_coeff = point_utils.build_sphere_harmonics(X, X, NV, NV, radius, L=L, nn_uplimit=16)
    NQ = dev((nv // 4).astype(np.int32), cuda)
    picked = sample.fps_(X, NV, NQ)
    Q = X[picked.long()].contiguous()
    _, pcnt, pidx, _ = nnquery.range_search_(X, Q, NV, NQ, radius=2 * radius, nnsample=32)
    nn3, d3 = nnquery.knn3_search_(Q, X, NQ, NV)
    w3 = point_utils.compute_unpool_weight(d3)
    torch.manual_seed(5)
    conv = point_layers.PCloudConv3d(C, C, (L + 1) ** 2 + 1, with_bn=False).to(cuda)
    params = list(conv.parameters())
    static_x = torch.randn(len(xyz), C, device=cuda, requires_grad=True)
    static_g = torch.randn(len(xyz), C, device=cuda)

    def step(x, g):
        y = conv(x, nn_cnt, nn_idx, filt_idx, filt_coeff)
        p = pool3d.maxPool(y, pcnt, pidx)
        z = y + unpool3d.interpolate(p, w3, nn3)
        return [z] + list(torch.autograd.grad(z, [x] + params, g))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(static_x, static_g)                            # warm-up: the pair orders are cached now
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_x, static_g)
    for i in range(3):
        gen = torch.Generator(device=cuda).manual_seed(300 + i)
        x = torch.randn(len(xyz), C, device=cuda, generator=gen)
        g = torch.randn(len(xyz), C, device=cuda, generator=gen)
        with torch.no_grad():
            static_x.copy_(x)
            static_g.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        eager = step(x.requires_grad_(True), g)
        torch.cuda.synchronize()
        for k, (a, b) in enumerate(zip(got, eager)):
            assert torch.equal(a, b), "replay %d: result %d differs from the eager step" % (i, k)


def test_point_argument_errors(cuda):
    say("case point errors")
    db, nvd = cloud(61, [50])
    D, ND = dev(db, cuda), dev(nvd, cuda)
    with pytest.raises(RuntimeError):
        nnquery.range_search_(D.cpu(), D, ND, ND, radius=0.1)
    with pytest.raises(RuntimeError):
        nnquery.range_search_(D, D, ND, ND, radius=-1.0)
    with pytest.raises(RuntimeError):
        point_nnquery.range(D, D, ND.long(), ND, 0.1, 5)               # the native layer takes int32 totals only
    _, cnt, idx, dst = nnquery.range_search_(D, D, ND, ND, radius=0.3)
    with pytest.raises(RuntimeError):
        buildkernel.SPH3Dkernel_(D, D, idx, dst, 0.3, kernel=[7, 2, 3])          # odd azimuth count
    x = torch.randn(50, 4, device=cuda)
    with pytest.raises(RuntimeError):
        conv3d.conv3d(x, torch.randn(3, 5, 1, device=cuda), cnt, idx, torch.zeros(len(idx), dtype=I32, device=cuda))
    with pytest.raises(RuntimeError):
        conv3d.conv3d(x, torch.randn(3, 4, 1, device=cuda), cnt, idx, torch.zeros(len(idx), dtype=torch.int64, device=cuda))
    # empty inputs
    e = nnquery.range_search_(D, D[:0], ND, ND * 0, radius=0.1)
    assert e[2].shape == (0, 2) and e[1].shape == (0,)
