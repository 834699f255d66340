"""Pins oracle/point_ref.py without a GPU.

The reference holds no fixtures for its point-cloud branch, so each function is pinned by something that does not
retype it: scipy's k-d tree for the searches, a brute-force statement of farthest point sampling, hand-placed
directions for the kernel bins, pure-Python loops on tiny inputs and autograd of a torch statement of the forward for
the convolution, pooling and unpooling gradients.
"""
import numpy as np
import pytest
import torch
from scipy.spatial import cKDTree

from oracle import point_ref as P


def cloud(seed, sizes, scale=1.0):
    rng = np.random.default_rng(seed)
    pts = [rng.uniform(0, scale, (n, 3)).astype(np.float32) + np.float32(10 * b) for b, n in enumerate(sizes)]
    return np.concatenate(pts), np.array(sizes, np.int32)


def subsample(seed, xyz, nv, frac):
    rng = np.random.default_rng(seed)
    out, cnt, start = [], [], 0
    for n in nv:
        k = max(1, int(n * frac))
        out.append(xyz[start + np.sort(rng.choice(n, k, replace=False))])
        cnt.append(k)
        start += n
    return np.concatenate(out), np.array(cnt, np.int32)


# ------------------------------------------------------------------ searches
@pytest.mark.parametrize("seed,limit", [(0, None), (1, 5), (2, 1)])
def test_range_search_matches_kdtree(seed, limit):
    db, nvd = cloud(seed, [300, 1, 120])
    q, nvq = subsample(seed, db, nvd, 0.4)
    radius = 0.2
    cnt_info, nn_count, nn_index, nn_dist = P.range_search(db, q, np.cumsum(nvd), np.cumsum(nvq), radius,
                                                           2147483647 if limit is None else limit)
    assert cnt_info[-1] == len(nn_index) == nn_count.sum() and np.array_equal(np.cumsum(nn_count), cnt_info)
    d0 = np.concatenate([[0], np.cumsum(nvd)])
    q0 = np.concatenate([[0], np.cumsum(nvq)])
    at = 0
    for b in range(len(nvd)):
        tree = cKDTree(db[d0[b]:d0[b + 1]].astype(np.float64))
        for j in range(q0[b], q0[b + 1]):
            got = nn_index[at:at + nn_count[j]]
            assert np.all(got[:, 0] == j)
            # neighbours whose distance is within rounding of the radius may fall on either side of a float64 tree query
            d = np.linalg.norm(db[d0[b]:d0[b + 1]].astype(np.float64) - q[j].astype(np.float64), axis=1)
            sure = np.nonzero(d < radius * (1 - 1e-6))[0] + d0[b]
            maybe = np.nonzero(d < radius * (1 + 1e-6))[0] + d0[b]
            assert set(sure) == set(i + d0[b] for i in tree.query_ball_point(q[j].astype(np.float64), radius * (1 - 1e-6)))
            if limit is None:
                assert set(sure) <= set(got[:, 1]) <= set(maybe)
            else:
                assert len(got) == min(limit, len(got)) and len(got) <= limit
                assert list(got[:, 1]) == sorted(got[:, 1]) and set(got[:, 1]) <= set(maybe)
                if len(sure) >= limit and len(sure) == len(maybe):
                    assert list(got[:, 1]) == sorted(sure)[:limit]          # the FIRST ones in database order
            assert np.all(np.diff(got[:, 1]) > 0)
            assert np.allclose(nn_dist[at:at + nn_count[j]], d[got[:, 1] - d0[b]], rtol=1e-5, atol=1e-7)
            at += nn_count[j]


def test_cube_search_hand_case_and_invariants():
    # query at the origin, cube of edge 2, 4 cells per axis of width 0.5: cell = floor((d + 1) / 0.5)
    db = np.array([[0.1, 0.1, 0.1], [-0.9, 0.9, 0.3], [1.5, 0, 0], [0.99, -0.99, -0.01], [0, 0, 1.0]], np.float32)
    q = np.zeros((1, 3), np.float32)
    cnt, count, idx = P.cube_search(db, q, [5], [1], 2.0, grid_size=4)
    assert count.tolist() == [3] and cnt.tolist() == [3]
    assert idx.tolist() == [[0, 0, (2 * 4 + 2) * 4 + 2], [0, 1, (0 * 4 + 3) * 4 + 2], [0, 3, (3 * 4 + 0) * 4 + 1]]
    # random: inside exactly when the Chebyshev distance is below half the edge; cells within range; limit keeps the first
    db, nvd = cloud(3, [200, 150])
    qq, nvq = subsample(3, db, nvd, 0.3)
    cnt, count, idx = P.cube_search(db, qq, np.cumsum(nvd), np.cumsum(nvq), 0.4, grid_size=3)
    assert idx[:, 2].min() >= 0 and idx[:, 2].max() < 27
    cheb = np.abs(db[idx[:, 1]] - qq[idx[:, 0]]).max(1)
    assert np.all(cheb < 0.2)
    total = 0
    d0 = np.concatenate([[0], np.cumsum(nvd)])
    q0 = np.concatenate([[0], np.cumsum(nvq)])
    for b in range(2):
        c = np.abs(db[None, d0[b]:d0[b + 1]] - qq[q0[b]:q0[b + 1], None]).max(2)
        total += int((c < np.float32(0.2)).sum())
    assert total == len(idx)
    _, count2, idx2 = P.cube_search(db, qq, np.cumsum(nvd), np.cumsum(nvq), 0.4, 2, 3)
    assert count2.max() <= 2 and np.array_equal(count2, np.minimum(count, 2))
    first_two = np.concatenate([idx[idx[:, 0] == j][:2] for j in range(len(qq))])
    assert np.array_equal(idx2, first_two)


def test_knn3_matches_kdtree_and_short_samples():
    db, nvd = cloud(4, [250, 2, 90])
    q, nvq = cloud(5, [40, 3, 25])
    idx, dst = P.knn3_search(db, q, np.cumsum(nvd), np.cumsum(nvq))
    d0 = np.concatenate([[0], np.cumsum(nvd)])
    q0 = np.concatenate([[0], np.cumsum(nvq)])
    for b in (0, 2):
        tree = cKDTree(db[d0[b]:d0[b + 1]].astype(np.float64))
        dd, ii = tree.query(q[q0[b]:q0[b + 1]].astype(np.float64), k=3)
        assert np.array_equal(idx[q0[b]:q0[b + 1]], ii + d0[b])
        assert np.allclose(dst[q0[b]:q0[b + 1]], dd, rtol=1e-5)
    # a sample with two points: the third slot keeps the sample's first point and an infinite distance
    short = idx[q0[1]:q0[2]]
    assert set(short[:, :2].ravel()) <= {d0[1], d0[1] + 1} and np.all(short[:, 2] == d0[1])
    assert np.all(np.isinf(dst[q0[1]:q0[2], 2])) and np.all(np.isfinite(dst[q0[1]:q0[2], :2]))
    assert np.all(dst[:, 0] <= dst[:, 1]) and np.all(dst[:, 1] <= dst[:, 2])


def test_fps_is_the_greedy_max_min_choice():
    xyz, nv = cloud(6, [120, 60])
    m = np.array([15, 60], np.int32)
    idx = P.fps(xyz, np.cumsum(nv), np.cumsum(m))
    assert len(idx) == 75 and idx[0] == 0 and idx[15] == 120
    assert len(set(idx[:15])) == 15 and sorted(idx[15:]) == list(range(120, 180))      # all points once, when asked for all
    pts = xyz[:120].astype(np.float64)
    chosen = [0]
    for j in range(1, 15):
        dmin = np.min(np.linalg.norm(pts[:, None] - pts[chosen][None], axis=2), axis=1)
        # the pick attains the largest distance to the chosen set (up to float32 rounding of that distance)
        assert dmin[idx[j]] >= dmin.max() * (1 - 1e-5)
        chosen.append(int(idx[j]))
    # equal distances: the lowest index wins
    sq = np.array([[0, 0, 0], [1, 0, 0], [-1, 0, 0], [0, 1, 0]], np.float32)
    assert P.fps(sq, [4], [3]).tolist() == [0, 1, 2]


# ------------------------------------------------------------------ kernel bins
def test_sph3d_bins_of_hand_placed_directions():
    q = np.zeros((1, 3), np.float32)
    n, p, qq = 8, 2, 3
    radius = 1.0
    # direction by azimuth / elevation, distance: expected (azimuth sector of 45 deg from -180, hemisphere, shell)
    cases = [((-170, -30, 0.5), (0, 0, 1)), ((-100, 30, 0.9), (1, 1, 2)), ((10, -60, 0.35), (4, 0, 1)),
             ((100, 45, 0.65), (6, 1, 1)), ((170, 10, 0.99), (7, 1, 2)), ((0.1, 0.1, 0.2), None)]
    db = []
    for (az, el, d), _ in cases:
        az, el = np.radians(az), np.radians(el)
        db.append([d * np.cos(el) * np.cos(az), d * np.cos(el) * np.sin(az), d * np.sin(el)])
    db = np.array(db, np.float32)
    nn_index = np.stack([np.zeros(len(db), np.int32), np.arange(len(db), dtype=np.int32)], 1)
    nn_dist = np.linalg.norm(db, axis=1).astype(np.float32)
    idx, _ = P.sph3d_kernel(db, q, nn_index, nn_dist, radius, (n, p, qq))
    want = [0 if c is None else c[2] * p * n + c[1] * n + c[0] + 1 for _, c in cases]
    assert idx.tolist() == want
    # fuzzy form: weights sum to one, the centre weight is 1 - d / radius, the elevation bins are neighbours
    fi, fc, _ = P.fuzzy_sph3d_kernel(db, q, nn_index, nn_dist, radius, (8, 4, 1))
    assert np.allclose(fc.sum(1), 1, atol=1e-6) and np.allclose(fc[:, 0], 1 - nn_dist, atol=1e-6) and np.all(fi[:, 0] == 0)
    own, other = (fi[:, 1] - 1) // 8, (fi[:, 2] - 1) // 8
    two = fi[:, 2] > 0
    assert np.all(np.abs(own - other)[two] == 1) and np.all(((fi[:, 1] - 1) % 8)[two] == ((fi[:, 2] - 1) % 8)[two])
    assert np.all(fc[:, 1] >= fc[:, 2])                              # the pair's own bin carries at least half
    # a direction in the middle of its elevation bin puts everything into that bin; at a bin border both share equally
    for el, share in ((-67.5, 0.0), (-45.0, 0.5)):
        e = np.radians(el)
        d1 = np.array([[0.5 * np.cos(e), 0.0, 0.5 * np.sin(e)]], np.float32)
        i1, c1, _ = P.fuzzy_sph3d_kernel(d1, q, np.array([[0, 0]], np.int32), np.array([0.5], np.float32), 1.0, (8, 4, 1))
        assert np.isclose(c1[0, 2], share * 0.5, atol=1e-4) and np.isclose(c1[0, 0], 0.5, atol=1e-6)


# ------------------------------------------------------------------ convolution, pooling, unpooling
def graph(seed, n_db=60, n_q=25, T=None, F=7):
    rng = np.random.default_rng(seed)
    db, nvd = cloud(seed, [n_db])
    q, nvq = subsample(seed, db, nvd, n_q / n_db)
    _, count, nn_index, nn_dist = P.range_search(db, q, np.cumsum(nvd), np.cumsum(nvq), 0.45)
    if T is None:
        bins, coeff = rng.integers(0, F, len(nn_index)).astype(np.int32), None
    else:
        bins = rng.integers(0, F, (len(nn_index), T)).astype(np.int32)
        coeff = rng.uniform(0, 1, (len(nn_index), T)).astype(np.float32)
    return db, q, count, nn_index, nn_dist, bins, coeff


@pytest.mark.parametrize("T", [None, 3])
@pytest.mark.parametrize("r", [1, 2])
def test_conv_against_loops_and_autograd(T, r):
    db, q, count, nn_index, _, bins, coeff = graph(7, T=T)
    rng = np.random.default_rng(8)
    C, F = 5, 7
    x, filt = rng.normal(size=(len(db), C)), rng.normal(size=(F, C, r))
    out = P.conv_fwd(x, filt, count, nn_index, bins, coeff)
    want = np.zeros((len(q), C * r))
    for p, (o, i) in enumerate(nn_index.tolist()):
        for c in range(C):
            for m in range(r):
                if coeff is None:
                    w = filt[bins[p], c, m]
                else:
                    w = sum(coeff[p, t] * filt[bins[p, t], c, m] for t in range(coeff.shape[1]))
                want[o, c * r + m] += x[i, c] * w / count[o]
    assert np.allclose(out, want, atol=1e-12)
    # gradients: autograd through a torch statement of the same forward
    xt, ft = torch.tensor(x, requires_grad=True), torch.tensor(filt, requires_grad=True)
    o_t, i_t = torch.tensor(nn_index[:, 0]).long(), torch.tensor(nn_index[:, 1]).long()
    if coeff is None:
        w = ft[torch.tensor(bins).long()]
    else:
        w = (torch.tensor(coeff, dtype=torch.float64)[:, :, None, None] * ft[torch.tensor(bins).long()]).sum(1)
    term = xt[i_t][:, :, None] * w / torch.tensor(count, dtype=torch.float64)[o_t][:, None, None]
    y = torch.zeros(len(q), C, r, dtype=torch.float64).index_add(0, o_t, term).reshape(len(q), -1)
    g = rng.normal(size=y.shape)
    y.backward(torch.tensor(g))
    gin, gfilt = P.conv_bwd(g, x, filt, count, nn_index, bins, coeff)
    assert np.allclose(gin, xt.grad.numpy(), atol=1e-12) and np.allclose(gfilt, ft.grad.numpy(), atol=1e-12)
    assert np.allclose(y.detach().numpy(), out, atol=1e-12)


def test_pooling_and_unpooling_against_loops_and_adjoints():
    db, q, count, nn_index, nn_dist, _, _ = graph(9)
    rng = np.random.default_rng(10)
    C = 4
    x = rng.normal(size=(len(db), C))
    x[5] = x[9]                                                       # equal values: the first pair keeps the maximum
    mx, idx = P.pool_max_fwd(x, count, nn_index)
    av = P.pool_avg_fwd(x, count, nn_index)
    for j in range(len(q)):
        nb = nn_index[nn_index[:, 0] == j, 1]
        assert np.array_equal(mx[j], x[nb].max(0)) and np.allclose(av[j], x[nb].mean(0))
        for c in range(C):
            assert idx[j, c] == nb[np.argmax(x[nb, c])]               # argmax = first among equals
    g = rng.normal(size=mx.shape)
    gm = P.pool_max_bwd(g, len(db), idx)
    assert np.isclose((gm * x).sum(), (g * mx).sum())                 # d<g, max> / dx . x = <g, max> (piecewise linear)
    ga = P.pool_avg_bwd(g, len(db), count, nn_index)
    assert np.isclose((ga * x).sum(), (g * av).sum())                 # adjoint of a linear map
    # a query without pairs
    mx0, idx0 = P.pool_max_fwd(x, np.array([0, 2], np.int32), np.array([[1, 3], [1, 4]], np.int32))
    assert np.all(mx0[0] == 0) and np.all(idx0[0] == -1) and np.array_equal(mx0[1], np.maximum(x[3], x[4]))
    # unpooling: three nearest coarse points with inverse-distance weights
    fine, nvf = cloud(11, [50])
    nn3, d3 = P.knn3_search(q, fine, [len(q)], [50])
    w = 1 / (d3 + 1e-8)
    w = w / w.sum(1, keepdims=True)
    y = rng.normal(size=(len(q), C))
    up = P.unpool_fwd(y, w, nn3)
    for o in range(50):
        assert np.allclose(up[o], sum(y[nn3[o, k]] * w[o, k] for k in range(3)))
    gu = rng.normal(size=up.shape)
    gy = P.unpool_bwd(gu, len(q), w, nn3)
    assert np.isclose((gy * y).sum(), (gu * up).sum())
    assert np.allclose(P.unpool_fwd(np.ones((len(q), 1)), w, nn3), 1)  # weights sum to one
