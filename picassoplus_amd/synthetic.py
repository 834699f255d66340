"""Seeded synthetic meshes, texture points and decimation-cluster maps.

The benchmark and the parity tests need inputs with the same structure as the
data the mesh ops consume in a real network: concatenated batches of triangle
meshes (vertex rows stacked, facet indices offset per sample, the convention of
picasso/mesh/dataset_shape.py:43-58 in the reference), per-facet texture-point
sets with barycentric coordinates, and the ``vt_replace`` / ``vt_map`` pair that
GPU decimation emits (picasso/mesh/pi_modules/decimate.py:23-28).  Everything
here is numpy on ``numpy.random.default_rng(seed)`` and therefore reproducible
on any host.
"""
import numpy as np

I32 = np.int32


# ------------------------------------------------------------------ primitives
def icosahedron():
    t = (1.0 + 5 ** 0.5) / 2.0
    v = np.array([[-1, t, 0], [1, t, 0], [-1, -t, 0], [1, -t, 0],
                  [0, -1, t], [0, 1, t], [0, -1, -t], [0, 1, -t],
                  [t, 0, -1], [t, 0, 1], [-t, 0, -1], [-t, 0, 1]], dtype=np.float64)
    f = np.array([[0, 11, 5], [0, 5, 1], [0, 1, 7], [0, 7, 10], [0, 10, 11],
                  [1, 5, 9], [5, 11, 4], [11, 10, 2], [10, 7, 6], [7, 1, 8],
                  [3, 9, 4], [3, 4, 2], [3, 2, 6], [3, 6, 8], [3, 8, 9],
                  [4, 9, 5], [2, 4, 11], [6, 2, 10], [8, 6, 7], [9, 8, 1]], dtype=np.int64)
    return v / np.linalg.norm(v, axis=1, keepdims=True), f


def subdivide(v, f):
    """Loop-style 1:4 split; shared edge midpoints are created once."""
    nv = v.shape[0]
    e = np.sort(np.concatenate([f[:, [0, 1]], f[:, [1, 2]], f[:, [2, 0]]]), axis=1)
    key = e[:, 0] * nv + e[:, 1]
    uniq, inv = np.unique(key, return_inverse=True)
    mid = 0.5 * (v[uniq // nv] + v[uniq % nv])
    nf = f.shape[0]
    m01, m12, m20 = nv + inv[:nf], nv + inv[nf:2 * nf], nv + inv[2 * nf:]
    f_new = np.concatenate([np.stack([f[:, 0], m01, m20], 1), np.stack([f[:, 1], m12, m01], 1),
                            np.stack([f[:, 2], m20, m12], 1), np.stack([m01, m12, m20], 1)])
    return np.concatenate([v, mid]), f_new


def icosphere(level):
    """Unit icosphere: level 5 has 10 242 vertices and 20 480 facets."""
    v, f = icosahedron()
    for _ in range(level):
        v, f = subdivide(v, f)
        v /= np.linalg.norm(v, axis=1, keepdims=True)
    return v, f.astype(I32)


def torus(nu, nv, R=1.0, r=0.35):
    """Closed torus: nu*nv vertices, 2*nu*nv facets, every vertex has valence 6."""
    a = np.arange(nu) * (2 * np.pi / nu)
    b = np.arange(nv) * (2 * np.pi / nv)
    A, B = np.meshgrid(a, b, indexing="ij")
    v = np.stack([(R + r * np.cos(B)) * np.cos(A), (R + r * np.cos(B)) * np.sin(A), r * np.sin(B)], -1)
    i, j = np.meshgrid(np.arange(nu), np.arange(nv), indexing="ij")
    p00 = i * nv + j
    p10 = ((i + 1) % nu) * nv + j
    p01 = i * nv + (j + 1) % nv
    p11 = ((i + 1) % nu) * nv + (j + 1) % nv
    f = np.concatenate([np.stack([p00, p10, p11], -1).reshape(-1, 3),
                        np.stack([p00, p11, p01], -1).reshape(-1, 3)])
    return v.reshape(-1, 3), f.astype(I32)


def grid_patch(rng, nx, ny, origin, ax_u, ax_v, spacing=None, flip_frac=0.5, fan_frac=0.0,
               collapse_frac=0.0):
    """Planar nx-by-ny quad grid, quads split into triangles.

    ``spacing``: None for unit steps, else (mean, sigma) of log-normal edge lengths.
    ``flip_frac``: share of quads whose diagonal is flipped (spreads valence over 4..8).
    ``fan_frac``: share of quads replaced by a 4-triangle fan around a new centre vertex
    (adds valence-4 vertices).
    ``collapse_frac``: share of grid vertices merged into their +u neighbour, as an edge
    collapse would (removes the two facets on that edge, leaves vertices of valence ~9-13).
    """
    if spacing is None:
        xs, ys = np.arange(nx + 1, dtype=np.float64), np.arange(ny + 1, dtype=np.float64)
    else:
        mu, sig = spacing
        xs = np.concatenate([[0.0], np.cumsum(np.exp(rng.normal(np.log(mu), sig, nx)))])
        ys = np.concatenate([[0.0], np.cumsum(np.exp(rng.normal(np.log(mu), sig, ny)))])
    X, Y = np.meshgrid(xs, ys, indexing="ij")
    origin, ax_u, ax_v = (np.asarray(t, dtype=np.float64) for t in (origin, ax_u, ax_v))
    v = origin + X[..., None] * ax_u + Y[..., None] * ax_v
    v = v.reshape(-1, 3)
    i, j = np.meshgrid(np.arange(nx), np.arange(ny), indexing="ij")
    i, j = i.reshape(-1), j.reshape(-1)
    p00, p10 = i * (ny + 1) + j, (i + 1) * (ny + 1) + j
    p01, p11 = p00 + 1, p10 + 1
    u = rng.random(i.shape[0])
    fan = u < fan_frac
    flip = (~fan) & (u < fan_frac + flip_frac * (1 - fan_frac))
    plain = ~(fan | flip)
    faces = [np.stack([p00[plain], p10[plain], p11[plain]], 1), np.stack([p00[plain], p11[plain], p01[plain]], 1),
             np.stack([p00[flip], p10[flip], p01[flip]], 1), np.stack([p10[flip], p11[flip], p01[flip]], 1)]
    if fan.any():
        ctr = 0.25 * (v[p00[fan]] + v[p10[fan]] + v[p01[fan]] + v[p11[fan]])
        c = v.shape[0] + np.arange(ctr.shape[0])
        v = np.concatenate([v, ctr])
        a, b, d, e = p00[fan], p10[fan], p11[fan], p01[fan]
        faces += [np.stack([a, b, c], 1), np.stack([b, d, c], 1), np.stack([d, e, c], 1), np.stack([e, a, c], 1)]
    f = np.concatenate(faces)
    if collapse_frac > 0 and nx >= 4:
        gi, gj = np.meshgrid(np.arange(1, nx - 1, 3), np.arange(ny + 1), indexing="ij")
        sel = rng.random(gi.shape) < min(1.0, 3 * collapse_frac)
        keep_v, gone_v = (gi[sel] * (ny + 1) + gj[sel]), ((gi[sel] + 1) * (ny + 1) + gj[sel])
        remap = np.arange(v.shape[0])
        remap[gone_v] = keep_v
        f = remap[f]
        f = f[(f[:, 0] != f[:, 1]) & (f[:, 1] != f[:, 2]) & (f[:, 0] != f[:, 2])]
        used = np.zeros(v.shape[0], bool)
        used[f.reshape(-1)] = True
        v, f = v[used], (np.cumsum(used) - 1)[f]
    # keep facets in scan order of their first corner so neighbouring facets stay close in memory
    f = f[np.argsort(f.min(axis=1), kind="stable")]
    return v, f.astype(I32)


def merge(parts):
    """Concatenate (vertex, facet) pairs with index offsets; returns counts per part too."""
    vs, fs, off = [], [], 0
    for v, f in parts:
        vs.append(v)
        fs.append(f.astype(np.int64) + off)
        off += v.shape[0]
    nv = np.array([v.shape[0] for v, _ in parts], I32)
    mf = np.array([f.shape[0] for _, f in parts], I32)
    return np.concatenate(vs), np.concatenate(fs).astype(I32), nv, mf


def room(rng, scale=1.0):
    """Room-like scene of axis-aligned planar grids: floor, four walls and boxes.

    About 300 k facets at scale 1; edge lengths are log-normal around 2 cm.
    """
    s = scale ** 0.5
    nx, ny, nz = int(210 * s), int(168 * s), int(107 * s)
    sp = (0.02, 0.5)
    kw = dict(spacing=sp, flip_frac=0.5, fan_frac=0.08, collapse_frac=0.04)
    parts = [grid_patch(rng, nx, ny, (0, 0, 0), (1, 0, 0), (0, 1, 0), **kw),
             grid_patch(rng, nx, nz, (0, 0, 0), (1, 0, 0), (0, 0, 1), **kw),
             grid_patch(rng, nx, nz, (0, ny * 0.02, 0), (1, 0, 0), (0, 0, 1), **kw),
             grid_patch(rng, ny, nz, (0, 0, 0), (0, 1, 0), (0, 0, 1), **kw),
             grid_patch(rng, ny, nz, (nx * 0.02, 0, 0), (0, 1, 0), (0, 0, 1), **kw)]
    for _ in range(6):
        bx, by, bz = (max(4, int(rng.integers(20, 40) * s)) for _ in range(3))
        o = np.array([rng.uniform(0.2, 2.5), rng.uniform(0.2, 2.0), 0.0])
        ex, ey, ez = bx * 0.02, by * 0.02, bz * 0.02
        parts += [grid_patch(rng, bx, by, o + (0, 0, ez), (1, 0, 0), (0, 1, 0), **kw),
                  grid_patch(rng, bx, bz, o, (1, 0, 0), (0, 0, 1), **kw),
                  grid_patch(rng, bx, bz, o + (0, ey, 0), (1, 0, 0), (0, 0, 1), **kw),
                  grid_patch(rng, by, bz, o, (0, 1, 0), (0, 0, 1), **kw),
                  grid_patch(rng, by, bz, o + (ex, 0, 0), (0, 1, 0), (0, 0, 1), **kw)]
    v, f, _, _ = merge(parts)
    return v, f


# ------------------------------------------------------------------ derived data
def triangle_normals_areas(v, f):
    p = v[f.astype(np.int64)]
    n = np.cross(p[:, 1] - p[:, 0], p[:, 2] - p[:, 0])
    l2 = np.linalg.norm(n, axis=1, keepdims=True)
    return n / (l2 + 1e-10), 0.5 * l2[:, 0]


def vertex_facet_count(f, vt_map, nv_out):
    """nf_count of the facet-to-vertex conv: (facet, corner) pairs per output vertex."""
    vo = vt_map[f.astype(np.int64)].reshape(-1)
    return np.bincount(vo[vo >= 0], minlength=nv_out).astype(I32)


def texture_points(rng, n_facets, counts):
    """``counts`` texture points per facet, barycentric coords ~ Dirichlet(1,1,1).

    Returns (num_texture (Nf,) int32, bary (T,3) float64, facet_of_point (T,) int64).
    """
    counts = np.broadcast_to(np.asarray(counts, I32), (n_facets,)).astype(I32)
    T = int(counts.sum())
    bary = rng.dirichlet((1.0, 1.0, 1.0), size=T)
    owner = np.repeat(np.arange(n_facets, dtype=np.int64), counts)
    return counts, bary, owner


def area_scaled_texture_counts(area, lo=1, hi=9):
    p95 = np.percentile(area, 95)
    return np.clip(np.rint(hi * area / p95), lo, hi).astype(I32)


def cluster_maps(rng, nv, mean=4.0, lo=1, hi=12, spatial=True, orphan_frac=0.0):
    """Decimation-style cluster maps over ``nv`` fine vertices.

    Cluster sizes are clip(Poisson(mean), lo, hi).  ``vt_replace[v]`` is ``-rep`` for a
    contracted vertex, 0 for a singleton and (size-1) for a representative;
    ``vt_map[v]`` is the coarse row of kept vertices (ascending with v) and -1
    elsewhere.  Vertex 0 is never the representative of a multi-member cluster, because
    ``-0`` could not mark its members.  ``spatial`` keeps members contiguous in vertex
    order (what edge collapses produce on a scan-ordered mesh); otherwise members are a
    random permutation.  ``orphan_frac`` marks that share of clusters as dropped
    (``vt_map = -1`` on the representative too).  Returns (vt_replace, vt_map, nv_out).
    """
    sizes = []
    total = 0
    while total < nv:
        s = np.clip(rng.poisson(mean, size=max(16, int(nv / mean) + 16)), lo, hi)
        sizes.append(s)
        total += int(s.sum())
    sizes = np.concatenate(sizes)
    cs = np.cumsum(sizes)
    n_cl = int(np.searchsorted(cs, nv, side="left")) + 1
    sizes = sizes[:n_cl].copy()
    sizes[-1] -= int(cs[n_cl - 1] - nv)
    order = np.arange(nv, dtype=np.int64) if spatial else rng.permutation(nv).astype(np.int64)
    start = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    pick = start + (rng.random(n_cl) * sizes).astype(np.int64)
    rep = order[pick]
    # vertex 0 must not represent other vertices: hand the role to another member
    bad = np.nonzero((rep == 0) & (sizes > 1))[0]
    for c in bad:
        members = order[start[c]:start[c] + sizes[c]]
        rep[c] = members[members != 0][0]
    cl_of = np.repeat(np.arange(n_cl), sizes)
    vt_replace = np.empty(nv, I32)
    vt_replace[order] = -rep[cl_of]
    vt_replace[rep] = sizes - 1
    kept = np.zeros(nv, bool)
    kept[rep] = True
    if orphan_frac > 0:
        kept[rep[rng.random(n_cl) < orphan_frac]] = False
    vt_map = np.where(kept, np.cumsum(kept) - 1, -1).astype(I32)
    return vt_replace, vt_map, int(kept.sum())


def random_rotation(rng):
    q, r = np.linalg.qr(rng.normal(size=(3, 3)))
    q *= np.sign(np.diag(r))
    if np.linalg.det(q) < 0:
        q[:, 0] = -q[:, 0]
    return q


# ------------------------------------------------------------------ workloads
def sphere_workload(seed=1000, level=5):
    """Single closed mesh: jittered, renormalised icosphere."""
    rng = np.random.default_rng(seed)
    v, f = icosphere(level)
    v = v + rng.normal(0, 0.002, v.shape)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    return dict(vertex=v, face=f, nv_in=np.array([v.shape[0]], I32), mf_in=np.array([f.shape[0]], I32))


def shapes_workload(seed=2000, n_meshes=16):
    """Batch of randomly posed icospheres / tori with 8k-32k facets each, radial noise 1 %."""
    parts = []
    for i in range(n_meshes):
        rng = np.random.default_rng(seed + i)
        if rng.random() < 0.5:
            v, f = icosphere(5)
        else:
            nu = int(rng.integers(80, 161))
            nf = int(rng.integers(8000, 32001))
            v, f = torus(nu, max(8, nf // (2 * nu)))
        v = v * (1.0 + rng.normal(0, 0.01, (v.shape[0], 1)))
        v = (v * rng.uniform(0.5, 2.0)) @ random_rotation(rng).T
        parts.append((v, f))
    v, f, nv_in, mf_in = merge(parts)
    return dict(vertex=v, face=f, nv_in=nv_in, mf_in=mf_in)


def scene_workload(seed=3000, n_rooms=8, scale=1.0):
    """Batch of room-like scenes, about 300 k facets each at scale 1."""
    parts = [room(np.random.default_rng(seed + i), scale) for i in range(n_rooms)]
    v, f, nv_in, mf_in = merge(parts)
    return dict(vertex=v, face=f, nv_in=nv_in, mf_in=mf_in)


def plane_workload(seed=4000, n=1024):
    """n-by-n vertex jittered planar grid: n*n vertices, 2*(n-1)^2 facets."""
    rng = np.random.default_rng(seed)
    v, f = grid_patch(rng, n - 1, n - 1, (0, 0, 0), (1, 0, 0), (0, 1, 0), flip_frac=0.0)
    v = v + rng.normal(0, 0.1, v.shape) * np.array([1.0, 1.0, 0.2])
    return dict(vertex=v, face=f, nv_in=np.array([v.shape[0]], I32), mf_in=np.array([f.shape[0]], I32))


def grid_cluster_maps(cells):
    """4:1 cluster maps from the (cells+1)^2 vertices of a ``cells``-by-``cells`` grid patch (vertex id
    ``i * (cells+1) + j``) to the (cells/2+1)^2 vertices of the grid of half the resolution: coarse vertex (I, J)
    collects the fine vertices {2I, 2I+1} x {2J, 2J+1} inside the patch; its representative is the last of them,
    so vertex 0 never represents others, and representatives ascend with the coarse id.
    Returns (vt_replace, vt_map, nv_out) with the meaning ``cluster_maps`` documents."""
    assert cells >= 2 and cells % 2 == 0
    nf, nc = cells + 1, cells // 2 + 1
    i, j = np.meshgrid(np.arange(nf), np.arange(nf), indexing="ij")
    I, J = i // 2, j // 2
    rep = np.minimum(2 * I + 1, cells) * nf + np.minimum(2 * J + 1, cells)        # fine id of my representative
    rep, fine = rep.reshape(-1), (i * nf + j).reshape(-1)
    size = np.bincount(rep, minlength=nf * nf)
    is_rep = rep == fine
    vt_replace = np.where(is_rep, size[fine] - 1, -rep).astype(I32)
    vt_map = np.where(is_rep, (I * nc + J).reshape(-1), -1).astype(I32)
    return vt_replace, vt_map, nc * nc


def hierarchy_workload(seed=5000, cells=1024, levels=4):
    """One planar scene-like mesh of 2*cells^2 facets with ``levels`` coarser versions of itself, each a jittered
    grid of half the resolution (a quarter of the vertices), and the 4:1 cluster maps between consecutive levels.
    Returns a list of ``levels + 1`` dicts: vertex, face, and (all but the last) vt_replace, vt_map, nv_out."""
    rng = np.random.default_rng(seed)
    out = []
    for l in range(levels + 1):
        n = cells >> l
        h = float(1 << l)
        v, f = grid_patch(rng, n, n, (0, 0, 0), (h, 0, 0), (0, h, 0), flip_frac=0.5)
        v = v + rng.normal(0, 0.1 * h, v.shape) * np.array([1.0, 1.0, 0.2])
        lev = dict(vertex=v, face=f)
        if l < levels:
            lev["vt_replace"], lev["vt_map"], lev["nv_out"] = grid_cluster_maps(n)
        out.append(lev)
    return out


def xavier_uniform(rng, shape, fan_in, fan_out):
    a = (6.0 / (fan_in + fan_out)) ** 0.5
    return rng.uniform(-a, a, shape)
