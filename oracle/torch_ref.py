"""TEST INFRASTRUCTURE ONLY: vectorised PyTorch-CPU restatement of the reference ops.

Same arithmetic as the brute-force loops in ``mesh_loops.inc`` but expressed with
``index_select`` / ``index_add_`` / ``scatter_reduce_`` / ``einsum`` so it runs at
benchmark sizes on all host cores.  It is dtype generic (float32 for the timed
CPU baseline, float64 as the parity answer).  Forward functions are built from
differentiable torch ops, so ``torch.autograd`` can confirm the explicit
backward formulas below.  The product never imports this module.

Paths cited are relative to picasso/mesh/pi_modules/source/ of the reference.
"""
import math

import torch


def _long(t):
    return t.to(torch.int64)


# --------------------------------------------------------------------------
# spherical harmonics  (picasso/mesh/layers.py:341-356, picasso/math_utils.py:10-62)
# --------------------------------------------------------------------------
def sph_harm(xyz, L):
    """Real SH basis values (N, (L+1)^2) at directions ``xyz`` (N, 3), angle form."""
    if L > 5:
        raise NotImplementedError
    nrm = torch.sqrt((xyz ** 2).sum(-1, keepdim=True))
    u = xyz / (nrm + 1e-10)
    phi = torch.atan2(u[:, 1], u[:, 0])
    th = torch.atan2(u[:, 2], torch.linalg.norm(u[:, :2], dim=-1))
    phi = torch.where(phi < 0, phi + 2 * math.pi, phi)
    th = math.pi / 2 - th
    s, c, pi = torch.sin(th), torch.cos(th), math.pi
    cp = [None] + [torch.cos(m * phi) for m in range(1, 6)]
    sp = [None] + [torch.sin(m * phi) for m in range(1, 6)]
    q = math.sqrt
    rows = [torch.full_like(s, 0.5 * q(1 / pi))]
    if L >= 1:
        rows += [0.5 * q(3 / 2 / pi) * s * cp[1], 0.5 * q(3 / pi) * c, 0.5 * q(3 / 2 / pi) * s * sp[1]]
    if L >= 2:
        a, b = 0.25 * q(15 / 2 / pi) * s ** 2, 0.5 * q(15 / 2 / pi) * s * c
        rows += [a * cp[2], b * cp[1], 0.25 * q(5 / pi) * (3 * c ** 2 - 1), a * sp[2], b * sp[1]]
    if L >= 3:
        a = 0.125 * q(35 / pi) * s ** 3
        b = 0.25 * q(105 / 2 / pi) * s ** 2 * c
        d = 0.125 * q(21 / pi) * s * (5 * c ** 2 - 1)
        rows += [a * cp[3], b * cp[2], d * cp[1], 0.25 * q(7 / pi) * (5 * c ** 3 - 3 * c),
                 a * sp[3], b * sp[2], d * sp[1]]
    if L >= 4:
        a = 3 / 16 * q(35 / 2 / pi) * s ** 4
        b = 3 / 8 * q(35 / pi) * s ** 3 * c
        d = 3 / 8 * q(5 / 2 / pi) * s ** 2 * (7 * c ** 2 - 1)
        e = 3 / 8 * q(5 / pi) * s * (7 * c ** 3 - 3 * c)
        rows += [a * cp[4], b * cp[3], d * cp[2], e * cp[1],
                 3 / 16 * q(1 / pi) * (35 * c ** 4 - 30 * c ** 2 + 3),
                 a * sp[4], b * sp[3], d * sp[2], e * sp[1]]
    if L >= 5:
        a = 3 / 32 * q(77 / pi) * s ** 5
        b = 3 / 16 * q(385 / 2 / pi) * s ** 4 * c
        d = 1 / 32 * q(385 / pi) * s ** 3 * (9 * c ** 2 - 1)
        e = 1 / 8 * q(1155 / 2 / pi) * s ** 2 * (3 * c ** 3 - c)
        g = 1 / 16 * q(165 / 2 / pi) * s * (21 * c ** 4 - 14 * c ** 2 + 1)
        rows += [a * cp[5], b * cp[4], d * cp[3], e * cp[2], g * cp[1],
                 1 / 16 * q(11 / pi) * (63 * c ** 5 - 70 * c ** 3 + 15 * c),
                 a * sp[5], b * sp[4], d * sp[3], e * sp[2], g * sp[1]]
    return torch.stack(rows, dim=1)


# --------------------------------------------------------------------------
# vertex2facet  (mesh_conv3d_gpu.cu:176-260)
# --------------------------------------------------------------------------
def v2f_fwd(x, filt, face):
    Nf, (_, C, r) = face.shape[0], filt.shape
    corners = x[_long(face)]                                   # (Nf, 3, C)
    return torch.einsum("fkc,kcm->fcm", corners, filt).reshape(Nf, C * r)


def v2f_bwd(gout, x, filt, face):
    Nf, (_, C, r) = face.shape[0], filt.shape
    g = gout.reshape(Nf, C, r)
    per_corner = torch.einsum("fcm,kcm->fkc", g, filt)         # (Nf, 3, C)
    gin = torch.zeros_like(x).index_add_(0, _long(face).reshape(-1), per_corner.reshape(-1, C))
    gfilt = torch.einsum("fcm,fkc->kcm", g, x[_long(face)])
    return gin, gfilt


# --------------------------------------------------------------------------
# facet2vertex  (mesh_conv3d_gpu.cu:299-426)
# --------------------------------------------------------------------------
def _f2v_corner_scale(face, nfcount, vtmap, dtype):
    vo = vtmap[_long(face)]                                    # (Nf, 3)
    ok = vo >= 0
    safe = _long(vo.clamp(min=0))
    scale = torch.where(ok, 1.0 / nfcount[safe].to(dtype), torch.zeros((), dtype=dtype))
    return safe, scale


def f2v_fwd(x, filt, coeff, face, nfcount, vtmap):
    Nf, C = x.shape
    K, _, r = filt.shape
    w = (coeff @ filt.reshape(K, C * r)).reshape(Nf, C, r)
    val = (w * x[:, :, None]).reshape(Nf, C * r)
    safe, scale = _f2v_corner_scale(face, nfcount, vtmap, x.dtype)
    out = torch.zeros(nfcount.shape[0], C * r, dtype=x.dtype)
    for j in range(3):
        out = out.index_add(0, safe[:, j], val * scale[:, j:j + 1])
    return out


def f2v_bwd(gout, x, filt, coeff, face, nfcount, vtmap):
    Nf, C = x.shape
    K, _, r = filt.shape
    w = (coeff @ filt.reshape(K, C * r)).reshape(Nf, C, r)
    safe, scale = _f2v_corner_scale(face, nfcount, vtmap, x.dtype)
    s = torch.zeros(Nf, C * r, dtype=x.dtype)
    for j in range(3):
        s = s + gout[safe[:, j]] * scale[:, j:j + 1]
    s = s.reshape(Nf, C, r)
    gin = (s * w).sum(-1)
    gfilt = torch.einsum("fk,fcm->kcm", coeff, s * x[:, :, None])
    return gin, gfilt


# --------------------------------------------------------------------------
# facet2facet  (mesh_conv3d_gpu.cu:6-168), factored through
#   G[f,ci,d] = (1/K_f) sum_{k in f} tex[k,ci] * bary[k,d]
# --------------------------------------------------------------------------
def _segments(cum, T):
    counts = torch.diff(cum, prepend=cum.new_zeros(1))
    seg = torch.repeat_interleave(torch.arange(cum.shape[0]), _long(counts), output_size=T)
    return counts, seg


def f2f_moments(tex, bary, cum):
    T, Cin = tex.shape
    counts, seg = _segments(cum, T)
    G = torch.zeros(cum.shape[0], Cin, bary.shape[1], dtype=tex.dtype)
    G = G.index_add(0, seg, tex[:, :, None] * bary[:, None, :])
    inv = torch.where(counts > 0, 1.0 / counts.clamp(min=1).to(tex.dtype), torch.zeros((), dtype=tex.dtype))
    return G * inv[:, None, None], inv, seg


def f2f_fwd(tex, filt, bary, cum):
    G, _, _ = f2f_moments(tex, bary, cum)
    return torch.einsum("fcd,ocd->fo", G, filt)


def f2f_bwd(gout, tex, filt, bary, cum):
    G, inv, seg = f2f_moments(tex, bary, cum)
    H = torch.einsum("fo,ocd->fcd", gout, filt)                # (Nf, Cin, F)
    gin = torch.einsum("kcd,kd->kc", H[seg], bary) * inv[seg][:, None]
    gfilt = torch.einsum("fo,fcd->ocd", gout, G)
    return gin, gfilt


def f2f_bwd_filter_pointwise(gout, tex, bary, cum, block=200_000):
    """The filter gradient in the reference's own point-wise form (mesh_conv3d_gpu.cu:85-135: every texture
    point k of facet f adds gout[f,co] * tex[k,ci] * bary[k,d] / K_f), as one product per block of points:
    gfilt[co,(ci,d)] = sum_k (gout[f(k),co] / K_f(k)) * (tex[k,ci] * bary[k,d]).  No per-facet moments are
    formed, so memory stays at block * Cin * F values: the form for scene-sized batches."""
    T, Cin = tex.shape
    F = bary.shape[1]
    counts, seg = _segments(cum, T)
    inv = torch.where(counts > 0, 1.0 / counts.clamp(min=1).to(tex.dtype), torch.zeros((), dtype=tex.dtype))
    gfilt = torch.zeros(gout.shape[1], Cin * F, dtype=tex.dtype)
    for k0 in range(0, T, block):
        k1 = min(k0 + block, T)
        s = seg[k0:k1]
        a = gout[s] * inv[s][:, None]
        b = (tex[k0:k1, :, None] * bary[k0:k1, None, :]).reshape(k1 - k0, Cin * F)
        gfilt += a.t() @ b
    return gfilt.reshape(gout.shape[1], Cin, F)


# --------------------------------------------------------------------------
# texture points from vertex features: tex[k] = sum_j bary[k,j] * x[face[f(k),j]] for the rows k of
# facet f's segment (the grouping of layers.py:57); the reference loads texture features from its
# dataset files (dataset_scene.py:29-33) and has no such routine -- the encoder-block workload chains
# facet2facet after vertex features this way
# --------------------------------------------------------------------------
def texture_fwd(x, face, bary, cum):
    _, seg = _segments(cum, bary.shape[0])
    corner = _long(face)[seg]                                   # (T, 3)
    return (x[corner] * bary[:, :, None]).sum(1)


def texture_bwd(gtex, nv, face, bary, cum):
    _, seg = _segments(cum, bary.shape[0])
    corner = _long(face)[seg]
    gin = torch.zeros(nv, gtex.shape[1], dtype=gtex.dtype)
    for j in range(3):
        gin = gin.index_add(0, corner[:, j], gtex * bary[:, j:j + 1])
    return gin


# --------------------------------------------------------------------------
# pooling / unpooling over decimation clusters
# (mesh_pool3d_gpu.cu:20-155, mesh_unpool3d_gpu.cu:5-46)
# --------------------------------------------------------------------------
def cluster_maps(vt_replace, vt_map):
    """Per fine vertex: coarse row (or -1) and the divisor avg-pool uses."""
    ids = torch.arange(vt_replace.shape[0], dtype=vt_replace.dtype)
    rep = _long(torch.where(vt_replace < 0, -vt_replace, ids))
    vo = vt_map[rep]
    cnt = vt_replace[rep] + 1
    return vo, cnt


def maxpool_fwd(x, vt_replace, vt_map, nv_out):
    """Returns (out, max_index); ties resolve to the smallest vertex id; rows without
    members keep value 0 / index 0 (mesh_pool3d.cpp:53-54).  NaN inputs not modelled."""
    Nv, C = x.shape
    vo, _ = cluster_maps(vt_replace, vt_map)
    ok = vo >= 0
    v_ok = torch.nonzero(ok).squeeze(1)
    idx = _long(vo[ok])[:, None].expand(-1, C)
    out = torch.zeros(nv_out, C, dtype=x.dtype)
    out = out.scatter_reduce(0, idx, x[ok], "amax", include_self=False)
    big = torch.iinfo(torch.int32).max
    cand = torch.where(x[ok] == out[_long(vo[ok])], v_ok[:, None].expand(-1, C),
                       torch.full((), big, dtype=torch.int64))
    arg = torch.full((nv_out, C), big, dtype=torch.int64)
    arg = arg.scatter_reduce(0, idx, cand, "amin", include_self=True)
    arg = torch.where(arg == big, torch.zeros((), dtype=torch.int64), arg)
    return out, arg.to(torch.int32)


def maxpool_bwd(gout, nv_in, max_index):
    C = gout.shape[1]
    gin = torch.zeros(nv_in, C, dtype=gout.dtype)
    # plain store semantics (mesh_pool3d_gpu.cu:100); distinct targets for valid cluster maps
    gin.scatter_(0, _long(max_index), gout)
    return gin


def avgpool_fwd(x, vt_replace, vt_map, nv_out):
    vo, cnt = cluster_maps(vt_replace, vt_map)
    ok = vo >= 0
    out = torch.zeros(nv_out, x.shape[1], dtype=x.dtype)
    return out.index_add(0, _long(vo[ok]), x[ok] / cnt[ok].to(x.dtype)[:, None])


def avgpool_bwd(gout, vt_replace, vt_map):
    vo, cnt = cluster_maps(vt_replace, vt_map)
    ok = vo >= 0
    g = gout[_long(vo.clamp(min=0))] / cnt.clamp(min=1).to(gout.dtype)[:, None]
    return torch.where(ok[:, None], g, torch.zeros((), dtype=gout.dtype))


def unpool_fwd(x, vt_replace, vt_map):
    vo, _ = cluster_maps(vt_replace, vt_map)
    ok = vo >= 0
    return torch.where(ok[:, None], x[_long(vo.clamp(min=0))], torch.zeros((), dtype=x.dtype))


def unpool_bwd(gout, nv_coarse, vt_replace, vt_map):
    vo, _ = cluster_maps(vt_replace, vt_map)
    ok = vo >= 0
    gin = torch.zeros(nv_coarse, gout.shape[1], dtype=gout.dtype)
    return gin.index_add(0, _long(vo[ok]), gout[ok])


# --------------------------------------------------------------------------
# helpers the callers of the path provide
# --------------------------------------------------------------------------
def count_vertex_adjface(face, vtmap, nv_out):
    """nf_count: number of (facet, corner) pairs landing on each output vertex
    (decimate_gpu.cu:813-831)."""
    vo = vtmap[_long(face)].reshape(-1)
    return torch.bincount(_long(vo[vo >= 0]), minlength=nv_out).to(torch.int32)


def face_normals(vertex, face):
    """Unit facet normals (picasso/mesh/pi_modules/decimate.py:70-85)."""
    p = vertex[_long(face)]
    n = torch.linalg.cross(p[:, 1] - p[:, 0], p[:, 2] - p[:, 0])
    return n / torch.linalg.norm(n, dim=-1, keepdim=True).clamp_min(1e-30)


def oriented_normals(normals, vertex, face):
    """Normals turned towards the origin as the viewpoint (picasso/networks/scene_seg.py:117-124): the sign of
    -centre . normal, with 0 counted as +1."""
    centre = vertex[_long(face)][:, :, :3].mean(1)
    sign = torch.sign((-centre * normals).sum(-1, keepdim=True))
    sign = torch.where(sign > -1, torch.ones_like(sign), sign)
    return normals * sign


# --------------------------------------------------------------------------
# pointwise tail of the conv modules  (picasso/mesh/layers.py:114-119, 169-174, 232-238)
# --------------------------------------------------------------------------
def dense_tail_fwd(x, w, b=None, relu=True, scale=None, shift=None):
    """act(x @ w + b) * scale + shift: matmul, bias, activation, then a batch norm that only applies
    its running statistics (scale = gamma / sqrt(var + eps), shift = beta - mean * scale)."""
    z = x @ w
    if b is not None:
        z = z + b
    if relu:
        z = torch.clamp_min(z, 0)
    if scale is not None:
        z = z * scale
    if shift is not None:
        z = z + shift
    return z


def dense_tail_bwd(gout, x, w, out=None):
    """Gradients of act(x @ w + b) for (x, w, b); ``out`` is the forward result when act is ReLU
    (entries with out > 0 pass the gradient), None for no activation."""
    gz = gout if out is None else torch.where(out > 0, gout, torch.zeros_like(gout))
    return gz @ w.t(), x.t() @ gz, gz.sum(0)


def bias_act_fwd(x, b=None, relu=True, scale=None, shift=None):
    """act(x + b) * scale + shift: the tail of F2FConv3d (picasso/mesh/layers.py:60-64)."""
    z = x if b is None else x + b
    if relu:
        z = torch.clamp_min(z, 0)
    if scale is not None:
        z = z * scale
    if shift is not None:
        z = z + shift
    return z


def bias_act_bwd(gout, out=None):
    """Gradients of act(x + b) for (x, b); ``out`` is the forward result when act is ReLU, else None."""
    gz = gout if out is None else torch.where(out > 0, gout, torch.zeros_like(gout))
    return gz, gz.sum(0)


def combine_clusters(rep_a, map_a, rep_b, map_b):
    """Cluster maps of two decimation steps -> maps of both together (decimate_gpu.cu:750-810): update_repB
    (:750-760) records, for every step-A survivor that also survives step B, its fine index; update_repA
    (:761-781) moves every fine vertex whose middle-level representative step B contracts to the fine index
    behind B's representative, which counts it; update_mapA (:782-794) chains the maps.  int32 tensors."""
    nv_a = rep_a.shape[0]
    ra, ma, rb, mb = (_long(t) for t in (rep_a, map_a, rep_b, map_b))
    idx = torch.arange(nv_a)
    owner = rb.clone()
    keep = ma >= 0
    keep_b = keep.clone()
    keep_b[keep] = rb[ma[keep]] >= 0
    owner[ma[keep_b]] = idx[keep_b]
    rep = ra.clone()
    vi = torch.where(ra < 0, -ra, idx)
    vo = ma[vi]
    hit = vo >= 0
    hit[hit.clone()] = owner[vo[hit]] < 0
    target = owner[-owner[vo[hit]]]
    rep[idx[hit]] = -target
    rep.index_add_(0, target, torch.ones_like(target))
    mapped = torch.full_like(ma, -1)
    mapped[keep] = mb[ma[keep]]
    return rep.to(torch.int32), mapped.to(torch.int32)
