"""TEST INFRASTRUCTURE ONLY: numpy restatement of the reference's point-cloud branch (picasso/point/pi_modules/source/*.cu):
neighbour queries, kernel-bin builders, farthest point sampling, the (fuzzy) depthwise point convolution, point
pooling and weighted unpooling.  The product never imports this module.

Searches and sampling compare float32 distances, so they are restated in float32 with every operation rounded on its
own (numpy's elementwise arithmetic; the device code switches contraction into fused multiply-adds off for the same
expressions), which makes their integer outputs exact.  The convolution, pooling and unpooling are dtype generic
(float64 as the parity answer).

Paths cited are relative to picasso/point/pi_modules/source/ of the reference.
"""
import numpy as np

F32 = np.float32


def _ranges(cum):
    cum = np.asarray(cum, np.int64)
    return np.concatenate([[0], cum[:-1]]), cum


def _sq_dist(q, d):
    """(M, N) float32 squared distances, each operation rounded: (dx*dx + dy*dy) + dz*dz."""
    dx = d[None, :, 0] - q[:, None, 0]
    dy = d[None, :, 1] - q[:, None, 1]
    dz = d[None, :, 2] - q[:, None, 2]
    return (dx * dx + dy * dy) + dz * dz, (dx, dy, dz)


def _first_hits(hit, limit):
    """keep the first ``limit`` True entries of every row (nnquery_gpu.cu:58, :118: ``cnt < nnSample``)."""
    rank = np.cumsum(hit, 1)
    return hit & (rank <= limit)


def range_search(database, query, nv_database, nv_query, radius, nn_sample=2147483647):
    """nnquery_gpu.cu:20-126 (count_sphereNN, build_sphereNN_idx): per query the database points of its sample with
    sqrt(d2) < radius, in ascending database order, at most nn_sample of them.
    returns (cnt_info int64 inclusive running total, nn_count int32, nn_index (Nout, 2) int32 [query, database], nn_dist)."""
    database, query = np.asarray(database, F32)[:, :3], np.asarray(query, F32)[:, :3]
    (d0, d1), (q0, q1) = _ranges(nv_database), _ranges(nv_query)
    counts = np.zeros(len(query), np.int64)
    pairs, dists = [], []
    for b in range(len(d1)):
        q, d = query[q0[b]:q1[b]], database[d0[b]:d1[b]]
        if len(q) == 0:
            continue
        dist = np.sqrt(_sq_dist(q, d)[0])
        hit = _first_hits(dist < F32(radius), nn_sample)
        qi, di = np.nonzero(hit)                                   # row-major: by query, then ascending database index
        counts[q0[b]:q1[b]] = hit.sum(1)
        pairs.append(np.stack([qi + q0[b], di + d0[b]], 1))
        dists.append(dist[qi, di])
    nn_index = np.concatenate(pairs).astype(np.int32) if pairs else np.zeros((0, 2), np.int32)
    nn_dist = np.concatenate(dists).astype(F32) if dists else np.zeros(0, F32)
    return np.cumsum(counts), counts.astype(np.int32), nn_index, nn_dist


def cube_search(database, query, nv_database, nv_query, length, nn_sample=2147483647, grid_size=4):
    """nnquery_gpu.cu:134-250: neighbours inside the axis-aligned cube of edge ``length`` and their cell of a
    grid_size^3 grid.  returns (cnt_info, nn_count, nn_index (Nout, 3) int32 [query, database, bin])."""
    database, query = np.asarray(database, F32)[:, :3], np.asarray(query, F32)[:, :3]
    (d0, d1), (q0, q1) = _ranges(nv_database), _ranges(nv_query)
    half, cell = F32(length) / F32(2), F32(length) / F32(grid_size)
    counts = np.zeros(len(query), np.int64)
    rows = []
    for b in range(len(d1)):
        q, d = query[q0[b]:q1[b]], database[d0[b]:d1[b]]
        if len(q) == 0:
            continue
        _, (dx, dy, dz) = _sq_dist(q, d)
        hit = _first_hits((np.abs(dx) < half) & (np.abs(dy) < half) & (np.abs(dz) < half), nn_sample)
        qi, di = np.nonzero(hit)
        ids = [((c[qi, di] + half) / cell).astype(np.int32) for c in (dx, dy, dz)]      # C truncation of a value >= 0
        counts[q0[b]:q1[b]] = hit.sum(1)
        rows.append(np.stack([qi + q0[b], di + d0[b], (ids[0] * grid_size + ids[1]) * grid_size + ids[2]], 1))
    nn_index = np.concatenate(rows).astype(np.int32) if rows else np.zeros((0, 3), np.int32)
    return np.cumsum(counts), counts.astype(np.int32), nn_index


def knn3_search(database, query, nv_database, nv_query):
    """nnquery_gpu.cu:262-330: the three nearest database points of the query's sample, ties to the lower index
    (strict ``<``).  With fewer than three points the missing slots keep index 0 of the sample and an infinite
    distance (1e40 is not a float).  returns (nn_index (Mp, 3), nn_dist (Mp, 3) sqrt distances)."""
    database, query = np.asarray(database, F32)[:, :3], np.asarray(query, F32)[:, :3]
    (d0, d1), (q0, q1) = _ranges(nv_database), _ranges(nv_query)
    idx = np.zeros((len(query), 3), np.int32)
    dst = np.full((len(query), 3), np.inf, F32)
    for b in range(len(d1)):
        q, d = query[q0[b]:q1[b]], database[d0[b]:d1[b]]
        idx[q0[b]:q1[b]] = d0[b]
        if len(q) == 0 or len(d) == 0:
            continue
        d2 = _sq_dist(q, d)[0]
        order = np.argsort(d2, axis=1, kind="stable")[:, :3]
        k = order.shape[1]
        idx[q0[b]:q1[b], :k] = order + d0[b]
        dst[q0[b]:q1[b], :k] = np.sqrt(np.take_along_axis(d2, order, 1))
    return idx, dst


def fps(xyz, nv_in, nv_out):
    """sample_gpu.cu:11-100: farthest point sampling per sample, starting from its first point; every further point
    maximises the distance to the chosen set.  DETERMINISTIC choice among equal distances: the lowest index (the
    reference's depends on its thread layout)."""
    xyz = np.asarray(xyz, F32)[:, :3]
    (n0, n1), (m0, m1) = _ranges(nv_in), _ranges(nv_out)
    out = np.zeros(int(m1[-1]) if len(m1) else 0, np.int32)
    for b in range(len(n1)):
        p = xyz[n0[b]:n1[b]]
        m = int(m1[b] - m0[b])
        if m == 0:
            continue
        best = np.full(len(p), 1e38, F32)
        cur = 0
        out[m0[b]] = n0[b]
        for j in range(1, m):
            dx, dy, dz = p[:, 0] - p[cur, 0], p[:, 1] - p[cur, 1], p[:, 2] - p[cur, 2]
            best = np.minimum((dx * dx + dy * dy) + dz * dz, best)
            cur = int(np.argmax(best))                              # first maximum
            out[m0[b] + j] = n0[b] + cur
    return out


def _angles(database, query, nn_index, nn_dist, n, p, q, radius):
    database, query = np.asarray(database, F32)[:, :3], np.asarray(query, F32)[:, :3]
    delta = database[nn_index[:, 1]] - query[nn_index[:, 0]]
    dist = np.asarray(nn_dist, F32)
    dist2d = np.sqrt(delta[:, 0] * delta[:, 0] + delta[:, 1] * delta[:, 1])
    pi = F32(np.pi)
    theta = np.arctan2(delta[:, 1], delta[:, 0])
    phi = np.arctan2(delta[:, 2], dist2d)
    theta = np.where(theta < pi, theta, -pi)
    theta = np.where(theta > -pi, theta, -pi) + pi
    phi = np.where(phi < pi / 2, phi, pi / 2)
    phi = np.where(phi > -pi / 2, phi, -pi / 2) + pi / 2
    alpha = theta * F32(n) / F32(2) / pi
    beta = phi * F32(p) / pi
    gamma = dist * F32(q) / F32(radius)
    return dist, alpha.astype(F32), beta.astype(F32), gamma.astype(F32)


def sph3d_kernel(database, query, nn_index, nn_dist, radius, kernel=(8, 2, 3)):
    """buildkernel_gpu.cu:20-76: bin of every neighbour pair in an (n azimuth, p elevation, q radial) spherical
    kernel; bin 0 is the centre (distance <= 0.3 radius).  returns (filt_index int32, (alpha, beta, gamma) the
    continuous bin coordinates, for tests to stay clear of bin borders)."""
    n, p, q = kernel
    dist, alpha, beta, gamma = _angles(database, query, nn_index, nn_dist, n, p, q, radius)
    nid = np.minimum(n - 1, alpha.astype(np.int32))
    pid = np.minimum(p - 1, beta.astype(np.int32))
    qid = np.minimum(q - 1, gamma.astype(np.int32))
    # the comparison runs in double: 0.3 is a double literal there
    outer = dist.astype(np.float64) > 0.3 * np.float64(F32(radius))
    return np.where(outer, qid * p * n + pid * n + nid + 1, 0).astype(np.int32), (alpha, beta, gamma)


def fuzzy_sph3d_kernel(database, query, nn_index, nn_dist, radius, kernel=(8, 4, 1)):
    """buildkernel_gpu.cu:84-155: three (bin, weight) slots per pair: the centre with weight max(0, 1 - dist/radius),
    and the pair's elevation bin shared with the neighbouring elevation bin on the side it leans to.
    returns (filt_index (Nout, 3), filt_coeff (Nout, 3), (alpha, beta, gamma))."""
    n, p, q = kernel
    dist, alpha, beta, gamma = _angles(database, query, nn_index, nn_dist, n, p, q, radius)
    self_c = np.maximum(0.0, 1 - (dist / F32(radius)).astype(np.float64)).astype(F32)     # max(0.0, float): in double
    nid = np.minimum(n - 1, alpha.astype(np.int32))
    p0 = np.minimum(p - 1, beta.astype(np.int32))
    qid = np.minimum(q - 1, gamma.astype(np.int32))
    b0 = beta - p0.astype(F32)
    p1 = np.where(b0 < F32(0.5), np.maximum(0, p0 - 1), np.minimum(p - 1, p0 + 1))
    single = p0 == p1
    w1 = np.where(single, F32(0), np.abs(b0 - F32(0.5))).astype(F32)
    w0 = (F32(1) - w1).astype(F32)
    idx = np.zeros((len(dist), 3), np.int32)
    coeff = np.zeros((len(dist), 3), F32)
    coeff[:, 0] = self_c
    idx[:, 1] = qid * p * n + p0 * n + nid + 1
    coeff[:, 1] = w0 * (F32(1) - self_c)
    idx[:, 2] = np.where(single, 0, qid * p * n + p1 * n + nid + 1)
    coeff[:, 2] = np.where(single, F32(0), w1 * (F32(1) - self_c))
    return idx, coeff, (alpha, beta, gamma)


# ----------------------------------------------------------------------------------------------- convolution
def _pair_weights(filt, bin_index, bin_coeff, dtype):
    """w[p, c, m] = sum_t coeff[p, t] * filter[bin[p, t], c, m]; the plain form has one bin of weight 1."""
    filt = np.asarray(filt, dtype)
    if bin_coeff is None:
        return filt[np.asarray(bin_index).reshape(-1)]
    return np.einsum("pt,ptcm->pcm", np.asarray(bin_coeff, dtype), filt[np.asarray(bin_index)])


def conv_fwd(x, filt, nn_count, nn_index, bin_index, bin_coeff=None, dtype=np.float64):
    """pcloud_conv3d_gpu.cu:8-26 (plain), :94-118 (fuzzy):
    out[o, c*r+m] = (1 / nn_count[o]) sum_{pairs (o, i)} x[i, c] * w[pair, c, m]."""
    x = np.asarray(x, dtype)
    w = _pair_weights(filt, bin_index, bin_coeff, dtype)
    o, i = nn_index[:, 0].astype(np.int64), nn_index[:, 1].astype(np.int64)
    term = x[i][:, :, None] * w / np.asarray(nn_count, dtype)[o][:, None, None]
    out = np.zeros((len(nn_count), w.shape[1], w.shape[2]), dtype)
    np.add.at(out, o, term)
    return out.reshape(len(nn_count), -1)


def conv_bwd(gout, x, filt, nn_count, nn_index, bin_index, bin_coeff=None, dtype=np.float64):
    """pcloud_conv3d_gpu.cu:28-84, :121-200 -> (grad_input (Np, C), grad_filter (F, C, r))."""
    x, filt = np.asarray(x, dtype), np.asarray(filt, dtype)
    F, C, r = filt.shape
    w = _pair_weights(filt, bin_index, bin_coeff, dtype)
    o, i = nn_index[:, 0].astype(np.int64), nn_index[:, 1].astype(np.int64)
    g = np.asarray(gout, dtype).reshape(-1, C, r)[o] / np.asarray(nn_count, dtype)[o][:, None, None]
    gin = np.zeros_like(x)
    np.add.at(gin, i, (g * w).sum(2))
    d = g * x[i][:, :, None]                                        # (pairs, C, r)
    gfilt = np.zeros_like(filt)
    if bin_coeff is None:
        np.add.at(gfilt, np.asarray(bin_index).reshape(-1), d)
    else:
        bc = np.asarray(bin_coeff, dtype)
        for t in range(bc.shape[1]):
            np.add.at(gfilt, np.asarray(bin_index)[:, t], bc[:, t, None, None] * d)
    return gin, gfilt


# ----------------------------------------------------------------------------------------------- pooling
def pool_max_fwd(x, nn_count, nn_index):
    """pcloud_pool3d_gpu.cu:20-79: per query and channel the largest neighbour value and the neighbour that holds it.
    DETERMINISTIC: among equal values the first pair in nn_index order; a query without neighbours gives 0 and index
    -1 (the reference leaves index 0 there)."""
    x = np.asarray(x)
    out = np.zeros((len(nn_count), x.shape[1]), x.dtype)
    idx = np.full((len(nn_count), x.shape[1]), -1, np.int32)
    seen = np.zeros(len(nn_count), bool)
    for o, i in nn_index[:, :2].tolist():
        if not seen[o]:
            out[o], idx[o], seen[o] = x[i], i, True
        else:
            better = x[i] > out[o]
            out[o] = np.where(better, x[i], out[o])
            idx[o] = np.where(better, i, idx[o])
    return out, idx


def pool_max_bwd(gout, n_in, max_index):
    """pcloud_pool3d_gpu.cu:83-96."""
    gin = np.zeros((n_in, gout.shape[1]), gout.dtype)
    o, c = np.nonzero(max_index >= 0)
    np.add.at(gin, (max_index[o, c], c), gout[o, c])
    return gin


def pool_avg_fwd(x, nn_count, nn_index, dtype=np.float64):
    """pcloud_pool3d_gpu.cu:99-114."""
    x = np.asarray(x, dtype)
    o, i = nn_index[:, 0].astype(np.int64), nn_index[:, 1].astype(np.int64)
    out = np.zeros((len(nn_count), x.shape[1]), dtype)
    np.add.at(out, o, x[i] / np.asarray(nn_count, dtype)[o][:, None])
    return out


def pool_avg_bwd(gout, n_in, nn_count, nn_index, dtype=np.float64):
    """pcloud_pool3d_gpu.cu:117-133."""
    gout = np.asarray(gout, dtype)
    o, i = nn_index[:, 0].astype(np.int64), nn_index[:, 1].astype(np.int64)
    gin = np.zeros((n_in, gout.shape[1]), dtype)
    np.add.at(gin, i, gout[o] / np.asarray(nn_count, dtype)[o][:, None])
    return gin


def unpool_fwd(x, weight, nn_index, dtype=np.float64):
    """pcloud_unpool3d_gpu.cu:1-19: out[o] = sum_k x[nn_index[o, k]] * weight[o, k]."""
    x, weight = np.asarray(x, dtype), np.asarray(weight, dtype)
    return np.einsum("okc,ok->oc", x[nn_index.astype(np.int64)], weight)


def unpool_bwd(gout, n_in, weight, nn_index, dtype=np.float64):
    """pcloud_unpool3d_gpu.cu:21-39."""
    gout, weight = np.asarray(gout, dtype), np.asarray(weight, dtype)
    gin = np.zeros((n_in, gout.shape[1]), dtype)
    for k in range(nn_index.shape[1]):
        np.add.at(gin, nn_index[:, k].astype(np.int64), gout * weight[:, k:k + 1])
    return gin
