"""Native neighbour queries: counterpart of the reference's ``point_nnquery`` extension
(picasso/point/pi_modules/source/nnquery.cpp:176-178), same three functions.  ``nv_database`` / ``nv_query`` are
inclusive running totals of the points per sample, as the reference's wrapper passes them."""
import torch

from ... import _lib
from ...mesh.pi_modules._check import F32, I32, check_input, same_device, stream_of


def _dims(database, query, nv_database, nv_query):
    check_input(database, "database", 2, F32)
    check_input(query, "query", 2, F32)
    check_input(nv_database, "nv_database", 1, I32)
    check_input(nv_query, "nv_query", 1, I32)
    if database.shape[1] != 3:
        raise RuntimeError("Shape of database points requires to be (Np, 3)")
    if query.shape[1] != 3:
        raise RuntimeError("Shape of query points requires to be (Mp, 3)")
    if nv_database.shape[0] != nv_query.shape[0]:
        raise RuntimeError("Shape of nv_database and nv_query should be identical")
    return database.shape[0], query.shape[0], nv_database.shape[0], same_device(database, query, nv_database, nv_query)


# Databases of at least this many points are searched through a cell grid (same outputs; the cost of a query then
# grows with its neighbours, not with its sample), smaller ones by the scan over the query's sample.
GRID_MIN_POINTS = 2048
GRID_MAX_SAMPLES = 1 << 20
KNN_CELLS_PER_POINT = 4.0        # cells of the nearest-neighbour grid per database point of a sample


def _search(kind, database, query, nv_database, nv_query, size, nn_sample, grid_size=None):
    Np, Mp, B, dev = _dims(database, query, nv_database, nv_query)
    if not nn_sample > 0:
        raise RuntimeError("BuildSphereNeighbor requires nn_sample>0")
    nn_sample = int(min(nn_sample, 2147483647))
    st = stream_of(database)
    args = (database.data_ptr(), query.data_ptr(), nv_database.data_ptr(), nv_query.data_ptr(), B, Np, Mp, float(size))
    with torch.cuda.device(dev):
        count = torch.zeros(Mp, dtype=I32, device=dev)
        if Mp and Np >= max(GRID_MIN_POINTS, 1) and 0 < B <= GRID_MAX_SAMPLES:
            grid = torch.empty(_lib.query("pmesh_point_grid_workspace_bytes", Np), dtype=torch.uint8, device=dev)
            _lib.call("pmesh_point_grid_build", database.data_ptr(), nv_database.data_ptr(), B, Np,
                      float(size) if kind == "range" else float(size) / 2, grid.data_ptr(), grid.numel(), st)
            args = (grid.data_ptr(),) + args
            kind_fn = kind + "_%s_grid"
        else:
            kind_fn = kind + "_%s"
        _lib.call("pmesh_point_" + kind_fn % "count", *args, nn_sample, count.data_ptr(), st)
        cnt_info = torch.cumsum(count, 0, dtype=torch.int64)
        n_out = int(cnt_info[-1]) if Mp else 0                   # the pair arrays are sized on the host, as in the reference
        width = 2 if kind == "range" else 3
        nn_index = torch.empty((n_out, width), dtype=I32, device=dev)
        if kind == "range":
            nn_dist = torch.empty(n_out, dtype=F32, device=dev)
            _lib.call("pmesh_point_" + kind_fn % "fill", *args, cnt_info.data_ptr(), n_out, nn_index.data_ptr(), nn_dist.data_ptr(), st)
            return cnt_info, nn_index, nn_dist
        _lib.call("pmesh_point_" + kind_fn % "fill", *args, int(grid_size), cnt_info.data_ptr(), n_out, nn_index.data_ptr(), st)
        return cnt_info, nn_index


def range(database, query, nv_database, nv_query, radius, nn_sample):
    """nnquery.cpp:29-78 -> (cnt_info int64 (Mp) running total of neighbours, nn_index (Nout,2) int32, nn_dist (Nout))."""
    if not radius > 0:
        raise RuntimeError("Range search requires radius>0")
    return _search("range", database, query, nv_database, nv_query, radius, nn_sample)


def cube(database, query, nv_database, nv_query, length, nn_sample, grid_size):
    """nnquery.cpp:81-129 -> (cnt_info, nn_index (Nout,3) int32: query, database point, grid cell)."""
    if not length > 0:
        raise RuntimeError("Cube size requires length>0")
    if not grid_size > 0:
        raise RuntimeError("Need grid_size>0")
    return _search("cube", database, query, nv_database, nv_query, length, nn_sample, grid_size)


def knn3(database, query, nv_database, nv_query):
    """nnquery.cpp:132-171 -> (nn_index (Mp,3) int32, nn_dist (Mp,3))."""
    Np, Mp, B, dev = _dims(database, query, nv_database, nv_query)
    with torch.cuda.device(dev):
        nn_index = torch.empty((Mp, 3), dtype=I32, device=dev)
        nn_dist = torch.empty((Mp, 3), dtype=F32, device=dev)
        if Mp and Np >= max(GRID_MIN_POINTS, 1) and 0 < B <= GRID_MAX_SAMPLES:
            # a cell grid with about KNN_CELLS_PER_POINT cells per point of a sample: a query looks at the cells around it
            grid = torch.empty(_lib.query("pmesh_point_grid_workspace_bytes", Np), dtype=torch.uint8, device=dev)
            st = stream_of(database)
            _lib.call("pmesh_point_grid_build", database.data_ptr(), nv_database.data_ptr(), B, Np, -float(KNN_CELLS_PER_POINT),
                      grid.data_ptr(), grid.numel(), st)
            _lib.call("pmesh_point_knn3_grid", grid.data_ptr(), database.data_ptr(), query.data_ptr(), nv_database.data_ptr(),
                      nv_query.data_ptr(), B, Np, Mp, nn_index.data_ptr(), nn_dist.data_ptr(), st)
            return nn_index, nn_dist
        _lib.call("pmesh_point_knn3", database.data_ptr(), query.data_ptr(), nv_database.data_ptr(), nv_query.data_ptr(), B, Np,
                  Mp, nn_index.data_ptr(), nn_dist.data_ptr(), stream_of(database))
    return nn_index, nn_dist
