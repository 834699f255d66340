"""Neighbour queries: API of picasso/point/pi_modules/nnquery.py (range_search_ :5, cube_search_ :37, knn3_search_ :69).
``nvDatabase`` / ``nvQuery`` are the per-sample point counts; extra feature columns of the point arrays are ignored."""
import torch

from . import point_nnquery as module

INT32_MAX = 2147483647


def _xyz(points):
    return points[..., :3].contiguous()


def _totals(counts):
    return torch.cumsum(counts, dim=-1, dtype=torch.int32)


def _per_query(cnt_info):
    return torch.cat([cnt_info[:1], cnt_info[1:] - cnt_info[:-1]], dim=0).contiguous().to(torch.int)


def range_search_(database, query, nvDatabase, nvQuery, radius=0.1, nnsample=None):
    """-> (cnt_info (Mp) int64 running total, nn_count (Mp) int32, nn_index (Nout,2) int32 [query, database point],
    nn_dist (Nout) float32): the database points of the query's sample closer than ``radius``, in ascending order, at
    most ``nnsample`` of them."""
    cnt_info, nn_index, nn_dist = module.range(_xyz(database), _xyz(query), _totals(nvDatabase), _totals(nvQuery), radius,
                                               INT32_MAX if nnsample is None else nnsample)
    return cnt_info, _per_query(cnt_info), nn_index, nn_dist


def cube_search_(database, query, nvDatabase, nvQuery, length=0.1, nnsample=None, gridsize=4):
    """-> (cnt_info, nn_count, nn_index (Nout,3) int32 [query, database point, cell of the gridsize^3 kernel])."""
    cnt_info, nn_index = module.cube(_xyz(database), _xyz(query), _totals(nvDatabase), _totals(nvQuery), length,
                                     INT32_MAX if nnsample is None else nnsample, gridsize)
    return cnt_info, _per_query(cnt_info), nn_index


def knn3_search_(database, query, nvDatabase, nvQuery):
    """-> (nn_index (Mp,3) int32, nn_dist (Mp,3) float32): the three nearest database points of every query."""
    return module.knn3(_xyz(database), _xyz(query), _totals(nvDatabase), _totals(nvQuery))
