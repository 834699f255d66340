"""Graph builders of the point-cloud branch with the names of picasso/point/utils.py."""
import numpy as np
import torch

from .layers import BuildSpharmCoeff
from .pi_modules.buildkernel import SPH3Dkernel_, fuzzySPH3Dkernel_
from .pi_modules.nnquery import cube_search_, knn3_search_, range_search_
from .pi_modules.sample import fps_


def range_search(xyz_data, xyz_query, nv_data, nv_query, radius, max_nn):
    """utils.py:15-18 -> (nn_cnt, nn_idx, nn_dst)."""
    cnt_info, nn_cnt, nn_idx, nn_dst = range_search_(xyz_data, xyz_query, nv_data, nv_query, radius=radius, nnsample=max_nn)
    return nn_cnt, nn_idx, nn_dst


def cube_search(xyz_data, xyz_query, nv_data, nv_query, length, nnsample=None, gridsize=4):
    """utils.py:21-24 -> (cnt_info, nn_cnt, nn_idx (Nout,3)).  (The reference unpacks four values from the three that
    its ``cube_search_`` returns and raises; this returns the three.)"""
    return cube_search_(xyz_data, xyz_query, nv_data, nv_query, length=length, nnsample=nnsample, gridsize=gridsize)


def knn3_search(xyz_data, xyz_query, nv_data, nv_query):
    """utils.py:27-29 -> (nn_idx (Mp,3), nn_dst (Mp,3))."""
    return knn3_search_(xyz_data, xyz_query, nv_data, nv_query)


def compute_unpool_weight(nn_dist):
    """Inverse-distance weights (utils.py:32-36).  The reference divides every row by the sum of the FIRST row
    (``torch.sum(...)[0]``); the same here."""
    weight = 1 / (nn_dist + np.finfo(float).eps)
    return weight / torch.sum(weight, dim=-1, keepdim=True)[0]


def fps(xyz_in, nv_xyz, num_sample):
    """utils.py:39-41."""
    return fps_(xyz_in, nv_xyz, num_sample)


def build_range_graph(xyz_data, xyz_query, nv_data, nv_query, radius, nn_uplimit=None, kernel_shape=None, fuzzy=True):
    """utils.py:44-59 -> (nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff or None)."""
    nn_cnt, nn_idx, nn_dst = range_search(xyz_data, xyz_query, nv_data, nv_query, radius=radius, max_nn=nn_uplimit)
    if fuzzy:
        filt_idx, filt_coeff = fuzzySPH3Dkernel_(xyz_data, xyz_query, nn_idx, nn_dst, radius, kernel=kernel_shape)
        return nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff
    filt_idx = SPH3Dkernel_(xyz_data, xyz_query, nn_idx, nn_dst, radius, kernel=kernel_shape)
    return nn_cnt, nn_idx, nn_dst, filt_idx, None


def build_cube_graph(xyz_data, xyz_query, nv_data, nv_query, radius, nn_uplimit=None, grid_size=None):
    """utils.py:62-69 -> (nn_cnt, nn_idx (Nout,2), None, filt_idx (Nout,), None)."""
    cnt_info, nn_cnt, nn_idx = cube_search(xyz_data, xyz_query, nv_data, nv_query, length=2 * radius, nnsample=nn_uplimit,
                                           gridsize=grid_size)
    return nn_cnt, nn_idx[:, :-1].contiguous(), None, nn_idx[:, -1].contiguous(), None


def build_sphere_harmonics(xyz_data, xyz_query, nv_data, nv_query, radius, L=2, nn_uplimit=None):
    """The graph ``DualBlock`` convolves on (utils.py:72-85, picasso/networks/pi2_blocks.py:56-62): range search, then per
    pair (L+1)^2 + 1 weighted bins: 1 - gamma for the centre and gamma * Y_lm(direction), gamma = distance / radius."""
    kernel_size = (L + 1) ** 2 + 1
    nn_cnt, nn_idx, nn_dst = range_search(xyz_data, xyz_query, nv_data, nv_query, radius=radius, max_nn=nn_uplimit)
    gamma = torch.clip(nn_dst[:, None] / radius, 0, 1)
    filt_coeff = BuildSpharmCoeff(L)(xyz_data, xyz_query, nn_idx)
    filt_coeff = torch.concat([1 - gamma, gamma * filt_coeff], dim=-1).contiguous()
    filt_idx = torch.arange(kernel_size, dtype=torch.int, device=filt_coeff.device)
    filt_idx = torch.tile(filt_idx, [filt_coeff.shape[0], 1]).contiguous()
    return nn_cnt, nn_idx, nn_dst, filt_idx, filt_coeff
