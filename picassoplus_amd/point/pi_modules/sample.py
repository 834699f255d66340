"""Farthest point sampling: API of picasso/point/pi_modules/sample.py (fps_ :5)."""
import torch

from . import point_sample as module


def fps_(xyz_in, nv_in, nv_out):
    """xyz_in (Np,3) float32, nv_in / nv_out (B,) int32 points per sample before / after -> sample_index (Mp,) int32
    into xyz_in: per sample its first point, then repeatedly the point farthest from those chosen."""
    nv_in = torch.cumsum(nv_in, dim=-1, dtype=torch.int32)
    nv_out = torch.cumsum(nv_out, dim=-1, dtype=torch.int32)
    return module.fps(xyz_in[..., :3].contiguous(), nv_in, nv_out)
