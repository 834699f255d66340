"""Differentiable mesh unpooling: API of picasso/mesh/pi_modules/unpool3d.py (interpolate :21)."""
import torch

from . import mesh_unpool3d as module


class InterpolateFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, vt_replace, vt_map):
        for t in (vt_replace, vt_map):
            if t.requires_grad:
                t.requires_grad = False
        output = module.forward(input, vt_replace, vt_map)
        ctx.save_for_backward(input, vt_replace, vt_map)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input = module.backward(grad_output.contiguous(), *ctx.saved_tensors)
        return grad_input, None, None


def interpolate(input, vt_replace, vt_map):
    return InterpolateFunction.apply(input, vt_replace, vt_map)
