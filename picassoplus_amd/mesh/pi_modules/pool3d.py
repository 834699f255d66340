"""Differentiable mesh pooling: API of picasso/mesh/pi_modules/pool3d.py (maxPool :23, avgPool :43)."""
import torch

from . import mesh_pool3d as module


def _no_grad_flags(*tensors):
    for t in tensors:
        if t.requires_grad:
            t.requires_grad = False


class MaxPoolFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, vt_replace, vt_map, vt_out):
        _no_grad_flags(vt_replace, vt_map, vt_out)
        output, max_index = module.max_forward(input, vt_replace, vt_map, vt_out)
        # the reference keeps (input, max_index) (pool3d.py:13); the two cluster maps ride along so
        # that backward can gather per fine vertex instead of zero-filling and scattering
        ctx.save_for_backward(input, max_index, vt_replace, vt_map)
        ctx.mark_non_differentiable(max_index)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input, max_index, vt_replace, vt_map = ctx.saved_tensors
        grad_input = module.max_backward(grad_output.contiguous(), input, max_index, vt_replace, vt_map)
        return grad_input, None, None, None


def maxPool(input, vt_replace, vt_map, vt_out):
    return MaxPoolFunction.apply(input, vt_replace, vt_map, vt_out)


class AvgPoolFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, vt_replace, vt_map, vt_out):
        _no_grad_flags(vt_replace, vt_map, vt_out)
        output = module.avg_forward(input, vt_replace, vt_map, vt_out)
        ctx.save_for_backward(input, vt_replace, vt_map)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        grad_input = module.avg_backward(grad_output.contiguous(), *ctx.saved_tensors)
        return grad_input, None, None, None


def avgPool(input, vt_replace, vt_map, vt_out):
    return AvgPoolFunction.apply(input, vt_replace, vt_map, vt_out)
