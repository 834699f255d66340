"""One generator for the six differentiable ops of the mesh layer.

Every op of picasso/mesh/pi_modules/{conv3d,pool3d,unpool3d}.py has the same shape: a native forward,
a native backward that receives ``grad_output`` followed by what forward saved, gradients for the
leading float inputs only, and index / coefficient inputs whose ``requires_grad`` flag the reference
clears in place (conv3d.py:8-9, pool3d.py:8-10, unpool3d.py:8-9).  ``native_op`` builds the
``torch.autograd.Function`` from that description.
"""
import torch


def native_op(name, forward, backward, n_inputs, n_grads, keep=None, selective=False):
    """Build the autograd Function ``name``.

    forward(*inputs)            -> output, or (output, *extras) where extras are saved, not returned
    backward(grad, *saved)      -> one gradient or a sequence of ``n_grads`` gradients, for inputs[:n_grads]
    keep(inputs, extras)        -> tuple of tensors to save (default: all inputs, then the extras)
    selective                   -> backward also takes ``needs=`` (one flag per gradient, from
                                   ``ctx.needs_input_grad``) and may return ``None`` where it is False
    Inputs past the first ``n_grads`` are indices / coefficients: they get ``None`` gradients and
    their ``requires_grad`` flag is cleared in place, as in the reference.
    """

    def fwd(ctx, *inputs):
        if len(inputs) != n_inputs:
            raise TypeError("%s expects %d arguments, got %d" % (name, n_inputs, len(inputs)))
        for t in inputs[n_grads:]:
            if t.requires_grad:
                t.requires_grad = False
        result = forward(*inputs)
        output, extras = (result[0], tuple(result[1:])) if isinstance(result, (tuple, list)) else (result, ())
        ctx.save_for_backward(*(keep(inputs, extras) if keep else tuple(inputs) + extras))
        return output

    def bwd(ctx, grad_output):
        if selective:
            grads = backward(grad_output.contiguous(), *ctx.saved_tensors, needs=tuple(ctx.needs_input_grad[:n_grads]))
        else:
            grads = backward(grad_output.contiguous(), *ctx.saved_tensors)
        grads = tuple(grads) if isinstance(grads, (tuple, list)) else (grads,)
        return grads + (None,) * (n_inputs - len(grads))

    return type(name, (torch.autograd.Function,), {"forward": staticmethod(fwd), "backward": staticmethod(bwd),
                                                   "__doc__": "autograd Function of %s" % name})
