"""The pointwise tail that follows every mesh convolution, as one native pass.

The reference writes it with separate PyTorch ops (picasso/mesh/layers.py:114-119, 169-174, 232-238):
``torch.matmul(outputs, depth_weights) + biases``, the activation, then batch norm.  ``dense_tail``
computes ``act(input @ weight + bias)`` in one kernel and, without gradients, can also apply an
inference-mode batch norm as a per-channel ``scale``/``shift``; its backward takes the ReLU mask from
the saved output, so no pre-activation tensor is kept.
"""
import torch

from ... import _lib
from ._check import F32, check_input, same_device, stream_of, workspace


MAX_CHANNELS = 896     # input channels of the forward, output channels of grad_input: one 32-column weight slab in LDS


def _dims(input, weight, bias):
    check_input(input, "input", 2, F32)
    check_input(weight, "weight", 2, F32)
    N, Ci = input.shape
    if weight.shape[0] != Ci:
        raise RuntimeError("weight must have shape (in_channels, out_channels)")
    Co = weight.shape[1]
    if Ci < 1 or Co < 1 or Ci > MAX_CHANNELS:
        raise RuntimeError("dense tail supports 1..896 input channels, got %d" % Ci)
    if bias is not None:
        check_input(bias, "bias", 1, F32)
        if bias.shape[0] != Co:
            raise RuntimeError("bias must have out_channels entries")
    return N, Ci, Co


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def dense_tail_forward(input, weight, bias=None, relu=True, scale=None, shift=None, with_bits=False):
    """(N,Ci),(Ci,Co),(Co,) -> act(input @ weight + bias) * scale + shift, float32 (N,Co).
    ``with_bits`` also returns the ReLU mask as bits: int32 (N, ceil(Co/32)), bit c%32 of word c//32 set where
    the activated value is positive -- what ``dense_tail_backward`` reads instead of the whole output."""
    N, Ci, Co = _dims(input, weight, bias)
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None:
            check_input(t, name, 1, F32)
            if t.shape[0] != Co:
                raise RuntimeError("%s must have out_channels entries" % name)
    dev = same_device(input, weight, *[t for t in (bias, scale, shift) if t is not None])
    with torch.cuda.device(dev):
        out = torch.empty((N, Co), dtype=F32, device=dev)
        bits = torch.empty((N, (Co + 31) // 32), dtype=torch.int32, device=dev) if with_bits else None
        _lib.call("pmesh_dense_fwd", input.data_ptr(), weight.data_ptr(), _ptr(bias), _ptr(scale), _ptr(shift),
                  1 if relu else 0, out.data_ptr(), _ptr(bits), N, Ci, Co, stream_of(input))
    return (out, bits) if with_bits else out


def dense_tail_backward(grad_output, input, weight, output=None, need_input=True, relu_bits=None):
    """Gradients of ``act(input @ weight + bias)``: ``output`` is the forward result when the activation
    was ReLU (its positive entries pass the gradient), or ``relu_bits`` the bit form of the same mask from
    ``dense_tail_forward(..., with_bits=True)``; both None for no activation.
    -> [grad_input (N,Ci) or None, grad_weight (Ci,Co), grad_bias (Co,)]."""
    N, Ci, Co = _dims(input, weight, None)
    check_input(grad_output, "grad_output", 2, F32)
    if tuple(grad_output.shape) != (N, Co):
        raise RuntimeError("grad_output must have shape (N, out_channels)")
    if output is not None:
        check_input(output, "output", 2, F32)
        if tuple(output.shape) != (N, Co):
            raise RuntimeError("output must have shape (N, out_channels)")
    if relu_bits is not None:
        check_input(relu_bits, "relu_bits", 2, torch.int32)
        if tuple(relu_bits.shape) != (N, (Co + 31) // 32):
            raise RuntimeError("relu_bits must have shape (N, ceil(out_channels / 32))")
    dev = same_device(grad_output, input, weight)
    with torch.cuda.device(dev):
        gin = torch.empty((N, Ci), dtype=F32, device=dev) if need_input else None
        gw = torch.empty((Ci, Co), dtype=F32, device=dev)
        gb = torch.empty((Co,), dtype=F32, device=dev)
        nbytes = _lib.query("pmesh_dense_bwd_workspace_bytes", N, Ci, Co)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_dense_bwd", grad_output.data_ptr(), input.data_ptr(), weight.data_ptr(), _ptr(output),
                  _ptr(relu_bits), _ptr(gin), gw.data_ptr(), gb.data_ptr(), ws.data_ptr(), nbytes, N, Ci, Co, stream_of(input))
    return [gin, gw, gb]


class DenseTailFunction(torch.autograd.Function):
    """autograd Function of dense_tail: gradients for input, weight and bias."""

    @staticmethod
    def forward(ctx, input, weight, bias, relu):
        # the backward pass reads the ReLU mask as bits (1/32 of the output) instead of the output
        if relu:
            out, bits = dense_tail_forward(input, weight, bias, True, with_bits=True)
        else:
            out, bits = dense_tail_forward(input, weight, bias, False), None
        ctx.save_for_backward(input, weight, bits)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight, bits = ctx.saved_tensors
        gin, gw, gb = dense_tail_backward(grad_output.contiguous(), input, weight, None,
                                          need_input=ctx.needs_input_grad[0], relu_bits=bits)
        return gin, gw if ctx.needs_input_grad[1] else None, gb if ctx.needs_input_grad[2] else None, None


def dense_tail(input, weight, bias, relu=True):
    """act(input @ weight + bias) with gradients; ``bias`` (Co,) float32."""
    return DenseTailFunction.apply(input, weight, bias, relu)


# ---------------------------------------------------------------- vertex2facet and its tail in one pass
def v2f_dense_supported(input, filter, weight):
    """The one-pass form takes depth multiplier 1, a multiple of 4 channels and what the tail itself takes."""
    C = input.shape[1]
    return (input.dtype == F32 and filter.shape[2] == 1 and C % 4 == 0 and 0 < C <= MAX_CHANNELS
            and weight.shape[1] >= 1 and input.data_ptr() % 16 == 0 and filter.data_ptr() % 16 == 0)


def v2f_dense_forward(input, filter, face, weight, bias=None, relu=True, scale=None, shift=None, with_bits=False,
                      keep_rows=False):
    """act(vertex2facet(input, filter, face) @ weight + bias) * scale + shift in one kernel: the facet rows of the
    convolution are formed inside the loads of the product.  input (Nv,C), filter (3,C,1), face (Nf,3) int32,
    weight (C,Co) -> (Nf,Co).  ``keep_rows`` also returns the convolution's rows (Nf,C), which the backward pass
    needs; ``with_bits`` the ReLU mask as bits.  Returns out, or (out, bits, rows) when either is asked for."""
    from .. import topology
    from ._check import I32
    check_input(input, "input", 2, F32)
    check_input(filter, "filter", 3, F32)
    check_input(face, "face", 2, I32)
    check_input(weight, "weight", 2, F32)
    Nv, C = input.shape
    Nf, Co = face.shape[0], weight.shape[1]
    if tuple(filter.shape) != (3, C, 1):
        raise RuntimeError("3 filters required, or input Channel size error of the filter")
    if face.shape[1] != 3:
        raise RuntimeError("face must have shape (NfIn, 3)")
    if weight.shape[0] != C:
        raise RuntimeError("weight must have shape (in_channels, out_channels)")
    if C % 4 or C > MAX_CHANNELS:
        raise RuntimeError("the one-pass vertex2facet tail takes a multiple of 4 channels, at most %d" % MAX_CHANNELS)
    for name, t in (("bias", bias), ("scale", scale), ("shift", shift)):
        if t is not None:
            check_input(t, name, 1, F32)
            if t.shape[0] != Co:
                raise RuntimeError("%s must have out_channels entries" % name)
    dev = same_device(input, filter, face, weight, *[t for t in (bias, scale, shift) if t is not None])
    if Nf:
        topology._check_range_cached(face, Nv)
    with torch.cuda.device(dev):
        out = torch.empty((Nf, Co), dtype=F32, device=dev)
        bits = torch.empty((Nf, (Co + 31) // 32), dtype=torch.int32, device=dev) if with_bits else None
        rows = torch.empty((Nf, C), dtype=F32, device=dev) if keep_rows else None
        _lib.call("pmesh_v2f_dense_fwd", input.data_ptr(), filter.data_ptr(), face.data_ptr(), weight.data_ptr(),
                  _ptr(bias), _ptr(scale), _ptr(shift), 1 if relu else 0, out.data_ptr(), _ptr(bits), _ptr(rows),
                  Nv, Nf, C, Co, stream_of(input))
    return (out, bits, rows) if (with_bits or keep_rows) else out


class V2FDenseFunction(torch.autograd.Function):
    """vertex2facet, the product with the pointwise weights, the bias and a ReLU (or no activation) as ONE native
    forward (picasso/mesh/layers.py:108-117 runs them as a native op and three PyTorch ops).  The convolution's rows
    are kept only when a gradient will need them.  Backward: the tail's gradients from the kept rows, then the
    convolution's from what the tail hands down."""

    @staticmethod
    def forward(ctx, input, filter, face, weight, bias, relu):
        if face.requires_grad:
            face.requires_grad = False
        need = any(ctx.needs_input_grad[i] for i in (0, 1, 3, 4))
        res = v2f_dense_forward(input, filter, face, weight, bias, relu, with_bits=bool(relu and need), keep_rows=need)
        out, bits, rows = res if need else (res, None, None)
        ctx.save_for_backward(input, filter, face, weight, bits, rows)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from . import mesh_conv3d
        input, filter, face, weight, bits, rows = ctx.saved_tensors
        need_conv = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        grows, gw, gb = dense_tail_backward(grad_output.contiguous(), rows, weight, None, need_input=need_conv, relu_bits=bits)
        gin = gfilt = None
        if need_conv:
            gin, gfilt = mesh_conv3d.vertex2facet_backward(grows, input, filter, face)
        return (gin if ctx.needs_input_grad[0] else None, gfilt if ctx.needs_input_grad[1] else None, None,
                gw if ctx.needs_input_grad[3] else None, gb if ctx.needs_input_grad[4] else None, None)


def v2f_dense(input, filter, face, weight, bias, relu=True):
    """act(vertex2facet(input, filter, face) @ weight + bias) with gradients for input, filter, weight and bias."""
    return V2FDenseFunction.apply(input, filter, face, weight, bias, relu)


# ---------------------------------------------------------------- facet2vertex and its tail in one pass
def f2v_dense_supported(input, filter, coeff, weight):
    """The one-pass form takes float32 rows, 16 coefficients per facet (degree 3), 32 or 64 convolution channels
    and 32, 64 or 128 output channels; the library decides (its product switches are part of the answer)."""
    if input.dtype != F32 or input.dim() != 2 or filter.dim() != 3 or coeff.dim() != 2 or weight.dim() != 2:
        return False
    K, C, r = filter.shape
    if input.shape[1] != C or coeff.shape[1] != K or weight.shape[0] != C * r:
        return False
    return bool(_lib.query("pmesh_f2v_dense_supported", input.shape[0], C, r, K, weight.shape[1], coeff.data_ptr()))


def f2v_dense_forward(input, filter, coeff, face, nf_count, vt_map, weight, bias=None, relu=True, scale=None, shift=None,
                      with_bits=False, keep_rows=False):
    """act(facet2vertex(input, filter, coeff, face, nf_count, vt_map) @ weight + bias) * scale + shift in one kernel: a
    wavefront multiplies the vertex rows of the convolution by the weights before they leave the chip.
    input (NfIn,C), filter (K,C,r), coeff (NfIn,K), weight (C*r,Co) -> (NvOut,Co).  ``keep_rows`` also returns the
    convolution's rows (NvOut,C*r), which the backward pass needs; ``with_bits`` the ReLU mask as bits.
    Returns out, or (out, bits, rows) when either is asked for."""
    from .. import topology
    from . import mesh_conv3d
    Nf, C, K, r, NvOut, NvIn = mesh_conv3d._f2v_dims(input, filter, coeff, face, nf_count, vt_map)
    check_input(weight, "weight", 2, F32)
    Co = weight.shape[1]
    if weight.shape[0] != C * r:
        raise RuntimeError("weight must have shape (in_channels * multiplier, out_channels)")
    for name, t in (("bias", bias), ("scale", scale), ("shift", shift)):
        if t is not None:
            check_input(t, name, 1, F32)
            if t.shape[0] != Co:
                raise RuntimeError("%s must have out_channels entries" % name)
    if not f2v_dense_supported(input, filter, coeff, weight):
        raise RuntimeError("the one-pass facet2vertex tail takes 16 coefficients, 32 or 64 convolution channels and "
                           "32, 64 or 128 output channels (got K=%d, C*r=%d, Co=%d)" % (K, C * r, Co))
    dev = same_device(input, filter, coeff, face, nf_count, vt_map, weight, *[t for t in (bias, scale, shift) if t is not None])
    rowptr, colidx = topology.vertex_csr(face, vt_map, NvOut)
    with torch.cuda.device(dev):
        out = torch.empty((NvOut, Co), dtype=F32, device=dev)
        bits = torch.empty((NvOut, Co // 32), dtype=torch.int32, device=dev) if with_bits else None
        rows = torch.empty((NvOut, C * r), dtype=F32, device=dev) if keep_rows else None
        nbytes = _lib.query("pmesh_f2v_dense_fwd_workspace_bytes", C, r, Co)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_f2v_dense_fwd", input.data_ptr(), filter.data_ptr(), coeff.data_ptr(), nf_count.data_ptr(),
                  rowptr.data_ptr(), colidx.data_ptr(), weight.data_ptr(), _ptr(bias), _ptr(scale), _ptr(shift),
                  1 if relu else 0, out.data_ptr(), _ptr(bits), _ptr(rows), ws.data_ptr(), nbytes, Nf, NvOut, C, r, K, Co,
                  stream_of(input))
    return (out, bits, rows) if (with_bits or keep_rows) else out


class F2VDenseFunction(torch.autograd.Function):
    """facet2vertex, the product with the pointwise weights, the bias and a ReLU (or no activation) as ONE native
    forward (picasso/mesh/layers.py:163-171 runs them as a native op and three PyTorch ops).  The convolution's rows
    are kept only when a gradient will need them.  Backward: the tail's gradients from the kept rows, then the
    convolution's from what the tail hands down."""

    @staticmethod
    def forward(ctx, input, filter, coeff, face, nf_count, vt_map, weight, bias, relu):
        for t in (coeff, face, nf_count, vt_map):
            if t.requires_grad:
                t.requires_grad = False
        need = any(ctx.needs_input_grad[i] for i in (0, 1, 6, 7))
        res = f2v_dense_forward(input, filter, coeff, face, nf_count, vt_map, weight, bias, relu,
                                with_bits=bool(relu and need), keep_rows=need)
        out, bits, rows = res if need else (res, None, None)
        ctx.save_for_backward(input, filter, coeff, face, nf_count, vt_map, weight, bits, rows)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from . import mesh_conv3d
        input, filter, coeff, face, nf_count, vt_map, weight, bits, rows = ctx.saved_tensors
        need_conv = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        grows, gw, gb = dense_tail_backward(grad_output.contiguous(), rows, weight, None, need_input=need_conv, relu_bits=bits)
        gin = gfilt = None
        if need_conv:
            gin, gfilt = mesh_conv3d.facet2vertex_backward(grows, input, filter, coeff, face, nf_count, vt_map)
        return (gin if ctx.needs_input_grad[0] else None, gfilt if ctx.needs_input_grad[1] else None, None, None, None, None,
                gw if ctx.needs_input_grad[6] else None, gb if ctx.needs_input_grad[7] else None, None)


def f2v_dense(input, filter, coeff, face, nf_count, vt_map, weight, bias, relu=True):
    """act(facet2vertex(...) @ weight + bias) with gradients for input, filter, weight and bias."""
    return F2VDenseFunction.apply(input, filter, coeff, face, nf_count, vt_map, weight, bias, relu)


# ---------------------------------------------------------------- the tail without a product
def bits_supported(C, *tensors):
    """The bit form of the ReLU mask of ``bias_act`` needs whole 32-column words and 16-byte aligned rows."""
    return C % 32 == 0 and all(t.data_ptr() % 16 == 0 for t in tensors)


def bias_act_forward(input, bias=None, relu=True, scale=None, shift=None, with_bits=False):
    """act(input + bias) * scale + shift for a convolution that mixes the channels itself (F2FConv3d,
    picasso/mesh/layers.py:60-64), one pass, float32 (N,C).  ``with_bits`` (C % 32 == 0) also returns the
    ReLU mask as bits, int32 (N, C/32), as ``dense_tail_forward`` does."""
    check_input(input, "input", 2, F32)
    N, C = input.shape
    if with_bits and not bits_supported(C, input):
        raise RuntimeError("the bit mask needs a multiple of 32 channels and 16-byte aligned rows")
    for name, t in (("bias", bias), ("scale", scale), ("shift", shift)):
        if t is not None:
            check_input(t, name, 1, F32)
            if t.shape[0] != C:
                raise RuntimeError("%s must have one entry per channel" % name)
    dev = same_device(input, *[t for t in (bias, scale, shift) if t is not None])
    with torch.cuda.device(dev):
        out = torch.empty((N, C), dtype=F32, device=dev)
        bits = torch.empty((N, C // 32), dtype=torch.int32, device=dev) if with_bits else None
        if C:
            _lib.call("pmesh_bias_act_fwd", input.data_ptr(), _ptr(bias), _ptr(scale), _ptr(shift), 1 if relu else 0,
                      out.data_ptr(), _ptr(bits), N, C, stream_of(input))
    return (out, bits) if with_bits else out


def bias_act_backward(grad_output, output=None, need_input=True, relu_bits=None):
    """-> [grad_input, grad_bias]: grad_input is grad_output where ``output`` > 0, or where ``relu_bits`` (the bit
    form from ``bias_act_forward(..., with_bits=True)``) is set; both None = no activation: grad_output itself;
    grad_bias its column sums."""
    check_input(grad_output, "grad_output", 2, F32)
    N, C = grad_output.shape
    if output is not None:
        check_input(output, "output", 2, F32)
        if tuple(output.shape) != (N, C):
            raise RuntimeError("output must have the shape of grad_output")
    if relu_bits is not None:
        check_input(relu_bits, "relu_bits", 2, torch.int32)
        if C % 32 or tuple(relu_bits.shape) != (N, C // 32):
            raise RuntimeError("relu_bits must have shape (N, channels / 32)")
    masked = output is not None or relu_bits is not None
    dev = same_device(grad_output) if output is None else same_device(grad_output, output)
    with torch.cuda.device(dev):
        gin = torch.empty((N, C), dtype=F32, device=dev) if (need_input and masked) else None
        gb = torch.empty((C,), dtype=F32, device=dev)
        nbytes = _lib.query("pmesh_bias_act_bwd_workspace_bytes", C)
        ws = workspace(nbytes, dev)
        _lib.call("pmesh_bias_act_bwd", grad_output.data_ptr(), _ptr(output), _ptr(relu_bits), _ptr(gin), gb.data_ptr(),
                  ws.data_ptr(), nbytes, N, C, stream_of(grad_output))
    if not masked and need_input:
        gin = grad_output
    return [gin, gb]


class BiasActFunction(torch.autograd.Function):
    """autograd Function of bias_act: gradients for input and bias."""

    @staticmethod
    def forward(ctx, input, bias, relu):
        out = bits = None
        if relu and bits_supported(input.shape[1], input):
            out, bits = bias_act_forward(input, bias, True, with_bits=True)
        else:
            out = bias_act_forward(input, bias, relu)
        ctx.save_for_backward(out if (relu and bits is None) else None, bits)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        out, bits = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if bits is not None and grad_output.data_ptr() % 16:
            grad_output = grad_output.clone()                  # the bit path reads 16-byte pieces
        gin, gb = bias_act_backward(grad_output, out, need_input=ctx.needs_input_grad[0], relu_bits=bits)
        return gin, gb if ctx.needs_input_grad[1] else None, None


def bias_act(input, bias, relu=True):
    """act(input + bias) with gradients; ``bias`` (C,) float32."""
    return BiasActFunction.apply(input, bias, relu)
