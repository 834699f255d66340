"""Argument checks shared by the native op wrappers.

Same contract as the reference's CHECK_INPUT macros (mesh_conv3d.cpp:24-30): device tensor,
contiguous, fixed rank -- violations raise RuntimeError -- plus the dtype check that the
reference gets from ``data_ptr<T>()``.
"""
import torch


def check_input(x, name, dims, dtype):
    if not isinstance(x, torch.Tensor):
        raise RuntimeError("%s must be a tensor" % name)
    if not x.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not x.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if x.dim() != dims:
        raise RuntimeError("%s must have dimension of %d" % (name, dims))
    if x.dtype != dtype:
        raise RuntimeError("expected scalar type %s for %s but found %s" % (dtype, name, x.dtype))


def same_device(*tensors):
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def stream_of(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


F32, I32, BF16 = torch.float32, torch.int32, torch.bfloat16


def feature_dtype(x, name):
    """float32, or bfloat16 for the reduced-precision variant (features in bf16 in HBM); anything else raises like
    a dtype mismatch in the reference's ``data_ptr<float>()``."""
    if isinstance(x, torch.Tensor) and x.dtype in (F32, BF16):
        return x.dtype
    raise RuntimeError("expected scalar type Float (or BFloat16 features) for %s but found %s"
                       % (name, getattr(x, "dtype", type(x))))
