"""Capacity cumsum -- mirror of the reference's jit_kernels/gating.py:13-22."""
import torch

from . import ops


def fast_cumsum_sub_one(data, dim=0):
    """cumsum(data, dim=0) - 1 of a 2-D integer mask on the GPU (int32 result, as the
    reference's CUDA path returns, custom_kernel.cpp:334)."""
    if data.dim() != 2 or dim != 0:
        raise Exception("Unimplemented fast_cumsum_sub_one() of data = %s and dim = %s" % (data.size(), dim))
    if not data.is_cuda:
        return torch.cumsum(data, dim=0) - 1        # host tensors: gating.py:13-15, 20-21
    return ops.cumsum_sub_one(data)
