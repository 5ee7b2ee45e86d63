"""Capacity cumsum -- mirror of the reference's jit_kernels/gating.py:13-22."""
from . import ops
from ._lib import PlanMoEError


def fast_cumsum_sub_one(data, dim=0):
    """cumsum(data, dim=0) - 1 of a 2-D integer mask on the GPU (int32 result, as the
    reference's CUDA path returns, custom_kernel.cpp:334)."""
    if data.dim() != 2 or dim != 0:
        raise Exception("Unimplemented fast_cumsum_sub_one() of data = %s and dim = %s" % (data.size(), dim))
    if not data.is_cuda:
        raise PlanMoEError("fast_cumsum_sub_one: CPU tensors are not supported by this build")
    return ops.cumsum_sub_one(data)
