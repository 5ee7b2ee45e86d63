"""planmoe_forward_int8_static: the forward chain through the entry point that allocates nothing
(its workspace is a buffer built into the library's device image) against planmoe_forward_int8
with a caller's workspace, bit for bit, on two calls in a row, the second on a smaller input
(the built-in buffer then still holds the first call's contents)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

KEYS = ("indices", "locations", "gates", "l_aux", "counts", "codes", "bias", "scale")


def _inputs(T, M, E, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    return x, wg


def _same(a, b):
    for key in KEYS:
        ta, tb = a[key], b[key]
        if ta.dtype in (torch.bfloat16, torch.float16):
            ta, tb = ta.view(torch.int16), tb.view(torch.int16)
        elif ta.dtype == torch.float32:
            ta, tb = ta.view(torch.int32), tb.view(torch.int32)
        assert torch.equal(ta, tb), key


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls():
    from planmoe_amd import ops
    for T, M, E, k, cf, seed in ((4096, 2048, 8, 2, 1.25, 11), (1000, 1024, 8, 2, 1.25, 12)):
        x, wg = _inputs(T, M, E, seed)
        C = ops.capacity(T, E, k, cf, 4)
        want = ops.forward_int8(x, wg, k, C, want_counts=True)
        got = {key: (torch.full_like(v, 77) if v is not None else None) for key, v in want.items()}
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(DEV)["allocation.all.allocated"]
        ops.forward_int8_static(x, wg, k, C, got)
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(DEV)["allocation.all.allocated"] == before     # no torch allocation either
        _same(want, got)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from planmoe_amd._lib import lib
    p = ctypes.c_void_p(256)
    # 4 M tokens need far more than the built-in 4 MiB: an error, and nothing is enqueued
    rc = lib.planmoe_forward_int8_static(p, p, 1, 1, None, 1 << 22, 512, 8, 2, 1, 16, p, p, p, 1 << 22, None, None,
                                         None, None, p, p, p, None)
    assert rc != 0 and b"built-in buffer" in lib.planmoe_last_error()
