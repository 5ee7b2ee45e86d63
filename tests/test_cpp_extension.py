"""The torch C++ extension with the reference's pybind surface: AbstractCompressor classes,
registry operations and torch.ops.tutel_ops.cumsum."""
import numpy as np
import pytest
import torch

import oracle
from helpers import bf16_bits, np_raw, raw

DEV = "cuda:0"


def test_module_surface_and_host_side_errors():
    from planmoe_amd import ext
    ck = ext.install_alias()
    import schemoe_custom_kernel
    assert schemoe_custom_kernel is ck
    for name in ("compress_operation", "comm_operation", "decompress_operation", "clear_ptr_lst",
                 "invoke_cpu_fp32", "invoke_cpu_fp64"):
        assert hasattr(ck, name)
    assert hasattr(torch.ops.tutel_ops, "cumsum")
    ck.clear_ptr_lst()
    with pytest.raises(RuntimeError, match="no matching compress_operation"):
        ck.decompress_operation(torch.zeros(4))
    with pytest.raises(RuntimeError, match="no matching compress_operation"):
        ck.comm_operation(torch.zeros(4))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ck.compress_operation(torch.zeros(4, 4, 8), "int8", "naive")
    ck.clear_ptr_lst()
    with pytest.raises(RuntimeError, match="no CPU kernels"):
        ck.invoke_cpu_fp32([torch.zeros(1)], [1, 1, 1], 0)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ck.compress_operation(torch.zeros(4, 4, 8), "lz", "naive")
    ck.clear_ptr_lst()


@pytest.mark.gpu
def test_zfp_shape_assertion_like_the_reference():
    from planmoe_amd import ext
    ck = ext.load()
    ck.clear_ptr_lst()
    with pytest.raises(RuntimeError, match="zfp fails."):
        ck.compress_operation(torch.zeros(4, 6, 8, device=DEV), "zfp", "naive")
    ck.clear_ptr_lst()


@pytest.mark.gpu
def test_pipeline_through_the_cpp_registry():
    from planmoe_amd import ext
    ck = ext.load()
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 64, 256, generator=g).to(DEV)
    ck.clear_ptr_lst()
    sent = [ck.compress_operation(x, name, "naive") for name in ("no", "int8", "zfp")]
    assert sent[0].data_ptr() == x.data_ptr()
    assert sent[1].dtype == torch.float32 and sent[1].numel() == x.numel() // 4
    assert sent[2].dtype == torch.float16 and sent[2].numel() == (oracle.zfp_max_bytes(2, 256, 256) + 1) // 2
    recv = [ck.comm_operation(s) for s in sent]
    assert all(r.data_ptr() != s.data_ptr() for r, s in zip(recv, sent))
    dec = [ck.decompress_operation(r) for r in recv]
    assert torch.equal(dec[0], x)
    rc, rb, rs = oracle.int8_compress(x.cpu().numpy())
    assert np.array_equal(sent[1].view(torch.uint8).cpu().numpy(), rc.reshape(-1))
    assert np.array_equal(raw(dec[1]), oracle.int8_decompress(rc, rb, rs).view(np.int32))
    st = oracle.zfp_compress(x.cpu().numpy().reshape(-1, 256), 2)
    assert np.array_equal(sent[2].view(torch.uint8).cpu().numpy()[:len(st)], st)
    assert np.array_equal(raw(dec[2]), oracle.zfp_decompress(st, 256, 256, 2).reshape(4, 64, 256).view(np.int32))
    with pytest.raises(RuntimeError):
        ck.decompress_operation(recv[0])                 # objects are single use
    bx = x.bfloat16()
    ck.clear_ptr_lst()
    d = ck.decompress_operation(ck.comm_operation(ck.compress_operation(bx, "int8", "pipe")))
    rc, rb, rs = oracle.int8_compress(bf16_bits(bx))
    assert d.dtype == torch.bfloat16 and np.array_equal(raw(d), np_raw(oracle.int8_decompress(rc, rb, rs)))


@pytest.mark.gpu
def test_lz_through_the_cpp_registry():
    from planmoe_amd import ext
    ck = ext.load()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(4, 64, 256, generator=g)
    x[1] = 0.0                                           # empty capacity slots
    x = x.to(DEV)
    ck.clear_ptr_lst()
    sent = ck.compress_operation(x, "lz", "naive")
    assert sent.data_ptr() == x.data_ptr()               # lz.cpp:40 returns its input
    recv = ck.comm_operation(sent)
    assert recv.data_ptr() != x.data_ptr() and not recv.any()     # g_output = zeros_like (lz.cpp:25)
    dec = ck.decompress_operation(recv)
    assert dec.data_ptr() == recv.data_ptr()             # decoded in place (lz.cpp:52-59)
    assert torch.equal(dec, x)
    ck.clear_ptr_lst()
    with pytest.raises(RuntimeError, match="Float"):
        ck.compress_operation(x.bfloat16(), "lz", "naive")
    ck.clear_ptr_lst()


@pytest.mark.gpu
def test_tutel_ops_cumsum():
    from planmoe_amd import ext
    ext.load()
    m = (torch.rand(3000, 8, generator=torch.Generator().manual_seed(0)) < 0.3).to(torch.int64)
    out = torch.ops.tutel_ops.cumsum(m.to(DEV))
    assert out.dtype == torch.int32 and np.array_equal(out.cpu().numpy(), oracle.cumsum_sub_one(m.numpy()))
