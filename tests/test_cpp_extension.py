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
    with pytest.raises(RuntimeError, match="expects 5 tensors"):
        ck.invoke_cpu_fp32([torch.zeros(1)], [1, 1, 1], 0)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ck.compress_operation(torch.zeros(4, 4, 8), "lz", "naive")
    ck.clear_ptr_lst()
    # the reference's NVRTC entry points exist and say what replaced them (custom_kernel.cpp:295-298)
    for call in (lambda: ck.update_sdk_home(torch.zeros(1)), lambda: ck.inject_source("__global__ void f() {}"),
                 lambda: ck.invoke([torch.zeros(1)], [1], 0)):
        with pytest.raises(RuntimeError, match="no run-time kernel compiler"):
            call()


def _load_example_plugin():
    """The example third-party compressor: built against include/planmoe/compressor/abstract.h by
    ext/build.py, linked against the extension module, registered under the name 'half'."""
    import ctypes
    import os
    from planmoe_amd import ext
    ck = ext.load()
    path = os.path.join(os.path.dirname(ext.PATH), "libexample_third_party_compressor.so")
    assert os.path.exists(path), "run python planmoe_amd/csrc/ext/build.py"
    ctypes.CDLL(path).register_example_compressor()
    return ck


def test_third_party_compressor_registers():
    ck = _load_example_plugin()
    assert "half" in ck.registered_compressors()


@pytest.mark.gpu
def test_third_party_compressor_runs_through_the_registry():
    """A subclass of AbstractCompressor compiled outside the extension goes through
    compress_operation / comm_operation / decompress_operation like a built-in one."""
    ck = _load_example_plugin()
    x = torch.randn(4, 64, 256, generator=torch.Generator().manual_seed(9)).to(DEV)
    ck.clear_ptr_lst()
    sent = ck.compress_operation(x, "half", "naive")
    assert sent.dtype == torch.float16 and torch.equal(sent, x.half())
    recv = ck.comm_operation(sent)
    assert recv.data_ptr() != sent.data_ptr()
    out = ck.decompress_operation(recv)
    assert out.dtype == torch.float32 and torch.equal(out, x.half().float())
    ck.clear_ptr_lst()


@pytest.mark.gpu
def test_comm_runs_on_its_own_stream_under_the_event_protocol():
    """Two chunks, each compress -> comm, then decompress in order (overlap.py:59-74 with degree 2):
    the copies are issued on the comm stream, the results equal those of one chunk at a time, and
    producing the next chunk's input on the compute stream right after cannot overtake a copy."""
    from planmoe_amd import compressor, ext
    ck = ext.load()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(8, 512, 1024, generator=g).bfloat16().to(DEV)
    for mod in (ck, compressor):
        old = compressor.SINGLE_RANK_COMM_COPIES
        compressor.SINGLE_RANK_COMM_COPIES = True
        try:
            mod.clear_ptr_lst()
            whole = mod.decompress_operation(mod.comm_operation(mod.compress_operation(x, "int8", "naive")))
            mod.clear_ptr_lst()
            halves = [h.contiguous() for h in x.split(256, dim=1)]
            recv = []
            for h in halves:
                recv.append(mod.comm_operation(mod.compress_operation(h, "int8", "naive")))
                h.zero_()            # the compute stream moves on and overwrites the chunk it has compressed
            got = torch.cat([mod.decompress_operation(r) for r in recv], dim=1)
            torch.cuda.synchronize()
            assert torch.equal(got, whole)
            mod.clear_ptr_lst()
        finally:
            compressor.SINGLE_RANK_COMM_COPIES = old


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


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_invoke_cpu_against_the_oracle_and_closed_forms(dtype):
    """invoke_cpu_fp32 / fp64 (custom_kernel.cpp:57-112): the reference's calls for host tensors.  The three
    kernel types against the oracle's restatement (bit for bit: same products, same order of sums)
    and against what torch computes for the same thing; dropped pairs (index < 0, location >=
    capacity), errors for GPU-side misuse."""
    from planmoe_amd import ext
    ck = ext.load()
    fn = ck.invoke_cpu_fp32 if dtype == torch.float32 else ck.invoke_cpu_fp64
    T, H, E, C = 37, 24, 5, 8
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, H, generator=g, dtype=dtype)
    gate = torch.rand(T, generator=g, dtype=dtype)
    idx = torch.randint(0, E, (T,), generator=g, dtype=torch.int32)
    # distinct slots for the live pairs, some pairs dropped either way
    perm = torch.randperm(E * C, generator=g)[:T]
    idx, loc = (perm // C).to(torch.int32), (perm % C).to(torch.int32)
    loc[3] = C + 2
    idx[5] = -1
    loc[8] = C
    live = (idx >= 0) & (loc < C)
    # 0: scatter into zeroed slots
    slots = torch.zeros(E * C, H, dtype=dtype)
    fn([gate, idx, loc, x, slots], [T, H, C], 0)
    want = oracle.dispatch(gate.numpy(), idx.numpy(), loc.numpy(), x.numpy(), np.zeros((E * C, H), dtype=x.numpy().dtype), C)
    assert np.array_equal(slots.numpy(), want)
    ref = torch.zeros(E * C, H, dtype=dtype)
    ref[(idx[live].long() * C + loc[live].long())] = gate[live, None] * x[live]
    assert torch.equal(slots, ref)
    fn([gate, idx, loc, x, slots], [T, H, C], 0)                  # it accumulates, as the reference does
    assert torch.equal(slots, ref + ref)
    # 1: gather back
    slots = torch.randn(E * C, H, generator=g, dtype=dtype)
    rows = torch.full((T, H), 7.0, dtype=dtype)
    fn([gate, idx, loc, rows, slots], [T, H, C], 1)
    assert np.array_equal(rows.numpy(), oracle.gather(gate.numpy(), idx.numpy(), loc.numpy(), slots.numpy(), T, C))
    assert bool((rows[~live] == 0).all()) and torch.equal(rows[live], gate[live, None] * slots[idx[live].long() * C + loc[live].long()])
    # 2: gate gradients
    gg = torch.full((T,), 9.0, dtype=dtype)
    fn([gg, idx, loc, x, slots], [T, H, C], 2)
    assert np.array_equal(gg.numpy(), oracle.bwd_gate(idx.numpy(), loc.numpy(), x.numpy(), slots.numpy(), C))
    assert bool((gg[~live] == 0).all())
    full = (slots[idx[live].long() * C + loc[live].long()].double() * x[live].double()).sum(1)
    assert torch.allclose(gg[live].double(), full, rtol=1e-5 if dtype == torch.float32 else 1e-12)
    # misuse
    with pytest.raises(RuntimeError, match="dtype of the entry point"):
        fn([gate.to(torch.float16), idx, loc, x, slots], [T, H, C], 0)
    with pytest.raises(RuntimeError, match="int32"):
        fn([gate, idx.long(), loc, x, slots], [T, H, C], 0)
    with pytest.raises(RuntimeError, match="outside the slots tensor"):
        fn([gate, idx + E, loc, x, slots], [T, H, C], 0)
    with pytest.raises(RuntimeError, match="contiguous"):
        fn([gate, idx, loc, x.t().contiguous().t(), slots], [T, H, C], 0)
