"""Host-side behaviour of the Python mirror that needs no GPU: argument checks, the
compressor registry protocol, plane packing, constructor errors."""
import pytest
import torch

import planmoe_amd
from planmoe_amd import compressor, ops
from planmoe_amd._lib import PlanMoEError


def test_public_names_match_the_reference_module():
    for name in ("fast_cumsum_sub_one", "fast_dispatcher", "extract_critical", "top_k_routing",
                 "fast_encode", "fast_decode", "moe_layer"):
        assert hasattr(planmoe_amd, name)
    assert planmoe_amd.top_k_routing is planmoe_amd.extract_critical


def test_fast_cumsum_sub_one_rejects_unsupported_calls():
    with pytest.raises(Exception, match="Unimplemented fast_cumsum_sub_one"):
        planmoe_amd.fast_cumsum_sub_one(torch.zeros(4, 4, dtype=torch.int32), dim=1)
    with pytest.raises(Exception, match="Unimplemented fast_cumsum_sub_one"):
        planmoe_amd.fast_cumsum_sub_one(torch.zeros(4, dtype=torch.int32))
    with pytest.raises(PlanMoEError):           # no CPU fall-back
        planmoe_amd.fast_cumsum_sub_one(torch.zeros(4, 4, dtype=torch.int32))


def test_cpu_tensors_fail_loudly():
    with pytest.raises(PlanMoEError):
        planmoe_amd.extract_critical(torch.rand(4, 2), 1)
    with pytest.raises(PlanMoEError):
        ops.int8_compress(torch.rand(4, 8))
    d = planmoe_amd.fast_dispatcher(2, 4, 8, torch.float32)
    with pytest.raises(PlanMoEError):
        d.update([torch.zeros(4, dtype=torch.int32)], [torch.zeros(4, dtype=torch.int32)], [torch.ones(4)], 4)


def test_plane_packing_detects_views():
    base = torch.arange(12, dtype=torch.int32).view(3, 4)
    t, stride = ops.planes([base[0], base[1], base[2]], torch.int32)
    assert stride == 4 and t.data_ptr() == base.data_ptr()
    a, b = torch.zeros(4, dtype=torch.int32), torch.ones(4, dtype=torch.int32)
    t, stride = ops.planes([a, b.clone()], torch.int32)
    assert stride == 4 and t.shape == (2, 4) and int(t[1].sum()) == 4
    t, stride = ops.planes([torch.zeros(4, dtype=torch.int64)], torch.int32)
    assert t.dtype == torch.int32


def test_registry_protocol_errors():
    compressor.clear_ptr_lst()
    with pytest.raises(PlanMoEError):
        compressor.decompress_operation(torch.zeros(4))
    with pytest.raises(PlanMoEError):
        compressor.comm_operation(torch.zeros(4))
    # the "no" compressor is pure host logic: FIFO matching and single use
    x0, x1 = torch.arange(8.0), torch.arange(8.0) + 100
    a = compressor.compress_operation(x0, "no", "naive")
    b = compressor.compress_operation(x1, "anything-else-is-no", "pipe")
    ra, rb = compressor.comm_operation(a), compressor.comm_operation(b)
    assert torch.equal(compressor.decompress_operation(ra), x0)
    assert torch.equal(compressor.decompress_operation(rb), x1)
    with pytest.raises(PlanMoEError):
        compressor.decompress_operation(ra)
    compressor.clear_ptr_lst()
    lz = compressor.get_compressor("lz", compressor.get_comm("naive"))
    assert isinstance(lz, compressor.LzCompressor)
    with pytest.raises(PlanMoEError, match="GPU"):
        lz.compress(torch.zeros(4, 4, 8))                # no CPU path
    with pytest.raises(PlanMoEError, match="Float"):
        lz.compress(torch.zeros(4, 4, 8, dtype=torch.bfloat16))


def test_registered_compressor_is_found_before_the_built_in_names():
    """A third-party subclass of the mirror's AbstractCompressor, added by name (the Python twin of
    the C++ extension's registry), goes through compress / comm / decompress_operation."""
    class Negate(compressor.NoCompressor):
        def compress(self, input):
            return super().compress(-input)

        def decompress(self, input):
            return -super().decompress(input)

    compressor.clear_ptr_lst()
    compressor.register("negate", Negate)
    try:
        assert "negate" in compressor.registered()
        x = torch.arange(6.0)
        sent = compressor.compress_operation(x, "negate", "naive")
        assert torch.equal(sent, -x)
        assert torch.equal(compressor.decompress_operation(compressor.comm_operation(sent)), x)
        with pytest.raises(TypeError):
            compressor.register("bad", 3)
    finally:
        compressor._registered.pop("negate", None)
        compressor.clear_ptr_lst()


def test_zfp_compressor_shape_check():
    c = compressor.ZfpCompressor(compressor.get_comm("naive"))
    assert c.compress_rate == 8.0
    with pytest.raises(PlanMoEError, match="zfp fails."):
        c.compress(torch.zeros(4, 6, 8))
    c.set_compress_rate(16.0)
    assert c.compress_rate == 16.0


def test_moe_layer_constructor_errors():
    with pytest.raises(Exception, match="Unrecognized argument provided to Tutel Moe-layer"):
        planmoe_amd.moe_layer({'type': 'top', 'k': 2}, 16, experts={'type': 'ffn', 'count_per_node': 2,
                              'hidden_size_per_expert': 8}, bogus=1)
    with pytest.raises(Exception, match="Unrecognized gate_type"):
        planmoe_amd.moe_layer({'type': 'nope', 'k': 2}, 16, experts={'type': 'ffn', 'count_per_node': 2,
                              'hidden_size_per_expert': 8})
    with pytest.raises(Exception, match="Unrecognized argument provided to Gating module"):
        planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'zzz': 3}, 16, experts={'type': 'ffn', 'count_per_node': 2,
                              'hidden_size_per_expert': 8})
    with pytest.raises(AssertionError):
        planmoe_amd.moe_layer({'type': 'top', 'k': 2}, 15, experts={'type': 'ffn', 'count_per_node': 2,
                              'hidden_size_per_expert': 8})
    m = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'capacity_factor': 1.25, 'fp32_gate': True}, 16,
                              experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 8},
                              compress_name='int8')
    assert m.num_global_experts == 4 and m.gates[0].top_k == 2 and m.gates[0].capacity_factor == 1.25
    assert m.gates[0].wg.weight.dtype == torch.float32 and m.compress_name == 'int8'


def test_overlap_degree_checks():
    from planmoe_amd.overlap import a2a_ffn_overlap_forward
    with pytest.raises(AssertionError):
        a2a_ffn_overlap_forward(torch.zeros(2, 8, 4), lambda t: t, 33, False, None, "no", "naive")
    with pytest.raises(AssertionError):
        a2a_ffn_overlap_forward(torch.zeros(2, 8, 4), lambda t: t, 3, False, None, "no", "naive")
    y = a2a_ffn_overlap_forward(torch.arange(64.0).view(2, 8, 4), lambda t: t * 2, 2, False, None, "no", "naive")
    assert torch.equal(y, torch.arange(64.0).view(2, 8, 4) * 2)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU's share of the path: --gpus N with N > 1 exits with a message that says
    so (before anything touches a device)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "--gpus 2 is not supported" in (r.stderr + r.stdout)
