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
    # host tensors: torch.cumsum - 1, as jit_kernels/gating.py:13-15 of the reference
    m = torch.tensor([[1, 0], [0, 1], [1, 1]], dtype=torch.int32)
    assert planmoe_amd.fast_cumsum_sub_one(m).tolist() == [[0, -1], [0, 0], [1, 1]]


def test_cpu_tensors_fail_loudly_in_the_gpu_entry_points():
    """The kernels' wrappers take GPU tensors only; host tensors have a route of their own (next
    test) that is entered by an explicit branch, never as a fall-back."""
    with pytest.raises(PlanMoEError):
        ops.int8_compress(torch.rand(4, 8))
    with pytest.raises(PlanMoEError):
        ops.route_topk(torch.rand(4, 2), 1)
    with pytest.raises(PlanMoEError):
        ops.dispatch_fwd(torch.rand(4, 8), [torch.zeros(4, dtype=torch.int32)], [torch.zeros(4, dtype=torch.int32)], None, 2, 4)


@pytest.mark.parametrize("dtype,k,cf,bpr,postscore", [(torch.float32, 2, 1.0, False, True), (torch.float32, 2, 0.5, False, False),
                                                      (torch.float64, 1, 1.0, False, True), (torch.float32, 3, 2.0, True, True),
                                                      (torch.float32, 2, 0.0, False, True), (torch.float32, 2, -0.5, False, False)])
def test_host_tensors_take_the_reference_cpu_route(dtype, k, cf, bpr, postscore):
    """fast_dispatch.py:105-113: host tensors go to invoke_cpu_fp32 / fp64 and torch's routing ops.
    Checked against the oracle (routing, dispatch, combine) and autograd identities."""
    import numpy as np
    import oracle
    from helpers import tie_free_scores
    T, E, M = 96, 4, 24
    scores = tie_free_scores(T, E, k, seed=3).to(dtype).requires_grad_(True)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(1)).to(dtype).requires_grad_(True)
    crit, l_loss = planmoe_amd.extract_critical(scores, k, capacity_factor=cf, batch_prioritized_routing=bpr)
    experts, idx_s, loc_s, gates_s, cap = crit
    sc = scores.detach().float().numpy()
    idx, loc, gates, _ = oracle.route_topk(sc, k)
    assert np.array_equal(torch.stack(idx_s).numpy(), idx)
    if not bpr:
        assert np.array_equal(torch.stack(loc_s).numpy(), loc)
        if cf > 0:
            assert cap == oracle.capacity(T, E, k, cf, 1)
    else:
        order = np.argsort(-sc.max(axis=1), kind="stable").astype(np.int32)
        want, _ = oracle.route_locations(idx, E, order)
        assert np.array_equal(torch.stack(loc_s).numpy(), want)
    assert torch.allclose(torch.stack(gates_s).detach().float(), torch.from_numpy(gates.astype(np.float32)), rtol=1e-5)
    assert abs(float(l_loss) - oracle.gshard_loss(sc, idx[0])) < 1e-5
    y = planmoe_amd.fast_encode(x, crit, is_postscore=postscore)
    assert y.shape == (E, cap, M) and y.dtype == dtype and not y.is_cuda
    g_in = None if postscore else [g.detach().float().numpy() for g in gates_s]
    locs_np = [l.numpy() for l in loc_s]
    want = oracle.encode(x.detach().float().numpy(), list(idx), locs_np, g_in, E, cap)
    assert torch.allclose(y.detach().float().reshape(-1, M), torch.from_numpy(want), rtol=1e-6, atol=1e-6)
    out = planmoe_amd.fast_decode(y, crit, is_postscore=postscore)
    g_out = [g.detach().float().numpy() for g in gates_s] if postscore else None
    want_out = oracle.decode(want, list(idx), locs_np, g_out, T, cap)
    assert torch.allclose(out.detach().float(), torch.from_numpy(want_out), rtol=1e-5, atol=1e-6)
    (out.square().sum() + l_loss).backward()
    assert x.grad is not None and scores.grad is not None and bool(torch.isfinite(x.grad).all())
    # dropped tokens get no gradient through the data path
    dropped = torch.stack([l >= cap for l in loc_s]).all(0)
    assert bool((x.grad[dropped] == 0).all())


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
