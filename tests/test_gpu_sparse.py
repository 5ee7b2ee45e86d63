"""GPU parity: dispatch / combine / gate-gradient kernels, bit-exact against the CPU oracle
for data movement and products, within tolerance for the gate-gradient dot products."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import raw, tie_free_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _routing(T, E, k, cf, seed, alignment=4):
    scores = tie_free_scores(T, E, k, seed).numpy()
    idx, loc, gates, _ = oracle.route_topk(scores, k)
    return idx, loc, gates, oracle.capacity(T, E, k, cf, alignment)


def _dev(planes):
    return [torch.from_numpy(np.ascontiguousarray(p)).to(DEV) for p in planes]


def _oracle_io(x, dtype):
    """The reference dispatcher computes in fp32 and casts back (fast_dispatch.py:91-93,121-131)."""
    return x.float().numpy()


@pytest.mark.parametrize("name", ["sparse_a", "sparse_b"])
def test_golden_fixtures(torch_golden, name):
    from planmoe_amd import ops
    c = case(torch_golden, name)
    E, C = int(c["E"][0]), int(c["C"][0])
    k, T = c["idx"].shape
    i, l, g = _dev(c["idx"]), _dev(c["loc"]), _dev(c["gates"])
    d = ops.dispatch_fwd(torch.from_numpy(c["x"]).to(DEV), i, l, g, E, C)
    assert np.array_equal(raw(d), c["dispatched"].view(np.int32))
    y = ops.combine_fwd(torch.from_numpy(c["eo"]).to(DEV), i, l, g, T, C)
    assert np.array_equal(raw(y), c["combined"].view(np.int32))
    gg = ops.bwd_gate(torch.from_numpy(c["x"]).to(DEV), torch.from_numpy(c["eo"]).to(DEV), i, l, C)
    assert np.allclose(gg.cpu().numpy(), c["grad_gates"], rtol=1e-5, atol=1e-5)   # fp32 rtol 1e-5


@pytest.mark.parametrize("T,M,E,k,cf,dtype", [
    (37, 24, 4, 2, 1.0, torch.float32), (37, 23, 4, 2, 1.0, torch.float32), (513, 256, 8, 2, 0.5, torch.float32),
    (513, 4096, 8, 2, 1.25, torch.bfloat16), (300, 1024, 16, 3, 1.0, torch.bfloat16),
    (100, 130, 4, 1, 1.0, torch.bfloat16), (64, 2048, 2, 2, 1.0, torch.float16), (1, 8, 1, 1, 1.0, torch.float32),
    (200, 9000, 4, 2, 1.0, torch.bfloat16)])
def test_dispatch_and_combine_bit_exact(T, M, E, k, cf, dtype):
    from planmoe_amd import ops
    idx, loc, gates, C = _routing(T, E, k, cf, seed=T + M)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, M, generator=g).to(dtype)
    eo = torch.randn(E * C, M, generator=g).to(dtype)
    i, l, gt = _dev(idx), _dev(loc), _dev(gates)
    for with_gates in (False, True):
        gl = list(gates) if with_gates else None
        want = torch.from_numpy(oracle.encode(x.float().numpy(), list(idx), list(loc), gl, E, C)).to(dtype)
        got = ops.dispatch_fwd(x.to(DEV), i, l, gt if with_gates else None, E, C)
        assert np.array_equal(raw(got), raw(want))
        wantc = torch.from_numpy(oracle.decode(eo.float().numpy(), list(idx), list(loc), gl, T, C)).to(dtype)
        gotc = ops.combine_fwd(eo.to(DEV), i, l, gt if with_gates else None, T, C)
        assert np.array_equal(raw(gotc), raw(wantc))


@pytest.mark.parametrize("T,M,E,k,dtype,rtol", [(300, 512, 8, 2, torch.float32, 1e-5), (300, 4096, 8, 2, torch.bfloat16, 1e-2),
                                                (50, 77, 4, 3, torch.float32, 1e-5), (40, 64, 16, 6, torch.float32, 1e-5)])
def test_bwd_gate(T, M, E, k, dtype, rtol):
    """fp64 restatement as the reference value; atol scaled by sum |terms| because the dot
    product cancels (the oracle's sequential fp32 sum is itself only that accurate)."""
    from planmoe_amd import ops
    idx, loc, gates, C = _routing(T, E, k, 0.75, seed=T)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, M, generator=g).to(dtype)
    d = torch.randn(E * C, M, generator=g).to(dtype)
    got = ops.bwd_gate(x.to(DEV), d.to(DEV), _dev(idx), _dev(loc), C).cpu().numpy()
    xd, dd = x.double().numpy(), d.double().numpy()
    for j in range(k):
        want = oracle.bwd_gate(idx[j], loc[j], xd, dd, C)
        mag = oracle.bwd_gate(idx[j], loc[j], np.abs(xd), np.abs(dd), C)
        assert (np.abs(got[j] - want) <= rtol * np.abs(want) + 1e-6 * mag).all()
        assert (got[j][loc[j] >= C] == 0).all()
        if dtype == torch.float32:          # and against the oracle's own sequential fp32 sum
            seq = oracle.bwd_gate(idx[j], loc[j], x.numpy(), d.numpy(), C)
            assert (np.abs(got[j] - seq) <= 1e-5 * np.abs(seq) + 2e-6 * mag).all()


def test_dropped_and_negative_indices():
    from planmoe_amd import ops
    x = torch.ones(3, 8)
    idx = [torch.tensor([0, -1, 1], dtype=torch.int32, device=DEV)]
    loc = [torch.tensor([0, 0, 5], dtype=torch.int32, device=DEV)]
    d = ops.dispatch_fwd(x.to(DEV), idx, loc, None, 2, 2).cpu()
    assert d[0].sum() == 8 and d[1:].abs().sum() == 0
    y = ops.combine_fwd(d.to(DEV), idx, loc, None, 3, 2).cpu()
    assert y[0].sum() == 8 and y[1:].abs().sum() == 0


def test_negative_zero_becomes_positive_zero_like_the_reference_accumulation():
    from planmoe_amd import ops
    x = torch.tensor([[-0.0, 1.0, -0.0, 2.0]])
    idx = [torch.zeros(1, dtype=torch.int32, device=DEV)]
    loc = [torch.zeros(1, dtype=torch.int32, device=DEV)]
    d = ops.dispatch_fwd(x.to(DEV), idx, loc, None, 1, 1).cpu()
    want = oracle.encode(x.numpy(), [np.zeros(1, np.int32)], [np.zeros(1, np.int32)], None, 1, 1)
    assert np.array_equal(raw(d), want.view(np.int32))
    assert not torch.signbit(d).any()


def test_many_choice_planes():
    """k = E = 80 > 64 lanes: the plane loop takes several rounds."""
    from planmoe_amd import ops
    T, M, E = 20, 16, 80
    idx, loc, gates, C = _routing(T, E, E, 1.0, seed=1, alignment=1)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(0))
    got = ops.dispatch_fwd(x.to(DEV), _dev(idx), _dev(loc), _dev(gates), E, C)
    want = oracle.encode(x.numpy(), list(idx), list(loc), list(gates), E, C)
    assert np.array_equal(raw(got), want.view(np.int32))
    y = ops.combine_fwd(got, _dev(idx), _dev(loc), _dev(gates), T, C)
    wy = oracle.decode(want, list(idx), list(loc), list(gates), T, C)
    assert np.array_equal(raw(y), wy.view(np.int32))


def test_config1_full_size_round_trip_fp32():
    """8192 x 2048 fp32, 2 experts top-2: decode(encode(x)) == x * sum of kept gates, and the
    dispatched buffer is exactly two copies of x (no drops, 100 % full)."""
    from planmoe_amd import ops
    T, M, E, k = 8192, 2048, 2, 2
    idx, loc, gates, C = _routing(T, E, k, 1.0, seed=0)
    assert C == 8192
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(0))
    i, l, g = _dev(idx), _dev(loc), _dev(gates)
    d = ops.dispatch_fwd(x.to(DEV), i, l, None, E, C)
    y = ops.combine_fwd(d, i, l, g, T, C).cpu()
    want = oracle.decode(oracle.encode(x.numpy(), list(idx), list(loc), None, E, C), list(idx), list(loc), list(gates), T, C)
    assert np.array_equal(raw(y), want.view(np.int32))
    d = d.cpu().view(E, C, M)
    for e in range(E):
        j = np.where(idx == e)        # plane / token of every row of expert e
        assert torch.equal(d[e][torch.from_numpy(loc[j])], x[torch.from_numpy(j[1])] + 0.0)


def test_config2_full_size_bf16_against_oracle():
    from planmoe_amd import ops
    T, M, E, k = 16384, 4096, 8, 2
    idx, loc, gates, C = _routing(T, E, k, 1.25, seed=0)
    assert C == 5120
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, M, generator=g).bfloat16()
    i, l, gt = _dev(idx), _dev(loc), _dev(gates)
    d = ops.dispatch_fwd(x.to(DEV), i, l, None, E, C)
    want = torch.from_numpy(oracle.encode(x.float().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
    assert np.array_equal(raw(d), raw(want))
    y = ops.combine_fwd(d, i, l, gt, T, C)
    wy = torch.from_numpy(oracle.decode(want.float().numpy(), list(idx), list(loc), list(gates), T, C)).bfloat16()
    assert np.array_equal(raw(y), raw(wy))


def test_buffers_beyond_two_to_the_31_elements():
    """600 000 tokens x 4096 bf16 (2.46 G elements, 4.9 GB per buffer): row addresses need 64 bits in
    every kernel of the path.  Checked through what holds at any size: dispatch then combine gives
    every kept token row back and zero rows for the dropped ones; the fused int8 kernels equal their
    two stages; the forward chain equals routing + the fused dispatch."""
    from planmoe_amd import ops
    T, M, E, k = 600000, 4096, 8, 1
    C = ops.capacity(T, E, k, 1.0, 4)
    g = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn(T, M, generator=g, device=DEV, dtype=torch.float32).bfloat16()
    wg = (torch.randn(E, M, generator=g, device=DEV) * M ** -0.5).bfloat16()
    r = ops.gate_route(x, wg, k)
    idx, loc = list(r["indices"]), list(r["locations"])
    kept = (loc[0] >= 0) & (loc[0] < C)
    assert 0 < int(kept.sum()) < T                                   # some tokens are dropped
    d = ops.dispatch_fwd(x, idx, loc, None, E, C)
    assert d.numel() > 2 ** 31
    slot = idx[0].long() * C + loc[0].long()
    last = int(torch.nonzero(kept)[-1])
    assert torch.equal(d[slot[last]], x[last])                       # the highest token row, the slot it went to
    y = ops.combine_fwd(d, idx, loc, None, T, C)
    assert torch.equal(y[kept].view(torch.int16), (x[kept] + 0.0).view(torch.int16))
    assert not y[~kept].any()
    del y
    codes, bias, scale = ops.dispatch_int8(x, idx, loc, None, E, C)
    c2, b2, s2 = ops.int8_compress(d)
    assert torch.equal(codes.view(-1), c2.view(-1))
    assert torch.equal(bias.view(torch.int16).view(-1), b2.view(torch.int16).view(-1))
    assert torch.equal(scale.view(torch.int16).view(-1), s2.view(torch.int16).view(-1))
    del c2, b2, s2
    dec = ops.int8_decompress(codes, bias, scale)
    y8 = ops.combine_int8(codes, bias, scale, idx, loc, list(r["gates"]), T, C)
    y2 = ops.combine_fwd(dec, idx, loc, list(r["gates"]), T, C)
    assert torch.equal(y8.view(torch.int16), y2.view(torch.int16))
    del dec, y8, y2
    # backward pieces: bwd_gate on sampled tokens against a dot product, the fused backward of
    # fast_decode against its stages (gated dispatch + int8, bwd_gate)
    gates = [t.float() for t in r["gates"]]
    gg = ops.bwd_gate(x, d, idx, loc, C)
    sample = torch.tensor([0, 1, T // 2, last, T - 1], device=DEV)
    want = (x[sample].float() * d[slot[sample].clamp(0, E * C - 1)].float()).sum(1) * kept[sample]
    assert torch.allclose(gg[0][sample], want, rtol=1e-2, atol=1e-2)
    c5, b5, s5, g5 = ops.combine_bwd_int8(x, d, idx, loc, gates, E, C)
    c6, b6, s6 = ops.dispatch_int8(x, idx, loc, gates, E, C)
    assert torch.equal(c5.view(-1), c6.view(-1)) and torch.equal(b5.view(torch.int16).view(-1), b6.view(torch.int16).view(-1))
    assert torch.allclose(g5[0], gg[0], rtol=1e-5, atol=1e-4)
    del c5, b5, s5, g5, c6, b6, s6, d
    f = ops.forward_int8(x, wg, k, C)
    assert torch.equal(f["indices"], r["indices"]) and torch.equal(f["locations"], r["locations"])
    assert torch.equal(f["codes"].view(-1), codes.view(-1))


def test_autograd_wiring_matches_the_reference_functions():
    """fast_encode / fast_decode backward: which gradients exist and what they equal."""
    import planmoe_amd
    T, M, E, k = 200, 64, 4, 2
    idx, loc, gates, C = _routing(T, E, k, 0.75, seed=21)
    crit = (E, _dev(idx), _dev(loc), [t.requires_grad_() for t in _dev(gates)], C)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, M, generator=g).to(DEV).requires_grad_()
    y = planmoe_amd.fast_encode(x, crit, is_postscore=True)
    assert y.shape == (E, C, M)
    dY = torch.randn(E, C, M, generator=g).to(DEV)
    y.backward(dY)
    g64 = None
    want_dx = oracle.decode(dY.cpu().view(E * C, M).numpy(), list(idx), list(loc), g64, T, C)
    assert np.array_equal(raw(x.grad), want_dx.view(np.int32))
    assert all(t.grad is None for t in crit[3])            # postscore: no gate gradient at encode

    eo = torch.randn(E, C, M, generator=g).to(DEV).requires_grad_()
    out = planmoe_amd.fast_decode(eo, crit, is_postscore=True)
    dOut = torch.randn(T, M, generator=g).to(DEV)
    out.backward(dOut)
    want_deo = oracle.encode(dOut.cpu().numpy(), list(idx), list(loc), list(gates), E, C)
    assert np.array_equal(raw(eo.grad.view(E * C, M)), want_deo.view(np.int32))
    for j in range(k):
        want = oracle.bwd_gate(idx[j], loc[j], dOut.cpu().double().numpy(), eo.detach().cpu().view(E * C, M).double().numpy(), C)
        assert np.allclose(crit[3][j].grad.cpu().numpy(), want, rtol=1e-5, atol=1e-4)


def test_prescore_mode_gates_at_encode():
    """is_postscore=False (fast_dispatch.py:40-45, 120-131): the gates scale the rows at encode,
    decode uses all-ones, and the gate gradient comes out of the encoder's backward."""
    import planmoe_amd
    T, M, E, k = 160, 48, 4, 2
    idx, loc, gates, C = _routing(T, E, k, 1.0, seed=9)
    gs = [t.requires_grad_() for t in _dev(gates)]
    crit = (E, _dev(idx), _dev(loc), gs, C)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, M, generator=g).to(DEV).requires_grad_()
    y = planmoe_amd.fast_encode(x, crit, is_postscore=False)
    want = oracle.encode(x.detach().cpu().numpy(), list(idx), list(loc), list(gates), E, C)
    assert np.array_equal(raw(y.view(E * C, M)), want.view(np.int32))
    dY = torch.randn(E, C, M, generator=g).to(DEV)
    y.backward(dY)
    want_dx = oracle.decode(dY.cpu().view(E * C, M).numpy(), list(idx), list(loc), list(gates), T, C)
    assert np.array_equal(raw(x.grad), want_dx.view(np.int32))
    for j in range(k):
        wg = oracle.bwd_gate(idx[j], loc[j], x.detach().cpu().double().numpy(), dY.cpu().view(E * C, M).double().numpy(), C)
        assert np.allclose(gs[j].grad.cpu().numpy(), wg, rtol=1e-5, atol=1e-4)
    out = planmoe_amd.fast_decode(y.detach(), crit, is_postscore=False)
    want_out = oracle.decode(want, list(idx), list(loc), None, T, C)
    assert np.array_equal(raw(out), want_out.view(np.int32))
