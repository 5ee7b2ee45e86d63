"""GPU parity: routing (top-k, capacity slots, gates, GShard loss) and the capacity cumsum,
bit-exact against the CPU oracle through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import bf16_bits, np_raw, raw, random_scores, tie_free_scores, to_np, zipf_bias

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(scores, k, normalize=True):
    from planmoe_amd import ops
    r = ops.route_topk(scores.to(DEV), k, normalize_gate=normalize, want_counts=True)
    s_np = to_np(scores)
    idx, loc, gates, counts = oracle.route_topk(s_np, k, normalize)
    assert np.array_equal(r["indices"].cpu().numpy(), idx)
    assert np.array_equal(r["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(r["gates"]), np_raw(gates))
    assert np.array_equal(r["counts"].cpu().numpy(), counts)
    want = oracle.gshard_loss(s_np, idx[0])
    tol = 1e-2 if scores.dtype == torch.bfloat16 else 1e-5      # fp32 rtol 1e-5, bf16 rtol 1e-2
    assert abs(float(r["l_aux"]) - want) <= tol * abs(want)
    return r


@pytest.mark.parametrize("name,k,norm", [("route_t2_e2", 2, True), ("route_t2_e8", 2, True),
                                         ("route_t1_e64", 1, True), ("route_t3_e16_nonorm", 3, False)])
def test_golden_fixtures(torch_golden, name, k, norm):
    from planmoe_amd import ops
    c = case(torch_golden, name)
    r = ops.route_topk(torch.from_numpy(c["scores"]).to(DEV), k, normalize_gate=norm, want_counts=True)
    assert np.array_equal(r["indices"].cpu().numpy(), c["indices"])
    assert np.array_equal(r["locations"].cpu().numpy(), c["locations"])
    assert np.array_equal(raw(r["gates"]), np_raw(c["gates"]))
    assert np.array_equal(r["counts"].cpu().numpy(), c["counts"])
    assert abs(float(r["l_aux"]) - float(c["l_aux"][0])) <= 1e-5 * abs(float(c["l_aux"][0]))


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (7, 2, 2), (255, 8, 2), (256, 8, 2), (257, 8, 2), (1000, 64, 1),
                                   (5000, 100, 3), (3000, 16, 16), (4097, 3, 2), (2000, 300, 2)])
def test_against_oracle(T, E, k):
    _check(tie_free_scores(T, E, k, seed=T + E), k)


@pytest.mark.parametrize("T,E,k", [(600000, 8, 2), (400000, 128, 2), (300001, 64, 1)])
def test_many_tokens(T, E, k):
    """Token counts an order of magnitude above the configs (thousands of routing tiles / groups)."""
    _check(tie_free_scores(T, E, k, seed=T + E), k)


def test_cumsum_many_rows():
    from planmoe_amd import ops
    mask = (torch.rand(600001, 64, generator=torch.Generator().manual_seed(9)) < 0.2).to(torch.int32).to(DEV)
    got = ops.cumsum_sub_one(mask)
    assert torch.equal(got, torch.cumsum(mask, 0, dtype=torch.int32) - 1)


def test_without_gate_normalisation():
    _check(tie_free_scores(700, 8, 2, seed=3), 2, normalize=False)


def test_bf16_scores():
    # bf16 scores tie almost surely; oracle and kernel share the lower-index rule
    _check(random_scores(3000, 8, seed=4, dtype=torch.bfloat16), 2)


def test_tied_scores_pick_lower_index_like_the_oracle():
    s = torch.full((300, 8), 0.125)
    s[::3, 5] = 0.25
    _check(s, 2)


def test_config1_full_size():
    # 8192 tokens, 2 experts, top-2: every expert receives every token, nothing is dropped
    r = _check(tie_free_scores(8192, 2, 2, seed=0), 2)
    from planmoe_amd import ops
    assert ops.capacity(8192, 2, 2, 1.0, 4) == 8192
    assert int(r["locations"].max()) == 8191
    assert r["counts"].sum(0).tolist() == [8192, 8192]


def test_config2_full_size():
    _check(tie_free_scores(16384, 8, 2, seed=0), 2)


def test_config3_full_size_zipf_overflow():
    from planmoe_amd import ops
    T, E = 32768, 64
    r = _check(tie_free_scores(T, E, 1, seed=0, bias=zipf_bias(E)), 1)
    C = ops.capacity(T, E, 1, 1.0, 4)
    assert C == 512
    counts = r["counts"][0].cpu().numpy()
    dropped = int((r["locations"][0] >= C).sum())
    assert dropped == int(np.maximum(counts - C, 0).sum()) and dropped > T // 4


def test_config5_full_size():
    _check(tie_free_scores(65536, 16, 2, seed=0), 2)


def test_logits_input_matches_scores_input():
    """With input_is_logits the kernel's own softmax feeds the same routing: feed the scores it
    reports back through the oracle, and compare them with an fp32 softmax within rtol 1e-5."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(8)
    logits = torch.randn(5000, 8, generator=g) * 2
    bias = zipf_bias(8)
    r = ops.route_topk(logits.to(DEV), 2, is_logits=True, logit_bias=bias, want_scores=True, want_counts=True)
    scores = r["scores"].cpu()
    assert torch.allclose(scores, torch.softmax(logits + bias, 1), rtol=1e-5, atol=1e-8)
    idx, loc, gates, counts = oracle.route_topk(scores.numpy(), 2)
    assert np.array_equal(r["indices"].cpu().numpy(), idx)
    assert np.array_equal(r["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(r["gates"]), np_raw(gates))


def test_empty_batch():
    from planmoe_amd import ops
    r = ops.route_topk(torch.zeros(0, 8, device=DEV), 2, want_counts=True)
    assert r["indices"].shape == (2, 0) and int(r["counts"].sum()) == 0


@pytest.mark.parametrize("T,E", [(1, 1), (5, 3), (1000, 8), (1024, 2), (4097, 64), (777, 130), (32768, 64)])
def test_cumsum_sub_one(T, E):
    import planmoe_amd
    g = torch.Generator().manual_seed(T)
    m = (torch.rand(T, E, generator=g) < 0.3).to(torch.int64)
    out = planmoe_amd.fast_cumsum_sub_one(m.to(DEV))
    assert out.dtype == torch.int32
    assert np.array_equal(out.cpu().numpy(), oracle.cumsum_sub_one(m.numpy()))


def test_extract_critical_structure():
    import planmoe_amd
    scores = tie_free_scores(1000, 8, 2, seed=12)
    (E, idxs, locs, gates, C), l_aux = planmoe_amd.extract_critical(scores.to(DEV), 2, capacity_factor=1.25, alignment=4)
    assert E == 8 and C == oracle.capacity(1000, 8, 2, 1.25, 4) and len(idxs) == len(locs) == len(gates) == 2
    idx, loc, g, _ = oracle.route_topk(scores.numpy(), 2)
    for j in range(2):
        assert idxs[j].dtype == torch.int32 and locs[j].dtype == torch.int32 and gates[j].dtype == torch.float32
        assert np.array_equal(idxs[j].cpu().numpy(), idx[j]) and np.array_equal(locs[j].cpu().numpy(), loc[j])
        assert np.array_equal(raw(gates[j]), np_raw(g[j]))
    assert abs(float(l_aux) - oracle.gshard_loss(scores.numpy(), idx[0])) < 1e-5
    # data-dependent capacity (capacity_factor = 0): max location + 1, aligned
    (_, _, _, _, C0), _ = planmoe_amd.extract_critical(scores.to(DEV), 2, capacity_factor=0, alignment=4)
    assert C0 == (int(loc.max()) + 1 + 3) // 4 * 4
    # capacity_factor < 0 (fast_dispatch.py:185-186): the data-dependent capacity, capped at
    # top_k * int(-cf * ceil(T / E)); both sides of the cap
    need = int(loc.max()) + 1
    per_expert = (1000 + 7) // 8
    for cf in (-0.25, -1.0, -64.0):
        (_, _, _, _, Cn), _ = planmoe_amd.extract_critical(scores.to(DEV), 2, capacity_factor=cf, alignment=4)
        assert Cn == (min(need, 2 * int(-cf * per_expert)) + 3) // 4 * 4
    assert 2 * int(0.25 * per_expert) < need < 2 * int(64.0 * per_expert)
    # custom loss callables see (scores, top-k ids [T, k])
    (_, _, _, _, _), l2 = planmoe_amd.extract_critical(scores.to(DEV), 2, loss_fn=lambda s, ids: ids.float().mean())
    assert abs(float(l2) - float(np.stack(list(idx), 1).mean())) < 1e-5


def _torch_routing_reference(scores64, idx, normalize, T, E):
    """gates and GShard loss from the scores with torch ops in float64 (indices fixed)."""
    idx_t = torch.from_numpy(idx.astype(np.int64))
    raw_g = [scores64.gather(1, idx_t[j][:, None])[:, 0] for j in range(idx.shape[0])]
    if normalize and len(raw_g) > 1:
        denom = torch.clamp(sum(raw_g), min=torch.finfo(torch.float32).eps)
        raw_g = [g / denom for g in raw_g]
    mask = torch.zeros(T, E, dtype=torch.float64)
    mask.scatter_(1, idx_t[0][:, None], E / T)
    l_aux = torch.sum(scores64.sum(0) * mask.sum(0)) / T
    return raw_g, l_aux


@pytest.mark.parametrize("T,E,k,normalize", [(500, 8, 2, True), (300, 16, 3, False), (257, 64, 1, True)])
def test_routing_gradients_match_autograd(T, E, k, normalize):
    """extract_critical's gates and l_aux carry gradients into the scores: compared with
    torch autograd of the same algebra in float64 (rtol 1e-5)."""
    import planmoe_amd
    scores = tie_free_scores(T, E, k, seed=T)
    s_dev = scores.to(DEV).requires_grad_()
    (_, idxs, locs, gates, C), l_aux = planmoe_amd.extract_critical(s_dev, k, normalize_gate=normalize)
    g = torch.Generator().manual_seed(1)
    w = [torch.randn(T, generator=g) for _ in range(k)]
    loss = sum((gates[j] * w[j].to(DEV)).sum() for j in range(k)) + 3.0 * l_aux
    loss.backward()
    s64 = scores.double().requires_grad_()
    idx = np.stack([i.cpu().numpy() for i in idxs])
    ref_g, ref_l = _torch_routing_reference(s64, idx, normalize, T, E)
    ref = sum((ref_g[j] * w[j].double()).sum() for j in range(k)) + 3.0 * ref_l
    ref.backward()
    assert torch.allclose(s_dev.grad.cpu().double(), s64.grad, rtol=1e-5, atol=1e-7)


def test_routing_gradients_through_the_fused_softmax():
    from planmoe_amd.fast_dispatch import route
    T, E, k = 400, 8, 2
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(T, E, generator=g)
    l_dev = logits.to(DEV).requires_grad_()
    gates, l_aux, indices, locations, counts = route(l_dev, k, True, True, True)
    w = torch.randn(k, T, generator=g)
    ((gates * w.to(DEV)).sum() + 2.0 * l_aux).backward()
    l64 = logits.double().requires_grad_()
    s64 = torch.softmax(l64, 1)
    ref_g, ref_l = _torch_routing_reference(s64, indices.cpu().numpy(), True, T, E)
    (sum((ref_g[j] * w[j].double()).sum() for j in range(k)) + 2.0 * ref_l).backward()
    assert torch.allclose(l_dev.grad.cpu().double(), l64.grad, rtol=1e-4, atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("T,E,k,with_order", [(1000, 8, 2, True), (1000, 8, 2, False), (4097, 64, 1, True),
                                              (300, 100, 4, True), (77, 3, 3, True), (20000, 16, 2, True)])
def test_route_locations(T, E, k, with_order):
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + E + k)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)], dim=1).to(torch.int32).contiguous()
    idx[0, ::17] = -1                                   # dead pairs take no slot
    idx[k - 1, 5::31] = E + 3
    order = torch.randperm(T, generator=g).to(torch.int32) if with_order else None
    loc, counts = ops.route_locations(idx.to(DEV), E, None if order is None else order.to(DEV), want_counts=True)
    want, wc = oracle.route_locations(idx.numpy(), E, None if order is None else order.numpy())
    assert np.array_equal(loc.cpu().numpy(), want)
    assert np.array_equal(counts.cpu().numpy(), wc)


@pytest.mark.gpu
@pytest.mark.parametrize("T,E,k", [(2048, 8, 2), (555, 16, 1), (16384, 8, 2)])
def test_batch_prioritized_routing(T, E, k):
    """extract_critical(batch_prioritized_routing=True): tokens with the larger top score get the
    lower slots; same indices, gates and loss as without."""
    import planmoe_amd as moe
    scores = tie_free_scores(T, E, k, seed=T)
    sd = scores.to(DEV)
    (n, idx_s, loc_s, gates_s, cap), l = moe.extract_critical(sd, k, capacity_factor=1.0, batch_prioritized_routing=True)
    (_, idx0, loc0, gates0, cap0), l0 = moe.extract_critical(sd, k, capacity_factor=1.0)
    assert cap == cap0 and float(l) == float(l0)
    for a, b in zip(idx_s, idx0):
        assert torch.equal(a, b)
    for a, b in zip(gates_s, gates0):
        assert torch.equal(a, b)
    idx = torch.stack(idx_s).cpu().numpy()
    order = torch.argsort(-scores.max(dim=1)[0], stable=True).numpy().astype(np.int32)
    want, _ = oracle.route_locations(idx, E, order)
    got = torch.stack(loc_s).cpu().numpy()
    assert np.array_equal(got, want)
    # dropped tokens (location >= capacity) of an expert are its least important ones
    top = scores.max(dim=1)[0].numpy()
    for e in range(E):
        m = idx[0] == e
        kept, dropped = top[m & (got[0] < cap)], top[m & (got[0] >= cap)]
        if len(kept) and len(dropped):
            assert kept.min() >= dropped.max()
