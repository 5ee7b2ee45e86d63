"""Pins of the routing part of the CPU oracle: torch.topk / scatter_ / cumsum chains on
tie-free inputs, brute force, and the slot invariants."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import bf16_bits, np_raw, tie_free_scores, zipf_bias


@pytest.mark.parametrize("name,k,norm", [("route_t2_e2", 2, True), ("route_t2_e8", 2, True),
                                         ("route_t1_e64", 1, True), ("route_t3_e16_nonorm", 3, False),
                                         ("route_bf16_t2_e4", 2, True)])
def test_golden(torch_golden, name, k, norm):
    c = case(torch_golden, name)
    idx, loc, gates, counts = oracle.route_topk(c["scores"], k, norm)
    assert np.array_equal(idx, c["indices"])
    assert np.array_equal(loc, c["locations"])
    assert np.array_equal(np_raw(gates), np_raw(c["gates"]))
    assert np.array_equal(counts, c["counts"])
    l = oracle.gshard_loss(c["scores"], idx[0])
    tol = 1e-2 if c["scores"].dtype == np.uint16 else 1e-5
    assert abs(l - float(c["l_aux"][0])) <= tol * abs(l)


def brute_force(scores, k):
    """O(T*E) pure-Python slot assignment for tiny inputs."""
    T, E = scores.shape
    idx = np.zeros((k, T), np.int32)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-scores[t, e], e))
        for j in range(k):
            idx[j, t] = order[j]
    loc = np.zeros((k, T), np.int32)
    for j in range(k):
        for t in range(T):
            e = idx[j, t]
            n = sum(1 for jj in range(j) for tt in range(T) if idx[jj, tt] == e)
            n += sum(1 for tt in range(t) if idx[j, tt] == e)
            loc[j, t] = n
    return idx, loc


@pytest.mark.parametrize("T,E,k", [(1, 1, 1), (9, 3, 2), (40, 5, 3), (17, 4, 4)])
def test_brute_force(T, E, k):
    scores = tie_free_scores(T, E, k, seed=T * 31 + E).numpy()
    idx, loc, gates, counts = oracle.route_topk(scores, k)
    bi, bl = brute_force(scores, k)
    assert np.array_equal(idx, bi) and np.array_equal(loc, bl)
    for j in range(k):
        assert np.array_equal(counts[j], np.bincount(idx[j], minlength=E))


def test_invariants_skewed():
    """Zipf-skewed top-1 routing: slots per expert are 0..n-1 in token order, the drop count
    at capacity C is sum_e max(0, n_e - C)."""
    T, E = 4096, 64
    scores = tie_free_scores(T, E, 1, seed=11, bias=zipf_bias(E)).numpy()
    idx, loc, gates, counts = oracle.route_topk(scores, 1)
    C = oracle.capacity(T, E, 1, 1.0, 4)
    assert C == 64
    for e in range(E):
        sel = np.nonzero(idx[0] == e)[0]
        assert np.array_equal(loc[0][sel], np.arange(len(sel)))
    dropped = int((loc[0] >= C).sum())
    assert dropped == int(np.maximum(counts[0] - C, 0).sum()) and dropped > 0
    assert np.array_equal(gates[0], scores[np.arange(T), idx[0]])


def test_second_choices_follow_first_choices():
    T, E, k = 500, 8, 2
    scores = tie_free_scores(T, E, k, seed=5).numpy()
    idx, loc, gates, counts = oracle.route_topk(scores, k)
    for e in range(E):
        first = np.nonzero(idx[0] == e)[0]
        second = np.nonzero(idx[1] == e)[0]
        assert np.array_equal(loc[0][first], np.arange(len(first)))
        assert np.array_equal(loc[1][second], len(first) + np.arange(len(second)))
    s = gates[0] + gates[1]
    assert np.abs(s - 1).max() <= 2 ** -22
    raw = scores[np.arange(T), idx[0]]
    assert np.array_equal(gates[0], raw / np.maximum(raw + scores[np.arange(T), idx[1]], np.float32(2 ** -23)))


@pytest.mark.parametrize("T,E,k,cf,al,want", [(8192, 2, 2, 1.0, 4, 8192), (16384, 8, 2, 1.25, 4, 5120),
                                               (32768, 64, 1, 1.0, 4, 512), (65536, 16, 2, 1.0, 4, 8192),
                                               (10, 3, 2, 1.0, 1, 8), (10, 3, 2, 1.0, 4, 8),
                                               (7, 4, 1, 1.5, 4, 4), (100, 8, 2, 1.2, 8, 32)])
def test_capacity_closed_form(T, E, k, cf, al, want):
    assert oracle.capacity(T, E, k, cf, al) == want


def test_cumsum_sub_one_against_torch():
    g = torch.Generator().manual_seed(0)
    for T, E in ((1, 1), (5, 3), (1025, 8), (3000, 64)):
        m = (torch.rand(T, E, generator=g) < 0.4).to(torch.int32)
        want = (torch.cumsum(m, dim=0) - 1).numpy()
        assert np.array_equal(oracle.cumsum_sub_one(m.numpy()), want)


def test_softmax_and_logits_against_torch():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(50, 96, generator=g)
    w = torch.randn(7, 96, generator=g) / 96 ** 0.5
    lg = oracle.gate_logits(x.numpy(), w.numpy())
    assert np.allclose(lg, (x.double() @ w.double().t()).numpy(), rtol=1e-12, atol=1e-12)
    xb, wb = x.bfloat16(), w.bfloat16()
    lgb = oracle.gate_logits(bf16_bits(xb), bf16_bits(wb))
    assert np.allclose(lgb, (xb.double() @ wb.double().t()).numpy(), rtol=1e-12, atol=1e-12)
    sm = oracle.softmax(lg.astype(np.float32))
    assert np.allclose(sm, torch.softmax(torch.from_numpy(lg.astype(np.float32)), 1).numpy(), rtol=1e-6)


def _torch_bpr_locations(scores, k):
    """The reference's tensor algebra for batch-prioritised routing (fast_dispatch.py:135-138,
    142-168) with torch ops, fast_cumsum_sub_one spelled as cumsum - 1."""
    T, E = scores.shape
    topk_indices = torch.topk(scores, k, dim=1).indices
    indices_s = [x.view(-1) for x in topk_indices.chunk(k, dim=1)]
    masks_se = [torch.nn.functional.one_hot(x, num_classes=E).to(torch.int64) for x in indices_s]
    importance = -1 * scores.max(dim=1)[0]

    def compute_location(x):
        order = importance.argsort(dim=0, stable=True)
        sorted_x = x[order]
        sorted_cumsum = (torch.cumsum(sorted_x, dim=0) - 1) * sorted_x
        return sorted_cumsum[order.argsort(dim=0)]

    locations = [torch.sum(compute_location(masks_se[0]) * masks_se[0], dim=1)]
    acc_base = None
    for j in range(1, k):
        s = torch.sum(masks_se[j - 1], dim=0, keepdim=True)
        acc_base = s if acc_base is None else acc_base + s
        loc2 = compute_location(masks_se[j]) + acc_base
        locations.append(torch.sum(loc2 * masks_se[j], dim=1))
    return torch.stack(indices_s).numpy().astype(np.int32), torch.stack(locations).numpy().astype(np.int32)


@pytest.mark.parametrize("T,E,k", [(257, 8, 2), (1000, 16, 3), (64, 4, 1), (500, 5, 5)])
def test_route_locations_against_the_torch_chain(T, E, k):
    """orc_route_locations with the importance order against the reference's own op chain, and
    without an order against orc_route_topk."""
    scores = tie_free_scores(T, E, k, seed=T + E)
    idx, want = _torch_bpr_locations(scores, k)
    order = torch.argsort(-scores.max(dim=1)[0], stable=True).numpy().astype(np.int32)
    loc, counts = oracle.route_locations(idx, E, order)
    assert np.array_equal(loc, want)
    idx2, loc2, _, counts2 = oracle.route_topk(scores.numpy(), k)
    assert np.array_equal(idx2, idx)
    loc3, counts3 = oracle.route_locations(idx, E)
    assert np.array_equal(loc3, loc2) and np.array_equal(counts3, counts2) and np.array_equal(counts, counts2)
    # an order only permutes who gets which slot of an expert
    for j in range(k):
        for e in range(E):
            m = idx[j] == e
            assert sorted(loc[j][m]) == sorted(loc2[j][m])


def test_route_locations_ignores_out_of_range_indices():
    idx = np.array([[0, 5, -1, 1, 0, 7]], np.int32)
    loc, counts = oracle.route_locations(idx, 2)
    assert loc.tolist() == [[0, -1, -1, 0, 1, -1]] and counts.tolist() == [[2, 1]]
