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
