"""Pins of the dispatch / combine / gate-gradient part of the CPU oracle: torch indexing
closed forms, the dense GShard einsum, round-trip and autograd identities."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import tie_free_scores


@pytest.mark.parametrize("name", ["sparse_a", "sparse_b"])
def test_golden(torch_golden, name):
    c = case(torch_golden, name)
    E, C = int(c["E"][0]), int(c["C"][0])
    k, T = c["idx"].shape
    d = oracle.encode(c["x"], list(c["idx"]), list(c["loc"]), list(c["gates"]), E, C)
    assert np.array_equal(d.view(np.int32), c["dispatched"].view(np.int32))
    y = oracle.decode(c["eo"], list(c["idx"]), list(c["loc"]), list(c["gates"]), T, C)
    assert np.array_equal(y.view(np.int32), c["combined"].view(np.int32))
    for j in range(k):
        gg = oracle.bwd_gate(c["idx"][j], c["loc"][j], c["x"].astype(np.float64), c["eo"].astype(np.float64), C)
        assert np.allclose(gg, c["grad_gates"][j], rtol=1e-12, atol=1e-12)


def _routing(T, E, k, cf, seed):
    scores = tie_free_scores(T, E, k, seed).numpy()
    idx, loc, gates, _ = oracle.route_topk(scores, k)
    return idx, loc, gates, oracle.capacity(T, E, k, cf, 1)


def test_dense_gshard_einsum_equivalence():
    """dispatch == einsum('sec,sm->ecm') and combine == einsum('sec,ecm->sm') with the dense
    combine-weights tensor of the GShard formulation."""
    T, M, E, k = 24, 6, 4, 2
    idx, loc, gates, C = _routing(T, E, k, 1.0, 3)
    x = np.random.default_rng(0).standard_normal((T, M))
    eo = np.random.default_rng(1).standard_normal((E * C, M))
    cw = np.zeros((T, E, C))
    for j in range(k):
        for t in range(T):
            if loc[j, t] < C:
                cw[t, idx[j, t], loc[j, t]] = gates[j, t]
    g64 = [g.astype(np.float64) for g in gates]
    d = oracle.encode(x, list(idx), list(loc), g64, E, C)
    assert np.allclose(d.reshape(E, C, M), np.einsum("sec,sm->ecm", cw, x), rtol=1e-13, atol=1e-13)
    y = oracle.decode(eo, list(idx), list(loc), g64, T, C)
    assert np.allclose(y, np.einsum("sec,ecm->sm", cw, eo.reshape(E, C, M)), rtol=1e-13, atol=1e-13)


def test_round_trip_and_drops():
    T, M, E, k = 200, 16, 4, 2
    idx, loc, gates, C = _routing(T, E, k, 0.5, 9)        # tight capacity: tokens are dropped
    x = np.random.default_rng(2).standard_normal((T, M)).astype(np.float32)
    d = oracle.encode(x, list(idx), list(loc), None, E, C)
    y = oracle.decode(d, list(idx), list(loc), list(gates), T, C)
    keep = (loc < C)
    w = (keep * gates).sum(0)
    assert np.allclose(y, x * w[:, None], rtol=1e-6, atol=1e-6)
    assert (~keep).any()
    used = np.zeros(E * C, bool)
    for j in range(k):
        used[(idx[j] * C + loc[j])[keep[j]]] = True
    assert (d[~used] == 0).all()


def test_backward_identities_with_autograd():
    """GatingEncoder.backward == combine with the same gates; GatingDecoder.backward ==
    dispatch; gate gradients == <dOut, expert_out[slot]> -- checked against torch autograd
    of an index-based restatement in float64."""
    T, M, E, k = 30, 8, 4, 2
    idx, loc, gates, C = _routing(T, E, k, 0.75, 4)
    rng = np.random.default_rng(5)
    x = torch.tensor(rng.standard_normal((T, M)), requires_grad=True)
    eo = torch.tensor(rng.standard_normal((E * C, M)), requires_grad=True)
    g = torch.tensor(gates.astype(np.float64), requires_grad=True)
    keep = torch.from_numpy(loc < C)
    slot = torch.from_numpy((idx.astype(np.int64) * C + loc))

    def enc(x_, g_):
        out = torch.zeros(E * C, M, dtype=torch.float64)
        for j in range(k):
            out = out.index_put((slot[j][keep[j]],), g_[j][keep[j], None] * x_[keep[j]], accumulate=True)
        return out

    def dec(eo_, g_):
        y = torch.zeros(T, M, dtype=torch.float64)
        for j in range(k):
            term = torch.zeros(T, M, dtype=torch.float64)
            term[keep[j]] = g_[j][keep[j], None] * eo_[slot[j][keep[j]]]
            y = y + term
        return y

    dY = torch.tensor(rng.standard_normal((E * C, M)))
    dx, dg = torch.autograd.grad(enc(x, g), (x, g), dY)
    g64 = [a.astype(np.float64) for a in gates]
    assert np.allclose(oracle.decode(dY.numpy(), list(idx), list(loc), g64, T, C), dx.numpy(), atol=1e-12)
    for j in range(k):
        assert np.allclose(oracle.bwd_gate(idx[j], loc[j], x.detach().numpy(), dY.numpy(), C), dg[j].numpy(), atol=1e-12)

    dOut = torch.tensor(rng.standard_normal((T, M)))
    deo, dg2 = torch.autograd.grad(dec(eo, g), (eo, g), dOut)
    assert np.allclose(oracle.encode(dOut.numpy(), list(idx), list(loc), g64, E, C), deo.numpy(), atol=1e-12)
    for j in range(k):
        assert np.allclose(oracle.bwd_gate(idx[j], loc[j], dOut.numpy(), eo.detach().numpy(), C), dg2[j].numpy(), atol=1e-12)


def test_negative_index_is_dropped():
    x = np.ones((3, 4), np.float32)
    idx = np.array([0, -1, 1], np.int32)
    loc = np.array([0, 0, 5], np.int32)
    d = oracle.encode(x, [idx], [loc], None, 2, 2)
    assert d[0].sum() == 4 and d[1:].sum() == 0
    y = oracle.gather(np.ones(3, np.float32), idx, loc, d, 3, 2)
    assert y[0].sum() == 4 and y[1:].sum() == 0
