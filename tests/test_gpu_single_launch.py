"""planmoe_forward_int8_single (one launch, x read once) against the oracle and the two-launch chain."""
import numpy as np
import pytest
import torch

import oracle
from helpers import np_raw, raw

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("T,E,k,cf,fp32_gate", [(16384, 8, 2, 1.25, True), (16384, 8, 2, 1.25, False), (16000, 8, 2, 1.25, True),
                                                (4096, 8, 2, 1.0, True), (100, 4, 2, 1.0, True), (9000, 16, 3, 0.5, True),
                                                (12288, 8, 1, 1.0, True), (5000, 12, 4, 2.0, False), (1, 3, 2, 1.0, True)])
def test_single_launch_forward(T, E, k, cf, fp32_gate, M=4096):
    from planmoe_amd import ops
    print("case", T, E, k, cf, fp32_gate, M, flush=True)
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    C = ops.capacity(T, E, k, cf, 4)
    out = ops.forward_int8_single(x, wg, k, C, fp32_gate=fp32_gate, want_scores=True, want_counts=True, want_logits=True)
    torch.cuda.synchronize()
    assert int(out["gave_up"]) == 0
    scores = out["scores"].float().cpu().numpy() if fp32_gate else None
    if fp32_gate:
        idx, loc, gates, counts = oracle.route_topk(scores, k)
    else:
        from helpers import bf16_bits
        idx, loc, gates, counts = oracle.route_topk(bf16_bits(out["scores"]), k)
    assert np.array_equal(out["indices"].cpu().numpy(), idx)
    assert np.array_equal(out["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(out["gates"]), np_raw(gates))
    assert np.array_equal(out["counts"].cpu().numpy(), counts)
    ref = ops.forward_int8(x, wg, k, C, fp32_gate=fp32_gate, want_scores=True, want_logits=True)
    assert torch.allclose(out["logits"].float(), ref["logits"].float(), rtol=1e-2 if not fp32_gate else 1e-5, atol=1e-5)
    want = oracle.gshard_loss(out["scores"].float().cpu().numpy(), idx[0])
    assert abs(float(out["l_aux"]) - want) <= 1e-5 * abs(want)
    # codes, bias and scale against the oracle itself: its dispatch of the rows to the slots it
    # worked out, then its restatement of Int8Compressor::compress on the bf16 rows
    from helpers import bf16_bits
    d = torch.from_numpy(oracle.encode(x.float().cpu().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
    rc, rb, rs = oracle.int8_compress(bf16_bits(d))
    del d
    assert np.array_equal(out["codes"].cpu().numpy().reshape(-1), rc.reshape(-1))
    assert np.array_equal(bf16_bits(out["bias"]).reshape(-1), rb.reshape(-1))
    assert np.array_equal(bf16_bits(out["scale"]).reshape(-1), rs.reshape(-1))


@pytest.mark.parametrize("T,M,E,k,cf,fp32_gate", [(16384, 2048, 8, 2, 1.25, True), (9000, 2048, 16, 3, 0.5, False),
                                                  (16384, 1024, 8, 2, 1.25, True), (5000, 1024, 4, 1, 1.0, True),
                                                  (12000, 3072, 8, 2, 1.25, True), (100, 3072, 12, 4, 2.0, False),
                                                  (1, 2048, 3, 2, 1.0, True),
                                                  # rows that end inside a wave's last pass over the codes
                                                  (16384, 768, 8, 2, 1.25, True), (7000, 1280, 16, 2, 1.0, False),
                                                  (16000, 2560, 8, 2, 1.25, True), (9000, 3584, 6, 3, 1.0, True),
                                                  (3000, 256, 4, 2, 1.0, True), (12345, 1792, 8, 1, 1.5, False),
                                                  (500, 3840, 16, 4, 2.0, True), (16384, 512, 8, 2, 1.25, True),
                                                  # two work-groups per compute unit: short rows, up to 128 tokens per unit
                                                  (32768, 1024, 8, 2, 1.25, True), (30000, 1792, 8, 2, 1.0, False),
                                                  (20000, 1536, 8, 3, 1.25, True)])
def test_single_launch_forward_other_row_lengths(T, M, E, k, cf, fp32_gate):
    """The one-launch kernel at other row lengths (multiples of 256 values): the same checks against the oracle."""
    test_single_launch_forward(T, E, k, cf, fp32_gate, M)


def test_the_library_says_which_shapes_the_single_launch_takes():
    """planmoe_forward_int8_single_serves against what the entry point then does: it launches exactly the
    shapes the query admits and refuses the others with an error (nothing enqueued)."""
    from planmoe_amd import ops
    from planmoe_amd._lib import PlanMoEError
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    cases = [(64 * cus, 4096, 8, 2, True), (64 * cus + 1, 4096, 8, 2, False), (128 * cus, 1024, 8, 2, True),
             (128 * cus + 1, 1024, 8, 2, False), (100, 4352, 8, 2, False), (100, 1000, 8, 2, False),
             (100, 1024, 17, 2, False), (100, 1024, 16, 5, False), (100, 1024, 3, 5, True), (1, 256, 1, 1, True)]
    for T, M, E, k, want in cases:
        print("case", T, M, E, k, flush=True)
        x = torch.randn(T, M, device=DEV).bfloat16()
        wg = (torch.randn(E, M, device=DEV) * M ** -0.5).bfloat16()
        assert ops.forward_int8_single_serves(x, wg, k) == want
        C = ops.capacity(T, E, k, 1.0, 4)
        if want:
            out = ops.forward_int8_single(x, wg, k, C)
            ref = ops.forward_int8(x, wg, k, C)
            torch.cuda.synchronize()
            assert int(out["gave_up"]) == 0 and torch.equal(out["codes"], ref["codes"]) and torch.equal(out["locations"], ref["locations"])
        else:
            with pytest.raises(PlanMoEError):
                ops.forward_int8_single(x, wg, k, C)
    assert not ops.forward_int8_single_serves(torch.randn(64, 1024, device=DEV), torch.randn(8, 1024, device=DEV), 2)   # fp32 rows


def test_single_launch_gives_up_cleanly_when_told_to():
    """spin_limit = 1 with more than one group: some group finds the others not in yet, gives up,
    writes none of its rows and raises the flag; every work-group still exits.  What the groups that
    finished wrote is the whole result's; the tokens of the groups that gave up are marked dropped and
    the loss is NaN, so a partial result cannot pass for a whole one."""
    from planmoe_amd import ops
    T, M, E, k, C = 16384, 4096, 8, 2, 5120
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    whole = ops.forward_int8_single(x, wg, k, C, want_scores=True)
    torch.cuda.synchronize()
    assert int(whole["gave_up"]) == 0
    out = ops.forward_int8_single(x, wg, k, C, spin_limit=1)
    torch.cuda.synchronize()
    assert int(out["gave_up"]) in (0, 1)
    assert torch.equal(out["indices"], whole["indices"])          # routing is every group's own work
    assert np.array_equal(raw(out["gates"]), raw(whole["gates"]))
    if int(out["gave_up"]) == 0:
        assert torch.equal(out["locations"], whole["locations"]) and torch.equal(out["codes"], whole["codes"])
        return
    assert bool(torch.isnan(out["l_aux"]))
    loc, ref = out["locations"], whole["locations"]
    done = (loc == ref).all(0)                                    # tokens whose group went through
    # a token of a group that gave up is dropped in every plane ...
    assert bool((loc[:, ~done] == C).all())
    # ... and work-groups give up as a whole: runs of 64 tokens
    assert bool((done.view(-1, 64).all(1) | (~done).view(-1, 64).all(1)).all())
    # the rows of the groups that went through are where the whole result has them, with its codes
    idx = out["indices"].long()
    for j in range(k):
        keep = done & (loc[j] < C)
        rows = (idx[j] * C + loc[j].long())[keep]
        assert torch.equal(out["codes"][rows], whole["codes"][rows])
        assert np.array_equal(raw(out["scale"][rows]), raw(whole["scale"][rows]))


def test_send_side_runs_the_two_launches_when_the_one_launch_gave_up(monkeypatch):
    """overlap.forward_int8_send_side never hands out a partial result: with a launch that gives up
    (forced through spin_limit) it returns what planmoe_forward_int8 returns."""
    from planmoe_amd import ops, overlap
    T, M, E, k, C = 16384, 4096, 8, 2, 5120
    g = torch.Generator().manual_seed(12)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    real = ops.forward_int8_single
    seen = []

    def hurried(*a, **kw):
        out = real(*a, spin_limit=1, **kw)
        seen.append(int(out["gave_up"]))
        return out

    monkeypatch.setattr(ops, "forward_int8_single", hurried)
    monkeypatch.setattr(overlap, "FORWARD_SINGLE_LAUNCH", True)
    got = overlap.forward_int8_send_side(x, wg, k, C, True, True, want_counts=True)
    ref = ops.forward_int8(x, wg, k, C, want_counts=True)
    torch.cuda.synchronize()
    assert seen and "gave_up" not in got
    if seen[0]:
        for key in ("indices", "locations", "codes", "counts"):
            assert torch.equal(got[key], ref[key]), key
    assert not bool(torch.isnan(got["l_aux"]))
    assert int(got["counts"][0].sum()) == T
    # the deferred form: the flag comes back as a check to ask later
    checks = []
    part = overlap.forward_int8_send_side(x, wg, k, C, True, True, checks=checks)
    assert len(checks) == 1 and bool(checks[0]) == bool(seen[-1]) and "gave_up" not in part


def test_layer_runs_again_in_two_launches_when_the_one_launch_gave_up(monkeypatch):
    """moe_layer with a one-launch send side that is made to give up: the layer's output, loss and
    gradients are those of the layer on the two-launch send side."""
    import planmoe_amd
    from planmoe_amd import ops, overlap

    class Identity(torch.nn.Module):
        def update(self, ctx):
            self.dummy = torch.nn.Parameter(torch.zeros(1))

        def forward(self, x, ctx):
            return x

    T, M, E = 16384, 4096, 8
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'capacity_factor': 1.25, 'fp32_gate': True}, M,
                                  experts={'type': 'custom', 'module': Identity(), 'count_per_node': E},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV).to(torch.bfloat16)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(0)).bfloat16().to(DEV)

    def run():
        xi = x.clone().requires_grad_(True)
        y = layer(xi)
        (y.float().square().mean() + y.l_aux.float()).backward()
        torch.cuda.synchronize()
        return y.detach(), float(y.l_aux.detach()), xi.grad

    monkeypatch.setattr(overlap, "FORWARD_SINGLE_LAUNCH", False)
    y0, l0, g0 = run()
    monkeypatch.setattr(overlap, "FORWARD_SINGLE_LAUNCH", True)
    real = ops.forward_int8_single
    seen = []

    def hurried(*a, **kw):
        out = real(*a, spin_limit=1, **kw)
        seen.append(int(out["gave_up"]))
        return out

    monkeypatch.setattr(ops, "forward_int8_single", hurried)
    y1, l1, g1 = run()
    assert seen
    if seen[0]:
        assert torch.equal(y0, y1) and l0 == l1 and torch.equal(g0, g1)
    assert bool(torch.isfinite(y1.float()).all()) and l1 == l1


def test_single_launch_and_two_launch_calls_take_turns_on_one_workspace():
    """The one-launch kernel's tags are its workspace's launch counter: no other entry point may
    write that region.  One workspace, one-launch calls at 16384 tokens between two-launch calls at
    512 tokens and routing-only calls, fresh inputs every time, everything against the oracle."""
    from helpers import bf16_bits
    from planmoe_amd import ops
    M, E, k = 4096, 8, 2
    g = torch.Generator().manual_seed(21)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    for it in range(6):
        T = 16384
        x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
        C = ops.capacity(T, E, k, 1.25, 4)
        out = ops.forward_int8_single(x, wg, k, C, want_scores=True)
        torch.cuda.synchronize()
        assert int(out["gave_up"]) == 0
        idx, loc, gates, counts = oracle.route_topk(out["scores"].float().cpu().numpy(), k)
        assert np.array_equal(out["indices"].cpu().numpy(), idx), it
        assert np.array_equal(out["locations"].cpu().numpy(), loc), it
        if it in (0, 5):
            d = torch.from_numpy(oracle.encode(x.float().cpu().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
            rc, rb, rs = oracle.int8_compress(bf16_bits(d))
            assert np.array_equal(out["codes"].cpu().numpy().reshape(-1), rc.reshape(-1)), it
        else:
            c2, _, _ = ops.dispatch_int8(x, list(out["indices"]), list(out["locations"]), None, E, C)
            assert torch.equal(out["codes"], c2), it
        # the same workspace (ops keeps one per device and stream) through the other entry points
        for Ts in (512, 448 + 64 * it):
            xs = torch.randn(Ts, M, generator=g).bfloat16().to(DEV)
            Cs = ops.capacity(Ts, E, k, 1.25, 4)
            small = ops.forward_int8(xs, wg, k, Cs, want_scores=True)
            si, sl, _, _ = oracle.route_topk(small["scores"].float().cpu().numpy(), k)
            assert np.array_equal(small["indices"].cpu().numpy(), si) and np.array_equal(small["locations"].cpu().numpy(), sl)
            ops.gate_route(xs, wg, k)


def test_single_launch_in_a_graph_replayed_with_fresh_inputs():
    """The captured launch carries the same arguments on every replay; the words the work-groups
    publish must still be told apart from those of the replay before (the workspace's launch counter
    does that).  Replays with fresh inputs, eager work between them, each against the eager result."""
    from planmoe_amd import ops
    T, M, E, k = 8192, 4096, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    plan = ops.ForwardInt8Plan(x, wg, k, C, single=True)
    plan.run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.run()
    # replays and eager calls take turns on the plan's one workspace: every launch must tell its own
    # published words from those of the launch before, whichever kind that was (tags that mixed a
    # per-call number into the launch counter once repeated here and let stale histograms through)
    for it in range(8):
        x.copy_(torch.randn(T, M, generator=g).bfloat16())
        if it % 3 == 2:
            plan.run()
        else:
            graph.replay()
        torch.cuda.synchronize()
        got = {key: v.clone() for key, v in plan.out.items() if v is not None}
        assert int(plan.gave_up) == 0
        want = ops.forward_int8_single(x, wg, k, C)
        ref = ops.forward_int8(x, wg, k, C)                      # the two-launch chain shares nothing with it
        for key in ("indices", "locations", "gates", "codes", "bias", "scale", "l_aux"):
            a, b = got[key], want[key]
            assert torch.equal(a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)), (it, key)
        same = (got["indices"] == ref["indices"]).all(0)
        assert float(same.float().mean()) > 0.99                 # (the two gate GEMMs sum in another order)
        if bool(same.all()):
            assert torch.equal(got["locations"], ref["locations"]) and torch.equal(got["codes"].view(-1), ref["codes"].view(-1))


def test_moe_layer_with_the_single_launch_send_side():
    """moe_layer (int8 compressor, identity experts) with overlap.FORWARD_SINGLE_LAUNCH: forward and
    backward against the same layer on the two-launch send side.  The two gate GEMMs add their
    partial sums in another order, so a token within an ulp of a tie may go elsewhere: all but a
    sliver of the rows must agree to the bit."""
    import planmoe_amd
    from planmoe_amd import overlap

    class Identity(torch.nn.Module):
        def update(self, ctx):
            self.dummy = torch.nn.Parameter(torch.zeros(1))

        def forward(self, x, ctx):
            return x

    T, M, E = 4096, 4096, 8
    results = []
    for single in (False, True):
        overlap.FORWARD_SINGLE_LAUNCH = single
        try:
            layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'capacity_factor': 1.25, 'fp32_gate': True}, M,
                                          experts={'type': 'custom', 'module': Identity(), 'count_per_node': E},
                                          seeds=(1, 2, 3), compress_name='int8').to(DEV).to(torch.bfloat16)
            x = torch.randn(T, M, generator=torch.Generator().manual_seed(0)).bfloat16().to(DEV).requires_grad_(True)
            y = layer(x)
            (y.float().square().mean() + y.l_aux.float()).backward()
            torch.cuda.synchronize()
            results.append((y.detach().float(), x.grad.float(), float(y.l_aux.detach()), layer.gates[0].wg.weight.grad.float()))
        finally:
            overlap.FORWARD_SINGLE_LAUNCH = True
    (y0, g0, l0, w0), (y1, g1, l1, w1) = results
    same_rows = (y0 == y1).all(dim=1).float().mean().item()
    assert same_rows > 0.999
    # x.grad carries the gate's share, which depends on the scores' last bits: bf16 tolerance
    assert torch.allclose(g0, g1, rtol=2e-2, atol=2e-2 * g0.abs().max().item())
    assert (g0 == g1).float().mean().item() > 0.99
    assert abs(l0 - l1) <= 1e-4 * abs(l0)
    assert torch.allclose(w0, w1, rtol=2e-2, atol=1e-3 * w0.abs().max().item())


@pytest.mark.parametrize("T,E,k,cap,normalize,with_bias,fp32_gate", [
    (3000, 8, 2, 400, False, False, True), (3000, 8, 2, 400, True, True, True), (2048, 3, 3, 700, True, True, False),
    (1000, 8, 2, 0, True, False, True), (777, 16, 4, 60, False, True, True), (16384, 8, 2, 8, True, False, True)])
def test_single_launch_options_against_the_two_launch_entry_point(T, E, k, cap, normalize, with_bias, fp32_gate):
    """normalize_gate off, a logit bias, capacity 0, a capacity that drops most tokens, top_k ==
    experts: wherever both entry points pick the same experts for every token (their gate GEMMs sum
    in another order, so a token within an ulp of a tie may differ) every output is the same bits."""
    from planmoe_amd import ops
    M = 4096
    g = torch.Generator().manual_seed(T + 7 * E + cap)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    lb = (torch.randn(E, generator=g) * 0.5).to(DEV) if with_bias else None
    kw = dict(fp32_gate=fp32_gate, logit_bias=lb, normalize_gate=normalize, want_scores=True, want_counts=True)
    got = ops.forward_int8_single(x, wg, k, cap, **kw)
    ref = ops.forward_int8(x, wg, k, cap, **kw)
    torch.cuda.synchronize()
    assert int(got["gave_up"]) == 0
    same = (got["indices"] == ref["indices"]).all(0)
    assert float(same.float().mean()) > 0.98
    assert torch.allclose(got["scores"].float(), ref["scores"].float(), rtol=1e-2 if not fp32_gate else 1e-5, atol=1e-6)
    assert torch.allclose(got["l_aux"].float(), ref["l_aux"].float(), rtol=1e-3)
    # the routing, against the oracle on the scores this launch reports (the two entry points' gate
    # GEMMs sum in another order, so a token within an ulp of a tie may go elsewhere in one of them)
    from helpers import bf16_bits
    sc = got["scores"].float().cpu().numpy() if fp32_gate else bf16_bits(got["scores"])
    idx, loc, gates, counts = oracle.route_topk(sc, k, normalize_gate=normalize)
    assert np.array_equal(got["indices"].cpu().numpy(), idx)
    assert np.array_equal(got["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(got["gates"]), np_raw(gates))
    assert np.array_equal(got["counts"].cpu().numpy(), counts)
    if cap > 0:
        # the codes, against the oracle's dispatch + compress of the rows to those slots
        d = torch.from_numpy(oracle.encode(x.float().cpu().numpy(), list(idx), list(loc), None, E, cap)).bfloat16()
        rc, rb, rs = oracle.int8_compress(bf16_bits(d))
        assert np.array_equal(got["codes"].cpu().numpy().reshape(-1), rc.reshape(-1))
        assert np.array_equal(bf16_bits(got["bias"]).reshape(-1), rb.reshape(-1))
        assert np.array_equal(bf16_bits(got["scale"]).reshape(-1), rs.reshape(-1))
    if bool(same.all()):
        for key in ("locations", "counts", "codes"):
            assert torch.equal(got[key], ref[key]), key


def test_ceiling_entry_point_runs_and_leaves_the_chain_alone():
    """planmoe_forward_int8_single_ceiling (the measuring stick of the one-launch kernel) writes every
    row of its code buffer in all three modes, shares the workspace's launch counter with the real
    kernel without disturbing it, and refuses the shapes it does not stand for."""
    from planmoe_amd import ops
    from planmoe_amd._lib import PlanMoEError
    T, M, E, k, C = 16384, 4096, 8, 2, 5120
    g = torch.Generator().manual_seed(31)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    ref = ops.forward_int8_single(x, wg, k, C)
    ceil = ops.ForwardCeiling(x, E, k, C)
    ceil.ws = ops._forward_workspace(T, E, k, x.device)           # the very workspace the real kernel uses
    for mode in (0, 1, 2, 0):
        ceil.codes.fill_(0xAA)
        ceil.run(mode)
        torch.cuda.synchronize()
        assert int(ceil.gave_up) == 0
        rows = ceil.codes.view(E, C, M)
        assert bool((rows[:, 4096:, :] == 0).all())               # the empty slots
        assert not bool((rows[:, :4096, :] == 0xAA).all(dim=2).any())   # every used slot was written
        again = ops.forward_int8_single(x, wg, k, C)
        torch.cuda.synchronize()
        assert int(again["gave_up"]) == 0
        assert torch.equal(again["codes"], ref["codes"]) and torch.equal(again["locations"], ref["locations"])
    with pytest.raises(PlanMoEError):
        ops.ForwardCeiling(x[:, :2048].contiguous(), E, k, C).run(0)
    with pytest.raises(PlanMoEError):
        ops.ForwardCeiling(x, 16, k, C).run(0)


def test_single_launch_on_two_streams_at_once():
    """Two one-launch kernels at the same time on one GPU could keep each other's work-groups from
    becoming resident; the library puts launches on one device in a row whatever their streams.
    Two different full-size batches, enqueued alternately on two streams without waiting: nobody
    gives up and every result is that of the same call made alone."""
    from planmoe_amd import ops
    T, M, E, k = 16384, 4096, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4)
    g = torch.Generator().manual_seed(41)
    xs = [torch.randn(T, M, generator=g).bfloat16().to(DEV) for _ in range(2)]
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    want = [ops.forward_int8_single(x, wg, k, C) for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[], []]
    for _ in range(6):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                got[i].append(ops.forward_int8_single(xs[i], wg, k, C))
    torch.cuda.synchronize()
    for i in (0, 1):
        for out in got[i]:
            assert int(out["gave_up"]) == 0
            for name in ("indices", "locations", "codes", "bias", "scale", "l_aux"):
                assert torch.equal(out[name].reshape(-1).view(torch.uint8), want[i][name].reshape(-1).view(torch.uint8)), name
