"""GPU parity: gate-logits GEMM (MFMA), the fused forward chain of config 2 and the
moe_layer mirror end to end."""
import numpy as np
import pytest
import torch

import oracle
from helpers import bf16_bits, np_raw, raw, to_np, zipf_bias

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("T,M,E,dtype", [(100, 512, 8, torch.bfloat16), (1000, 4096, 8, torch.bfloat16), (777, 2048, 64, torch.bfloat16),
                                         (100, 2048, 2, torch.float32), (50, 100, 5, torch.float32), (50, 1000, 20, torch.float32),
                                         (31, 136, 17, torch.bfloat16), (16, 4100, 8, torch.bfloat16), (10, 64, 100, torch.float32),
                                         (300, 2056, 32, torch.bfloat16), (129, 520, 128, torch.bfloat16), (65, 36, 24, torch.float32),
                                         (200, 264, 130, torch.bfloat16)])
def test_gate_logits(T, M, E, dtype):
    """fp32-accumulated logits against the oracle's fp64 dot products: rtol 1e-5 of the row scale
    (products of bf16 values are exact in fp32, only the summation order differs)."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, M, generator=g).to(dtype)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).to(dtype)
    out = ops.gate_logits(x.to(DEV), wg.to(DEV), torch.float32).cpu().numpy()
    ref = oracle.gate_logits(to_np(x), to_np(wg))
    mag = oracle.gate_logits(to_np(x.abs()), to_np(wg.abs()))
    assert (np.abs(out - ref) <= 1e-5 * np.abs(ref) + 1e-6 * mag).all()


def test_gate_logits_fp16_and_rounded_output():
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(6)
    x = torch.randn(64, 1024, generator=g).half()
    wg = (torch.randn(33, 1024, generator=g) / 32).half()
    out = ops.gate_logits(x.to(DEV), wg.to(DEV), torch.float32).cpu()
    assert torch.allclose(out.double(), x.double() @ wg.double().t(), rtol=1e-5, atol=1e-5)
    xb, wb = x.bfloat16(), wg.bfloat16()
    o32 = ops.gate_logits(xb.to(DEV), wb.to(DEV), torch.float32)
    o16 = ops.gate_logits(xb.to(DEV), wb.to(DEV), torch.bfloat16)
    assert torch.equal(o16, o32.bfloat16())


def _forward_chain(T, M, E, k, cf, seed, bias=None):
    """gate GEMM -> softmax/top-k/slots -> dispatch+int8, every stage checked against the
    oracle evaluated on the bits the previous HIP stage produced."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, M, generator=g).bfloat16()
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16()
    xd, wd = x.to(DEV), wg.to(DEV)
    logits = ops.gate_logits(xd, wd, torch.float32)
    ref = oracle.gate_logits(bf16_bits(x), bf16_bits(wg))
    assert np.abs(logits.cpu().numpy() - ref).max() <= 1e-5 * np.abs(ref).max()
    r = ops.route_topk(logits, k, is_logits=True, logit_bias=bias, want_scores=True, want_counts=True)
    scores = r["scores"].cpu()
    lg = logits.cpu() if bias is None else logits.cpu() + bias
    assert torch.allclose(scores, torch.softmax(lg, 1), rtol=1e-5, atol=1e-9)
    idx, loc, gates, counts = oracle.route_topk(scores.numpy(), k)
    assert np.array_equal(r["indices"].cpu().numpy(), idx) and np.array_equal(r["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(r["gates"]), np_raw(gates)) and np.array_equal(r["counts"].cpu().numpy(), counts)
    C = ops.capacity(T, E, k, cf, 4)
    codes, b, s = ops.dispatch_int8(xd, list(r["indices"]), list(r["locations"]), None, E, C)
    return x, idx, loc, gates, counts, C, codes, b, s


def test_config2_forward_chain_full_size():
    """16384 x 4096 bf16, 8 experts, top-2, cf 1.25: codes / bias / scale of the whole
    [8, 5120, 4096] buffer against the oracle, then the int8 round trip back to tokens."""
    from planmoe_amd import ops
    T, M, E, k = 16384, 4096, 8, 2
    x, idx, loc, gates, counts, C, codes, b, s = _forward_chain(T, M, E, k, 1.25, seed=0)
    assert C == 5120
    d = torch.from_numpy(oracle.encode(x.float().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
    rc, rb, rs = oracle.int8_compress(bf16_bits(d))
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(raw(b), np_raw(rb)) and np.array_equal(raw(s), np_raw(rs))
    dec = ops.int8_decompress(codes, b, s)
    assert np.array_equal(raw(dec), np_raw(oracle.int8_decompress(rc, rb, rs)))
    # decode(int8 round trip) stays within the codec's error of x * sum(kept gates)
    i = [torch.from_numpy(a).to(DEV) for a in idx]; l = [torch.from_numpy(a).to(DEV) for a in loc]
    gt = [torch.from_numpy(a).to(DEV) for a in gates]
    y = ops.combine_fwd(dec, i, l, gt, T, C).float().cpu()
    w = torch.from_numpy(((loc < C) * gates).sum(0))
    assert (y - x.float() * w[:, None]).abs().max() < 0.06


def test_config3_forward_chain_full_size_zipf():
    T, M, E = 32768, 2048, 64
    x, idx, loc, gates, counts, C, codes, b, s = _forward_chain(T, M, E, 1, 1.0, seed=0, bias=zipf_bias(E))
    assert C == 512
    kept = int((loc[0] < C).sum())
    assert kept == int(np.minimum(counts[0], C).sum()) and kept < T * 3 // 4
    # slots past an expert's fill are empty rows: codes 0, scale 0
    fill = np.minimum(counts[0], C)
    occupied = (np.arange(C)[None, :] < fill[:, None]).reshape(-1)
    sc = s.float().view(-1).cpu().numpy()
    assert (sc[~occupied] == 0).all() and (codes.view(E * C, M)[torch.from_numpy(~occupied).to(DEV)] == 0).all()
    # occupied rows hold their token's codes
    rows = np.nonzero(loc[0] < C)[0][::97]
    rc, rb, rs = oracle.int8_compress(bf16_bits(x[torch.from_numpy(rows)] + 0.0))
    slot = idx[0][rows].astype(np.int64) * C + loc[0][rows]
    assert np.array_equal(codes[torch.from_numpy(slot).to(DEV)].cpu().numpy(), rc)


def test_moe_layer_forward_matches_the_oracle_composition():
    """moe_layer with identity experts: out == decode(codec(encode(x))) assembled from the oracle."""
    import planmoe_amd

    class Identity(torch.nn.Module):
        def update(self, ctx):
            self.dummy = torch.nn.Parameter(torch.zeros(1, dtype=torch.bfloat16))

        def forward(self, x, ctx):
            return x

    T, M, E, k = 512, 256, 4, 2
    for compress in ("no", "int8"):
        layer = planmoe_amd.moe_layer({'type': 'top', 'k': k, 'capacity_factor': 1.0, 'fp32_gate': True}, M,
                                      experts={'type': 'custom', 'module': Identity(), 'count_per_node': E},
                                      seeds=(1, 2, 3), compress_name=compress).to(DEV).eval()
        x = torch.randn(2, T // 2, M, generator=torch.Generator().manual_seed(0)).bfloat16()
        with torch.no_grad():
            y = layer(x.to(DEV))
        assert y.shape == x.shape and y.dtype == torch.bfloat16
        from planmoe_amd import ops
        # the gate is kept in fp32 here: its logits (the weight as two bf16 parts) are what the layer routes on
        with torch.no_grad():
            logits = layer.gates[0](x.view(T, M).to(DEV))
        assert logits.dtype == torch.float32
        r = ops.route_topk(logits, k, is_logits=True, want_scores=True)
        idx, loc, gates, _ = oracle.route_topk(r["scores"].cpu().numpy(), k)
        C = oracle.capacity(T, E, k, 1.0, 4)
        d = torch.from_numpy(oracle.encode(x.view(T, M).float().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
        for _ in range(2):                                     # the pipeline applies the codec twice
            if compress == "int8":
                rc, rb, rs = oracle.int8_compress(bf16_bits(d))
                d = torch.from_numpy(oracle.int8_decompress(rc, rb, rs).view(np.int16)).view(torch.bfloat16)
        want = torch.from_numpy(oracle.decode(d.float().numpy(), list(idx), list(loc), list(gates), T, C)).bfloat16()
        assert np.array_equal(raw(y.view(T, M)), raw(want))
        assert abs(float(y.l_aux) - oracle.gshard_loss(r["scores"].cpu().numpy(), idx[0])) < 1e-4


def test_moe_layer_trains_with_builtin_ffn():
    import planmoe_amd
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True}, 64,
                                  experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 128},
                                  seeds=(1, 2, 3), compress_name='no').to(DEV)
    x = torch.randn(8, 32, 64, device=DEV, requires_grad=True)
    y = layer(x)
    (y.float().pow(2).mean() + y.l_aux).backward()
    assert x.grad is not None and torch.isfinite(x.grad).all()
    assert layer.experts.batched_fc1_w.grad is not None
    wg_grad = layer.gates[0].wg.weight.grad                    # gates and l_aux reach the gate weight
    assert wg_grad is not None and torch.isfinite(wg_grad).all() and wg_grad.abs().sum() > 0


def test_moe_layer_with_the_lossless_codec_equals_no_codec():
    """compress_name='lz' changes nothing but the sign of a zero: output and gradients equal
    those of compress_name='no', forward and backward, with two chunks per pass."""
    import planmoe_amd
    res = {}
    for compress in ("no", "lz"):
        layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 2.0}, 64,
                                      experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 128},
                                      seeds=(1, 2, 3), compress_name=compress, a2a_ffn_overlap_degree=2).to(DEV)
        x = torch.randn(8, 32, 64, generator=torch.Generator().manual_seed(5)).to(DEV).requires_grad_(True)
        y = layer(x)
        (y.float().pow(2).mean() + y.l_aux).backward()
        res[compress] = (y.detach(), x.grad, layer.experts.batched_fc1_w.grad, layer.gates[0].wg.weight.grad)
    for a, b in zip(res["no"], res["lz"]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("T,M,E,k,cf,dtype,fp32_gate,use_bias", [
    (1000, 512, 8, 2, 1.25, torch.bfloat16, True, False), (33, 256, 4, 2, 1.0, torch.bfloat16, True, False),
    (4096, 1024, 64, 1, 1.0, torch.bfloat16, True, True), (500, 2048, 2, 2, 1.0, torch.float32, True, False),
    (700, 264, 16, 3, 0.5, torch.bfloat16, False, False), (257, 128, 33, 4, 1.0, torch.float16, True, False),
    (31, 64, 5, 5, 2.0, torch.float32, False, True), (1500, 776, 48, 2, 1.25, torch.bfloat16, True, True),
    (900, 260, 24, 20, 1.0, torch.float32, True, False), (640, 512, 64, 17, 1.0, torch.bfloat16, False, False)])
def test_fused_forward_matches_unfused_and_oracle(T, M, E, k, cf, dtype, fp32_gate, use_bias):
    """planmoe_forward_int8 / planmoe_gate_route against the stage-by-stage entry points and the
    oracle (routing evaluated on the scores the kernel reports)."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, M, generator=g).to(dtype).to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).to(dtype).to(DEV)
    bias = zipf_bias(E) if use_bias else None
    C = ops.capacity(T, E, k, cf, 4)
    sdt = torch.float32 if (fp32_gate or dtype == torch.float32) else dtype
    for rep in range(2):                    # twice: the workspace counter must come back to zero
        out = ops.forward_int8(x, wg, k, C, fp32_gate=fp32_gate, logit_bias=bias, want_logits=True,
                               want_scores=True, want_counts=True)
        assert torch.equal(out["logits"], ops.gate_logits(x, wg, sdt))
        scores = out["scores"]
        assert scores.dtype == sdt and out["gates"].dtype == sdt
        lg = out["logits"].float().cpu() + (bias if use_bias else 0)
        if sdt != torch.float32:
            lg = lg.to(sdt).float()
        assert torch.allclose(scores.float().cpu(), torch.softmax(lg, 1), rtol=1e-5 if sdt == torch.float32 else 1e-2, atol=1e-8)
        if sdt == torch.float16:
            r = ops.route_topk(scores, k, want_counts=True)     # the oracle has no fp16 mode
            idx, loc, gates, counts = (r["indices"].cpu().numpy(), r["locations"].cpu().numpy(), None, r["counts"].cpu().numpy())
            assert torch.equal(out["gates"], r["gates"])
        else:
            idx, loc, gates, counts = oracle.route_topk(to_np(scores), k)
            assert np.array_equal(raw(out["gates"]), np_raw(gates))
        assert np.array_equal(out["indices"].cpu().numpy(), idx)
        assert np.array_equal(out["locations"].cpu().numpy(), loc)
        assert np.array_equal(out["counts"].cpu().numpy(), counts)
        if sdt != torch.float16:
            want = oracle.gshard_loss(to_np(scores), idx[0])
            assert abs(float(out["l_aux"]) - want) <= (1e-5 if sdt == torch.float32 else 1e-2) * abs(want)
        c2, b2, s2 = ops.dispatch_int8(x, list(out["indices"]), list(out["locations"]), None, E, C)
        assert torch.equal(out["codes"], c2)
        assert np.array_equal(raw(out["bias"]), raw(b2)) and np.array_equal(raw(out["scale"]), raw(s2))
        r2 = ops.gate_route(x, wg, k, fp32_gate=fp32_gate, logit_bias=bias, want_counts=True)
        for name in ("indices", "locations", "counts"):
            assert torch.equal(r2[name], out[name])
        assert np.array_equal(raw(r2["gates"]), raw(out["gates"]))
        # the two entry points add the per-group shares of the loss up in different orders
        assert abs(float(r2["l_aux"]) - float(out["l_aux"])) <= 1e-6 * abs(float(out["l_aux"]))


@pytest.mark.parametrize("T,M,E,k,cf,dtype,fp32_gate,use_bias", [
    (1000, 512, 8, 2, 1.25, torch.bfloat16, True, False), (33, 256, 4, 2, 1.0, torch.bfloat16, True, False),
    (4096, 1024, 64, 1, 1.0, torch.bfloat16, True, True), (500, 2048, 2, 2, 1.0, torch.float32, True, False),
    (700, 264, 16, 3, 0.5, torch.bfloat16, False, False), (257, 128, 33, 4, 1.0, torch.float16, True, False),
    (31, 64, 5, 5, 2.0, torch.float32, False, True), (900, 260, 24, 20, 1.0, torch.float32, True, False),
    (640, 512, 64, 17, 1.0, torch.bfloat16, False, False), (8192, 2048, 2, 2, 1.0, torch.float32, True, False)])
def test_forward_plain_matches_routing_plus_dispatch_and_the_oracle(T, M, E, k, cf, dtype, fp32_gate, use_bias):
    """planmoe_forward_plain (gate + routing + dispatch without a codec, two launches) against
    planmoe_gate_route + planmoe_dispatch_fwd bit for bit, and its buffer against the oracle's encode of
    the same routing (the last case is config 1 at full size)."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, M, generator=g).to(dtype)
    x[min(3, T - 1), :8] = -0.0                              # 0 + (-0) = +0 in the reference's accumulation
    x = x.to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).to(dtype).to(DEV)
    bias = zipf_bias(E) if use_bias else None
    C = ops.capacity(T, E, k, cf, 4)
    for rep in range(2):
        out = ops.forward_plain(x, wg, k, C, fp32_gate=fp32_gate, logit_bias=bias, want_scores=True, want_counts=True)
        r2 = ops.gate_route(x, wg, k, fp32_gate=fp32_gate, logit_bias=bias, want_scores=True, want_counts=True)
        for name in ("indices", "locations", "counts"):
            assert torch.equal(r2[name], out[name]), name
        assert np.array_equal(raw(r2["gates"]), raw(out["gates"])) and np.array_equal(raw(r2["scores"]), raw(out["scores"]))
        assert abs(float(r2["l_aux"]) - float(out["l_aux"])) <= 1e-6 * abs(float(out["l_aux"]))
        d2 = ops.dispatch_fwd(x, list(out["indices"]), list(out["locations"]), None, E, C)
        assert np.array_equal(raw(out["dispatched"]), raw(d2))
    if dtype != torch.float16:
        idx, loc = out["indices"].cpu().numpy(), out["locations"].cpu().numpy()
        want = oracle.encode(x.float().cpu().numpy(), list(idx), list(loc), None, E, C)
        assert np.array_equal(out["dispatched"].float().cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("T,M,E,k", [(300, 776, 24, 2), (200, 264, 8, 2), (130, 1032, 64, 1)])
def test_fused_forward_rows_of_one_sign(T, M, E, k):
    """Row min / max come out of the gate kernel's scan of the rows it streams: rows that do not
    straddle zero and a model_dim that is not a multiple of a K chunk (128 bf16 values) show a
    scan that picks up padding."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + M)
    x = (torch.randn(T, M, generator=g).abs() + 0.5)
    x[::3] *= -1
    x = x.bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    C = ops.capacity(T, E, k, 1.5, 4)
    out = ops.forward_int8(x, wg, k, C)
    c2, b2, s2 = ops.dispatch_int8(x, list(out["indices"]), list(out["locations"]), None, E, C)
    assert torch.equal(out["codes"], c2)
    assert np.array_equal(raw(out["bias"]), raw(b2)) and np.array_equal(raw(out["scale"]), raw(s2))
    rc, rb, rs = oracle.int8_compress(bf16_bits(ops.dispatch_fwd(x, list(out["indices"]), list(out["locations"]), None, E, C).cpu()))
    assert np.array_equal(c2.cpu().numpy().reshape(rc.shape), rc)


def test_cosine_gate_logits_and_layer():
    """CosineTopKGate against the reference's formula in fp32 torch ops (rtol 1e-5 of the logit
    scale), then a moe_layer with that gate and batch-prioritised routing trains one step."""
    import planmoe_amd
    from planmoe_amd.gates import CosineTopKGate
    torch.manual_seed(0)
    gate = CosineTopKGate(96, 12, k=2, fp32_gate=True, proj_dim=64).to(DEV)
    x = torch.randn(300, 96, device=DEV)
    got = gate(x)
    proj = torch.nn.functional.normalize(gate.cosine_projector(x), dim=1)
    want = (proj @ torch.nn.functional.normalize(gate.sim_matrix, dim=0)) * gate.temperature.exp()
    assert got.shape == (300, 12) and torch.allclose(got, want, rtol=1e-5, atol=1e-5 * float(gate.temperature.detach().exp()))

    layer = planmoe_amd.moe_layer({'type': 'cosine_top', 'k': 2, 'fp32_gate': True, 'proj_dim': 32}, 64,
                                  experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 128},
                                  seeds=(1, 2, 3), compress_name='no', batch_prioritized_routing=True).to(DEV)
    xin = torch.randn(8, 32, 64, device=DEV, requires_grad=True)
    y = layer(xin)
    (y.float().pow(2).mean() + y.l_aux).backward()
    assert torch.isfinite(xin.grad).all()
    g = layer.gates[0].sim_matrix.grad
    assert g is not None and torch.isfinite(g).all() and g.abs().sum() > 0


@pytest.mark.parametrize("T,M,E,k,cf,use_bias", [(16384, 4096, 8, 2, 1.25, False), (32768, 2048, 64, 1, 1.0, True),
                                                  (8192, 2048, 2, 2, 1.0, False)])
def test_forward_entry_point_full_size(T, M, E, k, cf, use_bias):
    """planmoe_forward_int8 (two launches) at the full size of configs 2, 3 and 1 (bf16 here):
    routing against the oracle on the scores the kernel reports, codes / bias / scale against the
    stand-alone dispatch + int8 entry point on that routing, counts and loss against the oracle."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    bias = zipf_bias(E) if use_bias else None
    C = ops.capacity(T, E, k, cf, 4)
    out = ops.forward_int8(x, wg, k, C, logit_bias=bias, want_scores=True, want_counts=True)
    scores = out["scores"].cpu().numpy()
    idx, loc, gates, counts = oracle.route_topk(scores, k)
    assert np.array_equal(out["indices"].cpu().numpy(), idx)
    assert np.array_equal(out["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(out["gates"]), np_raw(gates))
    assert np.array_equal(out["counts"].cpu().numpy(), counts)
    want = oracle.gshard_loss(scores, idx[0])
    assert abs(float(out["l_aux"]) - want) <= 1e-5 * abs(want)
    c2, b2, s2 = ops.dispatch_int8(x, list(out["indices"]), list(out["locations"]), None, E, C)
    assert torch.equal(out["codes"].view(-1), c2.view(-1))
    assert np.array_equal(raw(out["bias"]).reshape(-1), raw(b2).reshape(-1))
    assert np.array_equal(raw(out["scale"]).reshape(-1), raw(s2).reshape(-1))


def test_row_statistics_on_special_rows():
    """Row min / max as the three kernels that scan bf16 rows compute them (the gate kernel of the
    chain, the stand-alone dispatch + int8, the stand-alone compressor): rows that are all negative,
    all positive, mixed signs of zero, constant, tiny, huge, and -- where no gate has to digest them --
    rows with infinities and NaNs, against the literal torch-CPU chain on the dispatched buffer."""
    from planmoe_amd import ops
    T, M, E, k = 256, 512, 4, 2
    g = torch.Generator().manual_seed(12)
    x = torch.randn(T, M, generator=g)
    x[0] = -x[0].abs() - 1.0                      # all negative
    x[1] = x[1].abs() + 1.0                       # all positive
    x[2] = 0.0; x[2, ::2] = -0.0                  # zeros of both signs
    x[3] = -0.0
    x[4] = 3.25
    x[5] = -3.25
    x[6] *= 2.0 ** -120
    x[7] *= 2.0 ** 120
    x[8, 1:] = x[8, 1:].abs(); x[8, 0] = -0.0     # -0 as the only "negative"
    x[9] = -x[9].abs(); x[9, 5] = 0.0             # +0 as the only non-negative
    x = x.bfloat16()
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16()
    C = ops.capacity(T, E, k, 2.0, 4)

    def expect(buf):                              # Int8Compressor's chain, op by op in bf16 on the CPU
        b = torch.min(buf, -1, True)[0]; sc = torch.max(buf, -1, True)[0] - b
        codes = torch.mul(torch.div(torch.sub(buf, b), sc), 255.0)
        codes = torch.nan_to_num(codes, nan=0.0, posinf=0.0, neginf=0.0).to(torch.uint8)
        return codes, b, sc

    def same(got, ref):                           # bit for bit, any NaN for a NaN, either zero for a zero
        got, ref = got.cpu().view(-1).float(), ref.view(-1).float()
        nan = torch.isnan(ref)
        return torch.equal(torch.isnan(got), nan) and torch.equal(got[~nan], ref[~nan])

    xd, wd = x.to(DEV), wg.to(DEV)
    out = ops.forward_int8(xd, wd, k, C)
    idx, loc = list(out["indices"]), list(out["locations"])
    d = ops.dispatch_fwd(xd, idx, loc, None, E, C).cpu()
    codes, b, sc = expect(d)
    assert torch.equal(out["codes"].cpu(), codes) and same(out["bias"], b) and same(out["scale"], sc)
    # with infinities and NaNs in the rows: routing given, stand-alone kernels
    y = x.clone()
    y[10, 3] = float("inf"); y[11, 4] = float("-inf"); y[12, 5] = float("nan"); y[13] = float("inf")
    y[14, 0] = float("nan"); y[14, 1] = float("-inf"); y[15] = -y[15].abs(); y[15, 7] = float("nan")
    y[16] = -y[16].abs(); y[16, 9] = -float("nan")
    yd = y.to(DEV)
    d = ops.dispatch_fwd(yd, idx, loc, None, E, C).cpu()
    codes, b, sc = expect(d)
    c2, b2, s2 = ops.dispatch_int8(yd, idx, loc, None, E, C)
    assert torch.equal(c2.cpu(), codes) and same(b2, b) and same(s2, sc)
    c3, b3, s3 = ops.int8_compress(d.to(DEV))
    assert torch.equal(c3.cpu(), codes) and same(b3, b) and same(s3, sc)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_moe_layer_fused_int8_path_equals_the_stepwise_pipeline(dtype):
    """moe_layer with compress_name='int8': the fused send / receive sides (dispatch+compress,
    decompress+combine) against the step-by-step pipeline, outputs and every gradient bit for bit."""
    import planmoe_amd
    from planmoe_amd import overlap
    results = []
    for fuse in (True, False):
        overlap.FUSE_INT8, overlap.FUSE_GATE = fuse, False
        try:
            results.append(_layer_pass(planmoe_amd, dtype))
        finally:
            overlap.FUSE_INT8 = overlap.FUSE_GATE = True
    for a, b in zip(*results):
        assert torch.equal(a, b)
    assert results[0][1].abs().sum() > 0 and results[0][2].abs().sum() > 0


def test_moe_layer_fused_zfp_send_side_equals_the_stepwise_pipeline():
    """compress_name='zfp' (fp32): fast_encode + compress as planmoe_dispatch_zfp in forward and in
    the backward of fast_decode -- the output and the gradients that do not pass through the gate
    bit for bit against the steps; the gate gradients come from planmoe_bwd_gate_zfp, which sums in
    another order, so x.grad and the gate weight's gradient agree to rounding."""
    import planmoe_amd
    from planmoe_amd import overlap
    results = []
    for fuse in (True, False):
        overlap.FUSE_ZFP = fuse
        try:
            layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 1.25}, 128,
                                          experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 64},
                                          seeds=(1, 2, 3), compress_name='zfp').to(DEV)
            x = torch.randn(6, 50, 128, generator=torch.Generator().manual_seed(5)).to(DEV).requires_grad_(True)
            y = layer(x)
            (y.pow(2).mean() + y.l_aux).backward()
            results.append((y.detach(), x.grad.detach(), layer.gates[0].wg.weight.grad.detach(),
                            layer.experts.batched_fc1_w.grad.detach()))
        finally:
            overlap.FUSE_ZFP = True
    _same_but_for_the_gate_gradients(*results)
    assert results[0][1].abs().sum() > 0 and results[0][2].abs().sum() > 0


def _same_but_for_the_gate_gradients(fused, staged, exact_gate=False):
    """(y, x.grad, gate weight grad, fc1 grad): y and the expert gradient bit for bit; the two that
    pass through the gate gradients bit for bit (exact_gate) or to fp32 rounding."""
    assert torch.equal(fused[0], staged[0]) and torch.equal(fused[3], staged[3])
    for a, b in ((fused[1], staged[1]), (fused[2], staged[2])):
        if exact_gate:
            assert torch.equal(a, b)
        else:
            assert (a.float() - b.float()).abs().max().item() <= 1e-4 * max(b.float().abs().max().item(), 1e-6)


@pytest.mark.parametrize("compress,dtype", [("int8", torch.bfloat16), ("int8", torch.float32), ("zfp", torch.float32)])
def test_fused_paths_with_two_chunks_equal_the_stepwise_pipeline(compress, dtype):
    """a2a_ffn_overlap_degree = 2: the fused kernels code the whole buffer and only the expert call
    is sliced; the step-by-step pipeline codes slice by slice.  Same bits, forward and backward."""
    import planmoe_amd
    from planmoe_amd import overlap
    results = []
    for fuse in (True, False):
        overlap.FUSE_INT8 = overlap.FUSE_ZFP = fuse
        overlap.FUSE_GATE = False
        try:
            layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 1.25}, 128,
                                          experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 64},
                                          seeds=(1, 2, 3), compress_name=compress, a2a_ffn_overlap_degree=2).to(DEV).to(dtype)
            x = torch.randn(6, 50, 128, generator=torch.Generator().manual_seed(5)).to(dtype).to(DEV).requires_grad_(True)
            y = layer(x)
            (y.float().pow(2).mean() + y.l_aux.float()).backward()
            results.append((y.detach(), x.grad.detach(), layer.gates[0].wg.weight.grad.detach(),
                            layer.experts.batched_fc1_w.grad.detach()))
        finally:
            overlap.FUSE_INT8 = overlap.FUSE_ZFP = overlap.FUSE_GATE = True
    _same_but_for_the_gate_gradients(*results, exact_gate=(compress != "zfp"))


def _layer_pass(planmoe_amd, dtype):
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 1.25}, 128,
                                  experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 64},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV).to(dtype)
    x = torch.randn(6, 50, 128, generator=torch.Generator().manual_seed(5)).to(dtype).to(DEV).requires_grad_(True)
    y = layer(x)
    (y.float().pow(2).mean() + y.l_aux.float()).backward()
    return (y.detach(), x.grad.detach(), layer.gates[0].wg.weight.grad.detach(),
            layer.experts.batched_fc1_w.grad.detach(), y.l_aux.detach())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_moe_layer_with_the_gate_in_the_fused_send_side(dtype):
    """The layer's default for compress_name='int8': gate GEMM + routing + encode + compress as
    planmoe_forward_int8.  Its softmax sums in another order than the stand-alone routing, so
    the comparison with the staged pipeline is to rounding, forward and backward."""
    import planmoe_amd
    from planmoe_amd import overlap
    assert overlap.FUSE_GATE and overlap.FUSE_INT8
    fused = _layer_pass(planmoe_amd, dtype)
    overlap.FUSE_GATE = False
    try:
        staged = _layer_pass(planmoe_amd, dtype)
    finally:
        overlap.FUSE_GATE = True
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for name, a, b in zip(("y", "dx", "dwg", "dfc1", "l_aux"), fused, staged):
        a, b = a.float(), b.float()
        assert a.shape == b.shape
        err = (a - b).abs().max().item()
        assert err <= tol * max(b.abs().max().item(), 1e-6), (name, err)
    assert fused[2].abs().sum() > 0


@pytest.mark.parametrize("degree", [1, 2])
@pytest.mark.parametrize("compress,dtype", [("no", torch.bfloat16), ("no", torch.float32), ("lz", torch.float32),
                                            ("zfp", torch.float32)])
def test_moe_layer_with_gate_routing_and_encode_as_one_node(compress, dtype, degree):
    """The layer's default for the other compressors: gate GEMM + routing (planmoe_gate_route) and
    the encode as one autograd node, so that the two gradients of x meet in one GEMM epilogue.
    Against the staged pipeline (gate, routing and encode as separate nodes) to rounding: the
    fused softmax sums in another order, and the staged x.grad is rounded once more."""
    import planmoe_amd
    from planmoe_amd import overlap

    def run():
        layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 1.25}, 128,
                                      experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 64},
                                      seeds=(1, 2, 3), compress_name=compress,
                                      a2a_ffn_overlap_degree=degree).to(DEV).to(dtype)
        x = torch.randn(6, 50, 128, generator=torch.Generator().manual_seed(5)).to(dtype).to(DEV).requires_grad_(True)
        y = layer(x)
        (y.float().pow(2).mean() + y.l_aux.float()).backward()
        return (y.detach(), x.grad.detach(), layer.gates[0].wg.weight.grad.detach(),
                layer.experts.batched_fc1_w.grad.detach(), y.l_aux.detach())

    assert overlap.FUSE_GATE
    fused = run()
    overlap.FUSE_GATE = False
    try:
        staged = run()
    finally:
        overlap.FUSE_GATE = True
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for name, a, b in zip(("y", "dx", "dwg", "dfc1", "l_aux"), fused, staged):
        a, b = a.float(), b.float()
        assert a.shape == b.shape
        err = (a - b).abs().max().item()
        assert err <= tol * max(b.abs().max().item(), 1e-6), (name, err)
    assert fused[1].abs().sum() > 0 and fused[2].abs().sum() > 0


@pytest.mark.parametrize("T,M,E,dtype", [(4099, 256, 16, torch.bfloat16), (16384, 512, 8, torch.float32),
                                         (100, 64, 4, torch.float32), (1024, 128, 64, torch.float16)])
def test_gate_weight_gradient_split_over_token_chunks(T, M, E, dtype):
    """gates.weight_grad (a batched GEMM over token chunks + a sum) against the product in fp64:
    ragged token counts, the short-input fall-back, a gradient that is a transposed view."""
    from planmoe_amd import gates
    g0 = torch.Generator().manual_seed(T)
    x = torch.randn(T, M, generator=g0).to(dtype).to(DEV)
    g = (torch.randn(E, T, generator=g0) * 0.01).to(dtype).to(DEV).t()          # [T, E], not contiguous
    got = gates.weight_grad(g, x)
    assert got.dtype == dtype and got.shape == (E, M)
    ref = g.double().t() @ x.double()
    tol = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 2e-3}[dtype]
    assert (got.double() - ref).abs().max().item() <= tol * ref.abs().max().item()


@pytest.mark.parametrize("T,M,E,dtype", [(1000, 512, 8, torch.bfloat16), (257, 264, 3, torch.bfloat16), (4099, 1024, 7, torch.float16),
                                         (300, 100, 2, torch.float32), (1, 8, 1, torch.bfloat16), (16384, 4096, 8, torch.bfloat16)])
def test_gate_dx_accumulate(T, M, E, dtype):
    """planmoe_gate_dx_accumulate (dx += g @ wg in one pass over dx) against the product in fp64."""
    from planmoe_amd import ops
    g0 = torch.Generator().manual_seed(T + E)
    dx = torch.randn(T, M, generator=g0).to(dtype).to(DEV)
    w = (torch.randn(E, M, generator=g0) * M ** -0.5).to(dtype).to(DEV)
    g = (torch.randn(T, E, generator=g0) * 0.1).to(DEV)
    ref = dx.double() + g.to(dtype).double() @ w.double()
    guard = dx.clone()
    got = ops.gate_dx_accumulate(dx, g, w)
    assert got.data_ptr() == dx.data_ptr() and not torch.equal(dx, guard)
    ulp = {torch.float32: 2.0 ** -23, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    assert ((dx.double() - ref).abs() <= ulp * ref.abs() + 1e-6).all()
    with pytest.raises(Exception):
        ops.gate_dx_accumulate(dx, torch.zeros(T, 9, device=DEV), torch.zeros(9, M, device=DEV, dtype=dtype))


@pytest.mark.parametrize("E", [8, 96])
def test_fp32_gate_weight_next_to_fp16_activations(E):
    from planmoe_amd import gates
    T, M = 1000, 512
    g = torch.Generator().manual_seed(22)
    x = torch.randn(T, M, generator=g).half().to(DEV)
    gate = gates.LinearTopKGate(M, E, k=2, fp32_gate=True).to(DEV)
    with torch.no_grad():
        gate.wg.weight.copy_(torch.randn(E, M, generator=g) * M ** -0.5)
    ref = x.double() @ gate.wg.weight.double().t()
    assert (gate(x).double() - ref).abs().max().item() <= 2e-5


def test_fp32_gate_weight_next_to_bf16_activations():
    """fp32_gate with the gate kept in fp32 (top.py:21-26: x.float() @ wg.float()): the weight goes
    through the MFMA kernel as two bf16 parts, so the logits stay within fp32 summation noise of the
    fp32 product, where a weight rounded to bf16 is off by 1e-3 and re-routes tokens near a tie."""
    import planmoe_amd
    from planmoe_amd import gates
    T, M, E, k = 4096, 1024, 8, 2
    g = torch.Generator().manual_seed(21)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    gate = gates.LinearTopKGate(M, E, k=k, fp32_gate=True).to(DEV)
    assert gate.wg.weight.dtype == torch.float32
    with torch.no_grad():
        gate.wg.weight.copy_(torch.randn(E, M, generator=g) * M ** -0.5)
    logits = gate(x)
    assert logits.dtype == torch.float32
    ref = x.double() @ gate.wg.weight.double().t()
    err = (logits.double() - ref).abs().max().item()
    rounded = (x.double() @ gate.wg.weight.bfloat16().double().t() - ref).abs().max().item()
    assert err <= 2e-5 and rounded > 20 * err
    # same choices as the fp32 product wherever the runner-up is not within the noise
    top = torch.topk(ref, k + 1, dim=1)
    clear = (top.values[:, k - 1] - top.values[:, k]) > 1e-4
    mine = torch.topk(logits, k, dim=1).indices
    assert torch.equal(mine[clear], top.indices[clear][:, :k]) and clear.float().mean() > 0.99

    # the layer end to end with such a gate: experts in bf16, gate in fp32; gradients reach the fp32 weight
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'capacity_factor': 1.25}, 128,
                                  experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 64},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV)
    layer.experts.to(torch.bfloat16)
    assert layer.gates[0].wg.weight.dtype == torch.float32
    xin = torch.randn(300, 128, generator=g).bfloat16().to(DEV).requires_grad_(True)
    y = layer(xin)
    (y.float().pow(2).mean() + y.l_aux.float()).backward()
    wgrad = layer.gates[0].wg.weight.grad
    assert y.dtype == torch.bfloat16 and wgrad.dtype == torch.float32 and wgrad.abs().sum() > 0
    assert torch.isfinite(xin.grad).all() and xin.grad.abs().sum() > 0


def test_moe_layer_prescore_noise_and_load_importance_loss():
    """The remaining layer options run end to end: gates applied at encode (is_postscore=False),
    gate noise with the load-importance loss, a data-dependent capacity (capacity_factor = 0)."""
    import planmoe_amd
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'fp32_gate': True, 'gate_noise': 1.0, 'capacity_factor': 0.0},
                                  64, experts={'type': 'ffn', 'count_per_node': 4, 'hidden_size_per_expert': 96},
                                  seeds=(1, 2, 3), compress_name='int8', is_postscore=False,
                                  is_gshard_loss=False).to(DEV).train()
    x = torch.randn(4, 40, 64, device=DEV, requires_grad=True)
    y = layer(x)
    assert y.shape == x.shape and torch.isfinite(y).all() and torch.isfinite(y.l_aux)
    (y.pow(2).mean() + y.l_aux).backward()
    assert torch.isfinite(x.grad).all()
    wg = layer.gates[0].wg.weight.grad
    assert wg is not None and torch.isfinite(wg).all() and wg.abs().sum() > 0
