"""planmoe_ffn_fc1_int8: the experts' first GEMM straight from the int8 codes against the oracle's
decode followed by an fp64 matrix product (tolerance: rtol 1e-2 of bf16 outputs, the order of the
fp32 sums being the kernel's own), and against torch's batched GEMM on the decompressed tensor."""
import numpy as np
import pytest
import torch

import oracle
from helpers import bf16_bits, from_bf16_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("E,C,M,H,with_bias", [(2, 200, 256, 128, True), (3, 128, 64, 256, False), (1, 1, 512, 128, True),
                                               (4, 333, 1024, 384, True)])
def test_fc1_from_codes_against_the_oracle(E, C, M, H, with_bias):
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(E * 1000 + C)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    x[0, 0] = 0.0                                                    # an empty capacity slot: scale 0
    w = (torch.randn(E, H, M, generator=g) * M ** -0.5).bfloat16()
    fb = torch.randn(E, H, generator=g).bfloat16() if with_bias else None
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    got = ops.ffn_fc1_int8(codes, bias, scale, w.to(DEV), fb.to(DEV) if with_bias else None).float().cpu()
    rc, rb, rs = oracle.int8_compress(bf16_bits(x))
    assert np.array_equal(codes.cpu().numpy(), rc)
    dec = from_bf16_bits(oracle.int8_decompress(rc, rb, rs)).double()          # [E, C, M]
    ref = torch.einsum("ecm,ehm->ech", dec, w.double())
    mag = torch.einsum("ecm,ehm->ech", dec.abs(), w.double().abs())
    if with_bias:
        ref = ref + fb.double()[:, None, :]
        mag = mag + fb.double().abs()[:, None, :]
    # bf16 outputs: rtol 1e-2, plus the two bf16 roundings of sums whose terms may cancel (2^-8 of their magnitudes)
    assert ((got.double() - ref).abs() <= 1e-2 * ref.abs() + 2.0 ** -8 * mag + 1e-30).all()
    # and torch's own GEMM on the tensor the decompressor writes: same values up to summation order
    seen = ops.int8_decompress(codes, bias, scale)
    want = torch.matmul(seen, w.to(DEV).transpose(1, 2))
    if with_bias:
        want = want + fb.to(DEV)[:, None, :]
    assert torch.allclose(got, want.float().cpu(), rtol=2e-2, atol=float(mag.max()) * 2.0 ** -7)


def test_fc1_from_codes_config2_shape():
    """Config 2's receive side: 8 experts x 5120 slots x 4096, hidden 4096.  A sample of rows of every
    expert (tile edges included) against the oracle's decode and an fp64 product on the host."""
    from planmoe_amd import ops
    E, C, M, H = 8, 5120, 4096, 4096
    g = torch.Generator().manual_seed(1)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    w = (torch.randn(E, H, M, generator=g) * M ** -0.5).bfloat16()
    fb = torch.randn(E, H, generator=g).bfloat16()
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    got = ops.ffn_fc1_int8(codes, bias, scale, w.to(DEV), fb.to(DEV))
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 127, 128, 129, 2559, 2560, 4000, 5118, 5119])
    sample = got[:, rows].float().cpu().double()                      # [E, 10, H]
    rc, rb, rs = oracle.int8_compress(bf16_bits(x[:, rows].contiguous()))
    dec = from_bf16_bits(oracle.int8_decompress(rc, rb, rs)).double()
    ref = torch.einsum("ecm,ehm->ech", dec, w.double()) + fb.double()[:, None, :]
    mag = torch.einsum("ecm,ehm->ech", dec.abs(), w.double().abs()) + fb.double().abs()[:, None, :]
    assert ((sample - ref).abs() <= 1e-2 * ref.abs() + 2.0 ** -8 * mag).all()
    # every row was written: no row of the output is left as allocated
    assert bool(torch.isfinite(got.float()).all()) and float(got.float().abs().sum(dim=2).min()) > 0


def test_ffn_module_from_codes_equals_decompress_then_forward():
    """FusedExpertsNetwork.forward_from_codes against forward on the decompressed tensor (small
    shapes; bf16 tolerance), and the parameter shapes of the reference (ffn.py:33-56)."""
    import planmoe_amd
    from planmoe_amd import ops
    E, C, M, H = 4, 96, 256, 384
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2}, M,
                                  experts={'type': 'ffn', 'count_per_node': E, 'hidden_size_per_expert': H},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV).to(torch.bfloat16)
    ffn = layer.experts
    assert tuple(ffn.batched_fc1_w.shape) == (E, M, H) and tuple(ffn.batched_fc2_w.shape) == (E, H, M)
    assert tuple(ffn.batched_fc1_bias.shape) == (E, H) and tuple(ffn.batched_fc2_bias.shape) == (E, M)
    x = torch.randn(E, C, M, generator=torch.Generator().manual_seed(2)).bfloat16().to(DEV)
    codes, bias, scale = ops.int8_compress(x)
    with torch.no_grad():
        want = ffn(ops.int8_decompress(codes, bias, scale), layer)
        got = ffn.forward_from_codes(codes, bias, scale)
        got_exact = ffn.forward_from_codes(codes, bias, scale, exact=True)
    assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2 * float(want.float().abs().max()))
    assert torch.allclose(got_exact.float(), want.float(), rtol=2e-2, atol=2e-2 * float(want.float().abs().max()))


@pytest.mark.parametrize("E,C,M,H,with_bias", [(2, 200, 256, 128, True), (3, 256, 64, 512, False), (1, 1, 512, 256, True),
                                               (2, 700, 1024, 384, True)])
def test_fc1_affine_against_the_oracle(E, C, M, H, with_bias):
    """planmoe_ffn_fc1_int8_affine: codes on the matrix cores, scale / bias in the epilogue.  Against the
    oracle's decode + fp64 product with the same bf16 tolerance as the exact-decode kernel (the three
    roundings of the decompressor that it skips are of that size), and against that kernel."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(E * 1000 + C)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    x[0, 0] = 0.0
    w = (torch.randn(E, H, M, generator=g) * M ** -0.5).bfloat16()
    fb = torch.randn(E, H, generator=g).bfloat16() if with_bias else None
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    wd = w.to(DEV)
    got = ops.ffn_fc1_int8_affine(codes, bias, scale, wd, ops.ffn_weight_colsum(wd), fb.to(DEV) if with_bias else None).float().cpu()
    rc, rb, rs = oracle.int8_compress(bf16_bits(x))
    dec = from_bf16_bits(oracle.int8_decompress(rc, rb, rs)).double()
    ref = torch.einsum("ecm,ehm->ech", dec, w.double())
    mag = torch.einsum("ecm,ehm->ech", dec.abs(), w.double().abs())
    if with_bias:
        ref = ref + fb.double()[:, None, :]
        mag = mag + fb.double().abs()[:, None, :]
    assert ((got.double() - ref).abs() <= 1e-2 * ref.abs() + 2.0 ** -7 * mag + 1e-30).all()
    exact = ops.ffn_fc1_int8(codes, bias, scale, wd, fb.to(DEV) if with_bias else None).float().cpu()
    assert ((got - exact).abs().double() <= 1e-2 * ref.abs() + 2.0 ** -7 * mag + 1e-30).all()
    assert float((got[0, 0] - (fb[0].float() if with_bias else 0.0)).abs().max()) == 0.0     # the empty slot: bias only


def test_fc1_affine_gap_where_offsets_dwarf_ranges_and_weight_columns_cancel():
    """The case that separates the two forms: rows 100 + 2 N(0, 1) (bf16 spacing at 100 is 0.5, a code
    step 16 / 255) times weight columns that sum to zero, so the offset cancels and only the variation is
    left in the result.  The exact form stays at decompress + GEMM.  The affine form multiplies
    code / 255 * scale + bias without the decompressor's three roundings, so it differs by up to their
    share, 2^-8 of sum |w| |x| -- a bound in terms of the operands, not of the result: here more than a
    fifth of the outputs differ by over rtol 1e-2 of the result itself, which is why the layer takes
    the exact form unless told otherwise."""
    from planmoe_amd import ops
    E, C, M, H = 2, 128, 512, 128
    g = torch.Generator().manual_seed(7)
    x = (100.0 + 2.0 * torch.randn(E, C, M, generator=g)).bfloat16()
    half = (torch.randn(E, H, M // 2, generator=g) * M ** -0.5).bfloat16()
    w = torch.cat([half, -half], dim=2).contiguous()                   # every column of every expert sums to 0
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    wd = w.to(DEV)
    exact = ops.ffn_fc1_int8(codes, bias, scale, wd, None).float().cpu().double()
    affine = ops.ffn_fc1_int8_affine(codes, bias, scale, wd, ops.ffn_weight_colsum(wd), None).float().cpu().double()
    rc, rb, rs = oracle.int8_compress(bf16_bits(x))
    assert np.array_equal(codes.cpu().numpy(), rc)
    dec = from_bf16_bits(oracle.int8_decompress(rc, rb, rs)).double()
    ref = torch.einsum("ecm,ehm->ech", dec, w.double())
    mag = torch.einsum("ecm,ehm->ech", dec.abs(), w.double().abs())
    # exact form: the decompressor's values, fp32 sums (512 terms: 2^-15 mag at worst) and one bf16 rounding
    assert ((exact - ref).abs() <= 2.0 ** -8 * ref.abs() + 2.0 ** -14 * mag).all()
    # affine form: within the skipped roundings of the exact one ...
    gap = (affine - exact).abs()
    assert (gap <= 1.05 * 2.0 ** -8 * mag + 2.0 ** -7 * ref.abs()).all()
    # ... and that is not "an ulp of the result" here
    assert float((gap > 1e-2 * ref.abs()).double().mean()) > 0.2


def test_fc1_affine_config2_shape():
    from planmoe_amd import ops
    E, C, M, H = 8, 5120, 4096, 4096
    g = torch.Generator().manual_seed(1)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    w = (torch.randn(E, H, M, generator=g) * M ** -0.5).bfloat16()
    fb = torch.randn(E, H, generator=g).bfloat16()
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    wd = w.to(DEV)
    got = ops.ffn_fc1_int8_affine(codes, bias, scale, wd, None, fb.to(DEV))
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 2559, 2560, 4000, 5118, 5119])
    sample = got[:, rows].float().cpu().double()
    rc, rb, rs = oracle.int8_compress(bf16_bits(x[:, rows].contiguous()))
    dec = from_bf16_bits(oracle.int8_decompress(rc, rb, rs)).double()
    ref = torch.einsum("ecm,ehm->ech", dec, w.double()) + fb.double()[:, None, :]
    mag = torch.einsum("ecm,ehm->ech", dec.abs(), w.double().abs()) + fb.double().abs()[:, None, :]
    assert ((sample - ref).abs() <= 1e-2 * ref.abs() + 2.0 ** -7 * mag).all()
    assert bool(torch.isfinite(got.float()).all()) and float(got.float().abs().sum(dim=2).min()) > 0


def test_layer_inference_feeds_the_codes_to_the_experts(monkeypatch):
    """moe_layer under no_grad with the built-in FFN in bf16 and the int8 compressor: the receive
    side skips the decompress (experts.forward_from_codes is called) and the output agrees with the
    layer that decompresses first, to bf16 tolerance; with autograd on the usual path runs."""
    import planmoe_amd
    from planmoe_amd import overlap, experts
    T, M, E, H = 1024, 256, 4, 384
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'capacity_factor': 1.25}, M,
                                  experts={'type': 'ffn', 'count_per_node': E, 'hidden_size_per_expert': H},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV).to(torch.bfloat16)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(5)).bfloat16().to(DEV)
    monkeypatch.setattr(overlap, "FFN_FROM_CODES", True)
    calls = []
    real = experts.FusedExpertsNetwork.forward_from_codes

    def spy(self, *a, **kw):
        calls.append(1)
        return real(self, *a, **kw)
    monkeypatch.setattr(experts.FusedExpertsNetwork, "forward_from_codes", spy)
    with torch.no_grad():
        got = layer(x)
        assert len(calls) == 1
        monkeypatch.setattr(overlap, "FFN_FROM_CODES", False)
        want = layer(x)
        assert len(calls) == 1
    assert torch.allclose(got.float(), want.float(), rtol=3e-2, atol=3e-2 * float(want.float().abs().max()))
    monkeypatch.setattr(overlap, "FFN_FROM_CODES", True)
    y = layer(x.clone().requires_grad_(True))                     # autograd on: the training path
    assert len(calls) == 1 and y.requires_grad
    for fuse_gate in (False,):                                    # and the path with a separate gate + routing
        monkeypatch.setattr(overlap, "FUSE_GATE", fuse_gate)
        with torch.no_grad():
            got2 = layer(x)
        assert len(calls) == 2
        assert torch.allclose(got2.float(), want.float(), rtol=3e-2, atol=3e-2 * float(want.float().abs().max()))


def _ffn(E, M, H, seed=0):
    import types
    from planmoe_amd.experts import FusedExpertsNetwork
    torch.manual_seed(seed)
    net = FusedExpertsNetwork(H)
    net.update(types.SimpleNamespace(model_dim=M, num_local_experts=E))
    return net


@pytest.mark.parametrize("E,C,M,H", [(2, 200, 256, 384), (3, 64, 64, 128), (1, 517, 136, 72)])
def test_ffn_forward_and_backward_through_the_gemm_kernel(E, C, M, H):
    """FusedExpertsNetwork in bf16 on the GPU (both GEMMs and their four gradients through
    planmoe_gemm_nt_bf16 / planmoe_transpose_bf16) against the same network in fp64 on the host with
    the same bf16 parameters: experts/ffn.py:63-82 and its autograd."""
    net = _ffn(E, M, H, seed=E + C).bfloat16()
    ref = _ffn(E, M, H, seed=E + C)
    ref.load_state_dict({k: v.double() for k, v in net.state_dict().items()})
    ref = ref.double()
    g = torch.Generator().manual_seed(C)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    gy = torch.randn(E, C, M, generator=g).bfloat16()
    dev = net.to(DEV)
    xd = x.to(DEV).requires_grad_(True)
    y = dev(xd, None)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    xr = x.double().requires_grad_(True)
    yr = ref(xr, None)
    yr.backward(gy.double())

    def close(got, want, scale):
        # bf16 tolerance element by element for all but a sliver (a hidden unit within rounding of zero
        # passes relu on one side and not on the other: its whole term differs), and in the norm
        got, want = got.detach().double().cpu(), want.detach()
        ok = (got - want).abs() <= 2e-2 * want.abs() + 2e-2 * scale
        return float(ok.double().mean()) > 0.97 and float((got - want).norm() / want.norm()) < 3e-2
    assert close(y, yr, float(yr.detach().abs().mean()))
    assert close(xd.grad, xr.grad, float(xr.grad.abs().mean()))
    for name in ("batched_fc1_w", "batched_fc2_w", "batched_fc1_bias", "batched_fc2_bias"):
        got, want = getattr(dev, name).grad, getattr(ref, name).grad
        assert got is not None and close(got, want, float(want.abs().mean())), name
    # the weight forms are made again when the weights change
    with torch.no_grad():
        dev.batched_fc1_w.mul_(2.0)
        ref.batched_fc1_w.mul_(2.0)
        assert close(dev(x.to(DEV), None), ref(x.double(), None), float(yr.detach().abs().mean()))


def test_ffn_config2_size_forward_and_backward():
    """The built-in FFN at config 2's receive buffer with hidden 4096 (8 x [5120, 4096] -> 4096 -> 4096),
    forward and backward, no library GEMM involved.  Checked on samples against fp64 on the host:
    output rows and input-gradient rows of every expert, entries of both weight gradients, the biases'."""
    E, C, M, H = 8, 5120, 4096, 4096
    net = _ffn(E, M, H, seed=1).bfloat16().to(DEV)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(E, C, M, generator=g).bfloat16()
    gy = (torch.randn(E, C, M, generator=g) * 0.1).bfloat16()
    xd = x.to(DEV).requires_grad_(True)
    y = net(xd, None)
    y.backward(gy.to(DEV))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all()) and bool(torch.isfinite(xd.grad.float()).all())
    w1, w2 = net.batched_fc1_w.detach().cpu().double(), net.batched_fc2_w.detach().cpu().double()
    b1, b2 = net.batched_fc1_bias.detach().cpu().double(), net.batched_fc2_bias.detach().cpu().double()
    rows = torch.tensor([0, 255, 256, 2560, 5119])

    def close(got, want, scale):
        ok = (got.double().cpu() - want).abs() <= 2e-2 * want.abs() + 3e-2 * scale
        return float(ok.double().mean()) > 0.9 and float((got.double().cpu() - want).norm() / want.norm()) < 3e-2
    for e in (0, 3, 7):
        h1 = x[e, rows].double() @ w1[e] + b1[e]
        a = h1.clamp(min=0)
        yr = a @ w2[e] + b2[e]
        assert close(y[e, rows], yr, float(yr.abs().mean())), e
        da = gy[e, rows].double() @ w2[e].t()
        dxr = (da * (h1 > 0)) @ w1[e].t()
        assert close(xd.grad[e, rows], dxr, float(dxr.abs().mean())), e
        # weight gradients: all rows reduce into every entry; a few columns of each
        hs, ms = torch.tensor([0, 1, 2047, 4095]), torch.tensor([0, 5, 4094, 4095])
        h1_all = x[e].double() @ w1[e][:, hs] + b1[e][hs]                       # [C, 4]
        a_all = h1_all.clamp(min=0)
        dw2 = a_all.t() @ gy[e].double()[:, ms]                                 # [4, 4]
        assert close(net.batched_fc2_w.grad[e][hs][:, ms], dw2, float(dw2.abs().mean())), e
        da_all = gy[e].double() @ w2[e][hs].t()                                 # [C, 4]
        dh1 = da_all * (h1_all > 0)
        dw1 = x[e].double()[:, ms].t() @ dh1                                    # [4 (m), 4 (h)]
        assert close(net.batched_fc1_w.grad[e][ms][:, hs], dw1, float(dw1.abs().mean())), e
        assert close(net.batched_fc1_bias.grad[e][hs], dh1.sum(0), float(dh1.sum(0).abs().mean())), e
        db2 = gy[e].double().sum(0)[ms]
        assert close(net.batched_fc2_bias.grad[e][ms], db2, float(db2.abs().mean()) + 1e-3), e


def test_layer_with_the_builtin_ffn_at_config2_size():
    """moe_layer, int8 compressor, built-in FFN, 16384 tokens x 4096, 8 experts, hidden 4096: a forward
    and backward pass end to end.  The experts' part is checked by the tests above; here the layer
    must run at this size (no library GEMM at it), give finite results and gradients everywhere."""
    import planmoe_amd
    T, M, E, H = 16384, 4096, 8, 4096
    layer = planmoe_amd.moe_layer({'type': 'top', 'k': 2, 'capacity_factor': 1.25, 'fp32_gate': True}, M,
                                  experts={'type': 'ffn', 'count_per_node': E, 'hidden_size_per_expert': H},
                                  seeds=(1, 2, 3), compress_name='int8').to(DEV).to(torch.bfloat16)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(0)).bfloat16().to(DEV).requires_grad_(True)
    y = layer(x)
    (y.float().square().mean() + y.l_aux.float()).backward()
    torch.cuda.synchronize()
    assert y.shape == (T, M) and bool(torch.isfinite(y.float()).all())
    assert bool(torch.isfinite(x.grad.float()).all()) and float(x.grad.float().abs().sum()) > 0
    for p_ in layer.parameters():
        assert p_.grad is not None and bool(torch.isfinite(p_.grad.float()).all())
    with torch.no_grad():
        y2 = layer(x)
    assert torch.allclose(y2.float(), y.detach().float(), rtol=2e-2, atol=2e-2 * float(y.detach().float().abs().max()))
