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
