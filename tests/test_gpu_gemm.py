"""planmoe_gemm_nt_bf16 / planmoe_transpose_bf16: the batched bf16 products of the expert FFN
(experts/ffn.py:63-82) against an fp64 product of the same bf16 operands on the host.  A GEMM's
parity is tolerance-level: rtol 1e-2 of the bf16 result plus the bf16 roundings of sums whose terms
may cancel (2^-8 of the sum of their magnitudes); the order of the fp32 sums is the kernel's own."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(got, a, b, bias, relu):
    ref = torch.einsum("bmk,bnk->bmn", a.double(), b.double().expand(a.shape[0], -1, -1))
    mag = torch.einsum("bmk,bnk->bmn", a.double().abs(), b.double().abs().expand(a.shape[0], -1, -1))
    if bias is not None:
        ref = ref + bias.double()[:, None, :]
        mag = mag + bias.double().abs()[:, None, :]
    tol = 1e-2 * ref.abs() + 2.0 ** -7 * mag + 1e-30
    if relu:
        # an output within tol of zero may land on either side of the cut
        ok = ((got.double() - ref.clamp(min=0)).abs() <= tol)
    else:
        ok = (got.double() - ref).abs() <= tol
    assert bool(ok.all()), float((got.double() - ref).abs().max())


@pytest.mark.parametrize("B,m,n,k,with_bias,relu,shared_b", [
    (2, 200, 136, 72, True, False, False), (3, 300, 264, 128, False, False, False), (1, 1, 8, 8, True, True, False),
    (2, 513, 520, 200, True, True, False), (1, 256, 256, 64, False, False, False), (4, 130, 24, 1032, True, False, True),
    (2, 700, 512, 640, False, True, False),
    # more than 8 tile columns, not a multiple of 8, tile count not a multiple of 8: panels of 8 + 2 and 8 + 1
    # columns, an XCD's stretch of the tiles crossing batches, surplus work-groups
    (3, 700, 2312, 64, True, True, False), (5, 520, 2056, 128, False, False, True)])
def test_gemm_against_an_fp64_product(B, m, n, k, with_bias, relu, shared_b):
    from planmoe_amd import ops
    print("case", B, m, n, k, with_bias, relu, shared_b, flush=True)
    g = torch.Generator().manual_seed(B * 7 + m + n + k)
    a = torch.randn(B, m, k, generator=g).bfloat16()
    b = (torch.randn(1 if shared_b else B, n, k, generator=g) * k ** -0.5).bfloat16()
    bias = torch.randn(B, n, generator=g).bfloat16() if with_bias else None
    got = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV), bias.to(DEV) if with_bias else None, relu=relu)
    torch.cuda.synchronize()
    assert got.shape == (B, m, n) and got.dtype == torch.bfloat16
    _check(got.float().cpu(), a, b, bias, relu)


def test_gemm_matches_the_two_roundings_of_matmul_plus_add():
    """torch.add(torch.matmul(x, w), bias) in bf16 rounds the product, then the sum: with operands
    whose products are exact small integers the kernel's result is that, bit for bit."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(5)
    a = torch.randint(-3, 4, (2, 96, 64), generator=g).bfloat16()
    b = torch.randint(-3, 4, (2, 40, 64), generator=g).bfloat16()
    bias = (torch.randint(-5, 6, (2, 40), generator=g).float() + 0.3).bfloat16()
    got = ops.gemm_nt_bf16(a.to(DEV), b.to(DEV), bias.to(DEV)).cpu()
    want = torch.add(torch.matmul(a.float(), b.float().transpose(1, 2)).bfloat16(), bias.unsqueeze(1))
    assert torch.equal(got, want)


@pytest.mark.parametrize("B,R,C,pad", [(2, 100, 72, 1), (1, 64, 64, 64), (3, 5, 8, 64), (2, 333, 136, 8), (1, 1, 4096, 64)])
def test_transpose_with_zero_padding(B, R, C, pad):
    from planmoe_amd import ops
    x = torch.randn(B, R, C, generator=torch.Generator().manual_seed(R + C)).bfloat16().to(DEV)
    got = ops.transpose_bf16(x, pad)
    torch.cuda.synchronize()
    step = max(8, pad)
    Ro = (R + step - 1) // step * step
    assert got.shape == (B, C, Ro)
    assert torch.equal(got[:, :, :R], x.transpose(1, 2))
    assert bool((got[:, :, R:] == 0).all())


def test_gemm_config2_ffn_shape():
    """The expert FFN of config 2 with hidden 4096: 8 x [5120, 4096] x [4096, 4096]^T.  Sampled rows of
    every expert (tile edges included) against an fp64 product on the host."""
    from planmoe_amd import ops
    E, C, M, H = 8, 5120, 4096, 4096
    g = torch.Generator().manual_seed(2)
    a = torch.randn(E, C, M, generator=g).bfloat16()
    w = (torch.randn(E, H, M, generator=g) * M ** -0.5).bfloat16()
    bias = torch.randn(E, H, generator=g).bfloat16()
    got = ops.gemm_nt_bf16(a.to(DEV), w.to(DEV), bias.to(DEV), relu=True)
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 31, 32, 127, 128, 255, 256, 257, 2559, 2560, 4000, 5118, 5119])
    _check(got[:, rows].float().cpu(), a[:, rows], w, bias, True)
    assert bool(torch.isfinite(got.float()).all())


@pytest.mark.parametrize("B,k,m,n", [(1, 64, 8, 8), (2, 128, 256, 256), (3, 192, 264, 520), (2, 640, 1000, 136),
                                     (3, 64, 696, 2312), (1, 4096, 72, 200)])
def test_gemm_tn_equals_the_nt_form_on_transposed_copies(B, k, m, n):
    """c = a^T b with the operands as they lie (reduction index slow) against planmoe_gemm_nt_bf16 on
    transposed copies: same products, same order of the fp32 sums, hence the same bits; and against fp64."""
    from planmoe_amd import ops
    print("case", B, k, m, n, flush=True)
    g = torch.Generator().manual_seed(B + k + m + n)
    a = torch.randn(B, k, m, generator=g).bfloat16()
    b = (torch.randn(B, k, n, generator=g) * k ** -0.5).bfloat16()
    got = ops.gemm_tn_bf16(a.to(DEV), b.to(DEV))
    want = ops.gemm_nt_bf16(ops.transpose_bf16(a.to(DEV), 64), ops.transpose_bf16(b.to(DEV), 64))
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    ref = torch.einsum("bkm,bkn->bmn", a.double(), b.double())
    mag = torch.einsum("bkm,bkn->bmn", a.double().abs(), b.double().abs())
    assert ((got.double().cpu() - ref).abs() <= 2.0 ** -8 * ref.abs() + 2.0 ** -14 * mag + 1e-30).all()


@pytest.mark.parametrize("B,m,k,n,with_bias,relu", [(1, 8, 64, 8, True, False), (2, 300, 128, 264, False, True),
                                                    (3, 513, 192, 2312, True, True), (2, 1, 4096, 136, True, False)])
def test_gemm_nn_equals_the_nt_form_on_a_transposed_weight(B, m, k, n, with_bias, relu):
    """c = act(a w + bias) with the weight as the experts store it, [k, n], against planmoe_gemm_nt_bf16 on its
    transposed copy: the same bits."""
    from planmoe_amd import ops
    print("case", B, m, k, n, with_bias, relu, flush=True)
    g = torch.Generator().manual_seed(B + m + k + n)
    a = torch.randn(B, m, k, generator=g).bfloat16().to(DEV)
    w = (torch.randn(B, k, n, generator=g) * k ** -0.5).bfloat16().to(DEV)
    bias = torch.randn(B, n, generator=g).bfloat16().to(DEV) if with_bias else None
    got = ops.gemm_nn_bf16(a, w, bias, relu=relu)
    want = ops.gemm_nt_bf16(a, ops.transpose_bf16(w), bias, relu=relu)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
