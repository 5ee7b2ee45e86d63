"""Pins of the int8 part of the CPU oracle: the literal torch-CPU op chain in the tensor dtype."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import bf16_bits, from_bf16_bits, np_raw


def torch_chain(x):
    """min / max / sub / sub / div / mul 255 / to(uint8), then the decode chain: library ops
    applied in the order of the reference's compressor."""
    bias = torch.min(x, -1, True)[0]
    scale = torch.sub(torch.max(x, -1, True)[0], bias)
    q = torch.mul(torch.div(torch.sub(x, bias), scale), 255.0)
    codes = q.to(torch.uint8)
    dec = torch.add(torch.mul(torch.div(codes.to(x.dtype), 255.0), scale), bias)
    return codes, bias, scale, dec


@pytest.mark.parametrize("name", ["int8_f32", "int8_bf16"])
def test_golden(torch_golden, name):
    c = case(torch_golden, name)
    codes, bias, scale = oracle.int8_compress(c["x"])
    assert np.array_equal(codes, c["codes"])
    assert np.array_equal(np_raw(bias), np_raw(c["bias"]))
    assert np.array_equal(np_raw(scale), np_raw(c["scale"]))
    dec = oracle.int8_decompress(codes, bias, scale)
    assert np.array_equal(np_raw(dec), np_raw(c["decoded"]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_against_live_torch_chain(dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(64, 512, generator=g) * (10.0 ** torch.randint(-3, 4, (64, 1), generator=g).float())).to(dtype)
    x[5] = 0
    x[6] = -2.25
    codes_t, bias_t, scale_t, dec_t = torch_chain(x)
    xn = bf16_bits(x) if dtype == torch.bfloat16 else x.numpy()
    codes, bias, scale = oracle.int8_compress(xn)
    assert np.array_equal(codes, codes_t.numpy())
    conv = bf16_bits if dtype == torch.bfloat16 else (lambda t: t.numpy())
    assert np.array_equal(np_raw(bias), np_raw(conv(bias_t)))
    assert np.array_equal(np_raw(scale), np_raw(conv(scale_t)))
    assert np.array_equal(np_raw(oracle.int8_decompress(codes, bias, scale)), np_raw(conv(dec_t)))


def test_exhaustive_bf16_values_for_fixed_ranges():
    """Every finite bf16 value inside [lo, hi] placed in one row with fixed extremes."""
    allv = from_bf16_bits(np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)).float()
    for lo, hi in ((-1.0, 1.0), (0.0, 3.140625), (-250.0, 7.5), (1.0, 1.0078125)):
        vals = allv[torch.isfinite(allv) & (allv >= lo) & (allv <= hi)]
        vals = vals[vals != 0] if lo < 0 < hi else vals          # keep a single zero sign
        row = torch.cat([torch.tensor([lo, hi]), vals]).to(torch.bfloat16)[None, :]
        codes_t, bias_t, scale_t, dec_t = torch_chain(row)
        codes, bias, scale = oracle.int8_compress(bf16_bits(row))
        assert np.array_equal(codes, codes_t.numpy()), (lo, hi)
        assert np.array_equal(oracle.int8_decompress(codes, bias, scale).view(np.int16),
                              bf16_bits(dec_t).view(np.int16))


def test_invariants():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((32, 200)).astype(np.float32) * 5
    codes, bias, scale = oracle.int8_compress(x)
    rows = np.arange(32)
    assert (codes[rows, x.argmin(1)] == 0).all()           # row minimum -> 0
    assert (codes[rows, x.argmax(1)] == 255).all()         # row maximum -> 255
    order = np.argsort(x, axis=1)
    assert (np.diff(np.take_along_axis(codes.astype(np.int32), order, 1), axis=1) >= 0).all()   # monotone
    dec = oracle.int8_decompress(codes, bias, scale)
    assert (np.abs(dec - x) <= scale / 255.0 * 1.001).all()
    const = np.full((2, 16), 3.25, np.float32)
    c2, b2, s2 = oracle.int8_compress(const)
    assert (c2 == 0).all() and (s2 == 0).all() and (b2 == 3.25).all()
    assert (oracle.int8_decompress(c2, b2, s2) == 3.25).all()


def test_nan_row_like_torch():
    x = torch.randn(2, 32, generator=torch.Generator().manual_seed(82))
    x[1, 7] = float("nan")
    codes_t, bias_t, scale_t, _ = torch_chain(x)
    codes, bias, scale = oracle.int8_compress(x.numpy())
    assert np.array_equal(codes[0], codes_t.numpy()[0])
    assert np.isnan(bias[1]).all() and np.isnan(scale[1]).all() and np.isnan(bias_t.numpy()[1]).all()
    assert (codes[1] == 0).all()
