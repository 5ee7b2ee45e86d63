"""Seeded sweep over small random shapes: every stage of the path against the oracle, bit for bit
where the arithmetic is defined bit for bit.  Catches shape-dependent mistakes (ragged rows, one
token, top_k == experts, tiny capacities, alignment fall-backs) that the named cases miss."""
import numpy as np
import pytest
import torch

import oracle
from helpers import bf16_bits, from_bf16_bits, np_raw, raw, tie_free_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        E = int(rng.choice([1, 2, 3, 5, 8, 16, 17, 33, 64]))
        k = int(rng.integers(1, min(E, 4) + 1))
        T = int(rng.choice([1, 2, 63, 64, 65, 255, 257, 700]))
        M = int(rng.choice([8, 24, 72, 136, 520, 1000]))
        cf = float(rng.choice([0.25, 1.0, 2.0]))
        out.append((T, M, E, k, cf))
    return out


@pytest.mark.parametrize("T,M,E,k,cf", _shapes(24, 1))
def test_dispatch_codec_combine_bf16(T, M, E, k, cf):
    from planmoe_amd import ops
    scores = tie_free_scores(T, E, k, seed=T * 131 + E)
    r = ops.route_topk(scores.to(DEV), k, want_counts=True)
    idx, loc, gates, counts = oracle.route_topk(scores.numpy(), k)
    assert np.array_equal(r["indices"].cpu().numpy(), idx) and np.array_equal(r["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(r["gates"]), np_raw(gates)) and np.array_equal(r["counts"].cpu().numpy(), counts)
    C = ops.capacity(T, E, k, cf, 4)
    assert C == oracle.capacity(T, E, k, cf, 4)
    g = torch.Generator().manual_seed(M + T)
    x = torch.randn(T, M, generator=g).bfloat16()
    xd = x.to(DEV)
    i, l = list(r["indices"]), list(r["locations"])
    gt = [t.float() for t in r["gates"]]
    # dispatch, then the codec, against the oracle
    d = ops.dispatch_fwd(xd, i, l, None, E, C)
    want_d = torch.from_numpy(oracle.encode(x.float().numpy(), list(idx), list(loc), None, E, C)).bfloat16()
    assert np.array_equal(raw(d), raw(want_d))
    codes, bias, scale = ops.int8_compress(d)
    rc, rb, rs = oracle.int8_compress(bf16_bits(want_d))
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(raw(bias), np_raw(rb)) and np.array_equal(raw(scale), np_raw(rs))
    # the fused send side equals the two steps
    c2, b2, s2 = ops.dispatch_int8(xd, i, l, None, E, C)
    assert torch.equal(c2, codes) and np.array_equal(raw(b2), raw(bias)) and np.array_equal(raw(s2), raw(scale))
    # decompress + combine, stepwise and fused, against the oracle
    dec = ops.int8_decompress(codes, bias, scale)
    rd = oracle.int8_decompress(rc, rb, rs)
    assert np.array_equal(raw(dec), np_raw(rd))
    y = ops.combine_fwd(dec, i, l, gt, T, C)
    want_y = torch.from_numpy(oracle.decode(from_bf16_bits(rd).float().numpy(), list(idx), list(loc),
                                            [a.astype(np.float32) for a in gates], T, C)).bfloat16()
    assert np.array_equal(raw(y), raw(want_y))
    assert np.array_equal(raw(ops.combine_int8(codes, bias, scale, i, l, gt, T, C)), raw(want_y))


@pytest.mark.parametrize("T,M,E,k,cf", _shapes(16, 2))
def test_forward_entry_point(T, M, E, k, cf):
    """planmoe_forward_int8 on random shapes: routing against the oracle on the reported scores,
    codes against the stand-alone fused dispatch."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T * 7 + M)
    x = torch.randn(T, M, generator=g).bfloat16().to(DEV)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    C = ops.capacity(T, E, k, cf, 4)
    out = ops.forward_int8(x, wg, k, C, want_scores=True, want_counts=True)
    scores = out["scores"].cpu().numpy()
    idx, loc, gates, counts = oracle.route_topk(scores, k)        # (equal scores: the lower expert id, here as there)
    assert np.array_equal(out["indices"].cpu().numpy(), idx) and np.array_equal(out["locations"].cpu().numpy(), loc)
    assert np.array_equal(raw(out["gates"]), np_raw(gates)) and np.array_equal(out["counts"].cpu().numpy(), counts)
    c2, b2, s2 = ops.dispatch_int8(x, list(out["indices"]), list(out["locations"]), None, E, C)
    assert torch.equal(out["codes"].view(-1), c2.view(-1))
    assert np.array_equal(raw(out["bias"]).reshape(-1), raw(b2).reshape(-1))


@pytest.mark.parametrize("nx,ny,dims", [(4, 4, 2), (8, 4, 2), (4, 64, 2), (132, 8, 2), (1024, 12, 2), (4, 4, 1), (260, 4, 1), (4096, 4, 1)])
def test_zfp_random_fields(nx, ny, dims):
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(nx * 31 + ny)
    f = torch.randn(ny, nx, generator=g) * torch.exp(torch.randn(ny, 1, generator=g) * 4)
    f[0, :4] = 0
    stream = ops.zfp_compress(f.to(DEV), nx, ny, dims)
    n = ops.zfp_stream_bytes(dims, nx, ny)
    want = oracle.zfp_compress(f.numpy(), dims, 8.0)
    assert len(want) == n and np.array_equal(stream.cpu().numpy()[:n], want)
    dec = ops.zfp_decompress(stream, nx, ny, dims)
    assert np.array_equal(raw(dec), np_raw(oracle.zfp_decompress(want, ny, nx, dims, 8.0)))


@pytest.mark.parametrize("T,M,E,k,cf", _shapes(16, 3))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_and_backward_pieces(T, M, E, k, cf, dtype):
    """Gated dispatch, the gate gradient and the config-4 fusion on random shapes: fp32 results
    bit for bit against the oracle, bf16 against the stage-by-stage entry points."""
    from planmoe_amd import ops
    scores = tie_free_scores(T, E, k, seed=T * 17 + E)
    idx, loc, gates, _ = oracle.route_topk(scores.numpy(), k, normalize_gate=False)
    r = ops.route_topk(scores.to(DEV), k, normalize_gate=False)
    assert np.array_equal(r["locations"].cpu().numpy(), loc) and np.array_equal(raw(r["gates"]), np_raw(gates))
    C = ops.capacity(T, E, k, cf, 4)
    g = torch.Generator().manual_seed(M * 3 + T)
    x = torch.randn(T, M, generator=g).to(dtype)
    eo = torch.randn(E * C, M, generator=g).to(dtype)
    xd, eod = x.to(DEV), eo.to(DEV)
    i, l = list(r["indices"]), list(r["locations"])
    gt = [t.float() for t in r["gates"]]
    d = ops.dispatch_fwd(xd, i, l, gt, E, C)                      # gates applied at encode
    gg = ops.bwd_gate(xd, eod, i, l, C)
    if dtype == torch.float32:
        want = oracle.encode(x.numpy(), list(idx), list(loc), [a.astype(np.float32) for a in gates], E, C)
        assert np.array_equal(raw(d), want.view(np.int32))
        for j in range(k):
            w = oracle.bwd_gate(idx[j], loc[j], x.double().numpy(), eo.double().numpy(), C)
            scale = np.abs(x.double().numpy()).sum(1) * (np.abs(eo.numpy()).max() if eo.numel() else 0) + 1e-30
            assert (np.abs(gg[j].cpu().numpy() - w) <= 1e-5 * scale).all()
    # config-4 fusion == gated dispatch -> int8 compress, and its gate gradient == bwd_gate
    codes, bias, scale_, gg2 = ops.combine_bwd_int8(xd, eod, i, l, gt, E, C)
    c2, b2, s2 = ops.int8_compress(d)
    assert torch.equal(codes, c2) and np.array_equal(raw(bias), raw(b2)) and np.array_equal(raw(scale_), raw(s2))
    assert torch.equal(gg2, gg)


@pytest.mark.parametrize("seed", range(12))
def test_lz_random_buffers(seed):
    """GPULZ streams against the oracle on buffers of random size and texture: small alphabets
    (many matches of every length), runs, dense values, zeros of both signs, a ragged tail."""
    from planmoe_amd import ops
    rng = np.random.default_rng(100 + seed)
    nsym = int(rng.integers(1, 40 * 512))
    alphabet = int(rng.choice([1, 2, 3, 5, 17, 1000, 10 ** 6]))
    x = rng.integers(0, alphabet, size=nsym).astype(np.float32)
    for _ in range(int(rng.integers(0, 6))):                       # runs of one value
        a = int(rng.integers(0, nsym)); n = int(rng.integers(1, 700))
        x[a:a + n] = float(rng.choice([0.0, -0.0, 1.5, np.inf]))
    if seed % 3 == 0:
        x[rng.integers(0, nsym, size=5)] = np.nan
    padded = np.zeros((-(-nsym // 512) * 512,), np.float32)
    padded[:nsym] = x
    want = oracle.lz_compress(padded)
    xd = torch.from_numpy(x).to(DEV)
    got = ops.lz_compress(xd)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)
    out = torch.empty_like(xd)
    ops.lz_decompress(out, *got)
    ref = oracle.lz_decompress(*want)[:nsym]
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32))
