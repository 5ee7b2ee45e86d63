"""GPULZ ("lz") codec on the GPU against the CPU oracle: the four stream tensors byte for byte,
decoding of the oracle's streams, round trips, a ragged tail, and streams no coder wrote."""
import numpy as np
import pytest
import torch

import oracle
from planmoe_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def gpu_compress(x_np):
    x = torch.from_numpy(x_np).to(DEV)
    ws = torch.empty((max(int(_lib.lib.planmoe_lz_workspace_bytes(x_np.nbytes)), 16),), dtype=torch.uint8, device=DEV)
    return ops.lz_compress(x, workspace=ws)


def same_streams(got, want):
    for g, w, name in zip(got, want, ("flag_offsets", "data_offsets", "flags", "data")):
        g = g.cpu().numpy()
        assert g.shape == w.shape, name
        if not np.array_equal(g, w):
            bad = int(np.flatnonzero(g != w)[0])
            raise AssertionError("%s differs first at %d: %d != %d" % (name, bad, g[bad], w[bad]))


def check(x_np):
    x_np = np.ascontiguousarray(x_np, np.float32).reshape(-1)
    want = oracle.lz_compress(x_np)
    got = gpu_compress(x_np)
    same_streams(got, want)
    out = torch.full((x_np.size,), 7.0, dtype=torch.float32, device=DEV)
    ops.lz_decompress(out, *got)
    ref = oracle.lz_decompress(*want)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    return got


def distinct(n, start=1000.0):
    return (start + np.arange(n)).astype(np.float32)


def test_hand_worked_blocks():
    blocks = [np.full(512, 3.5, np.float32), distinct(512)]
    for prefix in ([1, 1, 2, 1, 2], [1, 2, 1, 3, 1, 4], [1, 2, 4, 1, 2, 3, 5, 1, 2, 3, 6],
                   [0.0, -0.0, float('nan'), float('nan')]):
        b = distinct(512)
        b[:len(prefix)] = prefix
        blocks.append(b)
    tail = distinct(512)
    tail[510:] = tail[508:510]
    blocks.append(tail)
    zeros = np.zeros(512, np.float32)
    zeros[0] = -0.0                                      # the literal keeps its sign, the copies lose it
    blocks += [zeros, np.full(512, np.nan, np.float32), np.full(512, np.inf, np.float32)]
    almost = np.full(512, 2.0, np.float32)
    almost[511] = 3.0                                    # one value short of the closed form
    blocks.append(almost)
    for b in blocks:
        check(b)
    check(np.concatenate(blocks))


@pytest.mark.parametrize("alphabet,nblocks,seed", [(2, 9, 0), (3, 64, 1), (8, 200, 2), (64, 1000, 3),
                                                   (100000, 777, 4)])
def test_random_alphabets(alphabet, nblocks, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, alphabet, size=nblocks * 512).astype(np.float32)
    check(x)


def test_dispatched_buffer_with_empty_slots():
    # what the codec sees in the layer: rows of activations, some capacity slots all zero
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4096, 1024)).astype(np.float32)
    x[rng.random(4096) < 0.3] = 0.0
    x[100, 17:900] = -0.0
    x[200, 5] = np.nan
    x[201, :] = np.inf
    fo, do, flags, data = check(x)
    assert int(do[-1]) < x.nbytes                        # the empty slots shrink


def test_many_blocks_and_scan_chunks():
    # 40 000 blocks: the offset tables span several chunks of the scan
    rng = np.random.default_rng(6)
    x = rng.integers(0, 5, size=40000 * 512).astype(np.float32)
    x[::3] += rng.standard_normal(x[::3].size).astype(np.float32)
    check(x)


def test_one_workspace_call_after_call():
    """What a call leaves in the workspace (class bytes, chunk totals) must not reach into the next:
    a long input, then shorter and different ones, on one workspace."""
    rng = np.random.default_rng(9)
    big = rng.integers(0, 3, size=5000 * 512).astype(np.float32)
    ws = torch.empty((int(_lib.lib.planmoe_lz_workspace_bytes(big.nbytes)),), dtype=torch.uint8, device=DEV)
    for x in (big, rng.standard_normal(700 * 512).astype(np.float32), np.zeros(2000 * 512, np.float32), big[::-1].copy()):
        got = ops.lz_compress(torch.from_numpy(x).to(DEV), workspace=ws)
        same_streams(got, oracle.lz_compress(x))


def test_config5_full_size():
    """The [16, 8192, 1024] fp32 buffer of config 5 (512 MiB, 262 144 blocks): a quarter of the
    capacity slots empty, some rows thinned out like an activation after a ReLU, the rest dense.
    All four stream tensors against the oracle, the decode against the input."""
    rng = np.random.default_rng(11)
    R, M = 16 * 8192, 1024
    x = rng.standard_normal((R, M), dtype=np.float32)
    kind = rng.random(R)
    x[kind < 0.25] = 0.0
    thin = (kind >= 0.25) & (kind < 0.35)
    x[thin] = np.maximum(x[thin], 0.0)
    want = oracle.lz_compress(x)
    xd = torch.from_numpy(x).to(DEV)
    got = ops.lz_compress(xd)
    same_streams(got, want)
    out = torch.empty_like(xd)
    ops.lz_decompress(out, *got)
    assert torch.equal(out.view(torch.int32), xd.view(torch.int32))      # no -0 and no NaN in this input
    assert int(got[1][-1]) < 0.8 * x.nbytes


def test_largest_input():
    """2^31 - 4096 bytes, the most the int32 offset tables can describe: nothing shrinks, so the last
    offsets sit right under 2^31.  Checked through what holds at any size: the tables are the
    prefix sums of a stored stream, the token bytes are the input, the decode gives it back."""
    nbytes = (1 << 31) - 4096
    x = torch.empty((nbytes // 4,), dtype=torch.float32, device=DEV)
    x.view(torch.int32).copy_(torch.arange(nbytes // 4, dtype=torch.int32, device=DEV))      # all symbols differ
    x.view(torch.int32).bitwise_and_(0x3fffffff)                                             # ... and none is a NaN
    fo, do, flags, data = ops.lz_compress(x)
    blocks = nbytes // 2048
    assert fo.numel() == blocks + 1 and int(fo[-1]) == blocks * 64 and int(do[-1]) == nbytes
    assert torch.equal(do, torch.arange(blocks + 1, dtype=torch.int64, device=DEV).mul_(2048).to(torch.int32))
    assert not flags.any()
    assert torch.equal(data.view(torch.int32), x.view(torch.int32))
    out = torch.empty_like(x)
    ops.lz_decompress(out, fo, do, flags, data)
    assert torch.equal(out.view(torch.int32), x.view(torch.int32))
    with pytest.raises(_lib.PlanMoEError, match="too large"):
        ops.lz_compress(torch.empty(((1 << 31) // 4,), dtype=torch.float32, device=DEV))


@pytest.mark.parametrize("nsym", [1, 8, 511, 513, 512 * 3 + 100, 512 * 17 - 1])
def test_ragged_tail(nsym):
    rng = np.random.default_rng(nsym)
    x = rng.integers(0, 4, size=nsym).astype(np.float32)
    padded = np.zeros((-(-nsym // 512) * 512,), np.float32)
    padded[:nsym] = x
    want = oracle.lz_compress(padded)                    # the tail block is coded as if zero-padded
    got = gpu_compress(x)
    same_streams(got, want)
    out = torch.full((nsym + 8,), 7.0, dtype=torch.float32, device=DEV)
    ops.lz_decompress(out[:nsym], *got)
    assert np.array_equal(out[:nsym].cpu().numpy(), x)
    assert np.all(out[nsym:].cpu().numpy() == 7.0)       # nothing written past the end


def test_empty():
    x = torch.empty((0,), dtype=torch.float32, device=DEV)
    fo, do, flags, data = ops.lz_compress(x)
    assert fo.tolist() == [0] and do.tolist() == [0] and flags.numel() == 0 and data.numel() == 0
    ops.lz_decompress(x, fo, do, flags, data)


def test_other_dtypes_are_taken_as_words():
    rng = np.random.default_rng(8)
    x = torch.from_numpy(rng.integers(0, 3, size=(64, 1024)).astype(np.float32)).to(DEV).bfloat16()
    got = ops.lz_compress(x)
    words = x.cpu().view(torch.int32).numpy().view(np.float32)
    same_streams(got, oracle.lz_compress(words))
    out = torch.empty_like(x)
    ops.lz_decompress(out, *got)
    assert torch.equal(out.view(torch.int16), x.view(torch.int16))


def test_foreign_streams_stay_in_bounds():
    # nothing a coder wrote: the decoder must neither fault nor touch memory outside `out`
    rng = np.random.default_rng(9)
    B = 300
    for kind in range(3):
        fo = rng.integers(-50, B * 64 + 50, size=B + 1).astype(np.int32)
        do = rng.integers(-50, B * 2048 + 50, size=B + 1).astype(np.int32)
        if kind == 1:
            fo, do = np.sort(fo), np.sort(do)
        if kind == 2:
            fo = (np.arange(B + 1) * 64).astype(np.int32)
            do = (np.arange(B + 1) * 1500).astype(np.int32)
        flags = rng.integers(0, 256, size=B * 64).astype(np.uint8)
        data = rng.integers(0, 256, size=B * 2048).astype(np.uint8)
        guard = torch.full((B * 512 + 1024,), 7.0, dtype=torch.float32, device=DEV)
        out = guard[512:512 + B * 512]
        ops.lz_decompress(out, *[torch.from_numpy(a).to(DEV) for a in (fo, do, flags, data)])
        torch.cuda.synchronize()
        g = guard.cpu().numpy()
        assert np.all(g[:512] == 7.0) and np.all(g[512 + B * 512:] == 7.0)
    check(np.full(1024, 2.0, np.float32))                # and the device still answers


def test_argument_errors():
    x = torch.zeros((1024,), dtype=torch.float32, device=DEV)
    with pytest.raises(_lib.PlanMoEError):
        ops.lz_compress(x, workspace=torch.empty((8,), dtype=torch.uint8, device=DEV))
    with pytest.raises(_lib.PlanMoEError):
        ops.lz_compress(torch.zeros((3,), dtype=torch.bfloat16, device=DEV))       # 6 bytes
    with pytest.raises(_lib.PlanMoEError):
        ops.lz_compress(torch.zeros((4,), dtype=torch.float32))                    # CPU tensor
