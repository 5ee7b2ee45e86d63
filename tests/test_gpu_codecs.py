"""GPU parity: the int8 codec (stand-alone and fused with dispatch) and the zfp fixed-rate
codec, bit-exact against the CPU oracle and the committed golden fixtures."""
import numpy as np
import pytest
import torch

import oracle
from conftest import case
from helpers import bf16_bits, from_bf16_bits, np_raw, raw, tie_free_scores, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ------------------------------------------------------------------------------ int8
@pytest.mark.parametrize("name", ["int8_f32", "int8_bf16"])
def test_int8_golden_fixtures(torch_golden, name):
    from planmoe_amd import ops
    c = case(torch_golden, name)
    x = from_bf16_bits(c["x"]) if c["x"].dtype == np.uint16 else torch.from_numpy(c["x"])
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    assert np.array_equal(codes.cpu().numpy(), c["codes"])
    assert np.array_equal(raw(bias), np_raw(c["bias"])) and np.array_equal(raw(scale), np_raw(c["scale"]))
    dec = ops.int8_decompress(codes, bias, scale)
    assert np.array_equal(raw(dec), np_raw(c["decoded"]))


@pytest.mark.parametrize("R,M,dtype", [(100, 4096, torch.bfloat16), (100, 2048, torch.float32), (33, 100, torch.float32),
                                       (33, 1001, torch.bfloat16), (10, 20000, torch.bfloat16), (7, 8, torch.bfloat16),
                                       (1, 1, torch.float32), (64, 512, torch.float16), (5, 16384, torch.float32)])
def test_int8_against_oracle(R, M, dtype):
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(R * 7 + M)
    x = (torch.randn(R, M, generator=g) * (10.0 ** torch.randint(-2, 3, (R, 1), generator=g).float())).to(dtype)
    x[0] = 0
    if R > 1:
        x[1] = 1.5
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    if dtype == torch.float16:
        # the oracle has no fp16 mode: compare with the literal torch-CPU chain instead
        b = torch.min(x, -1, True)[0]; s = torch.max(x, -1, True)[0] - b
        want = torch.mul(torch.div(torch.sub(x, b), s), 255.0).to(torch.uint8)
        assert np.array_equal(codes.cpu().numpy(), want.numpy())
        dec = torch.add(torch.mul(torch.div(want.to(dtype), 255.0), s), b)
        assert np.array_equal(raw(ops.int8_decompress(codes, bias, scale)), raw(dec))
        return
    rc, rb, rs = oracle.int8_compress(to_np(x))
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(raw(bias), np_raw(rb)) and np.array_equal(raw(scale), np_raw(rs))
    dec = ops.int8_decompress(codes, bias, scale)
    assert np.array_equal(raw(dec), np_raw(oracle.int8_decompress(rc, rb, rs)))
    assert (codes[0] == 0).all()                                  # empty slot: 0/0 -> code 0 -> decodes to 0
    assert (dec[0] == 0).all()


def test_int8_exhaustive_bf16():
    from planmoe_amd import ops
    allv = from_bf16_bits(np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)).float()
    for lo, hi in ((-1.0, 1.0), (0.0, 3.140625), (-250.0, 7.5), (0.0, 1.9921875), (-0.5, 0.5078125),
                   (-3.0517578125e-05, 2.2172927856445312e-05), (-1e20, 3e20), (0.33203125, 5.03125)):
        vals = allv[torch.isfinite(allv) & (allv >= lo) & (allv <= hi) & (allv != 0)]
        row = torch.cat([torch.tensor([lo, hi, 0.0]), vals])
        row = torch.cat([row, row.new_full(((-len(row)) % 8,), lo)]).to(torch.bfloat16)[None, :]
        codes, bias, scale = ops.int8_compress(row.to(DEV))
        rc, rb, rs = oracle.int8_compress(bf16_bits(row))
        assert np.array_equal(codes.cpu().numpy(), rc)
        assert np.array_equal(raw(ops.int8_decompress(codes, bias, scale)), np_raw(oracle.int8_decompress(rc, rb, rs)))


def test_int8_nan_row():
    from planmoe_amd import ops
    x = torch.randn(2, 64, generator=torch.Generator().manual_seed(72))
    x[1, 9] = float("nan")
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    rc, rb, rs = oracle.int8_compress(x.numpy())
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert torch.isnan(bias[1]).all() and torch.isnan(scale[1]).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("M", [64, 4096, 37])
def test_int8_rows_without_a_usable_scale(dtype, M):
    """Rows whose scale is 0, infinite or NaN (all codes 0) next to rows whose scale is merely
    extreme (IEEE division), against the literal torch-CPU op chain and the oracle."""
    from planmoe_amd import ops
    big = {torch.bfloat16: 3e38, torch.float32: 3e38, torch.float16: 6e4}[dtype]
    tiny = {torch.bfloat16: 2.0 ** -120, torch.float32: 2.0 ** -120, torch.float16: 2.0 ** -20}[dtype]
    x = torch.randn(12, M, generator=torch.Generator().manual_seed(M)).to(dtype)
    x[0] = 2.5                                             # constant
    x[1] = 0.0; x[1, ::2] = -0.0                           # +0 / -0
    x[2, 3] = float("inf")
    x[3, 5] = float("-inf")
    x[4] = float("inf")
    x[5] = float("-inf")
    x[6, 0] = big; x[6, 1] = -big                          # max - min overflows
    x[7, 7] = float("nan")
    x[8, 1] = float("inf"); x[8, 2] = float("-inf")
    g9 = torch.Generator().manual_seed(M + 1)
    x[9] = (torch.randn(M, generator=g9) * tiny).to(dtype)                          # tiny but usable scale
    x[10] = (torch.randn(M, generator=g9).clamp(-3, 3) * (big / 8)).to(dtype)       # huge but finite scale (|x| <= 3/8 big)
    codes, bias, scale = ops.int8_compress(x.to(DEV))
    b = torch.min(x, -1, True)[0]; sc = torch.max(x, -1, True)[0] - b
    want = torch.mul(torch.div(torch.sub(x, b), sc), 255.0).to(torch.uint8)
    usable = (sc.view(-1) > 0) & torch.isfinite(sc.view(-1))
    assert usable.tolist() == [False] * 9 + [True] * 3
    # float -> uint8 of NaN is not defined by torch; every backend here gives 0, the oracle pins 0
    want[~usable] = 0
    assert np.array_equal(codes.cpu().numpy(), want.numpy())

    def same(got, ref):                                    # bit for bit, any NaN for a NaN (inf - inf has no fixed sign)
        got, ref = got.cpu().view(-1), ref.view(-1)
        nan = torch.isnan(ref)
        return torch.equal(torch.isnan(got), nan) and np.array_equal(raw(got[~nan]), raw(ref[~nan]))
    assert same(bias, b) and same(scale, sc)
    if dtype != torch.float16:
        rc, rb, rs = oracle.int8_compress(to_np(x))
        assert np.array_equal(codes.cpu().numpy(), rc)


def test_int8_config2_full_size():
    """[8, 5120, 4096] bf16: codes checked on a row sample against the oracle, everything through
    invariants (row min -> 0, row max -> 255, |decode - x| <= scale/255 + bf16 rounding)."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(0)
    x = torch.randn(8 * 5120, 4096, generator=g).bfloat16()
    x[::5] = 0                                                     # empty capacity slots
    xd = x.to(DEV)
    codes, bias, scale = ops.int8_compress(xd)
    rows = torch.arange(0, x.size(0), 37)
    rc, rb, rs = oracle.int8_compress(bf16_bits(x[rows]))
    assert np.array_equal(codes[rows.to(DEV)].cpu().numpy(), rc)
    assert np.array_equal(raw(bias[rows.to(DEV)]), np_raw(rb))
    assert torch.equal(bias.view(-1), xd.amin(1)) and torch.equal(scale.view(-1), (xd.amax(1) - xd.amin(1)))
    live = scale.view(-1) > 0
    assert (codes.amin(1)[live] == 0).all() and (codes.amax(1)[live] == 255).all()
    dec = ops.int8_decompress(codes, bias, scale)
    err = (dec.float() - xd.float()).abs()
    bound = scale.float() / 255.0 + 2.0 ** -7 * (xd.float().abs() + scale.float())
    assert (err <= bound).all()


@pytest.mark.parametrize("T,M,E,k,cf,dtype", [(513, 4096, 8, 2, 1.25, torch.bfloat16), (300, 1024, 16, 3, 0.5, torch.bfloat16),
                                              (100, 2048, 2, 2, 1.0, torch.float32), (64, 64, 4, 1, 1.0, torch.float32),
                                              (50, 20000, 4, 2, 1.0, torch.bfloat16)])
def test_dispatch_int8_equals_dispatch_then_compress(T, M, E, k, cf, dtype):
    from planmoe_amd import ops
    scores = tie_free_scores(T, E, k, seed=T).numpy()
    idx, loc, gates, _ = oracle.route_topk(scores, k)
    C = oracle.capacity(T, E, k, cf, 4)
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(5)).to(dtype)
    i = [torch.from_numpy(a).to(DEV) for a in idx]
    l = [torch.from_numpy(a).to(DEV) for a in loc]
    gt = [torch.from_numpy(a).to(DEV) for a in gates]
    for with_gates in (False, True):
        codes, bias, scale = ops.dispatch_int8(x.to(DEV), i, l, gt if with_gates else None, E, C)
        d = torch.from_numpy(oracle.encode(x.float().numpy(), list(idx), list(loc), list(gates) if with_gates else None, E, C)).to(dtype)
        rc, rb, rs = oracle.int8_compress(to_np(d))
        assert np.array_equal(codes.cpu().numpy(), rc)
        assert np.array_equal(raw(bias), np_raw(rb)) and np.array_equal(raw(scale), np_raw(rs))
        # and against the unfused HIP path
        c2, b2, s2 = ops.int8_compress(ops.dispatch_fwd(x.to(DEV), i, l, gt if with_gates else None, E, C))
        assert torch.equal(codes, c2) and np.array_equal(raw(bias), raw(b2)) and np.array_equal(raw(scale), raw(s2))


# ------------------------------------------------------------------------------ zfp
def _zfp_cases(g):
    for k in g.files:
        if k.startswith("stream_"):
            _, name, d, r = k.split("_")
            yield k[7:], name, int(d[1]), float(r[1:])


def test_zfp_golden_streams_from_libzfp(zfp_golden):
    from planmoe_amd import ops
    n = 0
    for key, name, dims, rate in _zfp_cases(zfp_golden):
        f = zfp_golden["field_" + name]
        ny, nx = f.shape
        if (4 if dims == 1 else 16) * rate % 32:
            continue                                              # 1-D rate 4: 16-bit blocks, not built
        out = ops.zfp_compress(torch.from_numpy(f).to(DEV), nx, ny, dims, rate)
        want = zfp_golden["stream_" + key]
        assert out.numel() == int(zfp_golden["maxsize_" + key][0])
        assert np.array_equal(out.cpu().numpy()[:len(want)], want), key
        dec = ops.zfp_decompress(torch.from_numpy(np.concatenate([want, np.zeros(16, np.uint8)])).to(DEV), nx, ny, dims, rate)
        assert np.array_equal(raw(dec), zfp_golden["decoded_" + key].view(np.int32)), key
        n += 1
    assert n == 20


@pytest.mark.parametrize("ny,nx,dims", [(64, 128, 2), (64, 128, 1), (1024, 1024, 2), (4, 12, 1), (4, 4, 2), (12, 1028, 2), (20, 260, 1)])
def test_zfp_against_oracle(ny, nx, dims):
    from planmoe_amd import ops
    rng = np.random.default_rng(ny * nx + dims)
    f = rng.standard_normal((ny, nx)).astype(np.float32)
    f[0:4, 0:4] = 0
    if nx >= 12:
        f[0:4, 4:8] = 1e-40; f[0:4, 8:12] = 1e30; f[1, 6] = 0
    st = oracle.zfp_compress(f, dims)
    out = ops.zfp_compress(torch.from_numpy(f).to(DEV), nx, ny, dims)
    n = ops.zfp_stream_bytes(dims, nx, ny)
    assert n == len(st) and np.array_equal(out.cpu().numpy()[:n], st)
    dec = ops.zfp_decompress(out, nx, ny, dims)
    assert np.array_equal(raw(dec), oracle.zfp_decompress(st, ny, nx, dims).view(np.int32))


def _config5_field(rows, nx, seed=0):
    """Smooth N(0,1)-like field: per-row low-frequency sinusoid + box-filtered noise + noise."""
    g = torch.Generator().manual_seed(seed)
    j = torch.arange(nx, dtype=torch.float32)
    f_r = torch.randint(1, 4, (rows, 1), generator=g).float()
    phi = torch.rand(rows, 1, generator=g) * 2 * np.pi
    z = torch.randn(rows, nx + 8, generator=g)
    smooth = torch.nn.functional.avg_pool1d(z[:, None, :], 9, 1)[:, 0, :]
    v = 0.6 * smooth + torch.sin(2 * np.pi * f_r * j / nx + phi) + 0.05 * torch.randn(rows, nx, generator=g)
    return (v / v.std()).contiguous()


@pytest.mark.parametrize("rate", [2, 4, 8, 16])
def test_zfp_2d_field_kinds_and_rates(rate):
    """The 2-D coder at every block size it is built for, on fields that take the decoder's group-test
    walk through long zero runs, the block's last value, budgets that end in a run, all-zero blocks
    and planes below the sixteenth: streams and decoded fields against the oracle, bit for bit."""
    from planmoe_amd import ops
    rng = np.random.default_rng(3 + rate)
    ny, nx = 64, 512
    fields = {
        "gauss": rng.standard_normal((ny, nx)),
        "smooth": np.sin(np.arange(nx) / 37.0)[None, :] * np.cos(np.arange(ny) / 11.0)[:, None],
        "tiny": rng.standard_normal((ny, nx)) * 1e-30,
        "sparse": rng.standard_normal((ny, nx)) * (rng.random((ny, nx)) < 0.05),
        "spiky": rng.standard_normal((ny, nx)) * 10.0 ** rng.integers(-6, 6, (ny, nx)),
        "const": np.full((ny, nx), 3.25),
    }
    for name, f in fields.items():
        f = f.astype(np.float32)
        st = oracle.zfp_compress(f, 2, float(rate))
        want = oracle.zfp_decompress(st, ny, nx, 2, float(rate))
        got = ops.zfp_compress(torch.from_numpy(f).to(DEV), nx, ny, 2, float(rate)).cpu().numpy()
        assert np.array_equal(got[:len(st)], st), name
        dec = ops.zfp_decompress(torch.from_numpy(np.concatenate([st, np.zeros(16, np.uint8)])).to(DEV), nx, ny, 2, float(rate))
        assert np.array_equal(dec.cpu().numpy().view(np.uint32), want.view(np.uint32)), name


@pytest.mark.parametrize("dims", [2, 1])
def test_zfp_config5_full_size(dims):
    """[16, 8192, 1024] fp32 (65536 tokens x top-2 slots): whole stream against the oracle."""
    from planmoe_amd import ops
    ny, nx = 16 * 8192, 1024
    f = _config5_field(ny, nx)
    fd = f.to(DEV)
    out = ops.zfp_compress(fd, nx, ny, dims)
    n = ops.zfp_stream_bytes(dims, nx, ny)
    assert n == ny * nx                                            # 8 bits per value
    st = oracle.zfp_compress(f.numpy(), dims)
    assert np.array_equal(out.cpu().numpy()[:n], st)
    dec = ops.zfp_decompress(out, nx, ny, dims)
    assert np.array_equal(raw(dec), oracle.zfp_decompress(st, ny, nx, dims).view(np.int32))
    err = (dec - fd).abs().max().item()
    assert err < (0.25 if dims == 2 else 0.6)                      # rate 8 on a unit-variance smooth field
    # idempotence of the lossy round trip at the stream level
    again = ops.zfp_compress(dec, nx, ny, dims)
    dec2 = ops.zfp_decompress(again, nx, ny, dims)
    assert (dec2 - dec).abs().max().item() <= err


@pytest.mark.parametrize("T,M,E,k,cf", [(1000, 256, 8, 2, 1.25), (333, 1024, 16, 2, 0.5), (64, 4, 4, 4, 1.0),
                                        (5000, 132, 12, 1, 1.0), (7, 64, 4, 2, 4.0), (300, 2048, 4, 3, 1.0)])
def test_bwd_gate_zfp_equals_decompress_then_bwd_gate(T, M, E, k, cf):
    """planmoe_bwd_gate_zfp: the gate gradients from the stream of the expert output, against
    planmoe_zfp_decompress + planmoe_bwd_gate (another summation order: rtol 1e-5 on the sum of
    the terms' magnitudes) and against a dot product in fp64; exact zeros for dropped choices."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T * 3 + M)
    r = ops.route_topk(torch.softmax(torch.randn(T, E, generator=g), 1).to(DEV), k)
    C = ops.capacity(T, E, k, cf, 4)
    idx, loc = list(r["indices"]), list(r["locations"])
    y = torch.randn(E * C, M, generator=g).to(DEV)                   # expert outputs
    dout = torch.randn(T, M, generator=g).to(DEV)
    st = ops.zfp_compress(y, M, E * C, 2)
    seen = ops.zfp_decompress(st, M, E * C, 2)
    want = ops.bwd_gate(dout, seen, idx, loc, C)
    got = ops.bwd_gate_zfp(st, dout, idx, loc, E, C)
    assert got.shape == want.shape
    for j in range(k):
        kept = (loc[j] >= 0) & (loc[j] < C)
        slot = (idx[j].long() * C + loc[j].long()).clamp(0, max(E * C - 1, 0))
        rows = seen[slot] if E * C > 0 else torch.zeros_like(dout)
        ref = (dout.double() * rows.double()).sum(1) * kept
        mag = (dout.double() * rows.double()).abs().sum(1) * kept
        assert ((got[j].double() - ref).abs() <= 1e-5 * mag + 1e-30).all()
        # the oracle's leg: its own decode of its own stream, then its dot product in fp64
        if E * C > 0:
            n = ops.zfp_stream_bytes(2, M, E * C)
            ost = oracle.zfp_compress(y.cpu().numpy(), 2)
            assert np.array_equal(st.cpu().numpy()[:n], ost)
            orows = oracle.zfp_decompress(ost, E * C, M, 2).astype(np.float64)
            oref = oracle.bwd_gate(idx[j].cpu().numpy(), loc[j].cpu().numpy(), dout.double().cpu().numpy(), orows, C)
            assert (np.abs(got[j].double().cpu().numpy() - oref) <= 1e-5 * mag.cpu().numpy() + 1e-30).all()
        assert ((got[j].double() - want[j].double()).abs() <= 2e-5 * mag + 1e-30).all()
        assert (got[j][~kept] == 0).all()


def test_bwd_gate_zfp_without_slots_or_tokens():
    from planmoe_amd import ops
    T, M, E, k = 63, 64, 33, 2                                       # capacity_factor 0.25 leaves no slot
    C = ops.capacity(T, E, k, 0.25, 4)
    assert C == 0
    r = ops.route_topk(torch.softmax(torch.randn(T, E, generator=torch.Generator().manual_seed(0)), 1).to(DEV), k)
    empty = torch.empty((0,), dtype=torch.uint8, device=DEV)
    gg = ops.bwd_gate_zfp(empty, torch.randn(T, M, device=DEV), list(r["indices"]), list(r["locations"]), E, C)
    assert gg.shape == (k, T) and not gg.any()
    none = ops.bwd_gate_zfp(torch.zeros((4 * 64,), dtype=torch.uint8, device=DEV), torch.empty((0, M), device=DEV),
                            [torch.empty((0,), dtype=torch.int32, device=DEV)],
                            [torch.empty((0,), dtype=torch.int32, device=DEV)], 1, 4)
    assert none.shape == (1, 0)


def test_zfp_field_beyond_two_to_the_31_values():
    """A [8, 75000, 4096] fp32 buffer (2.46 G values, 9.8 GB; stream 2.46 GB): block and row addresses
    need 64 bits.  Blocks are coded independently, so the stream of the last 8 rows must be the
    stream of those rows coded alone, and the fused entry points must equal their two stages."""
    from planmoe_amd import ops
    T, M, E, k = 600000, 4096, 8, 1
    C = ops.capacity(T, E, k, 1.0, 4)
    R = E * C
    g = torch.Generator(device=DEV).manual_seed(2)
    x = torch.randn(T, M, generator=g, device=DEV, dtype=torch.float32)
    r = ops.route_topk(torch.softmax(torch.randn(T, E, generator=g, device=DEV), 1), k)
    idx, loc, gates = list(r["indices"]), list(r["locations"]), [t.float() for t in r["gates"]]
    d = ops.dispatch_fwd(x, idx, loc, None, E, C)
    assert d.numel() > 2 ** 31
    st = ops.zfp_compress(d, M, R, 2)
    n = ops.zfp_stream_bytes(2, M, R)
    tail = ops.zfp_compress(d[R - 8:].contiguous(), M, 8, 2)
    nt = ops.zfp_stream_bytes(2, M, 8)
    assert torch.equal(st[n - nt:n], tail[:nt])
    fused = ops.dispatch_zfp(x, idx, loc, None, E, C)
    assert torch.equal(fused[:n], st[:n])
    del fused
    dec = ops.zfp_decompress(st, M, R, 2)
    assert torch.equal(dec[R - 8:], ops.zfp_decompress(tail, M, 8, 2))
    del d
    y = ops.combine_fwd(dec, idx, loc, gates, T, C)
    del dec
    y2 = ops.combine_zfp(st, idx, loc, gates, T, E, C, M)
    assert torch.equal(y.view(torch.int32), y2.view(torch.int32))


@pytest.mark.parametrize("copies", [False, True])
def test_compressor_registry_round_trips(copies):
    """compress_operation / comm_operation / decompress_operation with 'no', 'int8', 'zfp', 'lz';
    the one-rank comm step hands the buffers over (default) or copies them."""
    from planmoe_amd import compressor
    compressor.SINGLE_RANK_COMM_COPIES = copies
    try:
        _registry_round_trips(compressor, copies)
    finally:
        compressor.SINGLE_RANK_COMM_COPIES = False


def _registry_round_trips(compressor, copies):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 64, 256, generator=g).to(DEV)
    compressor.clear_ptr_lst()
    outs = []
    for name in ("no", "int8", "zfp"):
        c = compressor.compress_operation(x, name, "naive")
        outs.append((name, c))
    assert outs[0][1] is x
    assert outs[1][1].dtype == torch.float32 and outs[1][1].numel() == x.numel() // 4
    assert outs[2][1].dtype == torch.float16 and outs[2][1].numel() == (oracle.zfp_max_bytes(2, 256, 256) + 1) // 2
    recv = [compressor.comm_operation(c) for _, c in outs]
    assert all((r.data_ptr() != c.data_ptr()) == copies for r, (_, c) in zip(recv, outs))
    dec = [compressor.decompress_operation(r) for r in recv]
    assert torch.equal(dec[0], x)
    rc, rb, rs = oracle.int8_compress(x.cpu().numpy())
    assert np.array_equal(raw(dec[1]), oracle.int8_decompress(rc, rb, rs).view(np.int32))
    st = oracle.zfp_compress(x.cpu().numpy().reshape(-1, 256), 2)
    assert np.array_equal(raw(dec[2]), oracle.zfp_decompress(st, 256, 256, 2).reshape(4, 64, 256).view(np.int32))
    # 'lz': the input comes back untouched, the streams travel, the decode fills g_output
    x[2] = 0.0
    c = compressor.compress_operation(x, "lz", "naive")
    assert c is x
    lz = compressor._compress_ptr_lst[-1]
    want = oracle.lz_compress(x.cpu().numpy())
    for got, ref in zip((lz.flagArrOffsetGlobal, lz.compressedDataOffsetGlobal, lz.flagArrGlobal,
                         lz.compressedDataGlobal), want):
        assert np.array_equal(got.cpu().numpy(), ref)
    r = compressor.comm_operation(c)
    assert r is not x and not r.any()
    d = compressor.decompress_operation(r)
    assert d is r and torch.equal(d, x)
    bx = x.bfloat16()
    c = compressor.compress_operation(bx, "int8", "naive")
    d = compressor.decompress_operation(compressor.comm_operation(c))
    assert d.dtype == torch.bfloat16 and d.shape == bx.shape
    rc, rb, rs = oracle.int8_compress(bf16_bits(bx))
    assert np.array_equal(raw(d), np_raw(oracle.int8_decompress(rc, rb, rs)))


@pytest.mark.parametrize("T,M,E,k,cf,dtype", [(300, 1024, 8, 2, 0.75, torch.bfloat16), (100, 256, 4, 3, 1.0, torch.float32),
                                              (64, 20000, 4, 2, 0.5, torch.bfloat16)])
def test_combine_bwd_int8_equals_the_unfused_backward(T, M, E, k, cf, dtype):
    """Config-4 fusion: scatter of gate * grad_out, gate gradients and the int8 compress of the
    gradient buffer in one launch against dispatch_fwd + bwd_gate + int8_compress and the oracle."""
    from planmoe_amd import ops
    scores = tie_free_scores(T, E, k, seed=T + 1).numpy()
    idx, loc, gates, _ = oracle.route_topk(scores, k)
    C = oracle.capacity(T, E, k, cf, 4)
    g = torch.Generator().manual_seed(7)
    dout = torch.randn(T, M, generator=g).to(dtype)
    eo = torch.randn(E * C, M, generator=g).to(dtype)
    i = [torch.from_numpy(a).to(DEV) for a in idx]
    l = [torch.from_numpy(a).to(DEV) for a in loc]
    gt = [torch.from_numpy(a).to(DEV) for a in gates]
    codes, bias, scale, gg = ops.combine_bwd_int8(dout.to(DEV), eo.to(DEV), i, l, gt, E, C)
    d = torch.from_numpy(oracle.encode(dout.float().numpy(), list(idx), list(loc), list(gates), E, C)).to(dtype)
    rc, rb, rs = oracle.int8_compress(to_np(d))
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(raw(bias), np_raw(rb)) and np.array_equal(raw(scale), np_raw(rs))
    c2, b2, s2 = ops.int8_compress(ops.dispatch_fwd(dout.to(DEV), i, l, gt, E, C))
    assert torch.equal(codes, c2) and np.array_equal(raw(bias), raw(b2))
    g2 = ops.bwd_gate(dout.to(DEV), eo.to(DEV), i, l, C)
    xd, ed = dout.double().numpy(), eo.double().numpy()
    rtol = 1e-5 if dtype == torch.float32 else 1e-2
    for j in range(k):
        want = oracle.bwd_gate(idx[j], loc[j], xd, ed, C)
        mag = oracle.bwd_gate(idx[j], loc[j], np.abs(xd), np.abs(ed), C)
        got = gg[j].cpu().numpy()
        assert (np.abs(got - want) <= rtol * np.abs(want) + 1e-6 * mag).all()
        assert (got[loc[j] >= C] == 0).all()
        assert np.allclose(got, g2[j].cpu().numpy(), rtol=1e-5, atol=1e-6 * mag.max())
    # the expert output handed over as int8 codes: decoded on the fly to what int8_decompress gives
    ec, eb, es = ops.int8_compress(eo.to(DEV))
    seen = ops.int8_decompress(ec, eb, es)
    c3, b3, s3, g3 = ops.combine_bwd_int8(dout.to(DEV), seen, i, l, gt, E, C)
    c4, b4, s4, g4 = ops.combine_bwd_int8(dout.to(DEV), (ec, eb, es), i, l, gt, E, C)
    assert torch.equal(c3, c4) and torch.equal(b3, b4) and torch.equal(s3, s4)
    assert np.array_equal(raw(g3), raw(g4))


def test_config4_backward_full_size():
    """Config 4 at its own shape: 16384 x 4096 bf16, 8 experts, top-2, cf 1.25 (capacity 5120), the
    routing of config 2 (x, wg seed 0), upstream gradient N(0,1) seed 1, expert output seed 2.
    (i) backward of combine fused with the int8 compress of the gradient buffer, expert output
    given as bf16 and as int8 codes: codes / bias / scale bit-exact against the oracle, gate
    gradients within rtol 1e-2 of the fp64 dot product (+ 1e-6 of the sum of the terms'
    magnitudes); (ii) int8 decompress bit-exact; (iii) backward of dispatch (gather-sum without
    gates) bit-exact, stand-alone and fused with the decompress."""
    from planmoe_amd import ops
    T, M, E, k = 16384, 4096, 8, 2
    g0 = torch.Generator().manual_seed(0)
    x = torch.randn(T, M, generator=g0).bfloat16()
    wg = (torch.randn(E, M, generator=g0) * M ** -0.5).bfloat16()
    r = ops.gate_route(x.to(DEV), wg.to(DEV), k, want_scores=True)
    idx, loc, gates, _ = oracle.route_topk(r["scores"].cpu().numpy(), k)
    assert np.array_equal(r["indices"].cpu().numpy(), idx) and np.array_equal(r["locations"].cpu().numpy(), loc)
    C = oracle.capacity(T, E, k, 1.25, 4)
    assert C == 5120
    dout = torch.randn(T, M, generator=torch.Generator().manual_seed(1)).bfloat16()
    eo = torch.randn(E * C, M, generator=torch.Generator().manual_seed(2)).bfloat16()
    i, l = list(r["indices"]), list(r["locations"])
    gt = [torch.from_numpy(a).to(DEV) for a in gates]
    dd, ed = dout.to(DEV), eo.to(DEV)
    codes, bias, scale, gg = ops.combine_bwd_int8(dd, ed, i, l, gt, E, C)
    # (i) the gradient buffer [E * C, M] = scatter of round(gate * dOut), then the codec
    d = torch.from_numpy(oracle.encode(dout.float().numpy(), list(idx), list(loc), list(gates), E, C)).bfloat16()
    rc, rb, rs = oracle.int8_compress(bf16_bits(d))
    del d
    assert np.array_equal(codes.cpu().numpy(), rc)
    assert np.array_equal(raw(bias), np_raw(rb)) and np.array_equal(raw(scale), np_raw(rs))
    xd, e64 = dout.double().numpy(), eo.double().numpy()
    for j in range(k):
        want = oracle.bwd_gate(idx[j], loc[j], xd, e64, C)
        mag = oracle.bwd_gate(idx[j], loc[j], np.abs(xd), np.abs(e64), C)
        got = gg[j].float().cpu().numpy()
        assert (np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6 * mag).all()
        assert (got[loc[j] >= C] == 0).all()
    del e64
    # the expert output as the int8 codes the receive side holds: what decompress would have given
    ec, eb, es = ops.int8_compress(ed)
    oc, ob, os_ = oracle.int8_compress(bf16_bits(eo))
    assert np.array_equal(ec.cpu().numpy(), oc)
    seen = from_bf16_bits(oracle.int8_decompress(oc, ob, os_)).double().numpy()
    c4, b4, s4, g4 = ops.combine_bwd_int8(dd, (ec, eb, es), i, l, gt, E, C)
    assert torch.equal(c4, codes) and torch.equal(b4, bias) and torch.equal(s4, scale)
    for j in range(k):
        want = oracle.bwd_gate(idx[j], loc[j], xd, seen, C)
        mag = oracle.bwd_gate(idx[j], loc[j], np.abs(xd), np.abs(seen), C)
        got = g4[j].float().cpu().numpy()
        assert (np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-6 * mag).all()
    del seen, xd
    # (ii) decompress of the gradient buffer, (iii) backward of dispatch: sum of the slot rows
    dec_ref = oracle.int8_decompress(rc, rb, rs)
    dec = ops.int8_decompress(codes, bias, scale)
    assert np.array_equal(raw(dec), np_raw(dec_ref))
    dx_ref = torch.from_numpy(oracle.decode(from_bf16_bits(dec_ref).float().numpy(), list(idx), list(loc), None, T, C)).bfloat16()
    assert np.array_equal(raw(ops.combine_fwd(dec, i, l, None, T, C)), raw(dx_ref))
    assert np.array_equal(raw(ops.combine_int8(codes, bias, scale, i, l, None, T, C)), raw(dx_ref))


@pytest.mark.parametrize("T,M,E,k,dtype,gated", [(1000, 512, 8, 2, torch.bfloat16, True), (300, 264, 5, 3, torch.bfloat16, False),
                                                  (257, 128, 4, 2, torch.float32, True), (64, 72, 3, 1, torch.float16, True),
                                                  (16384, 4096, 8, 2, torch.bfloat16, True)])
def test_combine_int8_equals_decompress_then_combine(T, M, E, k, dtype, gated):
    """planmoe_combine_int8 against planmoe_int8_decompress + planmoe_combine_fwd (bit for bit),
    and, for bf16 / fp32, that pair against the oracle."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + M)
    scores = torch.softmax(torch.randn(T, E, generator=g), 1)
    r = ops.route_topk(scores.to(DEV), k)
    C = ops.capacity(T, E, k, 1.0, 4)
    idx, loc = list(r["indices"]), list(r["locations"])
    gates = [x.float() for x in r["gates"]] if gated else None
    y = torch.randn(E * C, M, generator=g).to(dtype).to(DEV)          # expert outputs
    codes, bias, scale = ops.int8_compress(y)
    want = ops.combine_fwd(ops.int8_decompress(codes, bias, scale), idx, loc, gates, T, C)
    got = ops.combine_int8(codes, bias, scale, idx, loc, gates, T, C)
    assert np.array_equal(raw(got), raw(want))
    if dtype != torch.float16 and T <= 1000:
        rc, rb, rs = oracle.int8_compress(bf16_bits(y.cpu()) if dtype == torch.bfloat16 else y.cpu().numpy())
        dec = oracle.int8_decompress(rc, rb, rs)
        dec32 = from_bf16_bits(dec).float().numpy() if dtype == torch.bfloat16 else dec
        ref = oracle.decode(dec32, [a.cpu().numpy() for a in idx], [a.cpu().numpy() for a in loc],
                            [a.cpu().numpy() for a in gates] if gated else None, T, C)
        ref_t = torch.from_numpy(ref).to(dtype)
        assert np.array_equal(raw(got), raw(ref_t))


@pytest.mark.parametrize("T,M,E,k,cf,gated", [(1000, 256, 8, 2, 1.25, False), (333, 1024, 16, 2, 0.5, True),
                                              (64, 4, 4, 4, 1.0, True), (5000, 132, 12, 1, 1.0, False),
                                              (7, 64, 4, 2, 4.0, True)])
def test_dispatch_zfp_equals_dispatch_then_compress(T, M, E, k, cf, gated):
    """planmoe_dispatch_zfp: the stream of the dispatched buffer without the buffer, against the
    two stages and against the oracle."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T + M)
    x = torch.randn(T, M, generator=g)
    scores = torch.softmax(torch.randn(T, E, generator=g), dim=1)
    r = ops.route_topk(scores.to(DEV), k)
    C = ops.capacity(T, E, k, cf, 4)
    idx, loc = list(r["indices"]), list(r["locations"])
    gates = list(r["gates"]) if gated else None
    xd = x.to(DEV)
    got = ops.dispatch_zfp(xd, idx, loc, gates, E, C)
    staged = ops.zfp_compress(ops.dispatch_fwd(xd, idx, loc, gates, E, C), M, E * C, 2)
    assert torch.equal(got, staged)
    n = ops.zfp_stream_bytes(2, M, E * C)
    d = oracle.encode(x.numpy(), list(r["indices"].cpu().numpy()), list(r["locations"].cpu().numpy()),
                      list(r["gates"].cpu().numpy()) if gated else None, E, C)
    assert np.array_equal(got.cpu().numpy()[:n], oracle.zfp_compress(d.reshape(E * C, M), 2))


def test_dispatch_zfp_edge_cases():
    from planmoe_amd import ops
    from planmoe_amd._lib import PlanMoEError
    x = torch.randn(16, 64, device=DEV)
    idx = [torch.zeros(16, dtype=torch.int32, device=DEV)]
    loc = [torch.arange(16, dtype=torch.int32, device=DEV)]
    # every token dropped (capacity 0): nothing to code
    assert ops.dispatch_zfp(x, idx, loc, None, 4, 0).numel() == ops.zfp_max_bytes(2, 64, 0)
    # no token at all: a field of zeros
    e = torch.empty((0, 64), device=DEV)
    none = [torch.empty((0,), dtype=torch.int32, device=DEV)]
    out = ops.dispatch_zfp(e, none, none, None, 4, 8)
    assert not out.any()
    assert torch.equal(out, ops.zfp_compress(torch.zeros(32, 64, device=DEV), 64, 32, 2))
    with pytest.raises(PlanMoEError, match="zfp fails."):
        ops.dispatch_zfp(x, idx, loc, None, 3, 2)                      # 6 slot rows
    with pytest.raises(PlanMoEError):
        ops.dispatch_zfp(x.bfloat16(), idx, loc, None, 4, 8)


@pytest.mark.parametrize("T,M,E,k,cf,gated", [(1000, 256, 8, 2, 1.25, True), (333, 1024, 16, 2, 0.5, True),
                                              (64, 4, 4, 4, 1.0, True), (5000, 132, 12, 1, 1.0, False),
                                              (7, 64, 4, 2, 4.0, False), (900, 64, 4, 3, 0.25, True)])
def test_combine_zfp_equals_decompress_then_combine(T, M, E, k, cf, gated):
    """planmoe_combine_zfp: the token rows straight from the stream, bit for bit what the two
    stages give (dropped choices, empty slots, gates of both signs, zero rows)."""
    from planmoe_amd import ops
    g = torch.Generator().manual_seed(T * 3 + M)
    scores = torch.softmax(torch.randn(T, E, generator=g), dim=1)
    r = ops.route_topk(scores.to(DEV), k)
    C = ops.capacity(T, E, k, cf, 4)
    idx, loc = list(r["indices"]), list(r["locations"])
    gates = None
    if gated:
        gates = [(torch.randn(T, generator=g) * (torch.rand(T, generator=g) > 0.1)).to(DEV) for _ in range(k)]
    y = torch.randn(E * C, M, generator=g)
    y[::7] = 0.0
    stream = ops.zfp_compress(y.to(DEV), M, E * C, 2)
    got = ops.combine_zfp(stream, idx, loc, gates, T, E, C, M)
    dec = ops.zfp_decompress(stream, M, E * C, 2)
    want = ops.combine_fwd(dec, idx, loc, gates, T, C)
    assert np.array_equal(raw(got), raw(want))
    ref = oracle.decode(oracle.zfp_decompress(stream.cpu().numpy()[:ops.zfp_stream_bytes(2, M, E * C)], E * C, M, 2),
                        list(r["indices"].cpu().numpy()), list(r["locations"].cpu().numpy()),
                        [t.cpu().numpy() for t in gates] if gated else None, T, C)
    assert np.array_equal(raw(got), ref.view(np.int32))


def test_combine_zfp_edge_cases():
    from planmoe_amd import ops
    idx = [torch.zeros(16, dtype=torch.int32, device=DEV)]
    loc = [torch.arange(16, dtype=torch.int32, device=DEV)]
    none = torch.empty((0,), dtype=torch.uint8, device=DEV)
    out = ops.combine_zfp(ops.zfp_compress(torch.empty((0, 64), device=DEV), 64, 0, 2), idx, loc, None, 16, 4, 0, 64)
    assert out.shape == (16, 64) and not out.any()                        # capacity 0: every token dropped
    e = [torch.empty((0,), dtype=torch.int32, device=DEV)]
    stream = ops.zfp_compress(torch.randn(32, 64, device=DEV), 64, 32, 2)
    assert ops.combine_zfp(stream, e, e, None, 0, 4, 8, 64).shape == (0, 64)
    del none
