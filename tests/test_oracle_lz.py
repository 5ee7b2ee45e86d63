"""Pins of the GPULZ ("lz") part of the CPU oracle.

The reference holds no stream fixtures for this codec, so the oracle is pinned by what the
format fixes: streams worked out by hand for inputs where the matcher's rules (first run kept
on ties, a window symbol is consumed by a failed comparison, the run still open at the window's
end counts, float equality) each decide the outcome, closed forms for constant and all-distinct
blocks, and round trips through a decoder written here from the stream layout alone."""
import struct

import numpy as np
import pytest

import oracle


def distinct(n, start=1000.0):
    """n floats that equal nothing else in the block"""
    return (start + np.arange(n)).astype(np.float32)


def block_with(prefix):
    prefix = np.asarray(prefix, np.float32)
    return np.concatenate([prefix, distinct(512 - prefix.size)])


def lit(v):
    return struct.pack("<f", v)


def expect_stream(tokens):
    """tokens: list of ('L', value) / ('M', length, offset) -> (flag bytes, data bytes)"""
    flags = bytearray((len(tokens) + 7) // 8)
    data = bytearray()
    for t, tok in enumerate(tokens):
        if tok[0] == 'M':
            flags[t // 8] |= 1 << (t % 8)
            data += bytes([tok[1], tok[2]])
        else:
            data += lit(tok[1])
    return bytes(flags), bytes(data)


def check_block(blk, tokens):
    fo, do, flags, data = oracle.lz_compress(blk)
    f, d = expect_stream(tokens)
    assert fo.tolist() == [0, len(f)] and do.tolist() == [0, len(d)]
    assert flags[:len(f)].tobytes() == f
    assert data[:len(d)].tobytes() == d
    assert not flags[len(f):].any() and not data[len(d):].any()


def test_constant_block_closed_form():
    # position p sees min(p, 32) equal symbols behind it: tokens L, (1,1), (2,2), (4,4), (8,8),
    # (16,16), then (32,32) from 32 to the end -- 21 tokens, 3 flag bytes, 44 data bytes
    blk = np.full(512, 3.5, np.float32)
    tokens = [('L', 3.5)] + [('M', n, n) for n in (1, 2, 4, 8, 16)] + [('M', 32, 32)] * 15
    check_block(blk, tokens)
    fo, do, flags, data = oracle.lz_compress(blk)
    assert flags[:3].tolist() == [0xFE, 0xFF, 0x1F] and do[1] == 44


def test_all_distinct_block_is_stored():
    blk = distinct(512)
    fo, do, flags, data = oracle.lz_compress(blk)
    assert fo.tolist() == [0, 64] and do.tolist() == [0, 2048]
    assert not flags.any()
    assert data.tobytes() == blk.tobytes()


def test_failed_comparison_consumes_the_window_symbol():
    # a a b a b: at p=3 the run that starts at w=0 breaks at w=1, and w=1 is not tried again as a
    # start, so the two-symbol match (2, 2) is never seen: the token is (1, 3)
    a, b = 1.0, 2.0
    blk = block_with([a, a, b, a, b])
    tokens = [('L', a), ('M', 1, 1), ('L', b), ('M', 1, 3), ('M', 1, 2)] + [('L', v) for v in blk[5:]]
    check_block(blk, tokens)


def test_first_of_equal_runs_is_kept():
    # a b a c a d: at p=4 both a's match with length 1; the farther one (offset 4) came first
    a, b, c, d = 1.0, 2.0, 3.0, 4.0
    blk = block_with([a, b, a, c, a, d])
    tokens = [('L', a), ('L', b), ('M', 1, 2), ('L', c), ('M', 1, 4), ('L', d)] + [('L', v) for v in blk[6:]]
    check_block(blk, tokens)


def test_longer_later_run_wins():
    # a b x a b c y | a b c z: at p=7 the run at offset 7 has length 2, the one at offset 4 length 3
    a, b, c, x, y, z = 1.0, 2.0, 3.0, 4.0, 5.0, 6.0
    blk = block_with([a, b, x, a, b, c, y, a, b, c, z])
    tokens = [('L', a), ('L', b), ('L', x), ('M', 2, 3), ('L', c), ('L', y), ('M', 3, 4), ('L', z)]
    tokens += [('L', v) for v in blk[11:]]
    check_block(blk, tokens)


def test_float_equality_rules():
    # +0 and -0 are equal (the match turns the -0 into +0 when decoded); a NaN equals nothing
    nan = float('nan')
    blk = block_with([0.0, -0.0, nan, nan])
    fo, do, flags, data = oracle.lz_compress(blk)
    assert flags[0] == 0b00000010                       # L(+0) M(1,1) L(nan) L(nan) L...
    assert data[4:6].tolist() == [1, 1]
    out = oracle.lz_decompress(fo, do, flags, data)
    assert np.signbit(out[1]) == False and out[1] == 0.0     # noqa: E712
    assert np.isnan(out[2]) and np.isnan(out[3])
    assert np.array_equal(out[4:], blk[4:])


def test_match_stops_at_the_block_end():
    # the last two symbols repeat the two before them; the look-ahead may not leave the block
    blk = distinct(512)
    blk[510:] = blk[508:510]
    fo, do, flags, data = oracle.lz_compress(blk)
    assert do[1] == 510 * 4 + 2 and data[2040:2042].tolist() == [2, 2]
    blk2 = np.concatenate([blk, blk])                    # a second block never matches into the first
    fo2, do2, flags2, data2 = oracle.lz_compress(blk2)
    assert do2.tolist() == [0, 2042, 4084] and fo2.tolist() == [0, 64, 128]


def py_decode(fo, do, flags, data):
    """Decoder written from the stream layout (flag bit per token, LSB first; 4-byte literal or
    length/offset pair) -- shares no code with the oracle."""
    out = []
    for b in range(len(fo) - 1):
        blk, pos, t = [], int(do[b]), 0
        while len(blk) < 512:
            bit = (int(flags[int(fo[b]) + t // 8]) >> (t % 8)) & 1
            if bit:
                n, off = int(data[pos]), int(data[pos + 1])
                start = len(blk)
                for i in range(n):
                    blk.append(blk[start - off + i])
                pos += 2
            else:
                blk.append(bytes(data[pos:pos + 4]))
                pos += 4
            t += 1
        assert pos == int(do[b + 1]) and (t + 7) // 8 == int(fo[b + 1]) - int(fo[b])
        out += blk
    return np.frombuffer(b"".join(out), np.float32)


@pytest.mark.parametrize("alphabet,seed", [(2, 0), (3, 1), (8, 2), (64, 3), (100000, 4)])
def test_round_trip_and_token_validity(alphabet, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(1, alphabet + 1, size=6 * 512).astype(np.float32)
    x[512:1024] = 0.0                                     # an empty capacity slot
    fo, do, flags, data = oracle.lz_compress(x)
    assert np.array_equal(py_decode(fo, do, flags, data).view(np.uint32), x.view(np.uint32))
    assert np.array_equal(oracle.lz_decompress(fo, do, flags, data).view(np.uint32), x.view(np.uint32))
    assert np.all(np.diff(fo) >= 1) and np.all(np.diff(do) >= 2) and np.all(np.diff(do) <= 2048)
    assert not flags[fo[-1]:].any() and not data[do[-1]:].any()


def test_inconsistent_stream_is_rejected():
    fo = np.array([0, 1], np.int32)
    do = np.array([0, 2], np.int32)
    flags = np.zeros(64, np.uint8)
    flags[0] = 1
    data = np.zeros(2048, np.uint8)
    data[0], data[1] = 4, 9                               # a match that reaches before the block
    with pytest.raises(ValueError):
        oracle.lz_decompress(fo, do, flags, data)
