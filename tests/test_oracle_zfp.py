"""Pins of the zfp part of the CPU oracle: golden streams from stock libzfp 0.5.5."""
import numpy as np
import pytest

import oracle


def _cases(g):
    for k in g.files:
        if k.startswith("stream_"):
            _, name, d, r = k.split("_")
            yield k[7:], name, int(d[1]), float(r[1:])


def test_library_version(zfp_golden):
    assert int(zfp_golden["zfp_library_version"][0]) == 0x055


def test_streams_match_libzfp(zfp_golden):
    n = 0
    for key, name, dims, rate in _cases(zfp_golden):
        f = zfp_golden["field_" + name]
        st = oracle.zfp_compress(f, dims, rate)
        assert np.array_equal(st, zfp_golden["stream_" + key]), key
        n += 1
    assert n == 24


def test_decode_of_libzfp_streams_matches_libzfp(zfp_golden):
    for key, name, dims, rate in _cases(zfp_golden):
        f = zfp_golden["field_" + name]
        dec = oracle.zfp_decompress(zfp_golden["stream_" + key], f.shape[0], f.shape[1], dims, rate)
        assert np.array_equal(dec.view(np.uint32), zfp_golden["decoded_" + key].view(np.uint32)), key


def test_buffer_size_law(zfp_golden):
    for key, name, dims, rate in _cases(zfp_golden):
        ny, nx = zfp_golden["field_" + name].shape
        assert oracle.zfp_max_bytes(dims, nx, ny, rate) == int(zfp_golden["maxsize_" + key][0])
        n = 4 if dims == 1 else 16
        blocks = nx * ny // n
        bits = blocks * int(n * rate + 0.5)
        assert oracle.zfp_stream_bytes(dims, nx, ny, rate) == (bits + 63) // 64 * 8
        assert len(zfp_golden["stream_" + key]) == oracle.zfp_stream_bytes(dims, nx, ny, rate)


@pytest.mark.parametrize("nm,dims", [("f1", 1), ("f2", 2), ("i1", 1), ("i2", 2)])
def test_block_coder_against_low_level_api(zfp_golden, nm, dims):
    out = oracle.zfp_encode_block(zfp_golden["block_in_" + nm], dims, 8.0)
    assert np.array_equal(out, zfp_golden["block_out_" + nm])
    assert int(zfp_golden["block_bits_" + nm][0]) == (32 if dims == 1 else 128)


def test_zero_field_is_zero_stream():
    st = oracle.zfp_compress(np.zeros((8, 16), np.float32), 2, 8.0)
    assert st.sum() == 0 and len(st) == 8 * 16
    assert np.array_equal(oracle.zfp_decompress(st, 8, 16, 2, 8.0), np.zeros((8, 16), np.float32))


def test_round_trip_error_bound():
    rng = np.random.default_rng(1)
    f = rng.standard_normal((64, 64)).astype(np.float32)
    for dims, tol in ((1, 0.6), (2, 0.25)):
        dec = oracle.zfp_decompress(oracle.zfp_compress(f, dims, 8.0), 64, 64, dims, 8.0)
        assert np.abs(dec - f).max() < tol
    dec16 = oracle.zfp_decompress(oracle.zfp_compress(f, 2, 16.0), 64, 64, 2, 16.0)
    assert np.abs(dec16 - f).max() < 2e-3


def test_extent_not_multiple_of_four_is_rejected():
    with pytest.raises(ValueError):
        oracle.zfp_compress(np.zeros((6, 8), np.float32), 2, 8.0)
