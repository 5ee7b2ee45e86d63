"""Writes tests/golden/zfp_golden.npz: header-less fixed-rate streams and decoded fields
produced by the stock zfp 0.5.5 shared library (serial execution) for small float fields.

Run once in a container that has libzfp.so.0.5.5 (here: /opt/conda/lib); the .npz is
committed so the tests do not need the library.  Nothing from the reference tree is read.

    python tests/golden/make_zfp_golden.py
"""
import ctypes
import os
import sys

import numpy as np

LIBZFP = os.environ.get("LIBZFP", "/opt/conda/lib/libzfp.so.0.5.5")
ZFP_TYPE_FLOAT = 3


def load():
    z = ctypes.CDLL(LIBZFP)
    for name in ("zfp_field_1d", "zfp_field_2d", "zfp_stream_open", "stream_open"):
        getattr(z, name).restype = ctypes.c_void_p
    z.zfp_stream_set_rate.restype = ctypes.c_double
    z.zfp_stream_maximum_size.restype = ctypes.c_size_t
    z.zfp_compress.restype = ctypes.c_size_t
    z.zfp_decompress.restype = ctypes.c_size_t
    z.zfp_encode_block_float_1.restype = ctypes.c_uint
    z.zfp_encode_block_float_2.restype = ctypes.c_uint
    z.zfp_encode_block_int32_1.restype = ctypes.c_uint
    z.zfp_encode_block_int32_2.restype = ctypes.c_uint
    z.stream_flush.restype = ctypes.c_uint
    return z


def codec(z, field, dims, rate):
    """(stream bytes, maximum size, decoded field) for a [ny, nx] float32 array."""
    field = np.ascontiguousarray(field, np.float32)
    ny, nx = field.shape
    vp = ctypes.c_void_p

    def mkfield(arr):
        if dims == 2:
            return z.zfp_field_2d(arr.ctypes.data_as(vp), ZFP_TYPE_FLOAT, ctypes.c_uint(nx), ctypes.c_uint(ny))
        return z.zfp_field_1d(arr.ctypes.data_as(vp), ZFP_TYPE_FLOAT, ctypes.c_uint(nx * ny))

    f = mkfield(field)
    s = z.zfp_stream_open(None)
    z.zfp_stream_set_rate(vp(s), ctypes.c_double(rate), ZFP_TYPE_FLOAT, ctypes.c_uint(dims), 0)
    maxsize = z.zfp_stream_maximum_size(vp(s), vp(f))
    buf = np.zeros(maxsize, np.uint8)
    bs = z.stream_open(buf.ctypes.data_as(vp), ctypes.c_size_t(maxsize))
    z.zfp_stream_set_bit_stream(vp(s), vp(bs))
    length = z.zfp_compress(vp(s), vp(f))
    out = np.empty_like(field)
    f2 = mkfield(out)
    z.zfp_stream_rewind(vp(s))
    z.zfp_decompress(vp(s), vp(f2))
    z.zfp_field_free(vp(f)); z.zfp_field_free(vp(f2)); z.zfp_stream_close(vp(s)); z.stream_close(vp(bs))
    return buf[:length].copy(), maxsize, out


def block_api(z, block, dims, rate, as_int):
    """One block through the low-level zfp_encode_block_* entry points."""
    vp = ctypes.c_void_p
    s = z.zfp_stream_open(None)
    z.zfp_stream_set_rate(vp(s), ctypes.c_double(rate), ZFP_TYPE_FLOAT, ctypes.c_uint(dims), 0)
    buf = np.zeros(64, np.uint8)
    bs = z.stream_open(buf.ctypes.data_as(vp), ctypes.c_size_t(64))
    z.zfp_stream_set_bit_stream(vp(s), vp(bs))
    fn = getattr(z, "zfp_encode_block_%s_%d" % ("int32" if as_int else "float", dims))
    bits = fn(vp(s), block.ctypes.data_as(vp))
    z.stream_flush(vp(bs))
    z.zfp_stream_close(vp(s)); z.stream_close(vp(bs))
    return buf.copy(), bits


def fields():
    rng = np.random.default_rng(20261125)
    out = {}
    # smooth field: per-row sinusoid + filtered noise, the shape of config 5
    ny, nx = 32, 64
    j = np.arange(nx)
    rows = []
    for r in range(ny):
        f_r, phi = rng.integers(1, 4), rng.uniform(0, 2 * np.pi)
        noise = np.convolve(rng.standard_normal(nx + 8), np.ones(9) / 9, mode="valid")
        rows.append(0.6 * noise + np.sin(2 * np.pi * f_r * j / nx + phi) + 0.05 * rng.standard_normal(nx))
    out["smooth"] = np.asarray(rows, np.float32)
    out["gauss"] = rng.standard_normal((16, 32)).astype(np.float32)
    edge = rng.standard_normal((32, 32)).astype(np.float32)
    edge[0:4, 0:8] = 0.0                                   # all-zero blocks
    edge[4:8, 0:4] = -3.5                                  # constant negative
    edge[8:12, 0:4] = 1e-40                                # denormal block
    edge[8:12, 4:8] = 0.0; edge[9, 5] = 1e-41              # denormal maximum among zeros
    edge[12:16, 0:4] = 1e30                                # large magnitude
    edge[12:16, 4:8] = np.float32(3.0e38)                  # near FLT_MAX
    edge[16:20, 0:4] = 0.0; edge[17, 2] = 77.0             # single spike
    edge[20:24, 0:8] = 1e-30
    edge[24:28, 0:4] = np.where((np.add.outer(np.arange(4), np.arange(4)) % 2) == 0, 1.0, -1.0)  # alternating signs
    edge[24:28, 4:8] = 2.0 ** -100                         # scale factor overflows float
    edge[28:32, 0:4] = np.float32(2.0 ** 127)
    edge[28:32, 4:8] = -np.float32(2.0 ** -126)
    out["edge"] = edge
    out["tiny"] = rng.standard_normal((4, 4)).astype(np.float32)
    return out


def main():
    z = load()
    ver = ctypes.c_uint.in_dll(z, "zfp_library_version").value
    assert ver == 0x055, hex(ver)
    data = {"zfp_library_version": np.array([ver], np.uint32)}
    for name, fld in fields().items():
        data["field_" + name] = fld
        for dims in (1, 2):
            for rate in (8.0, 16.0, 4.0):
                st, maxsize, dec = codec(z, fld, dims, rate)
                key = "%s_d%d_r%d" % (name, dims, int(rate))
                data["stream_" + key] = st
                data["maxsize_" + key] = np.array([maxsize], np.uint64)
                data["decoded_" + key] = dec
    # low-level block entry points: pin the block coder separately from the float cast
    rng = np.random.default_rng(7)
    fb1 = rng.standard_normal(4).astype(np.float32)
    fb2 = rng.standard_normal(16).astype(np.float32)
    ib1 = rng.integers(-2 ** 29, 2 ** 29, 4).astype(np.int32)
    ib2 = rng.integers(-2 ** 29, 2 ** 29, 16).astype(np.int32)
    for nm, blk, dims, as_int in (("f1", fb1, 1, False), ("f2", fb2, 2, False),
                                  ("i1", ib1, 1, True), ("i2", ib2, 2, True)):
        buf, bits = block_api(z, blk, dims, 8.0, as_int)
        data["block_in_" + nm] = blk
        data["block_out_" + nm] = buf
        data["block_bits_" + nm] = np.array([bits], np.uint32)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "zfp_golden.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes,", len(data), "arrays")


if __name__ == "__main__":
    sys.exit(main())
