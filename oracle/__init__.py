"""CPU oracle for the PlanMoE MoE data path -- TEST INFRASTRUCTURE ONLY.

ctypes/numpy front end of ``oracle/planmoe_oracle.c``.  Only the test suite, the smoke
check and the benchmark's ``cpu_baseline`` leg may import this package; the product
(``planmoe_amd``) never does and fails loudly when its HIP library is missing.

All arrays are numpy.  bf16 data travels as ``uint16`` bit patterns (torch tensors convert
with ``t.view(torch.int16).numpy().view(numpy.uint16)``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libplanmoe_oracle.so")


def build(force=False):
    """Compile the C restatement with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "planmoe_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libplanmoe_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_gshard_loss.restype = ctypes.c_double
        _lib.orc_zfp_max_bytes.restype = ctypes.c_uint64
        _lib.orc_zfp_stream_bytes.restype = ctypes.c_uint64
        _lib.orc_capacity.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


_FT = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}


# --------------------------------------------------------------------------- sparse kernels
def dispatch(gate, idx, loc, x, dispatched, capacity):
    """dispatched[idx*C+loc] += gate * x  (in place, one choice plane)."""
    sfx = _FT[x.dtype]
    T, H = x.shape
    getattr(lib(), "orc_dispatch_" + sfx)(_p(_c(gate, x.dtype)), _p(_c(idx, np.int32)),
                                          _p(_c(loc, np.int32)), _p(x), _p(dispatched),
                                          ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(capacity))
    return dispatched


def gather(gate, idx, loc, dispatched, samples, capacity):
    """out[t] = gate[t] * dispatched[idx*C+loc] or zeros (one choice plane)."""
    sfx = _FT[dispatched.dtype]
    H = dispatched.shape[-1]
    out = np.empty((samples, H), dtype=dispatched.dtype)
    getattr(lib(), "orc_gather_" + sfx)(_p(_c(gate, dispatched.dtype)), _p(_c(idx, np.int32)),
                                        _p(_c(loc, np.int32)), _p(out), _p(dispatched),
                                        ctypes.c_int(samples), ctypes.c_int(H),
                                        ctypes.c_int(capacity))
    return out


def bwd_gate(idx, loc, x, dispatched, capacity):
    """grad_gate[t] = <dispatched[idx*C+loc], x[t]> summed sequentially in x's dtype."""
    sfx = _FT[x.dtype]
    T, H = x.shape
    out = np.empty((T,), dtype=x.dtype)
    getattr(lib(), "orc_bwd_gate_" + sfx)(_p(out), _p(_c(idx, np.int32)), _p(_c(loc, np.int32)),
                                          _p(x), _p(dispatched), ctypes.c_int(T), ctypes.c_int(H),
                                          ctypes.c_int(capacity))
    return out


def encode(x, idxs, locs, gates, experts, capacity):
    """All choice planes of GatingEncoder.forward: zeros, then one dispatch per plane.
    gates=None means the all-ones helper (is_postscore)."""
    T, H = x.shape
    out = np.zeros((experts * capacity, H), dtype=x.dtype)
    for j in range(len(idxs)):
        g = np.ones((T,), dtype=x.dtype) if gates is None else gates[j]
        dispatch(g, idxs[j], locs[j], x, out, capacity)
    return out


def decode(expert_out, idxs, locs, gates, samples, capacity):
    """GatingDecoder.forward: per-plane gathers summed left to right."""
    acc = None
    for j in range(len(idxs)):
        g = np.ones((samples,), dtype=expert_out.dtype) if gates is None else gates[j]
        y = gather(g, idxs[j], locs[j], expert_out, samples, capacity)
        acc = y if acc is None else acc + y
    return acc


# --------------------------------------------------------------------------- routing
def cumsum_sub_one(mask):
    mask = _c(mask, np.int32)
    out = np.empty_like(mask)
    lib().orc_cumsum_sub_one(_p(mask), _p(out), ctypes.c_int(mask.shape[0]),
                             ctypes.c_int(mask.shape[1]))
    return out


def capacity(samples, experts, top_k, capacity_factor=1.0, alignment=1):
    return lib().orc_capacity(ctypes.c_int(samples), ctypes.c_int(experts), ctypes.c_int(top_k),
                              ctypes.c_double(capacity_factor), ctypes.c_int(alignment))


def route_topk(scores, top_k, normalize_gate=True):
    """scores: float32 [T,E] or uint16 (bf16 bits) [T,E].
    Returns indices[k,T] int32, locations[k,T] int32, gates[k,T] (scores dtype), counts[k,E]."""
    is_bf16 = scores.dtype == np.uint16
    scores = np.ascontiguousarray(scores)
    T, E = scores.shape
    k = min(top_k, E)
    idx = np.empty((k, T), np.int32)
    loc = np.empty((k, T), np.int32)
    gates = np.empty((k, T), scores.dtype)
    counts = np.empty((k, E), np.int32)
    lib().orc_route_topk(_p(scores), ctypes.c_int(int(is_bf16)), ctypes.c_int(T), ctypes.c_int(E),
                         ctypes.c_int(k), ctypes.c_int(int(normalize_gate)), _p(idx), _p(loc),
                         _p(gates), _p(counts))
    return idx, loc, gates, counts


def route_locations(indices, experts, order=None):
    """indices int32 [k,T]; order int32 [T] or None.  Returns locations[k,T], counts[k,E]."""
    indices = _c(indices, np.int32)
    k, T = indices.shape
    loc = np.empty((k, T), np.int32)
    counts = np.empty((k, experts), np.int32)
    o = _c(order, np.int32) if order is not None else None
    lib().orc_route_locations(_p(indices), ctypes.c_int(T), ctypes.c_int(experts), ctypes.c_int(k),
                              _p(o) if o is not None else None, _p(loc), _p(counts))
    return loc, counts


def gshard_loss(scores, first_choice):
    is_bf16 = scores.dtype == np.uint16
    scores = np.ascontiguousarray(scores)
    T, E = scores.shape
    return lib().orc_gshard_loss(_p(scores), ctypes.c_int(int(is_bf16)),
                                 _p(_c(first_choice, np.int32)), ctypes.c_int(T), ctypes.c_int(E))


def softmax(logits):
    logits = _c(logits, np.float32)
    out = np.empty_like(logits)
    lib().orc_softmax_f32(_p(logits), _p(out), ctypes.c_int(logits.shape[0]),
                          ctypes.c_int(logits.shape[1]))
    return out


def gate_logits(x, wg):
    """float64 logits of x[T,M] . wg[E,M]^T; operands float32 or bf16 bits (uint16)."""
    is_bf16 = x.dtype == np.uint16
    x = np.ascontiguousarray(x)
    wg = np.ascontiguousarray(wg)
    out = np.empty((x.shape[0], wg.shape[0]), np.float64)
    lib().orc_gate_logits(_p(x), _p(wg), ctypes.c_int(int(is_bf16)), _p(out),
                          ctypes.c_int(x.shape[0]), ctypes.c_int(x.shape[1]),
                          ctypes.c_int(wg.shape[0]))
    return out


# --------------------------------------------------------------------------- int8 codec
def int8_compress(x):
    """x: [..., M] float32 or uint16 (bf16 bits). Returns codes uint8 [..., M], bias, scale [..., 1]."""
    x = np.ascontiguousarray(x)
    M = x.shape[-1]
    rows = x.size // M
    codes = np.empty(x.shape, np.uint8)
    bias = np.empty(x.shape[:-1] + (1,), x.dtype)
    scale = np.empty(x.shape[:-1] + (1,), x.dtype)
    fn = lib().orc_int8_compress_bf16 if x.dtype == np.uint16 else lib().orc_int8_compress_f32
    fn(_p(x), ctypes.c_int64(rows), ctypes.c_int(M), _p(codes), _p(bias), _p(scale))
    return codes, bias, scale


def int8_decompress(codes, bias, scale):
    codes = np.ascontiguousarray(codes)
    M = codes.shape[-1]
    rows = codes.size // M
    out = np.empty(codes.shape, bias.dtype)
    fn = lib().orc_int8_decompress_bf16 if bias.dtype == np.uint16 else lib().orc_int8_decompress_f32
    fn(_p(codes), _p(np.ascontiguousarray(bias)), _p(np.ascontiguousarray(scale)),
       ctypes.c_int64(rows), ctypes.c_int(M), _p(out))
    return out


# --------------------------------------------------------------------------- zfp codec
def zfp_max_bytes(dims, nx, ny, rate=8.0):
    return int(lib().orc_zfp_max_bytes(ctypes.c_int(dims), ctypes.c_int64(nx), ctypes.c_int64(ny),
                                       ctypes.c_double(rate)))


def zfp_stream_bytes(dims, nx, ny, rate=8.0):
    return int(lib().orc_zfp_stream_bytes(ctypes.c_int(dims), ctypes.c_int64(nx),
                                          ctypes.c_int64(ny), ctypes.c_double(rate)))


def zfp_compress(field, dims=2, rate=8.0):
    """field: float32 [ny, nx] (nx fastest).  Returns the header-less stream as uint8."""
    field = _c(field, np.float32)
    ny, nx = field.reshape(-1, field.shape[-1]).shape
    out = np.zeros((zfp_stream_bytes(dims, nx, ny, rate),), np.uint8)
    rc = lib().orc_zfp_compress(_p(field), ctypes.c_int(dims), ctypes.c_int64(nx),
                                ctypes.c_int64(ny), ctypes.c_double(rate), _p(out))
    if rc != 0:
        raise ValueError("zfp fails.")
    return out


def zfp_decompress(stream, ny, nx, dims=2, rate=8.0):
    stream = _c(stream, np.uint8)
    out = np.empty((ny, nx), np.float32)
    rc = lib().orc_zfp_decompress(_p(stream), ctypes.c_int(dims), ctypes.c_int64(nx),
                                  ctypes.c_int64(ny), ctypes.c_double(rate), _p(out))
    if rc != 0:
        raise ValueError("zfp fails.")
    return out


def zfp_encode_block(block, dims=2, rate=8.0):
    """One block through the block coder: float32 input -> float path, int32 input -> integer
    path (the library's zfp_encode_block_float_N / zfp_encode_block_int32_N).  64-byte buffer."""
    out = np.zeros((64,), np.uint8)
    if block.dtype == np.int32:
        lib().orc_zfp_encode_block_int32(_p(_c(block, np.int32)), ctypes.c_int(dims),
                                         ctypes.c_double(rate), _p(out))
    else:
        lib().orc_zfp_encode_block_float(_p(_c(block, np.float32)), ctypes.c_int(dims),
                                         ctypes.c_double(rate), _p(out))
    return out


# --------------------------------------------------------------------------- GPULZ ("lz") codec
LZ_BLOCK_BYTES = 2048


def lz_compress(x):
    """x: float32, size a multiple of 512.  Returns (flag_offsets int32 [B+1], data_offsets int32
    [B+1], flags uint8 [B*64], data uint8 [B*2048]); both byte arrays zero beyond their totals."""
    x = _c(x, np.float32).reshape(-1)
    assert x.size % 512 == 0
    B = x.size // 512
    fo = np.zeros((B + 1,), np.int32)
    do = np.zeros((B + 1,), np.int32)
    flags = np.zeros((B * 64,), np.uint8)
    data = np.zeros((B * 2048,), np.uint8)
    lib().orc_lz_compress(_p(x), ctypes.c_int64(B), _p(fo), _p(do), _p(flags), _p(data))
    return fo, do, flags, data


def lz_decompress(flag_offsets, data_offsets, flags, data):
    fo = _c(flag_offsets, np.int32)
    B = fo.size - 1
    out = np.zeros((B * 512,), np.float32)
    rc = lib().orc_lz_decompress(_p(out), ctypes.c_int64(B), _p(fo), _p(_c(data_offsets, np.int32)),
                                 _p(_c(flags, np.uint8)), _p(_c(data, np.uint8)))
    if rc != 0:
        raise ValueError("lz stream is inconsistent")
    return out
