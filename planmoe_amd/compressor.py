"""Compressor plug-ins and their registry -- Python mirror of the reference's
custom/compressor/* classes and of the compress / comm / decompress operations of
custom/custom_kernel.cpp:194-288 (the pybind surface of ``schemoe_custom_kernel``).

Objects are stateful and single use, exactly as in the reference: ``compress`` records what
``decompress`` needs.  With one GPU the all-to-all is the identity: ``comm_operation`` hands the
send buffers over as the receive buffers, or (``SINGLE_RANK_COMM_COPIES``) ``all_to_all`` copies
the send buffer into ``g_output`` and the per-row state into its receive-side twins, on a comm
stream under the reference's event protocol."""
import torch

from . import ops
from ._lib import PlanMoEError


# One rank: what the all-to-all delivers is what was sent.  With False the send buffers are handed
# over as the receive buffers (no device copy); with True they are copied into g_output, as a
# one-rank all_to_all of the reference would (naive.cpp:11-27).
SINGLE_RANK_COMM_COPIES = False


class AbstractComm:
    """comm/abstract.h:10-24 reduced to one rank: all_to_all(input, output, length) copies
    `length` bytes (naive.cpp:11-27 with g_world_size == 1)."""

    def __init__(self, name="naive"):
        self.name = name
        self.g_world_size, self.g_world_rank, self.g_local_size, self.g_local_rank = 1, 0, 1, 0

    def all_to_all(self, input, output, length):
        src = input.reshape(-1).view(torch.uint8)
        dst = output.reshape(-1).view(torch.uint8)
        dst[:length].copy_(src[:length])

    def pre_comm(self, input):
        pass


class AbstractCompressor:
    """compressor/abstract.h:11-22."""

    def __init__(self, comm_ptr):
        self.comm_ptr = comm_ptr
        self.g_output = None

    def compress(self, input):
        raise NotImplementedError

    def decompress(self, input):
        raise NotImplementedError

    def all_to_all(self, input, output):
        raise NotImplementedError

    def adopt(self, input):
        """One rank, no copy: the receive-side state is the send-side state."""
        self.g_output = input

    def pre_comm(self, stream):
        pass


class NoCompressor(AbstractCompressor):
    """compressor/no.cpp:3-20."""

    def compress(self, input):
        self.g_output = torch.empty_like(input)
        return input

    def decompress(self, input):
        return input

    def all_to_all(self, input, output):
        self.comm_ptr.all_to_all(input, output, input.numel() * input.element_size())


class Int8Compressor(AbstractCompressor):
    """compressor/int8.cpp:7-74: per-row min/max affine codes in uint8, shipped in an
    fp32-typed buffer of (N + 3) / 4 elements; bias and scale stay in the input dtype."""

    def compress(self, input):
        self.sizes = list(input.shape)
        self.dtype = input.dtype
        self.length = input.numel()
        fp_output = torch.empty(((self.length + 3) // 4,), dtype=torch.float32, device=input.device)
        _, self.bias, self.scale = ops.int8_compress(input.contiguous(), codes_out=fp_output)
        self.g_bias = torch.empty_like(self.bias)
        self.g_scale = torch.empty_like(self.scale)
        self.g_output = torch.empty_like(fp_output)
        return fp_output

    def decompress(self, input):
        codes = input.view(torch.uint8)[:self.length].view(self.sizes)
        return ops.int8_decompress(codes, self.g_bias, self.g_scale)

    def all_to_all(self, input, output):
        self.comm_ptr.all_to_all(input, output, self.length)
        self.comm_ptr.all_to_all(self.bias, self.g_bias, self.bias.numel() * self.bias.element_size())
        self.comm_ptr.all_to_all(self.scale, self.g_scale, self.scale.numel() * self.scale.element_size())

    def adopt(self, input):
        self.g_output, self.g_bias, self.g_scale = input, self.bias, self.scale


class ZfpCompressor(AbstractCompressor):
    """compressor/zfpc.cpp:23-97: zfp fixed rate (default 8 bits/value, zfpc.h:17) on the
    tensor's storage read as fp32, 2-D field nx = sizes[2], ny = sizes[0] * sizes[1]; the
    stream travels in an fp16-typed buffer of (bufsize + 1) / 2 elements."""

    def __init__(self, comm_ptr, compress_rate=8.0):
        super().__init__(comm_ptr)
        self.compress_rate = float(compress_rate)

    def set_compress_rate(self, compress_rate):
        self.compress_rate = float(compress_rate)

    def compress(self, input):
        self.sizes = list(input.shape)
        if len(self.sizes) != 3 or any(s % 4 for s in self.sizes):
            raise PlanMoEError("zfp fails.")
        if input.dtype != torch.float32:
            raise PlanMoEError("ZfpCompressor: the codec reads the buffer as fp32 (zfpc.cpp:31); "
                               "pass a float32 tensor")
        nx, ny = self.sizes[2], self.sizes[1] * self.sizes[0]
        bufsize = ops.zfp_max_bytes(2, nx, ny, self.compress_rate)
        output = torch.zeros(((bufsize + 1) // 2,), dtype=torch.float16, device=input.device)
        ops.zfp_compress(input.contiguous(), nx, ny, 2, self.compress_rate, out=output.view(torch.uint8))
        self.length = ops.zfp_stream_bytes(2, nx, ny, self.compress_rate)
        self.g_output = torch.empty_like(output)
        return output

    def decompress(self, input):
        nx, ny = self.sizes[2], self.sizes[1] * self.sizes[0]
        out = ops.zfp_decompress(input.view(torch.uint8), nx, ny, 2, self.compress_rate)
        return out.view(self.sizes)

    def all_to_all(self, input, output):
        self.comm_ptr.all_to_all(input, output, self.length)


class LzCompressor(AbstractCompressor):
    """compressor/lz.cpp:3-73: GPULZ lossless codec.  compress keeps the four stream tensors and
    returns its input; all_to_all ships the four tensors whole; decompress decodes into the
    tensor it is handed (g_output, a zeroed twin of the input).  float32 only, as the
    reference's data_ptr<float>() (gpulz.cu:15,451)."""

    def compress(self, input):
        if input.dtype != torch.float32:
            raise PlanMoEError("LzCompressor: expected scalar type Float but found %s" % input.dtype)
        x = input.contiguous()
        (self.flagArrOffsetGlobal, self.compressedDataOffsetGlobal, self.flagArrGlobal,
         self.compressedDataGlobal) = ops.lz_compress(x)
        self.g_flagArrOffsetGlobal = torch.empty_like(self.flagArrOffsetGlobal)
        self.g_compressedDataOffsetGlobal = torch.empty_like(self.compressedDataOffsetGlobal)
        self.g_flagArrGlobal = torch.empty_like(self.flagArrGlobal)
        self.g_compressedDataGlobal = torch.empty_like(self.compressedDataGlobal)
        self.g_output = torch.zeros_like(x)
        return input

    def decompress(self, input):
        if input.dtype != torch.float32:
            raise PlanMoEError("LzCompressor: expected scalar type Float but found %s" % input.dtype)
        return ops.lz_decompress(input, self.g_flagArrOffsetGlobal, self.g_compressedDataOffsetGlobal,
                                 self.g_flagArrGlobal, self.g_compressedDataGlobal)

    def all_to_all(self, input, output):
        for src, dst in ((self.flagArrOffsetGlobal, self.g_flagArrOffsetGlobal),
                         (self.compressedDataOffsetGlobal, self.g_compressedDataOffsetGlobal),
                         (self.flagArrGlobal, self.g_flagArrGlobal),
                         (self.compressedDataGlobal, self.g_compressedDataGlobal)):
            self.comm_ptr.all_to_all(src, dst, src.numel() * src.element_size())

    def adopt(self, input):
        # g_output stays the zeroed twin the decoder writes into
        self.g_flagArrOffsetGlobal, self.g_compressedDataOffsetGlobal = self.flagArrOffsetGlobal, self.compressedDataOffsetGlobal
        self.g_flagArrGlobal, self.g_compressedDataGlobal = self.flagArrGlobal, self.compressedDataGlobal


_registered = {}


def register(name, factory):
    """Add a compressor under `name`: factory(comm_ptr) -> AbstractCompressor.  Registered names
    are looked up before the built-in ones, as in the C++ extension's registry."""
    if not callable(factory):
        raise TypeError("register: factory must be callable (a subclass of AbstractCompressor or a function of comm_ptr)")
    _registered[str(name)] = factory


def registered():
    return sorted(_registered)


def get_compressor(name, comm_ptr):
    # custom_kernel.cpp:194-207
    if name in _registered:
        return _registered[name](comm_ptr)
    if name == "int8":
        return Int8Compressor(comm_ptr)
    if name == "zfp":
        return ZfpCompressor(comm_ptr)
    if name == "lz":
        return LzCompressor(comm_ptr)
    return NoCompressor(comm_ptr)


def get_comm(name):
    # custom_kernel.cpp:209-224: every algorithm is the identity on one GPU
    return AbstractComm(name)


# custom_kernel.cpp:226-288 -------------------------------------------------------------------
# When the comm step copies (SINGLE_RANK_COMM_COPIES), it runs on a comm stream of its own, at the
# priority of the compute stream, under the reference's event protocol: the event of a slot is
# recorded behind the compress (custom_kernel.cpp:251-253), the comm stream waits for it, carries
# the copies and records it again (:269-275), the decompress makes the compute stream wait for it
# (:281-283).  With a2a_ffn_overlap_degree > 1 a chunk's copy then runs beside the next chunk's
# compress.  Tensors that the comm stream touches are marked with record_stream, as int8.cpp:25-42
# does, so that the allocator does not hand their memory out while the copy is in flight.
_compress_ptr_lst = []
_events = []
_comm_cnt = 0
_decompress_cnt = 0
_comm_streams = {}


def comm_stream(device):
    """The comm stream of `device` (the reference's g_nccl_stream), created on first use."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _comm_streams:
        _comm_streams[index] = torch.cuda.Stream(device=index)          # default priority
    return _comm_streams[index]


def _tensors_of(c):
    return [v for v in vars(c).values() if isinstance(v, torch.Tensor) and v.is_cuda]


def clear_ptr_lst():
    global _comm_cnt, _decompress_cnt
    _compress_ptr_lst.clear()
    _events.clear()
    _comm_cnt = 0
    _decompress_cnt = 0


def compress_operation(input, name, comm_name):
    _compress_ptr_lst.append(get_compressor(name, get_comm(comm_name)))
    out = _compress_ptr_lst[-1].compress(input)
    event = None
    if SINGLE_RANK_COMM_COPIES and out.is_cuda:
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(out.device))
        side = comm_stream(out.device)
        for t in [out] + _tensors_of(_compress_ptr_lst[-1]):
            t.record_stream(side)
    _events.append(event)
    return out


def comm_operation(input):
    global _comm_cnt
    idx = _comm_cnt
    if idx >= len(_compress_ptr_lst) or _compress_ptr_lst[idx] is None:
        raise PlanMoEError("comm_operation: no matching compress_operation")
    _comm_cnt += 1
    c = _compress_ptr_lst[idx]
    c.pre_comm(None)
    if c.comm_ptr.g_world_size == 1 and not SINGLE_RANK_COMM_COPIES:
        c.adopt(input)
    elif _events[idx] is not None:
        side = comm_stream(input.device)
        side.wait_event(_events[idx])
        with torch.cuda.stream(side):
            c.all_to_all(input, c.g_output)
        _events[idx].record(side)
    else:
        c.all_to_all(input, c.g_output)
    return c.g_output


def decompress_operation(input):
    global _decompress_cnt
    idx = _decompress_cnt
    if idx >= len(_compress_ptr_lst) or _compress_ptr_lst[idx] is None:
        raise PlanMoEError("decompress_operation: no matching compress_operation")
    _decompress_cnt += 1
    if _events[idx] is not None and input.is_cuda:
        torch.cuda.current_stream(input.device).wait_event(_events[idx])
    output = _compress_ptr_lst[idx].decompress(input)
    _compress_ptr_lst[idx] = None
    return output
