"""Compress -> comm -> decompress pipeline -- mirror of the reference's impls/overlap.py.

One GPU: the comm step is the identity copy and the chunks run back to back on the current
stream (no comm streams to overlap with)."""
import torch

from . import compressor as _ck

MAX_NUM_SPLIT = 32     # AllToAllStatus.max_num_split of the reference (communicate.py)


class Compress(torch.autograd.Function):
    # overlap.py:12-21
    @staticmethod
    def forward(ctx, input, compress_name, comm_name):
        return _ck.compress_operation(input, compress_name, comm_name)

    @staticmethod
    def backward(ctx, grad):
        return _ck.decompress_operation(grad), None, None


class Decompress(torch.autograd.Function):
    # overlap.py:24-34
    @staticmethod
    def forward(ctx, input, compress_name, comm_name):
        ctx.compress_name = compress_name
        ctx.comm_name = comm_name
        return _ck.decompress_operation(input)

    @staticmethod
    def backward(ctx, grad):
        return _ck.compress_operation(grad, ctx.compress_name, ctx.comm_name), None, None


class Comm(torch.autograd.Function):
    # overlap.py:37-44
    @staticmethod
    def forward(ctx, input):
        return _ck.comm_operation(input)

    @staticmethod
    def backward(ctx, grad):
        return _ck.comm_operation(grad)


def a2a_ffn_overlap_forward(input, expert_fn, a2a_ffn_overlap_degree, use_2dh, group, compress_name,
                            comm_name):
    # overlap.py:47-76
    split_dim = 1
    assert a2a_ffn_overlap_degree <= MAX_NUM_SPLIT, \
        "Excepting a2a_ffn_overlap_degree (%d) <= AllToAllStatus.max_num_split (%d)." % (
            a2a_ffn_overlap_degree, MAX_NUM_SPLIT)
    assert input.shape[split_dim] % a2a_ffn_overlap_degree == 0, \
        "Excepting input.shape[%d] (%d) be multiple of a2a_ffn_overlap_degree (%d)." % (
            split_dim, input.shape[split_dim], a2a_ffn_overlap_degree)
    split_size = input.shape[split_dim] // a2a_ffn_overlap_degree
    input_split = list(input.split(split_size, dim=split_dim))
    _ck.clear_ptr_lst()

    for i in range(a2a_ffn_overlap_degree):
        input_split[i] = input_split[i].contiguous()
        input_split[i] = Compress.apply(input_split[i], compress_name, comm_name)
        input_split[i] = Comm.apply(input_split[i])

    for i in range(a2a_ffn_overlap_degree):
        input_split[i] = Decompress.apply(input_split[i], compress_name, comm_name)
        input_split[i] = expert_fn(input_split[i])
        input_split[i] = Compress.apply(input_split[i], compress_name, comm_name)
        input_split[i] = Comm.apply(input_split[i])
    for i in range(a2a_ffn_overlap_degree):
        input_split[i] = Decompress.apply(input_split[i], compress_name, comm_name)
    return torch.cat(input_split, dim=split_dim).contiguous()
