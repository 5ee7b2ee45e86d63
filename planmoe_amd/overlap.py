"""Compress -> comm -> decompress pipeline -- mirror of the reference's impls/overlap.py.

One GPU: the comm step is a copy on the device's comm stream between two events
(compressor.comm_operation), so with a2a_ffn_overlap_degree > 1 a chunk's copy runs beside the
next chunk's compress; the fused int8 / zfp paths below collapse the steps either side of it."""
import torch

from . import compressor as _ck
from . import ops
from .gates import weight_grad

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
    if compress_name not in ("int8", "zfp", "lz") and not _ck.SINGLE_RANK_COMM_COPIES:
        # NoCompressor on one rank: compress, comm and decompress all return their argument
        # (no.cpp:3-20, the comm hand-over), so the six autograd nodes around the experts are pure
        # host work; only the experts' slicing remains
        _ck.clear_ptr_lst()
        return _experts_in_chunks(expert_fn, input, a2a_ffn_overlap_degree).contiguous()
    split_size = input.shape[split_dim] // a2a_ffn_overlap_degree
    # (one slice: the tensor itself -- the backward of a split is a cat, i.e. a copy of the whole gradient)
    input_split = [input] if a2a_ffn_overlap_degree == 1 else list(input.split(split_size, dim=split_dim))
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
    if a2a_ffn_overlap_degree == 1:
        return input_split[0].contiguous()              # nothing to put together
    return torch.cat(input_split, dim=split_dim).contiguous()


def _experts_in_chunks(expert_fn, buf, degree):
    """The experts see the [E, C, M] buffer in a2a_ffn_overlap_degree slices along the capacity, as in
    a2a_ffn_overlap_forward.  The codecs work row by row (int8) or on 4-row blocks that never
    straddle a slice (zfp, capacity aligned to 4 * degree), so coding the whole buffer at once
    gives each slice the values it would get on its own."""
    if degree == 1:
        return expert_fn(buf)
    assert degree <= MAX_NUM_SPLIT, \
        "Excepting a2a_ffn_overlap_degree (%d) <= AllToAllStatus.max_num_split (%d)." % (degree, MAX_NUM_SPLIT)
    assert buf.shape[1] % degree == 0, \
        "Excepting input.shape[%d] (%d) be multiple of a2a_ffn_overlap_degree (%d)." % (1, buf.shape[1], degree)
    return torch.cat([expert_fn(c.contiguous()) for c in buf.split(buf.shape[1] // degree, dim=1)], dim=1)


# ------------------------------------------------------------------------------ fused int8 path
# With the "int8" compressor the steps either side of the all-to-all collapse (for any
# a2a_ffn_overlap_degree: only the expert call is sliced, see _experts_in_chunks):
#   send side     fast_encode + Compress      -> one pass (planmoe_dispatch_int8)
#   receive side  Decompress + fast_decode    -> one pass (planmoe_combine_int8)
# and the same two fusions serve the backward pass (Decompress.backward compresses the gradient,
# Compress.backward decompresses it, overlap.py:19-21, 32-34).  Results are bit-identical to the
# step-by-step pipeline; FUSE_INT8 = False keeps the reference's structure.
FUSE_INT8 = True
# one step further: the gate GEMM and the routing join the send side (planmoe_forward_int8)
FUSE_GATE = True
# and with this the send side is the one-launch kernel that reads the tokens once
# (planmoe_forward_int8_single) wherever it serves the shape.  The library keeps such launches on
# one device apart (each waits for the one before it, whatever their streams), and the layer
# reads the kernel's give-up flag before it uses any output: a launch whose work-groups did not
# all become resident in time (another long kernel holding compute units) is run again through the
# two launches of planmoe_forward_int8.  That read is one host synchronisation per forward pass;
# under a graph capture, where the host cannot read, the layer takes the two launches.
FORWARD_SINGLE_LAUNCH = True
# inference (no autograd) with the built-in expert FFN in bf16: the receive side hands the int8
# codes straight to the experts' first GEMM (planmoe_ffn_fc1_int8, which multiplies the values the
# decompressor would have written) instead of decompressing them into a tensor first.  Off by
# default since the experts' GEMMs are planmoe_gemm_nt_bf16: at 8 x 5120 x 4096 x 4096 the decode in
# the first GEMM's prologue makes that GEMM 1.9 ms, against 0.07 ms of planmoe_int8_decompress
# plus 1.35 ms of the plain GEMM; worth it only where the decompressed tensor's memory is what counts.
FFN_FROM_CODES = False
# the faster affine form of that GEMM (codes on the matrix cores, scale / bias in the epilogue):
# not bit-equal to decompress + GEMM, so it is something to opt into
FFN_FROM_CODES_AFFINE = False


def ffn_from_codes_fn(module, x, degree, reserve_dims):
    """The experts as a function of (codes, bias, scale) [E, C, ...] when the layer's receive side
    may skip the decompress, else None."""
    from .experts import FusedExpertsNetwork
    if not (FFN_FROM_CODES and not torch.is_grad_enabled() and type(module) is FusedExpertsNetwork and degree == 1 and
            reserve_dims == 1 and x.is_cuda and x.dtype == torch.bfloat16 and x.shape[-1] % 64 == 0 and
            module.hidden_size_per_expert % 128 == 0 and module.batched_fc1_w.dtype == torch.bfloat16 and
            module.output_dim in (None, x.shape[-1])):
        return None
    if FFN_FROM_CODES_AFFINE:
        return lambda codes, bias, scale: module.forward_from_codes(codes, bias, scale, exact=False)
    return module.forward_from_codes


class _GaveUp:
    """The give-up flag of a one-launch forward on its way to the host without stalling the stream:
    an asynchronous copy into pinned memory and an event behind it.  Asked at the end of the
    layer's forward pass, when the launch is long done, the answer costs no wait and the host has
    been free to enqueue everything behind the launch in the meantime."""
    _slots = {}

    def __init__(self, flag):
        dev = flag.device.index
        ring = _GaveUp._slots.get(dev)
        if ring is None:
            ring = _GaveUp._slots[dev] = [torch.zeros(64, dtype=torch.int32).pin_memory(), 0]
        ring[1] = (ring[1] + 1) % 64
        self.host = ring[0][ring[1]:ring[1] + 1]
        self.host.copy_(flag.reshape(1), non_blocking=True)
        self.event = torch.cuda.Event()
        self.event.record()

    def __bool__(self):
        self.event.synchronize()
        return int(self.host) != 0


def forward_int8_send_side(x, w, top_k, capacity, fp32_gate, normalize_gate, single=True, checks=None, **want):
    """ops.forward_int8_single where it serves the shape, else ops.forward_int8.  A one-launch result
    is valid only if no work-group gave up: with `checks` (a list) the flag's _GaveUp is appended for
    the caller to ask later (and to run the pass again with single=False if it is set); without, the
    flag is read here and the two launches run in its place if need be.  Never hands out a partial
    result unchecked."""
    if (single and FORWARD_SINGLE_LAUNCH and ops.forward_int8_single_serves(x, w, top_k, fp32_gate) and
            not torch.cuda.is_current_stream_capturing()):
        out = ops.forward_int8_single(x, w, top_k, capacity, fp32_gate=fp32_gate, normalize_gate=normalize_gate, **want)
        flag = out.pop("gave_up")
        if checks is not None:
            checks.append(_GaveUp(flag))
            return out
        if int(flag) == 0:
            return out
    return ops.forward_int8(x, w, top_k, capacity, fp32_gate=fp32_gate, normalize_gate=normalize_gate, **want)


class _EncodeInt8(torch.autograd.Function):
    """Decompress(Comm(Compress(fast_encode(x)))) for the all-ones gate helper (is_postscore)."""

    @staticmethod
    def forward(ctx, x, indices, locations, experts, capacity):
        codes, bias, scale = ops.dispatch_int8(x, list(indices), list(locations), None, experts, capacity)
        ctx.save_for_backward(indices, locations)
        ctx.samples, ctx.capacity = x.shape[0], capacity
        return ops.int8_decompress(codes, bias, scale)

    @staticmethod
    def backward(ctx, grad):
        indices, locations = ctx.saved_tensors
        codes, bias, scale = ops.int8_compress(grad.contiguous())
        dx = ops.combine_int8(codes, bias, scale, list(indices), list(locations), None, ctx.samples, ctx.capacity)
        return dx, None, None, None, None


class _DecodeInt8(torch.autograd.Function):
    """fast_decode(Decompress(Comm(Compress(y)))) with the gates applied at decode."""

    @staticmethod
    def forward(ctx, y, indices, locations, experts, capacity, samples, *gates):
        codes, bias, scale = ops.int8_compress(y.contiguous())
        out = ops.combine_int8(codes, bias, scale, list(indices), list(locations), list(gates), samples, capacity)
        ctx.save_for_backward(codes, bias, scale, indices, locations, *gates)
        ctx.experts, ctx.capacity = experts, capacity
        return out

    @staticmethod
    def backward(ctx, grad_out):
        codes, bias, scale, indices, locations, *gates = ctx.saved_tensors
        # the tensor fast_decode consumed is decoded from its codes on the fly
        gcodes, gbias, gscale, grad_gates = ops.combine_bwd_int8(
            grad_out.contiguous(), (codes, bias, scale), list(indices), list(locations), list(gates), ctx.experts,
            ctx.capacity)
        grad_y = ops.int8_decompress(gcodes, gbias, gscale)
        return (grad_y, None, None, None, None, None,
                *[grad_gates[j].to(g.dtype) for j, g in enumerate(gates)])


class _GateRouteEncodeInt8(torch.autograd.Function):
    """Gate GEMM + softmax / top-k / capacity slots + fast_encode + Compress in the one launch of
    planmoe_forward_int8_single (the two of planmoe_forward_int8 where that does not serve the
    shape), then Decompress.  Outputs: the [E*C, M] tensor the experts see, the
    gates [k, T] and l_aux (all three differentiable), indices and locations [k, T].
    Backward: the dispatch gradient as in _EncodeInt8; gates and l_aux go back through
    planmoe_route_bwd to the logits and from there into x and the gate weight (library GEMMs)."""

    @staticmethod
    def forward(ctx, x, w, top_k, capacity, fp32_gate, normalize_gate, single=True, checks=None):
        out = forward_int8_send_side(x, w, top_k, capacity, fp32_gate, normalize_gate, single=single, checks=checks,
                                     want_scores=True, want_counts=True)
        ctx.save_for_backward(x, w, out["scores"], out["indices"], out["locations"], out["counts"])
        ctx.capacity, ctx.normalize_gate = capacity, normalize_gate
        ctx.mark_non_differentiable(out["indices"], out["locations"])
        y = ops.int8_decompress(out["codes"], out["bias"], out["scale"])
        return y, out["gates"], out["l_aux"], out["indices"], out["locations"]

    @staticmethod
    def backward(ctx, grad_y, grad_gates, grad_l_aux, *unused):
        x, w, scores, indices, locations, counts = ctx.saved_tensors
        dx = None
        if grad_y is not None:
            codes, bias, scale = ops.int8_compress(grad_y.contiguous())
            dx = ops.combine_int8(codes, bias, scale, list(indices), list(locations), None, x.shape[0], ctx.capacity)
        dx, dw = _gate_backward(x, w, scores, indices, counts, ctx.normalize_gate, dx, grad_gates, grad_l_aux)
        return dx, dw, None, None, None, None, None, None


def _gate_backward(x, w, scores, indices, counts, normalize_gate, dx, grad_gates, grad_l_aux):
    """Gradients of the gates and of l_aux back through planmoe_route_bwd to the logits, and from
    there into x (added to dx, the gradient through the dispatched rows, in the GEMM's epilogue)
    and into the gate weight."""
    if grad_gates is None and grad_l_aux is None:
        return dx, None
    if grad_gates is None:
        grad_gates = torch.zeros((indices.shape[0], x.shape[0]), dtype=scores.dtype, device=x.device)
    grad_logits = ops.route_bwd(scores, indices, grad_gates.contiguous(), normalize_gate, grad_l_aux,
                                counts if grad_l_aux is not None else None, through_softmax=True)
    g = grad_logits.to(x.dtype)
    dw = weight_grad(g, x)
    vec = 4 if x.dtype == torch.float32 else 8
    if dx is None:
        dx = g @ w
    elif w.shape[0] <= 8 and x.shape[1] % vec == 0 and dx.is_contiguous():
        ops.gate_dx_accumulate(dx, grad_logits, w)           # one pass over dx instead of a GEMM with K = experts
    else:
        dx.addmm_(g, w)
    return dx, dw


class _GateRouteEncode(torch.autograd.Function):
    """Gate GEMM, routing and fast_encode as one node of the graph for the compressors without an
    int8 send side: x has one consumer, so its two gradients (through the dispatched rows and
    through the gate) meet in the epilogue of one GEMM instead of a pass of their own.
    codec 'plain': x -> the [E * C, M] buffer (planmoe_forward_plain: gate + routing, then a dispatch
                   launch that works out the slots itself);
    codec 'zfp':   x -> Decompress(Comm(Compress(buffer))) (planmoe_dispatch_zfp, as _EncodeZfp).
    Outputs as _GateRouteEncodeInt8."""

    @staticmethod
    def forward(ctx, x, w, top_k, experts, capacity, fp32_gate, normalize_gate, codec):
        if codec == 'zfp':
            out = ops.gate_route(x, w, top_k, fp32_gate=fp32_gate, normalize_gate=normalize_gate,
                                 want_scores=True, want_counts=True)
        else:
            # planmoe_forward_plain: the dispatch launch works out the slots itself (one launch less)
            out = ops.forward_plain(x, w, top_k, capacity, fp32_gate=fp32_gate, normalize_gate=normalize_gate,
                                    want_scores=True, want_counts=True)
        indices, locations = out["indices"], out["locations"]
        ctx.save_for_backward(x, w, out["scores"], indices, locations, out["counts"])
        ctx.experts, ctx.capacity, ctx.normalize_gate, ctx.codec = experts, capacity, normalize_gate, codec
        ctx.mark_non_differentiable(indices, locations)
        if codec == 'zfp':
            stream = ops.dispatch_zfp(x, list(indices), list(locations), None, experts, capacity)
            y = ops.zfp_decompress(stream, x.shape[1], experts * capacity, 2)
        else:
            y = out["dispatched"]
        return y, out["gates"], out["l_aux"], indices, locations

    @staticmethod
    def backward(ctx, grad_y, grad_gates, grad_l_aux, *unused):
        x, w, scores, indices, locations, counts = ctx.saved_tensors
        dx = None
        if grad_y is not None:
            grad_y = grad_y.contiguous()
            if ctx.codec == 'zfp':
                R, M = grad_y.shape
                stream = ops.zfp_compress(grad_y, M, R, 2)
                dx = ops.combine_zfp(stream, list(indices), list(locations), None, x.shape[0], ctx.experts,
                                     ctx.capacity, M)
            else:
                dx = ops.combine_fwd(grad_y, list(indices), list(locations), None, x.shape[0], ctx.capacity)
        dx, dw = _gate_backward(x, w, scores, indices, counts, ctx.normalize_gate, dx, grad_gates, grad_l_aux)
        return dx, dw, None, None, None, None, None, None


def gate_weight_fits(gate, x):
    """The chain's gate GEMM takes the weight in x's dtype.  A weight kept in fp32 next to 16-bit
    activations would have to be rounded for it, which moves tokens near a tie to another expert:
    those layers take the staged gate, which feeds the weight in as two 16-bit parts."""
    return gate.wg.weight.dtype == x.dtype


def gate_route_eligible(x, gate, experts, is_postscore):
    """Gate, routing and encode as one call chain (planmoe_gate_route) for any compressor."""
    from .gates import LinearTopKGate
    vec = 4 if x.dtype == torch.float32 else 8
    return (FUSE_GATE and is_postscore and type(gate) is LinearTopKGate and experts <= 64 and x.is_cuda and
            x.dtype in (torch.float32, torch.bfloat16, torch.float16) and x.shape[-1] % vec == 0 and
            x.shape[0] >= 1 and gate_weight_fits(gate, x))


def gate_route_encode(x, gate, top_k, capacity, normalize_gate, codec):
    """-> (buffer [E * C, M], gates [k, T], l_aux, indices [k, T], locations [k, T])."""
    w = gate.wg.weight
    if w.dtype != x.dtype:
        w = w.to(x.dtype)
    return _GateRouteEncode.apply(x.contiguous(), w.contiguous(), top_k, w.shape[0], capacity,
                                  bool(gate.fp32_gate), bool(normalize_gate), codec)


def fused_gate_eligible(x, gate, experts, compress_name, degree, is_postscore):
    """The whole send side (gate, routing, encode, compress) as planmoe_forward_int8."""
    from .gates import LinearTopKGate
    return (fused_int8_eligible(x, compress_name, degree, is_postscore) and type(gate) is LinearTopKGate and
            experts <= 64 and x.shape[0] >= 1 and gate_weight_fits(gate, x))


def fused_gate_forward(x, gate, top_k, capacity, normalize_gate, expert_fn, degree=1, codes_fn=None, single=True):
    """moe_layer's forward from the gate to the combine for the int8 compressor, the GShard loss
    and plain routing.  Returns (output [T, M], l_aux).  codes_fn (inference only): the experts as a
    function of the codes, see ffn_from_codes_fn.  The one-launch send side is checked at the end
    (by then its flag has long arrived): if a work-group gave up, the pass runs again in two launches."""
    w = gate.wg.weight
    if w.dtype != x.dtype:
        w = w.to(x.dtype)
    experts = w.shape[0]
    x = x.contiguous()
    checks = []
    if codes_fn is not None and not torch.is_grad_enabled():
        out = forward_int8_send_side(x, w.contiguous(), top_k, capacity, bool(gate.fp32_gate), bool(normalize_gate),
                                     single=single, checks=checks)
        M = x.shape[-1]
        y = codes_fn(out["codes"].view(experts, capacity, M), out["bias"].view(experts, capacity, 1),
                     out["scale"].view(experts, capacity, 1))
        codes, bias, scale = ops.int8_compress(y.reshape(experts * capacity, -1).to(x.dtype).contiguous())
        k = out["indices"].shape[0]
        res = ops.combine_int8(codes, bias, scale, list(out["indices"]), list(out["locations"]),
                               [out["gates"][j].float() for j in range(k)], x.shape[0], capacity)
        l_aux = out["l_aux"]
    else:
        y, gates, l_aux, indices, locations = _GateRouteEncodeInt8.apply(x, w.contiguous(), top_k, capacity, bool(gate.fp32_gate),
                                                                         bool(normalize_gate), single, checks)
        y = _experts_in_chunks(expert_fn, y.view(experts, capacity, x.shape[-1]), degree)
        y = y.reshape(experts * capacity, -1).to(x.dtype)
        k = indices.shape[0]
        res = _DecodeInt8.apply(y, indices, locations, experts, capacity, x.shape[0], *[gates[j].float() for j in range(k)])
    if any(bool(c) for c in checks):
        return fused_gate_forward(x, gate, top_k, capacity, normalize_gate, expert_fn, degree, codes_fn, single=False)
    return res, l_aux


# ------------------------------------------------------------------------------ fused zfp path
# With the "zfp" compressor (fp32 data) both sides collapse as well: fast_encode + Compress ->
# planmoe_dispatch_zfp (forward pass and, with the gates, the backward pass of fast_decode);
# Decompress + fast_decode -> planmoe_combine_zfp (forward pass and the backward pass of
# fast_encode).  Bit-identical to the steps.
class _EncodeZfp(torch.autograd.Function):
    """Decompress(Comm(Compress(fast_encode(x)))) for the all-ones gate helper (is_postscore)."""

    @staticmethod
    def forward(ctx, x, indices, locations, experts, capacity):
        R, M = experts * capacity, x.shape[1]
        stream = ops.dispatch_zfp(x, list(indices), list(locations), None, experts, capacity)
        ctx.save_for_backward(indices, locations)
        ctx.samples, ctx.experts, ctx.capacity = x.shape[0], experts, capacity
        return ops.zfp_decompress(stream, M, R, 2)

    @staticmethod
    def backward(ctx, grad):
        indices, locations = ctx.saved_tensors
        R, M = grad.shape
        stream = ops.zfp_compress(grad.contiguous(), M, R, 2)
        dx = ops.combine_zfp(stream, list(indices), list(locations), None, ctx.samples, ctx.experts, ctx.capacity, M)
        return dx, None, None, None, None


class _DecodeZfp(torch.autograd.Function):
    """fast_decode(Decompress(Comm(Compress(y)))) with the gates applied at decode.  The decoded
    buffer is not kept: the backward pass decodes the saved stream (a quarter of its size) again."""

    @staticmethod
    def forward(ctx, y, indices, locations, experts, capacity, samples, *gates):
        R, M = y.shape
        stream = ops.zfp_compress(y.contiguous(), M, R, 2)
        ctx.save_for_backward(stream, indices, locations, *gates)
        ctx.experts, ctx.capacity, ctx.shape = experts, capacity, (R, M)
        return ops.combine_zfp(stream, list(indices), list(locations), list(gates), samples, experts, capacity, M)

    @staticmethod
    def backward(ctx, grad_out):
        stream, indices, locations, *gates = ctx.saved_tensors
        R, M = ctx.shape
        grad_out = grad_out.contiguous()
        gstream = ops.dispatch_zfp(grad_out, list(indices), list(locations), list(gates), ctx.experts, ctx.capacity)
        grad_y = ops.zfp_decompress(gstream, M, R, 2)
        if FUSE_ZFP:
            # the gate gradients straight from the stream of the tensor fast_decode consumed
            gg = ops.bwd_gate_zfp(stream, grad_out, list(indices), list(locations), ctx.experts, ctx.capacity)
        else:
            seen = ops.zfp_decompress(stream, M, R, 2)
            gg = ops.bwd_gate(grad_out, seen, list(indices), list(locations), ctx.capacity)
        return (grad_y, None, None, None, None, None, *[gg[j].to(g.dtype) for j, g in enumerate(gates)])


FUSE_ZFP = True


def fused_zfp_eligible(x, compress_name, degree, is_postscore, experts, capacity):
    # the conditions under which ZfpCompressor.compress accepts the [E, C, M] buffer (zfpc.cpp:24-31)
    return (FUSE_ZFP and compress_name == 'zfp' and is_postscore and x.is_cuda and
            x.dtype == torch.float32 and x.shape[-1] % 4 == 0 and experts % 4 == 0 and capacity % 4 == 0 and
            capacity > 0)


def fused_zfp_forward(x, crit, expert_fn, degree=1):
    """encode -> [codec, comm, codec] -> experts -> [codec, comm, codec] -> decode for the
    zfp compressor.  crit = (experts, indices_s, locations_s, gates_s, capacity)."""
    experts, indices_s, locations_s, gates_s, capacity = crit
    indices = torch.stack([t.reshape(-1) for t in indices_s]).to(torch.int32).contiguous()     # [k, T]
    locations = torch.stack([t.reshape(-1) for t in locations_s]).to(torch.int32).contiguous()
    y = _EncodeZfp.apply(x.contiguous(), indices, locations, experts, capacity)
    y = _experts_in_chunks(expert_fn, y.view(experts, capacity, x.shape[-1]), degree)
    y = y.reshape(experts * capacity, -1).to(x.dtype)
    gates = [g.float() for g in gates_s]
    return _DecodeZfp.apply(y, indices, locations, experts, capacity, x.shape[0], *gates)


def zfp_experts_decode(y, expert_fn, degree, indices, locations, gates, samples):
    """The part of fused_zfp_forward after the encode: experts on the [E, C, M] buffer, then
    compress + decompress + decode in one pass."""
    experts, capacity, M = y.shape
    y = _experts_in_chunks(expert_fn, y, degree)
    y = y.reshape(experts * capacity, -1).to(torch.float32)
    return _DecodeZfp.apply(y, indices, locations, experts, capacity, samples, *[g.float() for g in gates])


def fused_int8_eligible(x, compress_name, degree, is_postscore):
    vec = 4 if x.dtype == torch.float32 else 8
    return (FUSE_INT8 and compress_name == 'int8' and is_postscore and x.is_cuda and
            x.dtype in (torch.float32, torch.bfloat16, torch.float16) and x.shape[-1] % vec == 0)


def fused_int8_forward(x, crit, expert_fn, degree=1, codes_fn=None):
    """encode -> [codec, comm, codec] -> experts -> [codec, comm, codec] -> decode for the
    int8 compressor.  crit = (experts, indices_s, locations_s, gates_s, capacity).  codes_fn
    (inference only): the experts as a function of the codes, see ffn_from_codes_fn."""
    experts, indices_s, locations_s, gates_s, capacity = crit
    indices = torch.stack([t.reshape(-1) for t in indices_s]).to(torch.int32).contiguous()     # [k, T]
    locations = torch.stack([t.reshape(-1) for t in locations_s]).to(torch.int32).contiguous()
    if codes_fn is not None and not torch.is_grad_enabled():
        x = x.contiguous()
        M = x.shape[-1]
        codes, bias, scale = ops.dispatch_int8(x, list(indices), list(locations), None, experts, capacity)
        y = codes_fn(codes.view(experts, capacity, M), bias.view(experts, capacity, 1), scale.view(experts, capacity, 1))
        codes, bias, scale = ops.int8_compress(y.reshape(experts * capacity, -1).to(x.dtype).contiguous())
        return ops.combine_int8(codes, bias, scale, list(indices), list(locations), [g.float() for g in gates_s],
                                x.shape[0], capacity)
    y = _EncodeInt8.apply(x.contiguous(), indices, locations, experts, capacity)
    y = _experts_in_chunks(expert_fn, y.view(experts, capacity, x.shape[-1]), degree)
    y = y.reshape(experts * capacity, -1).to(x.dtype)
    gates = [g.float() for g in gates_s]
    return _DecodeInt8.apply(y, indices, locations, experts, capacity, x.shape[0], *gates)

