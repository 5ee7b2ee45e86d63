"""Tensor-level wrappers of the libplanmoe_hip C ABI.

torch is used for what it is good at here -- device memory and the current HIP stream; all
arithmetic happens in the HIP kernels.  Every function enqueues on
``torch.cuda.current_stream()`` of the tensors' device and returns without synchronising.
"""
import ctypes

import torch

from . import _lib
from ._lib import PlanMoEError, check, lib

F32, BF16, F16 = 0, 1, 2
_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


def _dt(t, who):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise PlanMoEError("%s: unsupported dtype %s (float32, bfloat16 or float16)" % (who, t.dtype))


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _need_gpu(t, who):
    if not t.is_cuda:
        raise PlanMoEError("%s: tensors must live on the GPU (this build has no CPU path)" % who)


def _contig(t, who):
    if not t.is_contiguous():
        raise PlanMoEError("%s: tensor must be contiguous" % who)
    return t


def _ws(nbytes, device):
    return torch.empty((max(int(nbytes), 16),), dtype=torch.uint8, device=device)


def planes(tensors, dtype):
    """Pack a list of k 1-D tensors as k planes of one buffer.

    Returns (base tensor, plane stride in elements).  When the tensors already are equally
    spaced views of one allocation (as route_topk returns them) no copy is made."""
    k = len(tensors)
    n = tensors[0].numel()
    ok = all(t.dtype == dtype and t.dim() == 1 and t.numel() == n and t.is_contiguous() for t in tensors)
    if ok:
        if k == 1:
            return tensors[0], max(n, 1)
        es = tensors[0].element_size()
        d = tensors[1].data_ptr() - tensors[0].data_ptr()
        if d >= n * es and d % es == 0 and all(
                tensors[j].data_ptr() - tensors[0].data_ptr() == j * d for j in range(k)) and \
                tensors[0].untyped_storage().data_ptr() == tensors[-1].untyped_storage().data_ptr():
            return tensors[0], d // es
    stacked = torch.stack([t.reshape(-1).to(dtype) for t in tensors]).contiguous()
    return stacked, max(n, 1)


# ------------------------------------------------------------------------------ routing
def capacity(samples, experts, top_k, capacity_factor=1.0, alignment=1):
    out = ctypes.c_int(0)
    check(lib.planmoe_capacity(samples, experts, top_k, float(capacity_factor), int(alignment),
                               ctypes.byref(out)))
    return out.value


def cumsum_sub_one(mask):
    """int32 [T, E] -> int32 [T, E]: cumsum over dim 0, minus one."""
    _need_gpu(mask, "cumsum_sub_one")
    x = mask.to(torch.int32).contiguous()
    T, E = x.shape
    out = torch.empty_like(x)
    nbytes = lib.planmoe_cumsum_workspace_bytes(T, E)
    ws = _ws(nbytes, x.device)
    check(lib.planmoe_cumsum_sub_one(_ptr(x), _ptr(out), T, E, _ptr(ws), ws.numel(), _stream(x)))
    return out


def route_topk(inp, top_k, is_logits=False, logit_bias=None, normalize_gate=True,
               want_scores=False, want_l_aux=True, want_counts=False):
    """Top-k routing of scores (or logits) [T, E].

    Returns dict(indices [k,T] int32, locations [k,T] int32, gates [k,T] inp.dtype,
    scores [T,E] | None, l_aux 0-dim fp32 | None, counts [k,E] int32 | None)."""
    _need_gpu(inp, "route_topk")
    inp = _contig(inp, "route_topk")
    if inp.dim() != 2:
        raise PlanMoEError("route_topk: scores must be [samples, experts]")
    T, E = inp.shape
    k = min(int(top_k), E)
    dev = inp.device
    idx = torch.empty((k, T), dtype=torch.int32, device=dev)
    loc = torch.empty((k, T), dtype=torch.int32, device=dev)
    gates = torch.empty((k, T), dtype=inp.dtype, device=dev)
    scores = torch.empty_like(inp) if want_scores else None
    l_aux = torch.zeros((), dtype=torch.float32, device=dev) if want_l_aux else None
    counts = torch.empty((k, E), dtype=torch.int32, device=dev) if want_counts else None
    bias = None
    if logit_bias is not None:
        bias = logit_bias.to(device=dev, dtype=torch.float32).contiguous()
    ws = _ws(lib.planmoe_route_workspace_bytes(T, E, k), dev)
    check(lib.planmoe_route_topk(_ptr(inp), _dt(inp, "route_topk"), int(bool(is_logits)), _ptr(bias),
                                 T, E, k, int(bool(normalize_gate)), _ptr(idx), _ptr(loc), _ptr(gates),
                                 max(T, 1), _ptr(scores), _ptr(l_aux), _ptr(counts), _ptr(ws),
                                 ws.numel(), _stream(inp)))
    return dict(indices=idx, locations=loc, gates=gates, scores=scores, l_aux=l_aux, counts=counts)


def route_locations(indices, experts, order=None, want_counts=False):
    """Slot locations for existing routing decisions: indices int32 [k, T]; order int32 [T] =
    token served p-th (batch-prioritised routing), None = token order.
    Returns (locations [k, T] int32, counts [k, E] int32 | None)."""
    _need_gpu(indices, "route_locations")
    if indices.dtype != torch.int32 or indices.dim() != 2:
        raise PlanMoEError("route_locations: indices must be int32 [top_k, samples]")
    indices = _contig(indices, "route_locations")
    k, T = indices.shape
    dev = indices.device
    if order is not None:
        if order.numel() != T:
            raise PlanMoEError("route_locations: order must hold one entry per token")
        order = order.to(device=dev, dtype=torch.int32).contiguous()
    loc = torch.empty((k, T), dtype=torch.int32, device=dev)
    counts = torch.empty((k, int(experts)), dtype=torch.int32, device=dev) if want_counts else None
    ws = _ws(lib.planmoe_route_workspace_bytes(T, int(experts), k), dev)
    check(lib.planmoe_route_locations(_ptr(indices), max(T, 1), T, int(experts), k, _ptr(order), _ptr(loc),
                                      _ptr(counts), _ptr(ws), ws.numel(), _stream(indices)))
    return loc, counts


def route_bwd(scores, indices, grad_gates, normalize_gate=True, grad_l_aux=None, counts=None,
              through_softmax=False):
    """Gradient of route_topk's gates (and l_aux) with respect to the scores [T, E] (or the
    logits when through_softmax).  indices int32 [k, T], grad_gates [k, T] in scores.dtype."""
    _need_gpu(scores, "route_bwd")
    scores = _contig(scores, "route_bwd")
    T, E = scores.shape
    k = indices.shape[0]
    indices = _contig(indices, "route_bwd")
    gg = grad_gates.to(scores.dtype).contiguous()
    out = torch.empty_like(scores)
    dl = None if grad_l_aux is None else grad_l_aux.to(torch.float32).reshape(1).contiguous()
    c0 = None if counts is None else counts[0].contiguous()
    check(lib.planmoe_route_bwd(_ptr(scores), _dt(scores, "route_bwd"), _ptr(indices), _ptr(gg), max(T, 1), T, E, k,
                                int(bool(normalize_gate)), _ptr(dl), _ptr(c0), int(bool(through_softmax)),
                                _ptr(out), _stream(scores)))
    return out


def gate_logits(x, wg, out_dtype=None):
    """logits[T, E] = x[T, M] @ wg[E, M]^T with fp32 accumulation."""
    _need_gpu(x, "gate_logits")
    x = _contig(x, "gate_logits")
    wg = _contig(wg, "gate_logits")
    if x.dtype != wg.dtype:
        raise PlanMoEError("gate_logits: x and wg must share a dtype")
    out_dtype = out_dtype or x.dtype
    T, M = x.shape
    E = wg.shape[0]
    out = torch.empty((T, E), dtype=out_dtype, device=x.device)
    check(lib.planmoe_gate_logits(_ptr(x), _ptr(wg), _dt(x, "gate_logits"), _ptr(out), _DT[out_dtype],
                                  T, M, E, _stream(x)))
    return out


def gate_dx_accumulate(dx, grad_logits, wg):
    """dx[T, M] += grad_logits[T, E] @ wg[E, M] in place (up to 8 experts): the gate's share of x.grad."""
    _need_gpu(dx, "gate_dx_accumulate")
    dx = _contig(dx, "gate_dx_accumulate")
    wg = _contig(wg, "gate_dx_accumulate")
    if dx.dtype != wg.dtype:
        raise PlanMoEError("gate_dx_accumulate: dx and wg must share a dtype")
    g = grad_logits.to(torch.float32).contiguous()
    T, M = dx.shape
    E = wg.shape[0]
    if tuple(g.shape) != (T, E) or wg.shape[1] != M:
        raise PlanMoEError("gate_dx_accumulate: shapes do not fit")
    check(lib.planmoe_gate_dx_accumulate(_ptr(dx), _dt(dx, "gate_dx_accumulate"), _ptr(g), _ptr(wg), T, M, E,
                                         _stream(dx)))
    return dx


# ------------------------------------------------------------------------------ dispatch / combine
def _plane_args(indices, locations, gates, who):
    idx, s1 = planes(indices, torch.int32)
    loc, s2 = planes(locations, torch.int32)
    if s1 != s2:
        loc = torch.stack(list(locations)).contiguous()
        idx = torch.stack(list(indices)).contiguous()
        s1 = s2 = max(indices[0].numel(), 1)
    g = None
    if gates is not None:
        g, s3 = planes(gates, torch.float32)
        if s3 != s1:
            # bring all three to one stride
            idx = torch.stack(list(indices)).contiguous()
            loc = torch.stack(list(locations)).contiguous()
            g = torch.stack([t.to(torch.float32) for t in gates]).contiguous()
            s1 = max(indices[0].numel(), 1)
    return idx, loc, g, s1


def dispatch_fwd(x, indices, locations, gates, experts, capacity_):
    """[T, M] -> [experts*capacity, M]; gates=None is the all-ones helper."""
    _need_gpu(x, "dispatch_fwd")
    x = _contig(x, "dispatch_fwd")
    T, M = x.shape
    idx, loc, g, stride = _plane_args(indices, locations, gates, "dispatch_fwd")
    out = torch.empty((experts * capacity_, M), dtype=x.dtype, device=x.device)
    ws = _ws(lib.planmoe_dispatch_workspace_bytes(experts, capacity_), x.device)
    check(lib.planmoe_dispatch_fwd(_ptr(x), _dt(x, "dispatch_fwd"), _ptr(g), _ptr(idx), _ptr(loc),
                                   stride, len(indices), T, M, experts, capacity_, _ptr(out),
                                   _ptr(ws), ws.numel(), _stream(x)))
    return out


def combine_fwd(dispatched, indices, locations, gates, samples, capacity_):
    """[experts*capacity, M] -> [T, M]."""
    _need_gpu(dispatched, "combine_fwd")
    d = _contig(dispatched, "combine_fwd")
    M = d.shape[-1]
    idx, loc, g, stride = _plane_args(indices, locations, gates, "combine_fwd")
    out = torch.empty((samples, M), dtype=d.dtype, device=d.device)
    check(lib.planmoe_combine_fwd(_ptr(d), _dt(d, "combine_fwd"), _ptr(g), _ptr(idx), _ptr(loc), stride,
                                  len(indices), samples, M, capacity_, _ptr(out), _stream(d)))
    return out


def bwd_gate(x, dispatched, indices, locations, capacity_):
    """grad_gates[k, T] (fp32) = <dispatched[slot], x[t]>."""
    _need_gpu(x, "bwd_gate")
    x = _contig(x, "bwd_gate")
    d = _contig(dispatched, "bwd_gate")
    if x.dtype != d.dtype:
        raise PlanMoEError("bwd_gate: x and dispatched must share a dtype")
    T, M = x.shape
    idx, loc, _, stride = _plane_args(indices, locations, None, "bwd_gate")
    k = len(indices)
    out = torch.empty((k, stride), dtype=torch.float32, device=x.device)
    check(lib.planmoe_bwd_gate(_ptr(x), _ptr(d), _dt(x, "bwd_gate"), _ptr(idx), _ptr(loc), stride, k, T,
                               M, capacity_, _ptr(out), _stream(x)))
    return out[:, :T]


# ------------------------------------------------------------------------------ "int8" codec
def int8_compress(x, codes_out=None):
    """x [..., M] -> codes uint8 [..., M], bias [..., 1], scale [..., 1] (x's dtype).
    codes_out: optional contiguous uint8 storage of x.numel() bytes to write the codes into."""
    _need_gpu(x, "int8_compress")
    x = _contig(x, "int8_compress")
    M = x.shape[-1]
    rows = x.numel() // M if M else 0
    if codes_out is None:
        codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    else:
        codes = codes_out.view(torch.uint8).reshape(-1)[:x.numel()].view(x.shape)
    bias = torch.empty(x.shape[:-1] + (1,), dtype=x.dtype, device=x.device)
    scale = torch.empty_like(bias)
    check(lib.planmoe_int8_compress(_ptr(x), _dt(x, "int8_compress"), rows, M, _ptr(codes), _ptr(bias),
                                    _ptr(scale), _stream(x)))
    return codes, bias, scale


def int8_decompress(codes, bias, scale):
    _need_gpu(codes, "int8_decompress")
    codes = _contig(codes, "int8_decompress")
    M = codes.shape[-1]
    rows = codes.numel() // M if M else 0
    out = torch.empty(codes.shape, dtype=bias.dtype, device=codes.device)
    check(lib.planmoe_int8_decompress(_ptr(codes), _ptr(bias.contiguous()), _ptr(scale.contiguous()),
                                      _dt(bias, "int8_decompress"), rows, M, _ptr(out), _stream(codes)))
    return out


def combine_int8(codes, bias, scale, indices, locations, gates, samples, capacity_):
    """The int8 decompressor followed by fast_decode, in one pass: codes [experts*capacity, M]
    uint8 with their bias / scale -> [T, M] in bias.dtype."""
    _need_gpu(codes, "combine_int8")
    codes = _contig(codes, "combine_int8")
    M = codes.shape[-1]
    idx, loc, g, stride = _plane_args(indices, locations, gates, "combine_int8")
    out = torch.empty((samples, M), dtype=bias.dtype, device=codes.device)
    check(lib.planmoe_combine_int8(_ptr(codes), _ptr(bias.contiguous()), _ptr(scale.contiguous()),
                                   _dt(bias, "combine_int8"), _ptr(g), _ptr(idx), _ptr(loc), stride,
                                   len(indices), samples, M, capacity_, _ptr(out), _stream(codes)))
    return out


def dispatch_int8(x, indices, locations, gates, experts, capacity_):
    """fast_encode followed by the int8 compressor, in one pass.
    Returns codes [experts*capacity, M] uint8, bias, scale [experts*capacity, 1]."""
    _need_gpu(x, "dispatch_int8")
    x = _contig(x, "dispatch_int8")
    T, M = x.shape
    idx, loc, g, stride = _plane_args(indices, locations, gates, "dispatch_int8")
    R = experts * capacity_
    codes = torch.empty((R, M), dtype=torch.uint8, device=x.device)
    bias = torch.empty((R, 1), dtype=x.dtype, device=x.device)
    scale = torch.empty_like(bias)
    ws = _ws(lib.planmoe_dispatch_workspace_bytes(experts, capacity_), x.device)
    check(lib.planmoe_dispatch_int8(_ptr(x), _dt(x, "dispatch_int8"), _ptr(g), _ptr(idx), _ptr(loc),
                                    stride, len(indices), T, M, experts, capacity_, _ptr(codes),
                                    _ptr(bias), _ptr(scale), _ptr(ws), ws.numel(), _stream(x)))
    return codes, bias, scale


def combine_bwd_int8(grad_out, expert_out, indices, locations, gates, experts, capacity_):
    """GatingDecoder.backward + int8 compress of the gradient buffer in one pass.
    expert_out: the [E*C, M] tensor fast_decode consumed, or the (codes, bias, scale) triple it was
    decompressed from (same results, and the decompressed copy need not exist).
    Returns codes [E*C, M] uint8, bias, scale [E*C, 1], grad_gates [k, T] fp32."""
    _need_gpu(grad_out, "combine_bwd_int8")
    g_out = _contig(grad_out, "combine_bwd_int8")
    if isinstance(expert_out, (tuple, list)):
        e_codes, e_bias, e_scale = (_contig(t, "combine_bwd_int8") for t in expert_out)
        if e_bias.dtype != g_out.dtype or e_scale.dtype != g_out.dtype or e_codes.dtype != torch.uint8:
            raise PlanMoEError("combine_bwd_int8: coded expert output must be uint8 codes with bias / scale in grad_out's dtype")
        T, M = g_out.shape
        idx, loc, g, stride = _plane_args(indices, locations, gates, "combine_bwd_int8")
        k = len(indices)
        R = experts * capacity_
        codes = torch.empty((R, M), dtype=torch.uint8, device=g_out.device)
        bias = torch.empty((R, 1), dtype=g_out.dtype, device=g_out.device)
        scale = torch.empty_like(bias)
        gg = torch.empty((k, stride), dtype=torch.float32, device=g_out.device)
        ws = _ws(lib.planmoe_dispatch_workspace_bytes(experts, capacity_), g_out.device)
        check(lib.planmoe_combine_bwd_int8_coded(_ptr(g_out), _ptr(e_codes), _ptr(e_bias), _ptr(e_scale),
                                                 _dt(g_out, "combine_bwd_int8"), _ptr(g), _ptr(idx), _ptr(loc), stride,
                                                 k, T, M, experts, capacity_, _ptr(codes), _ptr(bias), _ptr(scale),
                                                 _ptr(gg), _ptr(ws), ws.numel(), _stream(g_out)))
        return codes, bias, scale, gg[:, :T]
    e_out = _contig(expert_out, "combine_bwd_int8")
    if g_out.dtype != e_out.dtype:
        raise PlanMoEError("combine_bwd_int8: grad_out and expert_out must share a dtype")
    T, M = g_out.shape
    idx, loc, g, stride = _plane_args(indices, locations, gates, "combine_bwd_int8")
    k = len(indices)
    R = experts * capacity_
    codes = torch.empty((R, M), dtype=torch.uint8, device=g_out.device)
    bias = torch.empty((R, 1), dtype=g_out.dtype, device=g_out.device)
    scale = torch.empty_like(bias)
    gg = torch.empty((k, stride), dtype=torch.float32, device=g_out.device)
    ws = _ws(lib.planmoe_dispatch_workspace_bytes(experts, capacity_), g_out.device)
    check(lib.planmoe_combine_bwd_int8(_ptr(g_out), _ptr(e_out), _dt(g_out, "combine_bwd_int8"), _ptr(g),
                                       _ptr(idx), _ptr(loc), stride, k, T, M, experts, capacity_, _ptr(codes),
                                       _ptr(bias), _ptr(scale), _ptr(gg), _ptr(ws), ws.numel(), _stream(g_out)))
    return codes, bias, scale, gg[:, :T]


# ------------------------------------------------------------------------------ fused forward chain
_forward_ws = {}


def _forward_workspace(T, E, k, device):
    """Workspace of the fused chain, grown on demand: one per device and stream (calls on one
    stream follow each other; calls on two streams must not share it)."""
    need = lib.planmoe_forward_workspace_bytes(T, E, k)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _forward_ws.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty((max(need, 1 << 20),), dtype=torch.uint8, device=device)
        # memory allocated during a graph capture belongs to the graph's private pool: such a
        # buffer serves this call only and is not kept for later eager calls
        if not torch.cuda.is_current_stream_capturing():
            _forward_ws[key] = ws
    return ws


def _forward_common(x, wg, top_k, fp32_gate, logit_bias, want_logits, want_scores, want_l_aux, want_counts):
    _need_gpu(x, "forward")
    x = _contig(x, "forward")
    wg = _contig(wg, "forward")
    if x.dtype != wg.dtype:
        raise PlanMoEError("forward: x and wg must share a dtype")
    T, M = x.shape
    E = wg.shape[0]
    k = min(int(top_k), E)
    dev = x.device
    sdt = torch.float32 if (fp32_gate or x.dtype == torch.float32) else x.dtype
    out = dict(
        indices=torch.empty((k, T), dtype=torch.int32, device=dev),
        locations=torch.empty((k, T), dtype=torch.int32, device=dev),
        gates=torch.empty((k, T), dtype=sdt, device=dev),
        logits=torch.empty((T, E), dtype=sdt, device=dev) if want_logits else None,
        scores=torch.empty((T, E), dtype=sdt, device=dev) if want_scores else None,
        l_aux=torch.zeros((), dtype=torch.float32, device=dev) if want_l_aux else None,
        counts=torch.empty((k, E), dtype=torch.int32, device=dev) if want_counts else None)
    bias = None
    if logit_bias is not None:
        bias = logit_bias.to(device=dev, dtype=torch.float32).contiguous()
    return x, wg, T, M, E, k, bias, out, _forward_workspace(T, E, k, dev)


def gate_route(x, wg, top_k, fp32_gate=True, logit_bias=None, normalize_gate=True, want_logits=False,
               want_scores=False, want_l_aux=True, want_counts=False):
    """Gate GEMM + softmax + top-k routing in two launches (experts <= 64)."""
    x, wg, T, M, E, k, bias, out, ws = _forward_common(x, wg, top_k, fp32_gate, logit_bias, want_logits,
                                                       want_scores, want_l_aux, want_counts)
    check(lib.planmoe_gate_route(_ptr(x), _ptr(wg), _dt(x, "gate_route"), int(bool(fp32_gate)), _ptr(bias),
                                 T, M, E, k, int(bool(normalize_gate)), _ptr(out["indices"]),
                                 _ptr(out["locations"]), _ptr(out["gates"]), max(T, 1), _ptr(out["logits"]),
                                 _ptr(out["scores"]), _ptr(out["l_aux"]), _ptr(out["counts"]), _ptr(ws),
                                 ws.numel(), _stream(x)))
    return out


def forward_int8(x, wg, top_k, capacity_, fp32_gate=True, logit_bias=None, normalize_gate=True,
                 want_logits=False, want_scores=False, want_l_aux=True, want_counts=False):
    """Gate GEMM + routing + dispatch + int8 compress in two launches.  Adds codes
    [E*capacity, M] uint8 and bias / scale [E*capacity, 1] to gate_route's outputs."""
    x, wg, T, M, E, k, bias, out, ws = _forward_common(x, wg, top_k, fp32_gate, logit_bias, want_logits,
                                                       want_scores, want_l_aux, want_counts)
    R = E * capacity_
    out["codes"] = torch.empty((R, M), dtype=torch.uint8, device=x.device)
    out["bias"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
    out["scale"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
    check(lib.planmoe_forward_int8(_ptr(x), _ptr(wg), _dt(x, "forward_int8"), int(bool(fp32_gate)), _ptr(bias),
                                   T, M, E, k, int(bool(normalize_gate)), capacity_, _ptr(out["indices"]),
                                   _ptr(out["locations"]), _ptr(out["gates"]), max(T, 1), _ptr(out["logits"]),
                                   _ptr(out["scores"]), _ptr(out["l_aux"]), _ptr(out["counts"]),
                                   _ptr(out["codes"]), _ptr(out["bias"]), _ptr(out["scale"]), _ptr(ws),
                                   ws.numel(), _stream(x)))
    return out


def forward_plain(x, wg, top_k, capacity_, fp32_gate=True, logit_bias=None, normalize_gate=True,
                  want_logits=False, want_scores=False, want_l_aux=True, want_counts=False):
    """Gate GEMM + routing + dispatch (no codec) in two launches: gate_route's outputs plus
    `dispatched` [E*capacity, M] in x's dtype, what fast_encode without gates makes of x (the second
    launch works out the slots itself, so the stand-alone routing's launch that finishes them and a
    pass over the routing planes are saved)."""
    x, wg, T, M, E, k, bias, out, ws = _forward_common(x, wg, top_k, fp32_gate, logit_bias, want_logits,
                                                       want_scores, want_l_aux, want_counts)
    out["dispatched"] = torch.empty((E * capacity_, M), dtype=x.dtype, device=x.device)
    check(lib.planmoe_forward_plain(_ptr(x), _ptr(wg), _dt(x, "forward_plain"), int(bool(fp32_gate)), _ptr(bias),
                                    T, M, E, k, int(bool(normalize_gate)), capacity_, _ptr(out["indices"]),
                                    _ptr(out["locations"]), _ptr(out["gates"]), max(T, 1), _ptr(out["logits"]),
                                    _ptr(out["scores"]), _ptr(out["l_aux"]), _ptr(out["counts"]),
                                    _ptr(out["dispatched"]), _ptr(ws), ws.numel(), _stream(x)))
    return out


_single_serves = {}


def forward_int8_single_serves(x, wg, top_k, fp32_gate=True):
    """The shapes planmoe_forward_int8_single takes: bf16 rows of 256 to 4096 values in steps of 256, up to
    16 experts, top_k <= 4, and so few tokens that all its work-groups are resident at once (64 per compute
    unit; 128 for rows of up to 1792 values).  The library is asked (planmoe_forward_int8_single_serves),
    once per shape and device."""
    if not (x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.shape[0] >= 1):
        return False
    key = (x.device.index, x.shape[0], x.shape[1], wg.shape[0], int(top_k), bool(fp32_gate))
    hit = _single_serves.get(key)
    if hit is None:
        with torch.cuda.device(x.device):
            hit = bool(lib.planmoe_forward_int8_single_serves(_dt(x, "forward_int8_single"), int(bool(fp32_gate)), x.shape[0],
                                                              x.shape[1], wg.shape[0], int(top_k)))
        if len(_single_serves) > 4096:
            _single_serves.clear()
        _single_serves[key] = hit
    return hit


def forward_int8_single(x, wg, top_k, capacity_, fp32_gate=True, logit_bias=None, normalize_gate=True,
                        want_logits=False, want_scores=False, want_l_aux=True, want_counts=False, spin_limit=0):
    """forward_int8 in one launch that reads x once (bf16 rows of 256 .. 4096 values in steps of 256, up to 16 experts,
    top_k <= 4, as many tokens as forward_int8_single_serves allows; anything else raises).  Adds `gave_up`, a device
    int32 that is 1 when a work-group ran out of `spin_limit` polls waiting for the others."""
    x, wg, T, M, E, k, bias, out, ws = _forward_common(x, wg, top_k, fp32_gate, logit_bias, want_logits,
                                                       want_scores, want_l_aux, want_counts)
    R = E * capacity_
    out["codes"] = torch.empty((R, M), dtype=torch.uint8, device=x.device)
    out["bias"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
    out["scale"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
    out["gave_up"] = torch.zeros((), dtype=torch.int32, device=x.device)
    check(lib.planmoe_forward_int8_single(_ptr(x), _ptr(wg), _dt(x, "forward_int8_single"), int(bool(fp32_gate)),
                                          _ptr(bias), T, M, E, k, int(bool(normalize_gate)), capacity_,
                                          _ptr(out["indices"]), _ptr(out["locations"]), _ptr(out["gates"]), max(T, 1),
                                          _ptr(out["logits"]), _ptr(out["scores"]), _ptr(out["l_aux"]),
                                          _ptr(out["counts"]), _ptr(out["codes"]), _ptr(out["bias"]),
                                          _ptr(out["scale"]), _ptr(ws), ws.numel(), int(spin_limit),
                                          _ptr(out["gave_up"]), _stream(x)))
    return out


class ForwardCeiling:
    """planmoe_forward_int8_single_ceiling with its buffers allocated once: the grid, loads, exchange
    and stores of the one-launch chain without its arithmetic (mode 0), without the wait at the
    exchange (mode 1), or with the two-half dealing (mode 2).  A measuring stick; the outputs mean
    nothing.  16384 x 4096 bf16, 8 experts, top-2."""

    def __init__(self, x, experts, top_k, capacity_):
        _need_gpu(x, "forward_ceiling")
        self.x = _contig(x, "forward_ceiling")
        T, M = x.shape
        dev = x.device
        self.shape = (T, M, int(experts), int(top_k), int(capacity_))
        R = experts * capacity_
        self.codes = torch.empty((R, M), dtype=torch.uint8, device=dev)
        self.bias = torch.empty((R,), dtype=torch.bfloat16, device=dev)
        self.scale = torch.empty((R,), dtype=torch.bfloat16, device=dev)
        self.planes = torch.empty((3 * top_k * T,), dtype=torch.int32, device=dev)
        self.gave_up = torch.zeros((), dtype=torch.int32, device=dev)
        self.ws = torch.empty((lib.planmoe_forward_workspace_bytes(T, experts, top_k),), dtype=torch.uint8, device=dev)

    def run(self, mode=0):
        T, M, E, k, C = self.shape
        check(lib.planmoe_forward_int8_single_ceiling(_ptr(self.x), T, M, E, k, C, _ptr(self.codes), _ptr(self.bias),
                                                      _ptr(self.scale), _ptr(self.planes), _ptr(self.ws), self.ws.numel(),
                                                      int(mode), 0, _ptr(self.gave_up), _stream(self.x)))


def forward_int8_static(x, wg, top_k, capacity_, out, fp32_gate=True, logit_bias=None, normalize_gate=True):
    """forward_int8 through the entry point that allocates nothing: the workspace is the library's
    built-in device buffer and every output is the caller's (`out`: the dict of tensors a
    forward_int8 call returned, or tensors of those shapes).  x, wg and logit_bias must be
    contiguous GPU tensors already (fp32 bias): nothing is copied or created here."""
    T, M = x.shape
    E = wg.shape[0]
    k = min(int(top_k), E)
    for t in (x, wg) + tuple(v for v in out.values() if v is not None):
        if not (t.is_cuda and t.is_contiguous()):
            raise PlanMoEError("forward_int8_static: contiguous GPU tensors only")
    check(lib.planmoe_forward_int8_static(_ptr(x), _ptr(wg), _dt(x, "forward_int8_static"), int(bool(fp32_gate)),
                                          _ptr(logit_bias), T, M, E, k, int(bool(normalize_gate)), capacity_,
                                          _ptr(out["indices"]), _ptr(out["locations"]), _ptr(out["gates"]),
                                          out["indices"].shape[1], _ptr(out.get("logits")), _ptr(out.get("scores")),
                                          _ptr(out.get("l_aux")), _ptr(out.get("counts")), _ptr(out["codes"]),
                                          _ptr(out["bias"]), _ptr(out["scale"]), _stream(x)))
    return out


class ForwardInt8Plan:
    """forward_int8 with every output and the workspace allocated once: `run()` is a single
    C-ABI call that enqueues the two launches (for serving loops that reuse their buffers)."""

    def __init__(self, x, wg, top_k, capacity_, fp32_gate=True, logit_bias=None, normalize_gate=True,
                 want_l_aux=True, want_counts=False, single=False):
        x, wg, T, M, E, k, bias, out, _ = _forward_common(x, wg, top_k, fp32_gate, logit_bias, False,
                                                          False, want_l_aux, want_counts)
        # a workspace of the plan's own: redispatch() reads the routing state run() left in it, which
        # another forward call on the same stream would overwrite in a shared one
        ws = torch.empty((max(lib.planmoe_forward_workspace_bytes(T, E, k), 256),), dtype=torch.uint8, device=x.device)
        R = E * capacity_
        out["codes"] = torch.empty((R, M), dtype=torch.uint8, device=x.device)
        out["bias"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
        out["scale"] = torch.empty((R, 1), dtype=x.dtype, device=x.device)
        self.out, self.x, self.wg, self._bias, self._ws = out, x, wg, bias, ws
        self._args = [_ptr(x), _ptr(wg), _dt(x, "forward_int8"), int(bool(fp32_gate)), _ptr(bias), T, M, E, k,
                      int(bool(normalize_gate)), capacity_, _ptr(out["indices"]), _ptr(out["locations"]),
                      _ptr(out["gates"]), max(T, 1), None, None, _ptr(out["l_aux"]), _ptr(out["counts"]),
                      _ptr(out["codes"]), _ptr(out["bias"]), _ptr(out["scale"]), _ptr(ws), ws.numel()]
        # single: the one-launch kernel that reads x once (planmoe_forward_int8_single; shapes it does
        # not serve raise at run()); gave_up is its device flag
        self.single = bool(single)
        self.gave_up = torch.zeros((), dtype=torch.int32, device=x.device)

    def run(self):
        if self.single:
            check(lib.planmoe_forward_int8_single(*self._args, 0, _ptr(self.gave_up), _stream(self.x)))
        else:
            check(lib.planmoe_forward_int8(*self._args, _stream(self.x)))
        return self.out

    def redispatch(self):
        """Only the last launch again (dispatch + int8 from the routing state of the last run)."""
        a = self._args
        check(lib.planmoe_forward_int8_redispatch(a[0], a[2], a[5], a[6], a[7], a[8], a[10], a[11], a[12], a[14],
                                                  a[19], a[20], a[21], a[22], a[23], _stream(self.x)))
        return self.out


# ------------------------------------------------------------------------------ expert FFN on codes
def ffn_weight_colsum(weight_k_major):
    """fp32 [E, H]: the sums over model_dim of the k-major first-GEMM weight (what the affine kernel's
    bias term multiplies); compute once per weight."""
    return weight_k_major.float().sum(-1).contiguous()


def ffn_fc1_int8(codes, bias, scale, weight_k_major, fc_bias=None, out=None):
    """First GEMM of the expert FFN straight from int8 codes: codes uint8 [E, C, M], bias / scale
    bf16 [E, C, 1] (what int8_compress returned), weight_k_major bf16 [E, H, M], fc_bias bf16
    [E, H] or None -> bf16 [E, C, H] = decompress(codes) @ weight_k_major^T (+ fc_bias)."""
    _need_gpu(codes, "ffn_fc1_int8")
    E, C, M = codes.shape
    H = weight_k_major.shape[1]
    if bias.dtype != torch.bfloat16 or weight_k_major.dtype != torch.bfloat16:
        raise PlanMoEError("ffn_fc1_int8: bf16 only")
    if tuple(weight_k_major.shape) != (E, H, M):
        raise PlanMoEError("ffn_fc1_int8: weight must be [experts, hidden, model_dim]")
    codes, weight_k_major = _contig(codes, "ffn_fc1_int8"), _contig(weight_k_major, "ffn_fc1_int8")
    bias, scale = _contig(bias, "ffn_fc1_int8"), _contig(scale, "ffn_fc1_int8")
    if fc_bias is not None:
        fc_bias = _contig(fc_bias.to(torch.bfloat16), "ffn_fc1_int8")
    if out is None:
        out = torch.empty((E, C, H), dtype=torch.bfloat16, device=codes.device)
    elif tuple(out.shape) != (E, C, H) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise PlanMoEError("ffn_fc1_int8: out must be a contiguous bf16 [experts, rows, hidden] tensor")
    check(lib.planmoe_ffn_fc1_int8(_ptr(codes), _ptr(bias), _ptr(scale), 1, _ptr(weight_k_major), _ptr(fc_bias),
                                   E, C, M, H, _ptr(out), _stream(codes)))
    return out


def ffn_fc1_int8_affine(codes, bias, scale, weight_k_major, weight_colsum=None, fc_bias=None, out=None):
    """ffn_fc1_int8 with the codes themselves on the matrix cores and scale / bias applied in the
    epilogue (planmoe_ffn_fc1_int8_affine): agrees with it to about an ulp of the bf16 result, and is
    the faster one.  weight_colsum = ffn_weight_colsum(weight_k_major) (computed here when None)."""
    _need_gpu(codes, "ffn_fc1_int8_affine")
    E, C, M = codes.shape
    H = weight_k_major.shape[1]
    if bias.dtype != torch.bfloat16 or weight_k_major.dtype != torch.bfloat16:
        raise PlanMoEError("ffn_fc1_int8_affine: bf16 only")
    if tuple(weight_k_major.shape) != (E, H, M):
        raise PlanMoEError("ffn_fc1_int8_affine: weight must be [experts, hidden, model_dim]")
    codes, weight_k_major = _contig(codes, "ffn_fc1_int8_affine"), _contig(weight_k_major, "ffn_fc1_int8_affine")
    bias, scale = _contig(bias, "ffn_fc1_int8_affine"), _contig(scale, "ffn_fc1_int8_affine")
    if weight_colsum is None:
        weight_colsum = ffn_weight_colsum(weight_k_major)
    if tuple(weight_colsum.shape) != (E, H) or weight_colsum.dtype != torch.float32 or not weight_colsum.is_contiguous():
        raise PlanMoEError("ffn_fc1_int8_affine: weight_colsum must be a contiguous fp32 [experts, hidden] tensor")
    if fc_bias is not None:
        fc_bias = _contig(fc_bias.to(torch.bfloat16), "ffn_fc1_int8_affine")
    if out is None:
        out = torch.empty((E, C, H), dtype=torch.bfloat16, device=codes.device)
    elif tuple(out.shape) != (E, C, H) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise PlanMoEError("ffn_fc1_int8_affine: out must be a contiguous bf16 [experts, rows, hidden] tensor")
    check(lib.planmoe_ffn_fc1_int8_affine(_ptr(codes), _ptr(bias), _ptr(scale), 1, _ptr(weight_k_major), _ptr(weight_colsum),
                                          _ptr(fc_bias), E, C, M, H, _ptr(out), _stream(codes)))
    return out


def transpose_bf16(x, pad_to=1):
    """[B, R, C] bf16 -> [B, C, R'] with R' = R rounded up to a multiple of pad_to (at least 8), the
    added columns zero (planmoe_transpose_bf16)."""
    _need_gpu(x, "transpose_bf16")
    x = _contig(x, "transpose_bf16")
    if x.dtype != torch.bfloat16 or x.dim() != 3:
        raise PlanMoEError("transpose_bf16: a bf16 [batches, rows, cols] tensor")
    B, R, C = x.shape
    if C % 8:
        raise PlanMoEError("transpose_bf16: cols must be a multiple of 8")
    step = max(8, int(pad_to))
    Ro = (R + step - 1) // step * step
    out = torch.empty((B, C, Ro), dtype=torch.bfloat16, device=x.device)
    check(lib.planmoe_transpose_bf16(_ptr(x), B, R, C, Ro, _ptr(out), _stream(x)))
    return out


def gemm_nt_bf16(a, b, bias=None, relu=False, out=None):
    """c[e] = act(bf16(bf16(a[e] @ b[e]^T) + bias[e])): a [B, m, k], b [B, n, k] (a [1, n, k] tensor is
    shared by all batches), bias [B, n] or None, all bf16 -> [B, m, n] bf16 (planmoe_gemm_nt_bf16)."""
    _need_gpu(a, "gemm_nt_bf16")
    a, b = _contig(a, "gemm_nt_bf16"), _contig(b, "gemm_nt_bf16")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or a.dim() != 3 or b.dim() != 3:
        raise PlanMoEError("gemm_nt_bf16: bf16 [batches, rows, k] operands")
    B, m, k = a.shape
    n = b.shape[1]
    if b.shape[2] != k or b.shape[0] not in (1, B):
        raise PlanMoEError("gemm_nt_bf16: operands disagree: a %s, b %s" % (tuple(a.shape), tuple(b.shape)))
    if k % 8 or n % 8:
        raise PlanMoEError("gemm_nt_bf16: k and n must be multiples of 8 (got k = %d, n = %d)" % (k, n))
    if bias is not None:
        bias = _contig(bias.to(torch.bfloat16), "gemm_nt_bf16")
        if tuple(bias.shape) != (B, n):
            raise PlanMoEError("gemm_nt_bf16: bias must be [batches, n]")
    if out is None:
        out = torch.empty((B, m, n), dtype=torch.bfloat16, device=a.device)
    elif tuple(out.shape) != (B, m, n) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise PlanMoEError("gemm_nt_bf16: out must be a contiguous bf16 [batches, m, n] tensor")
    check(lib.planmoe_gemm_nt_bf16(_ptr(a), _ptr(b), _ptr(bias), int(bool(relu)), B, m, n, k, k, k, n, m * k,
                                   n * k if b.shape[0] == B else 0, m * n, _ptr(out), _stream(a)))
    return out


def gemm_nn_bf16(a, b, bias=None, relu=False, out=None):
    """c[e] = act(bf16(bf16(a[e] @ b[e]) + bias[e])): a [B, m, k], b [B, k, n] (a weight as the experts store
    it), bias [B, n] or None, bf16 -> [B, m, n] bf16 (planmoe_gemm_nn_bf16; k a multiple of 64, n of 8)."""
    _need_gpu(a, "gemm_nn_bf16")
    a, b = _contig(a, "gemm_nn_bf16"), _contig(b, "gemm_nn_bf16")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or a.dim() != 3 or b.dim() != 3:
        raise PlanMoEError("gemm_nn_bf16: bf16 [batches, m, k] x [batches, k, n] operands")
    B, m, k = a.shape
    n = b.shape[2]
    if b.shape[0] != B or b.shape[1] != k:
        raise PlanMoEError("gemm_nn_bf16: operands disagree: a %s, b %s" % (tuple(a.shape), tuple(b.shape)))
    if k % 64 or n % 8:
        raise PlanMoEError("gemm_nn_bf16: k must be a multiple of 64, n of 8 (got k = %d, n = %d)" % (k, n))
    if bias is not None:
        bias = _contig(bias.to(torch.bfloat16), "gemm_nn_bf16")
        if tuple(bias.shape) != (B, n):
            raise PlanMoEError("gemm_nn_bf16: bias must be [batches, n]")
    if out is None:
        out = torch.empty((B, m, n), dtype=torch.bfloat16, device=a.device)
    elif tuple(out.shape) != (B, m, n) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise PlanMoEError("gemm_nn_bf16: out must be a contiguous bf16 [batches, m, n] tensor")
    check(lib.planmoe_gemm_nn_bf16(_ptr(a), _ptr(b), _ptr(bias), int(bool(relu)), B, m, n, k, k, n, n, m * k, k * n,
                                   m * n, _ptr(out), _stream(a)))
    return out


def gemm_tn_bf16(a, b, out=None):
    """c[e] = a[e]^T @ b[e]: a [B, k, m], b [B, k, n] bf16 -> [B, m, n] bf16 (planmoe_gemm_tn_bf16; k a
    multiple of 64, m and n multiples of 8)."""
    _need_gpu(a, "gemm_tn_bf16")
    a, b = _contig(a, "gemm_tn_bf16"), _contig(b, "gemm_tn_bf16")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16 or a.dim() != 3 or b.dim() != 3:
        raise PlanMoEError("gemm_tn_bf16: bf16 [batches, k, cols] operands")
    B, k, m = a.shape
    n = b.shape[2]
    if b.shape[0] != B or b.shape[1] != k:
        raise PlanMoEError("gemm_tn_bf16: operands disagree: a %s, b %s" % (tuple(a.shape), tuple(b.shape)))
    if k % 64 or m % 8 or n % 8:
        raise PlanMoEError("gemm_tn_bf16: k must be a multiple of 64, m and n of 8 (got k = %d, m = %d, n = %d)" % (k, m, n))
    if out is None:
        out = torch.empty((B, m, n), dtype=torch.bfloat16, device=a.device)
    elif tuple(out.shape) != (B, m, n) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise PlanMoEError("gemm_tn_bf16: out must be a contiguous bf16 [batches, m, n] tensor")
    check(lib.planmoe_gemm_tn_bf16(_ptr(a), _ptr(b), B, m, n, k, m, n, n, k * m, k * n, m * n, _ptr(out), _stream(a)))
    return out


# ------------------------------------------------------------------------------ zfp codec
def zfp_stream_bytes(dims, nx, ny, rate=8.0):
    return int(lib.planmoe_zfp_stream_bytes(dims, nx, ny, float(rate)))


def zfp_max_bytes(dims, nx, ny, rate=8.0):
    return int(lib.planmoe_zfp_max_bytes(dims, nx, ny, float(rate)))


def zfp_compress(field, nx, ny, dims=2, rate=8.0, out=None):
    """field: fp32 storage holding ny rows of nx values.  Returns a uint8 tensor of
    zfp_max_bytes (what the reference allocates) whose first zfp_stream_bytes are the stream."""
    _need_gpu(field, "zfp_compress")
    field = _contig(field, "zfp_compress")
    if out is None:
        # the kernel writes every byte of the stream; only the slack up to the maximum size
        # (what the reference's torch::zeros leaves as zeros) is cleared here
        out = torch.empty((zfp_max_bytes(dims, nx, ny, rate),), dtype=torch.uint8, device=field.device)
        out[zfp_stream_bytes(dims, nx, ny, rate):].zero_()
    check(lib.planmoe_zfp_compress(_ptr(field), dims, nx, ny, float(rate), _ptr(out), out.numel(),
                                   _stream(field)))
    return out


def zfp_decompress(stream, nx, ny, dims=2, rate=8.0):
    _need_gpu(stream, "zfp_decompress")
    out = torch.empty((ny, nx), dtype=torch.float32, device=stream.device)
    check(lib.planmoe_zfp_decompress(_ptr(stream), dims, nx, ny, float(rate), _ptr(out), _stream(stream)))
    return out


def dispatch_zfp(x, indices, locations, gates, experts, capacity_, rate=8.0, out=None):
    """fast_encode + zfp_compress (2-D, nx = M, ny = experts * capacity) in one pass: the stream of
    the dispatched buffer without the buffer.  x: fp32 [T, M].  Returns what zfp_compress returns."""
    _need_gpu(x, "dispatch_zfp")
    x = _contig(x, "dispatch_zfp")
    if x.dtype != torch.float32:
        raise PlanMoEError("dispatch_zfp: the codec reads its field as fp32; pass a float32 tensor")
    T, M = x.shape
    idx, loc, g, stride = _plane_args(indices, locations, gates, "dispatch_zfp")
    R = experts * capacity_
    if out is None:
        out = torch.empty((zfp_max_bytes(2, M, R, rate),), dtype=torch.uint8, device=x.device)
        out[zfp_stream_bytes(2, M, R, rate):].zero_()
    ws = _ws(lib.planmoe_dispatch_zfp_workspace_bytes(experts, capacity_), x.device)
    check(lib.planmoe_dispatch_zfp(_ptr(x), _ptr(g), _ptr(idx), _ptr(loc), stride, len(indices), T, M, experts,
                                   capacity_, float(rate), _ptr(out), out.numel(), _ptr(ws), ws.numel(), _stream(x)))
    return out


def combine_zfp(stream, indices, locations, gates, samples, experts, capacity_, model_dim, rate=8.0):
    """zfp_decompress (2-D, nx = model_dim, ny = experts * capacity) + fast_decode in one pass:
    [T, model_dim] fp32 straight from the stream."""
    _need_gpu(stream, "combine_zfp")
    stream = _contig(stream, "combine_zfp")
    idx, loc, g, stride = _plane_args(indices, locations, gates, "combine_zfp")
    out = torch.empty((samples, model_dim), dtype=torch.float32, device=stream.device)
    ws = _ws(lib.planmoe_combine_zfp_workspace_bytes(experts, capacity_), stream.device)
    check(lib.planmoe_combine_zfp(_ptr(stream), float(rate), _ptr(g), _ptr(idx), _ptr(loc), stride, len(indices),
                                  samples, model_dim, experts, capacity_, _ptr(out), _ptr(ws), ws.numel(),
                                  _stream(stream)))
    return out


def bwd_gate_zfp(stream, grad_out, indices, locations, experts, capacity_, rate=8.0):
    """grad_gates[k, T] (fp32) = <grad_out[t], decoded slot row> with the slot rows taken straight
    from the 2-D stream (nx = model_dim, ny = experts * capacity) of the tensor fast_decode consumed."""
    _need_gpu(stream, "bwd_gate_zfp")
    stream = _contig(stream, "bwd_gate_zfp")
    grad_out = _contig(grad_out, "bwd_gate_zfp")
    if grad_out.dtype != torch.float32:
        raise PlanMoEError("bwd_gate_zfp: grad_out must be float32 (the zfp codec reads its field as fp32)")
    T, M = grad_out.shape
    idx, loc, _, stride = _plane_args(indices, locations, None, "bwd_gate_zfp")
    k = len(indices)
    out = torch.empty((k, stride), dtype=torch.float32, device=grad_out.device)
    ws = _ws(lib.planmoe_combine_zfp_workspace_bytes(experts, capacity_), grad_out.device)
    check(lib.planmoe_bwd_gate_zfp(_ptr(stream), float(rate), _ptr(grad_out), _ptr(idx), _ptr(loc), stride, k, T, M,
                                   experts, capacity_, _ptr(out), _ptr(ws), ws.numel(), _stream(grad_out)))
    return out[:, :T]


# ------------------------------------------------------------------------------ GPULZ ("lz") codec
LZ_BLOCK_BYTES = 2048


def lz_compress(x, workspace=None):
    """x: any contiguous GPU tensor whose byte size is a multiple of 4 (the reference takes fp32).
    Returns the reference's four tensors (gpulz.cu:502-507): flag_offsets, data_offsets int32
    [blocks + 1], flags uint8 [blocks * 64], data uint8 [blocks * 2048]; the byte tensors are zero
    beyond flag_offsets[-1] / data_offsets[-1].  `workspace` (uint8, lz_workspace_bytes) is
    allocated when not given."""
    _need_gpu(x, "lz_compress")
    x = _contig(x, "lz_compress")
    nbytes = x.numel() * x.element_size()
    blocks = int(lib.planmoe_lz_blocks(nbytes))
    dev = x.device
    flag_offsets = torch.empty((blocks + 1,), dtype=torch.int32, device=dev)
    data_offsets = torch.empty((blocks + 1,), dtype=torch.int32, device=dev)
    flags = torch.empty((blocks * 64,), dtype=torch.uint8, device=dev)
    data = torch.empty((blocks * LZ_BLOCK_BYTES,), dtype=torch.uint8, device=dev)
    if workspace is None:
        workspace = _ws(lib.planmoe_lz_workspace_bytes(nbytes), dev)
    check(lib.planmoe_lz_compress(_ptr(x), nbytes, _ptr(flag_offsets), _ptr(data_offsets), _ptr(flags),
                                  _ptr(data), _ptr(workspace), workspace.numel(), _stream(x)))
    return flag_offsets, data_offsets, flags, data


def lz_decompress(out, flag_offsets, data_offsets, flags, data):
    """Decodes into `out` (the reference's lz_decompress writes its first argument, gpulz.cu:510-523)."""
    _need_gpu(out, "lz_decompress")
    if not out.is_contiguous():
        raise PlanMoEError("lz_decompress: out must be contiguous")
    nbytes = out.numel() * out.element_size()
    check(lib.planmoe_lz_decompress(_ptr(out), nbytes, _ptr(_contig(flag_offsets, "lz_decompress")),
                                    _ptr(_contig(data_offsets, "lz_decompress")),
                                    _ptr(_contig(flags, "lz_decompress")),
                                    _ptr(_contig(data, "lz_decompress")), _stream(out)))
    return out
