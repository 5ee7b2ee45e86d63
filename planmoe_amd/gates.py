"""Gates: the linear top-k gate (gates/top.py) and the cosine gate (gates/cosine_top.py)."""
import math

import torch

from . import ops


_SPLIT = 16          # token chunks of the weight gradient
_bmm_fp32_out = None  # whether torch.bmm can return fp32 for 16-bit inputs (probed on first use)


def weight_grad(g, x):
    """g^T @ x for g [T, E], x [T, M] (both in x's dtype): the gate weight's gradient.

    The product is a sum over tokens with a tiny output, which the library's GEMM heuristics
    serve badly (one pass over x at a quarter of the memory rate); split over _SPLIT token
    chunks as a batched GEMM plus a sum it runs at the rate x can be read (measured on
    16384 x 4096 x 8 bf16: 62 -> 29 us; 32768 x 2048 x 64: 111 -> 28 us).  The partial
    products are kept in fp32 where the library allows, so the result is rounded once."""
    global _bmm_fp32_out
    T = x.shape[0]
    main = (T // _SPLIT) * _SPLIT
    if main < 16 * _SPLIT:
        return g.t() @ x
    gs = g[:main].reshape(_SPLIT, main // _SPLIT, -1).transpose(1, 2)
    xs = x[:main].reshape(_SPLIT, main // _SPLIT, -1)
    parts = None
    if x.dtype != torch.float32 and _bmm_fp32_out is not False:
        try:
            parts = torch.bmm(gs, xs, out_dtype=torch.float32)
            _bmm_fp32_out = True
        except (TypeError, RuntimeError, NotImplementedError):
            _bmm_fp32_out = False
    if parts is None:
        parts = torch.bmm(gs, xs)
    out = parts.sum(0, dtype=torch.float32)
    if main < T:
        out = out + (g[main:].t() @ x[main:]).float()
    return out.to(x.dtype)


class _GateLogits(torch.autograd.Function):
    """logits = x @ w^T through the MFMA kernel; the two backward products are plain
    library GEMMs."""

    @staticmethod
    def forward(ctx, x, w, out_dtype):
        ctx.save_for_backward(x, w)
        return ops.gate_logits(x, w, out_dtype)

    @staticmethod
    def backward(ctx, grad):
        x, w = ctx.saved_tensors
        g = grad.to(x.dtype)
        return g @ w, weight_grad(g, x), None


class _GateLogitsSplit(torch.autograd.Function):
    """fp32 logits of 16-bit activations against an fp32 gate weight (the reference's fp32_gate
    case when the gate is kept in fp32, top.py:21-26) without reading x as fp32: the weight is
    split into two 16-bit parts, w = hi + lo up to 2^-17 of its magnitude, both go through the MFMA
    kernel as 2 E rows, and the two halves of the result are added.  Rounding the weight to one
    16-bit value instead would move logits by about 1e-3 and tokens near a tie to another expert."""

    @staticmethod
    def forward(ctx, x, w32):
        hi = w32.to(x.dtype)
        # fp16: the low part would sit among the subnormals; scaled by a power of two it does not
        up = 1024.0 if x.dtype == torch.float16 else 1.0
        lo = ((w32 - hi.float()) * up).to(x.dtype)
        E = w32.shape[0]
        if 2 * E <= 128:
            both = ops.gate_logits(x, torch.cat([hi, lo]).contiguous(), torch.float32)
            logits = both[:, :E] + both[:, E:] * (1.0 / up)
        else:
            logits = (ops.gate_logits(x, hi.contiguous(), torch.float32) +
                      ops.gate_logits(x, lo.contiguous(), torch.float32) * (1.0 / up))
        ctx.save_for_backward(x, hi)
        return logits

    @staticmethod
    def backward(ctx, grad):
        x, hi = ctx.saved_tensors
        g = grad.to(x.dtype)
        return g @ hi, weight_grad(g, x).float()


class LinearTopKGate(torch.nn.Module):
    # gates/top.py:6-26
    def __init__(self, model_dim, num_global_experts, k=1, fp32_gate=False, **options):
        super().__init__()
        try:
            self.wg = torch.nn.Linear(model_dim, num_global_experts, bias=False,
                                      dtype=torch.float32 if fp32_gate else None)
        except Exception:
            self.wg = torch.nn.Linear(model_dim, num_global_experts, bias=False)
        self.top_k = min(num_global_experts, int(k))
        self.fp32_gate = fp32_gate
        for opt in options:
            if opt not in ('capacity_factor', 'gate_noise'):
                raise Exception('Unrecognized argument provided to Gating module: %s' % opt)

    def forward(self, x):
        """Logits [T, E], fp32 when fp32_gate (top.py:21-26).

        The reference up-casts x and the weight to fp32 and runs an fp32 GEMM; here x is read
        once in its own dtype by the MFMA kernel, which accumulates in fp32.  A weight kept in
        fp32 next to 16-bit activations enters as two 16-bit parts (_GateLogitsSplit)."""
        w = self.wg.weight
        if self.fp32_gate and w.dtype == torch.float32 and x.dtype in (torch.bfloat16, torch.float16):
            return _GateLogitsSplit.apply(x.contiguous(), w)
        if x.dtype != w.dtype:
            w = w.to(x.dtype)
        return _GateLogits.apply(x.contiguous(), w.contiguous(),
                                 torch.float32 if self.fp32_gate else x.dtype)



class CosineTopKGate(torch.nn.Module):
    # gates/cosine_top.py:7-33
    def __init__(self, model_dim, num_global_experts, k=1, fp32_gate=False, proj_dim=256, init_t=0.5, **options):
        super().__init__()
        self.top_k = min(num_global_experts, int(k))
        self.fp32_gate = fp32_gate
        self.temperature = torch.nn.Parameter(torch.log(torch.full([1], 1.0 / init_t)), requires_grad=True)
        self.cosine_projector = torch.nn.Linear(model_dim, proj_dim)
        self.sim_matrix = torch.nn.Parameter(torch.randn(size=(proj_dim, num_global_experts)), requires_grad=True)
        torch.nn.init.normal_(self.sim_matrix, 0, 0.01)
        for opt in options:
            if opt not in ('capacity_factor', 'gate_noise'):
                raise Exception('Unrecognized argument provided to Gating module: %s' % opt)

    def forward(self, x):
        """Cosine similarity of the projected tokens with one vector per expert, scaled by a
        learnt temperature capped at 1 / 0.01.  The similarity product has the shape of the
        gate-logits GEMM ([T, proj_dim] x [E, proj_dim]^T) and runs through the same kernel."""
        w, b, sim = self.cosine_projector.weight, self.cosine_projector.bias, self.sim_matrix
        if self.fp32_gate:
            x, w, b, sim = x.float(), w.float(), b.float(), sim.float()
        elif x.dtype != w.dtype:
            w, b, sim = w.to(x.dtype), b.to(x.dtype), sim.to(x.dtype)
        proj = torch.nn.functional.normalize(torch.nn.functional.linear(x, w, b), dim=1)
        experts = torch.nn.functional.normalize(sim, dim=0).t()
        logits = _GateLogits.apply(proj.contiguous(), experts.contiguous(), proj.dtype)
        logit_scale = torch.clamp(self.temperature, max=math.log(1. / 0.01)).exp()
        return logits * logit_scale.to(logits.dtype)


Gate = LinearTopKGate
GATES = {'top': LinearTopKGate, 'cosine_top': CosineTopKGate}
