"""Linear top-k gate -- mirror of the reference's gates/top.py."""
import torch

from . import ops


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
        return g @ w, g.t() @ x, None


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
        once in its own dtype by the MFMA kernel, which accumulates in fp32.  An fp32 weight is
        rounded to x's dtype first when x is bf16/fp16 (exact if it holds such values)."""
        w = self.wg.weight
        if x.dtype != w.dtype:
            w = w.to(x.dtype)
        return _GateLogits.apply(x.contiguous(), w.contiguous(),
                                 torch.float32 if self.fp32_gate else x.dtype)


Gate = LinearTopKGate
