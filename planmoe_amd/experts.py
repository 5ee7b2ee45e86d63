"""Fused expert FFN -- mirror of the reference's experts/ffn.py (two batched GEMMs with bias and
activation between dispatch and combine).  On the GPU in bf16 both GEMMs, and the four of their
backward pass, are planmoe_gemm_nt_bf16 / _nn_ / _tn_ (one hand-written kernel for the matrix cores
that reads either operand either way round; no library GEMM is called at the layer's sizes); forward_from_codes() takes the int8 codes of the receive buffer
straight into the first GEMM."""
import torch


def _kernel_serves(x, w):
    """planmoe_gemm_nt_bf16 takes bf16 operands on the GPU whose row lengths are multiples of 8."""
    return (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 3 and
            w.shape[1] % 8 == 0 and w.shape[2] % 8 == 0 and x.shape[0] == w.shape[0] and x.shape[2] == w.shape[1])


class _WeightForms:
    """The [E, out, in] copy of a weight stored [E, in, out] (what the forward GEMM wants as its second
    operand), made again only when the weight has changed (in-place updates bump ._version, a .data
    swap changes the pointer)."""

    def __init__(self):
        self.key, self.value = None, None

    def k_major(self, w):
        from . import ops
        key = (w._version, w.data_ptr(), w.device, w.dtype, tuple(w.shape))
        if self.key != key:
            self.value = ops.transpose_bf16(w.detach())
            self.key = key
        return self.value


class _BatchedLinear(torch.autograd.Function):
    """y = act(x @ w + bias) over experts: x [E, R, in], w [E, in, out] (as the reference stores it),
    bias [E, out], act = relu or nothing; torch.add(torch.matmul(x, w), bias.unsqueeze(1)) of
    experts/ffn.py:77-79 with its two bf16 roundings.  All three products read their operands as they
    lie in memory when the reduction length is a multiple of 64 (planmoe_gemm_nn_bf16 for y,
    planmoe_gemm_nt_bf16 for dx = dy @ w^T, planmoe_gemm_tn_bf16 for dw = x^T @ dy); otherwise y takes a
    transposed copy of w (kept per weight version) and dw transposed copies of x and dy whose row index
    (the reduction) is padded with zeros to the kernel's k-tile.  dbias sums in fp32."""

    @staticmethod
    def forward(ctx, x, w, bias, relu, forms):
        from . import ops
        x = x.contiguous()
        b = bias.detach() if bias is not None else None
        if x.shape[2] % 64 == 0:
            y = ops.gemm_nn_bf16(x, w.detach().contiguous(), b, relu=relu)          # the weight as it is stored
        else:
            y = ops.gemm_nt_bf16(x, forms.k_major(w), b, relu=relu)
        ctx.save_for_backward(x, w, y if relu else None)
        ctx.relu, ctx.has_bias = relu, bias is not None
        return y

    @staticmethod
    def backward(ctx, gy):
        from . import ops
        x, w, y = ctx.saved_tensors
        gy = gy.contiguous()
        if ctx.relu:
            gy = torch.ops.aten.threshold_backward(gy, y, 0.0)      # relu's own backward: one pass over dy and y
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = ops.gemm_nt_bf16(gy, w.detach().contiguous())                    # [E, R, out] x [E, in, out]^T
        if ctx.needs_input_grad[1]:
            if x.shape[1] % 64 == 0:
                dw = ops.gemm_tn_bf16(x, gy)                                          # x^T dy, both as they lie
            else:
                dw = ops.gemm_nt_bf16(ops.transpose_bf16(x, 64), ops.transpose_bf16(gy, 64))      # [E, in, R'] x [E, out, R']^T
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = gy.sum(dim=1, dtype=torch.float32).to(gy.dtype)
        return dx, dw, db, None, None


class FusedExpertsNetwork(torch.nn.Module):
    # experts/ffn.py:13-82, one GPU (no expert sharding)
    def __init__(self, hidden_size_per_expert, activation_fn=None, activation_fn_with_self=None,
                 output_dim=None):
        super().__init__()
        self.hidden_size_per_expert = hidden_size_per_expert
        self.output_dim = output_dim
        if activation_fn_with_self is not None:
            assert activation_fn is None, "Option `activation_fn_with_self` has been specified, please keep exactly one of them."
            activation_fn = lambda x: activation_fn_with_self(x, self)
        self._relu = activation_fn is None          # the default activation: the first GEMM applies it itself
        if activation_fn is None:
            activation_fn = lambda x: torch.nn.functional.relu(x)
        self.activation_fn = activation_fn

    def update(self, ctx):
        model_dim = ctx.model_dim
        local_experts = ctx.num_local_experts
        hidden = self.hidden_size_per_expert
        out = self.output_dim or model_dim
        # parameter names and shapes as the reference's (ffn.py:33-56): fc1 [E, model_dim, hidden],
        # fc2 [E, hidden, out], so that its state dicts load here
        fc1_w = torch.empty(local_experts, model_dim, hidden)
        fc2_w = torch.empty(local_experts, hidden, out)
        fc1_b = torch.empty(local_experts, hidden)
        fc2_b = torch.empty(local_experts, out)
        for i in range(local_experts):
            fc1 = torch.nn.Linear(model_dim, hidden)
            fc2 = torch.nn.Linear(hidden, out)
            fc1_w[i], fc1_b[i] = fc1.weight.t(), fc1.bias
            fc2_w[i], fc2_b[i] = fc2.weight.t(), fc2.bias
        self.batched_fc1_w = torch.nn.Parameter(fc1_w)
        self.batched_fc2_w = torch.nn.Parameter(fc2_w)
        self.batched_fc1_bias = torch.nn.Parameter(fc1_b)
        self.batched_fc2_bias = torch.nn.Parameter(fc2_b)
        self._fc1_k_major = None
        self._fc1_forms, self._fc2_forms = _WeightForms(), _WeightForms()

    # a batched library GEMM is not issued above this many multiply-adds: at the layer's real sizes
    # ([8, 5120, 4096] x [8, 4096, 4096]) torch.matmul's batched bf16 kernel once ended a GPU run with
    # an illegal-address error whose cause could not be established, so the layer stays off that call
    LIBRARY_BATCHED_LIMIT = 1 << 32

    def _linear(self, x, w, bias, relu, forms):
        if _kernel_serves(x, w):
            return _BatchedLinear.apply(x, w, bias, relu, forms)
        # other dtypes / odd sizes: the reference's composite; large products one expert at a time
        if x.is_cuda and x.shape[0] > 1 and x.shape[0] * x.shape[1] * w.shape[1] * w.shape[2] > self.LIBRARY_BATCHED_LIMIT:
            y = torch.stack([torch.addmm(bias[e], x[e], w[e]) for e in range(x.shape[0])])
        else:
            y = torch.add(torch.matmul(x, w), bias.unsqueeze(1))
        return torch.nn.functional.relu(y) if relu else y

    def forward(self, x, ctx):
        # experts/ffn.py:63-82
        y = self._linear(x, self.batched_fc1_w, self.batched_fc1_bias, self._relu, self._fc1_forms)
        if not self._relu:
            y = self.activation_fn(y)
        return self._linear(y, self.batched_fc2_w, self.batched_fc2_bias, False, self._fc2_forms)

    def forward_from_codes(self, codes, bias, scale, exact=True):
        """The same forward with the int8 codes of the receive buffer as input (inference: no autograd
        through the first GEMM): the GEMM reads the codes, so the decompressed [E, C, model_dim]
        tensor is never written.  exact=True (the default): planmoe_ffn_fc1_int8 multiplies the
        decompressor's very values, so the result is that of decompress + GEMM up to the GEMM's
        summation order.  exact=False: planmoe_ffn_fc1_int8_affine puts the codes themselves on the
        matrix cores and applies scale / bias in the epilogue; it skips the decompressor's three
        roundings per element, which is about an ulp of the result for rows whose range is
        comparable to their offset and more than that where |bias| >> scale or the weights'
        column sum cancels -- an approximation to opt into, 1.4 x faster.
        bf16; model_dim % 64 == 0, hidden % 128 == 0."""
        from . import ops
        w = self.batched_fc1_w
        cached = self._fc1_k_major
        key = (w._version, w.data_ptr(), w.device, w.dtype)     # (.data swaps change the pointer, not the version)
        if cached is None or cached[0] != key:
            wk = w.detach().transpose(1, 2).contiguous()                        # [E, hidden, model_dim]
            cached = (key, wk, None if exact else ops.ffn_weight_colsum(wk))
            self._fc1_k_major = cached
        if not exact and cached[2] is None:
            cached = (key, cached[1], ops.ffn_weight_colsum(cached[1]))
            self._fc1_k_major = cached
        if exact:
            y = ops.ffn_fc1_int8(codes, bias, scale, cached[1], self.batched_fc1_bias.detach())
        else:
            y = ops.ffn_fc1_int8_affine(codes, bias, scale, cached[1], cached[2], self.batched_fc1_bias.detach())
        y = self.activation_fn(y)
        return self._linear(y, self.batched_fc2_w, self.batched_fc2_bias, False, self._fc2_forms)


ExpertModule = FusedExpertsNetwork
