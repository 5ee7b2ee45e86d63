"""Fused expert FFN -- mirror of the reference's experts/ffn.py (two batched GEMMs with bias and
activation between dispatch and combine).  forward() is the torch composite of the reference;
forward_from_codes() takes the int8 codes of the receive buffer straight into the first GEMM."""
import torch


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

    def forward(self, x, ctx):
        y = torch.add(torch.matmul(x, self.batched_fc1_w), self.batched_fc1_bias.unsqueeze(1))
        y = self.activation_fn(y)
        y = torch.add(torch.matmul(y, self.batched_fc2_w), self.batched_fc2_bias.unsqueeze(1))
        return y

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
        return torch.add(torch.matmul(y, self.batched_fc2_w), self.batched_fc2_bias.unsqueeze(1))


ExpertModule = FusedExpertsNetwork
