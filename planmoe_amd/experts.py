"""Fused expert FFN -- mirror of the reference's experts/ffn.py (two batched library GEMMs
with bias and activation).  It sits between dispatch and combine and is kept as a torch
composite: only the data path around it is hand-written here."""
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
        fc1_w = torch.empty(1, local_experts, hidden, model_dim)
        fc2_w = torch.empty(1, local_experts, hidden, out)
        fc1_b = torch.empty(1, local_experts, hidden)
        fc2_b = torch.empty(1, local_experts, out)
        for i in range(local_experts):
            fc1 = torch.nn.Linear(model_dim, hidden)
            fc2 = torch.nn.Linear(hidden, out)
            fc1_w[0, i], fc1_b[0, i] = fc1.weight, fc1.bias
            fc2_w[0, i], fc2_b[0, i] = fc2.weight.t(), fc2.bias
        self.batched_fc1_w = torch.nn.Parameter(fc1_w.squeeze(0))
        self.batched_fc2_w = torch.nn.Parameter(fc2_w.squeeze(0))
        self.batched_fc1_bias = torch.nn.Parameter(fc1_b.squeeze(0))
        self.batched_fc2_bias = torch.nn.Parameter(fc2_b.squeeze(0))

    def forward(self, x, ctx):
        w1 = self.batched_fc1_w.permute(0, 2, 1)
        y = torch.add(torch.matmul(x, w1), self.batched_fc1_bias.unsqueeze(1))
        y = self.activation_fn(y)
        y = torch.add(torch.matmul(y, self.batched_fc2_w), self.batched_fc2_bias.unsqueeze(1))
        return y


ExpertModule = FusedExpertsNetwork
