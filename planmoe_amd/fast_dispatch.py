"""Routing and dispatch/combine API -- mirror of the reference's impls/fast_dispatch.py.

Same names, arguments, defaults and return structure; the work is done by libplanmoe_hip
(one launch for all k choices instead of one JIT kernel launch per choice)."""
import torch

from . import host_route, losses, ops
from ._lib import PlanMoEError
from .gating import fast_cumsum_sub_one  # noqa: F401  (re-exported like the reference)


class GatingEncoder(torch.autograd.Function):
    """fast_dispatch.py:16-46: forward = dispatch; backward = combine (+ gate gradient when
    real gates were passed)."""

    @staticmethod
    def forward(ctx, config, reshaped_input, *gates_):
        ctx.reshaped_input = reshaped_input
        ctx.config = config
        ctx.gates = list(gates_) if gates_ else None
        if not reshaped_input.is_cuda:          # host tensors: the reference's CPU entry points, by name
            return host_route.scatter(config, reshaped_input, ctx.gates)
        return ops.dispatch_fwd(reshaped_input, config.indices_, config.locations_, ctx.gates,
                                config.num_global_experts, config.capacity)

    @staticmethod
    def backward(ctx, dispatched_input):
        cfg = ctx.config
        dispatched_input = dispatched_input.contiguous()
        if not dispatched_input.is_cuda:
            grad_gates = host_route.gate_gradients(cfg, ctx.reshaped_input, dispatched_input) if ctx.gates is not None else []
            return (None, host_route.gather(cfg, dispatched_input, ctx.gates), *grad_gates)
        grad_data = ops.combine_fwd(dispatched_input, cfg.indices_, cfg.locations_, ctx.gates,
                                    cfg.sample_size, cfg.capacity)
        grad_gates = []
        if ctx.gates is not None:
            gg = ops.bwd_gate(ctx.reshaped_input, dispatched_input, cfg.indices_, cfg.locations_,
                              cfg.capacity)
            grad_gates = [gg[j] for j in range(len(cfg.indices_))]
        return (None, grad_data, *grad_gates)


class GatingDecoder(torch.autograd.Function):
    """fast_dispatch.py:49-79: forward = combine; backward = dispatch of the gated gradient
    (+ gate gradient when real gates were passed)."""

    @staticmethod
    def forward(ctx, config, expert_output, *gates_):
        ctx.expert_output = expert_output
        ctx.config = config
        ctx.gates = list(gates_) if gates_ else None
        if not expert_output.is_cuda:
            return host_route.gather(config, expert_output, ctx.gates)
        return ops.combine_fwd(expert_output, config.indices_, config.locations_, ctx.gates,
                               config.sample_size, config.capacity)

    @staticmethod
    def backward(ctx, combined_output):
        cfg = ctx.config
        combined_output = combined_output.contiguous()
        if not combined_output.is_cuda:
            grad_gates = host_route.gate_gradients(cfg, combined_output, ctx.expert_output) if ctx.gates is not None else []
            return (None, host_route.scatter(cfg, combined_output, ctx.gates), *grad_gates)
        grad_expert_output = ops.dispatch_fwd(combined_output, cfg.indices_, cfg.locations_, ctx.gates,
                                              cfg.num_global_experts, cfg.capacity)
        grad_gates = []
        if ctx.gates is not None:
            gg = ops.bwd_gate(combined_output, ctx.expert_output, cfg.indices_, cfg.locations_,
                              cfg.capacity)
            grad_gates = [gg[j] for j in range(len(cfg.indices_))]
        return (None, grad_expert_output, *grad_gates)


class TutelMoeFastDispatcher:
    """fast_dispatch.py:82-131.  The compute dtype is fp32 for every input dtype but fp16
    on CUDA in the reference (:91-93); here the kernels read and write the input dtype directly
    and do the same fp32 arithmetic in registers, which gives the same bits without the two
    full-tensor casts."""

    def __init__(self, num_global_experts, capacity, model_dim, dispatch_dtype):
        self.num_global_experts = int(num_global_experts)
        self.capacity = int(capacity)
        self.model_dim = int(model_dim)
        self.dtype = torch.float32
        self.original_dtype = dispatch_dtype
        self.aligned_dim = model_dim
        self.is_cuda = None

    def update(self, indices_, locations_, gates_, capacity=None, is_postscore=True):
        self.indices_ = [x.to(torch.int32).view(-1) for x in indices_]
        self.locations_ = [x.to(torch.int32) for x in locations_]
        self.gates_ = [x.to(self.dtype) for x in gates_]
        self.is_postscore = is_postscore
        self.sample_size, self.capacity = int(self.indices_[0].size(0)), int(capacity) or self.capacity
        self.is_cuda = self.indices_[0].is_cuda

    def _host(self, data):
        # fast_dispatch.py:105-113: host routing tensors select the CPU kernels; they take fp32 / fp64
        # rows (jit_compiler.py:40-49), so other dtypes pass through the dispatcher's compute dtype
        if data.is_cuda:
            raise PlanMoEError("fast_dispatcher: routing tensors on the host, data on the GPU")
        return data.to(self.original_dtype if self.original_dtype is torch.float64 else self.dtype).contiguous()

    def encode(self, data):
        if not self.is_cuda:
            host = self._host(data)
            out = GatingEncoder.apply(self, host) if self.is_postscore else GatingEncoder.apply(self, host, *self.gates_)
            return out.to(self.original_dtype)
        data = data.to(self.original_dtype).contiguous()
        if self.is_postscore:
            return GatingEncoder.apply(self, data)
        return GatingEncoder.apply(self, data, *self.gates_)

    def decode(self, data):
        if not self.is_cuda:
            host = self._host(data)
            out = GatingDecoder.apply(self, host, *self.gates_) if self.is_postscore else GatingDecoder.apply(self, host)
            return out.to(self.original_dtype)
        data = data.to(self.original_dtype).contiguous()
        if self.is_postscore:
            return GatingDecoder.apply(self, data, *self.gates_)
        return GatingDecoder.apply(self, data)


fast_dispatcher = TutelMoeFastDispatcher


class _Route(torch.autograd.Function):
    """Routing with gradients: forward = the routing kernels, backward = planmoe_route_bwd.
    `inp` are scores, or logits when is_logits (softmax inside the kernel).  Outputs: gates
    [k, T] and l_aux (differentiable), indices / locations / counts / scores (not)."""

    @staticmethod
    def forward(ctx, inp, top_k, is_logits, normalize_gate, want_l_aux):
        r = ops.route_topk(inp.detach().contiguous(), top_k, is_logits=is_logits, normalize_gate=normalize_gate,
                           want_scores=is_logits, want_l_aux=want_l_aux, want_counts=True)
        scores = r["scores"] if is_logits else inp.detach().contiguous()
        ctx.save_for_backward(scores, r["indices"], r["counts"])
        ctx.normalize_gate, ctx.is_logits, ctx.want_l_aux = normalize_gate, is_logits, want_l_aux
        l_aux = r["l_aux"] if want_l_aux else inp.new_zeros(())
        ctx.mark_non_differentiable(r["indices"], r["locations"], r["counts"])
        return r["gates"], l_aux, r["indices"], r["locations"], r["counts"]

    @staticmethod
    def backward(ctx, grad_gates, grad_l_aux, *unused):
        scores, indices, counts = ctx.saved_tensors
        if grad_gates is None:
            grad_gates = torch.zeros((indices.shape[0], scores.shape[0]), dtype=scores.dtype, device=scores.device)
        dl = grad_l_aux if (ctx.want_l_aux and grad_l_aux is not None) else None
        grad = ops.route_bwd(scores, indices, grad_gates, ctx.normalize_gate, dl, counts if dl is not None else None,
                             through_softmax=ctx.is_logits)
        return grad, None, None, None, None


def route(inp, top_k, is_logits=False, normalize_gate=True, want_l_aux=True):
    """(gates [k,T], l_aux, indices [k,T], locations [k,T], counts [k,E]); gates and l_aux carry
    gradients back to `inp` when it requires them."""
    return _Route.apply(inp, top_k, is_logits, normalize_gate, want_l_aux)


def extract_critical(scores, top_k, loss_fn=losses.gshard_loss, capacity_factor=1.0,
                     batch_prioritized_routing=False, normalize_gate=True, group=None, alignment=1):
    """fast_dispatch.py:140-195.  Returns ((E, indices_s, locations_s, gates_s, capacity), l_loss).
    gates_s and the GShard l_loss carry gradients back into `scores`.

    batch_prioritized_routing (fast_dispatch.py:135-138, 152-154): tokens take their slots in
    the order of their largest score, highest first.  The reference sorts with an unstable
    argsort; here tokens with equal importance keep their token order."""
    if not scores.is_cuda:
        # host scores: the reference's torch ops (an explicit branch; GPU scores never take it)
        return host_route.extract_critical(scores, top_k, loss_fn, capacity_factor, batch_prioritized_routing,
                                           normalize_gate, alignment)
    num_global_experts = int(scores.size(1))
    top_k = min(top_k, num_global_experts)
    want_kernel_loss = loss_fn is losses.gshard_loss
    gates, l_aux, indices, locations, _ = route(scores, top_k, False, normalize_gate, want_kernel_loss)
    if batch_prioritized_routing:
        importance_scores = -1 * scores.detach().max(dim=1)[0]
        order = torch.argsort(importance_scores, dim=0, stable=True).to(torch.int32)
        locations, _ = ops.route_locations(indices, num_global_experts, order)
    indices_s = [indices[j] for j in range(top_k)]
    locations_s = [locations[j] for j in range(top_k)]
    gates_s = [gates[j] for j in range(top_k)]

    if loss_fn is None:
        l_loss = None
    elif want_kernel_loss:
        l_loss = l_aux.to(scores.dtype)
    else:
        topk_indices = torch.stack(indices_s, dim=1).to(torch.int64)
        l_loss = loss_fn(scores, topk_indices)

    samples = int(scores.size(0))
    if capacity_factor > 0:
        capacity = ops.capacity(samples, num_global_experts, top_k, capacity_factor, alignment)
    else:
        # data-dependent capacity (fast_dispatch.py:183-186); world size 1, so no all-reduce
        capacity = int(torch.max(locations)) + 1
        if capacity_factor < 0:
            per_expert = (samples + num_global_experts - 1) // num_global_experts
            capacity = min(capacity, top_k * int(-capacity_factor * per_expert))
        remainder = capacity % alignment
        if remainder > 0:
            capacity = capacity + alignment - remainder
    return (num_global_experts, indices_s, locations_s, gates_s, capacity), l_loss


def fast_encode(data, critial_data, is_postscore=True):
    # fast_dispatch.py:197-201
    num_global_experts = critial_data[0]
    dispatcher = TutelMoeFastDispatcher(num_global_experts, 0, data.size(-1), data.dtype)
    dispatcher.update(*critial_data[1:], is_postscore=is_postscore)
    return dispatcher.encode(data).view(num_global_experts, -1, data.size(-1))


def fast_decode(data, critial_data, is_postscore=True):
    # fast_dispatch.py:203-207
    num_global_experts = critial_data[0]
    dispatcher = TutelMoeFastDispatcher(num_global_experts, 0, data.size(-1), data.dtype)
    dispatcher.update(*critial_data[1:], is_postscore=is_postscore)
    return dispatcher.decode(data.reshape(-1, data.size(-1))).view(-1, data.size(-1))
