"""MOELayer -- mirror of the reference's impls/moe_layer.py for one GPU (world size 1).

routing -> fast_encode -> compress / (identity all-to-all) / decompress -> experts ->
compress / (identity all-to-all) / decompress -> fast_decode, with the reference's
constructor and forward signatures, defaults and dtype flow."""
import logging
import os
import re

import torch
from torch.nn import ModuleList

from . import experts as _experts
from . import gates as _gates
from . import losses, ops
from .fast_dispatch import extract_critical, fast_decode, fast_encode, route
from . import overlap as _overlap
from .overlap import (a2a_ffn_overlap_forward, fused_gate_eligible, fused_gate_forward, fused_int8_eligible,
                      fused_int8_forward, fused_zfp_eligible, fused_zfp_forward, gate_route_eligible,
                      gate_route_encode, zfp_experts_decode)


class MOELayer(torch.nn.Module):
    @staticmethod
    def global_expert_count(num_local_experts, group=None):
        # moe_layer.py:30-42 with world_size == 1
        if not isinstance(num_local_experts, int):
            num_local_experts = -int(1 / (num_local_experts + 1e-5))
        if num_local_experts == 0:
            raise Exception("Invalid value of num_local_experts: %d" % num_local_experts)
        if num_local_experts > 0:
            return num_local_experts
        assert 1 % -num_local_experts == 0, \
            "Excepting {-num_local_experts} devices to share an expert param, while global device count is {world_size}."
        return 1 // -num_local_experts

    def __init__(self, gate_type, model_dim, experts=None, scan_expert_func=None, result_func=None,
                 group=None, seeds=None, a2a_ffn_overlap_degree=1, is_postscore=True,
                 batch_prioritized_routing=False, normalize_gate=True, is_gshard_loss=True,
                 parallel_type='auto', use_2dh=False, index=0, compress_name='no', comm_name='naive',
                 **kwargs):
        super().__init__()
        assert model_dim % 2 == 0, "Model_dim (%s) must be even value, while this Model_dim mod 2 > 0." % model_dim
        if 'pad_samples' in kwargs:
            logging.warning("`pad_samples` option in Tutel Moe-layer has been deprecated, as Tutel always assumes `pad_samples=False` for better efficiency.")
            kwargs.pop('pad_samples')
        for k in kwargs:
            raise Exception('Unrecognized argument provided to Tutel Moe-layer: %s' % k)

        self.group = group
        self.result_func = result_func
        self.skip_moe = (int(os.environ.get('SKIP_MOE', '0')) != 0)
        self.num_local_experts = experts.pop('count_per_node', 1)
        self.num_global_experts = MOELayer.global_expert_count(self.num_local_experts, self.group)
        self.world_size = 1
        self.sharded_count = 1
        self.auto_parallel, self.use_model_parallel = False, False
        self.model_dim = model_dim
        self.is_postscore = is_postscore
        self.batch_prioritized_routing = batch_prioritized_routing
        if int(os.environ.get('BATCH_PRIO', 0)) != 0:
            self.batch_prioritized_routing = True
        self.normalize_gate = normalize_gate
        self.is_gshard_loss = is_gshard_loss
        self.a2a_ffn_overlap_degree = a2a_ffn_overlap_degree
        self.use_2dh = use_2dh
        self.compress_name = compress_name
        self.comm_name = comm_name

        if seeds is not None and seeds[1] is not None:
            torch.manual_seed(seeds[1])

        experts_type = experts.pop('type')
        if experts_type == 'custom':
            self.experts = experts['module']
        else:
            assert re.match(r'[a-zA-Z0-9\_]+', experts_type), \
                "Expert type must only include digits, letters and underline characters."
            if experts_type != 'ffn':
                raise Exception('Builtin expert type is not recognized: %s' % experts_type)
            assert 'fused_custom_fn' not in experts
            assert 'implicit_dropout_p' not in experts
            self.experts = _experts.ExpertModule(**experts)
        self.experts.update(self)

        if scan_expert_func is not None:
            for n, p in self.experts.named_parameters():
                scan_expert_func(n, p)
        for n, p in self.experts.named_parameters():
            setattr(p, '_tutel_expert', True)

        if isinstance(gate_type, str):
            assert re.match(r'^Top[0-9]+Gate$', gate_type), "Unrecognized gate_type: %s" % gate_type
            top_k = int(gate_type[3:-4])
            logging.warning(f"gate_type value `{gate_type}` in Tutel Moe-layer has been deprecated, please use gate_type = {{'type': 'top', 'k': {top_k}}} instead.")
            gate_type = {'type': 'top', 'k': top_k}
        if not isinstance(gate_type, list):
            gate_type = [gate_type]

        self.gates = []
        for gi, single_gate_type in enumerate(gate_type):
            gate_name = single_gate_type['type']
            single_gate_type.pop('type')
            assert re.match(r'[a-zA-Z0-9\_]+', gate_name), \
                "Gate type must only include digits, letters and underline characters."
            if seeds is not None and seeds[0] is not None:
                torch.manual_seed(seeds[0] + gi)
            if gate_name not in _gates.GATES:
                raise Exception("Unrecognized gate_type: %s" % gate_name)
            gate_module = _gates.GATES[gate_name](model_dim=self.model_dim, num_global_experts=self.num_global_experts,
                                                  **single_gate_type)
            if not hasattr(gate_module, 'gate_noise'):
                gate_module.gate_noise = single_gate_type.get('gate_noise', 0.0)
            if not hasattr(gate_module, 'capacity_factor'):
                gate_module.capacity_factor = single_gate_type.get(
                    'capacity_factor', float(os.environ.get('CAP_FACTOR', 1.0)))
            self.gates += [gate_module]
        self.gates = ModuleList(self.gates)

        if seeds is not None and len(seeds) > 2 and seeds[2] is not None:
            torch.manual_seed(seeds[2])
        self.save_count = 0

    def extra_repr(self):
        return 'Top-K(s) = %s, Total-Experts = %d [managed by %d device(s)],' % (
            [f'k={x.top_k}, noise={x.gate_noise}' for x in self.gates], self.num_global_experts,
            self.world_size)

    def get_parameter_iterator(self, param_type):
        if param_type == 'gate':
            return self.gates.named_parameters()
        elif param_type == 'local_experts':
            return self.experts.named_parameters()
        raise Exception("Specified parameter type is not recognized: %s. Valid `param_type` includes: gate, local_experts." % param_type)

    def expert_local(self, x, reserve_shape):
        y = self.experts(x.view(x.size(0), x.size(1), *reserve_shape), self)
        self.protected_shape = y.shape
        return y.reshape(y.size(0), y.size(1), -1)

    def forward(self, input, gate_index=0, capacity_factor=None, top_k=None, a2a_ffn_overlap_degree=None,
                reserve_dims=1):
        if self.skip_moe:
            result_output = input
            result_output.l_aux = None
            return self.result_func(result_output) if self.result_func is not None else result_output

        original_shape, original_dtype = input.shape, input.dtype
        assert len(original_shape) >= 2, "Input data must be at least 2D tensor: (s)amples, .., (m)odel_dim"
        x = input.reshape(-1, original_shape[-reserve_dims:].numel())
        for p in self.experts.parameters():
            x = x.to(p.dtype)
            break
        gctx = self.gates[gate_index]
        degree = a2a_ffn_overlap_degree if a2a_ffn_overlap_degree is not None else self.a2a_ffn_overlap_degree
        k = gctx.top_k if top_k is None else top_k
        cf = gctx.capacity_factor if capacity_factor is None else capacity_factor
        alignment = 4 * self.sharded_count * degree

        noisy = self.training and gctx.gate_noise > 0
        plain = (self.is_gshard_loss and not self.batch_prioritized_routing and cf > 0)
        if (plain and not noisy and _overlap.FUSE_GATE and
                fused_gate_eligible(x, gctx, self.num_global_experts, self.compress_name, degree, self.is_postscore)):
            # gate GEMM, routing, encode and compress as one two-launch call; decompress + decode
            # in one pass (same routing and the same bits per stage as the steps below)
            kk = min(k, self.num_global_experts)
            cap = ops.capacity(x.size(0), self.num_global_experts, kk, cf, alignment)
            if self.training:
                self.save_count = self.save_count + 1

            def expert_fn(expert_input):
                return self.expert_local(expert_input, original_shape[-reserve_dims:])
            y, l_aux = fused_gate_forward(x, gctx, kk, cap, self.normalize_gate, expert_fn, degree)
            l_aux = l_aux.to(torch.float32 if gctx.fp32_gate else x.dtype)
            y = y.view(list(original_shape)).to(original_dtype)
            self.l_aux = y.l_aux = l_aux
            return self.result_func(y) if self.result_func is not None else y

        if plain and not noisy and gate_route_eligible(x, gctx, self.num_global_experts, self.is_postscore):
            # gate GEMM + routing as one call and one node of the graph together with the encode (the
            # same routing and the same bits as the steps below); codec, comm and decode as below
            kk = min(k, self.num_global_experts)
            cap = ops.capacity(x.size(0), self.num_global_experts, kk, cf, alignment)
            zfp = fused_zfp_eligible(x, self.compress_name, degree, self.is_postscore, self.num_global_experts, cap)
            y, gates, l_aux, indices, locations = gate_route_encode(x, gctx, kk, cap, self.normalize_gate,
                                                                    'zfp' if zfp else 'plain')
            l_aux = l_aux.to(torch.float32 if gctx.fp32_gate else x.dtype)
            if self.training:
                self.save_count = self.save_count + 1

            def expert_fn(expert_input):
                return self.expert_local(expert_input, original_shape[-reserve_dims:])
            y = y.view(self.num_global_experts, cap, x.shape[-1])
            if zfp:
                y = zfp_experts_decode(y, expert_fn, degree, indices, locations, gates, x.shape[0])
            else:
                y = a2a_ffn_overlap_forward(y, expert_fn=expert_fn, a2a_ffn_overlap_degree=degree,
                                            use_2dh=self.use_2dh, group=self.group,
                                            compress_name=self.compress_name, comm_name=self.comm_name)
                crit = (self.num_global_experts, [indices[j] for j in range(kk)],
                        [locations[j] for j in range(kk)], [gates[j] for j in range(kk)], cap)
                y = fast_decode(y.to(x.dtype), crit, self.is_postscore)
            y = y.view(list(original_shape)).to(original_dtype)
            self.l_aux = y.l_aux = l_aux
            return self.result_func(y) if self.result_func is not None else y

        # routing (moe_layer.py:230-256)
        logits = gctx(x)
        if noisy:
            logits_w_noise = logits + gctx.gate_noise * torch.randn_like(logits) / self.num_global_experts
        else:
            logits_w_noise = logits
        if plain:
            # softmax, top-k, slots, gates and the GShard loss in one routing call
            kk = min(k, self.num_global_experts)
            gates, l_aux, indices, locations, _ = route(logits_w_noise.contiguous(), kk, True,
                                                        self.normalize_gate, True)
            cap = ops.capacity(x.size(0), self.num_global_experts, kk, cf, alignment)
            crit = (self.num_global_experts, [indices[j] for j in range(kk)],
                    [locations[j] for j in range(kk)], [gates[j] for j in range(kk)], cap)
            l_aux = l_aux.to(logits.dtype)
        else:
            scores = torch.softmax(logits_w_noise, dim=1)
            if self.is_gshard_loss:
                loss_fn = losses.gshard_loss
            else:
                def loss_fn(gates, topk_ids):
                    return losses.load_importance_loss(torch.softmax(logits, dim=1),
                                                       logits_w_noise.gather(index=topk_ids, dim=1),
                                                       self.num_global_experts, gctx.gate_noise)
            crit, l_aux = extract_critical(scores, top_k=k, loss_fn=loss_fn, capacity_factor=cf,
                                           batch_prioritized_routing=self.batch_prioritized_routing,
                                           normalize_gate=self.normalize_gate, group=self.group,
                                           alignment=alignment)

        if fused_int8_eligible(x, self.compress_name, degree, self.is_postscore):
            # encode + compress and decompress + decode in one pass each (bit-identical to the steps)
            if self.training:
                self.save_count = self.save_count + 1

            def expert_fn(expert_input):
                return self.expert_local(expert_input, original_shape[-reserve_dims:])
            y = fused_int8_forward(x, crit, expert_fn, degree)
            y = y.view(list(original_shape)).to(original_dtype)
            self.l_aux = y.l_aux = l_aux
            return self.result_func(y) if self.result_func is not None else y

        if fused_zfp_eligible(x, self.compress_name, degree, self.is_postscore, crit[0], crit[4]):
            # encode + compress in one pass, forward and (with the gates) backward
            if self.training:
                self.save_count = self.save_count + 1

            def expert_fn(expert_input):
                return self.expert_local(expert_input, original_shape[-reserve_dims:])
            y = fused_zfp_forward(x, crit, expert_fn, degree)
            y = y.view(list(original_shape)).to(original_dtype)
            self.l_aux = y.l_aux = l_aux
            return self.result_func(y) if self.result_func is not None else y

        # the reference casts x to the logits dtype around fast_encode / fast_decode
        # (moe_layer.py:265, 306); the kernels do that fp32 arithmetic in registers
        y = fast_encode(x, crit, self.is_postscore)

        if self.training:
            self.save_count = self.save_count + 1

        def expert_fn(expert_input):
            return self.expert_local(expert_input, original_shape[-reserve_dims:])
        y = a2a_ffn_overlap_forward(y, expert_fn=expert_fn, a2a_ffn_overlap_degree=degree,
                                    use_2dh=self.use_2dh, group=self.group,
                                    compress_name=self.compress_name, comm_name=self.comm_name)

        y = fast_decode(y.to(x.dtype), crit, self.is_postscore)
        y = y.view(list(original_shape)).to(original_dtype)
        self.l_aux = y.l_aux = l_aux
        return self.result_func(y) if self.result_func is not None else y


moe_layer = MOELayer
