"""MOELayer for one GPU (world size 1) behind the interface of the reference's impls/moe_layer.py:
the constructor and forward signatures, defaults, environment knobs (SKIP_MOE, BATCH_PRIO,
CAP_FACTOR), error texts and dtype flow of moe_layer.py:44-311.

    gate -> routing -> fast_encode -> compress / (identity all-to-all) / decompress -> experts
         -> compress / (identity all-to-all) / decompress -> fast_decode

forward() picks, per call, the most fused send / receive side whose conditions the call meets
(`_SendPlan`); every choice gives the routing and the bits of the step-by-step pipeline, which is
the last choice and the reference's own structure.  Two exceptions, both in the experts and both
tolerance-level as any GEMM is: under no_grad the built-in FFN's first GEMM reads the int8 codes
(the decompressor's very values, summed in this kernel's order, overlap.FFN_FROM_CODES), and
overlap.FFN_FROM_CODES_AFFINE opts into a faster form that skips the decompressor's roundings."""
import logging
import os
import re

import torch

from . import experts as _experts
from . import gates as _gates
from . import losses, ops
from . import overlap as _overlap
from .fast_dispatch import extract_critical, fast_decode, fast_encode, route

_NAME = re.compile(r'[a-zA-Z0-9\_]+')
_LEGACY_GATE = re.compile(r'^Top[0-9]+Gate$')


def _env_flag(name):
    return int(os.environ.get(name, '0')) != 0


class MOELayer(torch.nn.Module):
    # ------------------------------------------------------------------ construction
    @staticmethod
    def global_expert_count(num_local_experts, group=None):
        """Experts over all ranks (moe_layer.py:30-42); one rank here.  A fractional count 1/n means
        n devices share one expert, which one device can only do for n == 1."""
        world_size = 1
        if not isinstance(num_local_experts, int):
            num_local_experts = -int(1 / (num_local_experts + 1e-5))
        if num_local_experts == 0:
            raise Exception("Invalid value of num_local_experts: %d" % num_local_experts)
        if num_local_experts > 0:
            return num_local_experts * world_size
        sharing = -num_local_experts
        assert world_size % sharing == 0, \
            f"Excepting {sharing} devices to share an expert param, while global device count is {world_size}."
        return world_size // sharing

    def __init__(self, gate_type, model_dim, experts=None, scan_expert_func=None, result_func=None,
                 group=None, seeds=None, a2a_ffn_overlap_degree=1, is_postscore=True,
                 batch_prioritized_routing=False, normalize_gate=True, is_gshard_loss=True,
                 parallel_type='auto', use_2dh=False, index=0, compress_name='no', comm_name='naive',
                 **kwargs):
        super().__init__()
        assert model_dim % 2 == 0, "Model_dim (%s) must be even value, while this Model_dim mod 2 > 0." % model_dim
        self._reject_unknown(kwargs)
        seeds = tuple(seeds) + (None,) * 3 if seeds is not None else (None,) * 3

        # what the caller asked for
        self.model_dim = model_dim
        self.group, self.result_func = group, result_func
        self.is_postscore, self.normalize_gate, self.is_gshard_loss = is_postscore, normalize_gate, is_gshard_loss
        self.batch_prioritized_routing = batch_prioritized_routing or _env_flag('BATCH_PRIO')
        self.a2a_ffn_overlap_degree, self.use_2dh = a2a_ffn_overlap_degree, use_2dh
        self.compress_name, self.comm_name = compress_name, comm_name
        self.skip_moe = _env_flag('SKIP_MOE')
        # what one rank makes of it
        self.world_size, self.sharded_count = 1, 1
        self.auto_parallel, self.use_model_parallel = False, False
        self.num_local_experts = experts.pop('count_per_node', 1)
        self.num_global_experts = MOELayer.global_expert_count(self.num_local_experts, group)

        self.experts = self._make_experts(experts, seeds[1], scan_expert_func)
        self.gates = torch.nn.ModuleList(self._make_gates(gate_type, seeds[0]))
        if seeds[2] is not None:
            torch.manual_seed(seeds[2])
        self.save_count = 0

    @staticmethod
    def _reject_unknown(kwargs):
        if 'pad_samples' in kwargs:
            logging.warning("`pad_samples` option in Tutel Moe-layer has been deprecated, as Tutel always assumes `pad_samples=False` for better efficiency.")
        for name in kwargs:
            if name != 'pad_samples':
                raise Exception('Unrecognized argument provided to Tutel Moe-layer: %s' % name)

    def _make_experts(self, spec, seed, scan_expert_func):
        """experts = {'type': 'ffn' | 'custom', ...} (moe_layer.py:119-146); the dict is consumed."""
        if seed is not None:
            torch.manual_seed(seed)
        kind = spec.pop('type')
        if kind == 'custom':
            module = spec['module']
        else:
            assert _NAME.match(kind), "Expert type must only include digits, letters and underline characters."
            if kind != 'ffn':
                raise Exception('Builtin expert type is not recognized: %s' % kind)
            assert 'fused_custom_fn' not in spec
            assert 'implicit_dropout_p' not in spec
            module = _experts.ExpertModule(**spec)
        module.update(self)
        for name, param in module.named_parameters():
            if scan_expert_func is not None:
                scan_expert_func(name, param)
            setattr(param, '_tutel_expert', True)
        return module

    def _make_gates(self, gate_type, seed):
        """One gate module per entry of gate_type (moe_layer.py:148-190); 'TopNGate' strings are the
        deprecated spelling of {'type': 'top', 'k': N}."""
        if isinstance(gate_type, str):
            assert _LEGACY_GATE.match(gate_type), "Unrecognized gate_type: %s" % gate_type
            top_k = int(gate_type[3:-4])
            logging.warning(f"gate_type value `{gate_type}` in Tutel Moe-layer has been deprecated, please use gate_type = {{'type': 'top', 'k': {top_k}}} instead.")
            gate_type = {'type': 'top', 'k': top_k}
        modules = []
        for position, spec in enumerate(gate_type if isinstance(gate_type, list) else [gate_type]):
            name = spec.pop('type')
            assert _NAME.match(name), "Gate type must only include digits, letters and underline characters."
            if seed is not None:
                torch.manual_seed(seed + position)
            if name not in _gates.GATES:
                raise Exception("Unrecognized gate_type: %s" % name)
            gate = _gates.GATES[name](model_dim=self.model_dim, num_global_experts=self.num_global_experts, **spec)
            if not hasattr(gate, 'gate_noise'):
                gate.gate_noise = spec.get('gate_noise', 0.0)
            if not hasattr(gate, 'capacity_factor'):
                gate.capacity_factor = spec.get('capacity_factor', float(os.environ.get('CAP_FACTOR', 1.0)))
            modules.append(gate)
        return modules

    # ------------------------------------------------------------------ introspection
    def extra_repr(self):
        gates = ['k=%s, noise=%s' % (g.top_k, g.gate_noise) for g in self.gates]
        return 'Top-K(s) = %s, Total-Experts = %d [managed by %d device(s)],' % (gates, self.num_global_experts,
                                                                               self.world_size)

    def get_parameter_iterator(self, param_type):
        owners = {'gate': self.gates, 'local_experts': self.experts}
        if param_type not in owners:
            raise Exception("Specified parameter type is not recognized: %s. Valid `param_type` includes: gate, local_experts." % param_type)
        return owners[param_type].named_parameters()

    def expert_local(self, x, reserve_shape):
        y = self.experts(x.view(x.size(0), x.size(1), *reserve_shape), self)
        self.protected_shape = y.shape
        return y.reshape(y.size(0), y.size(1), -1)

    # ------------------------------------------------------------------ forward
    def _deliver(self, y, l_aux, shape, dtype):
        """Common tail of every path (moe_layer.py:306-311)."""
        y = y.view(list(shape)).to(dtype)
        self.l_aux = y.l_aux = l_aux
        return self.result_func(y) if self.result_func is not None else y

    def forward(self, input, gate_index=0, capacity_factor=None, top_k=None, a2a_ffn_overlap_degree=None,
                reserve_dims=1):
        if self.skip_moe:
            input.l_aux = None
            return self.result_func(input) if self.result_func is not None else input

        shape, dtype = input.shape, input.dtype
        assert len(shape) >= 2, "Input data must be at least 2D tensor: (s)amples, .., (m)odel_dim"
        reserve_shape = shape[-reserve_dims:]
        x = input.reshape(-1, reserve_shape.numel())
        first = next(iter(self.experts.parameters()), None)
        if first is not None:
            x = x.to(first.dtype)

        gate = self.gates[gate_index]
        E = self.num_global_experts
        degree = self.a2a_ffn_overlap_degree if a2a_ffn_overlap_degree is None else a2a_ffn_overlap_degree
        k = gate.top_k if top_k is None else top_k
        cf = gate.capacity_factor if capacity_factor is None else capacity_factor
        alignment = 4 * self.sharded_count * degree
        noisy = self.training and gate.gate_noise > 0
        # "plain" routing: what the routing kernels cover (GShard loss, token order, static capacity)
        plain = self.is_gshard_loss and not self.batch_prioritized_routing and cf > 0

        def expert_fn(expert_input):
            return self.expert_local(expert_input, reserve_shape)

        def count_step():
            if self.training:
                self.save_count = self.save_count + 1

        def pipeline(buffer):
            # compress -> comm -> decompress around the experts, in a2a_ffn_overlap_degree slices
            return _overlap.a2a_ffn_overlap_forward(buffer, expert_fn=expert_fn, a2a_ffn_overlap_degree=degree,
                                                    use_2dh=self.use_2dh, group=self.group,
                                                    compress_name=self.compress_name, comm_name=self.comm_name)

        if plain and not noisy:
            kk = min(k, E)
            cap = ops.capacity(x.size(0), E, kk, cf, alignment)
            loss_dtype = torch.float32 if getattr(gate, 'fp32_gate', False) else x.dtype
            if _overlap.FUSE_GATE and _overlap.fused_gate_eligible(x, gate, E, self.compress_name, degree,
                                                                   self.is_postscore):
                # gate GEMM, routing, encode and compress as one call; decompress + decode in one pass
                count_step()
                y, l_aux = _overlap.fused_gate_forward(x, gate, kk, cap, self.normalize_gate, expert_fn, degree,
                                                       _overlap.ffn_from_codes_fn(self.experts, x, degree, reserve_dims))
                return self._deliver(y, l_aux.to(loss_dtype), shape, dtype)
            if _overlap.gate_route_eligible(x, gate, E, self.is_postscore):
                # gate GEMM + routing as one call and one node of the graph together with the encode
                zfp = _overlap.fused_zfp_eligible(x, self.compress_name, degree, self.is_postscore, E, cap)
                y, gates, l_aux, indices, locations = _overlap.gate_route_encode(
                    x, gate, kk, cap, self.normalize_gate, 'zfp' if zfp else 'plain')
                count_step()
                y = y.view(E, cap, x.shape[-1])
                if zfp:
                    y = _overlap.zfp_experts_decode(y, expert_fn, degree, indices, locations, gates, x.shape[0])
                else:
                    crit = (E, list(indices.unbind(0)), list(locations.unbind(0)), list(gates.unbind(0)), cap)
                    y = fast_decode(pipeline(y).to(x.dtype), crit, self.is_postscore)
                return self._deliver(y, l_aux.to(loss_dtype), shape, dtype)

        crit, l_aux = self._route(gate, x, k, cf, alignment, noisy, plain)

        if _overlap.fused_int8_eligible(x, self.compress_name, degree, self.is_postscore):
            # encode + compress and decompress + decode in one pass each
            count_step()
            codes_fn = _overlap.ffn_from_codes_fn(self.experts, x, degree, reserve_dims)
            return self._deliver(_overlap.fused_int8_forward(x, crit, expert_fn, degree, codes_fn), l_aux, shape, dtype)
        if _overlap.fused_zfp_eligible(x, self.compress_name, degree, self.is_postscore, crit[0], crit[4]):
            count_step()
            return self._deliver(_overlap.fused_zfp_forward(x, crit, expert_fn, degree), l_aux, shape, dtype)

        # the reference's own sequence.  It casts x to the logits dtype around fast_encode / fast_decode
        # (moe_layer.py:265, 306); the kernels do that fp32 arithmetic in registers.
        y = fast_encode(x, crit, self.is_postscore)
        count_step()
        y = fast_decode(pipeline(y).to(x.dtype), crit, self.is_postscore)
        return self._deliver(y, l_aux, shape, dtype)

    def _route(self, gate, x, k, cf, alignment, noisy, plain):
        """The routing closure of moe_layer.py:230-256 -> (crit, l_aux).  Everything torch computes
        here runs with autocast off, as the reference's closure does (:258-260)."""
        E = self.num_global_experts
        logits = gate(x)
        with torch.autocast(device_type=x.device.type, enabled=False):
            if noisy:
                logits_w_noise = logits + gate.gate_noise * torch.randn_like(logits) / E
            else:
                logits_w_noise = logits
            if plain:
                # softmax, top-k, slots, gates and the GShard loss in one routing call
                kk = min(k, E)
                gates, l_aux, indices, locations, _ = route(logits_w_noise.contiguous(), kk, True,
                                                            self.normalize_gate, True)
                cap = ops.capacity(x.size(0), E, kk, cf, alignment)
                crit = (E, list(indices.unbind(0)), list(locations.unbind(0)), list(gates.unbind(0)), cap)
                return crit, l_aux.to(logits.dtype)
            scores = torch.softmax(logits_w_noise, dim=1)
            if self.is_gshard_loss:
                loss_fn = losses.gshard_loss
            else:
                def loss_fn(gates, topk_ids):
                    return losses.load_importance_loss(torch.softmax(logits, dim=1),
                                                       logits_w_noise.gather(index=topk_ids, dim=1), E,
                                                       gate.gate_noise)
            return extract_critical(scores, top_k=k, loss_fn=loss_fn, capacity_factor=cf,
                                    batch_prioritized_routing=self.batch_prioritized_routing,
                                    normalize_gate=self.normalize_gate, group=self.group, alignment=alignment)


moe_layer = MOELayer
