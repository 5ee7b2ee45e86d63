"""The reference's route for tensors that live on the HOST (fast_dispatch.py:105-113 picks the CPU
kernel triple for CPU tensors; jit_compiler.py:40-49 sends them to invoke_cpu_fp32 / invoke_cpu_fp64;
the routing around them is plain torch ops, fast_dispatch.py:140-195, with torch.cumsum in place of
the cumsum kernel, jit_kernels/gating.py:13-22).

Reached only through an explicit `not tensor.is_cuda` branch of the callers in fast_dispatch.py and
gating.py: a GPU tensor never ends up here, and nothing here touches the GPU.  It is the baseline
the reference runs without a GPU, single-threaded loops in the tensors' dtype, not a fast path."""
import torch

from . import losses


def _entry(dtype):
    from . import ext
    mod = ext.load()
    if dtype is torch.float32:
        return mod.invoke_cpu_fp32
    if dtype is torch.float64:
        return mod.invoke_cpu_fp64
    raise Exception("CPU kernel only supports float32 and float64!")


def _planes(cfg, gates):
    ones = None
    for j, (i, l) in enumerate(zip(cfg.indices_, cfg.locations_)):
        if gates is not None:
            yield gates[j].contiguous(), i.contiguous(), l.contiguous()
        else:
            if ones is None:
                ones = torch.ones(cfg.sample_size, dtype=cfg.dtype)
            yield ones, i.contiguous(), l.contiguous()


def _extra(cfg):
    return [cfg.sample_size, cfg.model_dim, cfg.capacity]


def scatter(cfg, rows, gates):
    """kernel type 0, one call per choice plane into a zeroed [E * capacity, model_dim] tensor."""
    rows = rows.contiguous()
    slots = torch.zeros(cfg.num_global_experts * cfg.capacity, cfg.model_dim, dtype=rows.dtype)
    call = _entry(rows.dtype)
    for g, i, l in _planes(cfg, gates):
        call([g.to(rows.dtype), i, l, rows, slots], _extra(cfg), 0)
    return slots


def gather(cfg, slots, gates):
    """kernel type 1 per choice plane, the planes added left to right."""
    slots = slots.contiguous()
    call = _entry(slots.dtype)
    total = None
    for g, i, l in _planes(cfg, gates):
        rows = torch.empty(cfg.sample_size, cfg.model_dim, dtype=slots.dtype)
        call([g.to(slots.dtype), i, l, rows, slots], _extra(cfg), 1)
        total = rows if total is None else total + rows
    return total


def gate_gradients(cfg, rows, slots):
    """kernel type 2 per choice plane: <slot row, token row>."""
    rows, slots = rows.contiguous(), slots.contiguous()
    call = _entry(rows.dtype)
    out = []
    for i, l in zip(cfg.indices_, cfg.locations_):
        g = torch.empty(cfg.sample_size, dtype=rows.dtype)
        call([g, i.contiguous(), l.contiguous(), rows, slots], _extra(cfg), 2)
        out.append(g)
    return out


def cumsum_sub_one(mask):
    return torch.cumsum(mask, dim=0) - 1


def extract_critical(scores, top_k, loss_fn, capacity_factor, batch_prioritized_routing, normalize_gate, alignment):
    """Routing of host scores with torch ops; same return structure as the GPU route."""
    T, E = int(scores.size(0)), int(scores.size(1))
    top_k = min(top_k, E)
    chosen = torch.topk(scores, top_k, dim=1).indices                      # [T, k]
    l_loss = loss_fn(scores, chosen) if loss_fn is not None else None
    masks = [losses._one_hot_with_dtype(chosen[:, j], num_classes=E, dtype=chosen.dtype) for j in range(top_k)]
    gates_s = [(scores * m).sum(dim=1) for m in masks]
    if batch_prioritized_routing:
        order = (-scores.max(dim=1)[0]).argsort(dim=0)
        back = order.argsort(dim=0)
        place = lambda m: (cumsum_sub_one(m[order]) * m[order])[back]
    else:
        place = cumsum_sub_one
    locations_s, taken = [], torch.zeros(1, E, dtype=chosen.dtype)
    for j, m in enumerate(masks):
        locations_s.append(((place(m) + taken) * m).sum(dim=1).to(torch.int32))
        taken = taken + m.sum(dim=0, keepdim=True)
    if top_k > 1 and normalize_gate:
        denom = torch.clamp(sum(gates_s), min=torch.finfo(gates_s[0].dtype).eps)
        gates_s = [g / denom for g in gates_s]
    indices_s = [chosen[:, j].to(torch.int32) for j in range(top_k)]
    per_expert = (T + E - 1) // E
    if capacity_factor > 0:
        capacity = top_k * int(capacity_factor * per_expert)
    else:
        capacity = int(torch.max(torch.cat(locations_s, dim=0))) + 1
        if capacity_factor < 0:
            capacity = min(capacity, top_k * int(-capacity_factor * per_expert))
    if capacity % alignment:
        capacity += alignment - capacity % alignment
    return (E, indices_s, locations_s, gates_s, capacity), l_loss
