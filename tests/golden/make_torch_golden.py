"""Writes tests/golden/torch_golden.npz: small input/output vectors for routing, the
dispatch/combine kernels and the int8 codec, produced with torch-CPU *library routines*
(topk, scatter_, cumsum, index ops, elementwise ops in the tensor dtype) arranged in the
order the reference's host code applies them.  The reference package itself cannot be
imported (it needs its CUDA extension), so nothing from it is executed or read here.

    python tests/golden/make_torch_golden.py
"""
import os

import numpy as np
import torch


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def tie_free(scores, k):
    """True when the top-(k+1) scores of every row are pairwise distinct."""
    kk = min(k + 1, scores.size(1))
    top = torch.topk(scores.float(), kk, dim=1).values
    return bool((top[:, :-1] > top[:, 1:]).all())


def routing_case(T, E, k, dtype, seed, normalize=True, bias=None):
    g = torch.Generator().manual_seed(seed)
    while True:
        logits = torch.randn(T, E, generator=g)
        if bias is not None:
            logits = logits + bias
        scores = torch.softmax(logits, dim=1).to(dtype)
        if tie_free(scores, k):
            break
    k = min(k, E)
    topk_indices = torch.topk(scores, k, dim=1).indices
    indices_s = [x.view(-1) for x in topk_indices.chunk(k, dim=1)]
    masks = []
    for x in indices_s:
        m = torch.zeros(T, E, dtype=torch.int64)
        m.scatter_(1, x.unsqueeze(-1), 1)
        masks.append(m)
    gates_s = [(scores * m).sum(dim=1) for m in masks]
    loc = torch.cumsum(masks[0], dim=0) - 1
    locations_s = [torch.sum(loc * masks[0], dim=1).to(torch.int32)]
    acc = None
    for j in range(1, k):
        s = torch.sum(masks[j - 1], dim=0, keepdim=True)
        acc = s if acc is None else acc + s
        loc = torch.cumsum(masks[j], dim=0) - 1 + acc
        locations_s.append(torch.sum(loc * masks[j], dim=1).to(torch.int32))
    if k > 1 and normalize:
        denom = torch.clamp(sum(gates_s), min=torch.finfo(gates_s[0].dtype).eps)
        gates_s = [x / denom for x in gates_s]
    # GShard loss
    mask0 = torch.zeros(T, E, dtype=scores.dtype)
    mask0.scatter_(1, topk_indices[:, :1], E / T)
    l_aux = torch.sum(torch.sum(scores, dim=0) * torch.sum(mask0, dim=0)) / T
    conv = bits if dtype == torch.bfloat16 else (lambda t: t.numpy().copy())
    return dict(scores=conv(scores), indices=torch.stack(indices_s).to(torch.int32).numpy(),
                locations=torch.stack(locations_s).numpy(), gates=conv(torch.stack(gates_s)),
                counts=torch.stack([m.sum(0) for m in masks]).to(torch.int32).numpy(),
                l_aux=np.array([float(l_aux)], np.float64))


def sparse_case(T, M, E, k, C, seed):
    g = torch.Generator().manual_seed(seed)
    scores = torch.softmax(torch.randn(T, E, generator=g), dim=1)
    top = torch.topk(scores, k, dim=1)
    idx = top.indices.t().contiguous().to(torch.int32)
    gates = top.values.t().contiguous()
    loc = torch.empty_like(idx)
    seen = torch.zeros(E, dtype=torch.int64)
    for j in range(k):
        for t in range(T):
            e = int(idx[j, t]); loc[j, t] = int(seen[e]); seen[e] += 1
    x = torch.randn(T, M, generator=g)
    eo = torch.randn(E * C, M, generator=g)
    keep = loc < C
    slot = (idx.long() * C + loc.long())
    disp = torch.zeros(E * C, M)
    for j in range(k):
        disp.index_put_((slot[j][keep[j]],), gates[j][keep[j], None] * x[keep[j]], accumulate=True)
    comb = torch.zeros(T, M)
    for j in range(k):
        term = torch.zeros(T, M)
        term[keep[j]] = gates[j][keep[j], None] * eo[slot[j][keep[j]]]
        comb = term if j == 0 else comb + term
    gg = torch.zeros(k, T, dtype=torch.float64)
    for j in range(k):
        gg[j][keep[j]] = (eo[slot[j][keep[j]]].double() * x[keep[j]].double()).sum(1)
    return dict(x=x.numpy(), eo=eo.numpy(), idx=idx.numpy(), loc=loc.numpy(), gates=gates.numpy(),
                C=np.array([C]), E=np.array([E]), dispatched=disp.numpy(), combined=comb.numpy(),
                grad_gates=gg.numpy())


def int8_case(R, M, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(R, M, generator=g) * torch.rand(R, 1, generator=g) * 4).to(dtype)
    x[0] = 0                       # empty capacity slot: 0/0
    x[1] = 1.5                     # constant row
    x[2, 0] = 1e4                  # outlier
    x[3] = x[3].abs()
    bias = torch.min(x, -1, True)[0]
    scale = torch.max(x, -1, True)[0]
    scale = torch.sub(scale, bias)
    out = torch.sub(x, bias)
    out = torch.div(out, scale)
    out = torch.mul(out, 255.0)
    codes = out.to(torch.uint8)
    dec = codes.to(dtype)
    dec = torch.div(dec, 255.0)
    dec = torch.mul(dec, scale)
    dec = torch.add(dec, bias)
    conv = bits if dtype == torch.bfloat16 else (lambda t: t.numpy().copy())
    return dict(x=conv(x), codes=codes.numpy(), bias=conv(bias), scale=conv(scale), decoded=conv(dec))


def main():
    data = {}
    cases = {
        "route_t2_e2": routing_case(64, 2, 2, torch.float32, 1),
        "route_t2_e8": routing_case(300, 8, 2, torch.float32, 2),
        "route_t1_e64": routing_case(257, 64, 1, torch.float32, 3,
                                     bias=torch.log(torch.arange(1, 65).float() ** -1.2)),
        "route_t3_e16_nonorm": routing_case(100, 16, 3, torch.float32, 4, normalize=False),
        "route_bf16_t2_e4": routing_case(40, 4, 2, torch.bfloat16, 5),
        "sparse_a": sparse_case(50, 24, 4, 2, 20, 6),
        "sparse_b": sparse_case(33, 40, 8, 1, 4, 7),
        "int8_f32": int8_case(12, 96, torch.float32, 8),
        "int8_bf16": int8_case(12, 128, torch.bfloat16, 9),
    }
    for name, d in cases.items():
        for k, v in d.items():
            data[name + "." + k] = v
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "torch_golden.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes; torch", torch.__version__)


if __name__ == "__main__":
    main()
