"""Shared helpers of the parity tests."""
import numpy as np
import torch


def bf16_bits(t):
    """torch bf16/fp16 tensor -> uint16 numpy bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bf16_bits(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def raw(t):
    """Bit pattern view of a tensor for exact comparisons."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy()
    return t.numpy()


def np_raw(a):
    if a.dtype == np.float32:
        return a.view(np.int32)
    if a.dtype == np.uint16:
        return a.view(np.int16)
    return a


def to_np(t):
    """torch tensor -> numpy as the oracle wants it (bf16 -> uint16 bits)."""
    if t.dtype == torch.bfloat16:
        return bf16_bits(t)
    return t.detach().cpu().numpy()


def tie_free_scores(T, E, k, seed, dtype=torch.float32, bias=None, scale=1.0):
    """Seeded softmax scores whose top-(k+1) entries are distinct in every row."""
    g = torch.Generator().manual_seed(seed)
    for _ in range(200):
        logits = torch.randn(T, E, generator=g) * scale
        if bias is not None:
            logits = logits + bias
        scores = torch.softmax(logits, dim=1).to(dtype)
        kk = min(k + 1, E)
        top = torch.topk(scores.float(), kk, dim=1).values
        if bool((top[:, :-1] > top[:, 1:]).all()):
            return scores
    raise RuntimeError("no tie-free draw (low-precision scores tie almost surely)")


def random_scores(T, E, seed, dtype=torch.float32):
    """Seeded softmax scores; rows may contain equal entries."""
    g = torch.Generator().manual_seed(seed)
    return torch.softmax(torch.randn(T, E, generator=g), dim=1).to(dtype)


def zipf_bias(E, s=1.2):
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -s
    return torch.log(p / p.sum()).float()
