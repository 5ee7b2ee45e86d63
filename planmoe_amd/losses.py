"""Auxiliary losses -- mirror of the reference's impls/losses.py.

gshard_loss is normally produced by the routing kernel itself (extract_critical recognises
this function and takes the kernel's value); the torch expressions below are kept so that the
functions stay callable on their own, as in the reference."""
import torch
from torch.distributions.normal import Normal


def _one_hot_with_dtype(data, num_classes, dtype, hot_value=1):
    # losses.py:7-10
    result = torch.zeros([data.size(0), num_classes], device=data.device, dtype=dtype)
    result.scatter_(1, data.unsqueeze(-1), hot_value)
    return result


def gshard_loss(scores_w_noise, top_ids):
    # losses.py:12-19
    num_samples, num_global_experts = int(scores_w_noise.size(0)), int(scores_w_noise.size(1))
    mask = _one_hot_with_dtype(top_ids[:, 0], num_global_experts, dtype=scores_w_noise.dtype,
                               hot_value=num_global_experts / num_samples)
    me = torch.sum(scores_w_noise, dim=0)
    ce = torch.sum(mask, dim=0)
    return torch.sum(me * ce) / num_samples


def load_importance_loss(scores_wo_noise, topk_logits, num_global_experts, gate_noise):
    # losses.py:21-42
    def cv2(v):
        v = v.float()
        return v.var() / (v.mean() ** 2 + 1e-10)

    normal = Normal(torch.tensor([0.0], device=scores_wo_noise.device),
                    torch.tensor([gate_noise / num_global_experts], device=scores_wo_noise.device))
    threshold = topk_logits[:, -1].view(-1, 1).float()
    load = normal.cdf(scores_wo_noise.float() - threshold).sum(0)
    importance = scores_wo_noise.float().sum(0)
    return (cv2(importance) + cv2(load)) / 2.0
