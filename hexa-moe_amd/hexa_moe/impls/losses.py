"""Auxiliary load-balancing losses of the router (reference: hexa_moe_cuda/hexa_moe/impls/losses.py).

Pure PyTorch: they are a few reductions over the [T, E] score matrix and carry the only gradient the
gate receives (the layer output is not weighted by the gate score).
"""
import torch


def gshard_loss(scores_w_noise, top_ids):
    """GShard loss (losses.py:12-19):  sum_e me[e] * ce[e] / T  with
    me[e] = sum_t scores[t, e]  and  ce[e] = (E / T) * #{t : top-1 expert of t is e}."""
    num_samples, num_experts = scores_w_noise.shape
    first_choice = top_ids[:, 0].reshape(-1).to(torch.int64)
    hits = torch.zeros(num_experts, device=scores_w_noise.device, dtype=scores_w_noise.dtype)
    hits.index_add_(0, first_choice, torch.ones_like(first_choice, dtype=scores_w_noise.dtype))
    ce = hits * (num_experts / num_samples)
    me = scores_w_noise.sum(dim=0)
    return (me * ce).sum() / num_samples


def _cv_squared(v):
    v = v.float()
    return v.var() / (v.mean() ** 2 + 1e-10)


def load_importance_loss(scores_wo_noise, topk_logits, num_global_experts, gate_noise):
    """Mean of the squared coefficients of variation of importance and load (losses.py:21-42).

    importance[e] = sum_t scores[t, e];   load[e] = sum_t Phi((scores[t, e] - thr[t]) / sigma) with
    thr[t] the k-th largest noisy logit of token t and sigma = gate_noise / E."""
    if not gate_noise > 0:
        raise AssertionError("`gate_noise` must be > 0 for normalization in load_importance_loss().")
    s = scores_wo_noise.float()
    threshold = topk_logits[:, -1].reshape(-1, 1).float()
    sigma = gate_noise / num_global_experts
    load = torch.special.ndtr((s - threshold) / sigma).sum(dim=0)
    importance = s.sum(dim=0)
    return (_cv_squared(importance) + _cv_squared(load)) / 2.0
