"""Fused routing front end: gate projection, softmax, top-k and the auxiliary loss (GShard or
load-importance) as HIP kernels with autograd glue.  It computes what the reference's routing() closure
computes (hexa_moe_cuda/hexa_moe/impls/cascaded_moe.py:515-531 with impls/layers.py:476-484 and
impls/losses.py:12-42); MoE_Cascaded uses it for GPU inputs with the linear gate and keeps the PyTorch
formulation for everything else (cosine gate, more than 8 slots, a single expert).
"""
import torch

from .. import ops


class GateProjection(torch.autograd.Function):
    """logits = x @ wg^T accumulated in fp32 whatever the tokens' type (the fp32 gate of
    gates/top.py:17-19), without materialising an fp32 copy of x."""

    @staticmethod
    def forward(ctx, x, wg):
        ctx.save_for_backward(x, wg)
        return ops.gate_logits(x, wg.float())

    @staticmethod
    def backward(ctx, dlogits):
        x, wg = ctx.saved_tensors
        dx, dwg = ops.gate_backward(dlogits, x, wg.float(), ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        if dwg is not None:
            dwg = dwg.to(wg.dtype)
        return dx, dwg


class RouterTopK(torch.autograd.Function):
    """(idx [T,k] int32, l_aux) = top-k of softmax(logits + scale*noise) and the GShard loss."""

    @staticmethod
    def forward(ctx, logits, noise, noise_scale, top_k):
        scores, idx, _me, ce, l_aux = ops.router_forward(logits, top_k, noise, noise_scale)
        ctx.save_for_backward(scores, ce)
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)    # no zero tensor for the index output's absent gradient
        return idx, l_aux

    @staticmethod
    def backward(ctx, _didx, dl_aux):
        if dl_aux is None:
            return None, None, None, None
        scores, ce = ctx.saved_tensors
        return ops.router_backward(scores, ce, dl_aux), None, None, None


class RouterTopKLoadImportance(torch.autograd.Function):
    """(idx [T,k] int32, l_aux) with the load-importance loss; sigma = gate_noise / E."""

    @staticmethod
    def forward(ctx, logits, noise, noise_scale, sigma, top_k):
        scores, idx, thr, stats = ops.router_forward_load_importance(logits, top_k, sigma, noise, noise_scale)
        ctx.save_for_backward(scores, idx, thr, stats)
        ctx.sigma = sigma
        ctx.mark_non_differentiable(idx)
        ctx.set_materialize_grads(False)
        return idx, stats[-1]

    @staticmethod
    def backward(ctx, _didx, dl_aux):
        if dl_aux is None:
            return None, None, None, None, None
        scores, idx, thr, stats = ctx.saved_tensors
        return ops.router_backward_load_importance(scores, thr, idx, stats, dl_aux, ctx.sigma), None, None, None, None


def fused_route_supported(gate, x, top_k, num_experts, is_gshard_loss):
    from ..gates.top import LinearTopKGate
    if not is_gshard_loss and not (2 <= num_experts <= 1024 and gate.gate_noise > 0):
        return False      # the PyTorch formulation raises the reference's error / yields its NaN
    return (x.is_cuda and isinstance(gate, LinearTopKGate) and 1 <= top_k <= min(8, num_experts)
            and num_experts <= 4096 and x.shape[1] % 8 == 0
            and x.dtype in (torch.float32, torch.float16, torch.bfloat16))


def fused_route(gate, x, top_k, num_experts, noise_scale, training, is_gshard_loss=True):
    """Returns (indices [T,k] int32, l_aux)."""
    w = gate.wg.weight
    if gate.fp32_gate or x.dtype == torch.float32:
        logits = GateProjection.apply(x, w)
    else:   # a gate kept in the tokens' type: the framework's own linear, as in the reference
        logits = gate(x).float()
    noise = None
    if training and noise_scale > 0:
        noise = torch.randn_like(logits)
    if not is_gshard_loss:
        return RouterTopKLoadImportance.apply(logits, noise, float(noise_scale), float(gate.gate_noise) / num_experts,
                                              int(top_k))
    return RouterTopK.apply(logits, noise, float(noise_scale), int(top_k))
