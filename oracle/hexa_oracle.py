"""CPU oracle for HEXA-MoE's expert-specific operators.  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it.  The shipped path (hexa_moe/*) must not.

It restates, in plain PyTorch on the CPU, the algorithm of the reference's hot path:

  routing segment pass  hexa_moe_cuda/hexa_moe/kernels/shared_cuda_core.cu:31-182 (count + prefix)
                        hexa_moe_cuda/hexa_moe/kernels/shared_cuda_core.cu:184-333 (assign)
  ESMM                  hexa_moe_cuda/hexa_moe/kernels/esmm_full.cu:58-246
  ESMM-bwd/ESTMM/ESS    hexa_moe_cuda/hexa_moe/kernels/fused_ops_full.cu:58-433 (as *specified* by the
                        paper's formula table, README.md:15-17; the shipped kernel has launch and
                        indexing defects and is not a numerical reference)
  MoE FFN fwd / bwd     hexa_moe_cuda/hexa_moe/impls/layers.py:99-277, 280-474 (data-centric branch)
  dense FFN             hexa_moe_cuda/hexa_moe/impls/layers.py:25-95
  auxiliary losses      hexa_moe_cuda/hexa_moe/impls/losses.py:12-42
  gate + routing        hexa_moe_cuda/hexa_moe/impls/cascaded_moe.py:515-531,
                        hexa_moe_cuda/hexa_moe/impls/layers.py:476-484

Parity pinning.  The reference ships no tests, golden vectors or fixtures for this path, and its
CUDA extension cannot be built in a ROCm image (nvcc, <mma.h>, and a header the repository does not
contain).  Every function below is therefore pinned by what the mathematics fixes, in
tests/test_oracle_*.py: torch.bincount / stable argsort and brute force for the segment pass;
nn.Linear (E=1), torch.bmm over gathered weights, identity weights and duplicated slots for ESMM;
torch.autograd through an independent dense formulation for ESTMM / ESS / the layer backward;
fp64 gradcheck at tiny sizes.  Not pinned by anything the reference holds: RNG-stream-identical
default initialisation (timm's trunc_normal_ is not installed) -- "parity unpinned" for that item.
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------
# routing segment pass
# --------------------------------------------------------------------------------------------
def token_count(routing_slot: torch.Tensor, num_experts: int, pad: int = 1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Histogram of one routing slot and the exclusive prefix of the counts rounded up to `pad`.

    Follows launch_count (shared_cuda_core.cu:126-182): tokens_per_expert[e] = #{t: routing[t]==e};
    expanded_tokens_per_expert[E+1] = exclusive scan of ceil(count/pad)*pad.  The reference fixes
    pad=16 (BLOCK_SIZE, shared_cuda_core.cu:17,167-169); pad=1 gives the exact, unpadded prefix.
    """
    r = routing_slot.reshape(-1).to(torch.int64)
    counts = torch.zeros(num_experts, dtype=torch.int64)
    for t in range(r.numel()):  # explicit loop = the definition; tests pin it against bincount
        counts[r[t]] += 1
    padded = ((counts + pad - 1) // pad) * pad
    expanded = torch.zeros(num_experts + 1, dtype=torch.int64)
    run = 0
    for e in range(num_experts):
        expanded[e] = run
        run += int(padded[e])
    expanded[num_experts] = run
    return counts.to(torch.int32), expanded.to(torch.int32)


def token_count_fast(routing_slot: torch.Tensor, num_experts: int, pad: int = 1):
    """Vectorised form of token_count for large T (pinned against token_count in the tests)."""
    r = routing_slot.reshape(-1).to(torch.int64)
    counts = torch.bincount(r, minlength=num_experts)
    padded = ((counts + pad - 1) // pad) * pad
    expanded = torch.zeros(num_experts + 1, dtype=torch.int64)
    expanded[1:] = torch.cumsum(padded, 0)
    return counts.to(torch.int32), expanded.to(torch.int32)


def token_assign(routing_slot: torch.Tensor, expanded: torch.Tensor, num_experts: int):
    """Scatter token ids into per-expert segments (launch_assign, shared_cuda_core.cu:284-333).

    token_idx_list[P], expert_idx_list[P] with P = expanded[E]; unused (padding) slots keep -1 as
    the caller pre-fills them (impls/layers.py:238-239).  The reference's order inside a segment
    depends on atomics; this oracle fixes it to ascending token id (a stable counting sort), which
    is one of the orders the reference can produce.
    """
    r = routing_slot.reshape(-1).to(torch.int64)
    P = int(expanded[num_experts])
    tok = torch.full((P,), -1, dtype=torch.int32)
    exp = torch.full((P,), -1, dtype=torch.int32)
    cursor = expanded[:num_experts].to(torch.int64).clone()
    for t in range(r.numel()):
        e = int(r[t])
        pos = int(cursor[e])
        tok[pos] = t
        exp[pos] = e
        cursor[e] += 1
    return tok, exp


def route_build(routing: torch.Tensor, num_experts: int):
    """All slots at once, unpadded: counts[k,E], offsets[k,E+1], token_ids[k,T] (ascending ids
    inside each expert segment).  Vectorised; pinned against token_count/token_assign (pad=1)."""
    assert routing.dim() == 2
    T, k = routing.shape
    counts = torch.zeros(k, num_experts, dtype=torch.int32)
    offsets = torch.zeros(k, num_experts + 1, dtype=torch.int32)
    token_ids = torch.zeros(k, T, dtype=torch.int32)
    for s in range(k):
        r = routing[:, s].to(torch.int64)
        c = torch.bincount(r, minlength=num_experts)
        counts[s] = c.to(torch.int32)
        offsets[s, 1:] = torch.cumsum(c, 0).to(torch.int32)
        token_ids[s] = torch.sort(r, stable=True).indices.to(torch.int32)
    return counts, offsets, token_ids


# --------------------------------------------------------------------------------------------
# the three expert-specific operators (operator-level contracts of the reference extension)
# --------------------------------------------------------------------------------------------
def _rows(token_ids: torch.Tensor, offsets: torch.Tensor, s: int, e: int) -> torch.Tensor:
    return token_ids[s, int(offsets[s, e]):int(offsets[s, e + 1])].to(torch.int64)


def esmm(x: torch.Tensor, W: torch.Tensor, b: Optional[torch.Tensor], token_ids: torch.Tensor,
         offsets: torch.Tensor, m2s: bool, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ESMM: out[(s),t,:] (+)= x[(s),t,:] @ W[e_s(t)] + b[e_s(t)]   (esmm_full.cu:58-246).

    W is [E, in, out]; b is [E, out] or None.
    m2s False: x [T,in] shared by the slots, result [k,T,out] (esmm_full.cu:216-244).
    m2s True : x [k,T,in], result [T,out] summed over the slots (esmm_full.cu:201-214).
    Arithmetic in the dtype of x (use fp32/fp64 inputs for a reference result).
    """
    k, T = token_ids.shape
    E, d_in, d_out = W.shape
    if out is None:
        out = torch.zeros((T, d_out) if m2s else (k, T, d_out), dtype=x.dtype)
    for s in range(k):
        for e in range(E):
            rows = _rows(token_ids, offsets, s, e)
            if rows.numel() == 0:
                continue
            xe = (x[s] if m2s else x).index_select(0, rows)
            ye = xe @ W[e]
            if b is not None:
                ye = ye + b[e]
            if m2s:
                out.index_add_(0, rows, ye)
            else:
                out[s].index_add_(0, rows, ye)
    return out


def estmm(dy: torch.Tensor, x: torch.Tensor, token_ids: torch.Tensor, offsets: torch.Tensor,
          m2s: bool, num_experts: int) -> torch.Tensor:
    """ESTMM: j_w[e] = sum_s sum_{t in seg(s,e)} dy[(s),t,:]^T x[(s),t,:]  -> [E, out, in]
    (fused_ops_full.cu:248-371 as specified; formula-table steps 5 and 9).

    m2s False (fc2 call, impls/layers.py:409-416): dy [T,out] shared, x [k,T,in] per slot.
    m2s True  (fc1 call, impls/layers.py:435-451): dy [k,T,out] per slot, x [T,in] shared.
    """
    k, T = token_ids.shape
    d_out = dy.shape[-1]
    d_in = x.shape[-1]
    jw = torch.zeros(num_experts, d_out, d_in, dtype=x.dtype)
    for s in range(k):
        for e in range(num_experts):
            rows = _rows(token_ids, offsets, s, e)
            if rows.numel() == 0:
                continue
            dye = (dy[s] if m2s else dy).index_select(0, rows)
            xe = (x if m2s else x[s]).index_select(0, rows)
            jw[e] += dye.t() @ xe
    return jw


def ess(dy: torch.Tensor, token_ids: torch.Tensor, offsets: torch.Tensor, m2s: bool,
        num_experts: int) -> torch.Tensor:
    """ESS: j_b[e] = sum_s sum_{t in seg(s,e)} dy[(s),t,:] -> [E, out]
    (fused_ops_full.cu:372-431 as specified; formula-table steps 4 and 8)."""
    k, T = token_ids.shape
    d_out = dy.shape[-1]
    jb = torch.zeros(num_experts, d_out, dtype=dy.dtype)
    for s in range(k):
        for e in range(num_experts):
            rows = _rows(token_ids, offsets, s, e)
            if rows.numel() == 0:
                continue
            jb[e] += (dy[s] if m2s else dy).index_select(0, rows).sum(0)
    return jb


def esmm_bwd(dy: torch.Tensor, w: torch.Tensor, token_ids: torch.Tensor, offsets: torch.Tensor,
             m2s: bool) -> torch.Tensor:
    """Backward ESMM: j_x[(s),t,:in] = dy[(s),t,:out] @ w[e]   with w [E,out,in], no bias
    (fused_ops_full.cu:117-247 as specified; formula-table steps 6 and 10).

    m2s False: dy [T,out] shared, j_x [k,T,in].   m2s True: dy [k,T,out], j_x [T,in] summed over slots.
    """
    # It is an ESMM whose weight is w viewed as [E, in'=out, out'=in] and whose row operand is dy;
    # the slot layout flips: shared input <-> per-slot output.
    return esmm(dy, w, None, token_ids, offsets, m2s=m2s)


def fused_grad(dy, w, x, token_ids, offsets, m2s: bool, with_bias: bool):
    """FUSED_GRAD / FUSED_GRAD_NO_BIAS contract (hexa_moe_ops.cpp:119-275): (j_b, j_x, j_w)."""
    E = w.shape[0]
    jx = esmm_bwd(dy, w, token_ids, offsets, m2s)
    jw = estmm(dy, x, token_ids, offsets, m2s, E)
    jb = ess(dy, token_ids, offsets, m2s, E) if with_bias else None
    return jb, jx, jw


# --------------------------------------------------------------------------------------------
# MoE FFN layer (formula table, steps 1-10) in the reference's parameter layout
# --------------------------------------------------------------------------------------------
def moe_ffn_forward(x, fc1_w, fc2_w, fc1_b, fc2_b, routing, act: Callable):
    """y[t] = sum_s ( act(x[t] W1[e]^T + b1[e]) W2[e] + b2[e] ),  e = routing[t,s]
    fc1_w [E,h,d_in], fc2_w [E,h,d_out], fc1_b [E,h]|None, fc2_b [E,d_out]|None
    (impls/layers.py:253-275; the layer output is NOT weighted by the gate score).
    Returns (y [T,d_out], y1 [k,T,h] pre-activation, y2 [k,T,h])."""
    E = fc1_w.shape[0]
    _, offsets, token_ids = route_build(routing, E)
    y1 = esmm(x, fc1_w.transpose(1, 2), fc1_b, token_ids, offsets, m2s=False)
    y2 = act(y1)
    y = esmm(y2, fc2_w, fc2_b, token_ids, offsets, m2s=True)
    return y, y1, y2


def moe_ffn_backward(dy, x, y1, fc1_w, fc2_w, has_b1: bool, has_b2: bool, routing,
                     act: Callable):
    """Steps 4-10 of the formula table; returns dx, dW1 [E,h,d_in], dW2 [E,h,d_out], db1, db2.
    act' is taken by autograd of act on y1 (elementwise activations only)."""
    E = fc1_w.shape[0]
    _, offsets, token_ids = route_build(routing, E)
    y1g = y1.detach().clone().requires_grad_(True)
    with torch.enable_grad():
        y2 = act(y1g)
    # fc2: j_y = dy [T,d_out] (shared), x-operand = y2 [k,T,h]; w = W2^T as [E,out=d_out,in=h]
    db2, dy2, dW2t = fused_grad(dy, fc2_w.transpose(1, 2), y2.detach(), token_ids, offsets,
                                m2s=False, with_bias=has_b2)
    dW2 = dW2t.transpose(1, 2).contiguous()            # [E,h,d_out]
    (dy1,) = torch.autograd.grad(y2, y1g, dy2)          # dy1 = dy2 * act'(y1)
    # fc1: j_y = dy1 [k,T,h] per slot, x-operand = x [T,d_in] shared; w = W1 as [E,out=h,in=d_in]
    db1, dx, dW1 = fused_grad(dy1, fc1_w, x, token_ids, offsets, m2s=True, with_bias=has_b1)
    return dx, dW1, dW2, db1, db2


def dense_mlp_forward(x, fc1_w, fc2_w, fc1_b, fc2_b, act: Callable):
    """Dense FFN depth (impls/layers.py:36-50): fc1_w [h,d_in], fc2_w [h,d_out]."""
    hid = x @ fc1_w.t()
    if fc1_b is not None:
        hid = hid + fc1_b
    y = act(hid) @ fc2_w
    if fc2_b is not None:
        y = y + fc2_b
    return y


# --------------------------------------------------------------------------------------------
# gate / auxiliary losses
# --------------------------------------------------------------------------------------------
def gshard_loss(scores: torch.Tensor, top_ids: torch.Tensor) -> torch.Tensor:
    """l_aux = sum_e( me[e] * ce[e] ) / T with me = sum_t scores, ce = (E/T)*#{t: top1(t)=e}
    (impls/losses.py:12-19)."""
    T, E = scores.shape
    ce = torch.bincount(top_ids[:, 0].to(torch.int64), minlength=E).to(scores.dtype) * (E / T)
    me = scores.sum(0)
    return (me * ce).sum() / T


def load_importance_loss(scores_wo_noise, topk_logits, num_global_experts, gate_noise):
    """(cv^2(importance) + cv^2(load)) / 2 (impls/losses.py:21-42)."""
    assert gate_noise > 0
    s = scores_wo_noise.float()
    thr = topk_logits[:, -1].reshape(-1, 1).float()
    sigma = gate_noise / num_global_experts
    prob = 0.5 * (1.0 + torch.erf((s - thr) / (sigma * math.sqrt(2.0))))
    load = prob.sum(0)
    l_load = load.var() / (load.mean() ** 2 + 1e-10)
    imp = s.sum(0)
    l_imp = imp.var() / (imp.mean() ** 2 + 1e-10)
    return (l_imp + l_load) / 2.0


def route_top_k(logits: torch.Tensor, top_k: int, noise: Optional[torch.Tensor] = None):
    """scores = softmax(logits (+noise)); indices = topk(scores, k) (cascaded_moe.py:515-531,
    layers.py:476-484).  Returns (scores, indices[T,k] int64)."""
    lw = logits if noise is None else logits + noise
    scores = F.softmax(lw, dim=1)
    idx = torch.topk(scores, min(top_k, scores.shape[1]), dim=1).indices
    return scores, idx


# --------------------------------------------------------------------------------------------
# timed CPU baseline (bench.py's cpu_baseline leg): the same math, vectorised per expert
# --------------------------------------------------------------------------------------------
def moe_layer_fwd_bwd_cpu(x, fc1_w, fc2_w, fc1_b, fc2_b, routing, dy, act=F.gelu):
    """One full MoE-layer forward + backward in fp32 on the host (formula-table steps 1-10)."""
    y, y1, _ = moe_ffn_forward(x, fc1_w, fc2_w, fc1_b, fc2_b, routing, act)
    grads = moe_ffn_backward(dy, x, y1, fc1_w, fc2_w, fc1_b is not None, fc2_b is not None,
                             routing, act)
    return (y,) + tuple(grads)
