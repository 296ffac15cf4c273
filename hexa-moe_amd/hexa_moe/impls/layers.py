"""Autograd functions of the cascaded MoE (reference: hexa_moe_cuda/hexa_moe/impls/layers.py).

FusedMoE_Shared_CudaCore is the MoE FFN of one depth in data-centric mode on one GPU: the ten steps
of the paper's formula table, each an expert-specific operator of libhexa_moe_hip.so:

    forward   1  y1 = ESMM(x, W1, b1)            3  y = ESMM(act(y1), W2, b2), summed over the slots
    backward  4  db2 = ESS(dy)                    5  dW2 = ESTMM(act(y1), dy)     6  dy2 = ESMM(dy, W2^T)
              7  dy1 = dy2 * act'(y1)             8  db1 = ESS(dy1)               9  dW1 = ESTMM(dy1, x)
              10 dx = ESMM(dy1, W1^T), summed over the slots

Against the reference (layers.py:99-277, 280-474) on the same math:
  * weights are read in their parameter layout ([E,h,d_in], [E,h,d_out]); nothing is concatenated,
    permuted or copied per call (layers.py:119-122, 307-309, 412, 438 copy every expert weight);
  * results are written in their final type; no fp32 staging buffers, zero-fills or cast kernels
    (layers.py:230-231, 260, 275);
  * the routing lists are built once per depth on the device, without .item() (layers.py:238), and the
    same metadata serves all six matmuls, both ESS calls and the backward;
  * gradients are returned for the Parameters that were passed in (the reference passes `.data`, so
    its expert gradients are dropped: cascaded_moe.py:553-559);
  * the activation is evaluated once: the backward differentiates the forward's own graph (or the
    fused GELU), not a second evaluation (layers.py:281-283, 407), so stochastic activations
    (dropout) use one mask.
"""
from typing import Any

import torch
import torch.nn.functional as F

from .. import _lib, ops
from . import losses


def is_plain_gelu(fn) -> bool:
    """True for activations known to be the exact (erf) GELU, which the kernels fuse."""
    return fn is F.gelu or getattr(fn, "hexa_fused", None) == "gelu"


def fused_gelu(x):
    """Marker activation: pass `activation_fn=fused_gelu` to get the fused GELU epilogue."""
    return F.gelu(x)


fused_gelu.hexa_fused = "gelu"


class MLP_Implement:
    """Dense FFN depth (reference: layers.py:25-95): y = act(x fc1_w^T + b1) fc2_w + b2 with
    fc1_w [h, d_in], fc2_w [h, d_out].  Plain differentiable PyTorch (rocBLAS GEMMs); on one GPU the
    reference's gradient all-reduces are the identity."""

    @staticmethod
    def apply(config: Any, tokens_input, fc1_w, fc2_w, fc1_bias, fc2_bias):
        dt = tokens_input.dtype
        hid = F.linear(tokens_input, fc1_w.to(dt), fc1_bias.to(dt) if fc1_bias is not None else None)
        out = config.activation_fn(hid) @ fc2_w.to(dt)
        if fc2_bias is not None:
            out = out + fc2_bias.to(dt)
        return out


def _weight_for(x, w, rows):
    """Kernels take weights in the tokens' 16-bit type or in fp32.  fp32 master weights under 16-bit
    tokens (autocast) are rounded to the tokens' type by the kernel as it stages them; from a few dozen
    routed rows per expert on it is cheaper to round them once here -- same values, and the forward and
    backward kernels then read half the bytes and take the fast path (measured at 72 rows per expert,
    768 -> 3072, 32 experts: forward + backward ESMM 218 + 188 us on fp32 weights, 72 + 60 us on the
    rounded copy, whose making moves 450 MB once)."""
    if w.dtype == x.dtype:
        return w
    if w.dtype == torch.float32 and x.dtype != torch.float32 and rows < 32 * w.shape[0]:
        return w
    return w.to(x.dtype)


class FusedMoE_Shared_CudaCore(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, config: Any, tokens_input, fc1_w, fc2_w, fc1_bias, fc2_bias):
        x = tokens_input.contiguous()
        if not x.is_cuda:
            raise RuntimeError("hexa_moe: the MoE FFN runs on the GPU only (no CPU fallback); move the module "
                               "and its input to a HIP device")
        E = int(config.num_global_experts)
        T, d_in = x.shape
        assert fc1_w.shape[0] == E and fc2_w.shape[0] == E and fc1_w.shape[2] == d_in
        assert fc1_w.shape[1] == fc2_w.shape[1]

        indices = getattr(config, "routing_", None)   # [T,k] tensor; else the reference's list of k vectors
        if indices is None:
            indices = config.indices_
        routing = indices if torch.is_tensor(indices) else torch.stack([i.reshape(-1) for i in indices], dim=1)
        blob = config.route_pool.slot(config.stage, T, routing.shape[1], E, x.device)
        route = ops.route_build(routing, E, blob=blob)
        if any(ctx.needs_input_grad):
            config.route_pool.bind(config.stage, route)  # keep the slot until this call's backward is done

        w1, w2 = _weight_for(x, fc1_w, T * routing.shape[1]), _weight_for(x, fc2_w, T * routing.shape[1])
        act = config.activation_fn
        fused = is_plain_gelu(act)
        ctx.act_graph = None
        if fused:
            y1, y2 = ops.esmm(x, w1, fc1_bias, route, False, _lib.HEXA_W_OUT_IN, gelu=True)
        else:
            y1 = ops.esmm(x, w1, fc1_bias, route, False, _lib.HEXA_W_OUT_IN)
            if any(ctx.needs_input_grad):
                with torch.enable_grad():
                    y1_leaf = y1.detach().requires_grad_(True)
                    y2_graph = act(y1_leaf)
                ctx.act_graph = (y1_leaf, y2_graph)
                y2 = y2_graph.detach()
            else:
                y2 = act(y1)
            if y2.dtype != x.dtype:
                y2 = y2.to(x.dtype)
        y = ops.esmm(y2.contiguous(), w2, fc2_bias, route, True, _lib.HEXA_W_IN_OUT)

        ctx.config = config
        ctx.route = route
        ctx.fused = fused
        ctx.has_b1, ctx.has_b2 = fc1_bias is not None, fc2_bias is not None
        ctx.param_dtypes = (fc1_w.dtype, fc2_w.dtype,
                            fc1_bias.dtype if fc1_bias is not None else None,
                            fc2_bias.dtype if fc2_bias is not None else None)
        ctx.save_for_backward(x, y1, y2 if fused else None, w1, w2)
        return y

    @staticmethod
    def backward(ctx: Any, j_tokens_output):
        x, y1, y2, w1, w2 = ctx.saved_tensors
        route = ctx.route
        dy = j_tokens_output.contiguous().to(x.dtype)
        need_x, need_w1, need_w2, need_b1, need_b2 = ctx.needs_input_grad[1:6]
        dt_w1, dt_w2, dt_b1, dt_b2 = ctx.param_dtypes
        if not ctx.fused:
            y1_leaf, y2_graph = ctx.act_graph
            y2 = y2_graph.detach().to(x.dtype).contiguous()

        def grad_dtype(param_dtype):  # fp32 master weights get fp32 grads, 16-bit weights 16-bit grads
            return torch.float32 if param_dtype == torch.float32 else x.dtype

        db2 = dw2 = db1 = dw1 = dx = None
        if ctx.has_b2 and need_b2:
            db2 = ops.ess(dy, route, False, out_dtype=grad_dtype(dt_b2)).to(dt_b2)
        if need_w2:
            # [E, h, d_out]: the per-slot operand act(y1) supplies the rows of dW2
            dw2 = ops.estmm(y2, dy, route, True, False, out_dtype=grad_dtype(dt_w2)).to(dt_w2)
        if need_x or need_w1 or (ctx.has_b1 and need_b1):
            bias1_done = False
            if ctx.fused and ctx.has_b1 and need_b1:
                # dy1 = (dy . W2^T) * gelu'(y1) and db1 = its per-expert row sums, from the same kernel
                dy1, db1 = ops.esmm_gelu_bwd_ess(dy, w2, route, _lib.HEXA_W_OUT_IN, y1, db_dtype=grad_dtype(dt_b1))
                db1 = db1.to(dt_b1)
                bias1_done = True
            elif ctx.fused:   # dy1 = (dy . W2^T) * gelu'(y1) in the ESMM epilogue
                dy1 = ops.esmm(dy, w2, None, route, False, _lib.HEXA_W_OUT_IN, gelu_bwd_of=y1)
            else:
                dy2 = ops.esmm(dy, w2, None, route, False, _lib.HEXA_W_OUT_IN)
                (dy1,) = torch.autograd.grad(y2_graph, y1_leaf, dy2.to(y2_graph.dtype))
                dy1 = dy1.to(x.dtype).contiguous()
            if ctx.has_b1 and need_b1 and not bias1_done:
                db1 = ops.ess(dy1, route, True, out_dtype=grad_dtype(dt_b1)).to(dt_b1)
            if need_w1:
                dw1 = ops.estmm(dy1, x, route, True, False, out_dtype=grad_dtype(dt_w1)).to(dt_w1)
            if need_x:
                dx = ops.esmm(dy1, w1, None, route, True, _lib.HEXA_W_IN_OUT)
        ctx.act_graph = None
        ctx.config.stage = ctx.config.stage - 1
        return (None, dx, dw1, dw2, db1, db2)


class _BlobOwner:
    """Keeps a route-pool slot bound while a backward that reads it is pending."""

    def __init__(self, blob):
        self.blob = blob


class FusedMoEDepth(torch.autograd.Function):
    """One MoE depth -- gate projection, softmax + top-k + auxiliary loss, the routing segment pass and the
    MoE FFN with the exact GELU -- as TWO library calls (hexa_moe_depth_forward / _backward) instead of one
    call per operator: the same kernels in the same order as the linear gate's routing followed by
    FusedMoE_Shared_CudaCore (reference: impls/cascaded_moe.py:508-568 and impls/layers.py:99-474), with the
    gate path's share of dx added inside the expert path's slot sum.  Returns (y, l_aux)."""

    events = None   # optional {"fwd": [torch.cuda.Event, ...], "bwd": [...]} recorded around the major kernels

    @staticmethod
    def forward(ctx: Any, config: Any, opts: Any, tokens_input, wg, fc1_w, fc2_w, fc1_bias, fc2_bias):
        top_k, noise_scale, is_gshard, sigma = opts
        x = tokens_input.contiguous()
        E = int(config.num_global_experts)
        T, d_in = x.shape
        hidden, d_out = fc1_w.shape[1], fc2_w.shape[2]
        assert fc1_w.shape == (E, hidden, d_in) and fc2_w.shape[:2] == (E, hidden) and wg.shape == (E, d_in)
        w1, w2 = _weight_for(x, fc1_w, T * top_k), _weight_for(x, fc2_w, T * top_k)
        if w1.dtype != w2.dtype:
            w1, w2 = w1.to(x.dtype), w2.to(x.dtype)
        w1, w2, wg32 = w1.contiguous(), w2.contiguous(), wg.float().contiguous()
        b1 = fc1_bias.contiguous() if fc1_bias is not None else None
        b2 = fc2_bias.contiguous() if fc2_bias is not None else None

        def grad_dtype(p):   # fp32 master parameters get fp32 gradients, 16-bit parameters 16-bit ones
            return None if p is None else (torch.float32 if p.dtype == torch.float32 else x.dtype)

        key = (T, top_k, E, d_in, hidden, d_out, x.dtype, w1.dtype, None if b1 is None else b1.dtype,
               None if b2 is None else b2.dtype, fc1_w.dtype, fc2_w.dtype, is_gshard, float(noise_scale), float(sigma))
        plans = config.__dict__.setdefault("depth_plans", {})
        plan = plans.get(key)
        if plan is None:
            plan = plans[key] = ops.DepthPlan(T, top_k, E, d_in, hidden, d_out, x.dtype, w1.dtype,
                                              None if b1 is None else b1.dtype, None if b2 is None else b2.dtype,
                                              grad_dtype(fc1_w), grad_dtype(fc2_w), grad_dtype(fc1_bias) or torch.float32,
                                              grad_dtype(fc2_bias) or torch.float32, 0 if is_gshard else 1,
                                              noise_scale, sigma)
        dev = x.device
        nstats = (2 if is_gshard else 4) * E + 1
        state = torch.empty(2 * T * E + T + nstats, dtype=torch.float32, device=dev)
        logits, scores = state[:T * E], state[T * E:2 * T * E]
        thr, stats = state[2 * T * E:2 * T * E + T], state[2 * T * E + T:]
        ints = torch.empty(T * top_k + _lib.estmm_plan_ints(E), dtype=torch.int32, device=dev)
        idx, estmm_plan = ints[:T * top_k].view(T, top_k), ints[T * top_k:]   # the backward's ESTMM work plan
        noise = torch.randn(T, E, dtype=torch.float32, device=dev) if noise_scale > 0 else None
        blob = config.route_pool.slot(config.stage, T, top_k, E, dev)
        y12 = torch.empty(2, top_k, T, hidden, dtype=x.dtype, device=dev)
        y = torch.empty(T, d_out, dtype=x.dtype, device=dev)
        ws = torch.empty(plan.fwd_bytes, dtype=torch.uint8, device=dev)
        ev = FusedMoEDepth.events
        ops.moe_depth_forward(plan, x, wg32, noise, w1, b1, w2, b2, logits, scores, idx, None if is_gshard else thr, stats,
                              blob, estmm_plan, y12[0], y12[1], y, ws, ev["fwd"] if ev else None)
        config.routing_ = idx
        if any(ctx.needs_input_grad):
            ctx.owner = _BlobOwner(blob)
            config.route_pool.bind(config.stage, ctx.owner)   # keep the slot until this call's backward is done
        ctx.config, ctx.plan, ctx.is_gshard = config, plan, is_gshard
        ctx.param_dtypes = (wg.dtype, fc1_w.dtype, fc2_w.dtype, None if fc1_bias is None else fc1_bias.dtype,
                            None if fc2_bias is None else fc2_bias.dtype)
        ctx.dims = (T, top_k, E, d_in, hidden, d_out)
        ctx.save_for_backward(x, wg32, w1, w2, state, ints, y12, blob)
        ctx.set_materialize_grads(False)
        return y, stats[nstats - 1]

    @staticmethod
    def backward(ctx: Any, dy, dl_aux):
        x, wg32, w1, w2, state, ints, y12, blob = ctx.saved_tensors
        T, top_k, E, d_in, hidden, d_out = ctx.dims
        idx, estmm_plan = ints[:T * top_k].view(T, top_k), ints[T * top_k:]
        dev = x.device
        need_x, need_wg, need_w1, need_w2, need_b1, need_b2 = ctx.needs_input_grad[2:8]
        dt_wg, dt_w1, dt_w2, dt_b1, dt_b2 = ctx.param_dtypes
        dy = torch.zeros(T, d_out, dtype=x.dtype, device=dev) if dy is None else dy.contiguous().to(x.dtype)
        g_aux = None if dl_aux is None else dl_aux.to(torch.float32).contiguous()

        def grad_dtype(p):
            return torch.float32 if p == torch.float32 else x.dtype

        def new(shape, dtype, want):
            return torch.empty(shape, dtype=dtype, device=dev) if want else None

        dx = new((T, d_in), x.dtype, need_x)
        dwg = new((E, d_in), torch.float32, need_wg and g_aux is not None)
        dw1 = new((E, hidden, d_in), grad_dtype(dt_w1), need_w1)
        dw2 = new((E, hidden, d_out), grad_dtype(dt_w2), need_w2)
        db1 = new((E, hidden), grad_dtype(dt_b1), dt_b1 is not None and need_b1)
        db2 = new((E, d_out), grad_dtype(dt_b2), dt_b2 is not None and need_b2)
        dy1 = torch.empty(top_k, T, hidden, dtype=x.dtype, device=dev)
        ws = torch.empty(ctx.plan.bwd_bytes, dtype=torch.uint8, device=dev)
        nstats = (2 if ctx.is_gshard else 4) * E + 1
        scores = state[T * E:2 * T * E]
        thr, stats = state[2 * T * E:2 * T * E + T], state[2 * T * E + T:2 * T * E + T + nstats]
        ev = FusedMoEDepth.events
        ops.moe_depth_backward(ctx.plan, dy, g_aux, x, wg32, w1, w2, scores, idx, None if ctx.is_gshard else thr, stats,
                               blob, estmm_plan, y12[0], y12[1], dx, dwg, dw1, db1, dw2, db2, dy1, ws, ev["bwd"] if ev else None)
        ctx.owner = None
        ctx.config.stage = ctx.config.stage - 1

        def cast(g, dt):
            return None if g is None else g.to(dt)

        return (None, None, dx, cast(dwg, dt_wg), cast(dw1, dt_w1), cast(dw2, dt_w2), cast(db1, dt_b1), cast(db2, dt_b2))


def topk_and_loss(scores, top_k, loss_fn=losses.gshard_loss):
    """Top-k expert choice as one [T,k] int64 tensor (what the routing pass reads directly) and the
    auxiliary loss."""
    top_k = min(int(top_k), int(scores.size(1)))
    topk_indices = torch.topk(scores, top_k, dim=1).indices
    l_loss = loss_fn(scores, topk_indices) if loss_fn is not None else None
    return topk_indices, l_loss


def simplified_extract_critical(scores, top_k, loss_fn=losses.gshard_loss):
    """Same contract as the reference's helper (layers.py:476-484): the k index vectors and the loss."""
    topk_indices, l_loss = topk_and_loss(scores, top_k, loss_fn)
    return [col.reshape(-1) for col in topk_indices.unbind(dim=1)], l_loss
