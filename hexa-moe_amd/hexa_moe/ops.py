"""Tensor-level wrappers of the C ABI: device memory and streams come from PyTorch, everything else
happens in libhexa_moe_hip.so.  All tensors must live on a HIP device; CPU tensors are rejected."""
import torch

from . import _lib

_DT = {torch.float32: _lib.HEXA_F32, torch.float16: _lib.HEXA_F16, torch.bfloat16: _lib.HEXA_BF16}


def _dt(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"hexa_moe: unsupported element type {t.dtype}")


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("hexa_moe: expert-specific operators run on the GPU only; got a CPU tensor "
                               "(there is no CPU fallback)")


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


class OpTimer:
    """Optional per-call device timing: while installed (set_timer), operator calls are bracketed by two
    events on the stream they launch on -- every call, or only those whose label is in `only` (an event
    pair costs about 4 us of stream time, which adds up over the ~25 calls of a layer step).
    durations() waits for the device."""

    def __init__(self, only=None):
        self.records = []
        self.only = None if only is None else frozenset(only)

    def durations(self):
        torch.cuda.synchronize()
        out = {}
        for label, a, b in self.records:
            out.setdefault(label, []).append(a.elapsed_time(b))  # ms
        return out


_timer = None


def set_timer(timer):
    global _timer
    _timer = timer


def _call(label, fn, *args):
    if _timer is None or (_timer.only is not None and label not in _timer.only):
        return fn(*args)
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    rc = fn(*args)
    b.record()
    _timer.records.append((label, a, b))
    return rc


class Route:
    """Routing metadata of one MoE depth: a view of a caller-owned int32 blob (see
    hexa_route_layout in include/hexa_moe_hip.h)."""

    def __init__(self, blob, T, k, E):
        self.blob, self.T, self.k, self.E = blob, int(T), int(k), int(E)
        self.layout = _lib.route_layout(T, k, E)
        self._plans = {}

    def estmm_plan(self, max_slots, out_dim=0, in_dim=0):
        """Work plan of estmm for this routing and result size (int32 [HEXA_ESTMM_PLAN_INTS]); made on first use,
        then shared by every estmm call on the routing whose result has as many 128 x 128 blocks.  The plan also
        holds the work queue of the persistent kernel, so calls that use it must not overlap (one stream)."""
        key = (int(max_slots), -(-int(out_dim) // 128) * -(-int(in_dim) // 128))
        plan = self._plans.get(key)
        if plan is None:
            plan = torch.empty(_lib.estmm_plan_ints(self.E), dtype=torch.int32, device=self.blob.device)
            rc = _call("estmm_plan", _lib.load().hexa_estmm_plan, _ptr(plan), _ptr(self.blob), self.T, self.k, self.E,
                       int(max_slots), int(out_dim), int(in_dim), _stream())
            _lib.check(rc, "hexa_estmm_plan")
            self._plans[key] = plan
        return plan

    def _part(self, start, n):
        return self.blob[start:start + n]

    @property
    def counts(self):
        return self._part(self.layout.counts, self.k * self.E).view(self.k, self.E)

    @property
    def offsets(self):
        return self._part(self.layout.offsets, self.k * (self.E + 1)).view(self.k, self.E + 1)

    @property
    def token_ids(self):
        return self._part(self.layout.token_ids, self.k * self.T).view(self.k, self.T)

    @property
    def expert_ids(self):
        return self._part(self.layout.expert_ids, self.k * self.T).view(self.k, self.T)

    @property
    def tile_count(self):
        return self._part(self.layout.tile_count, self.k)

    @property
    def tile_info(self):
        return self._part(self.layout.tile_info, self.k * self.layout.mt_ub * 4).view(self.k, self.layout.mt_ub, 4)

    @property
    def tile_count_l(self):
        return self._part(self.layout.tile_count_l, self.k)

    @property
    def tile_info_l(self):
        return self._part(self.layout.tile_info_l, self.k * self.layout.mt_ub_l * 4).view(self.k, self.layout.mt_ub_l, 4)


class RouteWorkspace:
    """One int32 device buffer reused by every MoE depth of a model (the depth-shared cache of
    routing metadata).  It grows to the largest (T, k, E) seen and is never shrunk."""

    def __init__(self):
        self.buf = None

    def get(self, T, k, E, device):
        need = _lib.route_layout(T, k, E).total_ints
        if self.buf is None or self.buf.numel() < need or self.buf.device != device:
            self.buf = torch.empty(max(int(need), 4), dtype=torch.int32, device=device)
        return self.buf


def route_blob_ints(T, k, E):
    return int(_lib.route_layout(T, k, E).total_ints)


def route_build(routing, num_experts, blob=None):
    """routing: [T, k] (or [T]) int32/int64 expert choices on the GPU -> Route."""
    _dev(routing)
    if routing.dim() == 1:
        routing = routing.unsqueeze(1)
    if routing.dtype not in (torch.int32, torch.int64):
        raise TypeError("hexa_moe: routing must be int32 or int64")
    T, k = routing.shape
    if blob is None:
        blob = torch.empty(max(route_blob_ints(T, k, num_experts), 4), dtype=torch.int32, device=routing.device)
    rc = _call("route_build", _lib.load().hexa_route_build, _ptr(routing), int(routing.dtype == torch.int64),
               routing.stride(0), routing.stride(1), T, k, num_experts, _ptr(blob), _stream())
    _lib.check(rc, "hexa_route_build")
    return Route(blob, T, k, num_experts)


def route_from_lists(token_idx_list, expert_idx_list, T, k, num_experts, blob=None):
    _dev(token_idx_list, expert_idx_list)
    if blob is None:
        blob = torch.empty(max(route_blob_ints(T, k, num_experts), 4), dtype=torch.int32, device=token_idx_list.device)
    rc = _lib.load().hexa_route_from_lists(_ptr(token_idx_list), _ptr(expert_idx_list), T, k, num_experts,
                                           _ptr(blob), _stream())
    _lib.check(rc, "hexa_route_from_lists")
    return Route(blob, T, k, num_experts)


def route_from_padded_lists(token_idx_list, expert_idx_list, slot_ends, T, k, num_experts, blob=None):
    """Route from the reference's concatenated, 16-padded lists; slot_ends is its device tensor of
    k+1 cumulative list lengths (cum_ids of impls/layers.py:245-248)."""
    _dev(token_idx_list, expert_idx_list, slot_ends)
    if slot_ends.dtype != torch.int32 or slot_ends.numel() < k + 1 or not slot_ends.is_contiguous():
        raise TypeError("slot_ends must be a contiguous int32 tensor of top_k + 1 entries")
    if blob is None:
        blob = torch.empty(max(route_blob_ints(T, k, num_experts), 4), dtype=torch.int32, device=token_idx_list.device)
    rc = _lib.load().hexa_route_from_padded_lists(_ptr(token_idx_list), _ptr(expert_idx_list), _ptr(slot_ends),
                                                  int(token_idx_list.numel()), T, k, num_experts, _ptr(blob), _stream())
    _lib.check(rc, "hexa_route_from_padded_lists")
    return Route(blob, T, k, num_experts)


def esmm(x, w, bias, route, m2s, w_layout, out=None, out_dtype=None, accumulate=False, gelu=False, gelu_bwd_of=None):
    """out[(s),t] (+)= x[(s),t] @ W[e] + bias[e].  Returns out, or (out, gelu(out)) when gelu=True.
    gelu_bwd_of=y1 multiplies the result by gelu'(y1) (y1 of out's shape and dtype)."""
    _dev(x, w, bias, out)
    T, k, E = route.T, route.k, route.E
    x = x.contiguous()
    w = w.contiguous()
    if w_layout == _lib.HEXA_W_IN_OUT:
        in_dim, out_dim = w.shape[1], w.shape[2]
    else:
        out_dim, in_dim = w.shape[1], w.shape[2]
    assert w.shape[0] == E and x.shape[-1] == in_dim
    assert tuple(x.shape) == ((k, T, in_dim) if m2s else (T, in_dim)), (x.shape, m2s, k, T, in_dim)
    if out is None:
        assert not accumulate
        out_dtype = out_dtype or x.dtype
        out = torch.empty((T, out_dim) if m2s else (k, T, out_dim), dtype=out_dtype, device=x.device)
    assert out.is_contiguous() and tuple(out.shape) == ((T, out_dim) if m2s else (k, T, out_dim))
    out_act = torch.empty_like(out) if gelu else None
    act = _lib.HEXA_ACT_GELU if gelu else _lib.HEXA_ACT_NONE
    if gelu_bwd_of is not None:
        assert not gelu and not m2s and not accumulate
        out_act = gelu_bwd_of.contiguous()
        assert out_act.shape == out.shape and out_act.dtype == out.dtype
        act = _lib.HEXA_ACT_GELU_BWD
    # scratch for summing the slots in one launch (see hexa_esmm in include/hexa_moe_hip.h)
    slot_ws = torch.empty((k - 1, T, out_dim), dtype=out.dtype, device=out.device) if (m2s and k > 1) else None
    if bias is not None:
        bias = bias.contiguous()
    label = f"esmm[{in_dim}->{out_dim},{'w_in_out' if w_layout == _lib.HEXA_W_IN_OUT else 'w_out_in'}" \
            f"{',sum_slots' if m2s else ''}{',gelu' if gelu else ''}{',gelu_bwd' if gelu_bwd_of is not None else ''}]"
    rc = _call(label, _lib.load().hexa_esmm, _ptr(out), _ptr(x), _ptr(w), _ptr(bias), _ptr(route.blob),
               int(bool(m2s)), int(w_layout), int(bool(accumulate)), T, k, in_dim, out_dim, E, _dt(x), _dt(w),
               _dt(bias) if bias is not None else 0, _dt(out),
               act, _ptr(out_act), _ptr(slot_ws), _stream())
    _lib.check(rc, "hexa_esmm")
    return (out, out_act) if gelu else out


def estmm(dy, x, route, dy_per_slot, x_per_slot, out=None, out_dtype=torch.float32, accumulate=False):
    """dw[e][o][i] (+)= sum over routed (slot, token) of dy[.., o] * x[.., i]  -> [E, out, in]."""
    _dev(dy, x, out)
    T, k, E = route.T, route.k, route.E
    dy = dy.contiguous()
    x = x.contiguous()
    assert dy.dtype == x.dtype
    out_dim, in_dim = dy.shape[-1], x.shape[-1]
    assert tuple(dy.shape) == ((k, T, out_dim) if dy_per_slot else (T, out_dim))
    assert tuple(x.shape) == ((k, T, in_dim) if x_per_slot else (T, in_dim))
    if out is None:
        assert not accumulate
        out = torch.empty(E, out_dim, in_dim, dtype=out_dtype, device=x.device)
    plan = scratch = None
    slots = 0
    if x.dtype != torch.float32:
        # a plan (made once per routing and result size) orders the work of the persistent kernel; with lists long
        # enough to be worth cutting it comes with scratch for up to 2E fp32 partial results, at most 256 MiB
        if T * k >= 128 * E and (out_dim * in_dim) % 4 == 0:
            slots = min(2 * E, (256 << 20) // (out_dim * in_dim * 4))
            slots = slots if slots >= 2 else 0
        plan = route.estmm_plan(slots, out_dim, in_dim)
        if slots:
            scratch = torch.empty(slots * out_dim * in_dim, dtype=torch.float32, device=x.device)
    rc = _call(f"estmm[{out_dim}x{in_dim}]", _lib.load().hexa_estmm, _ptr(out), _ptr(dy), _ptr(x), _ptr(route.blob),
               int(bool(dy_per_slot)), int(bool(x_per_slot)), int(bool(accumulate)), T, k, out_dim, in_dim, E,
               _dt(x), _dt(out), _ptr(plan), slots, _ptr(scratch), _stream())
    _lib.check(rc, "hexa_estmm")
    return out


def ess(dy, route, dy_per_slot, out=None, out_dtype=torch.float32, accumulate=False):
    """db[e][o] (+)= sum over routed (slot, token) of dy[.., o] -> [E, out]."""
    _dev(dy, out)
    T, k, E = route.T, route.k, route.E
    dy = dy.contiguous()
    out_dim = dy.shape[-1]
    assert tuple(dy.shape) == ((k, T, out_dim) if dy_per_slot else (T, out_dim))
    if out is None:
        assert not accumulate
        out = torch.empty(E, out_dim, dtype=out_dtype, device=dy.device)
    ws = None
    if T * k >= 256 * E:   # long token lists: scratch for the partial sums of up to 8 parts per list
        ws = torch.empty(8 * E * out_dim, dtype=torch.float32, device=dy.device)
    rc = _call(f"ess[{out_dim}{',per_slot' if dy_per_slot else ''}]", _lib.load().hexa_ess, _ptr(out), _ptr(dy),
               _ptr(route.blob), int(bool(dy_per_slot)), int(bool(accumulate)), T, k, out_dim, E, _dt(dy), _dt(out),
               _ptr(ws), 0 if ws is None else ws.numel(), _stream())
    _lib.check(rc, "hexa_ess")
    return out


def esmm_gelu_bwd_ess(x, w, route, w_layout, y1, db_dtype=torch.float32):
    """dy1 [k,T,out] = (x . w[e]) * gelu'(y1) and db [E,out] = per-expert row sums of dy1, in one call (the
    sums ride on the producing kernel's store loop on the 16-bit fast path)."""
    import ctypes
    _dev(x, w, y1)
    x, w, y1 = x.contiguous(), w.contiguous(), y1.contiguous()
    T, k, E = route.T, route.k, route.E
    in_dim = x.shape[-1]
    out_dim = w.shape[2] if w_layout == _lib.HEXA_W_IN_OUT else w.shape[1]
    assert tuple(x.shape) == (T, in_dim) and tuple(y1.shape) == (k, T, out_dim) and y1.dtype == x.dtype
    out = torch.empty(k, T, out_dim, dtype=x.dtype, device=x.device)
    db = torch.empty(E, out_dim, dtype=db_dtype, device=x.device)
    n = ctypes.c_int64()
    _lib.check(_lib.load().hexa_esmm_ess_ws_floats(T, k, out_dim, E, ctypes.byref(n)), "hexa_esmm_ess_ws_floats")
    ws = torch.empty(int(n.value), dtype=torch.float32, device=x.device)
    lay = "w_in_out" if w_layout == _lib.HEXA_W_IN_OUT else "w_out_in"
    rc = _call(f"esmm[{in_dim}->{out_dim},{lay},gelu_bwd+ess]", _lib.load().hexa_esmm_gelu_bwd_ess, _ptr(out), _ptr(db),
               _ptr(x), _ptr(w), _ptr(y1), _ptr(route.blob), int(w_layout), 0, T, k, in_dim, out_dim, E, _dt(x), _dt(w),
               _dt(db), _ptr(ws), int(ws.numel()), _stream())
    _lib.check(rc, "hexa_esmm_gelu_bwd_ess")
    return out, db


def gelu_bwd(dy2, y1):
    """dy1 = dy2 * gelu'(y1) (erf form)."""
    _dev(dy2, y1)
    dy2 = dy2.contiguous()
    y1 = y1.contiguous()
    assert dy2.shape == y1.shape and dy2.dtype == y1.dtype
    out = torch.empty_like(dy2)
    rc = _call("gelu_bwd", _lib.load().hexa_gelu_bwd, _ptr(out), _ptr(dy2), _ptr(y1), dy2.numel(), _dt(dy2),
               _stream())
    _lib.check(rc, "hexa_gelu_bwd")
    return out


def gate_logits(x, wg):
    """logits[t][e] = sum_d x[t][d] * wg[e][d] with fp32 accumulation; wg fp32 [E, d] -> fp32 [T, E]."""
    _dev(x, wg)
    x = x.contiguous()
    wg = wg.contiguous()
    assert wg.dtype == torch.float32 and x.dim() == 2 and wg.shape[1] == x.shape[1]
    T, d = x.shape
    E = wg.shape[0]
    logits = torch.empty(T, E, dtype=torch.float32, device=x.device)
    rc = _call("gate_logits", _lib.load().hexa_gate_logits, _ptr(logits), _ptr(x), _ptr(wg), T, d, E, _dt(x), _stream())
    _lib.check(rc, "hexa_gate_logits")
    return logits


def gate_backward(dlogits, x, wg, need_dx=True, need_dwg=True):
    """Backward of gate_logits: (dx [T, d] in x's type or None, dwg [E, d] fp32 or None)."""
    import ctypes
    _dev(dlogits, x, wg)
    dlogits = dlogits.contiguous()
    x = x.contiguous()
    wg = wg.contiguous()
    assert dlogits.dtype == torch.float32 and wg.dtype == torch.float32
    T, d = x.shape
    E = wg.shape[0]
    assert dlogits.shape == (T, E) and wg.shape == (E, d)
    dx = torch.empty_like(x) if need_dx else None
    dwg = ws = None
    if need_dwg:
        n = ctypes.c_int64()
        _lib.check(_lib.load().hexa_gate_ws_floats(T, d, E, ctypes.byref(n)), "hexa_gate_ws_floats")
        ws = torch.empty(int(n.value), dtype=torch.float32, device=x.device)
        dwg = torch.empty(E, d, dtype=torch.float32, device=x.device)
    rc = _call("gate_backward", _lib.load().hexa_gate_backward, _ptr(dx), _ptr(dwg), _ptr(dlogits), _ptr(x), _ptr(wg),
               T, d, E, _dt(x), _ptr(ws), _stream())
    _lib.check(rc, "hexa_gate_backward")
    return dx, dwg


def router_forward(logits, top_k, noise=None, noise_scale=0.0):
    """softmax + top-k + GShard loss.  Returns scores [T,E] fp32, idx [T,k] int32, me [E], ce [E], l_aux []."""
    import ctypes
    _dev(logits, noise)
    logits = logits.contiguous()
    assert logits.dtype == torch.float32 and logits.dim() == 2
    T, E = logits.shape
    dev = logits.device
    n = ctypes.c_int64()
    _lib.check(_lib.load().hexa_router_ws_floats(T, E, ctypes.byref(n)), "hexa_router_ws_floats")
    ws = torch.empty(int(n.value), dtype=torch.float32, device=dev)
    scores = torch.empty(T, E, dtype=torch.float32, device=dev)
    idx = torch.empty(T, top_k, dtype=torch.int32, device=dev)
    stats = torch.empty(2 * E + 1, dtype=torch.float32, device=dev)   # me, ce, l_aux
    me, ce, l_aux = stats[:E], stats[E:2 * E], stats[2 * E]
    if noise is not None:
        noise = noise.contiguous()
        assert noise.dtype == torch.float32 and noise.shape == logits.shape
    rc = _call("router_forward", _lib.load().hexa_router_forward, _ptr(scores), _ptr(idx), _ptr(me), _ptr(ce),
               l_aux.data_ptr(), _ptr(logits), _ptr(noise), float(noise_scale), T, E, int(top_k), _ptr(ws), _stream())
    _lib.check(rc, "hexa_router_forward")
    return scores, idx, me, ce, l_aux


def router_backward(scores, ce, grad_l_aux):
    """d l_aux / d logits scaled by grad_l_aux (a 0-dim fp32 device tensor)."""
    _dev(scores, ce, grad_l_aux)
    T, E = scores.shape
    g = grad_l_aux.to(torch.float32).contiguous()
    dlogits = torch.empty_like(scores)
    rc = _call("router_backward", _lib.load().hexa_router_backward, _ptr(dlogits), _ptr(scores), _ptr(ce), _ptr(g), T, E,
               _stream())
    _lib.check(rc, "hexa_router_backward")
    return dlogits


def router_forward_load_importance(logits, top_k, sigma, noise=None, noise_scale=0.0):
    """softmax + top-k + load-importance loss.  Returns scores (noise-free softmax) [T,E] fp32, idx [T,k]
    int32, thr [T], stats [4E+1] = importance, load, d l_aux/d importance, d l_aux/d load, l_aux."""
    import ctypes
    _dev(logits, noise)
    logits = logits.contiguous()
    assert logits.dtype == torch.float32 and logits.dim() == 2
    T, E = logits.shape
    dev = logits.device
    n = ctypes.c_int64()
    _lib.check(_lib.load().hexa_router_ws_floats(T, E, ctypes.byref(n)), "hexa_router_ws_floats")
    ws = torch.empty(int(n.value), dtype=torch.float32, device=dev)
    scores = torch.empty(T, E, dtype=torch.float32, device=dev)
    idx = torch.empty(T, top_k, dtype=torch.int32, device=dev)
    thr = torch.empty(T, dtype=torch.float32, device=dev)
    stats = torch.empty(4 * E + 1, dtype=torch.float32, device=dev)
    part = [stats[i * E:(i + 1) * E] for i in range(4)]
    if noise is not None:
        noise = noise.contiguous()
        assert noise.dtype == torch.float32 and noise.shape == logits.shape
    rc = _call("router_forward", _lib.load().hexa_router_forward_load_importance, _ptr(scores), _ptr(idx), _ptr(thr),
               _ptr(part[0]), _ptr(part[1]), _ptr(part[2]), _ptr(part[3]), stats[4 * E].data_ptr(), _ptr(logits),
               _ptr(noise), float(noise_scale), float(sigma), T, E, int(top_k), _ptr(ws), _stream())
    _lib.check(rc, "hexa_router_forward_load_importance")
    return scores, idx, thr, stats


def router_backward_load_importance(scores, thr, idx, stats, grad_l_aux, sigma):
    T, E = scores.shape
    grad_l_aux = grad_l_aux.to(torch.float32).contiguous()
    dlogits = torch.empty_like(scores)
    rc = _call("router_backward", _lib.load().hexa_router_backward_load_importance, _ptr(dlogits), _ptr(scores),
               _ptr(thr), _ptr(idx), _ptr(stats[2 * E:3 * E]), _ptr(stats[3 * E:4 * E]), _ptr(grad_l_aux), float(sigma),
               T, E, int(idx.shape[1]), _stream())
    _lib.check(rc, "hexa_router_backward_load_importance")
    return dlogits


# ---- one MoE depth per call ---------------------------------------------------------------------------------
class DepthPlan:
    """Descriptor and workspace sizes of hexa_moe_depth_forward / _backward for one (shape, dtypes, loss)."""

    def __init__(self, T, k, E, d_in, hidden, d_out, act_dtype, w_dtype, b1_dtype, b2_dtype, gw1, gw2, gb1, gb2,
                 loss, noise_scale, sigma):
        import ctypes
        dt = lambda t: _DT[t] if t is not None else 0   # noqa: E731
        self.desc = _lib.DepthDesc(int(T), int(k), int(E), int(d_in), int(hidden), int(d_out), dt(act_dtype), dt(w_dtype),
                                   dt(b1_dtype), dt(b2_dtype), dt(gw1), dt(gw2), dt(gb1), dt(gb2), int(loss),
                                   float(noise_scale), float(sigma), 0)
        f, b = ctypes.c_int64(), ctypes.c_int64()
        _lib.check(_lib.load().hexa_moe_depth_ws_bytes(ctypes.byref(self.desc), ctypes.byref(f), ctypes.byref(b)),
                   "hexa_moe_depth_ws_bytes")
        self.fwd_bytes, self.bwd_bytes = int(f.value), int(b.value)


def _event_array(events):
    """ctypes array of hipEvent_t handles from torch.cuda.Event objects (each recorded once before, so that
    its handle exists; None entries are skipped by the library), or (None, 0)."""
    import ctypes
    if not events:
        return None, 0
    arr = (ctypes.c_void_p * len(events))(*[None if e is None else e.cuda_event for e in events])
    return arr, len(events)


def moe_depth_forward(plan, x, wg, noise, fc1_w, fc1_b, fc2_w, fc2_b, logits, scores, idx, thr, stats, route_blob,
                      estmm_plan, y1, y2, y, ws, events=None):
    """estmm_plan: int32 [_lib.estmm_plan_ints(E)] that receives the work plan of the backward's ESTMM calls, or None."""
    import ctypes
    _dev(x, wg, noise, fc1_w, fc1_b, fc2_w, fc2_b, idx, route_blob, y1, y2, y, ws)
    ev, nev = _event_array(events)
    rc = _lib.load().hexa_moe_depth_forward(ctypes.byref(plan.desc), _ptr(x), _ptr(wg), _ptr(noise), _ptr(fc1_w),
                                            _ptr(fc1_b), _ptr(fc2_w), _ptr(fc2_b), _ptr(logits), _ptr(scores), _ptr(idx),
                                            _ptr(thr), _ptr(stats), _ptr(route_blob), _ptr(estmm_plan), _ptr(y1), _ptr(y2), _ptr(y),
                                            _ptr(ws), ws.numel() * ws.element_size(), ev, nev, _stream())
    _lib.check(rc, "hexa_moe_depth_forward")


def moe_depth_backward(plan, dy, grad_l_aux, x, wg, fc1_w, fc2_w, scores, idx, thr, stats, route_blob, estmm_plan, y1, y2,
                       dx, dwg, dw1, db1, dw2, db2, dy1, ws, events=None):
    """estmm_plan: the buffer moe_depth_forward filled for this routing, or None (the call then makes the plan)."""
    import ctypes
    _dev(dy, grad_l_aux, x, wg, fc1_w, fc2_w, route_blob, y1, y2, dx, dwg, dw1, db1, dw2, db2, dy1, ws)
    ev, nev = _event_array(events)
    rc = _lib.load().hexa_moe_depth_backward(ctypes.byref(plan.desc), _ptr(dy), _ptr(grad_l_aux), _ptr(x), _ptr(wg),
                                             _ptr(fc1_w), _ptr(fc2_w), _ptr(scores), _ptr(idx), _ptr(thr), _ptr(stats),
                                             _ptr(route_blob), _ptr(estmm_plan), _ptr(y1), _ptr(y2), _ptr(dx), _ptr(dwg), _ptr(dw1),
                                             _ptr(db1), _ptr(dw2), _ptr(db2), _ptr(dy1), _ptr(ws),
                                             ws.numel() * ws.element_size(), ev, nev, _stream())
    _lib.check(rc, "hexa_moe_depth_backward")
