"""MoE_Cascaded on the GPU vs the CPU oracle: forward, input gradient and every parameter gradient.

The module runs the HIP operators through the C ABI; the oracle evaluates the formula table on the
CPU in fp32/fp64 from the same parameters and the module's own routing decision (the top-k indices
are produced by the same torch ops on both sides, so they are compared bit-exactly)."""
import pytest
import torch
import torch.nn.functional as F

from _util import TOL, assert_close
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu


def _module(dims, moe_idx, E, k, bias=True, act=None, dtype=torch.float32, seed=1234, noise=1.0):
    from hexa_moe import moe as hmoe
    torch.manual_seed(seed)
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': k, 'gate_noise': noise, 'fp32_gate': True},
                          model_dim_list=dims, moe_idx_list=moe_idx, mlp_ratio=4, num_global_experts=E,
                          total_depth=len(dims), data_centric=True, mlp_fc1_bias=bias, mlp_fc2_bias=bias,
                          activation_fn=act if act is not None else (lambda x: F.gelu(x)))
    g = torch.Generator().manual_seed(seed)
    for name, p in m.named_parameters():          # U(+-1/sqrt(fan_in)) from the seed
        fan_in = p.shape[-1] if name.startswith(("batched_fc1_w", "mlp_fc1_w", "gates")) else p.shape[-2] if p.dim() > 1 else p.shape[-1]
        p.data.copy_((torch.rand(p.shape, generator=g) * 2 - 1) / fan_in ** 0.5)
    return m


def _oracle_depth(m, i, x, routing, dy, act, rd):
    W1, W2 = m.batched_fc1_w[i].detach().cpu().to(rd), m.batched_fc2_w[i].detach().cpu().to(rd)
    b1 = m.batched_fc1_bias[i].detach().cpu().to(rd) if m.has_fc1_bias else None
    b2 = m.batched_fc2_bias[i].detach().cpu().to(rd) if m.has_fc2_bias else None
    y, y1, _ = O.moe_ffn_forward(x.to(rd), W1, W2, b1, b2, routing, act)
    grads = O.moe_ffn_backward(dy.to(rd), x.to(rd), y1, W1, W2, b1 is not None, b2 is not None, routing, act)
    return y, grads


def test_readme_config_fp32(dev):
    """Tiny MoE_Cascaded as in the reference's README: dims 128 x4, MoE at depths 2 and 3, 8 experts,
    top-1, gate noise 1.0, fp32, 2048 tokens, loss = sum(y) + l_aux, train mode."""
    m = _module([128] * 4, [2, 3], E=8, k=1).to(dev).train()
    g = torch.Generator().manual_seed(1234)
    x0 = torch.randn(2048, 128, generator=g)
    x = x0.to(dev).requires_grad_(True)
    h = x
    captured = []
    dense = []
    aux = 0
    for depth in range(4):
        h_in = h
        h, l_aux = m(depth, h)
        if depth in (0, 1):
            assert l_aux == 0            # a dense depth has no auxiliary loss (cascaded_moe.py:506)
            dense.append((depth, h_in, h))
            h.retain_grad(); h_in.retain_grad()
        if depth in (2, 3):
            captured.append((depth, h_in, m.dispatch_params.routing_.clone(), h))
            h.retain_grad(); h_in.retain_grad()
            aux = aux + l_aux
    (h.sum() + aux).backward()
    torch.cuda.synchronize()
    for depth, h_in, routing, h_out in captured:
        i = m.moe_idx_list.index(depth)
        r = routing.cpu()
        # counts the device built are the bincount of the routing decision, bit for bit
        y_ref, (dx, dW1, dW2, db1, db2) = _oracle_depth(m, i, h_in.detach().cpu(), r, h_out.grad.cpu(), F.gelu, torch.float64)
        assert_close(h_out.detach(), y_ref, 1e-5, f"y depth {depth}")
        assert_close(m.batched_fc1_w[i].grad, dW1, 1e-5, "dW1")
        assert_close(m.batched_fc2_w[i].grad, dW2, 1e-5, "dW2")
        assert_close(m.batched_fc1_bias[i].grad, db1, 1e-5, "db1")
        assert_close(m.batched_fc2_bias[i].grad, db2, 1e-5, "db2")
        if depth == 3:   # h_in.grad of depth 3 is purely the layer's dx (+ the gate's aux-loss path)
            gate_free = h_in.grad.detach().cpu().double() - dx
            assert gate_free.abs().max() < 1e-2   # what is left is the small l_aux gradient through the gate
    # the dense depths (MLP_Implement) against the oracle's dense FFN, differentiated by autograd in fp64
    for depth, h_in, h_out in dense:
        i = [d_ for d_ in range(4) if d_ not in (2, 3)].index(depth)
        prm = [m.mlp_fc1_w[i], m.mlp_fc2_w[i], m.mlp_fc1_b[i], m.mlp_fc2_b[i]]
        ref_p = [q.detach().cpu().double().requires_grad_(True) for q in prm]
        xin = h_in.detach().cpu().double().requires_grad_(True)
        y_ref = O.dense_mlp_forward(xin, ref_p[0], ref_p[1], ref_p[2], ref_p[3], F.gelu)
        y_ref.backward(h_out.grad.cpu().double())
        assert_close(h_out.detach(), y_ref.detach(), 1e-5, f"dense y depth {depth}")
        assert_close(h_in.grad, xin.grad, 1e-5, f"dense dx depth {depth}")
        for q, r, name in zip(prm, ref_p, ["fc1_w", "fc2_w", "fc1_bias", "fc2_bias"]):
            assert_close(q.grad, r.grad, 1e-5, f"dense {name} depth {depth}")
    assert x.grad is not None and m.gates[0].wg.weight.grad is not None


@pytest.mark.parametrize("dtype,k,bias", [(torch.float32, 2, True), (torch.bfloat16, 1, True), (torch.bfloat16, 2, False),
                                          (torch.float16, 2, True)])
@pytest.mark.parametrize("act", [F.gelu, None], ids=["fused_gelu", "generic_activation"])
def test_single_depth_against_oracle(dev, dtype, k, bias, act):
    E, d, T = 16, 256, 3000
    m = _module([d], [0], E=E, k=k, bias=bias, noise=0.0, act=act).to(dev).to(dtype).eval()
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, d, generator=g).to(dtype)
    dy = torch.randn(T, d, generator=g).to(dtype)
    xd = x.to(dev).requires_grad_(True)
    y, l_aux = m(0, xd)
    routing = m.dispatch_params.routing_.cpu()
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    assert y.dtype == dtype and l_aux.dim() == 0
    # the device's per-expert counts equal the bincount of the decision
    rd = torch.float64 if dtype == torch.float32 else torch.float32
    y_ref, (dx, dW1, dW2, db1, db2) = _oracle_depth(m, 0, x, routing, dy, F.gelu, rd)
    tol = TOL[dtype]
    assert_close(y, y_ref, tol, "y")
    assert_close(xd.grad, dx, tol, "dx")
    assert_close(m.batched_fc1_w[0].grad, dW1, tol, "dW1")
    assert_close(m.batched_fc2_w[0].grad, dW2, tol, "dW2")
    if bias:
        assert_close(m.batched_fc1_bias[0].grad, db1, tol, "db1")
        assert_close(m.batched_fc2_bias[0].grad, db2, tol, "db2")
    assert m.batched_fc1_w[0].grad.dtype == dtype


def test_fused_gelu_equals_generic_activation_path(dev):
    """F.gelu itself is recognised and fused; a lambda goes through autograd of the callable."""
    E, d, T = 8, 128, 1500
    a = _module([d], [0], E=E, k=2, act=F.gelu, noise=0.0).to(dev).eval()
    b = _module([d], [0], E=E, k=2, act=lambda t: F.gelu(t), noise=0.0).to(dev).eval()
    b.load_state_dict(a.state_dict())
    x = torch.randn(T, d, device=dev)
    outs = []
    for m in (a, b):
        xi = x.clone().requires_grad_(True)
        y, _ = m(0, xi)
        y.square().sum().backward()
        outs.append((y.detach(), xi.grad, m.batched_fc1_w[0].grad, m.batched_fc2_bias[0].grad))
    torch.cuda.synchronize()
    for u, v in zip(*outs):
        assert_close(u, v, 2e-5, "fused vs generic")


def test_stochastic_activation_uses_one_mask(dev):
    """dropout(gelu(x)) as in the Swin model: the backward must see the forward's mask, so the layer's
    gradients equal those of the oracle evaluated with that same mask."""
    E, d, T = 4, 128, 1024
    masks = []

    def act(t):
        y = F.gelu(t)
        mk = (torch.rand_like(y) > 0.3).to(y.dtype) / 0.7
        masks.append(mk)
        return y * mk

    m = _module([d], [0], E=E, k=1, act=act, noise=0.0).to(dev).train()
    x = torch.randn(T, d, device=dev, requires_grad=True)
    y, _ = m(0, x)
    dy = torch.randn_like(y)
    y.backward(dy)
    torch.cuda.synchronize()
    assert len(masks) == 1, "the activation must be evaluated exactly once per forward+backward"
    mk = masks[0].cpu().double()
    routing = m.dispatch_params.routing_.cpu()
    y_ref, (dx, dW1, dW2, db1, db2) = _oracle_depth(m, 0, x.detach().cpu(), routing, dy.cpu(), lambda t: F.gelu(t) * mk, torch.float64)
    assert_close(y.detach(), y_ref, 1e-5, "y")
    assert_close(x.grad, dx, 1e-5, "dx")
    assert_close(m.batched_fc1_w[0].grad, dW1, 1e-5, "dW1")


def test_autocast_bf16_with_fp32_master_weights(dev):
    E, d, T = 8, 256, 2000
    m = _module([d, d], [1], E=E, k=2, noise=0.0).to(dev).eval()
    x = torch.randn(T, d, device=dev, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        h, _ = m(0, x)
        y, _ = m(1, h)
    assert y.dtype == torch.float32 or y.dtype == x.dtype
    dy = torch.randn_like(y)
    h.retain_grad()
    y.backward(dy)
    torch.cuda.synchronize()
    routing = m.dispatch_params.routing_.cpu()
    hb = h.detach().to(torch.bfloat16).float().cpu()
    W1 = m.batched_fc1_w[0].detach().to(torch.bfloat16).float().cpu()
    W2 = m.batched_fc2_w[0].detach().to(torch.bfloat16).float().cpu()
    b1, b2 = m.batched_fc1_bias[0].detach().cpu(), m.batched_fc2_bias[0].detach().cpu()
    y_ref, y1, _ = O.moe_ffn_forward(hb, W1, W2, b1, b2, routing, F.gelu)
    dx, dW1, dW2, db1, db2 = O.moe_ffn_backward(dy.to(torch.bfloat16).float().cpu(), hb, y1, W1, W2, True, True, routing, F.gelu)
    assert_close(y.detach().float(), y_ref, 2e-2, "y")
    assert m.batched_fc1_w[0].grad.dtype == torch.float32
    assert_close(m.batched_fc1_w[0].grad, dW1, 2e-2, "dW1")
    assert_close(m.batched_fc2_w[0].grad, dW2, 2e-2, "dW2")
    assert_close(m.batched_fc2_bias[0].grad, db2, 2e-2, "db2")


def test_route_pool_is_reused_across_steps_and_survives_pending_backward(dev):
    E, d, T = 8, 128, 512
    m = _module([d, d], [0, 1], E=E, k=1, noise=0.0).to(dev).eval()
    pool = m.dispatch_params.route_pool
    x = torch.randn(T, d, device=dev, requires_grad=True)
    y, _ = m(0, x)
    first = pool._slots[0][0]
    y.sum().backward()
    del y
    y, _ = m(0, x)
    assert pool._slots[0][0] is first, "a slot whose backward is done is reused, not reallocated"
    y2, _ = m(0, x)   # the first call's backward is still pending: its metadata must not be overwritten
    assert pool._slots[0][0] is not first
    (y.sum() + y2.sum()).backward()
    torch.cuda.synchronize()
    with torch.no_grad():
        m(1, x)
        before = pool._slots[1][0]
        m(1, x)
        assert pool._slots[1][0] is before


@pytest.mark.parametrize("loss", ["gshard", "load_importance"])
def test_nan_token_row_stays_routed_and_propagates(dev, loss):
    """A token whose features are NaN gets NaN gate logits.  torch.topk ranks NaN largest and still returns
    valid expert ids, so the reference routes the token, its output row is NaN and the auxiliary loss is NaN
    (which is what an AMP scaler looks for).  The fused router must not drop the token or leave its rows
    unwritten: valid ids, NaN in y and dx for that token only, NaN l_aux."""
    E, d, T, k = 8, 128, 700, 2
    m = _module([d], [0], E=E, k=k, act=F.gelu, noise=1.0).to(dev).train()
    m.is_gshard_loss = loss == "gshard"
    x = torch.randn(T, d, generator=torch.Generator().manual_seed(3))
    bad = 123
    x[bad] = float("nan")
    xd = x.to(dev).requires_grad_(True)
    y, l_aux = m(0, xd)
    idx = m.dispatch_params.routing_
    idx = idx if torch.is_tensor(idx) else torch.stack(list(idx), 1)
    y.sum().backward()
    torch.cuda.synchronize()
    assert int(idx.min()) >= 0 and int(idx.max()) < E
    assert torch.isnan(y[bad]).all() and torch.isnan(xd.grad[bad]).all()
    keep = torch.ones(T, dtype=torch.bool)
    keep[bad] = False
    assert torch.isfinite(y[keep.to(dev)]).all() and torch.isfinite(xd.grad[keep.to(dev)]).all()
    assert torch.isnan(l_aux)


@pytest.mark.parametrize("loss", ["gshard", "load_importance"])
@pytest.mark.parametrize("dtype,k,bias", [(torch.float32, 1, True), (torch.bfloat16, 2, True), (torch.float16, 2, False),
                                          (torch.bfloat16, 1, True)])
@pytest.mark.parametrize("batch", [0, 1, 2, "side"])
def test_depth_call_equals_operator_by_operator(dev, dtype, k, bias, loss, batch):
    """hexa_moe_depth_forward / _backward (one library call per direction) run the same kernels in the same
    order as the per-operator path: same routing, identical y, l_aux and parameter gradients; dx differs only
    by where the gate path's share is added (inside the slot sum instead of a separate addition)."""
    from hexa_moe import _lib
    E, d, T = 16, 256, 2500
    # batch 2: every small kernel of the backward in a launch of its own instead of the three batch launches; 1: four;
    # "side": the batches and the gate's backward on the library's second stream, beside the matmul kernels
    side = batch == "side"
    batch = 0 if side else batch
    _lib.check(_lib.load().hexa_set_option(b"batch", batch), "hexa_set_option")
    _lib.check(_lib.load().hexa_set_option(b"side_stream", 1 if side else 2), "hexa_set_option")
    m = _module([d], [0], E=E, k=k, bias=bias, act=F.gelu, noise=1.0).to(dev).to(dtype).eval()
    m.gates[0].wg.weight.data = m.gates[0].wg.weight.data.float()
    m.is_gshard_loss = loss == "gshard"
    g = torch.Generator().manual_seed(17)
    x = torch.randn(T, d, generator=g).to(dtype).to(dev)
    dy = torch.randn(T, d, generator=g).to(dtype).to(dev)
    res = []
    for fused_depth in (True, False):
        m.fused_depth = fused_depth
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        y, l_aux = m(0, xi)
        torch.autograd.backward([y, l_aux], [dy, torch.full((), 3.0, device=dev)])
        torch.cuda.synchronize()
        assert len(m.dispatch_params.indices_) == k and m.dispatch_params.indices_[0].dtype == torch.int32
        grads = [p.grad.clone() for p in (m.gates[0].wg.weight, m.batched_fc1_w[0], m.batched_fc2_w[0])]
        if bias:
            grads += [m.batched_fc1_bias[0].grad.clone(), m.batched_fc2_bias[0].grad.clone()]
        res.append((m.dispatch_params.routing_.clone().long(), y.detach().clone(), l_aux.detach().clone(), xi.grad.clone(), grads))
    _lib.check(_lib.load().hexa_set_option(b"batch", 0), "hexa_set_option")
    _lib.check(_lib.load().hexa_set_option(b"side_stream", 0), "hexa_set_option")
    (ra, ya, la, dxa, ga), (rb, yb, lb, dxb, gb) = res
    assert torch.equal(ra, rb) and torch.equal(ya, yb) and torch.equal(la, lb)
    for u, v in zip(ga, gb):
        assert torch.equal(u, v)
    assert_close(dxa, dxb, 1e-6 if dtype == torch.float32 else 1e-2, "dx")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,d,E,k,bias", [(2500, 256, 16, 2, True), (2300, 384, 8, 1, True), (1900, 128, 5, 3, False),
                                          (130, 512, 4, 2, True), (64, 128, 3, 1, True)])
def test_one_kernel_ffn_forward(dev, dtype, T, d, E, k, bias):
    """The depth call with fc1, GELU and fc2 in one kernel (library option "ffn_fused"): y against the oracle from
    the module's own routing, and y, dx and every parameter gradient (which go through the y1 / y2 the kernel
    saved) against the two-launch form."""
    from hexa_moe import _lib
    lib = _lib.load()
    m = _module([d], [0], E=E, k=k, bias=bias, act=F.gelu, noise=1.0).to(dev).to(dtype).eval()
    m.gates[0].wg.weight.data = m.gates[0].wg.weight.data.float()
    g = torch.Generator().manual_seed(23)
    x = torch.randn(T, d, generator=g).to(dtype).to(dev)
    dy = torch.randn(T, d, generator=g).to(dtype).to(dev)
    res = []
    try:
        for fused in (1, 0):
            _lib.check(lib.hexa_set_option(b"ffn_fused", fused), "hexa_set_option")
            m.zero_grad(set_to_none=True)
            xi = x.clone().requires_grad_(True)
            y, l_aux = m(0, xi)
            torch.autograd.backward([y, l_aux], [dy, torch.full((), 2.0, device=dev)])
            torch.cuda.synchronize()
            params = [m.batched_fc1_w[0], m.batched_fc2_w[0]] + ([m.batched_fc1_bias[0], m.batched_fc2_bias[0]] if bias else [])
            res.append((m.dispatch_params.routing_.clone().long().cpu(), y.detach().clone(), xi.grad.clone(), [p.grad.clone() for p in params]))
    finally:
        _lib.check(lib.hexa_set_option(b"ffn_fused", 0), "hexa_set_option")
    (ra, ya, dxa, ga), (rb, yb, dxb, gb) = res
    assert torch.equal(ra, rb)
    y_ref, _ = _oracle_depth(m, 0, x.float().cpu(), ra, dy.float().cpu(), F.gelu, torch.float32)
    assert_close(ya, y_ref, TOL[dtype], "y (one kernel) vs oracle")
    assert_close(ya, yb, TOL[dtype] / 4, "y (one kernel) vs two launches")
    assert_close(dxa, dxb, TOL[dtype] / 4, "dx")
    for u, v in zip(ga, gb):
        assert_close(u, v, TOL[dtype] / 4, "parameter gradient")


def _route_fields(blob, T, k, E):
    """The fields of a route blob that the routing pass defines (tile records up to each slot's count)."""
    from hexa_moe import _lib
    L = _lib.route_layout(T, k, E)
    b = blob.cpu()
    out = [b[L.counts:L.counts + k * E], b[L.offsets:L.offsets + k * (E + 1)], b[L.token_ids:L.token_ids + k * T],
           b[L.expert_ids:L.expert_ids + k * T], b[L.tile_count:L.tile_count + k], b[L.tile_count_l:L.tile_count_l + k]]
    for s in range(k):
        n, nl = int(b[L.tile_count + s]), int(b[L.tile_count_l + s])
        out.append(b[L.tile_info + 4 * s * L.mt_ub:L.tile_info + 4 * (s * L.mt_ub + min(n, L.mt_ub))])
        out.append(b[L.tile_info_l + 4 * s * L.mt_ub_l:L.tile_info_l + 4 * (s * L.mt_ub_l + min(nl, L.mt_ub_l))])
    return [t.clone() for t in out]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,d,E,k,train", [(2500, 256, 16, 2, True), (2300, 384, 32, 2, False), (1900, 128, 5, 3, True),
                                           (130, 264, 33, 2, True), (63, 8, 64, 1, False), (4097, 96, 7, 4, True),
                                           (700, 64, 100, 2, True), (900, 128, 240, 3, False), (500, 64, 130, 2, True)])
def test_gate_and_router_in_one_launch(dev, dtype, T, d, E, k, train):
    """The depth call's front end with the gate projection and the router in one kernel (the default up to 64
    experts) against the same call with the two as separate launches (library option "gate_router" = 2): the one
    kernel repeats the gate's sums in the same order, so routing, y, l_aux and every gradient are identical -- with
    gate noise (train mode, same seed), expert counts that are no multiple of 4 or span two 32-expert blocks, and a
    last workgroup with fewer than 64 tokens (above 64 experts the gate is a launch of its own either way).  Likewise
    the routing pass behind the router's histogram as one launch
    (default) against a scan and a scatter launch (option "route_kernels" = 3): every field of the route is identical."""
    from hexa_moe import _lib
    lib = _lib.load()
    m = _module([d], [0], E=E, k=k, act=F.gelu, noise=1.0).to(dev).to(dtype)
    m.train(train)
    m.gates[0].wg.weight.data = m.gates[0].wg.weight.data.float()
    m.fused_depth = True
    g = torch.Generator().manual_seed(29)
    x = torch.randn(T, d, generator=g).to(dtype).to(dev)
    dy = torch.randn(T, d, generator=g).to(dtype).to(dev)
    res = []
    try:
        for name, value in ((b"gate_router", 0), (b"gate_router", 2), (b"route_kernels", 3)):
            _lib.check(lib.hexa_set_option(b"gate_router", 0), "hexa_set_option")
            _lib.check(lib.hexa_set_option(b"route_kernels", 0), "hexa_set_option")
            _lib.check(lib.hexa_set_option(name, value), "hexa_set_option")
            torch.manual_seed(5)                      # the gate noise of both runs
            m.zero_grad(set_to_none=True)
            xi = x.clone().requires_grad_(True)
            y, l_aux = m(0, xi)
            torch.autograd.backward([y, l_aux], [dy, torch.full((), 2.0, device=dev)])
            torch.cuda.synchronize()
            blob = next(iter(m.dispatch_params.route_pool._slots.values()))[0]
            res.append((m.dispatch_params.routing_.clone(), y.detach().clone(), l_aux.detach().clone(), xi.grad.clone(),
                        [p.grad.clone() for p in m.parameters() if p.grad is not None], _route_fields(blob, T, k, E)))
    finally:
        _lib.check(lib.hexa_set_option(b"gate_router", 0), "hexa_set_option")
        _lib.check(lib.hexa_set_option(b"route_kernels", 0), "hexa_set_option")
    ra, ya, la, dxa, ga, fa = res[0]
    assert len(ga) >= 3
    for rb, yb, lb, dxb, gb, fb in res[1:]:
        assert torch.equal(ra, rb) and torch.equal(ya, yb) and torch.equal(la, lb) and torch.equal(dxa, dxb)
        assert len(ga) == len(gb) and len(fa) == len(fb)
        for u, v in zip(ga, gb):
            assert torch.equal(u, v)
        for u, v in zip(fa, fb):
            assert torch.equal(u, v)
