"""The benchmark's named configurations at their full sizes, GPU (through the C ABI) vs the CPU oracle.

  * ESMM alone at T=18432, d=384, h=1536, E=32, top-2, bf16 (uneven load from biased gate logits);
  * a full MoE layer forward + backward at T=4608, d=768, h=3072, E=32, top-1, bf16;
  * the skewed stress case T=32768, d=1024, h=4096, E=64, top-2 with Zipf(1.2) expert ranks and at
    least four experts without tokens: ESMM forward + ESTMM + ESS.

Tolerance 2e-2 (bf16 operands, fp32 accumulation) against the fp32 oracle on the bf16-rounded inputs;
routing counts and token lists bit-exact.  Where the full oracle would take minutes (the stress
case's weight gradient) the comparison is made on a seeded subset of experts plus properties that do
not depend on size: empty experts give exact zeros, the bias gradient equals the column sums of dy
regrouped, and the operator is linear in dy.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from _util import TOL, assert_close, gen, make_routing, uniform
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _check_route(route, routing, E):
    counts, offsets, token_ids = O.route_build(routing, E)
    assert torch.equal(route.counts.cpu(), counts)
    assert torch.equal(route.offsets.cpu(), offsets)
    assert torch.equal(route.token_ids.cpu(), token_ids)
    return counts, offsets, token_ids


def test_esmm_swin_stage3_shape(dev):
    from hexa_moe import _lib, ops
    T, d, h, E, k = 18432, 384, 1536, 32, 2
    print(f"config ESMM T={T} d={d} h={h} E={E} k={k} bf16 seed=1235", flush=True)
    g = gen(1235)
    x = torch.randn(T, d, generator=g).to(BF16)
    W = uniform((E, d, h), 1 / math.sqrt(d), g).to(BF16)
    b = uniform((E, h), 1 / math.sqrt(d), g).to(BF16)
    logits = torch.randn(T, E, generator=g) + 0.5 * torch.randn(E, generator=g)
    routing = torch.topk(torch.softmax(logits, 1), k, dim=1).indices
    route = ops.route_build(routing.to(dev), E)
    counts, offsets, token_ids = _check_route(route, routing, E)
    assert int(counts.sum(0).max()) > 1.5 * T * k / E      # the load is uneven
    want = O.esmm(x.float(), W.float(), b.float(), token_ids, offsets, False)
    got = ops.esmm(x.to(dev), W.to(dev), b.to(dev), route, False, _lib.HEXA_W_IN_OUT)
    got_t = ops.esmm(x.to(dev), W.transpose(1, 2).contiguous().to(dev), b.to(dev), route, False, _lib.HEXA_W_OUT_IN)
    torch.cuda.synchronize()
    assert got.shape == (k, T, h) and got.dtype == BF16
    assert_close(got, want, TOL[BF16], "esmm [E,in,out]")
    assert_close(got_t, want, TOL[BF16], "esmm [E,out,in]")


@pytest.mark.parametrize("act", [F.gelu, lambda t: F.gelu(t)], ids=["fused_gelu", "generic_activation"])
def test_layer_fwd_bwd_T4608_d768(dev, act):
    from hexa_moe import moe as hmoe
    T, d, E, k = 4608, 768, 32, 1
    print(f"config layer T={T} d={d} h={4 * d} E={E} k={k} bf16 seed=1236", flush=True)
    torch.manual_seed(1236)
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': k, 'gate_noise': 0.0, 'fp32_gate': True},
                          model_dim_list=[d], moe_idx_list=[0], mlp_ratio=4, num_global_experts=E, total_depth=1,
                          data_centric=True, mlp_fc1_bias=True, mlp_fc2_bias=True, activation_fn=act)
    g = gen(1236)
    for name, p in m.named_parameters():
        fan_in = p.shape[-1] if name.startswith(("batched_fc1_w", "gates")) else p.shape[-2] if p.dim() > 1 else p.shape[-1]
        p.data.copy_((torch.rand(p.shape, generator=g) * 2 - 1) / fan_in ** 0.5)
    m = m.to(dev).to(BF16).eval()
    x = torch.randn(T, d, generator=g).to(BF16)
    dy = torch.randn(T, d, generator=g).to(BF16)
    xd = x.to(dev).requires_grad_(True)
    y, _ = m(0, xd)
    routing = m.dispatch_params.routing_.cpu()
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    W1, W2 = m.batched_fc1_w[0].detach().cpu().float(), m.batched_fc2_w[0].detach().cpu().float()
    b1, b2 = m.batched_fc1_bias[0].detach().cpu().float(), m.batched_fc2_bias[0].detach().cpu().float()
    y_ref, y1, _ = O.moe_ffn_forward(x.float(), W1, W2, b1, b2, routing, F.gelu)
    dx, dW1, dW2, db1, db2 = O.moe_ffn_backward(dy.float(), x.float(), y1, W1, W2, True, True, routing, F.gelu)
    tol = TOL[BF16]
    assert_close(y, y_ref, tol, "y")
    assert_close(xd.grad, dx, tol, "dx")
    assert_close(m.batched_fc1_w[0].grad, dW1, tol, "dW1")
    assert_close(m.batched_fc2_w[0].grad, dW2, tol, "dW2")
    assert_close(m.batched_fc1_bias[0].grad, db1, tol, "db1")
    assert_close(m.batched_fc2_bias[0].grad, db2, tol, "db2")


def test_skewed_stress_T32768_E64(dev):
    from hexa_moe import _lib, ops
    T, d, h, E, k = 32768, 1024, 4096, 64, 2
    print(f"config stress T={T} d={d} h={h} E={E} k={k} bf16 zipf seed=1238", flush=True)
    routing = make_routing(T, E, k, seed=1238, skew="zipf", empty=4)
    g = gen(1238)
    x = torch.randn(T, d, generator=g).to(BF16)
    W = uniform((E, d, h), 1 / math.sqrt(d), g).to(BF16)
    b = uniform((E, h), 1 / math.sqrt(d), g).to(BF16)
    route = ops.route_build(routing.to(dev), E)
    counts, offsets, token_ids = _check_route(route, routing, E)
    load = counts.sum(0)
    empty = load == 0
    assert int(empty.sum()) >= 4 and int(load.max()) > 8 * int(load[load > 0].min())
    xd, Wd, bd = x.to(dev), W.to(dev), b.to(dev)

    # ESMM forward over every token; the oracle evaluates a seeded subset of the token rows
    y = ops.esmm(xd, Wd, bd, route, False, _lib.HEXA_W_IN_OUT)
    torch.cuda.synchronize()
    pick = torch.randperm(T, generator=g)[:4096]
    for s in range(k):
        e = routing[pick, s]
        want = torch.bmm(x[pick].float()[:, None, :], W.float()[e]).squeeze(1) + b.float()[e]
        assert_close(y[s, pick.to(dev)], want, TOL[BF16], f"esmm slot {s}")

    # ESTMM + ESS of a seeded dy (per-slot [k,T,h]) against the oracle on the busiest, the lightest
    # non-empty and four seeded experts; empty experts give exact zeros
    dy = torch.randn(k, T, h, generator=g).to(BF16)
    dyd = dy.to(dev)
    dw = ops.estmm(dyd, xd, route, True, False)
    db = ops.ess(dyd, route, True)
    torch.cuda.synchronize()
    assert dw.shape == (E, h, d) and db.shape == (E, h)
    live = torch.nonzero(~empty).flatten()
    order = live[torch.argsort(load[live])]
    chosen = {int(order[0]), int(order[-1])} | {int(live[i]) for i in torch.randperm(len(live), generator=g)[:4]}
    for e in sorted(chosen):
        dw_ref = torch.zeros(h, d)
        db_ref = torch.zeros(h)
        for s in range(k):
            rows = O._rows(token_ids, offsets, s, e)
            if rows.numel():
                dye = dy[s].index_select(0, rows).float()
                dw_ref += dye.t() @ x.index_select(0, rows).float()
                db_ref += dye.sum(0)
        assert_close(dw[e], dw_ref, TOL[BF16], f"estmm expert {e} ({int(load[e])} rows)")
        assert_close(db[e], db_ref, TOL[BF16], f"ess expert {e}")
    assert float(dw[empty.to(dev)].abs().max()) == 0.0 and float(db[empty.to(dev)].abs().max()) == 0.0
    # size-independent properties: the bias gradients add up to the column sums of dy, and both
    # operators are linear in dy (doubling is exact in binary floating point, so the results double exactly)
    assert_close(db.sum(0), dy.float().sum((0, 1)), TOL[BF16], "sum of db")
    dw2 = ops.estmm(dyd * 2, xd, route, True, False)
    db2 = ops.ess(dyd * 2, route, True)
    torch.cuda.synchronize()
    assert torch.equal(dw2, dw * 2) and torch.equal(db2, db * 2)


def test_large_token_count(dev):
    """300 000 tokens (more than 2^16 units of every kind: rows, tiles, routing units), small dimensions:
    every operator against the full oracle."""
    from hexa_moe import _lib, ops
    T, d_in, d_out, E, k = 300_000, 64, 72, 8, 2
    print(f"config large T={T} in={d_in} out={d_out} E={E} k={k} bf16 seed=1239", flush=True)
    g = gen(1239)
    routing = make_routing(T, E, k, seed=1239)
    x = torch.randn(T, d_in, generator=g).to(BF16)
    W = uniform((E, d_in, d_out), 1 / math.sqrt(d_in), g).to(BF16)
    b = uniform((E, d_out), 1 / math.sqrt(d_in), g).to(BF16)
    dy = torch.randn(k, T, d_out, generator=g).to(BF16)
    route = ops.route_build(routing.to(dev), E)
    counts, offsets, token_ids = _check_route(route, routing, E)
    tol = TOL[BF16]
    y = ops.esmm(x.to(dev), W.to(dev), b.to(dev), route, False, _lib.HEXA_W_IN_OUT)
    assert_close(y, O.esmm(x.float(), W.float(), b.float(), token_ids, offsets, False), tol, "esmm")
    ys = ops.esmm(dy.to(dev), W.transpose(1, 2).contiguous().to(dev), None, route, True, _lib.HEXA_W_IN_OUT)
    assert_close(ys, O.esmm(dy.float(), W.transpose(1, 2).float(), None, token_ids, offsets, True), tol, "esmm summed")
    dw = ops.estmm(dy.to(dev), x.to(dev), route, True, False)
    assert_close(dw, O.estmm(dy.float(), x.float(), token_ids, offsets, True, E), tol, "estmm")
    db = ops.ess(dy.to(dev), route, True)
    assert_close(db, O.ess(dy.float(), token_ids, offsets, True, E), tol, "ess")


def test_benchmark_step_T18432_top2_default_depth_path(dev):
    """The benchmark's own module and inputs (bench.make_module_and_inputs: T=18432, d=384, h=1536, E=32, top-2,
    bf16 experts, fp32 gate) through the default path -- one library call per direction -- against the oracle:
    y, dx and the four parameter gradients of the expert path, then dx and the gate's weight gradient with the
    auxiliary loss in the backward as the benchmark runs it (the gate's share from fp32 autograd of the oracle's
    loss on the same routing)."""
    import bench
    m, x, dy = bench.make_module_and_inputs(dev)
    T, k, E = bench.T, bench.K_TOP, bench.E
    print(f"config benchmark step T={T} d={bench.D} h={bench.H} E={E} k={k} bf16 seed={bench.SEED}", flush=True)
    tol = TOL[BF16]
    cpu = lambda t: t.detach().float().cpu()  # noqa: E731
    W1, W2 = cpu(m.batched_fc1_w[0]), cpu(m.batched_fc2_w[0])
    b1, b2 = cpu(m.batched_fc1_bias[0]), cpu(m.batched_fc2_bias[0])
    wg = cpu(m.gates[0].wg.weight)
    xc, dyc = cpu(x), cpu(dy)

    # expert path alone
    y, l_aux = m(0, x)
    routing = m.dispatch_params.routing_.cpu().long()
    y.backward(dy)
    torch.cuda.synchronize()
    logits = xc @ wg.t()
    scores_ref, routing_ref = O.route_top_k(logits, k)
    # the expert choice is that of torch.topk on the CPU's fp32 scores, except where two scores tie to within the
    # rounding of the projection's sums (a handful of tokens in 18432 at most); the oracle below gets the GPU's routing
    assert int((routing != routing_ref).any(1).sum()) <= 4
    assert abs(float(l_aux.detach()) - float(O.gshard_loss(scores_ref, routing))) < 1e-5
    y_ref, y1, _ = O.moe_ffn_forward(xc, W1, W2, b1, b2, routing, F.gelu)
    dx, dW1, dW2, db1, db2 = O.moe_ffn_backward(dyc, xc, y1, W1, W2, True, True, routing, F.gelu)
    assert_close(y, y_ref, tol, "y")
    assert_close(x.grad, dx, tol, "dx (expert path)")
    assert_close(m.batched_fc1_w[0].grad, dW1, tol, "dW1")
    assert_close(m.batched_fc2_w[0].grad, dW2, tol, "dW2")
    assert_close(m.batched_fc1_bias[0].grad, db1, tol, "db1")
    assert_close(m.batched_fc2_bias[0].grad, db2, tol, "db2")
    assert m.gates[0].wg.weight.grad is None

    # the benchmark's backward: y and the auxiliary loss together (weight 2e4 so that the gate's share is visible
    # next to the expert path's in bf16)
    x.grad = None
    for p in m.parameters():
        p.grad = None
    y, l_aux = m(0, x)
    torch.autograd.backward([y, l_aux], [dy, torch.full((), 2e4, device=dev)])
    torch.cuda.synchronize()
    xg = xc.clone().requires_grad_(True)
    wgg = wg.clone().requires_grad_(True)
    loss = O.gshard_loss(torch.softmax(xg @ wgg.t(), 1), routing)
    gx, gwg = torch.autograd.grad(loss * 2e4, [xg, wgg])
    assert float(gx.norm()) > 3e-2 * float(dx.norm())
    assert_close(x.grad, dx + gx, tol, "dx (expert path + gate)")
    assert_close(m.gates[0].wg.weight.grad, gwg, 1e-4, "dwg")
    assert_close(m.batched_fc1_w[0].grad, dW1, tol, "dW1 (with l_aux)")
