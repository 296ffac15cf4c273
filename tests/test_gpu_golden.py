"""The HIP library (through the C ABI) against the committed golden fixtures of tests/golden/: routing bit-exact,
fp32 operators and the layer at 1e-5, the routing front end's choices exact and its losses at 1e-5."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from _util import assert_close
from test_golden import load

pytestmark = pytest.mark.gpu


def f32(a, dev):
    return torch.from_numpy(np.asarray(a)).float().to(dev)


def want(a):
    return torch.from_numpy(np.asarray(a)).double()


def test_routing_fixture(dev):
    import hexa_moe_cuda
    from hexa_moe import ops
    g = load("routing")
    routing, E = torch.from_numpy(g["routing"]), int(g["E"])
    T, k = routing.shape
    route = ops.route_build(routing.to(dev), E)
    torch.cuda.synchronize()
    assert np.array_equal(route.counts.cpu().numpy(), g["counts"])
    assert np.array_equal(route.offsets.cpu().numpy(), g["offsets"])
    assert np.array_equal(route.token_ids.cpu().numpy(), g["token_ids"])
    # the reference's two ops in its 16-padded format, and the route rebuilt from those lists
    hexa_moe_cuda.set_pad(16)
    try:
        toks, exps, ends = [], [], [0]
        for s in range(k):
            r = routing[:, s].to(torch.int32).contiguous().to(dev)
            cnt = torch.zeros(E, dtype=torch.int32, device=dev)
            expd = torch.zeros(E + 1, dtype=torch.int32, device=dev)
            hexa_moe_cuda.TOKEN_COUNT(cnt, expd, r, T, E)
            P = int(expd[-1])
            tok = torch.full((P,), -1, dtype=torch.int32, device=dev)
            exp = torch.full((P,), -1, dtype=torch.int32, device=dev)
            hexa_moe_cuda.TOKEN_ASSIGN(tok, exp, expd, r, T, E)
            assert np.array_equal(cnt.cpu().numpy(), g[f"pad16_counts_{s}"])
            assert np.array_equal(expd.cpu().numpy(), g[f"pad16_expanded_{s}"])
            assert np.array_equal(tok.cpu().numpy(), g[f"pad16_tok_{s}"])
            assert np.array_equal(exp.cpu().numpy(), g[f"pad16_exp_{s}"])
            toks.append(tok); exps.append(exp); ends.append(ends[-1] + P)
    finally:
        hexa_moe_cuda.set_pad(1)
    again = ops.route_from_padded_lists(torch.cat(toks), torch.cat(exps), torch.tensor(ends, dtype=torch.int32, device=dev),
                                        T, k, E)
    torch.cuda.synchronize()
    assert torch.equal(again.token_ids, route.token_ids) and torch.equal(again.offsets, route.offsets)


def test_operator_fixture(dev):
    from hexa_moe import _lib, ops
    g = load("operators")
    routing, E = torch.from_numpy(g["routing"]), int(g["E"])
    route = ops.route_build(routing.to(dev), E)
    x, xs, W, b, dy, dys = (f32(g[k], dev) for k in ("x", "xs", "W", "b", "dy", "dy_shared"))
    assert_close(ops.esmm(x, W, b, route, False, _lib.HEXA_W_IN_OUT), want(g["esmm_per_slot"]), 1e-5, "esmm per slot")
    assert_close(ops.esmm(xs, W.transpose(1, 2).contiguous(), b, route, True, _lib.HEXA_W_OUT_IN), want(g["esmm_summed"]),
                 1e-5, "esmm summed")
    assert_close(ops.estmm(dy, x, route, True, False), want(g["estmm_dy_per_slot"]), 1e-5, "estmm")
    assert_close(ops.estmm(dys, xs, route, False, True), want(g["estmm_dy_shared"]), 1e-5, "estmm shared dy")
    assert_close(ops.ess(dy, route, True), want(g["ess_dy_per_slot"]), 1e-5, "ess")
    assert_close(ops.ess(dys, route, False), want(g["ess_dy_shared"]), 1e-5, "ess shared dy")


def test_layer_fixture(dev):
    from hexa_moe.impls.layers import FusedMoE_Shared_CudaCore
    from hexa_moe.impls.cascaded_moe import RoutePool
    g = load("layer")
    routing, E = torch.from_numpy(g["routing"]).to(dev), int(g["E"])
    x = f32(g["x"], dev).requires_grad_(True)
    prm = [f32(g[k], dev).requires_grad_(True) for k in ("W1", "W2", "b1", "b2")]

    class Cfg:
        pass
    cfg = Cfg()
    cfg.num_global_experts, cfg.indices_, cfg.stage, cfg.route_pool, cfg.activation_fn = E, routing, 0, RoutePool(), F.gelu
    y = FusedMoE_Shared_CudaCore.apply(cfg, x, *prm)
    y.backward(f32(g["dy"], dev))
    torch.cuda.synchronize()
    assert_close(y, want(g["y"]), 1e-5, "y")
    assert_close(x.grad, want(g["dx"]), 1e-5, "dx")
    for name, p in zip(("dW1", "dW2", "db1", "db2"), prm):
        assert_close(p.grad, want(g[name]), 1e-5, name)


def test_router_fixture(dev):
    from hexa_moe import ops
    g = load("router")
    logits, noise = f32(g["logits"], dev), f32(g["noise"], dev)
    k, gate_noise = int(g["k"]), float(g["gate_noise"])
    E = logits.shape[1]
    sigma = gate_noise / E
    scores, idx, _me, _ce, l_aux = ops.router_forward(logits, k, noise, sigma)
    torch.cuda.synchronize()
    assert np.array_equal(idx.cpu().numpy(), g["idx"])
    assert_close(scores, want(g["scores"]), 1e-6, "scores")
    assert_close(l_aux.reshape(1), want(g["gshard"]).reshape(1), 1e-5, "gshard loss")
    _s, idx2, _thr, stats = ops.router_forward_load_importance(logits, k, sigma, noise, sigma)
    torch.cuda.synchronize()
    assert np.array_equal(idx2.cpu().numpy(), g["idx"])
    assert_close(stats[-1].reshape(1), want(g["load_importance"]).reshape(1), 1e-5, "load-importance loss")
