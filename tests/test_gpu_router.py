"""Fused routing front end (gate projection, softmax + top-k + GShard loss and its backward) on the
GPU vs the PyTorch formulation the oracle uses.  Expert choices must be identical; fp32 values agree
to summation-order rounding."""
import pytest
import torch
import torch.nn.functional as F

from _util import assert_close, gen
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,d,E", [(1000, 384, 32), (77, 128, 8), (300, 256, 70), (18432, 384, 32)])
def test_gate_logits(dev, dtype, T, d, E):
    from hexa_moe import ops
    g = gen(T + E)
    x = torch.randn(T, d, generator=g).to(dtype)
    wg = torch.randn(E, d, generator=g) / d ** 0.5
    want = x.double() @ wg.double().t()
    got = ops.gate_logits(x.to(dev), wg.to(dev))
    torch.cuda.synchronize()
    assert got.dtype == torch.float32
    assert_close(got, want, 2e-6, "gate logits")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,d,E", [(1000, 384, 32), (77, 128, 8), (300, 264, 70), (18432, 384, 32), (33, 8, 3)])
def test_gate_backward(dev, dtype, T, d, E):
    """dx = dlogits . wg (in x's type) and dwg = dlogits^T . x (fp32), fp32 products and sums."""
    from hexa_moe import ops
    g = gen(T + E + d)
    x = torch.randn(T, d, generator=g).to(dtype)
    wg = torch.randn(E, d, generator=g) / d ** 0.5
    dl = torch.randn(T, E, generator=g)
    want_dx = dl.double() @ wg.double()
    want_dwg = dl.double().t() @ x.double()
    dx, dwg = ops.gate_backward(dl.to(dev), x.to(dev), wg.to(dev))
    torch.cuda.synchronize()
    assert dx.dtype == dtype and dwg.dtype == torch.float32
    assert_close(dwg, want_dwg, 2e-6, "gate dwg")
    assert_close(dx, want_dx, 2e-6 if dtype == torch.float32 else 2e-2, "gate dx")
    dx_only, none = ops.gate_backward(dl.to(dev), x.to(dev), wg.to(dev), need_dwg=False)
    assert none is None and torch.equal(dx_only, dx)
    # two runs give the same bits (fixed reduction order)
    _, dwg2 = ops.gate_backward(dl.to(dev), x.to(dev), wg.to(dev), need_dx=False)
    assert torch.equal(dwg, dwg2)


@pytest.mark.parametrize("T,E,k", [(1000, 32, 2), (18432, 32, 2), (2048, 8, 1), (513, 70, 3), (64, 4, 4), (257, 300, 2), (130, 9, 8),
                                   (200, 240, 5)])
@pytest.mark.parametrize("with_noise", [False, True])
def test_router_forward_and_backward(dev, T, E, k, with_noise):
    from hexa_moe import ops
    g = gen(T * k + E)
    logits = torch.randn(T, E, generator=g) + 0.5 * torch.randn(E, generator=g)
    noise = torch.randn(T, E, generator=g) if with_noise else None
    scale = 1.0 / E
    scores_ref, idx_ref = O.route_top_k(logits, k, noise * scale if with_noise else None)
    scores, idx, me, ce, l_aux = ops.router_forward(logits.to(dev), k, noise.to(dev) if with_noise else None, scale)
    torch.cuda.synchronize()
    assert_close(scores, scores_ref, 1e-6, "scores")
    # the choice is the top-k of the kernel's own scores, and agrees with the reference's choice
    assert torch.equal(idx.cpu().long(), torch.topk(scores.cpu(), k, dim=1).indices)
    assert torch.equal(idx.cpu().long(), idx_ref)
    assert_close(me, scores_ref.sum(0), 1e-5, "me")
    assert torch.equal(ce.cpu(), torch.bincount(idx_ref[:, 0], minlength=E).float() * (E / T))
    assert_close(l_aux.reshape(1), O.gshard_loss(scores_ref, idx_ref).reshape(1), 1e-5, "l_aux")
    # backward through the softmax
    lg = logits.clone().double().requires_grad_(True)
    s = F.softmax(lg + (noise.double() * scale if with_noise else 0), dim=1)
    (want,) = torch.autograd.grad(O.gshard_loss(s, idx_ref) * 3.0, lg)
    got = ops.router_backward(scores, ce, torch.tensor(3.0, device=dev))
    torch.cuda.synchronize()
    assert_close(got, want, 1e-5, "dlogits")


def _load_importance_fp64(logits, noisy, idx, sigma):
    """The loss in double precision, differentiable with respect to `logits` (noisy = logits + noise)."""
    s = F.softmax(logits, dim=1)
    thr = noisy.gather(1, idx[:, -1:])
    load = torch.special.ndtr((s - thr) / sigma).sum(0)
    imp = s.sum(0)
    return (imp.var() / (imp.mean() ** 2 + 1e-10) + load.var() / (load.mean() ** 2 + 1e-10)) / 2


@pytest.mark.parametrize("T,E,k", [(1000, 32, 1), (9216, 32, 1), (18432, 32, 2), (2048, 8, 2), (513, 70, 3), (64, 4, 4)])
@pytest.mark.parametrize("with_noise", [False, True])
@pytest.mark.parametrize("spread", [0.02, 1.0])
def test_router_load_importance(dev, T, E, k, with_noise, spread):
    """softmax + top-k + the load-importance loss and its backward against the PyTorch formulation:
    identical expert choices, loss against the oracle, gradient against fp64 autograd.  spread 0.02 is
    the regime of a freshly initialised gate (scores near 1/E, thresholds near 0: the normal CDF is in
    its steep part), spread 1.0 that of a trained one (saturated CDF)."""
    from hexa_moe import ops
    g = gen(T * k + E + 7)
    logits = spread * (torch.randn(T, E, generator=g) + 0.5 * torch.randn(E, generator=g))
    noise = torch.randn(T, E, generator=g) if with_noise else None
    gate_noise = 1.0
    sigma = gate_noise / E
    noisy = logits + noise * sigma if with_noise else logits
    _, idx_ref = O.route_top_k(noisy, k)
    want_l = O.load_importance_loss(F.softmax(logits, 1), noisy.gather(1, idx_ref), E, gate_noise)
    scores, idx, thr, stats = ops.router_forward_load_importance(logits.to(dev), k, sigma,
                                                                 noise.to(dev) if with_noise else None, sigma)
    torch.cuda.synchronize()
    assert torch.equal(idx.cpu().long(), idx_ref)
    assert_close(scores, F.softmax(logits.double(), 1), 1e-6, "scores")
    assert_close(thr, noisy.gather(1, idx_ref[:, -1:]).reshape(-1), 1e-6, "threshold")
    imp, load, l_aux = stats[:E], stats[E:2 * E], stats[4 * E]
    assert_close(imp, F.softmax(logits.double(), 1).sum(0), 1e-5, "importance")
    z = (F.softmax(logits.double(), 1) - noisy.double().gather(1, idx_ref[:, -1:])) / sigma
    assert_close(load, torch.special.ndtr(z).sum(0), 1e-4, "load")
    assert_close(l_aux.reshape(1), want_l.reshape(1).double(), 1e-3, "l_aux vs oracle (fp32)")
    lg = logits.double().requires_grad_(True)
    l64 = _load_importance_fp64(lg, lg + (noise.double() * sigma if with_noise else 0), idx_ref, sigma)
    assert_close(l_aux.reshape(1), l64.detach().reshape(1), 1e-4, "l_aux vs fp64")
    (want_g,) = torch.autograd.grad(l64 * 3.0, lg)
    got_g = ops.router_backward_load_importance(scores, thr, idx, stats, torch.tensor(3.0, device=dev), sigma)
    torch.cuda.synchronize()
    assert_close(got_g, want_g, 1e-4, "dlogits")


def test_ties_go_to_the_lower_index(dev):
    from hexa_moe import ops
    logits = torch.zeros(5, 6)
    logits[1, 3] = logits[1, 4] = 2.0
    _, idx, _, _, _ = ops.router_forward(logits.to(dev), 2)
    assert idx.cpu().tolist() == [[0, 1], [3, 4], [0, 1], [0, 1], [0, 1]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gshard", [True, False])
def test_module_fused_and_framework_routing_agree(dev, dtype, gshard):
    """MoE_Cascaded with the fused routing front end and with the PyTorch formulation of it.  The
    load-importance case runs in eval mode: it needs gate_noise > 0 for its sigma, and only without
    drawn noise do the two runs see the same logits."""
    from hexa_moe import moe as hmoe
    torch.manual_seed(3)
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': 2, 'gate_noise': 0.0 if gshard else 1.0, 'fp32_gate': True},
                          model_dim_list=[256], moe_idx_list=[0], num_global_experts=16, total_depth=1,
                          data_centric=True, activation_fn=F.gelu, is_gshard_loss=gshard)
    for p in m.parameters():
        torch.nn.init.uniform_(p.data, -0.06, 0.06)
    m = m.to(dev)
    if not gshard:
        m.eval()
    if dtype != torch.float32:
        m = m.to(dtype)
    x = torch.randn(3000, 256, device=dev).to(dtype)
    res = []
    for fused in (True, False):
        m.fused_router = fused
        m.zero_grad()
        xi = x.clone().requires_grad_(True)
        y, l_aux = m(0, xi)
        (y.float().sum() + 10.0 * l_aux).backward()
        res.append((m.dispatch_params.routing_.clone().long(), l_aux.detach(), y.detach(), xi.grad, m.gates[0].wg.weight.grad.clone()))
    torch.cuda.synchronize()
    a, b = res
    assert torch.equal(a[0], b[0]), "same expert choices"
    assert_close(a[1].reshape(1), b[1].reshape(1), 1e-5, "l_aux")
    assert torch.equal(a[2], b[2]), "same routing => bit-identical layer output"
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert_close(a[3], b[3], tol, "dx")
    assert_close(a[4], b[4], 1e-4 if dtype == torch.float32 else 2e-2, "gate weight grad")
