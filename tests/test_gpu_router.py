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


@pytest.mark.parametrize("T,E,k", [(1000, 32, 2), (18432, 32, 2), (2048, 8, 1), (513, 70, 3), (64, 4, 4)])
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


def test_ties_go_to_the_lower_index(dev):
    from hexa_moe import ops
    logits = torch.zeros(5, 6)
    logits[1, 3] = logits[1, 4] = 2.0
    _, idx, _, _, _ = ops.router_forward(logits.to(dev), 2)
    assert idx.cpu().tolist() == [[0, 1], [3, 4], [0, 1], [0, 1], [0, 1]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_fused_and_framework_routing_agree(dev, dtype):
    from hexa_moe import moe as hmoe
    torch.manual_seed(3)
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': 2, 'gate_noise': 0.0, 'fp32_gate': True}, model_dim_list=[256],
                          moe_idx_list=[0], num_global_experts=16, total_depth=1, data_centric=True,
                          activation_fn=F.gelu)
    for p in m.parameters():
        torch.nn.init.uniform_(p.data, -0.06, 0.06)
    m = m.to(dev)
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
        res.append((m.dispatch_params.indices_.clone().long(), l_aux.detach(), y.detach(), xi.grad, m.gates[0].wg.weight.grad.clone()))
    torch.cuda.synchronize()
    a, b = res
    assert torch.equal(a[0], b[0]), "same expert choices"
    assert_close(a[1].reshape(1), b[1].reshape(1), 1e-5, "l_aux")
    assert torch.equal(a[2], b[2]), "same routing => bit-identical layer output"
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert_close(a[3], b[3], tol, "dx")
    assert_close(a[4], b[4], 1e-4 if dtype == torch.float32 else 2e-2, "gate weight grad")
