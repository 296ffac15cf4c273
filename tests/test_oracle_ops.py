"""Pins the operator oracle (oracle/hexa_oracle.py) with checks chosen so that a dropped term, a wrong
index or a transposed operand fails one of them: an independent dense formulation (weights gathered
per token + einsum) differentiated by autograd, nn.Linear for E=1, identity weights, duplicated slots,
fp64 gradcheck, and closed forms of the auxiliary losses.  The reference holds no vectors for this path."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import hexa_oracle as O

torch.set_default_dtype(torch.float32)


def _problem(T, d, h, d_out, E, k, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, d, generator=g, dtype=dtype)
    W1 = torch.randn(E, h, d, generator=g, dtype=dtype) / math.sqrt(d)
    W2 = torch.randn(E, h, d_out, generator=g, dtype=dtype) / math.sqrt(h)
    b1 = torch.randn(E, h, generator=g, dtype=dtype)
    b2 = torch.randn(E, d_out, generator=g, dtype=dtype)
    logits = torch.randn(T, E, generator=g)
    routing = torch.topk(logits, k, dim=1).indices
    dy = torch.randn(T, d_out, generator=g, dtype=dtype)
    return x, W1, W2, b1, b2, routing, dy


def _dense_layer(x, W1, W2, b1, b2, routing, act):
    """Independent formulation: gather each token's expert weights, no segments, no sorting."""
    y = 0
    for s in range(routing.shape[1]):
        e = routing[:, s]
        hid = torch.einsum("td,thd->th", x, W1[e]) + (b1[e] if b1 is not None else 0)
        y = y + torch.einsum("th,tho->to", act(hid), W2[e]) + (b2[e] if b2 is not None else 0)
    return y


@pytest.mark.parametrize("k", [1, 2, 3])
@pytest.mark.parametrize("m2s", [False, True])
def test_esmm_against_gathered_bmm(k, m2s):
    T, d_in, d_out, E = 50, 12, 20, 5
    g = torch.Generator().manual_seed(k)
    routing = torch.topk(torch.randn(T, E, generator=g), k, dim=1).indices
    _, offsets, tok = O.route_build(routing, E)
    W = torch.randn(E, d_in, d_out, generator=g, dtype=torch.float64)
    b = torch.randn(E, d_out, generator=g, dtype=torch.float64)
    x = torch.randn((k, T, d_in) if m2s else (T, d_in), generator=g, dtype=torch.float64)
    got = O.esmm(x, W, b, tok, offsets, m2s)
    per_slot = [torch.bmm((x[s] if m2s else x)[:, None, :], W[routing[:, s]]).squeeze(1) + b[routing[:, s]] for s in range(k)]
    want = sum(per_slot) if m2s else torch.stack(per_slot)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)


def test_esmm_special_cases():
    T, d = 40, 16
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, d, generator=g, dtype=torch.float64)
    # E = 1 is a plain linear layer
    lin = torch.nn.Linear(d, 24, dtype=torch.float64)
    routing = torch.zeros(T, 1, dtype=torch.int64)
    _, off, tok = O.route_build(routing, 1)
    got = O.esmm(x, lin.weight.t()[None].detach(), lin.bias[None].detach(), tok, off, False)[0]
    assert torch.allclose(got, lin(x).detach(), atol=1e-12)
    # identity weights return each token's own row; every token to one expert
    routing = torch.full((T, 1), 2, dtype=torch.int64)
    _, off, tok = O.route_build(routing, 4)
    W = torch.eye(d, dtype=torch.float64).repeat(4, 1, 1) * torch.arange(1, 5, dtype=torch.float64)[:, None, None]
    assert torch.allclose(O.esmm(x, W, None, tok, off, False)[0], 3 * x)
    # two slots that pick the same expert double the (m2s) sum
    routing = torch.randint(0, 4, (T, 1), generator=g).repeat(1, 2)
    _, off, tok = O.route_build(routing, 4)
    Wr = torch.randn(4, d, 8, generator=g, dtype=torch.float64)
    one = O.esmm(x[None], Wr, None, tok[:1], off[:1], True)
    two = O.esmm(torch.stack([x, x]), Wr, None, tok, off, True)
    assert torch.allclose(two, 2 * one)


@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("bias", [True, False])
def test_layer_backward_against_autograd_of_dense_formulation(k, bias):
    x, W1, W2, b1, b2, routing, dy = _problem(T=60, d=12, h=20, d_out=10, E=6, k=k, seed=11 + k)
    if not bias:
        b1 = b2 = None
    leaves = [t.clone().requires_grad_(True) for t in (x, W1, W2) + ((b1, b2) if bias else ())]
    y_ref = _dense_layer(leaves[0], leaves[1], leaves[2], leaves[3] if bias else None, leaves[4] if bias else None,
                         routing, F.gelu)
    grads = torch.autograd.grad(y_ref, leaves, dy)
    y, y1, _ = O.moe_ffn_forward(x, W1, W2, b1, b2, routing, F.gelu)
    assert torch.allclose(y, y_ref.detach(), atol=1e-10)
    dx, dW1, dW2, db1, db2 = O.moe_ffn_backward(dy, x, y1, W1, W2, bias, bias, routing, F.gelu)
    assert torch.allclose(dx, grads[0], atol=1e-10)
    assert torch.allclose(dW1, grads[1], atol=1e-10)
    assert torch.allclose(dW2, grads[2], atol=1e-10)
    if bias:
        assert torch.allclose(db1, grads[3], atol=1e-10) and torch.allclose(db2, grads[4], atol=1e-10)
    else:
        assert db1 is None and db2 is None
    # experts nobody chose get exactly zero gradients
    unused = [e for e in range(6) if not (routing == e).any()]
    for e in unused:
        assert dW1[e].abs().max() == 0 and dW2[e].abs().max() == 0


def test_operator_contracts_against_autograd():
    """ESTMM / ESS / ESMM-bwd in the FUSED_GRAD layout are the gradients of the ESMM contract."""
    T, d_in, d_out, E, k = 45, 8, 14, 4, 2
    g = torch.Generator().manual_seed(5)
    routing = torch.topk(torch.randn(T, E, generator=g), k, dim=1).indices
    _, off, tok = O.route_build(routing, E)
    for m2s in (False, True):
        x = torch.randn((k, T, d_in) if m2s else (T, d_in), generator=g, dtype=torch.float64, requires_grad=True)
        W = torch.randn(E, d_in, d_out, generator=g, dtype=torch.float64, requires_grad=True)
        b = torch.randn(E, d_out, generator=g, dtype=torch.float64, requires_grad=True)
        per_slot = [torch.bmm((x[s] if m2s else x)[:, None, :], W[routing[:, s]]).squeeze(1) + b[routing[:, s]] for s in range(k)]
        y = sum(per_slot) if m2s else torch.stack(per_slot)
        jy = torch.randn(y.shape, generator=g, dtype=torch.float64)
        gx, gW, gb = torch.autograd.grad(y, (x, W, b), jy)
        # forward m2s=True (x per slot, y shared) pairs with FUSED_GRAD m2s=False (j_y shared, x per slot)
        jb, jx, jw = O.fused_grad(jy, W.detach().transpose(1, 2), x.detach(), tok, off, m2s=not m2s, with_bias=True)
        assert torch.allclose(jx, gx, atol=1e-10)
        assert torch.allclose(jw, gW.transpose(1, 2), atol=1e-10)
        assert torch.allclose(jb, gb, atol=1e-10)


def test_layer_gradcheck_fp64():
    x, W1, W2, b1, b2, routing, _ = _problem(T=32, d=6, h=8, d_out=5, E=3, k=2, seed=3)

    class Layer(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, W1, W2, b1, b2):
            y, y1, _ = O.moe_ffn_forward(x, W1, W2, b1, b2, routing, torch.tanh)
            ctx.save_for_backward(x, y1, W1, W2)
            return y

        @staticmethod
        def backward(ctx, dy):
            x, y1, W1, W2 = ctx.saved_tensors
            return O.moe_ffn_backward(dy, x, y1, W1, W2, True, True, routing, torch.tanh)

    args = [t.clone().requires_grad_(True) for t in (x, W1, W2, b1, b2)]
    assert torch.autograd.gradcheck(Layer.apply, args, eps=1e-6, atol=1e-6)


def test_dense_mlp_matches_linear_layers():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(20, 8, generator=g)
    fc1 = torch.nn.Linear(8, 32)
    fc2 = torch.nn.Linear(32, 8)
    want = fc2(F.gelu(fc1(x))).detach()
    got = O.dense_mlp_forward(x, fc1.weight.detach(), fc2.weight.t().detach(), fc1.bias.detach(), fc2.bias.detach(), F.gelu)
    assert torch.allclose(got, want, atol=1e-6)


def test_gshard_loss_closed_forms():
    T, E = 64, 8
    # uniform scores: me = T/E each, sum ce = E  ->  l_aux = (T/E) * E / T = 1, whatever the choice is
    scores = torch.full((T, E), 1.0 / E)
    ids = torch.randint(0, E, (T, 2))
    assert abs(float(O.gshard_loss(scores, ids)) - 1.0) < 1e-6
    # everything on expert 0 with score 1: me[0] = T, ce[0] = E  ->  l_aux = E
    scores = torch.zeros(T, E); scores[:, 0] = 1
    assert abs(float(O.gshard_loss(scores, torch.zeros(T, 1, dtype=torch.int64))) - E) < 1e-5
    # only the first slot counts
    s = torch.softmax(torch.randn(T, E), 1)
    ids = torch.topk(s, 2, dim=1).indices
    assert torch.allclose(O.gshard_loss(s, ids), O.gshard_loss(s, ids[:, :1]))


def test_load_importance_loss_closed_forms():
    T, E = 128, 4
    # identical rows: importance is a multiple of the row, load has zero variance when all scores equal
    scores = torch.full((T, E), 0.25)
    thr = torch.full((T, 1), 0.25)
    assert abs(float(O.load_importance_loss(scores, thr, E, 1.0))) < 1e-6
    # scores far above / below the threshold: load = T * indicator
    scores = torch.zeros(T, E); scores[:, 0] = 1.0
    thr = torch.full((T, 1), 0.5)
    imp = torch.tensor([float(T), 0, 0, 0]); load = torch.tensor([float(T), 0, 0, 0])
    want = (imp.var() / imp.mean() ** 2 + load.var() / load.mean() ** 2) / 2
    assert abs(float(O.load_importance_loss(scores, thr, E, 1e-3)) - float(want)) < 1e-4


def test_load_importance_loss_sigma_is_gate_noise_over_experts():
    """The width of the normal CDF is gate_noise / E (impls/losses.py:27-33: Normal(0, gate_noise / E)).
    An independent evaluation with torch.special.ndtr, in the steep regime (scores within a few sigma of
    the threshold), differs from one with sigma = gate_noise by far more than the tolerance, so a dropped
    `/ E` in the oracle fails here."""
    g = torch.Generator().manual_seed(11)
    T, E, noise = 512, 8, 0.16          # sigma = 0.02
    scores = torch.softmax(0.3 * torch.randn(T, E, generator=g), 1).double()
    thr = scores.mean(1, keepdim=True) + 0.01 * torch.randn(T, 1, generator=g).double()

    def independent(sigma):
        load = torch.special.ndtr((scores - thr) / sigma).sum(0)
        imp = scores.sum(0)
        cv2 = lambda v: v.var(unbiased=True) / (v.mean() ** 2 + 1e-10)   # noqa: E731
        return float((cv2(imp) + cv2(load)) / 2)

    got = float(O.load_importance_loss(scores.float(), thr.float(), E, noise))
    assert abs(got - independent(noise / E)) < 1e-5 * max(1.0, abs(got))
    assert abs(independent(noise) - independent(noise / E)) > 5e-4      # 50x the tolerance above: the scales are far apart


def test_nan_token_row_in_the_oracle():
    """Pins what the GPU test of a NaN token row expects: softmax of a row with a NaN is all NaN, torch.topk
    still returns ids in [0, E), the token stays in its experts' lists, and its output row is NaN while every
    other row is finite."""
    g = torch.Generator().manual_seed(5)
    T, d, h, E, k = 64, 16, 32, 4, 2
    x = torch.randn(T, d, generator=g)
    x[7] = float("nan")
    wg = torch.randn(E, d, generator=g)
    scores, idx = O.route_top_k(x @ wg.t(), k)
    assert torch.isnan(scores[7]).all() and int(idx.min()) >= 0 and int(idx.max()) < E
    counts, offsets, token_ids = O.route_build(idx, E)
    assert int(counts.sum()) == T * k and (token_ids == 7).sum() == k
    W1, W2 = torch.randn(E, h, d, generator=g), torch.randn(E, h, d, generator=g)
    y, _, _ = O.moe_ffn_forward(x, W1, W2, None, None, idx, F.gelu)
    assert torch.isnan(y[7]).all()
    keep = torch.ones(T, dtype=torch.bool); keep[7] = False
    assert torch.isfinite(y[keep]).all()
