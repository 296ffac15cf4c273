"""The operators inside their real caller: a Swin-MoE-S-shaped model (swin_moe_harness.SwinMoE) on the GPU.

  * a small fp32 run (4 images, 8 experts): at every MoE depth the FFN's output and the expert-weight
    gradients equal the CPU oracle's on the FFN input, routing and output gradient captured from the run
    (1e-5), and the routing pool holds one slot per MoE depth that is reused by the next step;
  * the benchmark's configuration -- 64 images of 192x192, dims 96/192/384/768, depths 2/2/18/2, window 12,
    MoE on every other block of stages 3 and 4, 32 experts, top-1, bf16 autocast over fp32 master weights,
    train mode (gate noise, stochastic depth) -- forward + backward: finite results, a gradient on every
    parameter, and two MoE depths (one per stage) against the oracle at 2e-2.  The step time is printed.
"""
import time

import pytest
import torch
import torch.nn.functional as F

from _util import TOL, assert_close
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu


class Capture:
    """Keeps, for chosen depths, what the FFN saw: input, routing decision, output (with gradient)."""

    def __init__(self, model, depths):
        self.model, self.depths, self.seen = model, set(depths), {}

    def __call__(self, depth, ffn_in, ffn_out):
        if depth in self.depths:
            ffn_out.retain_grad()
            self.seen[depth] = (ffn_in.detach(), self.model.cascaded_moe.dispatch_params.routing_.clone(), ffn_out)


def _check_depth(model, depth, seen, tol, rd):
    c = model.cascaded_moe
    i = c.moe_idx_list.index(depth)
    ffn_in, routing, ffn_out = seen[depth]
    x = ffn_in.reshape(-1, ffn_in.shape[-1]).cpu()
    dy = ffn_out.grad.reshape(-1, ffn_out.shape[-1]).cpu()
    if tol > 1e-4:     # the layer computes on the 16-bit roundings of its fp32 parameters and inputs
        q = lambda t: t.to(torch.bfloat16).to(rd)
    else:
        q = lambda t: t.to(rd)
    W1, W2 = q(c.batched_fc1_w[i].detach().cpu()), q(c.batched_fc2_w[i].detach().cpu())
    b2 = q(c.batched_fc2_bias[i].detach().cpu()) if c.has_fc2_bias else None
    y_ref, y1, _ = O.moe_ffn_forward(q(x), W1, W2, None, b2, routing.cpu(), F.gelu)
    _, dW1, dW2, _, db2 = O.moe_ffn_backward(q(dy), q(x), y1, W1, W2, False, b2 is not None, routing.cpu(), F.gelu)
    assert_close(ffn_out.detach().reshape(-1, ffn_out.shape[-1]), y_ref, tol, f"depth {depth} y")
    assert_close(c.batched_fc1_w[i].grad, dW1, tol, f"depth {depth} dW1")
    assert_close(c.batched_fc2_w[i].grad, dW2, tol, f"depth {depth} dW2")
    if b2 is not None:
        assert_close(c.batched_fc2_bias[i].grad, db2, tol, f"depth {depth} db2")


def test_small_fp32_every_moe_depth_matches_oracle(dev):
    import swin_moe_harness as S
    print("swin-shaped fp32: 4 images 96x96, depths 2/2/4/2, 8 experts top-2, seed 1237", flush=True)
    torch.manual_seed(1237)
    m = S.SwinMoE(img_size=96, depths=(2, 2, 4, 2), moe_blocks=((-1,), (-1,), (1, 3), (1,)), window_size=6,
                  num_experts=8, top_value=2, num_classes=10, drop_path_rate=0.0, gate_noise=0.0, mlp_fc2_bias=True,
                  is_gshard_loss=True, init_std=0.05).to(dev).train()
    g = torch.Generator().manual_seed(1237)
    images = torch.randn(4, 3, 96, 96, generator=g).to(dev)
    cap = Capture(m, m.moe_depths)
    logits, l_aux = m(images, ffn_hook=cap)
    (logits.square().sum() + l_aux).backward()
    torch.cuda.synchronize()
    assert m.moe_depths == [5, 7, 9]
    for depth in m.moe_depths:
        _check_depth(m, depth, cap.seen, 1e-5, torch.float64)
    # the routing pool: one buffer per MoE depth, taken again by the next step once nothing of this
    # step's autograd graph is alive any more
    pool = m.cascaded_moe.dispatch_params.route_pool
    before = {stage: entry[0].data_ptr() for stage, entry in pool._slots.items()}
    assert sorted(before) == [0, 1, 2]
    want = logits.detach().clone()
    cap.seen.clear()
    del logits, l_aux
    m.zero_grad(set_to_none=True)
    logits2, _ = m(images)
    logits2.sum().backward()
    torch.cuda.synchronize()
    assert torch.allclose(logits2, want)      # nothing stochastic in this configuration
    assert {stage: entry[0].data_ptr() for stage, entry in pool._slots.items()} == before


def test_swin_moe_s_batch64_bf16_autocast(dev):
    import swin_moe_harness as S
    print("swin-moe-s: 64 images 192x192, 32 experts top-1, bf16 autocast, train mode, seed 1237", flush=True)
    torch.manual_seed(1237)
    m = S.SwinMoE(num_experts=32, top_value=1, init_std=0.02).to(dev).train()
    g = torch.Generator().manual_seed(1237)
    images = torch.randn(64, 3, 192, 192, generator=g).to(dev)
    checked = (13, 23)                                   # a stage-3 depth (T=9216, d=384) and stage 4's (T=2304, d=768)
    cap = Capture(m, checked)

    def step(hook=None):
        m.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits, l_aux = m(images, ffn_hook=hook)
            loss = logits.float().square().mean() + l_aux
        loss.backward()
        return logits, loss

    logits, loss = step(cap)
    torch.cuda.synchronize()
    assert logits.shape == (64, 1000) and torch.isfinite(logits).all() and torch.isfinite(loss)
    missing = [n for n, p in m.named_parameters() if p.grad is None]
    assert not missing, missing
    assert all(torch.isfinite(p.grad).all() for p in m.parameters())
    c = m.cascaded_moe
    assert c.batched_fc1_w[0].dtype == torch.float32 and c.batched_fc1_w[0].grad.dtype == torch.float32
    for depth in checked:
        _check_depth(m, depth, cap.seen, TOL[torch.bfloat16], torch.float32)
    # step time with the routing pool warm (not a benchmark line: attention and the dense depths are stock torch)
    for _ in range(2):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 5
    print(f"swin-moe-s fwd+bwd: {dt * 1e3:.1f} ms per step of 64 images = {64 / dt:.0f} images/s", flush=True)
