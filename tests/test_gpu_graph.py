"""The depth calls under HIP graph capture: a MoE_Cascaded forward + backward captured once with torch.cuda.graph
and replayed with new inputs must give, bit for bit, what the eager calls give -- the library allocates nothing,
never synchronises and never reads a device value on the host (the reference's layer reads one list length per
slot with .item(): hexa_moe_cuda/hexa_moe/impls/layers.py:233-243), so a whole step can be one graph launch.
Between the replays the program runs its own eager work and synchronisations."""
import pytest
import torch
import torch.nn.functional as F

from _util import gen

pytestmark = pytest.mark.gpu


def _module(dev, T, d, E, k, dtype, seed):
    from hexa_moe import moe as hmoe
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': k, 'gate_noise': 0.0, 'fp32_gate': True},
                          model_dim_list=[d], moe_idx_list=[0], mlp_ratio=4, num_global_experts=E, total_depth=1,
                          data_centric=True, mlp_fc1_bias=True, mlp_fc2_bias=True, activation_fn=F.gelu)
    g = gen(seed)
    for p in m.parameters():
        p.data.copy_((torch.rand(p.shape, generator=g) * 2 - 1) * 0.06)
    m = m.to(dev)
    for plist in (m.batched_fc1_w, m.batched_fc2_w, m.batched_fc1_bias, m.batched_fc2_bias):
        for prm in plist:
            prm.data = prm.data.to(dtype)
    return m.train()


@pytest.mark.parametrize("T,d,E,k,dtype", [(2304, 128, 8, 2, torch.bfloat16), (1000, 256, 16, 1, torch.float16),
                                           (4608, 384, 32, 2, torch.bfloat16)])
def test_depth_forward_backward_replays_bit_equal_to_eager(dev, T, d, E, k, dtype):
    print(f"graph capture T={T} d={d} E={E} k={k} {dtype}", flush=True)
    m = _module(dev, T, d, E, k, dtype, seed=T + d)
    params = list(m.parameters())
    g = gen(T)
    inputs = [(torch.randn(T, d, generator=g).to(dtype).to(dev), torch.randn(T, d, generator=g).to(dtype).to(dev))
              for _ in range(4)]
    one = torch.ones((), device=dev)
    sx = inputs[0][0].clone().requires_grad_(True)      # the graph's static input and output-gradient buffers
    sdy = inputs[0][1].clone()

    def step():
        y, l_aux = m(0, sx)
        torch.autograd.backward([y, l_aux], [sdy, one])
        return y, l_aux

    def clear():
        sx.grad = None
        for p in params:
            p.grad = None

    def snapshot(y, l_aux):
        return [y.clone(), l_aux.clone(), sx.grad.clone(), m.dispatch_params.routing_.clone()] + [p.grad.clone() for p in params]

    # eager results for every input pair (also warms up lazily made plans, pools and kernel attributes)
    eager = []
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for x, dy in inputs:
            sx.data.copy_(x); sdy.copy_(dy)
            clear()
            eager.append(snapshot(*step()))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gy, gl = step()
    torch.cuda.synchronize()

    # replays in another order than the eager runs, each preceded by eager work of the program's own
    for i in (2, 0, 3, 1, 2):
        x, dy = inputs[i]
        sx.data.copy_(x); sdy.copy_(dy)
        junk = (x.float() @ x.float().t()[:, :64]).sum()     # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = snapshot(gy, gl)
        assert torch.isfinite(junk)
        names = ["y", "l_aux", "dx", "routing"] + [n for n, _ in m.named_parameters()]
        for name, a, b in zip(names, got, eager[i]):
            assert torch.equal(a, b), f"replay of input {i}: {name} differs from eager"
