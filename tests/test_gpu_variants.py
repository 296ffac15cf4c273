"""Every kernel variant of the 16-bit fast path (tile shapes, the pipelined persistent kernel, tile-to-XCD mapping,
general kernels) must give the same results: the operators are run under each setting of the library's
tuning knobs and compared with the CPU oracle."""
import pytest
import torch

from _util import TOL, assert_close, gen, make_linear, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu

SETTINGS = [{"tile": t} for t in range(1, 12)] + [
    {"pipe": 1}, {"pipe": 2}, {"tile": 12}, {"tile": 13},
    {"esmm_map": 2}, {"esmm_map": 2, "esmm_group": 16}, {"estmm_group": 1}, {"estmm_group": 4}, {"estmm_group": 12}, {"esmm_stream": 1}, {"esmm_stream": 2}, {"general_kernels": 1}, {"estmm_pipe": 1},
]
ALL = ("tile", "pipe", "esmm_map", "esmm_group", "estmm_group", "esmm_stream", "general_kernels", "estmm_pipe")


@pytest.fixture
def knobs():
    from hexa_moe import _lib
    lib = _lib.load()

    def apply(cfg):
        for name in ALL:
            _lib.check(lib.hexa_set_option(name.encode(), int(cfg.get(name, 0))), "hexa_set_option")
    yield apply
    apply({})


@pytest.mark.parametrize("cfg", SETTINGS, ids=lambda c: ",".join(f"{k}={v}" for k, v in c.items()))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dims", [(2300, 192, 392), (1700, 256, 320)], ids=["192x392", "256x320"])
def test_variant(dev, knobs, cfg, dtype, dims):
    """The second pair of dimensions (contractions of 256 and 320: multiples of 64, at least 256) is one the pipelined
    persistent kernel covers, in both directions; the first one it leaves to the one-tile kernels."""
    from hexa_moe import _lib, ops
    knobs(cfg)
    (T, d_in, d_out), E, k = dims, 6, 2
    g = gen(5)
    routing = make_routing(T, E, k, seed=6, skew="zipf", empty=1)
    _, offsets, token_ids = O.route_build(routing, E)
    route = ops.route_build(routing.to(dev), E)
    x, W, b = make_linear(T, d_in, d_out, E, k, seed=7, dtype=dtype, m2s=False)
    want = O.esmm(x.float(), W.float(), b.float(), token_ids, offsets, False)
    # per-slot result, both weight layouts, fused GELU and GELU'
    y1, y2 = ops.esmm(x.to(dev), W.to(dev), b.to(dev), route, False, _lib.HEXA_W_IN_OUT, gelu=True)
    assert_close(y1, want, TOL[dtype], "esmm in_out")
    assert_close(y2, torch.nn.functional.gelu(want), TOL[dtype], "esmm gelu")
    Wt = W.transpose(1, 2).contiguous().to(dev)
    got = ops.esmm(x.to(dev), Wt, b.to(dev), route, False, _lib.HEXA_W_OUT_IN)
    assert_close(got, want, TOL[dtype], "esmm out_in")
    base = torch.randn(want.shape, generator=g).to(dtype)
    acc = base.clone().to(dev)
    ops.esmm(x.to(dev), Wt, b.to(dev), route, False, _lib.HEXA_W_OUT_IN, out=acc, accumulate=True)
    assert_close(acc, want + base.float(), TOL[dtype], "esmm accumulating")
    y1r = y1.float().cpu().double().requires_grad_(True)
    lin = O.esmm(x.float(), W.float(), None, token_ids, offsets, False)
    (want_g,) = torch.autograd.grad(torch.nn.functional.gelu(y1r), y1r, lin.double())
    got = ops.esmm(x.to(dev), Wt, None, route, False, _lib.HEXA_W_OUT_IN, gelu_bwd_of=y1)
    assert_close(got, want_g, TOL[dtype], "esmm * gelu'")
    got, db = ops.esmm_gelu_bwd_ess(x.to(dev), Wt, route, _lib.HEXA_W_OUT_IN, y1)
    assert_close(got, want_g, TOL[dtype], "esmm * gelu' (with column sums)")
    assert_close(db, O.ess(got.float().cpu(), token_ids, offsets, True, E), 1e-5, "column sums of the stored result")
    # sum over slots (per-slot operand), accumulating
    xs = torch.randn(k, T, d_out, generator=g).to(dtype)
    W2 = ((torch.rand(E, d_out, d_in, generator=g) * 2 - 1) / d_out ** 0.5).to(dtype)
    b2 = torch.randn(E, d_in, generator=g).to(dtype)
    want2 = O.esmm(xs.float(), W2.float(), b2.float(), token_ids, offsets, True)
    got2 = ops.esmm(xs.to(dev), W2.to(dev), b2.to(dev), route, True, _lib.HEXA_W_IN_OUT)
    assert_close(got2, want2, TOL[dtype], "esmm sum over slots")
    # ESTMM, 16-bit and fp32 results
    want_dw = O.estmm(xs.float(), x.float(), token_ids, offsets, True, E)
    assert_close(ops.estmm(xs.to(dev), x.to(dev), route, True, False), want_dw, TOL[dtype], "estmm")
    assert_close(ops.estmm(xs.to(dev), x.to(dev), route, True, False, out_dtype=dtype), want_dw, TOL[dtype], "estmm 16-bit")
    torch.cuda.synchronize()
