"""The Triton sibling's operator surface (counter, ESMM, es_fused; reference hexa_moe_triton/hexa_moe/kernels)
on the HIP library, through its own list format -- chunks of 16 per expert, -1 padding, callers add 1 -- against
the CPU oracle."""
import pytest
import torch

from _util import TOL, assert_close, gen, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu


def _lists(routing_slot, E, dev):
    from hexa_moe.kernels import counter
    n, start, tok, exp = counter(routing_slot.to(dev), E)
    return n, start, tok, exp


@pytest.mark.parametrize("T,E", [(1000, 8), (37, 5), (4096, 32)])
def test_counter_format(dev, T, E):
    routing = make_routing(T, E, 1, seed=T + E, skew="zipf", empty=1)[:, 0]
    n, start, tok, exp = _lists(routing, E, dev)
    counts, expanded = O.token_count(routing.to(torch.int32), E, pad=16)
    assert n == int(expanded[-1]) and torch.equal(start.cpu(), expanded.to(torch.int32))
    assert tok.shape == (n,) and exp.shape == (n // 16,) and tok.dtype == torch.int32 and exp.dtype == torch.int32
    tok, exp = tok.cpu(), exp.cpu()
    for e in range(E):
        seg = tok[int(expanded[e]):int(expanded[e + 1])]
        real = seg[seg >= 0]
        assert torch.equal(real, torch.nonzero(routing == e).flatten().to(torch.int32))      # ascending, complete
        assert (seg[len(real):] == -1).all()
        assert (exp[int(expanded[e]) // 16:int(expanded[e + 1]) // 16] == e).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [True, False])
def test_esmm_and_es_fused(dev, dtype, with_bias):
    from hexa_moe.kernels import ESMM, es_fused
    T, d_in, d_out, E = 1500, 136, 264, 6
    g = gen(41)
    routing = make_routing(T, E, 1, seed=42, skew="zipf", empty=1)
    _, offsets, token_ids = O.route_build(routing, E)
    n, start, tok, exp = _lists(routing[:, 0], E, dev)
    tok1b = (tok + 1).contiguous()                                    # what the reference's layer passes on
    x = torch.randn(T, d_in, generator=g).to(dtype)
    W = ((torch.rand(E, d_in, d_out, generator=g) * 2 - 1) / d_in ** 0.5).to(dtype)
    b = torch.randn(E, d_out, generator=g).to(dtype)
    rd = torch.float64 if dtype == torch.float32 else torch.float32
    tol = TOL[dtype]
    got = ESMM(x.to(dev), W.to(dev), b.to(dev) if with_bias else torch.empty(0, device=dev), tok1b, exp)
    want = O.esmm(x.to(rd), W.to(rd), b.to(rd) if with_bias else None, token_ids, offsets, False)[0]
    assert got.shape == (T, d_out) and got.dtype == dtype
    assert_close(got, want, tol, "ESMM")
    # backward step: tok1 = dy [T, out], tok2 = x [T, in], w [E, out, in]
    dy = torch.randn(T, d_out, generator=g).to(dtype)
    Wt = W.transpose(1, 2).contiguous()
    res = es_fused(dy.to(dev), x.to(dev), Wt.to(dev), tok1b, exp, start, E, bias=with_bias)
    jb, jx, jw = O.fused_grad(dy.to(rd), Wt.to(rd), x.to(rd)[None], token_ids, offsets, False, True)
    if with_bias:
        r_ess, r_esmm, r_estmm = res
        assert_close(r_ess, jb, tol, "es_fused: ESS")
    else:
        r_esmm, r_estmm = res
    assert_close(r_esmm, jx[0], tol, "es_fused: ESMM")
    assert_close(r_estmm, jw, tol, "es_fused: ESTMM")
    assert r_estmm.shape == (E, d_out, d_in) and r_esmm.shape == (T, d_in)
    torch.cuda.synchronize()
