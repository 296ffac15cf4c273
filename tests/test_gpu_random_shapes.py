"""A seeded sweep over irregular problem shapes: every operator through the C ABI against the CPU oracle.

The hand-picked shapes of the other files cover the corners that are known to matter; this one draws
40 problems from a fixed seed (token counts that are not multiples of anything, 1..40 experts of which
some may be empty, 1..4 slots, dimensions that are multiples of 8 but of no tile size, all three element
types, every routing recipe) so that a tiling assumption that only holds for "nice" sizes has somewhere
to fail.  Tolerances as everywhere: 1e-5 for fp32, 2e-2 for bf16 / fp16.
"""
import random

import pytest
import torch

from _util import TOL, assert_close, gen, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16


def _problems(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        E = rnd.choice([1, 2, 3, 5, 8, 13, 32, 40])
        k = rnd.randint(1, min(4, E))
        T = rnd.choice([1, 5, 63, 64, 65, 127, 129, 257, 700, 1025, 2999])
        d_in = 8 * rnd.randint(1, 65)
        d_out = 8 * rnd.randint(1, 65)
        dtype = rnd.choice([F32, BF16, F16])
        skew = rnd.choice([None, "zipf", "one"]) if E >= k + 2 else None
        out.append((i, T, d_in, d_out, E, k, dtype, skew))
    return out


@pytest.mark.parametrize("i,T,d_in,d_out,E,k,dtype,skew", _problems(40, 20261125),
                         ids=lambda v: str(v).replace("torch.", ""))
def test_random_problem(dev, i, T, d_in, d_out, E, k, dtype, skew):
    from hexa_moe import _lib, ops
    print(f"problem {i}: T={T} in={d_in} out={d_out} E={E} k={k} {dtype} {skew}", flush=True)
    g = gen(1000 + i)
    routing = make_routing(T, E, k, seed=2000 + i, skew=skew, empty=1 if skew == "zipf" else 0)
    counts, offsets, token_ids = O.route_build(routing, E)
    route = ops.route_build(routing.to(dev), E)
    assert torch.equal(route.counts.cpu(), counts) and torch.equal(route.token_ids.cpu(), token_ids)
    rd = torch.float64 if dtype == F32 else torch.float32
    tol = TOL[dtype]
    x = torch.randn(T, d_in, generator=g).to(dtype)
    xs = torch.randn(k, T, d_in, generator=g).to(dtype)
    W = ((torch.rand(E, d_in, d_out, generator=g) * 2 - 1) / d_in ** 0.5).to(dtype)
    b = (torch.rand(E, d_out, generator=g) - 0.5).to(dtype)
    # ESMM, both slot layouts, both weight layouts
    y = ops.esmm(x.to(dev), W.to(dev), b.to(dev), route, False, _lib.HEXA_W_IN_OUT)
    assert_close(y, O.esmm(x.to(rd), W.to(rd), b.to(rd), token_ids, offsets, False), tol, "esmm per-slot result")
    ys = ops.esmm(xs.to(dev), W.transpose(1, 2).contiguous().to(dev), None, route, True, _lib.HEXA_W_OUT_IN)
    assert_close(ys, O.esmm(xs.to(rd), W.to(rd), None, token_ids, offsets, True), tol, "esmm summed over slots")
    # ESTMM and ESS, both layouts of dy
    dy = torch.randn(k, T, d_out, generator=g).to(dtype)
    dw = ops.estmm(dy.to(dev), x.to(dev), route, True, False)
    assert_close(dw, O.estmm(dy.to(rd), x.to(rd), token_ids, offsets, True, E), tol, "estmm")
    db = ops.ess(dy.to(dev), route, True)
    assert_close(db, O.ess(dy.to(rd), token_ids, offsets, True, E), tol, "ess per-slot dy")
    dy_shared = torch.randn(T, d_out, generator=g).to(dtype)
    db2 = ops.ess(dy_shared.to(dev), route, False)
    assert_close(db2, O.ess(dy_shared.to(rd), token_ids, offsets, False, E), tol, "ess shared dy")
    dw2 = ops.estmm(dy_shared.to(dev), xs.to(dev), route, False, True)
    assert_close(dw2, O.estmm(dy_shared.to(rd), xs.to(rd), token_ids, offsets, False, E), tol, "estmm shared dy")
    # the fused GELU' + bias-gradient call
    y1 = torch.randn(k, T, d_out, generator=g).to(dtype)
    t = y1.to(rd)
    pre = O.esmm(x.to(rd), W.to(rd), None, token_ids, offsets, False)
    want = pre * (0.5 * (1 + torch.erf(t / 2 ** 0.5)) + t * torch.exp(-0.5 * t * t) / (2 * torch.pi) ** 0.5)
    got, dbg = ops.esmm_gelu_bwd_ess(x.to(dev), W.to(dev), route, _lib.HEXA_W_IN_OUT, y1.to(dev))
    torch.cuda.synchronize()
    assert_close(got, want, tol, "gelu' product")
    assert_close(dbg, O.ess(want, token_ids, offsets, True, E), tol, "its bias gradient")
    empty = counts.sum(0) == 0
    if empty.any():
        for name, t_ in (("dw", dw), ("db", db), ("dbg", dbg)):
            assert float(t_.cpu()[empty].abs().max()) == 0.0, name
