"""The persistent ESTMM kernel (option estmm_pipe = 1: one workgroup per CU takes (expert, 128 x 128 block) items from
a queue) against the CPU oracle and against the one-item-per-workgroup kernel: ragged and empty experts, every
token on one expert (the plan then cuts that expert's list into parts whose fp32 partial results the fix-up task
adds), one to three routing slots, either operand per slot, 16-bit and fp32 results, accumulation, and a result
that does not depend on which workgroup took which item (two runs are bit-identical; the queue's counters are back
at zero after every launch)."""
import pytest
import torch

from _util import TOL, assert_close, gen, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu
BF, HF, F32 = torch.bfloat16, torch.float16, torch.float32

CASES = [
    # T, M, N, E, k, dtype, skew, empty, out dtype, (dy per slot, x per slot), accumulate
    (2300, 128, 128, 6, 2, BF, None, 0, F32, (True, False), False),
    (2300, 192, 392, 6, 2, BF, "zipf", 1, F32, (True, False), False),
    (1700, 256, 320, 6, 2, HF, "zipf", 1, HF, (True, False), False),
    (900, 136, 72, 5, 1, BF, None, 0, BF, (True, False), False),
    (5000, 384, 128, 4, 3, BF, "one", 0, F32, (True, False), False),       # one expert holds everything: cut into parts
    (5000, 256, 128, 4, 3, BF, "one", 0, BF, (True, False), True),
    (3000, 256, 256, 8, 2, BF, None, 0, F32, (False, True), False),
    (3000, 256, 256, 8, 2, BF, None, 0, F32, (True, False), True),
    (3000, 256, 256, 8, 2, HF, None, 0, HF, (True, False), True),
    (37, 8, 8, 3, 1, BF, None, 0, F32, (True, False), False),
    (6000, 640, 384, 40, 2, BF, "zipf", 4, BF, (True, False), False),
]


@pytest.fixture
def pipe_knob():
    from hexa_moe import _lib
    lib = _lib.load()
    yield lambda v: _lib.check(lib.hexa_set_option(b"estmm_pipe", int(v)), "hexa_set_option")
    lib.hexa_set_option(b"estmm_pipe", 0)


@pytest.mark.parametrize("T,M,N,E,k,dtype,skew,empty,out_dtype,per_slot,acc", CASES)
def test_persistent_estmm(dev, pipe_knob, T, M, N, E, k, dtype, skew, empty, out_dtype, per_slot, acc):
    from hexa_moe import _lib, ops
    print(f"estmm_pipe T={T} M={M} N={N} E={E} k={k} {dtype} skew={skew} out={out_dtype} per_slot={per_slot} acc={acc}", flush=True)
    g = gen(T + M)
    routing = make_routing(T, E, k, seed=T + 1, skew=skew, empty=empty)
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn((k, T, M) if per_slot[0] else (T, M), generator=g).to(dtype)
    x = torch.randn((k, T, N) if per_slot[1] else (T, N), generator=g).to(dtype)
    want = O.estmm(dy.float(), x.float(), token_ids, offsets, per_slot[0], E)
    base = torch.randn(E, M, N, generator=g).to(out_dtype) if acc else None
    if acc:
        want = want + base.float()
    route = ops.route_build(routing.to(dev), E)

    def run(knob):
        pipe_knob(knob)
        out = base.clone().to(dev) if acc else None
        return ops.estmm(dy.to(dev), x.to(dev), route, per_slot[0], per_slot[1], out=out, out_dtype=out_dtype, accumulate=acc)

    got = run(1)
    plan = next(iter(route._plans.values()))
    torch.cuda.synchronize()
    tol = TOL[dtype] if out_dtype != F32 else max(TOL[dtype] / 100, 1e-4)
    assert_close(got, want, tol, "persistent estmm vs oracle")
    # the queue (behind the plan's 4E + 1 ints) is left at zero for the next launch
    assert int(plan[4 * E + 1:4 * E + 17].abs().sum()) == 0
    again = run(1)
    assert torch.equal(got, again), "two runs differ"
    other = run(0)
    # same products, another order of the fp32 sums: equal to rounding
    assert_close(got, other.float(), 1e-5 if out_dtype == F32 else TOL[dtype], "persistent vs one-item-per-workgroup kernel")
    empty_e = (route.counts.sum(0) == 0).cpu()
    if empty_e.any() and not acc:
        assert float(got[empty_e.to(dev)].abs().max()) == 0.0
