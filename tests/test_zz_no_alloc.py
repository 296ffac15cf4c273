"""hexa_ess_noalloc (the entry point that allocates nothing: its partial sums live in an array built into the
library) against hexa_ess with caller scratch, through the C ABI: bit-identical results, on two calls in a
row of which the second is smaller (the built-in array keeps the first call's contents), and against the
CPU oracle.  Sizes beyond the built-in array are rejected with an error code."""
import pytest
import torch

from _util import TOL, assert_close, gen, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu

DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _ess_pair(dev, T, d_out, E, k, per_slot, dtype, seed):
    """db from hexa_ess (caller scratch of 8*E*out floats) and from hexa_ess_noalloc, plus the oracle's."""
    from hexa_moe import _lib, ops
    lib = _lib.load()
    g = gen(seed)
    routing = make_routing(T, E, k, seed=seed + 1, skew="zipf", empty=1)
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn((k, T, d_out) if per_slot else (T, d_out), generator=g).to(dtype)
    want = O.ess(dy.to(torch.float64 if dtype == torch.float32 else torch.float32), token_ids, offsets, per_slot, E)
    route = ops.route_build(routing.to(dev), E)
    dyd = dy.to(dev)
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(8 * E * d_out, dtype=torch.float32, device=dev)
    a = torch.full((E, d_out), float("nan"), dtype=torch.float32, device=dev)
    b = torch.full((E, d_out), float("nan"), dtype=torch.float32, device=dev)
    print(f"ess_noalloc T={T} out={d_out} E={E} k={k} per_slot={per_slot} {dtype}", flush=True)
    _lib.check(lib.hexa_ess(a.data_ptr(), dyd.data_ptr(), route.blob.data_ptr(), int(per_slot), 0, T, k, d_out, E,
                            DT[dtype], 0, ws.data_ptr(), ws.numel(), st), "hexa_ess")
    _lib.check(lib.hexa_ess_noalloc(b.data_ptr(), dyd.data_ptr(), route.blob.data_ptr(), int(per_slot), 0, T, k, d_out,
                                    E, DT[dtype], 0, st), "hexa_ess_noalloc")
    torch.cuda.synchronize()
    return a, b, want


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_noalloc_matches_ess_twice_second_smaller(dev, dtype):
    # first call: long lists (split walk through the built-in array); second: fewer tokens, experts and columns
    for T, d_out, E, k, per_slot, seed in [(9000, 264, 8, 2, True, 301), (4100, 72, 5, 2, False, 311)]:
        a, b, want = _ess_pair(dev, T, d_out, E, k, per_slot, dtype, seed)
        assert torch.equal(a, b), "hexa_ess_noalloc differs from hexa_ess"
        assert_close(b, want, TOL[dtype], "ess_noalloc vs oracle")


def test_noalloc_short_lists_and_accumulate(dev):
    """Lists too short for the split walk (one pass, no scratch), and accumulate into an existing result."""
    from hexa_moe import _lib, ops
    lib = _lib.load()
    a, b, want = _ess_pair(dev, 300, 40, 6, 2, True, torch.bfloat16, 321)
    assert torch.equal(a, b)
    assert_close(b, want, TOL[torch.bfloat16], "short lists")
    T, d_out, E, k = 5000, 128, 4, 1
    g = gen(331)
    routing = make_routing(T, E, k, seed=332)
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn(T, d_out, generator=g)
    base = torch.randn(E, d_out, generator=g)
    route = ops.route_build(routing.to(dev), E)
    out = base.clone().to(dev)
    dyd = dy.to(dev)
    _lib.check(lib.hexa_ess_noalloc(out.data_ptr(), dyd.data_ptr(), route.blob.data_ptr(), 0, 1, T, k, d_out, E, 0, 0,
                                    torch.cuda.current_stream().cuda_stream), "hexa_ess_noalloc")
    torch.cuda.synchronize()
    assert_close(out, O.ess(dy.double(), token_ids, offsets, False, E) + base.double(), 1e-5, "accumulate")


def test_noalloc_rejects_sizes_beyond_the_builtin_scratch(dev):
    from hexa_moe import _lib, ops
    lib = _lib.load()
    E, d_out, T = 64, 8192, 64            # 8*E*out = 4 Mi floats > 2 Mi
    routing = make_routing(T, E, 1, seed=5)
    route = ops.route_build(routing.to(dev), E)
    dy = torch.zeros(T, d_out, device=dev)
    db = torch.zeros(E, d_out, device=dev)
    rc = lib.hexa_ess_noalloc(db.data_ptr(), dy.data_ptr(), route.blob.data_ptr(), 0, 0, T, 1, d_out, E, 0, 0,
                              torch.cuda.current_stream().cuda_stream)
    assert rc == -2 and b"built-in scratch" in lib.hexa_last_error()


def test_noalloc_allocates_nothing(dev):
    """The property the entry point exists for: after a warm call, further calls leave the device's free memory
    as it was (hipMemGetInfo through torch: neither the library nor the runtime took or returned a byte)."""
    from hexa_moe import _lib, ops
    lib = _lib.load()
    T, d_out, E, k = 9000, 264, 8, 2
    routing = make_routing(T, E, k, seed=341, skew="zipf")
    route = ops.route_build(routing.to(dev), E)
    dy = torch.randn(k, T, d_out, device=dev, dtype=torch.bfloat16)
    db = torch.zeros(E, d_out, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    call = lambda: lib.hexa_ess_noalloc(db.data_ptr(), dy.data_ptr(), route.blob.data_ptr(), 1, 0, T, k, d_out, E,  # noqa: E731
                                        DT[torch.bfloat16], 0, st)
    assert call() == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(5):
        assert call() == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_reserved() == reserved0
