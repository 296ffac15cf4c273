"""Routing segment pass on the GPU vs the CPU oracle: bit-exact counts, offsets and token lists."""
import numpy as np
import pytest
import torch

from _util import make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu

CASES = [
    # T, E, k, skew, empty
    (1, 1, 1, None, 0),
    (7, 3, 1, None, 0),
    (64, 8, 2, None, 0),
    (513, 5, 3, None, 0),
    (2048, 8, 1, None, 0),
    (4608, 32, 1, None, 0),
    (18432, 32, 2, None, 0),
    (4099, 64, 2, "zipf", 6),
    (32768, 64, 2, "zipf", 4),
    (1000, 16, 2, "one", 0),
    (3000, 300, 2, None, 0),
    (70000, 16, 2, None, 0),
    (65536, 256, 1, "zipf", 20),
]


@pytest.fixture(params=[0, 1, 3], ids=["auto", "one_launch", "three_launches"])
def route_kernels(request):
    """The pass runs as one launch for small token counts, else as a histogram launch and one that scans and
    scatters (up to 256 experts), else as three; every case runs under the automatic choice, with one launch forced
    (it covers up to 65536 tokens and 256 experts; beyond that the two- or three-launch form runs) and with three
    forced."""
    from hexa_moe import _lib
    lib = _lib.load()
    _lib.check(lib.hexa_set_option(b"route_kernels", request.param), "hexa_set_option")
    yield request.param
    _lib.check(lib.hexa_set_option(b"route_kernels", 0), "hexa_set_option")


@pytest.mark.parametrize("T,E,k,skew,empty", CASES)
@pytest.mark.parametrize("as_i64", [False, True])
def test_route_build_matches_oracle(dev, route_kernels, T, E, k, skew, empty, as_i64):
    from hexa_moe import ops
    print(f"case T={T} E={E} k={k} skew={skew} i64={as_i64} route_kernels={route_kernels}", flush=True)
    routing = make_routing(T, E, k, seed=100 + T + E, skew=skew, empty=empty)
    counts, offsets, token_ids = O.route_build(routing, E)
    r = routing if as_i64 else routing.to(torch.int32)
    route = ops.route_build(r.to(dev), E)
    torch.cuda.synchronize()
    assert torch.equal(route.counts.cpu(), counts)
    assert torch.equal(route.offsets.cpu(), offsets)
    assert torch.equal(route.token_ids.cpu(), token_ids)
    # expert of every list position, and the row-tile records the matmul kernels walk
    exp = route.expert_ids.cpu()
    tiles = route.tile_info.cpu()
    ntile = route.tile_count.cpu()
    for s in range(k):
        assert torch.equal(exp[s], routing[token_ids[s].long(), s].to(torch.int32))
        want = []
        for e in range(E):
            c, o = int(counts[s, e]), int(offsets[s, e])
            for j in range(0, c, 128):
                want.append((e, o + j, min(128, c - j), 0))
        assert int(ntile[s]) == len(want)
        got = [tuple(int(v) for v in row) for row in tiles[s, :len(want)]]
        assert got == want
        want_l = []
        for e in range(E):
            c, o = int(counts[s, e]), int(offsets[s, e])
            for j in range(0, c, 256):
                want_l.append((e, o + j, min(256, c - j), 0))
        assert int(route.tile_count_l[s]) == len(want_l)
        assert [tuple(int(v) for v in row) for row in route.tile_info_l.cpu()[s, :len(want_l)]] == want_l
    if skew == "zipf":
        assert int((counts.sum(0) == 0).sum()) >= empty


def test_route_transposed_slots_and_noncontiguous(dev):
    """k contiguous slot vectors ([k,T] storage) give the same lists as [T,k] storage."""
    from hexa_moe import ops
    routing = make_routing(3000, 16, 2, seed=5)
    a = ops.route_build(routing.to(dev), 16)
    b = ops.route_build(routing.t().contiguous().to(dev).t(), 16)
    torch.cuda.synchronize()
    assert torch.equal(a.token_ids, b.token_ids) and torch.equal(a.offsets, b.offsets)


def test_route_out_of_range_ids_are_skipped(dev):
    from hexa_moe import ops
    routing = make_routing(1000, 8, 1, seed=6).to(torch.int32)
    routing[::7, 0] = 8
    routing[3::11, 0] = -1
    keep = ((routing[:, 0] >= 0) & (routing[:, 0] < 8)).nonzero().flatten()
    route = ops.route_build(routing.to(dev), 8)
    torch.cuda.synchronize()
    n = int(route.offsets[0, 8])
    assert n == keep.numel()
    want = keep[torch.sort(routing[keep, 0], stable=True).indices].to(torch.int32)
    assert torch.equal(route.token_ids[0, :n].cpu(), want)


@pytest.mark.parametrize("pad", [1, 16])
def test_legacy_count_assign(dev, pad):
    """TOKEN_COUNT / TOKEN_ASSIGN one to one, including the reference's 16-padded format."""
    import hexa_moe_cuda
    from oracle import route_oracle as RO
    T, E = 5000, 32
    routing = make_routing(T, E, 1, seed=9, skew="zipf", empty=3)[:, 0].to(torch.int32)
    c_ref, x_ref = RO.token_count(routing.numpy(), E, pad)
    t_ref, e_ref = RO.token_assign(routing.numpy(), E, x_ref)
    r = routing.to(dev)
    cnt = torch.zeros(E, dtype=torch.int32, device=dev)
    expd = torch.zeros(E + 1, dtype=torch.int32, device=dev)
    hexa_moe_cuda.set_pad(pad)
    try:
        hexa_moe_cuda.TOKEN_COUNT(cnt, expd, r, T, E)
        P = int(expd[-1].item())
        tok = torch.zeros(P, dtype=torch.int32, device=dev) - 1
        exp = torch.zeros(P, dtype=torch.int32, device=dev) - 1
        hexa_moe_cuda.TOKEN_ASSIGN(tok, exp, expd, r, T, E)
    finally:
        hexa_moe_cuda.set_pad(1)
    torch.cuda.synchronize()
    assert np.array_equal(cnt.cpu().numpy(), c_ref)
    assert np.array_equal(expd.cpu().numpy(), x_ref)
    assert np.array_equal(tok.cpu().numpy(), t_ref)
    assert np.array_equal(exp.cpu().numpy(), e_ref)


@pytest.mark.parametrize("T,E,k,skew,empty", [(5000, 32, 2, "zipf", 3), (777, 5, 3, None, 0), (18432, 32, 2, None, 0)])
def test_route_from_padded_lists(dev, T, E, k, skew, empty):
    """The reference's list format (segments padded to 16 with -1, slots concatenated, cumulative
    lengths in a device array) gives the same route as the routing decision itself.  The lists are
    written by the C oracle; within a segment they are then permuted with a seeded shuffle, since the
    reference's order inside a segment is whatever its atomics produced."""
    from hexa_moe import ops
    from oracle import route_oracle as RO
    print(f"padded lists T={T} E={E} k={k} skew={skew}", flush=True)
    routing = make_routing(T, E, k, seed=300 + T, skew=skew, empty=empty).to(torch.int32)
    rng = np.random.default_rng(T)
    toks, exps, ends = [], [], [0]
    for s in range(k):
        r = routing[:, s].contiguous().numpy()
        _, x_ref = RO.token_count(r, E, 16)
        t_ref, e_ref = RO.token_assign(r, E, x_ref)
        toks.append(t_ref); exps.append(e_ref); ends.append(ends[-1] + len(t_ref))
    tok = torch.from_numpy(np.concatenate(toks)).to(dev)
    exp = torch.from_numpy(np.concatenate(exps)).to(dev)
    cum = torch.tensor(ends, dtype=torch.int32, device=dev)
    want = ops.route_build(routing.to(dev), E)
    got = ops.route_from_padded_lists(tok, exp, cum, T, k, E)
    torch.cuda.synchronize()
    for name in ("counts", "offsets", "token_ids", "expert_ids", "tile_count", "tile_count_l"):
        assert torch.equal(getattr(got, name), getattr(want, name)), name
    for s in range(k):
        n, nl = int(want.tile_count[s]), int(want.tile_count_l[s])
        assert torch.equal(got.tile_info[s, :n], want.tile_info[s, :n])
        assert torch.equal(got.tile_info_l[s, :nl], want.tile_info_l[s, :nl])
    # shuffled inside each segment: same counts and offsets, each segment the same set of tokens
    counts, offsets, _ = O.route_build(routing.long(), E)
    shuf = [t.copy() for t in toks]
    for s in range(k):
        _, x_ref = RO.token_count(routing[:, s].contiguous().numpy(), E, 16)
        for e in range(E):
            a, c = int(x_ref[e]), int(counts[s, e])
            rng.shuffle(shuf[s][a:a + c])
    got2 = ops.route_from_padded_lists(torch.from_numpy(np.concatenate(shuf)).to(dev), exp, cum, T, k, E)
    torch.cuda.synchronize()
    assert torch.equal(got2.counts.cpu(), counts) and torch.equal(got2.offsets.cpu(), offsets)
    ids = got2.token_ids.cpu()
    for s in range(k):
        for e in range(E):
            a, b = int(offsets[s, e]), int(offsets[s, e + 1])
            assert torch.equal(torch.sort(ids[s, a:b]).values, want.token_ids[s, a:b].cpu())
