"""ESMM / ESTMM / ESS / fused backward on the GPU (through the C ABI) vs the CPU oracle.

Tolerances: rel-err 1e-5 for fp32, 2e-2 for bf16 / fp16 (fp32 accumulation), measured both over the
whole tensor (Frobenius) and on the worst element against the largest reference magnitude.  Inputs are
rounded to the tested type first; the oracle runs in fp32 (fp64 for the fp32 cases) on those values.
"""
import pytest
import torch

from _util import TOL, assert_close, gen, make_linear, make_routing
from oracle import hexa_oracle as O

pytestmark = pytest.mark.gpu

F32, BF16, F16 = torch.float32, torch.bfloat16, torch.float16


def _ref_dtype(dtype):
    return torch.float64 if dtype == F32 else torch.float32


SHAPES = [
    # T, d_in, d_out, E, k, skew
    (37, 8, 8, 3, 1, None),
    (300, 64, 136, 5, 2, None),
    (1000, 384, 256, 8, 2, None),
    (700, 200, 72, 4, 1, "one"),
    (2048, 128, 512, 8, 1, None),
    (900, 320, 136, 6, 1, None),      # one slot, a contraction the pipelined kernel takes (also when accumulating)
    (1500, 264, 392, 16, 2, "zipf"),
    (1100, 512, 384, 8, 2, None),     # a 384-wide result: one tile spans it
    (900, 96, 328, 5, 2, "zipf"),
    (500, 64, 72, 16, 8, None),       # eight slots: the most the fast path's slot tables hold
    (300, 32, 40, 12, 9, None),       # nine: the general kernels take over where the tables end
]


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("m2s", [False, True])
@pytest.mark.parametrize("layout", ["in_out", "out_in"])
@pytest.mark.parametrize("T,d_in,d_out,E,k,skew", SHAPES)
def test_esmm(dev, dtype, m2s, layout, T, d_in, d_out, E, k, skew):
    from hexa_moe import _lib, ops
    print(f"esmm {dtype} m2s={m2s} {layout} T={T} in={d_in} out={d_out} E={E} k={k} {skew}", flush=True)
    routing = make_routing(T, E, k, seed=T + E, skew=skew, empty=2 if skew == "zipf" else 0)
    x, W, b = make_linear(T, d_in, d_out, E, k, seed=d_in + d_out, dtype=dtype, m2s=m2s)
    _, offsets, token_ids = O.route_build(routing, E)
    rd = _ref_dtype(dtype)
    want = O.esmm(x.to(rd), W.to(rd), b.to(rd), token_ids, offsets, m2s)
    route = ops.route_build(routing.to(dev), E)
    Wd = W.to(dev) if layout == "in_out" else W.transpose(1, 2).contiguous().to(dev)
    lay = _lib.HEXA_W_IN_OUT if layout == "in_out" else _lib.HEXA_W_OUT_IN
    got = ops.esmm(x.to(dev), Wd, b.to(dev), route, m2s, lay)
    torch.cuda.synchronize()
    assert got.dtype == dtype
    assert_close(got, want, TOL[dtype], "esmm")
    # no bias, and accumulation into an existing result
    want_nb = O.esmm(x.to(rd), W.to(rd), None, token_ids, offsets, m2s)
    base = torch.randn(want.shape, generator=gen(1)).to(dtype)
    out = base.clone().to(dev)
    ops.esmm(x.to(dev), Wd, None, route, m2s, lay, out=out, accumulate=True)
    torch.cuda.synchronize()
    assert_close(out, want_nb + base.to(rd), TOL[dtype], "esmm accumulate")


@pytest.mark.parametrize("dtype", [BF16, F16])
@pytest.mark.parametrize("layout", ["in_out", "out_in"])
def test_esmm_fp32_weights_and_fp32_result(dev, dtype, layout):
    """'mix' of the reference: 16-bit tokens, fp32 weights and bias; also an fp32 result buffer."""
    from hexa_moe import _lib, ops
    T, d_in, d_out, E, k = 900, 128, 264, 6, 2
    routing = make_routing(T, E, k, seed=3)
    x, W, b = make_linear(T, d_in, d_out, E, k, seed=4, dtype=F32, m2s=False)
    x = x.to(dtype)
    _, offsets, token_ids = O.route_build(routing, E)
    # the kernel rounds the fp32 weights to the tokens' type; the oracle sees the rounded values
    want = O.esmm(x.float(), W.to(dtype).float(), b, token_ids, offsets, False)
    route = ops.route_build(routing.to(dev), E)
    Wd = W.to(dev) if layout == "in_out" else W.transpose(1, 2).contiguous().to(dev)
    lay = _lib.HEXA_W_IN_OUT if layout == "in_out" else _lib.HEXA_W_OUT_IN
    got = ops.esmm(x.to(dev), Wd, b.to(dev), route, False, lay, out_dtype=F32)
    torch.cuda.synchronize()
    assert got.dtype == F32
    assert_close(got, want, 1e-5, "esmm mix, fp32 result")
    got16 = ops.esmm(x.to(dev), Wd, b.to(dev), route, False, lay)
    torch.cuda.synchronize()
    assert_close(got16, want, TOL[dtype], "esmm mix")


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
def test_esmm_fused_gelu(dev, dtype):
    from hexa_moe import _lib, ops
    T, d_in, d_out, E, k = 640, 96, 200, 4, 2
    routing = make_routing(T, E, k, seed=8)
    x, W, b = make_linear(T, d_in, d_out, E, k, seed=9, dtype=dtype, m2s=False)
    _, offsets, token_ids = O.route_build(routing, E)
    rd = _ref_dtype(dtype)
    want = O.esmm(x.to(rd), W.to(rd), b.to(rd), token_ids, offsets, False)
    route = ops.route_build(routing.to(dev), E)
    y1, y2 = ops.esmm(x.to(dev), W.to(dev), b.to(dev), route, False, _lib.HEXA_W_IN_OUT, gelu=True)
    torch.cuda.synchronize()
    assert_close(y1, want, TOL[dtype], "pre-activation")
    assert_close(y2, torch.nn.functional.gelu(want), TOL[dtype], "gelu")


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("m2s", [False, True])
@pytest.mark.parametrize("T,d_in,d_out,E,k,skew", SHAPES)
def test_fused_grad(dev, dtype, m2s, T, d_in, d_out, E, k, skew):
    """ESMM-bwd + ESTMM + ESS in the reference's FUSED_GRAD layout, fp32 results."""
    from hexa_moe import _lib, ops
    print(f"fused_grad {dtype} m2s={m2s} T={T} in={d_in} out={d_out} E={E} k={k} {skew}", flush=True)
    g = gen(T + d_in)
    routing = make_routing(T, E, k, seed=T + E + 1, skew=skew, empty=2 if skew == "zipf" else 0)
    _, offsets, token_ids = O.route_build(routing, E)
    jy = torch.randn((k, T, d_out) if m2s else (T, d_out), generator=g).to(dtype)
    x = torch.randn((T, d_in) if m2s else (k, T, d_in), generator=g).to(dtype)
    w = ((torch.rand(E, d_out, d_in, generator=g) * 2 - 1) / d_out ** 0.5).to(dtype)
    rd = _ref_dtype(dtype)
    jb_ref, jx_ref, jw_ref = O.fused_grad(jy.to(rd), w.to(rd), x.to(rd), token_ids, offsets, m2s, True)
    route = ops.route_build(routing.to(dev), E)
    jb = torch.zeros(E, d_out, dtype=F32, device=dev)
    jx = torch.zeros(jx_ref.shape, dtype=F32, device=dev)
    jw = torch.zeros(E, d_out, d_in, dtype=F32, device=dev)
    jy_d, w_d, x_d = jy.to(dev), w.to(dev), x.to(dev)  # kept alive: only raw pointers cross the C ABI
    rc = _lib.load().hexa_fused_grad(jb.data_ptr(), jx.data_ptr(), jw.data_ptr(), jy_d.data_ptr(),
                                     w_d.data_ptr(), x_d.data_ptr(), route.blob.data_ptr(), int(m2s), 1,
                                     T, k, d_in, d_out, E, ops._dt(jy), ops._dt(w), 0, 0, 0, None,
                                     None, 0, None, None, 0, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "hexa_fused_grad")
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert_close(jx, jx_ref, tol, "j_x")
    assert_close(jw, jw_ref, tol, "j_w")
    assert_close(jb, jb_ref, tol, "j_b")
    # experts without tokens get exact zeros from the non-accumulating operators
    dw = ops.estmm(jy.to(dev), x.to(dev), route, m2s, not m2s)
    db = ops.ess(jy.to(dev), route, m2s)
    torch.cuda.synchronize()
    empty = (route.counts.sum(0) == 0).cpu()
    assert_close(dw, jw_ref, tol, "estmm")
    assert_close(db, jb_ref, tol, "ess")
    if empty.any():
        assert float(dw.cpu()[empty].abs().max()) == 0.0 and float(db.cpu()[empty].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [BF16, F16])
def test_estmm_16bit_result(dev, dtype):
    from hexa_moe import ops
    T, d_in, d_out, E, k = 800, 136, 264, 6, 2
    g = gen(77)
    routing = make_routing(T, E, k, seed=78)
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn(k, T, d_out, generator=g).to(dtype)
    x = torch.randn(T, d_in, generator=g).to(dtype)
    want = O.estmm(dy.float(), x.float(), token_ids, offsets, True, E)
    route = ops.route_build(routing.to(dev), E)
    got = ops.estmm(dy.to(dev), x.to(dev), route, True, False, out_dtype=dtype)
    db = ops.ess(dy.to(dev), route, True, out_dtype=dtype)
    torch.cuda.synchronize()
    assert got.dtype == dtype
    assert_close(got, want, TOL[dtype], "estmm 16-bit result")
    assert_close(db, O.ess(dy.float(), token_ids, offsets, True, E), TOL[dtype], "ess 16-bit result")


def test_estmm_many_cut_experts(dev):
    """More than 64 experts whose lists the plan cuts (70 of 1000 experts hold every token): the fix-up task finds
    the j-th cut expert of the plan beyond the first 64 ranks, and workgroups past the last cut expert do nothing."""
    from hexa_moe import ops
    E, busy, rows, M, N = 1000, 70, 1900, 64, 64
    T = busy * rows
    g = gen(311)
    experts = torch.randperm(E, generator=g)[:busy]
    routing = experts[torch.randint(0, busy, (T, 1), generator=g)]
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn(1, T, M, generator=g).to(BF16)
    x = torch.randn(T, N, generator=g).to(BF16)
    want = O.estmm(dy.float(), x.float(), token_ids, offsets, True, E)
    route = ops.route_build(routing.to(dev), E)
    got = ops.estmm(dy.to(dev), x.to(dev), route, True, False)
    plan = next(iter(route._plans.values())).cpu()
    assert int((plan[E:2 * E] > 1).sum()) == busy, "every busy expert's list is cut"
    again = ops.estmm(dy.to(dev), x.to(dev), route, True, False)
    torch.cuda.synchronize()
    assert_close(got, want, 1e-4, "estmm with 70 cut experts")
    assert torch.equal(got, again)
    idle = torch.ones(E, dtype=torch.bool)
    idle[experts] = False
    assert float(got[idle.to(dev)].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("per_slot", [False, True])
def test_ess_long_lists(dev, dtype, per_slot):
    """Token lists long enough for the split walk (partial sums through scratch, folded in order)."""
    from hexa_moe import ops
    T, d_out, E, k = 6000, 200, 8, 2
    g = gen(91)
    routing = make_routing(T, E, k, seed=92, skew="zipf", empty=1)
    _, offsets, token_ids = O.route_build(routing, E)
    dy = torch.randn((k, T, d_out) if per_slot else (T, d_out), generator=g).to(dtype)
    rd = _ref_dtype(dtype)
    want = O.ess(dy.to(rd), token_ids, offsets, per_slot, E)
    route = ops.route_build(routing.to(dev), E)
    got = ops.ess(dy.to(dev), route, per_slot)
    again = ops.ess(dy.to(dev), route, per_slot)
    torch.cuda.synchronize()
    assert_close(got, want, TOL[dtype], "ess")
    assert torch.equal(got, again)
    base = torch.randn(E, d_out, generator=g)
    out = base.clone().to(dev)
    ops.ess(dy.to(dev), route, per_slot, out=out, accumulate=True)
    torch.cuda.synchronize()
    assert_close(out, want + base.to(rd), TOL[dtype], "ess accumulate")


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
def test_gelu_bwd(dev, dtype):
    from hexa_moe import ops
    g = gen(5)
    y1 = (torch.randn(3, 1001, 40, generator=g) * 2).to(dtype)
    dy2 = torch.randn(3, 1001, 40, generator=g).to(dtype)
    yr = y1.double().requires_grad_(True)
    (want,) = torch.autograd.grad(torch.nn.functional.gelu(yr), yr, dy2.double())
    got = ops.gelu_bwd(dy2.to(dev), y1.to(dev))
    torch.cuda.synchronize()
    assert_close(got, want, 2e-6 if dtype == F32 else TOL[dtype], "gelu_bwd")


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("d_in,d_out", [(96, 200), (200, 96), (384, 1536)])
def test_esmm_fused_gelu_bwd(dev, dtype, d_in, d_out):
    """dy1 = (dy . W^T) * gelu'(y1) in one ESMM (weights stored [E, out, in] as in the backward)."""
    from hexa_moe import _lib, ops
    T, E, k = 900, 6, 2
    g = gen(d_in)
    routing = make_routing(T, E, k, seed=31)
    x, W, _ = make_linear(T, d_in, d_out, E, k, seed=32, dtype=dtype, m2s=False)
    y1 = (torch.randn(k, T, d_out, generator=g) * 2).to(dtype)
    _, offsets, token_ids = O.route_build(routing, E)
    rd = _ref_dtype(dtype)
    lin = O.esmm(x.to(rd), W.to(rd), None, token_ids, offsets, False)
    yr = y1.double().requires_grad_(True)
    (want,) = torch.autograd.grad(torch.nn.functional.gelu(yr), yr, lin.double())
    route = ops.route_build(routing.to(dev), E)
    for lay, Wd in ((_lib.HEXA_W_OUT_IN, W.transpose(1, 2).contiguous()), (_lib.HEXA_W_IN_OUT, W)):
        got = ops.esmm(x.to(dev), Wd.to(dev), None, route, False, lay, gelu_bwd_of=y1.to(dev))
        torch.cuda.synchronize()
        assert_close(got, want, TOL[dtype], "esmm * gelu'")


@pytest.mark.parametrize("dtype", [F32, BF16, F16])
@pytest.mark.parametrize("T,d_in,d_out,E,k,skew", [(1100, 96, 200, 5, 2, "zipf"), (2300, 384, 1536, 8, 2, None),
                                                   (700, 64, 136, 4, 1, "one"), (37, 8, 8, 3, 1, None)])
def test_esmm_gelu_bwd_with_bias_gradient(dev, dtype, T, d_in, d_out, E, k, skew):
    """dy1 = (x . W[e]) * gelu'(y1) and db = per-expert row sums of dy1 from one call; the sums must be those
    of the tensor as stored (what ESS of dy1 gives), and both must match the oracle."""
    from hexa_moe import _lib, ops
    print(f"esmm+gelu'+ess {dtype} T={T} in={d_in} out={d_out} E={E} k={k} {skew}", flush=True)
    g = gen(T + d_out)
    routing = make_routing(T, E, k, seed=T + 3, skew=skew, empty=1 if skew == "zipf" else 0)
    _, offsets, token_ids = O.route_build(routing, E)
    x = torch.randn(T, d_in, generator=g).to(dtype)
    W = ((torch.rand(E, d_out, d_in, generator=g) * 2 - 1) / d_in ** 0.5).to(dtype)     # [E,out,in]
    y1 = torch.randn(k, T, d_out, generator=g).to(dtype)
    rd = _ref_dtype(dtype)
    pre = O.esmm(x.to(rd), W.transpose(1, 2).to(rd), None, token_ids, offsets, False)
    t = y1.to(rd)
    want = pre * (0.5 * (1 + torch.erf(t / 2 ** 0.5)) + t * torch.exp(-0.5 * t * t) / (2 * torch.pi) ** 0.5)
    route = ops.route_build(routing.to(dev), E)
    got, db = ops.esmm_gelu_bwd_ess(x.to(dev), W.to(dev), route, _lib.HEXA_W_OUT_IN, y1.to(dev))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert got.dtype == dtype and db.dtype == F32 and db.shape == (E, d_out)
    assert_close(got, want, tol, "dy1")
    assert_close(db, O.ess(want, token_ids, offsets, True, E), tol, "db vs oracle")
    # against the sums of the stored tensor: only the order of the fp32 additions differs
    assert_close(db, O.ess(got.cpu().to(torch.float64), token_ids, offsets, True, E), 1e-5, "db vs stored dy1")
    empty = (route.counts.sum(0) == 0).cpu()
    if empty.any():
        assert float(db.cpu()[empty].abs().max()) == 0.0


@pytest.mark.parametrize("pad", [1, 16])
def test_reference_style_ops(dev, pad):
    """The five operator names of the reference extension, called the way impls/layers.py calls them:
    with exact lists (pad 1) and with the reference's own format, every expert's segment padded to a
    multiple of 16 with -1 and the slots' lists concatenated (pad 16)."""
    import hexa_moe_cuda
    hexa_moe_cuda.set_pad(pad)
    try:
        _reference_style_ops(dev, pad)
    finally:
        hexa_moe_cuda.set_pad(1)


def _reference_style_ops(dev, pad):
    import hexa_moe_cuda
    hexa_moe_cuda.clear_route_cache()
    T, d_in, d_out, E, k = 600, 64, 128, 8, 2
    routing = make_routing(T, E, k, seed=21).to(torch.int32)
    x, W, b = make_linear(T, d_in, d_out, E, k, seed=22, dtype=F32, m2s=False)
    _, offsets, token_ids = O.route_build(routing, E)
    want = O.esmm(x.double(), W.double(), b.double(), token_ids, offsets, False)
    rd = routing.to(dev)
    tpe = torch.zeros(E, dtype=torch.int32, device=dev)
    expd = torch.zeros(E + 1, dtype=torch.int32, device=dev)
    tok_lists, exp_lists = [], []
    for i in range(k):
        tpe.zero_(); expd.zero_()
        hexa_moe_cuda.TOKEN_COUNT(tpe, expd, rd[:, i].contiguous(), T, E)
        n = expd[-1].item()
        tok_lists.append(torch.zeros(n, dtype=torch.int32, device=dev) - 1)
        exp_lists.append(torch.zeros(n, dtype=torch.int32, device=dev) - 1)
        hexa_moe_cuda.TOKEN_ASSIGN(tok_lists[i], exp_lists[i], expd, rd[:, i].contiguous(), T, E)
        assert n % pad == 0 and (n > T) == (pad > 1) and int((tok_lists[i] >= 0).sum()) == T
    cum = torch.zeros(k + 1, dtype=torch.int32, device=dev)
    for i in range(k):
        cum[i + 1] = cum[i] + len(exp_lists[i])
    tok = torch.cat(tok_lists).contiguous()
    exp = torch.cat(exp_lists).contiguous()
    hid = torch.zeros(k, T, d_out, dtype=F32, device=dev)
    hexa_moe_cuda.ESMM_TENSOR_CORE(hid.reshape(-1), x.to(dev).reshape(-1), W.to(dev).reshape(-1), b.to(dev).reshape(-1),
                                   tok, exp, cum, True, True, True, False, T, k, d_in, d_out, E)
    torch.cuda.synchronize()
    assert_close(hid, want, 1e-5, "ESMM_TENSOR_CORE")
    g = gen(23)
    jy = torch.randn(k, T, d_out, generator=g)
    w = W.transpose(1, 2).contiguous()  # [E,out,in]
    jb_ref, jx_ref, jw_ref = O.fused_grad(jy.double(), w.double(), x.double(), token_ids, offsets, True, True)
    jb = torch.zeros(E, d_out, device=dev); jx = torch.zeros(T, d_in, device=dev); jw = torch.zeros(E, d_out, d_in, device=dev)
    hexa_moe_cuda.FUSED_GRAD(jb.reshape(-1), jx.reshape(-1), jw.reshape(-1), jy.to(dev).reshape(-1),
                             w.to(dev).reshape(-1), x.to(dev).reshape(-1), tok, exp, cum, True, True, True, T, k, d_in,
                             d_out, E)
    jx2 = torch.zeros(T, d_in, device=dev); jw2 = torch.zeros(E, d_out, d_in, device=dev)
    hexa_moe_cuda.FUSED_GRAD_NO_BIAS(jx2.reshape(-1), jw2.reshape(-1), jy.to(dev).reshape(-1), w.to(dev).reshape(-1),
                                     x.to(dev).reshape(-1), tok, exp, cum, True, True, True, T, k, d_in, d_out, E)
    torch.cuda.synchronize()
    assert_close(jb, jb_ref, 1e-5, "j_b"); assert_close(jx, jx_ref, 1e-5, "j_x"); assert_close(jw, jw_ref, 1e-5, "j_w")
    assert torch.equal(jx, jx2) and torch.equal(jw, jw2)
    # the three matmul ops shared ONE build of the routing metadata (keyed on the list tensors); 16-bit operands
    # with lists this long also take the balanced ESTMM (a plan made once per routing) and the split ESS walk
    assert len(hexa_moe_cuda._route_cache) == 1
    jb16 = torch.zeros(E, d_out, device=dev); jx16 = torch.zeros(T, d_in, device=dev, dtype=BF16)
    jw16 = torch.zeros(E, d_out, d_in, device=dev)
    hexa_moe_cuda.FUSED_GRAD(jb16.reshape(-1), jx16.reshape(-1), jw16.reshape(-1), jy.to(dev).to(BF16).reshape(-1),
                             w.to(dev).to(BF16).reshape(-1), x.to(dev).to(BF16).reshape(-1), tok, exp, cum, False, False,
                             True, T, k, d_in, d_out, E)
    torch.cuda.synchronize()
    assert len(hexa_moe_cuda._route_cache) == 1
    assert_close(jb16, jb_ref, 2e-2, "j_b bf16"); assert_close(jx16, jx_ref, 2e-2, "j_x bf16"); assert_close(jw16, jw_ref, 2e-2, "j_w bf16")
    # lists rewritten in place (same storage, new version) are not served from the cache
    tok.add_(0)
    jx3 = torch.zeros(T, d_in, device=dev); jw3 = torch.zeros(E, d_out, d_in, device=dev)
    hexa_moe_cuda.FUSED_GRAD_NO_BIAS(jx3.reshape(-1), jw3.reshape(-1), jy.to(dev).reshape(-1), w.to(dev).reshape(-1),
                                     x.to(dev).reshape(-1), tok, exp, cum, True, True, True, T, k, d_in, d_out, E)
    torch.cuda.synchronize()
    assert len(hexa_moe_cuda._route_cache) == 2 and torch.equal(jx3, jx2)
    hexa_moe_cuda.clear_route_cache()


def test_token_assign_into_the_same_lists_rebuilds_the_routing_metadata(dev):
    """A caller that keeps ONE pair of preallocated list tensors (k = 1, so the lists are passed as they are) and
    refills them with TOKEN_ASSIGN for a new routing: the matmul op behind it must see the new routing.  The
    operators write through raw pointers, which leaves the tensors' version counters alone."""
    import hexa_moe_cuda
    hexa_moe_cuda.clear_route_cache()
    T, d_in, d_out, E = 512, 64, 128, 4
    x, W, b = make_linear(T, d_in, d_out, E, 1, seed=31, dtype=F32, m2s=False)
    tok = torch.empty(T, dtype=torch.int32, device=dev)
    exp = torch.empty(T, dtype=torch.int32, device=dev)
    tpe = torch.zeros(E, dtype=torch.int32, device=dev)
    expd = torch.zeros(E + 1, dtype=torch.int32, device=dev)
    cum = torch.tensor([0, T], dtype=torch.int32, device=dev)
    for seed in (41, 42, 43):
        routing = make_routing(T, E, 1, seed=seed).to(torch.int32)
        _, offsets, token_ids = O.route_build(routing, E)
        want = O.esmm(x.double(), W.double(), b.double(), token_ids, offsets, False)
        col = routing[:, 0].contiguous().to(dev)
        hexa_moe_cuda.TOKEN_COUNT(tpe, expd, col, T, E)
        hexa_moe_cuda.TOKEN_ASSIGN(tok, exp, expd, col, T, E)       # same tensors every time, no torch op in between
        hid = torch.zeros(1, T, d_out, dtype=F32, device=dev)
        hexa_moe_cuda.ESMM_TENSOR_CORE(hid.reshape(-1), x.to(dev).reshape(-1), W.to(dev).reshape(-1), b.to(dev).reshape(-1),
                                       tok, exp, cum, True, True, True, False, T, 1, d_in, d_out, E)
        torch.cuda.synchronize()
        assert_close(hid, want, 1e-5, f"ESMM_TENSOR_CORE after re-assignment, seed {seed}")
        assert len(hexa_moe_cuda._route_cache) == 1
    hexa_moe_cuda.clear_route_cache()


def test_cpu_tensors_are_rejected(dev):
    from hexa_moe import ops
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.route_build(torch.zeros(4, 1, dtype=torch.int32), 2)


def test_unsupported_granularity_raises(dev):
    from hexa_moe import _lib, ops
    routing = make_routing(64, 2, 1, seed=1)
    route = ops.route_build(routing.to(dev), 2)
    x = torch.randn(64, 12, device=dev, dtype=BF16)
    W = torch.randn(2, 12, 16, device=dev, dtype=BF16)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        ops.esmm(x, W, None, route, False, _lib.HEXA_W_IN_OUT)
