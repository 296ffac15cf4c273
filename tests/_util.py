"""Shared helpers of the parity tests: seeded problems and error measures."""
import math

import torch

# Tolerances of the parity bar: relative error of the whole tensor (Frobenius) and of the worst
# element against the largest reference magnitude.
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def rel_err(a, b):
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    den = b.norm().item()
    fro = (a - b).norm().item() / den if den > 0 else (a - b).norm().item()
    mx = b.abs().max().item()
    worst = (a - b).abs().max().item() / mx if mx > 0 else (a - b).abs().max().item()
    return fro, worst


def assert_close(a, b, tol, what=""):
    assert a.shape == b.shape, (what, a.shape, b.shape)
    fro, worst = rel_err(a, b)
    assert fro <= tol and worst <= tol, f"{what}: rel-err fro={fro:.3e} worst={worst:.3e} > {tol:.1e}"


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def make_routing(T, E, k, seed, skew=None, empty=0):
    """[T,k] int64 routing on the CPU.  skew None: top-k of softmax(logits + per-expert bias), the
    benchmark's recipe; 'zipf': Zipf(1.2) ranks over a seeded expert permutation with `empty`
    experts never chosen; 'one': every token to expert E-1."""
    g = gen(seed)
    if skew == "one":
        idx = torch.full((T, k), E - 1, dtype=torch.int64)
        for s in range(1, k):
            idx[:, s] = (E - 1 - s) % E
        return idx
    if skew == "zipf":
        live = E - empty
        w = 1.0 / torch.arange(1, live + 1, dtype=torch.float64) ** 1.2
        perm = torch.randperm(E, generator=g)[:live]
        idx = torch.empty(T, k, dtype=torch.int64)
        first = torch.multinomial(w, T, replacement=True, generator=g)
        idx[:, 0] = perm[first]
        for s in range(1, k):  # next distinct draw
            nxt = torch.multinomial(w, T, replacement=True, generator=g)
            clash = nxt == first
            nxt[clash] = (nxt[clash] + 1) % live
            idx[:, s] = perm[nxt]
        return idx
    logits = torch.randn(T, E, generator=g) + 0.5 * torch.randn(E, generator=g)
    return torch.topk(torch.softmax(logits, 1), k, dim=1).indices


def uniform(shape, bound, g):
    return (torch.rand(shape, generator=g) * 2 - 1) * bound


def make_linear(T, d_in, d_out, E, k, seed, dtype, m2s):
    """Seeded ESMM problem.  Values are rounded to `dtype` first so oracle and GPU see the same numbers."""
    g = gen(seed)
    b = 1.0 / math.sqrt(d_in)
    x = torch.randn((k, T, d_in) if m2s else (T, d_in), generator=g).to(dtype)
    W = uniform((E, d_in, d_out), b, g).to(dtype)
    bias = uniform((E, d_out), b, g).to(dtype)
    return x, W, bias
