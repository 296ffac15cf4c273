"""Writes the golden fixtures of this directory from the CPU oracle (fp64).

The reference ships no test vectors for this path, so the fixtures are made by this build's own oracle,
whose functions are pinned by mathematics in tests/test_oracle_*.py.  They freeze today's oracle: a later
change to the oracle that moves any of these numbers fails tests/test_golden.py on the CPU, and the HIP
library is checked against the same files on the GPU.  Everything is small (.npz with fp32 inputs and fp64
expected outputs, about 110 KB together, loaded with allow_pickle=False).

    python tests/golden/make_golden.py        # rewrites tests/golden/*.npz
"""
import math
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

from _util import gen, make_routing  # noqa: E402
from oracle import hexa_oracle as O  # noqa: E402
from oracle import route_oracle as RO  # noqa: E402


def _np(t):
    return t.detach().cpu().numpy()


def _f32_exact(t):
    """Inputs are rounded to fp32 (so that they can be stored as float32 without loss) and used in fp64."""
    return t.float().double()


def routing_fixture():
    T, E, k = 203, 7, 2
    routing = make_routing(T, E, k, seed=11, skew="zipf", empty=1)
    counts, offsets, token_ids = O.route_build(routing, E)
    out = {"routing": _np(routing), "E": np.int64(E), "counts": _np(counts), "offsets": _np(offsets),
           "token_ids": _np(token_ids)}
    for s in range(k):                       # the reference's 16-padded lists of every slot
        r = _np(routing[:, s]).astype(np.int32)
        c, x = RO.token_count(r, E, 16)
        tok, exp = RO.token_assign(r, E, x)
        out[f"pad16_counts_{s}"], out[f"pad16_expanded_{s}"] = c, x
        out[f"pad16_tok_{s}"], out[f"pad16_exp_{s}"] = tok, exp
    return out


def operators_fixture():
    T, d_in, d_out, E, k = 45, 16, 24, 4, 2
    g = gen(12)
    routing = make_routing(T, E, k, seed=12, skew="zipf", empty=1)
    _, offsets, token_ids = O.route_build(routing, E)
    x = _f32_exact(torch.randn(T, d_in, generator=g, dtype=torch.float64))
    xs = _f32_exact(torch.randn(k, T, d_in, generator=g, dtype=torch.float64))
    W = _f32_exact((torch.rand(E, d_in, d_out, generator=g, dtype=torch.float64) * 2 - 1) / math.sqrt(d_in))
    b = _f32_exact(torch.rand(E, d_out, generator=g, dtype=torch.float64) - 0.5)
    dy = _f32_exact(torch.randn(k, T, d_out, generator=g, dtype=torch.float64))
    dy_shared = _f32_exact(torch.randn(T, d_out, generator=g, dtype=torch.float64))
    return {
        "routing": _np(routing), "E": np.int64(E), "x": _np(x.float()), "xs": _np(xs.float()), "W": _np(W.float()),
        "b": _np(b.float()), "dy": _np(dy.float()), "dy_shared": _np(dy_shared.float()),
        "esmm_per_slot": _np(O.esmm(x, W, b, token_ids, offsets, False)),
        "esmm_summed": _np(O.esmm(xs, W, b, token_ids, offsets, True)),
        "estmm_dy_per_slot": _np(O.estmm(dy, x, token_ids, offsets, True, E)),
        "estmm_dy_shared": _np(O.estmm(dy_shared, xs, token_ids, offsets, False, E)),
        "ess_dy_per_slot": _np(O.ess(dy, token_ids, offsets, True, E)),
        "ess_dy_shared": _np(O.ess(dy_shared, token_ids, offsets, False, E)),
    }


def layer_fixture():
    T, d, h, E, k = 40, 8, 24, 3, 2
    g = gen(13)
    routing = make_routing(T, E, k, seed=13)
    x = _f32_exact(torch.randn(T, d, generator=g, dtype=torch.float64))
    dy = _f32_exact(torch.randn(T, d, generator=g, dtype=torch.float64))
    W1 = _f32_exact((torch.rand(E, h, d, generator=g, dtype=torch.float64) * 2 - 1) / math.sqrt(d))
    W2 = _f32_exact((torch.rand(E, h, d, generator=g, dtype=torch.float64) * 2 - 1) / math.sqrt(h))
    b1 = _f32_exact(torch.rand(E, h, generator=g, dtype=torch.float64) - 0.5)
    b2 = _f32_exact(torch.rand(E, d, generator=g, dtype=torch.float64) - 0.5)
    y, y1, _ = O.moe_ffn_forward(x, W1, W2, b1, b2, routing, F.gelu)
    dx, dW1, dW2, db1, db2 = O.moe_ffn_backward(dy, x, y1, W1, W2, True, True, routing, F.gelu)
    return {"routing": _np(routing), "E": np.int64(E), "x": _np(x.float()), "dy": _np(dy.float()), "W1": _np(W1.float()),
            "W2": _np(W2.float()), "b1": _np(b1.float()), "b2": _np(b2.float()), "y": _np(y), "dx": _np(dx), "dW1": _np(dW1), "dW2": _np(dW2),
            "db1": _np(db1), "db2": _np(db2)}


def router_fixture():
    T, E, k = 120, 6, 2
    g = gen(14)
    logits = torch.randn(T, E, generator=g, dtype=torch.float32) * 0.5
    noise = torch.randn(T, E, generator=g, dtype=torch.float32)
    gate_noise = 1.0
    sigma = gate_noise / E
    scores, idx = O.route_top_k(logits, k, noise * sigma)
    return {"logits": _np(logits), "noise": _np(noise), "k": np.int64(k), "gate_noise": np.float64(gate_noise),
            "scores": _np(scores), "idx": _np(idx), "gshard": _np(O.gshard_loss(scores, idx)),
            "load_importance": _np(O.load_importance_loss(F.softmax(logits, 1), (logits + noise * sigma).gather(1, idx),
                                                          E, gate_noise))}


FIXTURES = {"routing": routing_fixture, "operators": operators_fixture, "layer": layer_fixture, "router": router_fixture}


if __name__ == "__main__":
    for name, make in FIXTURES.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **make())
        print(path, os.path.getsize(path), "bytes")
