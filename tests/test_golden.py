"""The CPU oracle against the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_golden.py from the oracle itself): a guard against the oracle drifting between rounds.
The HIP library is checked against the same files in tests/test_gpu_golden.py."""
import os

import numpy as np
import torch
import torch.nn.functional as F

from oracle import hexa_oracle as O
from oracle import route_oracle as RO

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLD, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def t64(a):
    return torch.from_numpy(np.asarray(a)).double()


def close(a, b, tol=1e-12):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.abs(a - b).max() <= tol * max(1.0, np.abs(b).max())


def test_routing_fixture():
    g = load("routing")
    routing, E = torch.from_numpy(g["routing"]), int(g["E"])
    counts, offsets, token_ids = O.route_build(routing, E)
    assert np.array_equal(counts.numpy(), g["counts"]) and np.array_equal(offsets.numpy(), g["offsets"])
    assert np.array_equal(token_ids.numpy(), g["token_ids"])
    for s in range(routing.shape[1]):
        r = g["routing"][:, s].astype(np.int32)
        c, x = RO.token_count(r, E, 16)
        tok, exp = RO.token_assign(r, E, x)
        assert np.array_equal(c, g[f"pad16_counts_{s}"]) and np.array_equal(x, g[f"pad16_expanded_{s}"])
        assert np.array_equal(tok, g[f"pad16_tok_{s}"]) and np.array_equal(exp, g[f"pad16_exp_{s}"])


def test_operator_fixture():
    g = load("operators")
    routing, E = torch.from_numpy(g["routing"]), int(g["E"])
    _, offsets, token_ids = O.route_build(routing, E)
    x, xs, W, b, dy, dys = (t64(g[k]) for k in ("x", "xs", "W", "b", "dy", "dy_shared"))
    assert close(O.esmm(x, W, b, token_ids, offsets, False), g["esmm_per_slot"])
    assert close(O.esmm(xs, W, b, token_ids, offsets, True), g["esmm_summed"])
    assert close(O.estmm(dy, x, token_ids, offsets, True, E), g["estmm_dy_per_slot"])
    assert close(O.estmm(dys, xs, token_ids, offsets, False, E), g["estmm_dy_shared"])
    assert close(O.ess(dy, token_ids, offsets, True, E), g["ess_dy_per_slot"])
    assert close(O.ess(dys, token_ids, offsets, False, E), g["ess_dy_shared"])


def test_layer_fixture():
    g = load("layer")
    routing = torch.from_numpy(g["routing"])
    x, dy, W1, W2, b1, b2 = (t64(g[k]) for k in ("x", "dy", "W1", "W2", "b1", "b2"))
    y, y1, _ = O.moe_ffn_forward(x, W1, W2, b1, b2, routing, F.gelu)
    grads = O.moe_ffn_backward(dy, x, y1, W1, W2, True, True, routing, F.gelu)
    assert close(y, g["y"])
    for name, got in zip(("dx", "dW1", "dW2", "db1", "db2"), grads):
        assert close(got, g[name]), name


def test_router_fixture():
    g = load("router")
    logits, noise = torch.from_numpy(g["logits"]), torch.from_numpy(g["noise"])
    k, gate_noise = int(g["k"]), float(g["gate_noise"])
    E = logits.shape[1]
    sigma = gate_noise / E
    scores, idx = O.route_top_k(logits, k, noise * sigma)
    assert np.array_equal(idx.numpy(), g["idx"]) and close(scores, g["scores"], 1e-7)
    assert close(O.gshard_loss(scores, idx), g["gshard"], 1e-7)
    li = O.load_importance_loss(F.softmax(logits, 1), (logits + noise * sigma).gather(1, idx), E, gate_noise)
    assert close(li, g["load_importance"], 1e-6)
