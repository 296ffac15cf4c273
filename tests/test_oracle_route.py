"""Pins the routing-pass oracle (oracle/hexa_oracle.py and oracle/route_oracle.c) against what the
mathematics fixes: numpy bincount / stable argsort, brute force on tiny inputs, the partition
invariants, and the reference's 16-padding rule.  The reference holds no vectors for this path."""
import subprocess
import os

import numpy as np
import pytest
import torch

from oracle import hexa_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def RO():
    subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "oracle")], check=True)
    from oracle import route_oracle
    return route_oracle


def _rand_routing(T, E, k, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, E, (T, k), generator=g)


@pytest.mark.parametrize("T,E,pad", [(0, 3, 1), (1, 1, 1), (17, 4, 1), (100, 7, 16), (1000, 32, 16), (513, 5, 3)])
def test_count_against_bincount(RO, T, E, pad):
    r = _rand_routing(T, E, 1, T + E)[:, 0]
    want_c = np.bincount(r.numpy(), minlength=E)
    want_x = np.concatenate([[0], np.cumsum(-(-want_c // pad) * pad)])
    for counts, expanded in (O.token_count(r, E, pad), O.token_count_fast(r, E, pad), RO.token_count(r.numpy(), E, pad)):
        assert np.array_equal(np.asarray(counts), want_c)
        assert np.array_equal(np.asarray(expanded), want_x)


@pytest.mark.parametrize("T,E,pad", [(1, 1, 1), (17, 4, 1), (100, 7, 16), (777, 9, 16)])
def test_assign_is_a_stable_sort_with_padding(RO, T, E, pad):
    r = _rand_routing(T, E, 1, 3 * T + E)[:, 0]
    _, expanded = O.token_count(r, E, pad)
    order = np.argsort(r.numpy(), kind="stable")
    counts = np.bincount(r.numpy(), minlength=E)
    for tok, exp in (O.token_assign(r, expanded, E), RO.token_assign(r.numpy(), E, expanded.numpy())):
        tok, exp = np.asarray(tok), np.asarray(exp)
        pos = 0
        for e in range(E):
            s = int(expanded[e])
            assert s % pad == 0
            seg = tok[s:s + counts[e]]
            assert np.array_equal(seg, order[pos:pos + counts[e]])          # ascending ids = stable order
            assert np.all(exp[s:s + counts[e]] == e)
            assert np.all(tok[s + counts[e]:int(expanded[e + 1])] == -1)     # fillers keep the caller's -1
            assert np.all(exp[s + counts[e]:int(expanded[e + 1])] == -1)
            pos += counts[e]


def test_brute_force_tiny():
    # every routing of 4 tokens over 3 experts
    for code in range(3 ** 4):
        r = torch.tensor([(code // 3 ** i) % 3 for i in range(4)])
        counts, offsets, tok = O.route_build(r[:, None], 3)
        want = [[t for t in range(4) if r[t] == e] for e in range(3)]
        assert counts[0].tolist() == [len(w) for w in want]
        assert tok[0].tolist() == [t for w in want for t in w]
        assert offsets[0].tolist() == [0, len(want[0]), len(want[0]) + len(want[1]), 4]


@pytest.mark.parametrize("T,E,k", [(64, 8, 2), (1000, 32, 2), (2048, 8, 1), (300, 64, 3)])
def test_route_build_invariants_and_c_port(RO, T, E, k):
    r = _rand_routing(T, E, k, T * k)
    counts, offsets, tok = O.route_build(r, E)
    c2, o2, t2 = RO.route_build(r.numpy(), E)
    assert np.array_equal(counts.numpy(), c2) and np.array_equal(offsets.numpy(), o2) and np.array_equal(tok.numpy(), t2)
    for s in range(k):
        assert int(counts[s].sum()) == T and int(offsets[s, E]) == T
        assert torch.equal(torch.sort(tok[s]).values, torch.arange(T, dtype=torch.int32))   # a permutation
        assert torch.all(offsets[s, 1:] >= offsets[s, :-1])
        for e in range(E):
            seg = tok[s, offsets[s, e]:offsets[s, e + 1]].long()
            assert torch.all(r[seg, s] == e)
            assert torch.all(seg[1:] > seg[:-1])
        # unpadded pad=1 path of the two reference ops gives the same lists
        c1, x1 = O.token_count(r[:, s], E, 1)
        t1, _ = O.token_assign(r[:, s], x1, E)
        assert torch.equal(c1, counts[s]) and torch.equal(x1, offsets[s]) and torch.equal(t1, tok[s])


def test_c_port_rejects_bad_ids(RO):
    with pytest.raises(ValueError):
        RO.token_count(np.array([0, 5], np.int32), 3)
