"""Host-side logic that needs no GPU: the module API, the state-dict contract, routing and losses
against the oracle, the dense depths, error behaviour, and that the C-ABI library loads and exports
every symbol the public header declares (no compute calls)."""
import ctypes
import os
import re

import pytest
import torch
import torch.nn.functional as F

from oracle import hexa_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GATE = {'type': 'top', 'k': 1, 'gate_noise': 1.0, 'fp32_gate': True}


def _readme_module(**kw):
    from hexa_moe import moe as hmoe
    args = dict(gate_type=dict(GATE), model_dim_list=[128, 128, 128, 128], moe_idx_list=[2, 3], mlp_ratio=4,
                mlp_proportion=None, num_global_experts=8, total_depth=4, data_centric=True, mlp_fc1_bias=True,
                mlp_fc2_bias=True, activation_fn=lambda x: F.gelu(x))
    args.update(kw)
    return hmoe.MoE_Cascaded(**args)


def test_header_symbols_are_exported():
    from hexa_moe import _lib
    header = open(os.path.join(ROOT, "include", "hexa_moe_hip.h")).read()
    declared = set(re.findall(r"^(?:int|const char\*)\s+(hexa_\w+)\s*\(", header, flags=re.M))
    assert len(declared) >= 12
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/hexa_moe_hip.h but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert lib.hexa_abi_version() == 9


def test_abi_argument_errors_without_a_gpu():
    from hexa_moe import _lib
    lib = _lib.load()
    assert lib.hexa_esmm(None, None, None, None, None, 0, 0, 0, 16, 1, 8, 8, 2, 0, 0, 0, 0, 0, None, None, None) == -1
    assert b"null pointer" in lib.hexa_last_error()
    assert lib.hexa_route_layout_get(-1, 1, 1, ctypes.byref(_lib.RouteLayout())) == -1
    assert lib.hexa_token_count(None, None, None, 4, 2, 1, None, None) == -1
    L = _lib.route_layout(18432, 2, 32)
    assert L.mt_ub == 18432 // 128 + 32 and L.units == 36 and L.tile_info % 4 == 0
    assert L.mt_ub_l == 18432 // 256 + 32 and L.tile_info_l % 4 == 0
    parts = [L.counts, L.offsets, L.token_ids, L.expert_ids, L.tile_count, L.tile_info, L.tile_count_l, L.tile_info_l,
             L.scratch, L.total_ints]
    assert parts == sorted(parts)


def test_state_dict_names_and_shapes():
    m = _readme_module(seeds=(11, 12, 13))
    sd = m.state_dict()
    want = {"batched_fc1_w.0": (8, 512, 128), "batched_fc2_w.1": (8, 512, 128), "batched_fc1_bias.0": (8, 512),
            "batched_fc2_bias.1": (8, 128), "mlp_fc1_w.0": (512, 128), "mlp_fc2_w.1": (512, 128),
            "mlp_fc1_b.0": (512,), "mlp_fc2_b.1": (128,), "gates.0.wg.weight": (8, 128), "gates.1.wg.weight": (8, 128)}
    for k, shape in want.items():
        assert tuple(sd[k].shape) == shape, k
    assert len(sd) == 18
    assert m.gates[0].wg.weight.dtype == torch.float32
    assert float(m.batched_fc1_bias[0].detach().abs().max()) == 0.0
    w = m.batched_fc1_w[0].detach()                                   # trunc_normal(std=0.005), cut at +-2 (absolute)
    # (a uniform draw of exactly -1 maps to the lower cut itself, -2: one element in 2^24, so the bulk is checked, not the maximum)
    bulk = w[w.abs() < 0.05]
    assert bulk.numel() > 0.9999 * w.numel() and 0.004 < float(bulk.std()) < 0.006 and float(w.abs().max()) <= 2.0
    nb = _readme_module(mlp_fc1_bias=False, mlp_fc2_bias=False)
    assert not any("bias" in k or "_b." in k for k in nb.state_dict())
    assert nb.batched_fc1_bias[0] is None


def test_gate_spec_is_not_modified_and_seeds_work():
    spec = dict(GATE)
    a = _readme_module(gate_type=spec, seeds=(1, 2, 3))
    assert spec == GATE
    b = _readme_module(gate_type=spec, seeds=(1, 2, 3))
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    cos = _readme_module(gate_type={'type': 'cosine_top', 'k': 2, 'proj_dim': 32})
    assert cos.gates[1].sim_matrix.shape == (32, 8) and cos.gates[0].top_k == 2
    legacy = _readme_module(gate_type='Top2Gate')
    assert legacy.gates[0].top_k == 2
    with pytest.raises(Exception, match="Unrecognized"):
        _readme_module(gate_type={'type': 'top', 'k': 1, 'bogus': 3})


def test_unsupported_modes_are_refused():
    with pytest.raises(NotImplementedError):
        _readme_module(data_centric=False)
    with pytest.raises(NotImplementedError):
        _readme_module(mlp_proportion=[0.5, 0.5])


def test_dense_depth_matches_oracle_and_backpropagates():
    m = _readme_module()
    for p in m.parameters():
        torch.nn.init.uniform_(p.data, -0.1, 0.1)
    x = torch.randn(4, 16, 128, requires_grad=True)
    y, l_aux = m(1, x)
    assert l_aux == 0 and y.shape == x.shape
    want = O.dense_mlp_forward(x.detach().reshape(-1, 128), m.mlp_fc1_w[1].detach(), m.mlp_fc2_w[1].detach(),
                               m.mlp_fc1_b[1].detach(), m.mlp_fc2_b[1].detach(), F.gelu)
    assert torch.allclose(y.detach().reshape(-1, 128), want, atol=1e-5)
    y.sum().backward()
    assert x.grad is not None and m.mlp_fc1_w[1].grad is not None and m.mlp_fc1_w[0].grad is None


def test_moe_depth_on_cpu_fails_loudly():
    m = _readme_module()
    with pytest.raises(RuntimeError, match="GPU only"):
        m(2, torch.randn(8, 128))


def test_routing_and_losses_match_oracle():
    from hexa_moe.impls import losses
    from hexa_moe.impls.layers import simplified_extract_critical, topk_and_loss
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(300, 8, generator=g)
    noise = torch.randn(300, 8, generator=g) / 8
    scores, idx = O.route_top_k(logits, 2, noise)
    got_idx, l = topk_and_loss(F.softmax(logits + noise, dim=1), 2)
    assert torch.equal(got_idx, idx)
    assert torch.allclose(l, O.gshard_loss(scores, idx))
    lists, l2 = simplified_extract_critical(F.softmax(logits + noise, dim=1), 2)
    assert len(lists) == 2 and torch.equal(lists[1], idx[:, 1]) and torch.equal(l, l2)
    topk_logits = (logits + noise).gather(1, idx)
    a = losses.load_importance_loss(F.softmax(logits, 1), topk_logits, 8, 1.0)
    b = O.load_importance_loss(F.softmax(logits, 1), topk_logits, 8, 1.0)
    assert torch.allclose(a, b, rtol=1e-5)


def test_module_routing_is_deterministic_in_eval_and_noisy_in_train():
    m = _readme_module()
    x = torch.randn(64, 128)
    m.eval()
    a, _ = m._route(m.gates[0], x, 1)
    b, _ = m._route(m.gates[0], x, 1)
    assert torch.equal(a, b)
    want = torch.topk(F.softmax(F.linear(x, m.gates[0].wg.weight), 1), 1).indices
    assert torch.equal(a, want)


def test_moe_buffer_round_trip():
    from hexa_moe import moe as hmoe
    m = _readme_module()
    buf = hmoe.MoE_Buffer([128, 128], 8, 2, mlp_ratio=4)
    assert set(buf.state_dict()) == {k for k in m.state_dict() if k.startswith("batched_")}
    for p in buf.parameters():
        torch.nn.init.normal_(p.data)
    m.load_ckpt(buf)
    assert torch.equal(m.batched_fc2_w[1].data, buf.batched_fc2_w[1].data)
    out = hmoe.MoE_Buffer([128, 128], 8, 2, mlp_ratio=4)
    m.save_ckpt(out)
    for (k1, v1), (k2, v2) in zip(buf.state_dict().items(), out.state_dict().items()):
        assert k1 == k2 and torch.equal(v1, v2)
    assert m.cuda_cache() is None and m.cache_gather(0) is None


def test_skip_moe_env(monkeypatch):
    monkeypatch.setenv("SKIP_MOE", "1")
    m = _readme_module()
    x = torch.randn(8, 128)
    y, l = m(2, x)
    assert y is x and l is None


def test_triton_sibling_surface_signatures():
    """hexa_moe.kernels exports counter / ESMM / es_fused with the argument lists of
    hexa_moe_triton/hexa_moe/kernels (basics.py:89, esmm.py:249, fused.py:382)."""
    import inspect
    from hexa_moe import kernels
    from hexa_moe.kernels import constant
    assert constant.MAX_TOKEN_CHUNK == 16
    assert list(inspect.signature(kernels.counter).parameters) == ["routing", "num_exps"]
    assert list(inspect.signature(kernels.ESMM).parameters) == ["toks", "w", "b", "tok_ids_list", "exp_ids_list"]
    assert list(inspect.signature(kernels.es_fused).parameters) == ["tok1", "tok2", "w", "tok_ids_list", "exp_ids_list",
                                                                    "exp_start_list", "num_exps", "bias"]
    import torch
    with __import__("pytest").raises(RuntimeError):
        kernels.counter(torch.zeros(8, dtype=torch.int32), 4)       # CPU tensors are rejected: no fallback
