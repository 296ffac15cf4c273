"""MoE_Cascaded / MoE_Buffer: every FFN and MoE layer of a model in one module
(reference: hexa_moe_cuda/hexa_moe/impls/cascaded_moe.py:38-80, 82-568).

Constructor arguments, forward signature, parameter names and shapes follow the reference so that a
model written against `hexa_moe.moe` (the Swin-MoE model, the README example) runs unchanged and its
state dict round-trips:
    batched_fc1_w.{i} [E,h,d_in]   batched_fc2_w.{i} [E,h,d_out]   batched_fc1_bias.{i} [E,h]
    batched_fc2_bias.{i} [E,d_out] mlp_fc1_w.{j} [h,d_in]  mlp_fc2_w.{j} [h,d_out]  mlp_fc1_b.{j}  mlp_fc2_b.{j}
    gates.{i}.wg.weight [E,d]

This build is one GPU, data-centric: each device holds every expert in full, so the reference's
weight cache pool + all-gather (cascaded_moe.py:244-256, 387-410) has nothing to move; what is shared
across the depths instead is a pool of routing-metadata buffers (one slot per MoE depth, allocated
once and reused every step).  Expert, hidden-dim and model sharding are not implemented and are
refused (`data_centric=False`, a non-trivial `mlp_proportion`).

Behaviour that differs from the reference on purpose: no process group is needed; routing is
evaluated once per call (the reference evaluates it twice on CUDA and draws the gate noise twice,
cascaded_moe.py:533-536); the gate configuration passed in is not modified (cascaded_moe.py:299-317
pops 'type' from the caller's dict); expert Parameters receive gradients (the reference passes
`.data`, cascaded_moe.py:553-559).
"""
import importlib
import logging
import os
import re
import weakref
from types import SimpleNamespace

import torch
import torch.distributed as dist
import torch.nn.functional as F
from torch import nn

from .. import ops
from . import losses, router
from .layers import (FusedMoE_Shared_CudaCore, FusedMoEDepth, MLP_Implement, is_plain_gelu,  # noqa: F401
                     simplified_extract_critical, topk_and_loss)


def cast_if_autocast_enabled(tensor):
    """Cast to the autocast dtype of the tensor's device when autocast is on
    (reference: cascaded_moe.py:23-36)."""
    kind = tensor.device.type
    if kind not in ("cuda", "cpu"):
        raise RuntimeError("User specified autocast device_type must be 'cuda' or 'cpu'")
    if torch.is_autocast_enabled(kind):
        return tensor.to(dtype=torch.get_autocast_dtype(kind))
    return tensor


def _param_list(shapes):
    return nn.ParameterList([nn.Parameter(torch.empty(*s)) if s is not None else None for s in shapes])


class MoE_Buffer(nn.Module):
    """Host-side holder of the full expert parameters, used to load / save checkpoints
    (reference: cascaded_moe.py:38-80).  Same parameter names and shapes as MoE_Cascaded's experts."""

    def __init__(self, model_dim_list_moe, num_global_experts, total_depth_moe, mlp_ratio=4.,
                 output_dim_list_moe=None, mlp_fc1_bias=True, mlp_fc2_bias=True):
        super().__init__()
        E = int(num_global_experts)
        self.total_depth_moe = total_depth_moe
        self.num_global_experts = E
        self.input_dim_list_moe = list(model_dim_list_moe)
        self.output_dim_list_moe = list(output_dim_list_moe or model_dim_list_moe)
        self.hidden_size_list_moe = [int(mlp_ratio * d) for d in model_dim_list_moe]
        self.has_fc1_bias, self.has_fc2_bias = mlp_fc1_bias, mlp_fc2_bias
        depths = range(total_depth_moe)
        hid, din, dout = self.hidden_size_list_moe, self.input_dim_list_moe, self.output_dim_list_moe
        self.batched_fc1_w = _param_list([(E, hid[i], din[i]) for i in depths])
        self.batched_fc2_w = _param_list([(E, hid[i], dout[i]) for i in depths])
        self.batched_fc1_bias = _param_list([(E, hid[i]) if mlp_fc1_bias else None for i in depths])
        self.batched_fc2_bias = _param_list([(E, dout[i]) if mlp_fc2_bias else None for i in depths])


class RoutePool:
    """Routing-metadata buffers shared across the MoE depths: one int32 device buffer per depth,
    allocated on first use and reused by every later step.  A buffer still referenced by a pending
    backward (its Route object is alive) is left alone and a new one takes its slot."""

    def __init__(self):
        self._slots = {}

    def slot(self, stage, T, k, E, device):
        need = ops.route_blob_ints(T, k, E)
        entry = self._slots.get(stage)
        if entry is not None:
            blob, owner = entry
            free = owner is None or owner() is None
            if free and blob.numel() >= need and blob.device == device:
                return blob
        blob = torch.empty(max(need, 4), dtype=torch.int32, device=device)
        self._slots[stage] = (blob, None)
        return blob

    def bind(self, stage, route):
        entry = self._slots.get(stage)
        if entry is not None and entry[0] is route.blob:
            self._slots[stage] = (entry[0], weakref.ref(route))

    def clear(self):
        self._slots.clear()


class MoE_Cascaded(nn.Module):
    def __init__(self, gate_type, model_dim_list, moe_idx_list, num_global_experts, total_depth, data_centric=True,
                 mlp_ratio=4., mlp_proportion=None, output_dim_list=None, mlp_fc1_bias=True, mlp_fc2_bias=True,
                 activation_fn=None, activation_fn_with_self=None, result_func=None, group=None, seeds=None,
                 a2a_ffn_overlap_degree=1, batch_prioritized_routing=False, normalize_gate=True,
                 is_gshard_loss=True, parallel_type='adaptive:1', use_2dh=False):
        super().__init__()
        if not data_centric:
            raise NotImplementedError("hexa_moe (MI355X build): model-centric mode shards experts over several "
                                      "GPUs and is not part of this one-GPU build; use data_centric=True")
        if mlp_proportion is not None and not (len(mlp_proportion) == 1 and abs(mlp_proportion[0] - 1.0) < 1e-3):
            raise NotImplementedError("hexa_moe (MI355X build): mlp_proportion splits the hidden dimension over "
                                      "devices; this build keeps every expert whole on one GPU")
        self.group = group
        self.result_func = result_func
        self.skip_moe = int(os.environ.get('SKIP_MOE', '0')) != 0
        self.batch_prioritized_routing = batch_prioritized_routing or int(os.environ.get('BATCH_PRIO', 0)) != 0
        self.normalize_gate = normalize_gate
        self.is_gshard_loss = is_gshard_loss
        self.a2a_ffn_overlap_degree = a2a_ffn_overlap_degree
        self.use_2dh = use_2dh
        self.parallel_type = parallel_type
        self.fused_router = True   # set False to route with the PyTorch formulation
        self.fused_depth = True    # set False to run a depth operator by operator instead of as two library calls
        # One device holds every expert in full; a process group, if there is one, only replicates.
        self.world_size, self.local_rank = 1, 0
        if dist.is_available() and dist.is_initialized():
            self.local_rank = dist.get_rank(group)
        self.mlp_proportion = [1.0]

        if seeds is not None and seeds[1] is not None:
            torch.manual_seed(seeds[1])

        E = int(num_global_experts)
        self.num_global_experts = E
        self.moe_idx_list = list(moe_idx_list)
        self.mlp_idx_list = [i for i in range(total_depth) if i not in self.moe_idx_list]
        self.total_depth_moe, self.total_depth_mlp = len(self.moe_idx_list), len(self.mlp_idx_list)
        out_dims = output_dim_list or model_dim_list
        self.input_dim_list_moe = [model_dim_list[i] for i in self.moe_idx_list]
        self.output_dim_list_moe = [out_dims[i] for i in self.moe_idx_list]
        self.hidden_size_list_moe = [int(d * mlp_ratio) for d in self.input_dim_list_moe]
        self.input_dim_list_mlp = [model_dim_list[i] for i in self.mlp_idx_list]
        self.output_dim_list_mlp = [out_dims[i] for i in self.mlp_idx_list]
        self.hidden_size_list_mlp = [int(d * mlp_ratio) for d in self.input_dim_list_mlp]
        self.has_fc1_bias, self.has_fc2_bias = mlp_fc1_bias, mlp_fc2_bias
        # the whole hidden dimension of every MoE depth lives here (reference: dim_split, :341-361)
        self.local_dim_list = list(self.hidden_size_list_moe)
        self.local_dim_list_all = [self.local_dim_list]
        self.ids_list_global = [[list(range(h)) for h in self.hidden_size_list_moe]]

        hid, din, dout = self.hidden_size_list_moe, self.input_dim_list_moe, self.output_dim_list_moe
        moe = range(self.total_depth_moe)
        self.batched_fc1_w = _param_list([(E, hid[i], din[i]) for i in moe])
        self.batched_fc2_w = _param_list([(E, hid[i], dout[i]) for i in moe])
        self.batched_fc1_bias = _param_list([(E, hid[i]) if mlp_fc1_bias else None for i in moe])
        self.batched_fc2_bias = _param_list([(E, dout[i]) if mlp_fc2_bias else None for i in moe])
        hid, din, dout = self.hidden_size_list_mlp, self.input_dim_list_mlp, self.output_dim_list_mlp
        mlp = range(self.total_depth_mlp)
        self.mlp_fc1_w = _param_list([(hid[j], din[j]) for j in mlp])
        self.mlp_fc2_w = _param_list([(hid[j], dout[j]) for j in mlp])
        self.mlp_fc1_b = _param_list([(hid[j],) if mlp_fc1_bias else None for j in mlp])
        self.mlp_fc2_b = _param_list([(dout[j],) if mlp_fc2_bias else None for j in mlp])

        if activation_fn_with_self is not None:
            assert activation_fn is None, \
                "Option `activation_fn_with_self` has been specified, please keep exactly one of them."
            activation_fn = lambda x: activation_fn_with_self(x, self)  # noqa: E731
        if activation_fn is None:
            activation_fn = F.relu

        self.dispatch_params = SimpleNamespace(
            activation_fn=activation_fn, stage=0, world_size=1, local_rank=self.local_rank,
            has_fc1_bias=mlp_fc1_bias, has_fc2_bias=mlp_fc2_bias, data_centric=True,
            input_dim_list_moe=self.input_dim_list_moe, output_dim_list_moe=self.output_dim_list_moe,
            hidden_size_list_moe=self.hidden_size_list_moe, local_dim_list=self.local_dim_list,
            num_global_experts=E, indices_=None, routing_=None, route_pool=RoutePool())

        self._init_moe()
        self._build_gates(gate_type, seeds)
        if seeds is not None and len(seeds) > 2 and seeds[2] is not None:
            torch.manual_seed(seeds[2])

    # ---- construction helpers ------------------------------------------------------------------
    def _init_moe(self):
        """trunc_normal(std=0.005) weights, zero biases (reference: cascaded_moe.py:324-339)."""
        for plist in (self.batched_fc1_w, self.batched_fc2_w, self.mlp_fc1_w, self.mlp_fc2_w):
            for p in plist:
                nn.init.trunc_normal_(p.data, std=0.005)
        for plist in (self.batched_fc1_bias, self.batched_fc2_bias, self.mlp_fc1_b, self.mlp_fc2_b):
            for p in plist:
                if p is not None:
                    nn.init.zeros_(p.data)

    def _build_gates(self, gate_type, seeds):
        if isinstance(gate_type, str):
            assert re.match(r'^Top[0-9]+Gate$', gate_type), "Unrecognized gate_type: %s" % gate_type
            top_k = int(gate_type[3:-4])
            logging.warning(f"gate_type value `{gate_type}` has been deprecated, please use "
                            f"gate_type = {{'type': 'top', 'k': {top_k}}} instead.")
            gate_type = {'type': 'top', 'k': top_k}
        if not isinstance(gate_type, list):
            gate_type = [gate_type]
        self.gate_len = len(gate_type)
        gates = []
        for depth in range(self.total_depth_moe):
            for gi, spec in enumerate(gate_type):
                options = dict(spec)  # the caller's dict is left untouched
                kind = options.pop('type')
                assert re.match(r'[a-zA-Z0-9\_]+', kind), \
                    "Gate type must only include digits, letters and underline characters."
                if seeds is not None and seeds[0] is not None:
                    torch.manual_seed(seeds[0] + gi)
                try:
                    module = importlib.import_module(f'...gates.{kind}', __name__)
                except ModuleNotFoundError:
                    raise Exception("Unrecognized gate_type: %s" % kind)
                gate = module.Gate(model_dim=self.input_dim_list_moe[depth],
                                   num_global_experts=self.num_global_experts, **options)
                if not hasattr(gate, 'gate_noise'):
                    gate.gate_noise = options.get('gate_noise', 0.0)
                gates.append(gate)
        self.gates = nn.ModuleList(gates)

    # ---- the reference's cache / checkpoint entry points -----------------------------------------
    def cuda_cache(self):
        """Reference: moves the weight cache pool to the GPU (cascaded_moe.py:380-385).  Here the
        parameters are the full weights, so there is no pool to move; kept for callers."""
        return None

    def cache_gather(self, depth_idx=0):
        """Reference: all-gathers the hidden-dim shards of depth `depth_idx` (cascaded_moe.py:387-410).
        One GPU holds whole experts: nothing to gather."""
        return None

    def _expert_lists(self):
        return (("batched_fc1_w", True), ("batched_fc2_w", True),
                ("batched_fc1_bias", self.has_fc1_bias), ("batched_fc2_bias", self.has_fc2_bias))

    def load_ckpt(self, load_moe, src_rank=0):
        """Copy expert parameters from a MoE_Buffer (reference: cascaded_moe.py:412-472, where rank
        `src_rank` scatters hidden-dim shards; here the whole tensors are copied)."""
        with torch.no_grad():
            for name, present in self._expert_lists():
                if not present:
                    continue
                for dst, src in zip(getattr(self, name), getattr(load_moe, name)):
                    dst.copy_(src.to(dst.device, dst.dtype))

    def save_ckpt(self, dst_moe, dst_rank=0):
        """Copy expert parameters into a MoE_Buffer (the Triton sibling's save_ckpt,
        hexa_moe_triton/hexa_moe/impls/cascaded_moe.py:413-464)."""
        with torch.no_grad():
            for name, present in self._expert_lists():
                if not present:
                    continue
                for src, dst in zip(getattr(self, name), getattr(dst_moe, name)):
                    dst.copy_(src.to(dst.device, dst.dtype))

    # ---- forward -----------------------------------------------------------------------------------
    def _route(self, gate, x, top_k):
        """gate -> (+noise) -> softmax -> top-k and the auxiliary loss (reference: cascaded_moe.py:515-531).
        GPU inputs with the linear gate take the fused kernels (impls/router.py)."""
        if self.fused_router and router.fused_route_supported(gate, x, top_k, self.num_global_experts,
                                                              self.is_gshard_loss):
            return router.fused_route(gate, x, top_k, self.num_global_experts,
                                      gate.gate_noise / self.num_global_experts, self.training, self.is_gshard_loss)
        logits = gate(x)
        if self.training and gate.gate_noise > 0:
            logits_w_noise = logits + gate.gate_noise * torch.randn_like(logits) / self.num_global_experts
        else:
            logits_w_noise = logits
        scores = F.softmax(logits_w_noise, dim=1)
        if self.is_gshard_loss:
            loss_fn = losses.gshard_loss
        else:
            def loss_fn(gates, topk_ids):
                return losses.load_importance_loss(F.softmax(logits, dim=1), logits_w_noise.gather(index=topk_ids, dim=1),
                                                   self.num_global_experts, gate.gate_noise)
        return topk_and_loss(scores, top_k, loss_fn)

    def _depth_call_supported(self, gate, x, top_k):
        """The one-call-per-depth path covers the linear fp32 gate with the fused router and the exact GELU."""
        return (self.fused_depth and self.fused_router and is_plain_gelu(self.dispatch_params.activation_fn)
                and router.fused_route_supported(gate, x, top_k, self.num_global_experts, self.is_gshard_loss)
                and (gate.fp32_gate or x.dtype == torch.float32))

    def forward(self, depth_idx, input, gate_index=0, top_k=None, a2a_ffn_overlap_degree=None, reserve_dims=1):
        is_moe = depth_idx in self.moe_idx_list
        if self.skip_moe:
            return (self.result_func(input) if self.result_func is not None else input), None

        original_shape, original_dtype = input.shape, input.dtype
        assert len(original_shape) >= 2, "Input data must be at least 2D tensor: (s)amples, .., (m)odel_dim"
        x = input.reshape(-1, original_shape[-reserve_dims:].numel())
        if torch.is_autocast_enabled(x.device.type):
            x = cast_if_autocast_enabled(x)
        else:
            first = next(self.parameters(), None)
            if first is not None:
                x = x.to(first.dtype)

        if not is_moe:
            j = self.mlp_idx_list.index(depth_idx)
            y = MLP_Implement.apply(self.dispatch_params, x, self.mlp_fc1_w[j], self.mlp_fc2_w[j],
                                    self.mlp_fc1_b[j], self.mlp_fc2_b[j]).to(original_dtype)
            y = y.view(list(original_shape[:-reserve_dims]) + list(y.shape[-reserve_dims:]))
            return (self.result_func(y) if self.result_func is not None else y), 0

        i = self.moe_idx_list.index(depth_idx)
        gate = self.gates[i * self.gate_len + gate_index]
        if a2a_ffn_overlap_degree is not None:
            self.a2a_ffn_overlap_degree = a2a_ffn_overlap_degree
        cfg = self.dispatch_params
        cfg.stage = i
        k = min(int(top_k or gate.top_k), self.num_global_experts)
        if self._depth_call_supported(gate, x, k):
            # the whole depth as two library calls (forward, backward)
            noise_scale = gate.gate_noise / self.num_global_experts if (self.training and gate.gate_noise > 0) else 0.0
            opts = (k, noise_scale, bool(self.is_gshard_loss), gate.gate_noise / self.num_global_experts)
            y, l_aux = FusedMoEDepth.apply(cfg, opts, x.contiguous(), gate.wg.weight, self.batched_fc1_w[i],
                                           self.batched_fc2_w[i], self.batched_fc1_bias[i], self.batched_fc2_bias[i])
            y = y.to(original_dtype)
        else:
            indices, l_aux = self._route(gate, x, k)
            cfg.routing_ = indices  # [T,k] int64 / int32, read in place by the routing pass
            y = FusedMoE_Shared_CudaCore.apply(cfg, x.contiguous(), self.batched_fc1_w[i], self.batched_fc2_w[i],
                                               self.batched_fc1_bias[i], self.batched_fc2_bias[i]).to(original_dtype)
        # the reference's form of the decision (cascaded_moe.py:545): k int32 vectors of T expert ids
        cfg.indices_ = [col.to(torch.int32) for col in cfg.routing_.unbind(dim=1)]
        y = y.view(list(original_shape[:-reserve_dims]) + list(y.shape[-reserve_dims:]))
        return (self.result_func(y) if self.result_func is not None else y), l_aux
