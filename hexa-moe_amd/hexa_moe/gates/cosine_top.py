"""Cosine-similarity top-k router (reference: hexa_moe_cuda/hexa_moe/gates/cosine_top.py:7-37).

logits = exp(min(temperature, log 100)) * <normalize(proj(x)), normalize(sim_matrix)>
Parameters keep the reference's names: temperature [1], cosine_projector (Linear model_dim ->
proj_dim), sim_matrix [proj_dim, E].
"""
import math

import torch
from torch import nn
from torch.nn import functional as F

_ALLOWED_EXTRA = frozenset({"capacity_factor", "gate_noise"})


class CosineTopKGate(nn.Module):
    def __init__(self, model_dim, num_global_experts, k=1, fp32_gate=False, proj_dim=256, init_t=0.5, **options):
        super().__init__()
        unknown = set(options) - _ALLOWED_EXTRA
        if unknown:
            raise Exception("Unrecognized argument provided to Gating module: %s" % sorted(unknown)[0])
        self.fp32_gate = bool(fp32_gate)
        self.top_k = min(int(num_global_experts), int(k))
        self.clamp_max = math.log(1.0 / 0.01)
        self.temperature = nn.Parameter(torch.full([1], math.log(1.0 / init_t)))
        self.cosine_projector = nn.Linear(model_dim, proj_dim)
        self.sim_matrix = nn.Parameter(torch.empty(proj_dim, num_global_experts))
        nn.init.normal_(self.sim_matrix, 0.0, 0.01)

    def _logits(self, x, w, b, sim):
        q = F.normalize(F.linear(x, w, b), dim=1)
        keys = F.normalize(sim, dim=0)
        scale = self.temperature.clamp(max=self.clamp_max).exp()
        return (q @ keys) * scale.to(q.dtype)

    def forward(self, x):
        proj = self.cosine_projector
        if self.fp32_gate:
            with torch.autocast(device_type=x.device.type, enabled=False):
                return self._logits(x.float(), proj.weight.float(), proj.bias.float(), self.sim_matrix.float())
        return self._logits(x.to(proj.weight.dtype), proj.weight, proj.bias, self.sim_matrix)


Gate = CosineTopKGate
