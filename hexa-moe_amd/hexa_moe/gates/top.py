"""Linear top-k router (reference: hexa_moe_cuda/hexa_moe/gates/top.py:5-22).

logits = x @ wg^T with a bias-free projection `wg` ([E, model_dim]); with fp32_gate the projection is
created and evaluated in fp32 whatever the tokens' type.  The state-dict key stays `wg.weight`.
"""
import torch
from torch import nn

_ALLOWED_EXTRA = frozenset({"capacity_factor", "gate_noise"})


class LinearTopKGate(nn.Module):
    def __init__(self, model_dim, num_global_experts, k=1, fp32_gate=False, **options):
        super().__init__()
        unknown = set(options) - _ALLOWED_EXTRA
        if unknown:
            raise Exception("Unrecognized argument provided to Gating module: %s" % sorted(unknown)[0])
        self.fp32_gate = bool(fp32_gate)
        self.top_k = min(int(num_global_experts), int(k))
        self.wg = nn.Linear(model_dim, num_global_experts, bias=False,
                            dtype=torch.float32 if self.fp32_gate else None)

    def forward(self, x):
        if self.fp32_gate:
            # keep the router out of autocast: the expert choice is made on fp32 logits
            with torch.autocast(device_type=x.device.type, enabled=False):
                return nn.functional.linear(x.float(), self.wg.weight.float())
        return self.wg(x.to(self.wg.weight.dtype))


Gate = LinearTopKGate
