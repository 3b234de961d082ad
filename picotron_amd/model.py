"""The SwiGLU MLP that expert and shared-expert weights live in.

Mirrors picotron/model.py:236-258 (class ``MLP``): three bias-free linears ``up_proj``, ``gate_proj``,
``down_proj`` and ``down(silu(gate(x)) * up(x))``.  The forward runs the grouped SwiGLU kernels with
a single expert; there is no eager path.
"""

import math

import torch
import torch.nn as nn


class MLP(nn.Module):
    def __init__(self, config) -> None:
        super().__init__()
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)
        self.reset_parameters()

    def reset_parameters(self):
        for lin in (self.up_proj, self.gate_proj, self.down_proj):
            bound = math.sqrt(1.0 / lin.weight.size(1))
            torch.nn.init.uniform_(lin.weight, -bound, bound)

    def forward(self, x):
        from picotron_amd.expert_parallel import megakernel

        lead = x.shape[:-1]
        rows = x.reshape(-1, x.shape[-1])
        counts = torch.full((1,), rows.shape[0], dtype=torch.int64, device=rows.device)
        y = megakernel.fused_moe(
            rows, counts, self.gate_proj.weight.unsqueeze(0), self.up_proj.weight.unsqueeze(0), self.down_proj.weight.unsqueeze(0)
        )
        return y.reshape(*lead, y.shape[-1])
