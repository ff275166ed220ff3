"""RMSNorm in front of the MoE block (oracle; test infrastructure only).

Restates the torch formula the reference keeps as its own fallback and parity target
(turboquant_utils/norm_kernels.py:186-195, i.e. Qwen3_5MoeRMSNorm.forward): everything in fp32,
weight enters as (1 + weight), one final cast to the activation dtype.
"""

from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    out = x.to(torch.float32)
    out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + eps)
    return (out * (1.0 + weight.float())).type_as(x)
