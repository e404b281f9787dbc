"""Oracle (test infrastructure): normalisation layers.

Follows core/nn/norm/rms_norm.py and core/nn/norm/layernorm.py of the reference.
"""

from typing import Optional

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """core/nn/norm/rms_norm.py:47-50.

    x * rsqrt(mean(x^2) + eps) evaluated in x's dtype (the float round trip on
    line 49 changes nothing), then multiplied by the weight.
    """
    out = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    out = out.float().type_as(x)
    return out * weight


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float = 1e-5):
    """core/nn/norm/layernorm.py:75-86 (`torch` optimisation type)."""
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), weight, bias, eps)
