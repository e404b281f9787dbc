"""Oracle (test infrastructure): MLP activations.

Follows core/nn/mlp.py of the reference.
"""

from typing import Optional

import torch
import torch.nn.functional as F


def swiglu(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """core/nn/mlp.py:248-249: silu(x) * gate."""
    return F.silu(x) * gate


def swiglu_grad(x: torch.Tensor, gate: torch.Tensor, dout: torch.Tensor):
    """Closed-form gradient of `swiglu` (what autograd derives from mlp.py:248-249).

    d/dx = dout * gate * sigma(x) * (1 + x * (1 - sigma(x))),  d/dgate = dout * silu(x).
    """
    sig = torch.sigmoid(x)
    return dout * gate * sig * (1 + x * (1 - sig)), dout * x * sig


def swiglu_mlp(x, w_in, w_gate, w_out, b_in=None, b_gate=None, b_out=None):
    """core/nn/mlp.py:269-282 at tensor-parallel size 1."""
    return F.linear(swiglu(F.linear(x, w_in, b_in), F.linear(x, w_gate, b_gate)), w_out, b_out)


def gelu_mlp(x, w_in, w_out, b_in: Optional[torch.Tensor] = None, b_out: Optional[torch.Tensor] = None):
    """core/nn/mlp.py:107-122 (`ParallelMLP` with the default GELU) at tensor-parallel size 1."""
    return F.linear(F.gelu(F.linear(x, w_in, b_in)), w_out, b_out)
