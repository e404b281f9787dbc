"""TEST INFRASTRUCTURE (see oracle/__init__.py).  LM head and weighted token-level cross entropy.

Restates, with explicit log-sum-exp arithmetic (so that torch.nn.functional.cross_entropy stays available as an
independent library check), transformer/model/losses/cross_entropy.py:18-32 and :58-88 and the projection of
transformer/model/layers/lm_head.py:58-59.
"""

from typing import Dict, Tuple

import torch


def token_losses(logits: torch.Tensor, targets: torch.Tensor, ignore_index: int = -100) -> torch.Tensor:
    """cross_entropy.py:24-28: per-row -log softmax(x)[t] on ``logits.float()`` (:74); rows whose target is
    ``ignore_index`` (torch's default) contribute 0."""
    x = logits.float() if logits.dtype != torch.float64 else logits
    mx = x.max(dim=-1, keepdim=True).values
    lse = (x - mx).exp().sum(dim=-1).log() + mx.squeeze(-1)
    ignored = targets == ignore_index
    safe_t = torch.where(ignored, torch.zeros_like(targets), targets)
    picked = x.gather(-1, safe_t.unsqueeze(-1)).squeeze(-1)
    return torch.where(ignored, torch.zeros_like(lse), lse - picked)


def cross_entropy_loss(activations: torch.Tensor, target_token_ids: torch.Tensor,
                       loss_weights: torch.Tensor) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """cross_entropy.py:58-88: loss = sum(losses * w) / sum(w) (:30); accuracy = hit rate of argmax over the
    tokens with w > 0 (:81-86)."""
    w = loss_weights.float().flatten() if activations.dtype != torch.float64 else loss_weights.double().flatten()
    logits = activations.reshape(-1, activations.shape[-1])
    logits = logits.float() if logits.dtype != torch.float64 else logits
    t = target_token_ids.flatten()
    losses = token_losses(logits, t)
    loss = torch.sum(losses * w) / w.sum()
    mask = (w > 0).to(w.dtype)
    hits = (logits.argmax(-1) == t).to(w.dtype)
    return loss, {"accuracy": torch.sum(hits * mask) / mask.sum()}


def lm_head(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """lm_head.py:58-59: logits = x @ weight^T, no bias (ColumnParallelLinear at model-parallel size 1)."""
    return torch.nn.functional.linear(x, weight)
