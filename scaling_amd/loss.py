"""Loss side of the path: LM head and token-level cross entropy on the HIP kernel.

Mirrors transformer/model/losses/cross_entropy.py:12-88 (``CrossEntropyLoss``) and
transformer/model/layers/lm_head.py:15-68 (``TransformerLMHead``, parameter ``linear.weight``), plus a fused
entry point that never materialises the ``[tokens, vocab]`` logits.  u-muP scaling is outside this layer's scope
and raises.
"""

from typing import Dict, Optional, Tuple

import torch

from . import ops
from .config import TransformerArchitectureConfig
from .layer import TransformerLayerIO


class CrossEntropyLoss(torch.nn.Module):
    """``forward(output, batch) -> (loss, {"accuracy": ...})`` as losses/cross_entropy.py:58-88.

    ``output.activations`` are logits ``[b, s, vocab]``; ``batch.target_token_ids`` ``[b, s]`` int64 and
    ``batch.loss_weights`` ``[b, s]``.  loss = sum(losses * w) / sum(w) (:30), accuracy = weighted hit rate of the
    row argmax over the tokens with w > 0 (:81-86)."""

    def __init__(self, loss_config=None, umup_config=None) -> None:
        super().__init__()
        if umup_config is not None and getattr(umup_config, "enable", False):
            raise NotImplementedError("u-muP loss scaling is not part of the hip layer")

    def forward(self, output: TransformerLayerIO, batch) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
        assert batch.target_token_ids is not None, "target_token_ids not set in batch"
        assert batch.loss_weights is not None, "loss_weights not set in batch"
        logits = output.activations.reshape(-1, output.activations.shape[-1])
        targets = batch.target_token_ids.flatten()
        weights = batch.loss_weights.float().flatten()
        losses, argmax = ops.cross_entropy(logits, targets)
        loss = torch.sum(losses * weights) / weights.sum()
        return loss, {"accuracy": _accuracy(argmax, targets, weights)}


def _accuracy(argmax: torch.Tensor, targets: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    mask = (weights > 0).float()
    hits = (argmax.to(torch.int64) == targets).float()
    return torch.sum(hits * mask) / mask.sum()


class TransformerLMHead(torch.nn.Module):
    """Untied output projection, layers/lm_head.py:15-68: ``linear.weight`` is ``[vocab, hidden]``, no bias.

    ``forward`` keeps the reference behaviour (logits on a PyTorch GEMM); ``loss`` fuses the head with the cross
    entropy so the logits of only ``chunk_rows`` tokens exist at any time."""

    def __init__(self, architecture_config: TransformerArchitectureConfig, init_method=None, topology=None,
                 device: Optional[torch.device] = None) -> None:
        super().__init__()
        cfg = architecture_config
        if len(getattr(cfg, "finetunable_token_ids", []) or []) > 0:
            raise NotImplementedError("finetunable_token_ids masks are not part of the hip layer")
        self.linear = torch.nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False, device=device, dtype=cfg.precision.dtype)
        if init_method is not None:
            init_method(self.linear.weight)

    def forward(self, x: TransformerLayerIO) -> TransformerLayerIO:
        return TransformerLayerIO(activations=self.linear(x.activations), position_ids=x.position_ids,
                                  cumulative_seq_lengths=x.cumulative_seq_lengths,
                                  cumulative_seq_lengths_padded=x.cumulative_seq_lengths_padded,
                                  loss_weights=x.loss_weights, inference_settings=x.inference_settings,
                                  embeddings=x.embeddings)

    def loss(self, x: TransformerLayerIO, batch, chunk_rows: int = 8192) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
        h = x.activations.reshape(-1, x.activations.shape[-1])
        targets = batch.target_token_ids.flatten()
        weights = batch.loss_weights.float().flatten()
        loss, argmax = ops.linear_cross_entropy(h, self.linear.weight, targets, weights, chunk_rows)
        return loss, {"accuracy": _accuracy(argmax, targets, weights)}
