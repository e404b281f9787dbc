"""Decoder stack and greedy generation with a pre-allocated KV cache.

Mirrors the inference path of the reference at tensor-parallel size 1: layer order EmbeddingInput ->
N x TransformerLayer -> LayerNormWrapper -> LM head (transformer/model/model.py:84-181), the no-grad
layer loop (core/nn/parallel_module/inference_module.py:100-109), prefill + one-token-per-step cached
decoding with greedy sampling (transformer/inference/inference_model.py:223-263, inference/sample.py:5-6)
and the per-layer checkpoint files `model_state_layer_{i}_{Class}.pt`
(core/nn/parallel_module/partitioned_module.py:246-408).  Unlike the reference the cached path accepts
a batch of prompts of equal length (the reference asserts batch size 1, attention.py:855-857).
Embedding lookup, LM head matmul and arg-max stay on PyTorch-ROCm.
"""

import glob
import os
import re
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from .config import TransformerArchitectureConfig, architecture_from_config_file
from .data import get_cumulative_seq_lengths, get_position_ids
from .layer import InferenceSettings, LayerNormWrapper, TransformerLayer, TransformerLayerIO
from .loss import TransformerLMHead

# class names written by older versions of the reference (partitioned_module.py:25-32)
LEGACY_CLASS_NAMES = {"LuminousEmbeddingInput": "EmbeddingInput", "LuminousLayer": "TransformerLayer",
                      "LuminousLMHead": "TransformerLMHead", "LuminousLMHeadTied": "TransformerLMHeadTied"}


def sample_argmax(logits: torch.Tensor) -> torch.Tensor:
    """transformer/inference/sample.py:5-6: greedy choice at the last position, one id per batch row."""
    return torch.argmax(logits, dim=-1)[:, -1]


class EmbeddingInput(torch.nn.Module):
    def __init__(self, cfg: TransformerArchitectureConfig, device=None):
        super().__init__()
        self.embedding = torch.nn.Embedding(cfg.vocab_size, cfg.hidden_size, device=device, dtype=cfg.precision.dtype)

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return self.embedding(token_ids)


class TransformerInferenceModule(torch.nn.Module):
    """`_layers[i]` holds the i-th layer in the reference's order, so checkpoint indices line up."""

    def __init__(self, architecture_config: TransformerArchitectureConfig, device: Union[str, torch.device] = "cuda",
                 init_std: float = 0.02, seed: Optional[int] = None) -> None:
        super().__init__()
        cfg = architecture_config
        self.architecture_config = cfg
        self.device = torch.device(device)
        gen = None
        if seed is not None:
            gen = torch.Generator(device="cpu").manual_seed(seed)

        def init(w: torch.Tensor) -> torch.Tensor:
            if gen is None:
                return torch.nn.init.normal_(w, mean=0.0, std=init_std)
            w.data.copy_((torch.randn(w.shape, generator=gen) * init_std).to(w.dtype))
            return w

        layers: List[torch.nn.Module] = [EmbeddingInput(cfg, self.device)]
        for i in range(cfg.num_layers):
            layers.append(TransformerLayer(cfg, layer_index=i, init_method=init, device=self.device))
        layers.append(LayerNormWrapper(cfg, layer_index=cfg.num_layers, device=self.device))
        layers.append(TransformerLMHead(cfg, device=self.device))
        self._layers = torch.nn.ModuleList(layers)
        init(self._layers[0].embedding.weight)
        if cfg.weight_tying:
            self._layers[-1].linear.weight = self._layers[0].embedding.weight
        else:
            init(self._layers[-1].linear.weight)
        # core/nn/parallel_module/inference_module.py:98: an inference module is in eval mode from construction, so the
        # dropouts of a training config (after attention, after the MLP, on the attention probabilities) are off
        self.eval()

    # ---- checkpoint files ------------------------------------------------------------------------------
    def load_checkpoint(self, checkpoint_dir: Union[str, Path]) -> None:
        """Loads `model_state_layer_{index}_{ClassName}.pt` files written by the reference."""
        pattern = re.compile(r"model_state_layer_(\d+)_([A-Za-z]+)\.pt$")
        found: Dict[int, str] = {}
        for f in glob.glob(os.path.join(str(checkpoint_dir), "model_state_layer_*.pt")):
            m = pattern.search(os.path.basename(f))
            if m:
                found[int(m.group(1))] = f
        for idx, layer in enumerate(self._layers):
            if idx not in found:
                if idx == len(self._layers) - 1 and self.architecture_config.weight_tying:
                    continue
                raise FileNotFoundError(f"no checkpoint file for layer {idx} in {checkpoint_dir}")
            sd = torch.load(found[idx], map_location=self.device, weights_only=True)
            cls = pattern.search(os.path.basename(found[idx])).group(2)
            cls = LEGACY_CLASS_NAMES.get(cls, cls)
            if cls.startswith("TransformerLMHead"):
                sd = {("linear.weight" if k in ("embedding.weight", "linear.weight") else k): v for k, v in sd.items()}
            layer.load_state_dict(sd, strict=True)

    def save_checkpoint(self, checkpoint_dir: Union[str, Path]) -> None:
        os.makedirs(str(checkpoint_dir), exist_ok=True)
        names = ["EmbeddingInput"] + ["TransformerLayer"] * self.architecture_config.num_layers + ["LayerNormWrapper", "TransformerLMHead"]
        for idx, (layer, name) in enumerate(zip(self._layers, names)):
            torch.save(layer.state_dict(), os.path.join(str(checkpoint_dir), f"model_state_layer_{idx}_{name}.pt"))

    @classmethod
    def from_checkpoint(cls, checkpoint_dir: Union[str, Path], device="cuda", config_file: Optional[Path] = None):
        config_file = Path(checkpoint_dir) / "config.yml" if config_file is None else config_file
        module = cls(architecture_from_config_file(config_file, kernel="hip"), device=device)
        module.load_checkpoint(checkpoint_dir)
        return module

    # ---- forward -------------------------------------------------------------------------------------------
    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, position_ids: Optional[torch.Tensor] = None,
                cumulative_seq_lengths: Optional[torch.Tensor] = None,
                inference_settings: Optional[InferenceSettings] = None, last_token_only: bool = False) -> torch.Tensor:
        """token_ids [b, s] -> logits [b, s, vocab]; ids / lengths default to the reference's batch
        construction (transformer/data/text_dataset_batch.py:110-126).  last_token_only=True applies the
        final norm and the LM head to the last position only (logits [b, 1, vocab]): greedy decoding reads
        nothing else, and a [32, 4096, 128256] logits tensor would not be worth its 33 GB."""
        token_ids = token_ids.to(self.device)
        if cumulative_seq_lengths is None:
            cumulative_seq_lengths = get_cumulative_seq_lengths(token_ids, self.architecture_config.reset_attention_mask)
        if position_ids is None:
            position_ids = get_position_ids(token_ids, self.architecture_config.reset_position_ids)
        x = TransformerLayerIO(activations=self._layers[0](token_ids), position_ids=position_ids.to(self.device),
                               cumulative_seq_lengths=cumulative_seq_lengths.to(self.device),
                               inference_settings=inference_settings)
        for layer in self._layers[1:-2]:
            x = layer(x)
        if last_token_only:
            x.activations = x.activations[:, -1:, :].contiguous()
        x = self._layers[-2](x)
        return self._layers[-1].linear(x.activations)

    def logits(self, input_tokens: Sequence[int]) -> torch.Tensor:
        return self.forward(torch.tensor([list(input_tokens)])).squeeze(0)

    # ---- generation ---------------------------------------------------------------------------------------
    @torch.no_grad()
    def generate_graph(self, max_tokens: int, input_tokens: Union[Sequence[int], torch.Tensor]) -> List[List[int]]:
        """Greedy cached completion whose per-token step (all layers, LM head, arg-max, cache append) is
        captured once as a HIP graph and replayed: the host issues one launch per token instead of a few
        hundred.  No early stop; returns the completion ids per prompt.  Same arithmetic as `generate`."""
        ids = torch.as_tensor(input_tokens)
        if ids.dim() == 1:
            ids = ids.unsqueeze(0)
        ids = ids.to(self.device)
        b, n_prompt = ids.shape
        layers = list(self._layers[1:-2])
        assert n_prompt + max_tokens <= layers[0].self_attention._cache_capacity(), "KV cache too small"
        logits = self.forward(ids, inference_settings=InferenceSettings(use_cache=True, reset_cache=True), last_token_only=True)
        tok = sample_argmax(logits).unsqueeze(1).contiguous()             # [b, 1] static buffer
        pos = torch.full((b,), n_prompt, dtype=torch.int64, device=self.device)
        out = torch.zeros(b, max_tokens, dtype=torch.int64, device=self.device)
        out[:, 0] = tok[:, 0]
        step = torch.ones(1, dtype=torch.int64, device=self.device)      # column of `out` the next token goes to
        if max_tokens == 1:
            return out.tolist()
        for layer in layers:                                              # decode workspaces exist before capture
            att = layer.self_attention
            cache = att.cache[0]
            if cache.workspace is None:
                from . import ops
                cache.workspace = ops.decode_workspace(b, att.num_attention_heads, att.hidden_size_per_attention_head,
                                                       cache.max_ctx, self.device)

        # every layer has seen the same tokens: one device-side context-length vector serves all caches and is
        # advanced once per step instead of once per layer
        shared_ctx = layers[0].self_attention.cache[0].ctx_len
        for layer in layers[1:]:
            layer.self_attention.cache[0].ctx_len = shared_ctx

        from .nn import RMSNorm
        from . import ops
        final_norm = self._layers[-2].norm
        fuse_add_norm = all(isinstance(n, RMSNorm) for layer in layers for n in (layer.input_layernorm, layer.post_attention_layernorm)) \
            and isinstance(final_norm, RMSNorm)

        # arg-max over the vocabulary by the streaming cross-entropy kernel (first index of the maximum, as
        # torch.argmax): ~8 us for [32, 128256] against ~48 us for torch's reduction
        no_target = torch.zeros(b, dtype=torch.int64, device=self.device)

        def one_step():
            h = self._layers[0](tok)
            shared_ctx.add_(1)
            if fuse_add_norm:
                # every residual add is folded into the RMSNorm that follows it (same rounding points as the
                # separate add and norm of layer.decode_step)
                n = layers[0].input_layernorm(h)
                for i, layer in enumerate(layers):
                    a = layer.self_attention.decode_forward(n, pos, advance=False)
                    h, n = ops.add_rms_norm(h, a, layer.post_attention_layernorm.weight, layer.post_attention_layernorm.eps)
                    nxt_norm = layers[i + 1].input_layernorm if i + 1 < len(layers) else final_norm
                    h, n = ops.add_rms_norm(h, layer.mlp(n), nxt_norm.weight, nxt_norm.eps)
                lg = self._layers[-1].linear(n)
            else:
                for layer in layers:
                    h = layer.decode_step(h, pos, advance=False)
                lg = self._layers[-1].linear(final_norm(h))
            nxt = ops.cross_entropy_forward(lg.view(b, -1), no_target)[1].to(torch.int64).view(b, 1)
            out.index_copy_(1, step, nxt)
            tok.copy_(nxt)
            pos.add_(1)
            step.add_(1)

        n_eager = min(2, max_tokens - 1)                                  # warm-up steps run eagerly
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(n_eager):
                one_step()
        torch.cuda.current_stream().wait_stream(side)
        remaining = max_tokens - 1 - n_eager
        if remaining > 0:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                one_step()
            for _ in range(remaining):   # capture only records; every remaining token is one replay
                graph.replay()
        for i, layer in enumerate(layers):
            cache = layer.self_attention.cache[0]
            cache.length = n_prompt + max_tokens - 1
            if i > 0:
                cache.ctx_len = shared_ctx.clone()      # each cache owns its lengths again
        return out.tolist()

    @torch.no_grad()
    def generate(self, max_tokens: int, input_tokens: Union[Sequence[int], torch.Tensor], use_cache: bool = True,
                 stop_tokens: Optional[Sequence[int]] = None) -> Tuple[List[List[int]], torch.Tensor]:
        """Greedy completion.  input_tokens: one prompt (list of ids) or a [batch, length] tensor of prompts
        of equal length.  Returns (completion ids per prompt, logits [batch, steps, vocab]).  A batch of 1
        stops at the first id in `stop_tokens` (the reference's rule); larger batches run all steps."""
        ids = torch.as_tensor(input_tokens)
        if ids.dim() == 1:
            ids = ids.unsqueeze(0)
        ids = ids.to(self.device)
        b, n_prompt = ids.shape
        stop = set(stop_tokens or [])
        completions: List[List[int]] = [[] for _ in range(b)]
        step_logits = []
        if use_cache:
            settings = InferenceSettings(use_cache=True, reset_cache=True)
            cur, pos = ids, None
            for k in range(max_tokens):
                logits = self.forward(cur, position_ids=pos, inference_settings=settings, last_token_only=True)
                nxt = sample_argmax(logits)
                step_logits.append(logits[:, -1, :])
                for i, t in enumerate(nxt.tolist()):
                    completions[i].append(t)
                settings = InferenceSettings(use_cache=True, reset_cache=False)
                cur = nxt.unsqueeze(1)
                pos = torch.full((b, 1), n_prompt + k, dtype=torch.int64, device=self.device)
                if b == 1 and completions[0][-1] in stop:
                    break
        else:
            cur = ids
            for _ in range(max_tokens):
                logits = self.forward(cur)
                nxt = sample_argmax(logits)
                step_logits.append(logits[:, -1, :])
                for i, t in enumerate(nxt.tolist()):
                    completions[i].append(t)
                cur = torch.cat([cur, nxt.unsqueeze(1)], dim=-1)
                if b == 1 and completions[0][-1] in stop:
                    break
        return completions, torch.stack(step_logits, dim=1)
