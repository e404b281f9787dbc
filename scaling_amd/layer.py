"""Pre-norm transformer layer and final-norm wrapper with the reference's module and parameter names.

Mirror of transformer/model/layers/layer.py:45-345, layers/base.py:12-81 and layers/layernorm.py:11-59
at tensor-parallel size 1 with u-muP off (the residual split / add are then identities plus a sum,
core/nn/residual.py:49-65).
"""

from typing import Callable, List, Optional

import torch

from .config import MLPType, TransformerArchitectureConfig
from .nn import ParallelMLP, ParallelSelfAttention, ParallelSwiGLUMLP, get_norm


class InferenceSettings:
    """transformer/data/inference_settings.py:20-54 (control parameters are outside the hot path)."""

    def __init__(self, use_cache: bool, reset_cache: bool, cache_index: int = 0,
                 embedding_layers: Optional[List[int]] = None) -> None:
        self.use_cache = use_cache
        self.reset_cache = reset_cache
        self.cache_index = cache_index
        self.embedding_layers = embedding_layers if embedding_layers is not None else [-1]
        self.control_log_additive_batch = True


class TransformerLayerIO:
    """transformer/model/layers/base.py:12-81: what one layer hands to the next."""

    def __init__(self, activations: torch.Tensor, position_ids: Optional[torch.Tensor],
                 cumulative_seq_lengths_padded: Optional[torch.Tensor] = None,
                 cumulative_seq_lengths: Optional[torch.Tensor] = None, loss_weights: Optional[torch.Tensor] = None,
                 inference_settings: Optional[InferenceSettings] = None, embeddings: Optional[torch.Tensor] = None,
                 embeddings_head: Optional[torch.Tensor] = None,
                 attention_scores_manipulation: Optional[torch.Tensor] = None) -> None:
        self.activations = activations
        self.position_ids = position_ids
        self.cumulative_seq_lengths = cumulative_seq_lengths
        self.cumulative_seq_lengths_padded = cumulative_seq_lengths_padded
        self.loss_weights = loss_weights
        self.inference_settings = inference_settings
        self.embeddings = embeddings
        self.embeddings_head = embeddings_head
        self.attention_scores_manipulation = attention_scores_manipulation


def _check_architecture(cfg: TransformerArchitectureConfig) -> None:
    unsupported = {
        "umup.enable": cfg.umup.enable, "adapter_config": cfg.adapter_config, "lora_config": cfg.lora_config,
        "bitfit_bias_config": cfg.bitfit_bias_config, "fp8_config_attention": cfg.fp8_config_attention,
        "fp8_config_attention_dense_out": cfg.fp8_config_attention_dense_out, "fp8_config_mlp": cfg.fp8_config_mlp,
        "fp8_config_mlp_dense_out": cfg.fp8_config_mlp_dense_out,
    }
    bad = [k for k, v in unsupported.items() if v]
    if bad:
        raise NotImplementedError(f"architecture options outside the hip layer's scope are set: {bad}")


class TransformerLayer(torch.nn.Module):
    def __init__(self, architecture_config: TransformerArchitectureConfig, layer_index: int, topology=None,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = torch.nn.init.xavier_normal_,
                 device: Optional[torch.device] = None) -> None:
        super().__init__()
        if topology is not None:
            raise NotImplementedError("tensor-parallel size 1 only; pass topology=None")
        cfg = architecture_config
        _check_architecture(cfg)
        self.architecture_config = cfg
        self.topology = None
        self.layer_index = layer_index
        dtype = cfg.precision.dtype
        self.input_layernorm = get_norm(cfg.norm_type, cfg.layernorm, cfg.hidden_size, device, dtype)
        self.self_attention = ParallelSelfAttention(
            hidden_size=cfg.hidden_size, num_attention_heads=cfg.num_attention_heads,
            num_local_attention_heads=cfg.num_local_attention_heads,
            local_attention_window_size=cfg.local_attention_window_size, masked_softmax_config=cfg.masked_softmax,
            causal=cfg.causal, dropout_attention_probs=cfg.dropout_attention_probs, rotary_config=cfg.rotary_config(),
            relative_position_embedding_type=cfg.relative_position_embedding_type, bias=cfg.attention_bias,
            device=device, dtype=dtype, init_method=init_method, norm_type=cfg.norm_type,
            key_query_norm=cfg.key_query_norm, layernorm_config=cfg.layernorm, qkv_in_one=cfg.attention_qkv_in_one,
            num_kv_heads=cfg.attention_num_kv_heads, use_matmul=cfg.attention_use_matmul)
        self.dropout_attention = torch.nn.Dropout(cfg.dropout_after_attention)
        self.post_attention_layernorm = get_norm(cfg.norm_type, cfg.layernorm, cfg.hidden_size, device, dtype)
        mlp_class = ParallelSwiGLUMLP if cfg.mlp_type == MLPType.SWIGLU else ParallelMLP   # layer.py:150-189 of the reference
        self.mlp = mlp_class(io_features=cfg.hidden_size, intermediate_feature_factor=cfg.mlp_factor,
                             bias=cfg.mlp_bias, device=device, dtype=dtype, init_method=init_method)
        self.dropout_mlp = torch.nn.Dropout(cfg.dropout_after_mlp)

    def attention_block(self, hidden_state: torch.Tensor, cumulative_seq_lengths: torch.Tensor,
                        position_ids: Optional[torch.Tensor], use_cache: bool = False, reset_cache: bool = False,
                        cache_index: int = 0, attention_scores_manipulation=None,
                        attentions_score_manipulation_log_additive=True) -> torch.Tensor:
        residual = self.input_layernorm(hidden_state)
        residual = self.self_attention(residual, cumulative_seq_lengths=cumulative_seq_lengths,
                                       attention_scores_manipulation=attention_scores_manipulation,
                                       attentions_score_manipulation_log_additive=attentions_score_manipulation_log_additive,
                                       position_ids=position_ids, use_cache=use_cache, reset_cache=reset_cache,
                                       cache_index=cache_index)
        return self.dropout_attention(residual) + hidden_state

    def mlp_block(self, hidden_state: torch.Tensor) -> torch.Tensor:
        residual = self.mlp(self.post_attention_layernorm(hidden_state))
        return self.dropout_mlp(residual) + hidden_state

    def decode_step(self, hidden_state: torch.Tensor, position_ids: torch.Tensor, cache_index: int = 0,
                    advance: bool = True) -> torch.Tensor:
        """Cached single-token step on plain tensors, free of host synchronisation (HIP-graph capturable)."""
        h = hidden_state + self.self_attention.decode_forward(self.input_layernorm(hidden_state), position_ids, cache_index,
                                                              advance=advance)
        return h + self.mlp(self.post_attention_layernorm(h))

    def forward(self, x: TransformerLayerIO) -> TransformerLayerIO:
        s = x.inference_settings
        use_cache, reset_cache, cache_index = (False, False, 0) if s is None else (s.use_cache, s.reset_cache, s.cache_index)
        assert x.cumulative_seq_lengths is not None
        h = self.attention_block(x.activations, x.cumulative_seq_lengths, x.position_ids, use_cache=use_cache,
                                 reset_cache=reset_cache, cache_index=cache_index,
                                 attention_scores_manipulation=x.attention_scores_manipulation)
        h = self.mlp_block(h)
        return TransformerLayerIO(activations=h, cumulative_seq_lengths=x.cumulative_seq_lengths,
                                  cumulative_seq_lengths_padded=x.cumulative_seq_lengths_padded,
                                  attention_scores_manipulation=x.attention_scores_manipulation,
                                  loss_weights=x.loss_weights, position_ids=x.position_ids,
                                  inference_settings=x.inference_settings, embeddings=x.embeddings)


class LayerNormWrapper(torch.nn.Module):
    """Final norm, transformer/model/layers/layernorm.py:11-59 (sub-module name `norm`)."""

    def __init__(self, architecture_config: TransformerArchitectureConfig, layer_index: int, topology=None,
                 umup_on_residual: Optional[bool] = None, device: Optional[torch.device] = None) -> None:
        super().__init__()
        cfg = architecture_config
        self.architecture_config = cfg
        self.layer_index = layer_index
        self.norm = get_norm(cfg.norm_type, cfg.layernorm, cfg.hidden_size, device, cfg.precision.dtype, topology=topology)

    def forward(self, x: TransformerLayerIO) -> TransformerLayerIO:
        return TransformerLayerIO(activations=self.norm(x.activations), position_ids=x.position_ids,
                                  cumulative_seq_lengths=x.cumulative_seq_lengths,
                                  cumulative_seq_lengths_padded=x.cumulative_seq_lengths_padded,
                                  loss_weights=x.loss_weights, inference_settings=x.inference_settings,
                                  embeddings=x.embeddings)
