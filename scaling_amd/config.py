"""Configuration surface of the layer hot path.

Field names, defaults and enum values follow the reference's frozen Pydantic configs so that an
existing `transformer_architecture` block validates unchanged; the only addition is the
`MaskedSoftmaxKernel.HIP` member that selects the gfx950 kernels of this package.

Reference: core/config/base.py:39-91 (BaseConfig), core/nn/masked_softmax/masked_softmax_config.py:8-36,
core/nn/rotary_config.py:6-11, core/nn/norm/layernorm_config.py:8-20, core/nn/norm/get_norm.py:12-14,
core/nn/attention/attention.py:274-277, transformer/context/config.py:28-48 and :229-432.
"""

import json
from enum import Enum
from pathlib import Path
from typing import Any, Optional, Type, TypeVar, Union

import torch
import yaml
from pydantic import BaseModel, ConfigDict, Field

T = TypeVar("T", bound="BaseConfig")


def _merge(dst: dict, src: dict) -> None:
    for key, value in src.items():
        if isinstance(value, dict):
            _merge(dst.setdefault(key, {}), value)
        else:
            dst[key] = value


def _plain(x: Any) -> Any:
    if isinstance(x, dict):
        return {k: _plain(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_plain(v) for v in x]
    if isinstance(x, Enum):
        return x.value
    if isinstance(x, Path):
        return str(x)
    return x


class BaseConfig(BaseModel):
    """Immutable config; unknown keys are validation errors; enums serialise by value."""

    model_config = ConfigDict(extra="forbid", frozen=True, protected_namespaces=())

    def as_dict(self) -> dict:
        return _plain(self.model_dump())

    @classmethod
    def from_dict(cls: Type[T], d: dict, overwrite_values: Optional[dict] = None) -> T:
        if overwrite_values is not None:
            _merge(d, overwrite_values)
        return cls(**d)

    def as_str(self) -> str:
        return json.dumps(self.as_dict())

    @classmethod
    def from_str(cls: Type[T], s: str) -> T:
        return cls.from_dict(json.loads(s))

    @classmethod
    def from_yaml(cls: Type[T], yml_filename: Union[str, Path], overwrite_values: Optional[dict] = None) -> T:
        with open(yml_filename) as f:
            d = yaml.safe_load(f)
        return cls.from_dict(d, overwrite_values)

    def save(self, out_file: Union[str, Path], indent: int = 4) -> None:
        with open(out_file, "w", encoding="UTF-8") as f:
            json.dump(self.as_dict(), f, indent=indent)


class MaskedSoftmaxKernel(Enum):
    TORCH = "torch"
    FLASH_ATTENTION = "flash_attention"
    HIP = "hip"  # hand-written gfx950 kernels of this package


class MaskedSoftmaxConfig(BaseConfig):
    kernel: MaskedSoftmaxKernel = Field(MaskedSoftmaxKernel.TORCH, description="attention core implementation")
    softmax_in_fp32: bool = Field(False, description="fp32 softmax (the hip kernel always computes in fp32)")
    scale: float = Field(1.0, description="factor the scores are multiplied with before the softmax")
    deterministic_flash_attn_bwd: bool = Field(False, description="flash-attention only; the hip backward is always deterministic")


class RotaryConfig(BaseConfig):
    dimensions: int = Field(0, description="number of rotated features per head")
    base: int = Field(10000, description="")
    max_seq_length: int = Field(2048, description="rows of the cos / sin tables")


class LayerNormOptimizationType(Enum):
    TORCH = "torch"


class LayerNormConfig(BaseConfig):
    optimization_type: LayerNormOptimizationType = Field(LayerNormOptimizationType.TORCH, description="")
    layernorm_epsilon: float = Field(1.0e-5, description="value added to the denominator for numerical stability")


class NormType(Enum):
    LAYERNORM = "layernorm"
    RMS = "rms"


class RelativePositionEmbeddingType(Enum):
    NONE = "none"
    ROTARY = "rotary"
    ROTARY_COMPLEX = "rotary_complex"


class Precision(Enum):
    FLOAT16 = "float16"
    BFLOAT16 = "bfloat16"
    FLOAT32 = "float32"

    @property
    def dtype(self) -> torch.dtype:
        return {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}[self.value]


class MLPType(Enum):
    DEFAULT = "default"
    SWIGLU = "swiglu"


class UMuPConfig(BaseConfig):
    enable: bool = Field(False, description="enables u-mup (not supported by the hip layer)")
    allow_non_umup_params: bool = Field(False, description="")
    normalize_depth_to_num_layers: bool = Field(False, description="")
    attn_mult: float = Field(1.0, description="")
    act_mult: float = Field(1.0, description="")
    residual_mult: float = Field(1.0, description="")
    residual_attn_ratio: float = Field(1.0, description="")
    loss_mult: float = Field(1.0, description="")


class TransformerArchitectureConfig(BaseConfig):
    """Same fields as the reference's architecture config.  Blocks that configure subsystems outside
    the layer hot path (fp8, bitfit, softprompt, adapter, LoRA, embedding head) are accepted as plain
    dicts so existing files validate; the hip layer refuses to be built when one of them is set."""

    vocab_size: int = Field(0, description="")
    vocab_file: Optional[Path] = Field(None, description="")
    hidden_size: int = Field(0, description="")
    num_layers: int = Field(0, description="")
    num_attention_heads: int = Field(0, description="")
    num_local_attention_heads: int = Field(0, description="")
    local_attention_window_size: Optional[int] = Field(None, description="")
    rotary_embedding_base: int = Field(10000, description="")
    rotary_percentage: float = Field(1.0, description="")
    sequence_length: int = Field(2048, description="")
    norm_type: NormType = Field(NormType.LAYERNORM, description="")
    relative_position_embedding_type: RelativePositionEmbeddingType = Field(RelativePositionEmbeddingType.ROTARY, description="")
    mlp_type: MLPType = Field(MLPType.DEFAULT, description="")
    mlp_factor: float = Field(4.0, description="")
    attention_bias: bool = Field(True, description="")
    attention_qkv_in_one: bool = Field(True, description="")
    attention_num_kv_heads: Optional[int] = Field(None, description="")
    attention_use_matmul: bool = Field(False, description="")
    reset_attention_mask: bool = Field(True, description="")
    reset_position_ids: bool = Field(True, description="")
    mlp_bias: bool = Field(True, description="")
    key_query_norm: bool = Field(False, description="")
    weight_tying: bool = Field(True, description="")
    masked_softmax: MaskedSoftmaxConfig = Field(MaskedSoftmaxConfig(), description="")
    layernorm: LayerNormConfig = Field(LayerNormConfig(), description="")
    precision: Precision = Field(Precision.FLOAT32, description="")
    fp8_config_attention: Optional[dict] = Field(None, description="")
    fp8_config_attention_dense_out: Optional[dict] = Field(None, description="")
    fp8_config_mlp: Optional[dict] = Field(None, description="")
    fp8_config_mlp_dense_out: Optional[dict] = Field(None, description="")
    fp8_config_lm_head: Optional[dict] = Field(None, description="")
    dropout_embedding: float = Field(0.0, ge=0.0, le=1.0, description="")
    dropout_attention_probs: float = Field(0.0, ge=0.0, le=1.0, description="")
    dropout_after_attention: float = Field(0.0, ge=0.0, le=1.0, description="")
    dropout_after_mlp: float = Field(0.0, ge=0.0, le=1.0, description="")
    bitfit_bias_config: Optional[dict] = Field(None, description="")
    finetunable_token_ids: list = Field(default_factory=list, description="")
    image_encoder: bool = Field(False, description="")
    dropout_image_encoder: float = Field(0.0, ge=0.0, le=1.0, description="")
    softprompt_config: Optional[dict] = Field(None, description="")
    adapter_config: Optional[dict] = Field(None, description="")
    lora_config: Optional[dict] = Field(None, description="")
    embedding_head_config: Optional[dict] = Field(None, description="")
    lm_head: bool = Field(True, description="")
    causal: bool = Field(True, description="")
    umup: UMuPConfig = Field(UMuPConfig(), description="")

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def rotary_config(self) -> RotaryConfig:
        """transformer/model/layers/layer.py:95-103."""
        return RotaryConfig(dimensions=int(self.rotary_percentage * self.head_dim),
                            max_seq_length=self.sequence_length, base=self.rotary_embedding_base)


def architecture_from_config_file(config_file: Union[str, Path], kernel: Optional[str] = "hip") -> TransformerArchitectureConfig:
    """Reads the `transformer_architecture` block of a training config file.

    The reference's inference loader overwrites `masked_softmax.kernel` from a boolean
    (transformer/inference/inference_model.py:48-58); here the kernel is a parameter (None keeps the
    value stored in the file)."""
    with open(config_file) as f:
        d = yaml.safe_load(f)
    arch = d["transformer_architecture"]
    if kernel is not None:
        arch.setdefault("masked_softmax", {})["kernel"] = kernel
    return TransformerArchitectureConfig.from_dict(arch)
