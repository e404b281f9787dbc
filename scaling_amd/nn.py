"""Drop-in layer modules at tensor-parallel size 1 backed by the gfx950 kernels.

Constructor arguments, forward signatures, sub-module names and parameter names follow the
reference's modules (see each class), so state dicts and the per-layer checkpoint files of the
reference load unchanged.  Linear projections stay on PyTorch-ROCm matmul.  Everything else on the
path (norm, rotary, attention core, SwiGLU) runs the HIP kernels of this package; options the kernels
do not cover raise `NotImplementedError` instead of silently taking another path.
"""

import math
from typing import Callable, Dict, Optional, Tuple

import torch
import torch.nn.functional as F

from . import ops
from .config import (LayerNormConfig, MaskedSoftmaxConfig, MaskedSoftmaxKernel, NormType,
                     RelativePositionEmbeddingType, RotaryConfig)

InitMethod = Callable[[torch.Tensor], torch.Tensor]


def _default_device(device, topology=None) -> torch.device:
    if topology is not None:
        raise NotImplementedError("scaling_amd modules cover tensor-parallel size 1 only; pass topology=None")
    if device is not None:
        return torch.device(device)
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")


_CHECKED: Dict[str, tuple] = {}


def _checked_once(kind: str, t: torch.Tensor, extra: tuple, compute: Callable[[], bool]) -> bool:
    """Result of a device-side validation of tensor `t` that needs a host read-back: computed once per tensor and
    kind, so the layers of one forward share it.  The tensor is identified by address, layout and version counter,
    and the last validated one is kept alive here, so its memory cannot be handed to another tensor meanwhile.

    Limits: tensors created under torch.inference_mode() carry no version counter and are validated on every
    call; writes through this package's raw-pointer kernels (ops.*) do not bump the counter, so a tensor that is
    overwritten in place that way keeps its cached answer; while the current stream is being captured into a graph
    a read-back is impossible, so a tensor that is not the one validated last is passed as valid (the kernels
    clamp out-of-range position ids instead of faulting): validate once before the capture."""
    try:
        version = t._version
    except RuntimeError:                   # inference tensors do not track a version counter
        version = None
    key = (t.data_ptr(), tuple(t.shape), tuple(t.stride()), version, t.device, extra)
    hit = _CHECKED.get(kind)
    if version is not None and hit is not None and hit[0] == key:
        return hit[1]
    if t.is_cuda and torch.cuda.is_current_stream_capturing():
        return True
    ok = compute()
    _CHECKED[kind] = (key, ok, t)
    return ok


class _Linear(torch.nn.Module):
    """weight [out, in] (+ bias [out]): the parameter layout of the reference's Column/RowParallelLinear
    at model-parallel size 1 (core/nn/linear/column_parallel_linear.py:109-116, row_parallel_linear.py:117-124)."""

    def __init__(self, in_features: int, out_features: int, bias: bool, device, dtype, init_method: InitMethod):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=dtype))
        init_method(self.weight)
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(out_features, device=device, dtype=dtype))
        else:
            self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)


class RMSNorm(torch.nn.Module):
    """Mirror of core/nn/norm/rms_norm.py:19-106 (u-muP and sequence-parallel branches excluded)."""

    def __init__(self, dimensions: int, device: Optional[torch.device] = None, config: Optional[LayerNormConfig] = None,
                 dtype: torch.dtype = torch.float32, topology=None, umup_on_residual: Optional[bool] = None) -> None:
        super().__init__()
        device = _default_device(device, topology)
        self.config = config if config is not None else LayerNormConfig()
        self.eps = self.config.layernorm_epsilon
        self.topology = None
        self.weight = torch.nn.Parameter(torch.ones(dimensions, dtype=dtype, device=device))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rms_norm(x, self.weight, self.eps)


class LayerNorm(torch.nn.Module):
    """Mirror of core/nn/norm/layernorm.py:16-86 (`optimization_type: torch`; u-muP and bitfit bias names
    excluded): weight ones, bias zeros, torch.nn.functional.layer_norm semantics."""

    def __init__(self, config: Optional[LayerNormConfig], normalized_shape: int, device: Optional[torch.device] = None,
                 dtype: torch.dtype = torch.float32, bitfit_bias_name: Optional[str] = None, topology=None,
                 umup_on_residual: Optional[bool] = None) -> None:
        super().__init__()
        if bitfit_bias_name:
            raise NotImplementedError("bitfit bias names are outside the layer hot path of this package")
        device = _default_device(device, topology)
        self.config = config if config is not None else LayerNormConfig()
        self.eps = self.config.layernorm_epsilon
        self.normalized_shape = torch.Size((normalized_shape,))
        self.topology = None
        self.weight = torch.nn.Parameter(torch.ones(normalized_shape, dtype=dtype, device=device))
        self.bias = torch.nn.Parameter(torch.zeros(normalized_shape, dtype=dtype, device=device))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layer_norm(x, self.weight, self.bias, self.eps)


def get_norm(norm_type: NormType, layernorm_config: Optional[LayerNormConfig], dimensions: int,
             device: Optional[torch.device], dtype: torch.dtype, bitfit_bias_name: Optional[str] = None,
             topology=None, umup_on_residual: Optional[bool] = None) -> torch.nn.Module:
    """Mirror of core/nn/norm/get_norm.py:17-49."""
    if norm_type == NormType.RMS:
        return RMSNorm(dimensions=dimensions, device=device, config=layernorm_config, dtype=dtype, topology=topology)
    if norm_type == NormType.LAYERNORM:
        return LayerNorm(config=layernorm_config, normalized_shape=dimensions, device=device, dtype=dtype,
                         bitfit_bias_name=bitfit_bias_name, topology=topology)
    raise NotImplementedError(f"norm_type {norm_type} is not known")


class RotaryEmbedding(torch.nn.Module):
    """Mirror of core/nn/rotary.py:142-213: fp32 table construction, tables cast to the module dtype and
    kept as non-persistent buffers `cos` / `sin` of shape [max_seq, 1, 1, dim]."""

    def __init__(self, config: RotaryConfig, device: torch.device, dtype: torch.dtype = torch.float32) -> None:
        super().__init__()
        assert config.dimensions > 1, "RotaryEmbedding cannot use `dim` == 1"
        dim, n = config.dimensions, config.max_seq_length
        self.inv_freq = 1.0 / (config.base ** (torch.arange(0, dim, 2).float() / dim))
        ang = torch.outer(torch.arange(n).float(), self.inv_freq)
        ang = torch.cat((ang, ang), dim=-1).to(device).float()
        self.register_buffer("cos", ang.cos().reshape(n, 1, 1, dim).to(dtype), persistent=False)
        self.register_buffer("sin", ang.sin().reshape(n, 1, 1, dim).to(dtype), persistent=False)
        self.dimensions = dim
        self.max_seq_length = n

    def tables(self) -> Tuple[torch.Tensor, torch.Tensor]:
        return self.cos.view(self.max_seq_length, self.dimensions), self.sin.view(self.max_seq_length, self.dimensions)

    def rotate_tokens(self, x: torch.Tensor, position_ids: Optional[torch.Tensor], seq_len: int) -> torch.Tensor:
        """x [tokens, heads, head_dim] (tokens = flattened (b s)); position_ids int64 [tokens] or None."""
        cos, sin = self.tables()
        return ops.rotary_embedding(x, cos, sin, position_ids, seq_len_for_null_ids=seq_len)

    def forward(self, query: torch.Tensor, key: torch.Tensor, query_position_ids: Optional[torch.Tensor] = None,
                key_position_ids: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """query [s_q, b, n_q, d], key [s_k, b, n_kv, d], ids [s, b] as in the reference."""
        def one(x, ids):
            s, b, n, d = x.shape
            tok = x.permute(1, 0, 2, 3).reshape(b * s, n, d)
            flat = None if ids is None else ids.transpose(0, 1).reshape(-1).contiguous()
            return self.rotate_tokens(tok, flat, s).view(b, s, n, d).permute(1, 0, 2, 3)
        return one(query, query_position_ids), one(key, key_position_ids)


class RotaryEmbeddingComplex(torch.nn.Module):
    """Mirror of core/nn/rotary.py:216-255: interleaved pairs (2i, 2i+1), fp32 arithmetic; the real and
    imaginary parts of freqs_cis (rotary.py:45-56) are non-persistent buffers [max_seq, dim/2]."""

    def __init__(self, config: RotaryConfig, device: torch.device) -> None:
        super().__init__()
        assert config.dimensions > 1, "RotaryEmbedding cannot use `dim` == 1"
        dim, n = config.dimensions, config.max_seq_length
        freqs = 1.0 / (float(config.base) ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
        ang = torch.outer(torch.arange(n), freqs).float().to(device)
        self.register_buffer("freqs_cis_real", ang.cos(), persistent=False)
        self.register_buffer("freqs_cis_imag", ang.sin(), persistent=False)
        self.dimensions = dim
        self.max_seq_length = n

    def tables(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """fp32 [max_seq, dim / 2] real and imaginary parts (no copy unless the buffers were cast)."""
        return self.freqs_cis_real.float().contiguous(), self.freqs_cis_imag.float().contiguous()

    def rotate_tokens(self, x: torch.Tensor, position_ids: Optional[torch.Tensor], seq_len: int) -> torch.Tensor:
        assert x.shape[-1] == self.dimensions, "the interleaved variant rotates the whole head (rotary.py:69-70)"
        real, imag = self.tables()
        return ops.rotary_embedding_complex(x, real, imag, position_ids, seq_len)

    def forward(self, query: torch.Tensor, key: torch.Tensor, query_position_ids: Optional[torch.Tensor] = None,
                key_position_ids: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        def one(x, ids):
            s, b, n, d = x.shape
            tok = x.permute(1, 0, 2, 3).reshape(b * s, n, d)
            flat = None if ids is None else ids.transpose(0, 1).reshape(-1).contiguous()
            return self.rotate_tokens(tok, flat, s).view(b, s, n, d).permute(1, 0, 2, 3)
        return one(query, query_position_ids), one(key, key_position_ids)


class ParallelSwiGLUMLP(torch.nn.Module):
    """Mirror of core/nn/mlp.py:149-282: dense_out(silu(dense_in(x)) * siglu_weight(x))."""

    def __init__(self, io_features: int, intermediate_feature_factor: float, bias: bool = True,
                 device: Optional[torch.device] = None, dtype: torch.dtype = torch.float32, topology=None,
                 init_method: InitMethod = torch.nn.init.xavier_normal_, bitfit_bias_name: Optional[str] = None,
                 umup_mult: Optional[float] = None, umup_is_first_layer: Optional[bool] = None,
                 umup_is_last_layer: Optional[bool] = None, umup_on_residual: Optional[bool] = None,
                 fp8_config=None, fp8_config_dense_out=None) -> None:
        super().__init__()
        device = _default_device(device, topology)
        if fp8_config is not None or fp8_config_dense_out is not None or bitfit_bias_name is not None:
            raise NotImplementedError("fp8 / bitfit options are outside the layer hot path of this package")
        assert float(int(io_features * intermediate_feature_factor)) == io_features * intermediate_feature_factor, \
            "io_features * intermediate_feature_factor does not result in a natural number for feature dimensions"
        inter = int(io_features * intermediate_feature_factor)
        self.topology = None
        self.dense_in = _Linear(io_features, inter, bias, device, dtype, init_method)
        self.siglu_weight = _Linear(io_features, inter, bias, device, dtype, init_method)
        self.dense_out = _Linear(inter, io_features, bias, device, dtype, init_method)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.dense_out(ops.swiglu(self.dense_in(x), self.siglu_weight(x)))


class ParallelMLP(torch.nn.Module):
    """Mirror of core/nn/mlp.py:25-146 with the GELU activation (activation_function.py:13-14):
    dense_out(gelu(dense_in(x)))."""

    def __init__(self, io_features: int, intermediate_feature_factor: float, bias: bool = True,
                 device: Optional[torch.device] = None, dtype: torch.dtype = torch.float32, topology=None,
                 init_method: InitMethod = torch.nn.init.xavier_normal_, bitfit_bias_name: Optional[str] = None,
                 activation_function: str = "gelu", umup_mult: Optional[float] = None,
                 umup_is_first_layer: Optional[bool] = None, umup_is_last_layer: Optional[bool] = None,
                 umup_on_residual: Optional[bool] = None, fp8_config=None, fp8_config_dense_out=None) -> None:
        super().__init__()
        device = _default_device(device, topology)
        if fp8_config is not None or fp8_config_dense_out is not None or bitfit_bias_name is not None:
            raise NotImplementedError("fp8 / bitfit options are outside the layer hot path of this package")
        if getattr(activation_function, "value", activation_function) != "gelu":
            raise NotImplementedError("ParallelMLP has a HIP kernel for the GELU activation only")
        assert float(int(io_features * intermediate_feature_factor)) == io_features * intermediate_feature_factor, \
            "io_features * intermediate_feature_factor does not result in a natural number for feature dimensions"
        inter = int(io_features * intermediate_feature_factor)
        self.topology = None
        self.dense_in = _Linear(io_features, inter, bias, device, dtype, init_method)
        self.dense_out = _Linear(inter, io_features, bias, device, dtype, init_method)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.dense_out(ops.gelu(self.dense_in(x)))


class MaskedSoftmax(torch.nn.Module):
    """Mirror of core/nn/masked_softmax/masked_softmax.py:37-52: holds the config and resolves the kernel.  As for the
    reference's fused flash-attention kernel, `kernel` is None for `hip` (the softmax runs inside the attention
    kernels, always in fp32, with `config.scale` folded into the score scale) and calling the module asserts;
    any other kernel raises NotImplementedError at construction."""

    def __init__(self, config: MaskedSoftmaxConfig) -> None:
        super().__init__()
        self.config = config
        self.kernel: Optional[torch.nn.Module]
        if self.config.kernel == MaskedSoftmaxKernel.HIP:
            self.kernel = None
        else:
            raise NotImplementedError(f"kernel {self.config.kernel} not implemented (this package provides masked_softmax.kernel = 'hip' only)")

    def forward(self, x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        assert self.kernel is not None
        return self.kernel(x=x, mask=mask)


class ScaledDotProductAttention(torch.nn.Module):
    """Mirror of core/nn/attention/attention.py:280-395 backed by the fused kernels: same constructor, attributes
    (`head_dim`, `dropout_p`, `softmax_fn`, `dropout_fn`, `masked_softmax_config`, `query_key_scaling_factor`,
    `causal`, `use_matmul`) and forward signature.  `forward` takes the reference's layout (query [s_q, b, n, d],
    key / value [s_k, b, n_kv, d]; the KV heads need not be repeated) and returns [(b n), s_q, d];
    `forward_tokens` is the copy-free form on token-major tensors that ParallelSelfAttention uses."""

    def __init__(self, head_dim: int, dropout_p: float, masked_softmax_config: MaskedSoftmaxConfig, causal: bool,
                 use_matmul: bool = False, umup_mult: Optional[float] = None):
        super().__init__()
        if umup_mult is not None:
            raise NotImplementedError("u-muP scaling is outside the hip kernel's scope")
        self.head_dim = head_dim
        self.dropout_p = dropout_p
        self.softmax_fn = MaskedSoftmax(masked_softmax_config)
        self.dropout_fn = torch.nn.Dropout(p=dropout_p)   # kept for the module tree; the kernels draw their own mask
        self.masked_softmax_config = masked_softmax_config
        self.query_key_scaling_factor: float = 1 / (head_dim ** 0.5)
        self.causal = causal
        self.use_matmul = use_matmul
        self.umup_mult = None
        self._use_umup = False

    @property
    def softmax_scale(self) -> float:
        """alpha of the score product times masked_softmax.scale (attention.py:154-160 with masked_softmax.py:21-22)."""
        return self.query_key_scaling_factor * self.masked_softmax_config.scale

    def forward_tokens(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cumulative_seq_lengths: torch.Tensor,
                       cumulative_seq_lengths_key: Optional[torch.Tensor] = None, rotary=None) -> torch.Tensor:
        """q [tokens, n, d], k / v [tokens_k, n_kv, d] (views with contiguous features) -> [tokens, n, d]."""
        return ops.attention(q, k, v, cumulative_seq_lengths, cumulative_seq_lengths_key, self.causal, self.softmax_scale,
                             dropout_p=self.dropout_p if self.training else 0.0, rotary=rotary,
                             deterministic=self.masked_softmax_config.deterministic_flash_attn_bwd)

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, cumulative_seq_lengths: torch.Tensor,
                attention_scores_manipulation: Optional[torch.Tensor] = None,
                attentions_score_manipulation_log_additive=True) -> torch.Tensor:
        if attention_scores_manipulation is not None:
            raise NotImplementedError("attention_scores_manipulation is not available with the hip kernel")
        s_q, b, n, d = query.shape

        def tokens(x):
            return x.permute(1, 0, 2, 3).reshape(b * x.shape[0], x.shape[2], d)

        cu = cumulative_seq_lengths.to(torch.int32)
        if key.shape[0] != s_q:   # cached decoding in the reference's layout: every row is one document with its own key length
            assert cu.numel() == b + 1, "differing query and key lengths need one document per batch row"
            cu_k = torch.arange(0, b * key.shape[0] + 1, key.shape[0], dtype=torch.int32, device=cu.device)
        else:
            cu_k = None
        out = self.forward_tokens(tokens(query), tokens(key), tokens(value), cu, cu_k)
        return out.view(b, s_q, n, d).permute(0, 2, 1, 3).reshape(b * n, s_q, d)


class KVCache:
    """Pre-allocated cache of post-rotary K and un-repeated V, indexed [batch, token, kv head, d], replacing
    the reference's per-step torch.cat (core/nn/attention/attention.py:862-869).  Storage is head-major
    ([batch, kv head, token, d]): the decode kernel streams one (sequence, kv head) pair per workgroup, and
    a contiguous 1 MB stream per pair measures ~6 % more HBM bandwidth than 256-byte pieces 2 KB apart."""

    def __init__(self, batch: int, max_ctx: int, n_kv: int, head_dim: int, dtype, device) -> None:
        self.k = torch.zeros(batch, n_kv, max_ctx, head_dim, dtype=dtype, device=device).transpose(1, 2)
        self.v = torch.zeros(batch, n_kv, max_ctx, head_dim, dtype=dtype, device=device).transpose(1, 2)
        self.ctx_len = torch.zeros(batch, dtype=torch.int32, device=device)
        self.length = 0          # host copy of the (uniform) context length
        self.max_ctx = max_ctx
        self.workspace: Optional[torch.Tensor] = None


class ParallelSelfAttention(torch.nn.Module):
    """Mirror of core/nn/attention/attention.py:509-969 for `masked_softmax.kernel = hip`.

    Same constructor arguments and forward signature.  Differences, all documented errors rather than
    silent fall-backs: attention-score manipulation, LoRA, local attention windows, u-muP and fp8 are not
    available; attention-probability dropout is applied inside the kernels in training mode (its mask comes
    from a counter-based hash, not from torch's generator stream, and its rate is quantised to 1/256);
    float32 (the reference's default precision) runs separate exact-fp32 kernels without dropout, fused rotary or
    KV cache.  The KV cache is pre-allocated (see `KVCache`), supports batches of
    single-document rows and is filled/extended in place.
    """

    def __init__(self, hidden_size: int, num_attention_heads: int, masked_softmax_config: MaskedSoftmaxConfig,
                 causal: bool = True, num_local_attention_heads: int = 0,
                 local_attention_window_size: Optional[int] = None, dropout_attention_probs: float = 0.0,
                 rotary_config: Optional[RotaryConfig] = None,
                 relative_position_embedding_type: RelativePositionEmbeddingType = RelativePositionEmbeddingType.ROTARY,
                 bias: bool = True, device: Optional[torch.device] = None, dtype: torch.dtype = torch.float32,
                 topology=None, init_method: InitMethod = torch.nn.init.xavier_normal_,
                 bitfit_bias_name: Optional[str] = None, lora_config=None, norm_type: NormType = NormType.LAYERNORM,
                 key_query_norm: bool = False, layernorm_config: Optional[LayerNormConfig] = None,
                 qkv_in_one: bool = True, num_kv_heads: Optional[int] = None, use_matmul: bool = False,
                 umup_mult: Optional[float] = None, umup_is_first_layer: Optional[bool] = None,
                 umup_is_last_layer: Optional[bool] = None, umup_on_residual: Optional[bool] = None,
                 fp8_config=None, fp8_config_dense_out=None, max_cache_length: Optional[int] = None) -> None:
        super().__init__()
        self._device = _default_device(device, topology)
        assert hidden_size % num_attention_heads == 0, \
            f"hidden size ({hidden_size}) must be divisible by num_attention_heads ({num_attention_heads})"
        assert 0.0 <= dropout_attention_probs < 1.0, "dropout_attention_probs must be in [0, 1)"
        self.dropout_attention_probs = float(dropout_attention_probs)   # applied in training mode only
        # attention.py:734-743; raises NotImplementedError for any masked_softmax.kernel other than `hip`
        self.scaled_dot_product_attention = ScaledDotProductAttention(
            head_dim=hidden_size // num_attention_heads, dropout_p=self.dropout_attention_probs,
            masked_softmax_config=masked_softmax_config, causal=causal, use_matmul=use_matmul)
        if num_local_attention_heads > 0 or lora_config is not None or fp8_config is not None or \
                fp8_config_dense_out is not None or bitfit_bias_name is not None:
            raise NotImplementedError("local attention, LoRA, fp8 and bitfit are outside the hip kernel's scope")
        if dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise NotImplementedError("the hip attention kernels take bfloat16, float16 or float32 tensors")
        if dtype == torch.float32 and self.dropout_attention_probs > 0.0:
            raise NotImplementedError("attention-probability dropout needs precision bfloat16 or float16 with the hip kernel")

        self.hidden_size_per_attention_head = hidden_size // num_attention_heads
        self.num_attention_heads = num_attention_heads
        self.num_attention_heads_per_partition = num_attention_heads
        self.causal = causal
        self.masked_softmax_config = masked_softmax_config
        self.use_flash_attention = False
        self.dtype = dtype
        self.lora_config = None
        self.topology = None
        self.qkv_in_one = qkv_in_one
        self.num_kv_heads = num_kv_heads
        if num_kv_heads:
            assert not qkv_in_one, "for a differing number of kv heads, qkv cannot be stored in one"
            assert num_attention_heads % num_kv_heads == 0
            self.num_kv_heads_per_partition = num_kv_heads
        else:
            self.num_kv_heads_per_partition = num_attention_heads
        self.num_repeat_kv = num_attention_heads // self.num_kv_heads_per_partition
        d = self.hidden_size_per_attention_head
        if d not in (32, 64, 96, 128):
            raise NotImplementedError(f"head_dim {d} is not supported by the hip attention kernels (32, 64, 96, 128)")

        if qkv_in_one:
            self.query_key_value = _Linear(hidden_size, 3 * hidden_size, bias, self._device, dtype, init_method)
        else:
            self.query = _Linear(hidden_size, hidden_size, bias, self._device, dtype, init_method)
            self.key = _Linear(hidden_size, hidden_size // self.num_repeat_kv, bias, self._device, dtype, init_method)
            self.value = _Linear(hidden_size, hidden_size // self.num_repeat_kv, bias, self._device, dtype, init_method)

        self.rotary_embedding = None
        if relative_position_embedding_type == RelativePositionEmbeddingType.ROTARY:
            assert rotary_config is not None
            self.rotary_embedding = RotaryEmbedding(config=rotary_config, device=self._device, dtype=dtype)
        elif relative_position_embedding_type == RelativePositionEmbeddingType.ROTARY_COMPLEX:
            assert rotary_config is not None
            self.rotary_embedding = RotaryEmbeddingComplex(config=rotary_config, device=self._device)
        # rotary can be applied inside the attention kernels (on the Q/K load), either pairing
        # when it covers the whole head
        # (16-bit tensors only: float32 runs the stand-alone rotary kernel in front of the fp32 attention core)
        self._fusable_rotary = self.rotary_embedding is not None and dtype != torch.float32 and \
            rotary_config.dimensions == self.hidden_size_per_attention_head and self.hidden_size_per_attention_head in (64, 128)

        self.key_query_norm = key_query_norm
        self.norm_query = self.norm_key = None
        if key_query_norm:
            self.norm_query = get_norm(norm_type, layernorm_config, d, self._device, dtype)
            self.norm_key = get_norm(norm_type, layernorm_config, d, self._device, dtype)

        # softmax_fn scale: alpha * masked_softmax.scale (attention.py:297 with masked_softmax.py:21-22)
        self.query_key_scaling_factor = self.scaled_dot_product_attention.query_key_scaling_factor
        self.softmax_scale = self.scaled_dot_product_attention.softmax_scale
        self.dense = _Linear(hidden_size, hidden_size, bias, self._device, dtype, init_method)
        self.cache: Dict[int, Optional[KVCache]] = dict()
        self.max_cache_length = max_cache_length

    # ---- helpers --------------------------------------------------------------------------------
    def _project(self, x: torch.Tensor):
        b, s, _ = x.shape
        nq, nkv, d = self.num_attention_heads, self.num_kv_heads_per_partition, self.hidden_size_per_attention_head
        if self.qkv_in_one:
            qkv = self.query_key_value(x).view(b * s, nq, 3 * d)       # per head: q then k then v (attention.py:790-796)
            return qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
        if not torch.is_grad_enabled() and not self.training:
            # inference (eval mode, so that a no-grad forward that activation checkpointing recomputes with grad takes
            # the same GEMMs both times): one projection GEMM over the row-stacked weights; q, k, v are column slices
            w, bias = self._fused_qkv()
            out = F.linear(x, w, bias).view(b * s, (nq + 2 * nkv) * d)
            return (out[:, :nq * d].view(b * s, nq, d), out[:, nq * d:(nq + nkv) * d].view(b * s, nkv, d),
                    out[:, (nq + nkv) * d:].view(b * s, nkv, d))
        q = self.query(x).view(b * s, nq, d)
        k = self.key(x).view(b * s, nkv, d)
        v = self.value(x).view(b * s, nkv, d)
        return q, k, v

    def _fused_qkv(self):
        """The weights (and biases) of `query`, `key`, `value` as row blocks of one tensor.  Built on first use: the
        three parameters are re-pointed at views of the stacked copy, so values, names and the state dict stay as
        they are while a single GEMM can read all of them.  Rebuilt if a parameter was moved or replaced."""
        mods = (self.query, self.key, self.value)
        rows = [m.weight.shape[0] for m in mods]
        offs = [0, rows[0], rows[0] + rows[1]]
        fused = self.__dict__.get("_qkv_fused")

        def aliased(t, name):
            return t is not None and all(getattr(m, name).data_ptr() == t[o:o + r].data_ptr() and getattr(m, name).device == t.device
                                         for m, o, r in zip(mods, offs, rows))

        has_bias = mods[0].bias is not None
        if fused is None or not aliased(fused[0], "weight") or (has_bias and not aliased(fused[1], "bias")):
            w = torch.cat([m.weight.data for m in mods], dim=0)
            bias = torch.cat([m.bias.data for m in mods], dim=0) if has_bias else None
            for m, o, r in zip(mods, offs, rows):
                m.weight.data = w[o:o + r]
                if has_bias:
                    m.bias.data = bias[o:o + r]
            fused = (w, bias)
            self.__dict__["_qkv_fused"] = fused
        return fused

    @staticmethod
    def _decode_operand(t: torch.Tensor) -> torch.Tensor:
        """q / k / v of one token per sequence as the decode kernel takes them: [heads, d] contiguous per sequence."""
        ok = t.stride(2) == 1 and t.stride(1) == t.shape[2] and t.stride(0) % 8 == 0
        return t if ok else t.contiguous()

    def _rows_are_single_documents(self, cu: torch.Tensor, b: int, s: int) -> bool:
        """True when every batch row is one document.  A decode step (s == 1) needs the shape only: cumulative lengths
        as transformer/data/utils.py:40-74 builds them contain every multiple of s, and b + 1 of them on b tokens can
        only be 0..b (a caller that breaks that contract is not detected here).  A prefill compares on the device and
        reads the answer back once per cumulative-lengths tensor (all layers of a forward receive the same one)."""
        if cu.numel() != b + 1:
            return False
        if s == 1:
            return True
        return _checked_once("single_documents", cu, (b, s),
                             lambda: bool(torch.equal(cu, torch.arange(0, b * s + 1, s, dtype=cu.dtype, device=cu.device))))

    def _check_positions(self, pos: Optional[torch.Tensor]) -> None:
        """The reference gathers cos / sin rows by position id (rotary.py:128-131) and raises on an id outside the
        table; the kernels would clamp instead, so the ids are validated here, once per position-id tensor."""
        if pos is None or self.rotary_embedding is None or pos.numel() == 0:
            return
        rows = self.rotary_embedding.max_seq_length
        ok = _checked_once("positions", pos, (rows,), lambda: bool(((pos >= 0) & (pos < rows)).all()))
        if not ok:
            raise IndexError(f"position ids outside the rotary table of {rows} rows")

    def forward(self, x: torch.Tensor, cumulative_seq_lengths: torch.Tensor, position_ids: Optional[torch.Tensor],
                cumulative_seq_lengths_key: Optional[torch.Tensor] = None, use_cache: bool = False,
                reset_cache: bool = False, cache_index: int = 0, attention_scores_manipulation=None,
                attentions_score_manipulation_log_additive=True) -> torch.Tensor:
        if attention_scores_manipulation is not None:
            raise NotImplementedError("attention_scores_manipulation is not available with the hip kernel")
        b, s, hidden = x.shape
        nq, nkv, d = self.num_attention_heads, self.num_kv_heads_per_partition, self.hidden_size_per_attention_head
        q, k, v = self._project(x)
        if self.key_query_norm:
            q = self.norm_query(q)
            k = self.norm_key(k)
        pos = None if position_ids is None else position_ids.reshape(-1).contiguous()
        cu = cumulative_seq_lengths.to(torch.int32)
        sdpa = self.scaled_dot_product_attention

        if use_cache:
            if not self.causal:
                raise ValueError("KV caching is only supported for causal attention.")
            if self.dtype == torch.float32:
                raise NotImplementedError("the KV-cache decode kernels take bfloat16 or float16 tensors")
            assert self._rows_are_single_documents(cu, b, s), "sequence packing is not supported with cache"
            if not reset_cache:
                return self.dense(self._decode_step(q, k, v, pos, b, s, cache_index).view(b, s, nq * d))
        elif reset_cache:
            self.cache[cache_index] = None
        self._check_positions(pos)
        cu_k = None if cumulative_seq_lengths_key is None else cumulative_seq_lengths_key.to(torch.int32)

        if self._fusable_rotary and pos is not None and not use_cache:
            # rotary is applied while the kernels load Q and K (forward and backward); nothing rotated is stored
            cos, sin = self.rotary_embedding.tables()
            ctx = sdpa.forward_tokens(q, k, v, cu, cu_k, rotary=(cos, sin, pos, pos))
            return self.dense(ctx.view(b, s, nq * d))
        if self.rotary_embedding is not None:
            q = self.rotary_embedding.rotate_tokens(q, pos, s)
            k = self.rotary_embedding.rotate_tokens(k, pos, s)
        if use_cache:  # prefill: keep post-rotary K and V (attention.py:861-862)
            self._fill_cache(k, v, b, s, cache_index)
        ctx = sdpa.forward_tokens(q, k, v, cu, cu_k)
        return self.dense(ctx.view(b, s, nq * d))

    # ---- KV cache ----------------------------------------------------------------------------------
    def merge_lora_weights(self) -> None:
        """attention.py:1033-1034: the trainer calls this on every attention module when it is told to merge LoRA
        weights after loading a checkpoint; this module never holds any (its constructor refuses `lora_config`)."""
        raise AssertionError("Merge of LoRa weights called without proper configuration.")

    def _cache_capacity(self) -> int:
        if self.max_cache_length is not None:
            return self.max_cache_length
        if self.rotary_embedding is not None:
            return self.rotary_embedding.max_seq_length
        raise ValueError("set max_cache_length when the module has no rotary table to size the cache from")

    def _fill_cache(self, k: torch.Tensor, v: torch.Tensor, b: int, s: int, cache_index: int) -> None:
        nkv, d = self.num_kv_heads_per_partition, self.hidden_size_per_attention_head
        cap = max(self._cache_capacity(), s)
        cache = self.cache.get(cache_index)
        if cache is None or cache.k.shape[0] != b or cache.max_ctx < cap:
            cache = KVCache(b, cap, nkv, d, k.dtype, k.device)
            self.cache[cache_index] = cache
        cache.k[:, :s].copy_(k.detach().view(b, s, nkv, d))
        cache.v[:, :s].copy_(v.detach().view(b, s, nkv, d))
        cache.length = s
        cache.ctx_len.fill_(s)

    def decode_forward(self, x: torch.Tensor, position_ids: torch.Tensor, cache_index: int = 0,
                       advance: bool = True) -> torch.Tensor:
        """One cached decode step without any host synchronisation (usable under HIP graph capture):
        x [b, 1, H], position_ids int64 [b].  The caller guarantees a prefilled cache with room for one
        more token per sequence; only the device-side context lengths are advanced here (advance=False when
        the caller shares one context-length tensor between layers and has advanced it already)."""
        b = x.shape[0]
        nq, d = self.num_attention_heads, self.hidden_size_per_attention_head
        q, k, v = self._project(x)
        if self.key_query_norm:
            q, k = self.norm_query(q), self.norm_key(k)
        cache = self.cache[cache_index]
        if advance:
            cache.ctx_len.add_(1)
        rotary = None
        if self.rotary_embedding is not None:
            if self._fusable_rotary:
                cos, sin = self.rotary_embedding.tables()
                rotary = (cos, sin, position_ids)
            else:
                q = self.rotary_embedding.rotate_tokens(q, position_ids, 1)
                k = self.rotary_embedding.rotate_tokens(k, position_ids, 1)
        ctx = ops.decode_attention(self._decode_operand(q), cache.k, cache.v, cache.ctx_len, self._decode_operand(k),
                                   self._decode_operand(v), rotary=rotary, softmax_scale=self.softmax_scale, workspace=cache.workspace)
        return self.dense(ctx.view(b, 1, nq * d))

    def _decode_step(self, q, k, v, pos, b: int, s: int, cache_index: int) -> torch.Tensor:
        cache = self.cache.get(cache_index)
        assert cache is not None, "decode step without a prefilled cache"
        if s != 1:
            raise NotImplementedError("cached attention extends the context one token per sequence and step")
        assert cache.k.shape[0] == b and cache.length + 1 <= cache.max_ctx, "KV cache too small or batch changed"
        nq, nkv, d = self.num_attention_heads, self.num_kv_heads_per_partition, self.hidden_size_per_attention_head
        cache.length += 1
        cache.ctx_len.add_(1)
        rotary = None
        if self.rotary_embedding is not None:
            if cache.length > self.rotary_embedding.max_seq_length:
                raise IndexError(f"position {cache.length - 1} is outside the rotary table of {self.rotary_embedding.max_seq_length} rows")
            if pos is None:
                pos = torch.full((b,), cache.length - 1, dtype=torch.int64, device=q.device)
            if self._fusable_rotary:
                cos, sin = self.rotary_embedding.tables()
                rotary = (cos, sin, pos)
            else:  # partial rotary: stand-alone kernel, then a plain append
                q = self.rotary_embedding.rotate_tokens(q, pos, 1)
                k = self.rotary_embedding.rotate_tokens(k, pos, 1)
        if cache.workspace is None:
            cache.workspace = ops.decode_workspace(b, nq, d, cache.max_ctx, q.device)
        return ops.decode_attention(self._decode_operand(q), cache.k, cache.v, cache.ctx_len, self._decode_operand(k),
                                    self._decode_operand(v), rotary=rotary, softmax_scale=self.softmax_scale, workspace=cache.workspace)
