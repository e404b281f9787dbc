"""Oracle (test infrastructure): self-attention module math, the pre-norm transformer
layer and the greedy cached / uncached decode loop, at tensor-parallel size 1.

Follows core/nn/attention/attention.py:772-969, transformer/model/layers/layer.py:241-345,
core/nn/residual.py:49-65, transformer/model/layers/layernorm.py:36-59 and
transformer/inference/inference_model.py:188-263 of the reference.  Weights are passed
as plain dicts that use the reference's state-dict key names.
"""

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

from .attention import multi_head_attention, repeat_kv
from .data_utils import get_cumulative_seq_lengths, get_position_ids
from .mlp import gelu_mlp, swiglu_mlp
from .norm import layer_norm, rms_norm
from .rotary import RotaryTables, apply_rotary, apply_rotary_complex, rotary_tables


@dataclass
class LayerSpec:
    """The architecture fields that parameterise the path (transformer/context/config.py:229-432)."""

    hidden_size: int
    num_attention_heads: int
    num_kv_heads: Optional[int] = None          # attention_num_kv_heads
    qkv_in_one: bool = True                     # attention_qkv_in_one
    norm_type: str = "layernorm"                # "layernorm" | "rms"
    mlp_type: str = "default"                   # "default" (GELU) | "swiglu"
    layernorm_epsilon: float = 1e-5
    rotary: str = "rotary"                      # "none" | "rotary" | "rotary_complex"
    rotary_base: int = 10000
    rotary_percentage: float = 1.0
    sequence_length: int = 2048                 # rotary table length
    causal: bool = True
    softmax_in_fp32: bool = False
    softmax_scale: float = 1.0
    dtype: torch.dtype = torch.float32

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def n_kv(self) -> int:
        return self.num_kv_heads or self.num_attention_heads

    @property
    def rotary_dim(self) -> int:
        return int(self.rotary_percentage * self.head_dim)  # layer.py:96-103

    def tables(self) -> RotaryTables:
        return rotary_tables(self.rotary_dim, self.sequence_length, self.rotary_base, self.dtype)


KVCache = Dict[int, Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]]


def _norm(spec: LayerSpec, x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """core/nn/norm/get_norm.py:17-49."""
    if spec.norm_type == "rms":
        return rms_norm(x, w[prefix + ".weight"], spec.layernorm_epsilon)
    return layer_norm(x, w[prefix + ".weight"], w.get(prefix + ".bias"), spec.layernorm_epsilon)


def self_attention(spec: LayerSpec, w: Dict[str, torch.Tensor], x: torch.Tensor,
                   cumulative_seq_lengths: torch.Tensor, position_ids: Optional[torch.Tensor],
                   prefix: str = "self_attention", tables: Optional[RotaryTables] = None,
                   use_cache: bool = False, reset_cache: bool = False, cache: Optional[KVCache] = None,
                   cache_index: int = 0) -> torch.Tensor:
    """core/nn/attention/attention.py:772-969, `torch` kernel branch.

    x [b, s, H] -> [b, s, H].  The fused projection stores, per head, q then k
    then v (each head_dim wide, lines 790-796).  The cache keeps post-rotary,
    un-repeated K/V and grows by concatenation (lines 852-873).
    """
    b, s, _ = x.shape
    nq, nkv, d = spec.num_attention_heads, spec.n_kv, spec.head_dim
    if spec.qkv_in_one:
        qkv = F.linear(x, w[prefix + ".query_key_value.weight"], w.get(prefix + ".query_key_value.bias"))
        qkv = qkv.view(b, s, nq, 3 * d).permute(1, 0, 2, 3)  # "b sq (np hn) -> sq b np hn"
        q, k, v = qkv[..., :d], qkv[..., d:2 * d], qkv[..., 2 * d:]
    else:
        q = F.linear(x, w[prefix + ".query.weight"], w.get(prefix + ".query.bias")).view(b, s, nq, d).permute(1, 0, 2, 3)
        k = F.linear(x, w[prefix + ".key.weight"], w.get(prefix + ".key.bias")).view(b, s, nkv, d).permute(1, 0, 2, 3)
        v = F.linear(x, w[prefix + ".value.weight"], w.get(prefix + ".value.bias")).view(b, s, nkv, d).permute(1, 0, 2, 3)

    # query / key norm over head_dim, before the rotary embedding (attention.py:712-732, 819-834)
    if prefix + ".norm_query.weight" in w:
        q = _norm(spec, q, w, prefix + ".norm_query")
        k = _norm(spec, k, w, prefix + ".norm_key")

    ids = None if position_ids is None else position_ids.transpose(0, 1)  # "b sq -> sq b", line 838-839
    if spec.rotary == "rotary":
        q, k = apply_rotary(q, k, tables if tables is not None else spec.tables(), ids, ids)
    elif spec.rotary == "rotary_complex":
        q, k = apply_rotary_complex(q, k, spec.rotary_dim, spec.sequence_length, spec.rotary_base, ids, ids)

    if use_cache:
        assert spec.causal and b == 1 and cache is not None
        assert cumulative_seq_lengths.tolist() == [0, s], "sequence packing is not supported with cache"
        if not reset_cache:
            past_k, past_v = cache[cache_index]
            k = torch.cat((past_k, k), dim=0)
            v = torch.cat((past_v, v), dim=0)
        cache[cache_index] = (k, v)
    elif reset_cache and cache is not None:
        cache[cache_index] = (None, None)

    n_rep = nq // nkv
    ctx = multi_head_attention(q, repeat_kv(k, n_rep), repeat_kv(v, n_rep), cumulative_seq_lengths,
                               causal=spec.causal, query_key_scaling_factor=1.0 / (d ** 0.5),
                               softmax_in_fp32=spec.softmax_in_fp32, softmax_scale=spec.softmax_scale)
    ctx = ctx.view(b, nq, s, d).permute(0, 2, 1, 3).reshape(b, s, nq * d)  # "(b np) sq hn -> b sq (np hn)"
    return F.linear(ctx, w[prefix + ".dense.weight"], w.get(prefix + ".dense.bias"))


def attention_block(spec, w, hidden, cumulative_seq_lengths, position_ids, **kw) -> torch.Tensor:
    """transformer/model/layers/layer.py:241-274 (dropout 0, u-muP off, no adapters)."""
    return hidden + self_attention(spec, w, _norm(spec, hidden, w, "input_layernorm"),
                                   cumulative_seq_lengths, position_ids, **kw)


def mlp_block(spec: LayerSpec, w: Dict[str, torch.Tensor], hidden: torch.Tensor) -> torch.Tensor:
    """transformer/model/layers/layer.py:276-293."""
    h = _norm(spec, hidden, w, "post_attention_layernorm")
    if spec.mlp_type == "swiglu":
        h = swiglu_mlp(h, w["mlp.dense_in.weight"], w["mlp.siglu_weight.weight"], w["mlp.dense_out.weight"],
                       w.get("mlp.dense_in.bias"), w.get("mlp.siglu_weight.bias"), w.get("mlp.dense_out.bias"))
    else:
        h = gelu_mlp(h, w["mlp.dense_in.weight"], w["mlp.dense_out.weight"],
                     w.get("mlp.dense_in.bias"), w.get("mlp.dense_out.bias"))
    return hidden + h


def transformer_layer(spec, w, hidden, cumulative_seq_lengths, position_ids, **kw) -> torch.Tensor:
    """transformer/model/layers/layer.py:295-345."""
    return mlp_block(spec, w, attention_block(spec, w, hidden, cumulative_seq_lengths, position_ids, **kw))


def final_norm(spec: LayerSpec, w: Dict[str, torch.Tensor], hidden: torch.Tensor) -> torch.Tensor:
    """transformer/model/layers/layernorm.py:36-59."""
    return _norm(spec, hidden, w, "norm")


# ---------------------------------------------------------------------------------------------
# decoder stack + greedy generation (embedding -> layers -> final norm -> LM head)
# ---------------------------------------------------------------------------------------------

def _logits(spec, model, token_ids, position_ids, cu, caches, use_cache, reset_cache):
    """core/nn/parallel_module/inference_module.py:100-109: one no-grad pass through all layers."""
    h = F.embedding(token_ids, model["embedding.weight"])
    tables = spec.tables() if spec.rotary == "rotary" else None
    for i, w in enumerate(model["layers"]):
        h = transformer_layer(spec, w, h, cu, position_ids, tables=tables, use_cache=use_cache,
                              reset_cache=reset_cache, cache=caches[i] if caches is not None else None)
    h = final_norm(spec, model["final"], h)
    return F.linear(h, model["lm_head.weight"])


@torch.no_grad()
def generate_uncached(spec: LayerSpec, model: dict, input_tokens: List[int], max_tokens: int):
    """transformer/inference/inference_model.py:188-221: re-run the whole prefix every step."""
    ids = torch.tensor(input_tokens).unsqueeze(0)
    tokens = []
    logits = None
    for _ in range(max_tokens):
        cu = get_cumulative_seq_lengths(ids)
        logits = _logits(spec, model, ids, get_position_ids(ids), cu, None, False, False)
        nxt = int(logits[0, -1].argmax())  # transformer/inference/sample.py:5-6
        tokens.append(nxt)
        ids = torch.cat((ids, torch.tensor([[nxt]])), dim=-1)
    return tokens, logits[0, len(input_tokens) - 1:]


@torch.no_grad()
def generate_cached(spec: LayerSpec, model: dict, input_tokens: List[int], max_tokens: int):
    """transformer/inference/inference_model.py:223-263: prefill, then one token per step."""
    ids = torch.tensor(input_tokens).unsqueeze(0)
    caches: List[KVCache] = [dict() for _ in model["layers"]]
    pos = get_position_ids(ids)
    reset = True
    tokens, step_logits = [], []
    for k in range(max_tokens):
        cu = get_cumulative_seq_lengths(ids)
        logits = _logits(spec, model, ids, pos, cu, caches, True, reset)
        reset = False
        nxt = int(logits[0, -1].argmax())
        tokens.append(nxt)
        step_logits.append(logits[0, -1:])
        ids = torch.tensor([[nxt]])
        pos = torch.tensor([[len(input_tokens) + k]])
    return tokens, torch.cat(step_logits)
