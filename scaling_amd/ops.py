"""Tensor-level entry points of the HIP kernels (through the C ABI) and their autograd wrappers.

Every function here launches a hand-written gfx950 kernel on the current stream.  None of them falls
back to PyTorch arithmetic: tensors must live on the GPU, and shapes or dtypes a kernel does not
support raise.  Autograd functions keep tensors with ``ctx.save_for_backward`` only, so they work
under saved-tensor hooks (activation checkpointing) and are deterministic under recomputation.
"""

import ctypes
import math
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import MiAttnArgs, MiAttnBwdArgs, MiDecodeArgs, check, dtype_code, ptr, stream_ptr

__all__ = [
    "rms_norm", "swiglu", "rotary_embedding", "rotary_embedding_complex", "attention", "attention_forward", "attention_backward",
    "decode_attention", "rms_norm_forward", "rms_norm_backward", "swiglu_forward", "swiglu_backward",
    "cross_entropy", "cross_entropy_forward", "linear_cross_entropy", "add_rms_norm",
]


def _need_cuda(*tensors):
    _lib.require_device()
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("scaling_amd ops take GPU tensors only (got a CPU tensor); there is no CPU path")


# ------------------------------------------------------------------------------------------------
# RMSNorm
# ------------------------------------------------------------------------------------------------
def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """(x + residual, rms_norm(x + residual) * weight) in one launch (inference; no autograd).  The sum is rounded
    to the tensor dtype before it is normalised, as the separate add and norm would do."""
    _need_cuda(x, residual, weight)
    assert x.shape == residual.shape and x.dtype == residual.dtype == weight.dtype and x.shape[-1] == weight.shape[0]
    x2, r2 = x.contiguous().view(-1, x.shape[-1]), residual.contiguous().view(-1, x.shape[-1])
    total, y = torch.empty_like(x2), torch.empty_like(x2)
    check(_lib.load().mi_add_rmsnorm_fwd(ptr(x2), ptr(r2), ptr(weight.contiguous()), ptr(total), ptr(y), x2.shape[0], x2.shape[1],
                                         float(eps), dtype_code(x.dtype), stream_ptr()), "mi_add_rmsnorm_fwd")
    return total.view(x.shape), y.view(x.shape)


def rms_norm_forward(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _need_cuda(x, weight)
    assert x.shape[-1] == weight.shape[0] and weight.dtype == x.dtype
    x2 = x.contiguous().view(-1, x.shape[-1])
    w = weight.contiguous()
    y = torch.empty_like(x2)
    check(_lib.load().mi_rmsnorm_fwd(ptr(x2), ptr(w), ptr(y), None, x2.shape[0], x2.shape[1], float(eps),
                                     dtype_code(x.dtype), stream_ptr()), "mi_rmsnorm_fwd")
    return y.view(x.shape)


def rms_norm_backward(x: torch.Tensor, weight: torch.Tensor, dy: torch.Tensor, eps: float):
    _need_cuda(x, weight, dy)
    lib = _lib.load()
    if x.numel() == 0:                   # no rows: no launch, the weight gradient is a sum over nothing
        return torch.empty_like(x), torch.zeros_like(weight)
    x2 = x.contiguous().view(-1, x.shape[-1])
    dy2 = dy.contiguous().view(-1, x.shape[-1])
    w = weight.contiguous()
    dx = torch.empty_like(x2)
    dw = torch.empty_like(w)
    nbytes = lib.mi_rmsnorm_bwd_workspace_bytes(x2.shape[0], x2.shape[1])
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    check(lib.mi_rmsnorm_bwd(ptr(x2), ptr(w), ptr(dy2), ptr(dx), ptr(dw), ptr(ws), nbytes, x2.shape[0], x2.shape[1],
                             float(eps), dtype_code(x.dtype), stream_ptr()), "mi_rmsnorm_bwd")
    return dx.view(x.shape), dw


class _RMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        ctx.save_for_backward(x, weight)
        ctx.eps = eps
        return rms_norm_forward(x, weight, eps)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dx, dw = rms_norm_backward(x, weight, dy, ctx.eps)
        return dx, dw, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2, -1) + eps) * weight (fp32 math, one rounding)."""
    return _RMSNorm.apply(x, weight, eps)


# ------------------------------------------------------------------------------------------------
# LayerNorm, GELU (the reference's default norm / activation)
# ------------------------------------------------------------------------------------------------
def layer_norm_forward(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
                       save_stats: bool = False):
    """y, or (y, stats) with stats an fp32 [2, n_rows] tensor (row means, then reciprocal standard deviations)
    for layer_norm_backward when save_stats is set."""
    _need_cuda(x, weight, bias)
    assert x.shape[-1] == weight.shape[0] and weight.dtype == x.dtype
    x2 = x.contiguous().view(-1, x.shape[-1])
    w = weight.contiguous()
    b = bias.contiguous() if bias is not None else None
    y = torch.empty_like(x2)
    stats = torch.empty(2, x2.shape[0], dtype=torch.float32, device=x.device) if save_stats else None
    check(_lib.load().mi_layernorm_fwd(ptr(x2), ptr(w), ptr(b), ptr(y), ptr(stats[0]) if save_stats else None,
                                       ptr(stats[1]) if save_stats else None, x2.shape[0], x2.shape[1], float(eps),
                                       dtype_code(x.dtype), stream_ptr()), "mi_layernorm_fwd")
    return (y.view(x.shape), stats) if save_stats else y.view(x.shape)


def layer_norm_backward(x: torch.Tensor, weight: torch.Tensor, dy: torch.Tensor, eps: float, need_bias_grad: bool = True,
                        stats: Optional[torch.Tensor] = None):
    """(dx, dweight, dbias).  `stats` is what layer_norm_forward(save_stats=True) returned for the same x, or
    None to have the statistics recomputed."""
    _need_cuda(x, weight, dy)
    lib = _lib.load()
    if x.numel() == 0:                   # no rows: no launch, the parameter gradients are sums over nothing
        return torch.empty_like(x), torch.zeros_like(weight), (torch.zeros_like(weight) if need_bias_grad else None)
    if stats is not None:
        assert stats.dtype == torch.float32 and stats.is_contiguous() and stats.shape == (2, x.numel() // x.shape[-1])
    x2 = x.contiguous().view(-1, x.shape[-1])
    dy2 = dy.contiguous().view(-1, x.shape[-1])
    w = weight.contiguous()
    dx = torch.empty_like(x2)
    dw = torch.empty_like(w)
    db = torch.empty_like(w) if need_bias_grad else None
    nbytes = lib.mi_layernorm_bwd_workspace_bytes(x2.shape[0], x2.shape[1])
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    check(lib.mi_layernorm_bwd(ptr(x2), ptr(w), ptr(dy2), ptr(stats[0]) if stats is not None else None,
                               ptr(stats[1]) if stats is not None else None, ptr(dx), ptr(dw), ptr(db), ptr(ws), nbytes,
                               x2.shape[0], x2.shape[1], float(eps), dtype_code(x.dtype), stream_ptr()), "mi_layernorm_bwd")
    return dx.view(x.shape), dw, db


class _LayerNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        y, stats = layer_norm_forward(x, weight, bias, eps, save_stats=True)
        ctx.save_for_backward(x, weight, stats)
        ctx.eps = eps
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, stats = ctx.saved_tensors
        dx, dw, db = layer_norm_backward(x, weight, dy, ctx.eps, ctx.has_bias, stats)
        return dx, dw, db, None


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, eps: float = 1e-5) -> torch.Tensor:
    """(x - mean) * rsqrt(var + eps) * weight + bias over the last dimension (fp32 math, one rounding)."""
    return _LayerNorm.apply(x, weight, bias, eps)


def gelu_forward(x: torch.Tensor) -> torch.Tensor:
    _need_cuda(x)
    x = x.contiguous()
    y = torch.empty_like(x)
    check(_lib.load().mi_gelu_fwd(ptr(x), ptr(y), x.numel(), dtype_code(x.dtype), stream_ptr()), "mi_gelu_fwd")
    return y


def gelu_backward(x: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    _need_cuda(x, dy)
    x, dy = x.contiguous(), dy.contiguous()
    dx = torch.empty_like(x)
    check(_lib.load().mi_gelu_bwd(ptr(x), ptr(dy), ptr(dx), x.numel(), dtype_code(x.dtype), stream_ptr()), "mi_gelu_bwd")
    return dx


class _GELU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return gelu_forward(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return gelu_backward(x, dy)


def gelu(x: torch.Tensor) -> torch.Tensor:
    """Exact (erf) GELU."""
    return _GELU.apply(x)


# ------------------------------------------------------------------------------------------------
# SwiGLU
# ------------------------------------------------------------------------------------------------
def swiglu_forward(a: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    _need_cuda(a, gate)
    assert a.shape == gate.shape and a.dtype == gate.dtype
    a, gate = a.contiguous(), gate.contiguous()
    out = torch.empty_like(a)
    check(_lib.load().mi_swiglu_fwd(ptr(a), ptr(gate), ptr(out), a.numel(), dtype_code(a.dtype), stream_ptr()),
          "mi_swiglu_fwd")
    return out


def swiglu_backward(a: torch.Tensor, gate: torch.Tensor, dout: torch.Tensor):
    _need_cuda(a, gate, dout)
    a, gate, dout = a.contiguous(), gate.contiguous(), dout.contiguous()
    da, dg = torch.empty_like(a), torch.empty_like(gate)
    check(_lib.load().mi_swiglu_bwd(ptr(a), ptr(gate), ptr(dout), ptr(da), ptr(dg), a.numel(), dtype_code(a.dtype),
                                    stream_ptr()), "mi_swiglu_bwd")
    return da, dg


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, gate):
        ctx.save_for_backward(a, gate)
        return swiglu_forward(a, gate)

    @staticmethod
    def backward(ctx, dout):
        a, gate = ctx.saved_tensors
        return swiglu_backward(a, gate, dout)


def swiglu(a: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """silu(a) * gate."""
    return _SwiGLU.apply(a, gate)


# ------------------------------------------------------------------------------------------------
# rotary (stand-alone kernel)
# ------------------------------------------------------------------------------------------------
def _rotary_launch(x, cos, sin, position_ids, seq_len_for_null_ids, inverse, out=None):
    """x: [tokens, heads, head_dim] view whose last dim is contiguous; cos/sin: [rows, rot_dim]."""
    _need_cuda(x, cos, sin, position_ids)
    assert x.dim() == 3 and x.stride(2) == 1
    assert cos.is_contiguous() and sin.is_contiguous() and cos.shape == sin.shape and cos.dim() == 2
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if position_ids is not None:
        position_ids = position_ids.contiguous()
        assert position_ids.dtype == torch.int64 and position_ids.numel() == x.shape[0]
    check(_lib.load().mi_rotary(ptr(x), ptr(out), ptr(cos), ptr(sin), ptr(position_ids), x.shape[0], x.shape[1],
                                x.shape[2], cos.shape[1], x.stride(0), x.stride(1), out.stride(0), out.stride(1),
                                cos.shape[0], int(seq_len_for_null_ids), int(bool(inverse)), dtype_code(x.dtype),
                                dtype_code(cos.dtype), stream_ptr()), "mi_rotary")
    return out


class _Rotary(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos, sin, position_ids, seq_len_for_null_ids):
        ctx.save_for_backward(cos, sin, position_ids if position_ids is not None else torch.empty(0, device=x.device))
        ctx.has_ids = position_ids is not None
        ctx.seq_len = seq_len_for_null_ids
        return _rotary_launch(x, cos, sin, position_ids, seq_len_for_null_ids, False)

    @staticmethod
    def backward(ctx, dout):
        cos, sin, ids = ctx.saved_tensors
        if dout.stride(-1) != 1:
            dout = dout.contiguous()
        dx = _rotary_launch(dout, cos, sin, ids if ctx.has_ids else None, ctx.seq_len, True)
        return dx, None, None, None, None


def rotary_embedding(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                     position_ids: Optional[torch.Tensor] = None, seq_len_for_null_ids: int = 0) -> torch.Tensor:
    """Rotate-half rotary on x [tokens, heads, head_dim]; position_ids int64 [tokens] (flattened (b s))."""
    return _Rotary.apply(x, cos, sin, position_ids, seq_len_for_null_ids)


def _rotary_complex_launch(x, cos, sin, position_ids, seq_len_for_null_ids, inverse):
    _need_cuda(x, cos, sin, position_ids)
    assert x.dim() == 3 and x.stride(2) == 1
    assert cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
    assert cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == x.shape[2]
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    if position_ids is not None:
        position_ids = position_ids.contiguous()
        assert position_ids.dtype == torch.int64 and position_ids.numel() == x.shape[0]
    check(_lib.load().mi_rotary_complex(ptr(x), ptr(out), ptr(cos), ptr(sin), ptr(position_ids), x.shape[0], x.shape[1],
                                        x.shape[2], x.stride(0), x.stride(1), out.stride(0), out.stride(1), cos.shape[0],
                                        int(seq_len_for_null_ids), int(bool(inverse)), dtype_code(x.dtype), stream_ptr()),
          "mi_rotary_complex")
    return out


class _RotaryComplex(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cos, sin, position_ids, seq_len_for_null_ids):
        ctx.save_for_backward(cos, sin, position_ids if position_ids is not None else torch.empty(0, device=x.device))
        ctx.has_ids = position_ids is not None
        ctx.seq_len = seq_len_for_null_ids
        return _rotary_complex_launch(x, cos, sin, position_ids, seq_len_for_null_ids, False)

    @staticmethod
    def backward(ctx, dout):
        cos, sin, ids = ctx.saved_tensors
        if dout.stride(-1) != 1:
            dout = dout.contiguous()
        return _rotary_complex_launch(dout, cos, sin, ids if ctx.has_ids else None, ctx.seq_len, True), None, None, None, None


def rotary_embedding_complex(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                             position_ids: Optional[torch.Tensor] = None, seq_len_for_null_ids: int = 0) -> torch.Tensor:
    """Interleaved-pair rotary on x [tokens, heads, head_dim]; cos / sin fp32 [rows, head_dim/2]."""
    return _RotaryComplex.apply(x, cos, sin, position_ids, seq_len_for_null_ids)


# ------------------------------------------------------------------------------------------------
# cross entropy over vocabulary rows
# ------------------------------------------------------------------------------------------------
def cross_entropy_forward(logits: torch.Tensor, targets: torch.Tensor, row_scale: Optional[torch.Tensor] = None,
                          dlogits: Optional[torch.Tensor] = None, want_lse: bool = False):
    """One launch over logits [rows, vocab]: returns (losses fp32 [rows], argmax int32 [rows]) (+ lse if asked).

    With ``dlogits`` (same shape and dtype, may be ``logits`` itself) the gradient
    ``row_scale[r] * (softmax(x_r) - onehot(t_r))`` is written in the same pass."""
    _need_cuda(logits, targets, row_scale, dlogits)
    assert logits.dim() == 2 and logits.stride(1) == 1, "logits must be [rows, vocab] with contiguous vocab"
    assert targets.dtype == torch.int64 and targets.is_contiguous() and targets.numel() == logits.shape[0]
    if row_scale is not None:
        assert row_scale.dtype == torch.float32 and row_scale.is_contiguous() and row_scale.numel() == logits.shape[0]
    if dlogits is not None:
        assert dlogits.shape == logits.shape and dlogits.dtype == logits.dtype and dlogits.stride(1) == 1
    n, v = logits.shape
    losses = torch.empty(n, dtype=torch.float32, device=logits.device)
    argmax = torch.empty(n, dtype=torch.int32, device=logits.device)
    # with a gradient, rows that are very long, not a whole number of 16-byte vectors or not 16-byte aligned take two
    # launches that hand the log-sum-exp over: always supply the (rows x 4 bytes) buffer
    need_lse = want_lse or dlogits is not None
    lse = torch.empty(n, dtype=torch.float32, device=logits.device) if need_lse else None
    check(_lib.load().mi_cross_entropy(ptr(logits), ptr(targets), ptr(row_scale), ptr(losses), ptr(lse), ptr(argmax), ptr(dlogits),
                                       n, v, logits.stride(0), dlogits.stride(0) if dlogits is not None else 0,
                                       dtype_code(logits.dtype), stream_ptr()), "mi_cross_entropy")
    return (losses, argmax, lse) if want_lse else (losses, argmax)


class _CrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, targets):
        losses, argmax = cross_entropy_forward(logits, targets)
        ctx.save_for_backward(logits, targets)
        ctx.mark_non_differentiable(argmax)
        return losses, argmax

    @staticmethod
    def backward(ctx, dlosses, _dargmax):
        logits, targets = ctx.saved_tensors
        dlogits = torch.empty_like(logits)
        cross_entropy_forward(logits, targets, row_scale=dlosses.float().contiguous(), dlogits=dlogits)
        return dlogits, None


def cross_entropy(logits: torch.Tensor, targets: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Differentiable per-row losses (fp32) and the row argmax (int32) of logits [rows, vocab]."""
    if logits.stride(1) != 1:
        logits = logits.contiguous()
    return _CrossEntropy.apply(logits, targets.contiguous())


class _LinearCrossEntropy(torch.autograd.Function):
    """loss = sum_r w_r * CE(h_r W^T, t_r) / sum_r w_r without ever holding the [rows, vocab] logits: rows are
    processed in chunks, each chunk's logits become its gradient in place and are folded into dh / dW at once."""

    @staticmethod
    def forward(ctx, h, weight, targets, loss_weights, chunk_rows):
        n = h.shape[0]
        w32 = loss_weights.float().contiguous()
        total = w32.sum()
        row_scale = (w32 / total).contiguous()
        need_dh, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        dh = torch.empty_like(h) if need_dh else None
        dw = None      # one chunk: the product itself; several chunks: their sum, accumulated in fp32
        losses = torch.empty(n, dtype=torch.float32, device=h.device)
        argmax = torch.empty(n, dtype=torch.int32, device=h.device)
        for r0 in range(0, n, chunk_rows):
            r1 = min(n, r0 + chunk_rows)
            logits = torch.matmul(h[r0:r1], weight.t())                       # PyTorch GEMM, [chunk, vocab]
            grad_buf = logits if (need_dh or need_dw) else None
            lc, ac = cross_entropy_forward(logits, targets[r0:r1], row_scale=row_scale[r0:r1], dlogits=grad_buf)
            losses[r0:r1] = lc
            argmax[r0:r1] = ac
            if need_dh:
                torch.matmul(logits, weight, out=dh[r0:r1])
            if need_dw:
                prod = torch.matmul(logits.t(), h[r0:r1])
                if n <= chunk_rows:
                    dw = prod
                elif dw is None:
                    dw = prod.float()
                else:
                    dw.add_(prod)
        loss = (losses * w32).sum() / total
        ctx.save_for_backward(dh if need_dh else torch.empty(0), dw if need_dw else torch.empty(0))
        ctx.flags = (need_dh, need_dw, weight.dtype)
        ctx.mark_non_differentiable(argmax)
        return loss, argmax

    @staticmethod
    def backward(ctx, dloss, _dargmax):
        dh, dw = ctx.saved_tensors
        need_dh, need_dw, wdtype = ctx.flags
        return (dh * dloss.to(dh.dtype) if need_dh else None, (dw * dloss).to(wdtype) if need_dw else None, None, None, None)


def linear_cross_entropy(h: torch.Tensor, weight: torch.Tensor, targets: torch.Tensor, loss_weights: torch.Tensor,
                         chunk_rows: int = 8192) -> Tuple[torch.Tensor, torch.Tensor]:
    """LM head + weighted cross entropy, chunked over rows.  h [rows, hidden], weight [vocab, hidden].
    The transient logits take chunk_rows * vocab * 2 bytes (2.1 GB at the default and a 128k vocabulary); larger
    chunks keep the three GEMMs efficient and the fp32 accumulation of dweight rare (measured at 8192 rows x 128256:
    23.4 ms with one chunk, 28.4 ms with four, 39.9 ms with eight).

    Returns (loss, argmax int32 [rows]); the gradients of h and weight are computed in the forward pass."""
    _need_cuda(h, weight, targets, loss_weights)
    assert h.dim() == 2 and weight.dim() == 2 and h.shape[1] == weight.shape[1] and h.dtype == weight.dtype
    return _LinearCrossEntropy.apply(h.contiguous(), weight, targets.contiguous().view(-1), loss_weights.contiguous().view(-1),
                                     int(chunk_rows))


# ------------------------------------------------------------------------------------------------
# attention core
# ------------------------------------------------------------------------------------------------
def _fused_rotary_kind(cos: torch.Tensor, sin: torch.Tensor, head_dim: int, dtype: torch.dtype) -> bool:
    """Checks the tables of a fused rotary; True for the interleaved-pair variant (fp32 tables [rows, head_dim / 2],
    RotaryEmbeddingComplex), False for rotate-half (tables [rows, head_dim] in the tensors' dtype)."""
    assert cos.is_contiguous() and sin.is_contiguous() and cos.shape == sin.shape and cos.dim() == 2
    if cos.dtype == torch.float32 and cos.shape[1] * 2 == head_dim and dtype != torch.float32:
        assert sin.dtype == torch.float32
        return True
    assert cos.dtype == dtype and sin.dtype == dtype and cos.shape[1] == head_dim, \
        "fused rotary takes [rows, head_dim] tables in the data dtype or fp32 [rows, head_dim / 2] tables (interleaved pairs)"
    return False


def _fill_attn_args(q, k, v, o, lse, cu_q, cu_k, causal, scale, rotary=None, flags=0, dropout=None, q_rot=None) -> MiAttnArgs:
    a = MiAttnArgs()
    a.flags = int(flags)
    a.q, a.k, a.v, a.o, a.lse = ptr(q), ptr(k), ptr(v), ptr(o), ptr(lse)
    a.cu_seqlens_q, a.cu_seqlens_k = ptr(cu_q), ptr(cu_k)
    a.n_docs = cu_q.numel() - 1
    a.causal = int(bool(causal))
    a.total_q, a.total_k = q.shape[0], k.shape[0]
    a.n_q_heads, a.n_kv_heads, a.head_dim = q.shape[1], k.shape[1], q.shape[2]
    a.dtype = dtype_code(q.dtype)
    a.q_stride_token, a.q_stride_head = q.stride(0), q.stride(1)
    a.k_stride_token, a.k_stride_head = k.stride(0), k.stride(1)
    a.v_stride_token, a.v_stride_head = v.stride(0), v.stride(1)
    a.o_stride_token, a.o_stride_head = o.stride(0), o.stride(1)
    a.softmax_scale = float(scale)
    if rotary is not None:
        cos, sin, pos_q, pos_k = rotary
        a.rotary_cos, a.rotary_sin = ptr(cos), ptr(sin)
        a.position_ids_q, a.position_ids_k = ptr(pos_q), ptr(pos_k)
        a.rotary_table_rows = cos.shape[0]
        a.rotary_interleaved = int(_fused_rotary_kind(cos, sin, q.shape[2], q.dtype))
        a.q_rot_out = ptr(q_rot)
    if dropout is not None and dropout[0] > 0.0:
        a.dropout_p, a.dropout_seed = float(dropout[0]), int(dropout[1]) & 0xFFFFFFFFFFFFFFFF
    a.stream = stream_ptr()
    return a


def _check_qkv(q, k, v, cu_q, cu_k):
    _need_cuda(q, k, v, cu_q, cu_k)
    for t in (q, k, v):
        assert t.dim() == 3 and t.stride(2) == 1, "q/k/v must be [tokens, heads, head_dim] with contiguous features"
    assert k.shape == v.shape and q.shape[2] == k.shape[2]
    assert cu_q.dtype == torch.int32 and cu_q.is_contiguous()
    if cu_k is not None:
        assert cu_k.dtype == torch.int32 and cu_k.is_contiguous() and cu_k.numel() == cu_q.numel()


SPLIT_P = 4   # MI_ATTN_SPLIT_P


def attention_forward(q, k, v, cu_seqlens_q, cu_seqlens_k=None, causal=True, softmax_scale=None, rotary=None, flags=0,
                      dropout=None, return_rotated_q=False, precise=False):
    """Returns (o [tokens, n_q_heads, head_dim], lse fp32 [n_q_heads, tokens]) (+ the rotated q if asked).

    rotary: optional (cos, sin, position_ids_q, position_ids_k), q and k are rotated while they are loaded:
    rotate-half with [rows, head_dim] tables in q's dtype, interleaved pairs with fp32 [rows, head_dim / 2] tables.
    position_ids_k = None: k is rotated already, only q is rotated in the kernel (the cheaper arrangement, see
    include/mi355_layer.h); return_rotated_q then also returns the rotated q (strides of q) for the backward.

    dropout: optional (p, seed) for dropout on the attention probabilities; the backward needs the same pair.

    flags: 0 lets the library pick the tiling; 1 / 2 pin one / two query groups per wavefront.
    precise: accuracy mode (probabilities enter P V as two bf16 terms; no dropout, rotary on q only)."""
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[2])
    if precise:
        flags |= SPLIT_P
    q_rot = None
    if rotary is not None:
        cos, sin, pos_q, pos_k = rotary
        _fused_rotary_kind(cos, sin, q.shape[2], q.dtype)
        assert pos_q.dtype == torch.int64 and pos_q.is_contiguous() and pos_q.numel() == q.shape[0]
        assert pos_k is None or (pos_k.dtype == torch.int64 and pos_k.is_contiguous() and pos_k.numel() == k.shape[0])
        if return_rotated_q:
            q_rot = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
    else:
        assert not return_rotated_q
    o = torch.empty((q.shape[0], q.shape[1], q.shape[2]), dtype=q.dtype, device=q.device)
    lse = torch.empty((q.shape[1], q.shape[0]), dtype=torch.float32, device=q.device)
    a = _fill_attn_args(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, causal, softmax_scale, rotary, flags, dropout, q_rot)
    check(_lib.load().mi_attn_fwd(ctypes.byref(a)), "mi_attn_fwd")
    return (o, lse, q_rot) if return_rotated_q else (o, lse)


def attention_backward(do, q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k=None, causal=True, softmax_scale=None,
                       flags=0, buffers=None, dropout=None, rotary=None, precise=False):
    """Returns (dq, dk, dv).  The summation order is fixed: results are bit-reproducible
    (what masked_softmax.deterministic_flash_attn_bwd asks of the reference's fused kernel holds always).

    rotary = (cos, sin, position_ids_q, position_ids_k): q and k are the ROTATED tensors the forward attended with, and
    dq / dk come back as gradients of the unrotated ones (rotated back inside the kernels, one rounding).

    flags: 0 runs the whole backward; 16 / 32 / 64 run only the delta / dK-dV / dQ kernel (timing aid).
    buffers: optional (dq, dk, dv, workspace) to reuse across calls.
    precise: accuracy mode (P and dS enter their MFMAs as two bf16 terms each; no dropout)."""
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k)
    lib = _lib.load()
    if precise:
        flags |= SPLIT_P
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[2])
    if do.stride() != o.stride():
        do = do.contiguous()
        assert do.stride() == o.stride()
    if buffers is not None:
        dq, dk, dv, ws = buffers
        assert dq.stride() == q.stride()
    else:
        dq = torch.empty_like(q)
        if dq.stride() != q.stride():
            dq = torch.empty_strided(q.shape, q.stride(), dtype=q.dtype, device=q.device)
        dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
        nbytes = lib.mi_attn_bwd_workspace_bytes_kv(q.shape[0], k.shape[0], q.shape[1], k.shape[1], q.shape[2])
        ws = torch.empty(max(nbytes // 4, 4), dtype=torch.float32, device=q.device)
    b = MiAttnBwdArgs()
    b.fwd = _fill_attn_args(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, causal, softmax_scale, rotary, flags, dropout)
    b.d_o, b.dq, b.dk, b.dv = ptr(do), ptr(dq), ptr(dk), ptr(dv)
    b.dk_stride_token, b.dk_stride_head = dk.stride(0), dk.stride(1)
    b.dv_stride_token, b.dv_stride_head = dv.stride(0), dv.stride(1)
    b.workspace, b.workspace_bytes = ptr(ws), ws.numel() * 4
    check(lib.mi_attn_bwd(ctypes.byref(b)), "mi_attn_bwd")
    return dq, dk, dv


class _Attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cu_q, cu_k, causal, scale, dropout_p, dropout_seed, cos, sin, pos_q, pos_k, precise):
        dropout = (dropout_p, dropout_seed) if dropout_p > 0.0 else None
        ctx.precise = precise
        if cos is None:
            o, lse = attention_forward(q, k, v, cu_q, cu_k, causal, scale, dropout=dropout, precise=precise)
            ctx.save_for_backward(q, k, v, o, lse, cu_q, cu_k if cu_k is not None else cu_q)
        else:
            # rotary: k is rotated once by the stand-alone kernel, q while the attention kernel loads it; the rotated
            # tensors are what the backward kernels stream, so they are kept instead of q and k
            interleaved = _fused_rotary_kind(cos, sin, q.shape[2], q.dtype)
            k_rot = (_rotary_complex_launch if interleaved else _rotary_launch)(k, cos, sin, pos_k, 0, False)
            if any(ctx.needs_input_grad[:3]):
                o, lse, q_rot = attention_forward(q, k_rot, v, cu_q, cu_k, causal, scale, rotary=(cos, sin, pos_q, None),
                                                  dropout=dropout, return_rotated_q=True, precise=precise)
                ctx.save_for_backward(q_rot, k_rot, v, o, lse, cu_q, cu_k if cu_k is not None else cu_q, cos, sin, pos_q, pos_k)
            else:   # nothing to differentiate: the rotated q is not written out
                o, lse = attention_forward(q, k_rot, v, cu_q, cu_k, causal, scale, rotary=(cos, sin, pos_q, None), dropout=dropout,
                                           precise=precise)
        ctx.causal, ctx.scale, ctx.dropout, ctx.rotary = causal, scale, dropout, cos is not None
        return o

    @staticmethod
    def backward(ctx, do):
        saved = ctx.saved_tensors           # read once: saved-tensor hooks (activation checkpointing) unpack on access
        q, k, v, o, lse, cu_q, cu_k = saved[:7]
        rotary = tuple(saved[7:11]) if ctx.rotary else None
        dq, dk, dv = attention_backward(do, q, k, v, o, lse, cu_q, cu_k, ctx.causal, ctx.scale, dropout=ctx.dropout, rotary=rotary,
                                        precise=ctx.precise)
        return (dq, dk, dv) + (None,) * 11


def next_dropout_seed(device: torch.device) -> int:
    """A fresh 64-bit seed from the device's default generator without touching the GPU: (seed, offset) of the
    Philox state, with the offset advanced as torch's own random kernels do.  The state is part of what
    torch.utils.checkpoint saves and restores, so a recomputed forward draws the same seed."""
    gen = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4)
    return (seed * 0x9E3779B97F4A7C15 + offset * 0xD1B54A32D192ED03 + 0x2545F4914F6CDD1D) & 0xFFFFFFFFFFFFFFFF


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens_q: torch.Tensor,
              cu_seqlens_k: Optional[torch.Tensor] = None, causal: bool = True,
              softmax_scale: Optional[float] = None, dropout_p: float = 0.0,
              dropout_seed: Optional[int] = None, rotary=None, deterministic: bool = False, precise: bool = False) -> torch.Tensor:
    """Differentiable attention core on q [tokens, n_q, d], k/v [tokens_k, n_kv, d] (bfloat16, float16 or float32;
    float32 tensors run separate kernels on the fp32 matrix pipe with exact fp32 probabilities, without dropout).

    Tokens are the flattened (batch seq) axis; cu_seqlens are int32 offsets on it.  Returns
    o [tokens, n_q, d].  dropout_p > 0 drops attention probabilities (attention.py:204-207) with a mask that
    is a function of (dropout_seed, head, query, key); without a seed one is drawn from the device generator.
    The drop probability is quantised to round(256 p) / 256.

    rotary = (cos, sin, position_ids_q, position_ids_k) applies the rotary embedding of the whole head to q and k
    (attention.py:836-845; table formats as for attention_forward) and differentiates through it: q is rotated while
    the forward kernel loads it, k by one stand-alone launch, and the backward kernels rotate dq / dk back in their
    epilogues, with or without autograd, with or without dropout.
    deterministic mirrors masked_softmax.deterministic_flash_attn_bwd of the reference; the kernels sum in a fixed
    order whatever its value.
    precise selects the accuracy mode of forward and backward: P and dS enter their products as two bf16 terms, which
    brings outputs and gradients within max-abs 2e-2 / mean-relative 1e-3 of the fp32 reference (the default mode
    rounds P once to bf16 as the reference does); bench.py times both modes (`accuracy_mode.time_over_default`); no
    dropout.  Exception: with `rotary` the rotated q and k are rounded once to the I/O dtype before the score product
    in either mode, which leaves a mean-relative error of about 2e-3 against the fp32 reference (0.5 - 0.75 x what the
    reference's own bf16 path shows there).
    """
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(q.shape[2])
    if dropout_p > 0.0 and dropout_seed is None:
        dropout_seed = next_dropout_seed(q.device)
    cos = sin = pos_q = pos_k = None
    if rotary is not None and q.dtype == torch.float32:
        # float32 tensors: the rotation runs as the stand-alone (differentiable) kernel in front of the fp32 attention core
        cos, sin, pos_q, pos_k = rotary
        rot = rotary_embedding_complex if cos.shape[1] * 2 == q.shape[2] else rotary_embedding
        q, k = rot(q, cos, sin, pos_q), rot(k, cos, sin, pos_k)
        rotary = cos = sin = pos_q = pos_k = None
    if rotary is not None:
        cos, sin, pos_q, pos_k = rotary
        _fused_rotary_kind(cos, sin, q.shape[2], q.dtype)
        assert pos_q.dtype == torch.int64 and pos_q.is_contiguous() and pos_q.numel() == q.shape[0]
        assert pos_k.dtype == torch.int64 and pos_k.is_contiguous() and pos_k.numel() == k.shape[0]
    return _Attention.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, causal, float(softmax_scale), float(dropout_p),
                            int(dropout_seed) if dropout_seed is not None else 0, cos, sin, pos_q, pos_k, bool(precise))


# ------------------------------------------------------------------------------------------------
# decode attention over a pre-allocated KV cache
# ------------------------------------------------------------------------------------------------
def decode_workspace(batch: int, n_q_heads: int, head_dim: int, max_ctx: int, device) -> torch.Tensor:
    nbytes = _lib.load().mi_attn_decode_workspace_bytes(batch, n_q_heads, head_dim, max_ctx)
    return torch.empty(nbytes // 4, dtype=torch.float32, device=device)


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, ctx_len: torch.Tensor,
                     k_new: Optional[torch.Tensor] = None, v_new: Optional[torch.Tensor] = None,
                     rotary: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None,
                     softmax_scale: Optional[float] = None, workspace: Optional[torch.Tensor] = None,
                     n_splits: int = 0, out: Optional[torch.Tensor] = None, static_scratch: bool = False) -> torch.Tensor:
    """One decode step.  q [B, n_q, d]; caches [B, max_ctx, n_kv, d]; ctx_len int32 [B] counts the valid
    keys INCLUDING the token appended by this call (k_new/v_new [B, n_kv, d], written at ctx_len-1).
    rotary = (cos, sin, position_ids[B]) rotates q and k_new inside the kernels (table formats as for
    attention_forward: rotate-half or interleaved pairs).  q, k_new and v_new may be
    column slices of one projection output: only their [heads, d] part has to be contiguous.
    static_scratch=True calls the entry point that allocates nothing (partial results in the library's static
    device array; `out` should be given too, and calls on one GPU must not overlap)."""
    _need_cuda(q, k_cache, v_cache, ctx_len)
    B, nq, d = q.shape

    def _rows(t):
        assert t.stride(2) == 1 and t.stride(1) == d and t.stride(0) % 8 == 0, "each sequence's [heads, d] block must be contiguous"
        return t.stride(0)

    assert k_cache.dim() == 4 and k_cache.shape == v_cache.shape
    assert k_cache.stride() == v_cache.stride() and k_cache.stride(3) == 1
    assert ctx_len.dtype == torch.int32 and ctx_len.numel() == B
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if workspace is None and not static_scratch:
        workspace = decode_workspace(B, nq, d, k_cache.shape[1], q.device)
    if out is None:
        out = torch.empty((B, nq, d), dtype=q.dtype, device=q.device)
    a = MiDecodeArgs()
    a.q, a.k_cache, a.v_cache, a.o, a.ctx_len = ptr(q), ptr(k_cache), ptr(v_cache), ptr(out), ptr(ctx_len)
    a.q_stride_batch = _rows(q)
    if k_new is not None:
        assert k_new.shape == (B, k_cache.shape[2], d) and v_new.shape == k_new.shape
        a.k_new, a.v_new = ptr(k_new), ptr(v_new)
        a.k_new_stride_batch, a.v_new_stride_batch = _rows(k_new), _rows(v_new)
    if rotary is not None:
        cos, sin, pos = rotary
        a.rotary_interleaved = int(_fused_rotary_kind(cos, sin, d, q.dtype))
        assert pos.dtype == torch.int64 and pos.numel() == B and pos.is_contiguous()
        a.rotary_cos, a.rotary_sin, a.position_ids = ptr(cos), ptr(sin), ptr(pos)
        a.rotary_table_rows = cos.shape[0]
    a.batch, a.max_ctx, a.n_q_heads, a.n_kv_heads, a.head_dim = B, k_cache.shape[1], nq, k_cache.shape[2], d
    a.dtype = dtype_code(q.dtype)
    a.cache_stride_batch, a.cache_stride_token, a.cache_stride_head = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    a.softmax_scale = float(softmax_scale)
    a.n_splits = int(n_splits)
    a.stream = stream_ptr()
    if static_scratch:
        check(_lib.load().mi_attn_decode_static(ctypes.byref(a)), "mi_attn_decode_static")
        return out
    a.workspace, a.workspace_bytes = ptr(workspace), workspace.numel() * 4
    check(_lib.load().mi_attn_decode(ctypes.byref(a)), "mi_attn_decode")
    return out
