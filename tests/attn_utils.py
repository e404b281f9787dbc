"""Helpers shared by the attention GPU tests: seeded inputs, layout conversion, oracle evaluation."""

import math

import torch

import oracle


def make_cu(b, s, cuts=()):
    """int32 cumulative lengths containing every multiple of s plus the given extra cut points."""
    return torch.tensor(sorted(set(i * s for i in range(b + 1)) | set(cuts)), dtype=torch.int32)


def random_docs_cu(total, lo, hi, seed):
    """Document lengths uniform in [lo, hi], last one truncated so the lengths sum to `total`."""
    g = torch.Generator().manual_seed(seed)
    cu = [0]
    while cu[-1] < total:
        n = int(torch.randint(lo, hi + 1, (1,), generator=g))
        cu.append(min(total, cu[-1] + n))
    return torch.tensor(cu, dtype=torch.int32)


def position_ids_from_cu(cu, total):
    pos = torch.zeros(total, dtype=torch.int64)
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        pos[a:b] = torch.arange(b - a)
    return pos


def make_qkv(b, s, nq, nkv, d, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b * s, nq, d, generator=g).to(dtype)
    k = torch.randn(b * s, nkv, d, generator=g).to(dtype)
    v = torch.randn(b * s, nkv, d, generator=g).to(dtype)
    do = torch.randn(b * s, nq, d, generator=g).to(dtype)
    return q, k, v, do


def to_sbnd(x, b, s):
    return x.view(b, s, x.shape[1], x.shape[2]).permute(1, 0, 2, 3)


def from_bn_s_d(o, b, n):
    # [(b n), s, d] -> [(b s), n, d]
    s, d = o.shape[1], o.shape[2]
    return o.view(b, n, s, d).permute(0, 2, 1, 3).reshape(b * s, n, d)


def _lowbias32(x):
    import numpy as np
    x = x.astype(np.uint32)
    x ^= x >> np.uint32(16); x = (x * np.uint32(0x7FEB352D)).astype(np.uint32)
    x ^= x >> np.uint32(15); x = (x * np.uint32(0x846CA68B)).astype(np.uint32)
    x ^= x >> np.uint32(16)
    return x


def dropout_keep_mask(seed, n_heads, total_q, total_k, p):
    """The keep mask the kernels generate (integer arithmetic documented with mi_attn_args in include/mi355_layer.h):
    returns (keep bool [heads, total_q, total_k], effective drop probability)."""
    import numpy as np
    thr = min(255, max(1, int(p * 256.0 + 0.5)))
    seed32 = np.uint32((seed & 0xFFFFFFFF) ^ ((seed >> 32) & 0xFFFFFFFF))
    heads = np.arange(n_heads, dtype=np.uint64)
    with np.errstate(over="ignore"):
        inner = _lowbias32(((heads * 0x9E3779B9 + 0x7F4A7C15) & 0xFFFFFFFF).astype(np.uint32))
        base = _lowbias32(inner ^ seed32).astype(np.uint64)
        q = np.arange(total_q, dtype=np.uint64)
        k = np.arange(total_k, dtype=np.uint64)
        x = (base[:, None, None] + ((q >> 1) * 0x9E3779B1)[None, :, None] + ((k >> 1) * 0x85EBCA77)[None, None, :]) & 0xFFFFFFFF
        h = _lowbias32(x.astype(np.uint32))
    shift = (16 * (q & 1))[None, :, None] + (8 * (k & 1))[None, None, :]
    byte = (h >> shift.astype(np.uint32)) & np.uint32(0xFF)
    return torch.from_numpy(byte >= thr), thr / 256.0


def oracle_attention(q, k, v, cu, b, s, causal, scale, dtype=torch.float32, do=None, softmax_in_fp32=True, dropout=None):
    """Runs the oracle on token-major tensors; returns o (and dq, dk, dv when `do` is given) in token layout.

    dropout = (keep [heads, b*s, b*s] bool, effective p): the diagonal blocks of the token-level mask are handed
    to the oracle in its [b, n, s, s] layout."""
    nq, nkv = q.shape[1], k.shape[1]
    qq, kk, vv = (t.to(dtype).clone().requires_grad_(do is not None) for t in (q, k, v))
    extra = {}
    if dropout is not None:
        keep, p_eff = dropout
        extra = dict(dropout_p=p_eff, dropout_keep=torch.stack([keep[:, i * s:(i + 1) * s, i * s:(i + 1) * s] for i in range(b)]))
    out = oracle.multi_head_attention(
        to_sbnd(qq, b, s), oracle.repeat_kv(to_sbnd(kk, b, s), nq // nkv), oracle.repeat_kv(to_sbnd(vv, b, s), nq // nkv),
        cu, causal, scale, softmax_in_fp32=softmax_in_fp32, **extra)
    o = from_bn_s_d(out, b, nq)
    if do is None:
        return o.detach()
    o.backward(do.to(dtype))
    return o.detach(), qq.grad, kk.grad, vv.grad


def rows_reference(q, k, v, lo_hi, rows, head, kv_head, scale, reference_bf16_order=False):
    """Attention of selected query rows of one head against keys [lo, hi) per row (size-independent check).

    Default: fp64 truth.  reference_bf16_order=True reproduces the reference's rounding points for
    bf16 tensors instead (scores rounded to bf16, fp32 softmax, probabilities rounded to bf16, output bf16).
    """
    outs = []
    for r in rows:
        lo, hi = lo_hi(r)
        if reference_bf16_order:
            sc = ((k[lo:hi, kv_head].float() @ q[r, head].float()) * scale).bfloat16().float()
            p = torch.softmax(sc, 0).bfloat16().float()
            outs.append((p @ v[lo:hi, kv_head].float()).bfloat16().float())
        else:
            sc = (k[lo:hi, kv_head].double() @ q[r, head].double()) * scale
            p = torch.softmax(sc, 0)
            outs.append((p @ v[lo:hi, kv_head].double()).float())
    return torch.stack(outs)


DEFAULT_SCALE = lambda d: 1.0 / math.sqrt(d)  # noqa: E731
