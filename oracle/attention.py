"""Oracle (test infrastructure): dense mask, masked softmax and the attention core.

Follows core/nn/attention/attention.py and core/nn/masked_softmax/masked_softmax.py
of the reference.
"""

from typing import Optional

import torch

MASK_FILL = -10000.0  # core/nn/masked_softmax/masked_softmax.py:28


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """core/nn/attention/attention.py:60-69: query head h reads kv head h // n_rep.

    x is [s, b, n_kv, d]; result [s, b, n_kv * n_rep, d].
    """
    if n_rep == 1:
        return x
    return torch.repeat_interleave(x, n_rep, dim=2)


def get_max_seq_length(cumulative_seq_lengths: torch.Tensor) -> int:
    """core/nn/attention/attention.py:72-73: length of the longest document."""
    return int(torch.diff(cumulative_seq_lengths).max())


def cumulative_seq_lengths_to_dense_attention_mask(cumulative_seq_lengths: torch.Tensor,
                                                   seq_length_per_batch_item: int, causal: bool) -> torch.Tensor:
    """core/nn/attention/attention.py:76-105.

    Returns bool [b, 1, s, s] with True = masked.  Entries of the cumulative
    lengths that are multiples of the per-item sequence length cut the list
    into batch items (line 81); inside an item every document is a square block
    of allowed pairs, lower-triangular when causal.
    """
    s = int(seq_length_per_batch_item)
    cu = [int(v) for v in cumulative_seq_lengths.tolist()]
    cut_positions = [i for i, v in enumerate(cu) if v % s == 0]
    items = []
    for lo, hi in zip(cut_positions[:-1], cut_positions[1:]):
        lengths = [cu[i + 1] - cu[i] for i in range(lo, hi)]
        allowed = torch.zeros(sum(lengths), sum(lengths), dtype=torch.bool, device=cumulative_seq_lengths.device)
        start = 0
        for n in lengths:
            allowed[start:start + n, start:start + n] = True
            start += n
        items.append(allowed)
    allowed = torch.stack(items)
    if causal:
        allowed = torch.tril(allowed)
    return ~allowed.unsqueeze(1)


def masked_softmax(scores: torch.Tensor, mask: torch.Tensor, softmax_in_fp32: bool = False,
                   scale: float = 1.0) -> torch.Tensor:
    """core/nn/masked_softmax/masked_softmax.py:14-34 (the `torch` kernel).

    Optional upcast to fp32, optional multiplication by `scale`, masked entries
    overwritten by -10000, softmax over the key axis, cast back.
    """
    in_dtype = scores.dtype
    x = scores.float() if (softmax_in_fp32 and in_dtype != torch.float32) else scores
    if scale != 1.0:
        x = x * scale
    x = x.masked_fill(mask, MASK_FILL)
    probs = torch.softmax(x, dim=-1)
    return probs.to(in_dtype)


def multi_head_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                         cumulative_seq_lengths: torch.Tensor, causal: bool,
                         query_key_scaling_factor: float, softmax_in_fp32: bool = False,
                         softmax_scale: float = 1.0, dropout_p: float = 0.0,
                         mask: Optional[torch.Tensor] = None,
                         dropout_keep: Optional[torch.Tensor] = None) -> torch.Tensor:
    """core/nn/attention/attention.py:108-213 with `MaskedSoftmaxTorch` as softmax_fn.

    query [s_q, b, n, d]; key, value [s_k, b, n, d] (kv heads already repeated).
    Returns [(b n), s_q, d].  Scores are alpha * Q K^T *in the input dtype*
    (`baddbmm`, lines 154-160), the mask comes from the query-side cumulative
    lengths with s_q as the per-item length (lines 166-168), probabilities are
    cast to the value dtype before P V (line 211).  Dropout (lines 204-207, torch.nn.Dropout on the
    probabilities) is restated with an explicit keep mask `dropout_keep` [b, n, s_q, s_k] (bool) so that a
    test can supply the mask the kernels generate: probs * keep / (1 - dropout_p).  Attention-score
    manipulation is outside the restated path.
    """
    assert (dropout_p == 0.0) == (dropout_keep is None), "dropout needs both the rate and the keep mask"
    s_q, b, n, d = query.shape
    q = query.permute(1, 2, 0, 3).reshape(b * n, s_q, d)
    k = key.permute(1, 2, 0, 3).reshape(b * n, key.shape[0], d)
    v = value.permute(1, 2, 0, 3).reshape(b * n, value.shape[0], d)
    scores = torch.baddbmm(
        torch.empty(b * n, s_q, k.shape[1], dtype=q.dtype, device=q.device),
        q, k.transpose(1, 2), beta=0.0, alpha=query_key_scaling_factor,
    )
    scores = scores.view(b, n, s_q, k.shape[1])
    if mask is None:
        mask = cumulative_seq_lengths_to_dense_attention_mask(cumulative_seq_lengths, s_q, causal)
    probs = masked_softmax(scores, mask, softmax_in_fp32=softmax_in_fp32, scale=softmax_scale)
    if dropout_keep is not None:
        probs = probs * dropout_keep.to(probs.dtype) * (1.0 / (1.0 - dropout_p))
    probs = probs.reshape(b * n, s_q, k.shape[1])
    return torch.bmm(probs.to(v.dtype), v)
