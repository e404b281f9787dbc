"""Integer index construction for packed batches (host / device agnostic, no Python loops).

Same results, bit for bit, as transformer/data/utils.py:4-108 of the reference: cumulative sequence
lengths are int32 offsets on the flattened (batch seq) axis, position ids are int64 [batch, seq].
"""

import torch

EOD_TOKEN = 0  # the reference hard-codes the end-of-document id (transformer/data/utils.py:43)


def get_cumulative_seq_lengths(input_token_ids: torch.Tensor, reset_attention_mask: bool = True,
                               eod_token: int = EOD_TOKEN) -> torch.Tensor:
    b, s = input_token_ids.shape
    dev = input_token_ids.device
    if not reset_attention_mask:
        return torch.arange(0, b * s + 1, s, dtype=torch.int32, device=dev)
    is_end = input_token_ids == eod_token
    is_end = is_end | (torch.arange(s, device=dev) == s - 1)
    ends = torch.nonzero(is_end.reshape(-1)).reshape(-1) + 1
    return torch.cat((torch.zeros(1, dtype=torch.int32, device=dev), ends.to(torch.int32)))


def get_max_seq_length(cumulative_seq_lengths: torch.Tensor) -> int:
    """core/nn/attention/attention.py:72-73: length of the longest document (a host integer; the reference hands it
    to its flash-attention call, the hip kernels size their loops from the cumulative lengths themselves)."""
    return int(torch.diff(cumulative_seq_lengths).max().item())


def get_position_ids(input_token_ids: torch.Tensor, reset_position_ids: bool = True,
                     eod_token: int = EOD_TOKEN) -> torch.Tensor:
    b, s = input_token_ids.shape
    dev = input_token_ids.device
    idx = torch.arange(s, dtype=torch.long, device=dev).unsqueeze(0).expand(b, s)
    if not reset_position_ids:
        return idx
    # a document starts right after an end-of-document token (which itself closes the previous one)
    starts = torch.zeros(b, s, dtype=torch.long, device=dev)
    starts[:, 1:] = torch.where(input_token_ids[:, :-1] == eod_token, idx[:, 1:], torch.zeros_like(idx[:, 1:]))
    return (idx - torch.cummax(starts, dim=1).values).to(input_token_ids.dtype)


def add_cumulative_seq_lengths_padding(cumulative_seq_lengths: torch.Tensor, pad_to: int,
                                       padding_value: int = -1) -> torch.Tensor:
    assert pad_to >= len(cumulative_seq_lengths)
    pad = torch.full((pad_to - len(cumulative_seq_lengths),), padding_value, dtype=torch.int32,
                     device=cumulative_seq_lengths.device)
    return torch.cat((cumulative_seq_lengths, pad))


def remove_cumulative_seq_lengths_padding(cumulative_seq_lengths: torch.Tensor, padding_value: int = -1) -> torch.Tensor:
    return cumulative_seq_lengths[cumulative_seq_lengths != padding_value]
