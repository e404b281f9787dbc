"""Oracle (test infrastructure): integer index construction for packed batches.

Follows transformer/data/utils.py of the reference; all results are integer and
must be bit-exact.
"""

import torch

EOD_TOKEN = 0  # hard-coded end-of-document id, transformer/data/utils.py:43,80


def get_cumulative_seq_lengths(input_token_ids: torch.Tensor, reset_attention_mask: bool = True,
                               eod_token: int = EOD_TOKEN) -> torch.Tensor:
    """transformer/data/utils.py:40-74.

    Offsets on the flattened (batch seq) token axis: 0, then one past every token
    that is an EOD or the last of its row.  Without reset: every multiple of seq.
    Result dtype int32.
    """
    b, s = input_token_ids.shape
    if not reset_attention_mask:
        return torch.arange(0, b * s + 1, s, dtype=torch.int32, device=input_token_ids.device)
    ends = input_token_ids == eod_token
    ends = ends.clone()
    ends[:, s - 1] = True
    flat = torch.nonzero(ends.reshape(-1), as_tuple=False).reshape(-1)  # row-major order
    out = torch.empty(flat.numel() + 1, dtype=torch.int32, device=input_token_ids.device)
    out[0] = 0
    out[1:] = (flat + 1).to(torch.int32)
    return out


def get_position_ids(input_token_ids: torch.Tensor, reset_position_ids: bool = True,
                     eod_token: int = EOD_TOKEN) -> torch.Tensor:
    """transformer/data/utils.py:77-108.

    Positions restart at 0 after each EOD (the EOD itself still belongs to the
    document it closes).  int64, shape [b, s].
    """
    b, s = input_token_ids.shape
    if not reset_position_ids:
        return torch.arange(s, dtype=torch.long, device=input_token_ids.device).unsqueeze(0).expand(b, s)
    out = torch.zeros_like(input_token_ids)
    for row in range(b):
        pos = 0
        for col in range(s):
            out[row, col] = pos
            pos += 1
            if int(input_token_ids[row, col]) == eod_token:
                pos = 0
    return out


def add_cumulative_seq_lengths_padding(cumulative_seq_lengths: torch.Tensor, pad_to: int,
                                       padding_value: int = -1) -> torch.Tensor:
    """transformer/data/utils.py:4-22: right-pad with -1 (int32) to a fixed length."""
    n = cumulative_seq_lengths.numel()
    assert pad_to >= n
    pad = torch.full((pad_to - n,), padding_value, dtype=torch.int32, device=cumulative_seq_lengths.device)
    return torch.cat((cumulative_seq_lengths, pad))


def remove_cumulative_seq_lengths_padding(cumulative_seq_lengths: torch.Tensor,
                                          padding_value: int = -1) -> torch.Tensor:
    """transformer/data/utils.py:25-37."""
    return cumulative_seq_lengths[cumulative_seq_lengths != padding_value]
