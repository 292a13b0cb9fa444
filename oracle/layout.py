"""Oracle: packed <-> padded index arithmetic.

axon/utils/torch/ops.py:339-348 (``get_unpad_data``) and
axon/utils/fsdp/forward_utils.py:131,164-182 (label roll, pad back, shift right).
"""

from __future__ import annotations

import torch


def unpad_data(attention_mask):
    lens = attention_mask.sum(-1).to(torch.int32)
    indices = attention_mask.flatten().nonzero().flatten()
    cu = torch.zeros(lens.numel() + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    return indices, cu, int(lens.max()) if lens.numel() else 0


def head_outputs_to_token_positions(packed_values, indices, batch, seqlen):
    """Scatter packed head outputs to [B,T], then shift right by one with a zero in column 0."""
    full = torch.zeros(batch * seqlen, dtype=packed_values.dtype)
    full[indices] = packed_values
    full = full.view(batch, seqlen)
    out = torch.zeros_like(full)
    out[:, 1:] = full[:, :-1]
    return out
