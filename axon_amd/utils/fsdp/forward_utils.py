"""Packed-batch layout helpers around the fused LM head.

Index arithmetic of axon/utils/fsdp/forward_utils.py:88-182 (``unpad_inputs``,
``prepare_rmpad_inputs``, ``rmpad_postprocess``) and ``get_unpad_data``
(axon/utils/torch/ops.py:339-348), restated with torch index ops (the reference
uses flash_attn.bert_padding for the same gathers).  These are tiny gathers over
[B, T] integers and run on whatever device the inputs live on.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def get_unpad_data(attention_mask: torch.Tensor):
    """``(indices, cu_seqlens int32 [B+1], max_seqlen)`` of the valid positions."""
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    max_len = int(seqlens.max().item()) if seqlens.numel() else 0
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    return indices, cu_seqlens, max_len


def unpad_input_ids(input_ids: torch.Tensor, attention_mask: torch.Tensor):
    """[B, T] ids -> packed ``(1, N)`` ids, flat ``indices`` [N], ``cu_seqlens``."""
    indices, cu_seqlens, _ = get_unpad_data(attention_mask)
    packed = input_ids.flatten()[indices].unsqueeze(0)
    return packed, indices, cu_seqlens


def rolled_labels(packed_ids: torch.Tensor) -> torch.Tensor:
    """Next-token labels over the whole packed stream (forward_utils.py:131).  The label of
    a sequence's last token is the next sequence's first token; it lands where
    ``response_mask`` is 0 after ``shift_to_token_positions``."""
    return torch.roll(packed_ids, shifts=-1, dims=-1)


def pad_packed(values: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int) -> torch.Tensor:
    """Scatter packed per-token values [N] back to [B, T] (zeros elsewhere)."""
    out = torch.zeros(batch * seqlen, device=values.device, dtype=values.dtype)
    out[indices] = values.reshape(-1)
    return out.view(batch, seqlen)


def shift_to_token_positions(full: torch.Tensor) -> torch.Tensor:
    """``full[b, t]`` predicts token t+1; return ``r`` with ``r[b, t]`` = value for token t and
    ``r[b, 0] = 0`` (forward_utils.py:180-182)."""
    return F.pad(full[:, :-1], (1, 0), value=0.0)


def rmpad_postprocess(t: torch.Tensor, *, indices: torch.Tensor, batch_size: int, seqlen: int) -> torch.Tensor:
    """Packed head output -> [B, T] aligned to token positions."""
    return shift_to_token_positions(pad_packed(t, indices, batch_size, seqlen))


def shift_packed(values: torch.Tensor, cu_seqlens: torch.Tensor) -> torch.Tensor:
    """The same re-alignment without leaving the packed layout: ``out[p] = values[p-1]`` for a
    token that is not first in its sequence, ``0`` for a first token."""
    out = torch.roll(values, shifts=1, dims=0)
    starts = cu_seqlens[:-1].long()
    out[starts[starts < values.numel()]] = 0
    return out


def packed_logprobs(hidden, weight, packed_ids, cu_seqlens, temperature: float = 1.0, logit_softcapping=None,
                    response_mask=None):
    """Head of the remove-padding path in one call: packed hidden states ``[N, H]`` and the packed token ids
    ``[N]`` (or ``[1, N]``) in, ``(log_probs, entropy)`` ``[N]`` aligned to token positions out — what
    ``rolled_labels`` + the fused head + ``shift_packed`` produce, without the roll and shift passes
    (forward_utils.py:131,164-182 in packed form).

    ``response_mask`` ``[N]`` (optional; the reference has no such argument and runs the head over every
    token): the positions where it is zero — the prompt — come back as 0 and their rows stay out of the
    head, forward and backward.  Every consumer of these values weighs them with the same mask (``agg_loss``,
    axon/trainer/algos/loss/utils.py:120-251), so losses, gradients and masked metrics do not change.  Costs
    one readback (the number of response positions)."""
    from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy

    ids = packed_ids.reshape(-1)
    if response_mask is None:
        return linear_cross_entropy(hidden, weight, ids, float(temperature), "none", None, logit_softcapping,
                                    cu_seqlens)
    n = ids.numel()
    wanted = response_mask.reshape(-1) != 0
    if wanted.numel() != n:
        raise ValueError(f"response_mask has {wanted.numel()} entries for {n} packed tokens")
    starts = cu_seqlens[:-1].long()
    wanted[starts[starts < n]] = False  # a sequence's first token has no prediction (comparison made a new tensor)
    wanted[:1] = False
    pos = torch.nonzero(wanted).flatten()  # position p is predicted from the hidden state at p - 1
    lp_c, ent_c = linear_cross_entropy(hidden.reshape(n, -1).index_select(0, pos - 1), weight,
                                       ids.index_select(0, pos), float(temperature), "none", None,
                                       logit_softcapping)
    zeros = torch.zeros(n, device=lp_c.device, dtype=lp_c.dtype)
    return zeros.index_copy(0, pos, lp_c), zeros.index_copy(0, pos, ent_c)


def _from_logits(logits, labels, temperature: float, calculate_entropy: bool):
    """The non-fused head (forward_utils.py:287-304): divide the logits by the temperature in place, then
    log-probability and entropy from one pass over them."""
    from axon_amd.utils.torch.ops import logprobs_and_entropy_from_logits, logprobs_from_logits

    logits.div_(temperature)
    if calculate_entropy:
        return logprobs_and_entropy_from_logits(logits, labels)
    return logprobs_from_logits(logits, labels, inplace_backward=True), None


def fsdp_model_forward(module, micro_batch: dict, temperature: float, calculate_entropy: bool = False, *,
                       use_remove_padding: bool = True, use_fused_kernels: bool = True, ulysses_sp_size: int = 1,
                       skip_prompt_rows: bool = False, **_unused):
    """Forward one micro-batch through a model whose ``forward`` is the fused-head one
    (``forward_with_hip_backend``) and return ``(entropy, log_probs)``, both ``[batch, seq]``: position 0 is 0,
    position t holds log P(token_t | tokens before it).  Mirror of the fused branches of ``fsdp_model_forward``
    (forward_utils.py:185-318): with remove-padding the ids are unpadded, rolled over the packed stream and
    handed to the model as ``pre_rolled_labels`` (:236-265), the packed outputs are scattered back and shifted
    right (``rmpad_postprocess``, :164-182); without it the outputs are shifted right directly (:282-285).
    With ``use_fused_kernels=False`` the model writes the logits and ``axon_amd.utils.torch.ops`` turns them into
    log-probabilities and entropy (:287-304).  Ulysses sequence parallelism (more than one GPU) is not part of
    this build.

    ``skip_prompt_rows`` (no counterpart in the reference, off by default; fused branches only): positions where
    ``micro_batch["response_mask"]`` ``[batch, seq]`` is zero come back as 0 and their rows stay out of the head."""
    head_kwargs = {}
    if skip_prompt_rows and use_fused_kernels and "response_mask" in micro_batch:
        # hidden position t predicts token t + 1: keep it when the response mask covers t + 1
        keep = F.pad(micro_batch["response_mask"][:, 1:] != 0, (0, 1), value=False)
    if ulysses_sp_size > 1:
        raise NotImplementedError("Ulysses sequence parallelism needs more than one GPU")
    input_ids = micro_batch["input_ids"]
    batch_size, seqlen = input_ids.shape
    attention_mask = micro_batch["attention_mask"]
    position_ids = micro_batch["position_ids"]
    if position_ids.dim() == 3:  # mrope layout (channels first), forward_utils.py:224-225
        position_ids = position_ids.transpose(0, 1)
    if use_remove_padding:
        indices, cu_seqlens, _ = get_unpad_data(attention_mask)
        if indices.numel() == 0:  # all-zero mask: nothing to predict (forward_utils.py:122-127, 176-177)
            zeros = torch.zeros(batch_size, seqlen, device=input_ids.device, dtype=torch.float32)
            return (zeros if calculate_entropy else None), zeros.clone()
        fwd_ids = input_ids.flatten()[indices].unsqueeze(0)
        if position_ids.dim() == 3:
            fwd_pos = position_ids.flatten(1)[:, indices].unsqueeze(1)
        else:
            fwd_pos = position_ids.flatten()[indices].unsqueeze(0)
        labels = rolled_labels(fwd_ids)
        if use_fused_kernels:
            if skip_prompt_rows and "response_mask" in micro_batch:
                head_kwargs["head_row_mask"] = keep.flatten()[indices].unsqueeze(0)
            output = module(input_ids=fwd_ids, attention_mask=None, position_ids=fwd_pos, use_cache=False,
                            temperature=temperature, return_dict=True, pre_rolled_labels=labels, **head_kwargs)
            lp_packed = output.log_probs.reshape(-1)
            ent_packed = output.entropy.reshape(-1) if calculate_entropy else None
        else:  # the model writes the logits (forward_utils.py:287-292)
            output = module(input_ids=fwd_ids, attention_mask=None, position_ids=fwd_pos, use_cache=False)
            lp_packed, ent_packed = _from_logits(output.logits.squeeze(0), labels.reshape(-1), temperature,
                                                 calculate_entropy)
        log_probs = rmpad_postprocess(lp_packed, indices=indices, batch_size=batch_size, seqlen=seqlen)
        entropy = None
        if calculate_entropy:
            entropy = rmpad_postprocess(ent_packed, indices=indices, batch_size=batch_size, seqlen=seqlen)
        return entropy, log_probs
    if use_fused_kernels:
        if skip_prompt_rows and "response_mask" in micro_batch:
            head_kwargs["head_row_mask"] = keep
        output = module(input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids,
                        use_cache=False, temperature=temperature, return_dict=True, **head_kwargs)
        log_probs = shift_to_token_positions(output.log_probs.view(batch_size, seqlen))
        entropy = shift_to_token_positions(output.entropy.view(batch_size, seqlen)) if calculate_entropy else None
        return entropy, log_probs
    # padded, non-fused (forward_utils.py:294-304): logits[:, t] predicts token t + 1
    output = module(input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids, use_cache=False)
    lp, ent = _from_logits(output.logits[:, :-1, :], input_ids[:, 1:], temperature, calculate_entropy)
    log_probs = F.pad(lp, (1, 0), value=0.0)
    entropy = F.pad(ent, (1, 0), value=0.0) if calculate_entropy else None
    return entropy, log_probs
