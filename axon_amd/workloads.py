"""Seeded synthetic inputs for the five benchmark configurations.

Everything is drawn on the CPU from ``torch.Generator().manual_seed(seed)`` so the
same tensors can be fed to the HIP path and to the CPU oracle.  Shapes and
distributions follow the workload descriptions: uniform / log-normal ragged
lengths, ``-Exp(1)`` log-probs with small Gaussian perturbations, Bernoulli
rewards placed on the last valid token, groups of 8 (or 16) samples per prompt.
"""

from __future__ import annotations

import numpy as np
import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def ragged_lengths(total: int, g: torch.Generator, mu=6.5, sigma=0.8, lo=32, hi=8192) -> list[int]:
    """Sequence lengths ~ round(LogNormal(mu, sigma)) clipped to [lo, hi], summing to ``total`` exactly."""
    lens: list[int] = []
    left = total
    while left > 0:
        x = int(torch.exp(torch.randn((), generator=g) * sigma + mu).round().clamp(lo, hi))
        if left - x < lo:  # the remainder could not form a sequence: close with what is left
            x = left if left <= hi else x
            if left - x != 0 and left - x < lo:
                x = left - lo
        lens.append(x)
        left -= x
    assert sum(lens) == total and all(1 <= v <= hi for v in lens)
    return lens


def cu_from_lengths(lens) -> torch.Tensor:
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(lens, dtype=torch.int64), 0).to(torch.int32)
    return cu


def uids_for(n_rows: int, group: int) -> np.ndarray:
    return np.array([f"g{i // group}" for i in range(n_rows)], dtype=object)


def c1_loss_only(seed=1, groups=16, samples=8, seqlen=1024):
    """Padded [B, T] GRPO + PPO inputs (config 1)."""
    g = _gen(seed)
    b = groups * samples
    lens = torch.randint(64, seqlen + 1, (b,), generator=g)
    mask = (torch.arange(seqlen)[None, :] < lens[:, None]).float()
    old = -torch.empty(b, seqlen).exponential_(1.0, generator=g)
    new = old + 0.05 * torch.randn(b, seqlen, generator=g)
    reward = torch.bernoulli(torch.full((b,), 0.5), generator=g)
    tlr = torch.zeros(b, seqlen)
    tlr[torch.arange(b), lens - 1] = reward
    return dict(old_log_probs=old, log_probs=new, sampler_log_probs=old.clone(), response_mask=mask,
                token_level_rewards=tlr, uid=uids_for(b, samples), lengths=lens)


def lmhead_inputs(n_tokens, hidden, vocab, seed, label_dtype=torch.int32):
    """hidden ~ N(0,1), weight ~ N(0,0.02) in bf16, uniform labels (configs 2, 3, 5)."""
    g = _gen(seed)
    h = torch.randn(n_tokens, hidden, generator=g).bfloat16()
    w = (torch.randn(vocab, hidden, generator=g) * 0.02).bfloat16()
    labels = torch.randint(0, vocab, (n_tokens,), generator=g).to(label_dtype)
    return h, w, labels


def packed_rl_inputs(n_tokens, seed, group=8, reward_p=0.5, lengths=None):
    """Packed per-token RL inputs over ragged sequences (configs 3-5): cu_seqlens, response
    mask (all but each sequence's first token), per-sequence Bernoulli rewards on the last token."""
    g = _gen(seed)
    lens = lengths if lengths is not None else ragged_lengths(n_tokens, g)
    cu = cu_from_lengths(lens)
    s = len(lens)
    mask = torch.ones(n_tokens)
    mask[cu[:-1].long()] = 0.0
    reward = torch.bernoulli(torch.full((s,), reward_p), generator=g)
    tlr = torch.zeros(n_tokens)
    tlr[cu[1:].long() - 1] = reward
    return dict(cu_seqlens=cu, lengths=lens, response_mask=mask, token_level_rewards=tlr, uid=uids_for(s, group),
                rewards=reward)


def c4_correction(seed=4, n_tokens=65536):
    """Sampler-trainer correction + GSPO inputs (config 4)."""
    g = _gen(seed)
    d = packed_rl_inputs(n_tokens, seed + 1000)
    old = -torch.empty(n_tokens).exponential_(1.0, generator=g)
    samp = old + 0.01 * torch.randn(n_tokens, generator=g)
    outlier = torch.bernoulli(torch.full((n_tokens,), 0.001), generator=g).bool()
    samp = torch.where(outlier, samp + 2.0 * torch.randn(n_tokens, generator=g), samp)
    new = old + 0.05 * torch.randn(n_tokens, generator=g)
    d.update(old_log_probs=old, sampler_log_probs=samp, log_probs=new)
    return d


def uniform_lengths(n_seqs, lo, hi, g) -> list[int]:
    return torch.randint(lo, hi + 1, (n_seqs,), generator=g).tolist()
