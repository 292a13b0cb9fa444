"""Oracle: LM-head log-prob and entropy, forward and backward, on the CPU.

Follows axon/utils/torch/fused_linear.py:26-89 (the torch implementation the
north star names) and the formulas of axon/utils/kernel/kernels.py:250-265,
356-370, 827-834.  The arithmetic is evaluated on fp32 upcasts of the bf16
inputs (fp32 accumulate), which is what the Triton kernel computes and what a
1e-3 tolerance can be checked against; ``forward_bf16_torch_path`` keeps the
reference torch backend's own rounding (bf16 logits) and is used only as the
timed CPU baseline.
"""

from __future__ import annotations

import torch


def _softcap(logits, softcap):
    """fused_linear.py:19-23: tanh(logits / cap) * cap, applied to the raw logits before the temperature."""
    return logits if softcap is None else torch.tanh(logits / softcap) * softcap


def forward(hidden, weight, labels, temperature: float = 1.0, chunk: int = 512, softcap: float | None = None):
    """logits = softcap(h @ W^T)/T in fp32; returns (logprob[label], entropy) as fp32 [N].

    fused_linear.py:33-44: log_softmax + gather, entropy = logsumexp - sum softmax*logits.
    Token-chunked like the reference (:125-136) to bound memory.
    """
    h = hidden.reshape(-1, hidden.shape[-1]).float()
    w = weight.float()
    ids = labels.reshape(-1).long()
    n = h.shape[0]
    logp = torch.empty(n, dtype=torch.float32)
    ent = torch.empty(n, dtype=torch.float32)
    for s in range(0, n, chunk):
        e = min(s + chunk, n)
        logits = _softcap(h[s:e] @ w.t(), softcap) / temperature
        lse = torch.logsumexp(logits, dim=-1)
        probs = torch.softmax(logits, dim=-1)
        logp[s:e] = logits.gather(-1, ids[s:e, None]).squeeze(-1) - lse
        ent[s:e] = lse - (probs * logits).sum(-1)
    return logp, ent


def backward(dlogp, dent, hidden, weight, labels, temperature: float = 1.0, chunk: int = 512,
             round_dlogits_bf16: bool = False, softcap: float | None = None):
    """Closed-form gradients (fused_linear.py:49-89):

        dlogits = [ g*(onehot - p) - gH * p * (log p + H) ] / T   (* (1 - tanh^2(raw / cap)) with a softcap, :80-83)
        d_hidden = dlogits @ W,   d_weight = dlogits^T @ hidden      (fp32)

    ``round_dlogits_bf16`` reproduces the rounding of dlogits to the input dtype
    that both reference backends apply before the two matmuls (fused_linear.py:77,
    kernels.py:1527).
    """
    h = hidden.reshape(-1, hidden.shape[-1]).float()
    w = weight.float()
    ids = labels.reshape(-1).long()
    n = h.shape[0]
    d_h = torch.zeros_like(h)
    d_w = torch.zeros_like(w)
    for s in range(0, n, chunk):
        e = min(s + chunk, n)
        raw = h[s:e] @ w.t()
        logits = _softcap(raw, softcap) / temperature
        logp_all = torch.log_softmax(logits, dim=-1)
        p = logp_all.exp()
        dl = torch.zeros_like(logits)
        if dlogp is not None:
            onehot = torch.zeros_like(logits).scatter_(-1, ids[s:e, None], 1.0)
            dl = dl + dlogp[s:e].float()[:, None] * (onehot - p)
        if dent is not None:
            entropy = -(p * logp_all).sum(-1, keepdim=True)
            dl = dl - dent[s:e].float()[:, None] * p * (logp_all + entropy)
        dl = dl / temperature
        if softcap is not None:
            dl = dl * (1.0 - torch.tanh(raw / softcap) ** 2)
        if round_dlogits_bf16:
            dl = dl.bfloat16().float()
        d_h[s:e] = dl @ w
        d_w += dl.t() @ h[s:e]
    return d_h, d_w


def forward_bf16_torch_path(hidden, weight, labels, temperature: float = 1.0, chunk: int = 512):
    """The reference torch backend as it runs under bf16 (fused_linear.py:26-46, 120-136):
    the matmul result is bf16, softmax in fp32, outputs rounded back to bf16.  CPU baseline only."""
    n = hidden.shape[0]
    logp = hidden.new_zeros(n)
    ent = hidden.new_zeros(n)
    ids = labels.long()
    for s in range(0, n, chunk):
        e = min(s + chunk, n)
        logits = (hidden[s:e] @ weight.t()) / temperature
        lf = logits.float()
        probs = lf.softmax(-1)
        logp[s:e] = lf.log_softmax(-1).gather(-1, ids[s:e, None]).squeeze(-1).to(logits.dtype)
        ent[s:e] = (torch.logsumexp(lf, -1) - (probs * lf).sum(-1)).to(logits.dtype)
    return logp, ent


def backward_bf16_torch_path(dlogp, hidden, weight, labels, temperature: float = 1.0, chunk: int = 512):
    """Reference torch backend backward in bf16 (fused_linear.py:49-89, 180-202), dentropy None."""
    n = hidden.shape[0]
    ids = labels.long()
    d_h = torch.zeros_like(hidden)
    d_w = torch.zeros_like(weight)
    for s in range(0, n, chunk):
        e = min(s + chunk, n)
        logits = ((hidden[s:e] @ weight.t()) / temperature)
        dt = logits.dtype
        p = logits.float().softmax(-1)
        onehot = torch.zeros_like(p).scatter_(-1, ids[s:e, None], 1.0)
        dl = (dlogp[s:e].float()[:, None] * (onehot - p)).to(dt) / temperature
        d_h[s:e] += dl @ weight
        d_w += dl.t() @ hidden[s:e]
    return d_h, d_w


def logprobs_from_logits(logits, labels):
    """axon/utils/torch/ops.py:39-102 in fp32: ``log_softmax(logits)[labels]`` (the definition the reference's own
    test uses, tests/utils/torch/test_ops.py:36-42)."""
    lp = torch.log_softmax(logits.float(), dim=-1)
    return lp.gather(-1, labels.long().unsqueeze(-1)).squeeze(-1)


def entropy_from_logits(logits):
    """axon/utils/torch/ops.py:105-120 in fp32: ``logsumexp - sum softmax * logits``."""
    z = logits.float()
    return torch.logsumexp(z, dim=-1) - (torch.softmax(z, dim=-1) * z).sum(-1)
