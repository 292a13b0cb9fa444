#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle.

    python tests/golden/make_fixtures.py

Every array is produced by this repository's own oracle (``oracle/``) on seeded inputs; no
reference code is imported or run.  The fixtures freeze inputs AND expected outputs, so that
(1) a later change of the oracle that moves a result is caught on the CPU, and (2) the HIP path
is checked on the GPU against numbers that do not depend on the oracle being importable in the
same way there.  Files are ``.npz`` (plain arrays, loaded with ``allow_pickle=False``); bf16
tensors are stored as their 16-bit patterns (``int16``).

  lmhead_n64_h128_v1000.npz   fused LM head: hidden/weight bf16, labels, temperature 0.7;
                              logprob, entropy, dHidden, dWeight (fp32) for given dlogp/dentropy
  ppo_regions.npz             one token per PPO clip region (both advantage signs, below /
                              inside / above the clip interval, dual clip, the clamp at +-20):
                              per-token loss and gradient
  gspo_ragged.npz             GSPO on 4 ragged sequences (padded layout + cu_seqlens): loss,
                              gradient, metrics
  sampler_boundaries.npz      log-ratios within 20 ulps of +-ln 2 and ln 1e-4: rejection mask,
                              veto mask, truncated IS weights
  grpo_groups.npz             GRPO advantages for group sizes 1/2/3/8 incl. an all-equal group
  gae_returns.npz             GAE, chunked GAE, REINFORCE++ and ReMax on 6 rows of 300 tokens with
                              observation gaps in the response: advantages and returns
  value_kl_cov.npz            clipped value loss and KL-Cov loss on 8 x 257 tokens: loss, gradient,
                              metrics, the tokens KL-Cov picks
"""

from __future__ import annotations

import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import advantage as OA  # noqa: E402
from oracle import lmhead as OM  # noqa: E402
from oracle import loss as OL  # noqa: E402
from oracle import returns as OR  # noqa: E402
from oracle import sampler as OS  # noqa: E402


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy()


def save(name, **arrays):
    path = os.path.join(HERE, name)
    np.savez_compressed(path, **{k: (v.numpy() if isinstance(v, torch.Tensor) else np.asarray(v))
                                 for k, v in arrays.items()})
    print(f"{name}: {os.path.getsize(path) / 1024:.1f} KiB")


def lmhead():
    g = torch.Generator().manual_seed(1234)
    n, h, v, temp = 64, 128, 1000, 0.7
    hid = torch.randn(n, h, generator=g).bfloat16()
    w = (torch.randn(v, h, generator=g) * 0.05).bfloat16()
    lab = torch.randint(0, v, (n,), generator=g).to(torch.int32)
    dlp = torch.randn(n, generator=g)
    dent = 0.1 * torch.randn(n, generator=g)
    lp, ent = OM.forward(hid, w, lab, temp)
    dh, dw = OM.backward(dlp, dent, hid, w, lab, temp)
    save("lmhead_n64_h128_v1000.npz", hidden_bf16=bf16_bits(hid), weight_bf16=bf16_bits(w), labels=lab,
         temperature=np.float32(temp), dlogprobs=dlp, dentropy=dent, logprobs=lp, entropy=ent,
         dhidden=dh.float(), dweight=dw.float())


# (log_probs - old_log_probs, advantage): every branch of the dual-clip PPO objective with
# clip_low 0.2, clip_high 0.28, c 3.0
PPO_REGIONS = [
    (-0.5, 1.0), (-0.1, 1.0), (0.0, 1.0), (0.1, 2.0), (0.3, 1.5), (1.5, 0.5),       # A > 0
    (-0.5, -1.0), (-0.1, -2.0), (0.0, -1.0), (0.2, -1.0), (0.3, -0.5), (1.0, -1.0),  # A < 0
    (1.2, -1.0), (2.0, -3.0),                                                        # A < 0, ratio > c
    (25.0, 1.0), (-25.0, 1.0), (25.0, -1.0), (-25.0, -1.0),                          # clamp at +-20
    (0.4, 0.0),                                                                      # A = 0
]


def ppo_regions():
    d = torch.tensor([[x for x, _ in PPO_REGIONS]])
    adv = torch.tensor([[a for _, a in PPO_REGIONS]])
    old = torch.full_like(d, -1.0)
    lp = (old + d).requires_grad_(True)
    mask = torch.ones_like(d)
    # token_reduce=sum, batch_reduce=token-mean -> loss = mean over tokens; per-token loss = grad wrt a unit weight
    loss, m = OL.ppo_loss(lp, old, adv, mask, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0)
    loss.backward()
    save("ppo_regions.npz", log_probs=lp.detach(), old_log_probs=old, advantages=adv, response_mask=mask,
         loss=loss.detach(), grad=lp.grad, pg_clipfrac=np.float64(m["pg_clipfrac"]), ppo_kl=np.float64(m["ppo_kl"]),
         pg_clipfrac_lower=np.float64(m["pg_clipfrac_lower"]))


def gspo_ragged():
    g = torch.Generator().manual_seed(77)
    lens = [5, 1, 37, 12]
    b, t = len(lens), max(lens)
    mask = (torch.arange(t)[None] < torch.tensor(lens)[:, None]).float()
    mask[2, 0] = 0.0  # a masked token inside a sequence
    old = -torch.empty(b, t).exponential_(1.0, generator=g)
    new = old + 2e-3 * torch.randn(b, t, generator=g)  # sequence ratios straddle the 3e-4 / 4e-4 clip
    adv = torch.tensor([1.0, -1.0, 0.7, -0.4])[:, None] * mask
    isw = (1.0 + 0.1 * torch.randn(b, t, generator=g)).clamp(max=2.0) * mask
    lp = new.clone().requires_grad_(True)
    loss, m = OL.gspo_loss(lp, old, adv, mask, clip_ratio_low=3e-4, clip_ratio_high=4e-4, sampler_is_weights=isw,
                           token_reduce="mean", batch_reduce="step-mean")
    loss.backward()
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    save("gspo_ragged.npz", lengths=np.asarray(lens, np.int32), cu_seqlens=cu, log_probs=new, old_log_probs=old,
         advantages=adv, response_mask=mask, sampler_is_weights=isw, loss=loss.detach(), grad=lp.grad,
         pg_clipfrac=np.float64(m["pg_clipfrac"]), ppo_kl=np.float64(m["ppo_kl"]))


def sampler_boundaries():
    vals = []
    for c in (math.log(2.0), -math.log(2.0), math.log(1e-4)):
        x = torch.tensor(c, dtype=torch.float32)
        up, dn = x.clone(), x.clone()
        vals.append(x.clone())
        for _ in range(20):
            up = torch.nextafter(up, torch.tensor(math.inf))
            dn = torch.nextafter(dn, torch.tensor(-math.inf))
            vals += [up.clone(), dn.clone()]
    lr = torch.stack(vals)  # 123 values
    lr = torch.cat([lr, torch.tensor([0.0, 10.0, -5.0, 70.0, -70.0])]).view(8, 16)
    old, samp = lr.clone(), torch.zeros_like(lr)
    mask = torch.ones_like(lr)
    mask[5, 3] = 0.0
    w, rs_mask, _ = OS.correction(old, samp, mask, sampler_is="token", sampler_is_threshold=2.0, sampler_rs="token",
                                  sampler_rs_threshold=2.0)
    _, veto_mask, mv = OS.correction(old, samp, mask, sampler_token_veto_threshold=1e-4)
    # one token per row: the row-level veto flag at the boundary
    col = lr.reshape(-1, 1)
    _, veto_rows, _ = OS.correction(col, torch.zeros_like(col), torch.ones_like(col),
                                    sampler_token_veto_threshold=1e-4)
    save("sampler_boundaries.npz", old_log_probs=old, sampler_log_probs=samp, response_mask=mask, is_weights=w,
         rs_mask=rs_mask, veto_mask=veto_mask, veto_rows=veto_rows,
         veto_fraction=np.float64(mv["sampler_is_veto_fraction"]))


def grpo_groups():
    g = torch.Generator().manual_seed(5)
    sizes = [1, 2, 3, 8, 8]
    gidx = torch.cat([torch.full((s,), i) for i, s in enumerate(sizes)])
    b, t = gidx.numel(), 12
    lens = torch.randint(1, t + 1, (b,), generator=g)
    mask = (torch.arange(t)[None] < lens[:, None]).float()
    score = torch.bernoulli(torch.full((b,), 0.5), generator=g)
    score[-8:] = 1.0  # an all-equal group
    score[1:3] = torch.tensor([0.25, 1.75])
    tlr = torch.zeros(b, t)
    tlr[torch.arange(b), lens - 1] = score
    perm = torch.randperm(b, generator=g)  # groups interleaved, as uids are in a batch
    tlr, mask, gidx = tlr[perm], mask[perm], gidx[perm]
    out = {}
    for norm in (True, False):
        out[f"adv_norm{int(norm)}"] = OA.grpo_advantage(tlr, mask, gidx, eps=1e-6, norm_adv_by_std=norm)
    mean, std, cnt = OA.group_mean_std(tlr.sum(-1), gidx, 1e-6)
    save("grpo_groups.npz", token_level_rewards=tlr, response_mask=mask, gidx=gidx.to(torch.int64), mean=mean,
         std=std, count=cnt, **out)


def gae_returns():
    g = torch.Generator().manual_seed(6)
    b, t = 6, 300
    rewards = torch.randn(b, t, generator=g) * (torch.rand(b, t, generator=g) > 0.8)
    values = torch.randn(b, t, generator=g)
    lens = torch.tensor([300, 1, 64, 257, 150, 299])
    mask = (torch.arange(t)[None] < lens[:, None]).float() * (torch.rand(b, t, generator=g) > 0.2)
    mask[1, 0] = 1
    base = torch.randn(b, generator=g)
    gae_adv, gae_ret = OR.gae_advantage(rewards, values, mask, 0.99, 0.95)
    raw_adv, _ = OR.gae_raw(rewards, values, mask, 0.99, 0.95)
    ch_adv, ch_ret = OR.chunked_gae_advantage(rewards, values, mask, 0.99, 0.95)
    rpp_adv, rpp_ret = OR.reinforce_plus_plus_advantage(rewards, mask, 0.97)
    rm_adv, rm_ret = OR.remax_advantage(rewards, mask, base)
    save("gae_returns.npz", rewards=rewards, values=values, response_mask=mask, reward_baselines=base,
         gae_raw=raw_adv, gae_adv=gae_adv, gae_ret=gae_ret, chunked_adv=ch_adv, chunked_ret=ch_ret, rpp_adv=rpp_adv,
         rpp_ret=rpp_ret, remax_adv=rm_adv, remax_ret=rm_ret)


def value_kl_cov():
    g = torch.Generator().manual_seed(8)
    b, t = 8, 257
    values = torch.randn(b, t, generator=g)
    vpreds = values + 0.4 * torch.randn(b, t, generator=g)
    returns = values + torch.randn(b, t, generator=g)
    mask = (torch.rand(b, t, generator=g) > 0.3).float()
    mask[5] = 0
    vp = vpreds.clone().requires_grad_(True)
    vloss, vm = OR.value_loss(vp, values, returns, mask, cliprange_value=0.3)
    vloss.backward()
    old = -torch.empty(b, t).exponential_(1.0, generator=g)
    lp = (old + 0.1 * torch.randn(b, t, generator=g)).requires_grad_(True)
    adv = torch.randn(b, 1, generator=g).expand(b, t).contiguous() + 0.1 * torch.randn(b, t, generator=g)
    kloss, km, picked = OL.kl_cov_loss(lp, old, adv, mask, kl_cov_ratio=0.01, ppo_kl_coef=1.0)
    kloss.backward()
    save("value_kl_cov.npz", values=values, vpreds=vpreds, returns=returns, response_mask=mask,
         value_loss=vloss.detach(), value_grad=vp.grad, vf_clipfrac=np.float32(vm["vf_clipfrac"]),
         vpred_mean=np.float32(vm["vpred_mean"]), old_log_probs=old, log_probs=lp.detach(), advantages=adv,
         kl_cov_loss=kloss.detach(), kl_cov_grad=lp.grad, kl_cov_ppo_kl=np.float32(km["ppo_kl"]),
         kl_cov_picked=torch.sort(picked).values)


if __name__ == "__main__":
    torch.set_num_threads(1)  # summation order of the CPU reductions independent of the machine
    lmhead()
    ppo_regions()
    gspo_ragged()
    sampler_boundaries()
    grpo_groups()
    gae_returns()
    value_kl_cov()
