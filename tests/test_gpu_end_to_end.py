"""GPU parity of the whole chain at reduced size: head forward -> shift -> GRPO advantage ->
PPO loss -> loss backward -> head backward, against the same chain in the CPU oracle; plus
size-independent properties at the full Qwen3-8B shape."""

import numpy as np
import pytest
import torch

from axon_amd import workloads as W
from axon_amd.protocol import DataProto
from axon_amd.trainer.algos.advantages import compute_advantage
from axon_amd.trainer.algos.loss import compute_loss_fn
from axon_amd.utils.fsdp.forward_utils import shift_packed
from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
from oracle import advantage as OA
from oracle import lmhead as OM
from oracle import loss as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def hip_chain(hid, w, labels, rl, old_lp, temp=1.0):
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    cu = rl["cu_seqlens"].to(DEV)
    lp_head, ent = linear_cross_entropy(hd, wd, labels.to(DEV), temp, "none")
    lp_tok = shift_packed(lp_head, cu)
    data = DataProto.from_dict(
        tensors={"token_level_rewards": rl["token_level_rewards"].to(DEV), "response_mask": rl["response_mask"].to(DEV)},
        meta_info={"cu_seqlens": cu})
    data.non_tensor_batch["uid"] = rl["uid"]  # one uid per sequence; the packed tensors are per token
    adv = compute_advantage(data, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}).batch["advantages"]
    loss_data = DataProto.from_dict(
        tensors={"log_probs": lp_tok, "old_log_probs": old_lp.to(DEV), "advantages": adv,
                 "response_mask": rl["response_mask"].to(DEV)}, meta_info={"cu_seqlens": cu})
    loss, metrics = compute_loss_fn(loss_data, "ppo", {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28})
    loss.backward()
    return loss, lp_head, ent, hd.grad, wd.grad, adv


def oracle_chain(hid, w, labels, rl, old_lp, temp=1.0):
    lp_head, ent = OM.forward(hid, w, labels, temp)
    cu = rl["cu_seqlens"].long()
    lens = (cu[1:] - cu[:-1]).tolist()
    s, tmax = len(lens), max(lens)
    lp_tok = torch.zeros_like(lp_head)
    lp_tok[1:] = lp_head[:-1]
    lp_tok[cu[:-1]] = 0.0
    pad = lambda x: torch.stack([torch.nn.functional.pad(x[a:b], (0, tmax - (b - a))) for a, b in zip(cu[:-1], cu[1:])])
    gidx = torch.tensor(np.unique(rl["uid"], return_inverse=True)[1])
    mask = pad(rl["response_mask"])
    adv = OA.grpo_advantage(pad(rl["token_level_rewards"]), mask, gidx, 1e-6)
    lp_pad = pad(lp_tok).requires_grad_(True)
    loss, _ = OL.ppo_loss(lp_pad, pad(old_lp), adv, mask, clip_ratio_low=0.2, clip_ratio_high=0.28)
    loss.backward()
    g_tok = torch.cat([lp_pad.grad[b, :l] for b, l in enumerate(lens)])
    g_head = torch.zeros_like(g_tok)
    g_head[:-1] = g_tok[1:]          # adjoint of the shift
    g_head[cu[1:] - 1] = 0.0          # a sequence's last head output feeds no token
    dh, dw = OM.backward(g_head, None, hid, w, labels, temp)
    return loss, lp_head, ent, dh, dw, torch.cat([adv[b, :l] for b, l in enumerate(lens)])


def test_chain_small_vs_oracle():
    n, h, v = 1500, 128, 2000
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=21)
    w = (w.float() * 6).bfloat16()
    rl = W.packed_rl_inputs(n, seed=22, lengths=[400, 33, 500, 64, 300, 203])
    rl["uid"] = W.uids_for(6, 3)
    g = torch.Generator().manual_seed(23)
    old = OM.forward(hid, w, lab)[0]
    old_tok = torch.zeros_like(old)
    old_tok[1:] = old[:-1]
    old_tok = old_tok - 0.05 * torch.randn(n, generator=g)
    got = hip_chain(hid, w, lab, rl, old_tok)
    ref = oracle_chain(hid, w, lab, rl, old_tok)
    assert got[0].item() == pytest.approx(ref[0].item(), rel=1e-4, abs=1e-8)
    assert (got[1].cpu() - ref[1]).abs().max() < 1e-3 and (got[2].cpu() - ref[2]).abs().max() < 1e-3
    assert torch.allclose(got[5].cpu(), ref[5], rtol=1e-5, atol=1e-6)
    assert rel_l2(got[3], ref[3]) < 2e-2 and rel_l2(got[4], ref[4]) < 2e-2


def test_qwen3_8b_shape_properties():
    """Config 3 at full size (32768 x 4096 x 151936): size-independent checks.

    - log-probs are <= 0, entropy in [0, ln V], and a token subset matches the oracle;
    - sum_v dlogit = 0 per token => d_hidden . 1-direction test: with g = const the column sums of
      d_weight equal  sum_t g_t (onehot - p)^T h  whose sum over v is 0 => sum_v d_weight[v] = 0;
    - linearity: backward(2g) = 2 backward(g)."""
    import math
    n, h, v = 32768, 4096, 151936
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=3)
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    from axon_amd import _ops
    lp, ent, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    assert torch.isfinite(lp).all() and (lp <= 1e-4).all()
    assert (ent >= -1e-4).all() and (ent <= math.log(v) + 1e-3).all()
    idx = torch.arange(0, n, 509)
    ref_lp, ref_ent = OM.forward(hid[idx], w, lab[idx])
    assert (lp.cpu()[idx] - ref_lp).abs().max() < 1e-3 and (ent.cpu()[idx] - ref_ent).abs().max() < 1e-3
    g = torch.randn(n, device=DEV) / n
    dh, dw = _ops.lmhead_backward(g, None, hd, wd, ld, lse, eb, 1.0)
    assert torch.isfinite(dh.float()).all() and torch.isfinite(dw.float()).all()
    col = dw.float().sum(0)
    scale = dw.float().abs().sum(0)
    assert (col.abs() / scale.clamp_min(1e-20)).max().item() < 2e-2
    ref_dh, _ = OM.backward(g.cpu()[idx], None, hid[idx], w, lab[idx])
    assert rel_l2(dh[idx.to(DEV)], ref_dh) < 2e-2
    dh2, dw2 = _ops.lmhead_backward(2 * g, None, hd, wd, ld, lse, eb, 1.0)
    assert rel_l2(dh2, 2 * dh.float()) < 1e-2 and rel_l2(dw2, 2 * dw.float()) < 1e-2


from head_reference import _fp32_torch_head_reference, _spread_rows  # noqa: E402


def _stash_backward(hd, wd, ld, g_lp, g_en, plain_forward):
    """Forward with a stash (its outputs must be those of the plain forward, bit for bit) and the backward
    that decodes it."""
    from axon_amd import _ops
    saved, _ops.LMHEAD_STASH = _ops.LMHEAD_STASH, True
    try:
        *out, stash = _ops.lmhead_forward(hd, wd, ld, 1.0, stash=True)
    finally:
        _ops.LMHEAD_STASH = saved
    assert stash is not None and all(torch.equal(a, b) for a, b in zip(out, plain_forward))
    return _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, out[2], out[3], 1.0, stash=stash)


def test_qwen3_8b_dweight_rows_vs_fp32_torch():
    """Config 3 at full size: d_weight on ~120 vocabulary rows spread over all five vocabulary chunks of the
    backward (rows >= 131072 and the last tile included), log-prob and entropy of every token, against an
    fp32 torch reference computed on the GPU.  Tolerances: 1e-3 absolute, 2e-2 relative L2."""
    n, h, v = 32768, 4096, 151936
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=3)
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    from axon_amd import _ops
    lp, ent, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    gen = torch.Generator().manual_seed(33)
    g_lp = (torch.randn(n, generator=gen) / n).to(DEV)
    g_en = (0.3 * torch.randn(n, generator=gen) / n).to(DEV)
    dh, dw = _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0)
    rows = _spread_rows(v)
    assert (rows >= 131072).sum() >= 10 and len(rows) >= 64
    ref_lp, ref_ent, ref_dw = _fp32_torch_head_reference(hd, wd, ld, g_lp, g_en, rows)
    assert (lp - ref_lp).abs().max().item() < 1e-3
    assert (ent - ref_ent).abs().max().item() < 1e-3
    got = dw[rows.to(DEV)].double()
    assert rel_l2(got, ref_dw) < 2e-2
    per_row = (got - ref_dw).norm(dim=1) / ref_dw.norm(dim=1).clamp_min(1e-30)
    assert per_row.max().item() < 5e-2, (per_row.argmax().item(), per_row.max().item())  # no single row is off
    # the same from the forward's stash (10 GB at this shape) instead of the recomputed logits
    dh_s, dw_s = _stash_backward(hd, wd, ld, g_lp, g_en, (lp, ent, lse, eb))
    got_s = dw_s[rows.to(DEV)].double()
    assert rel_l2(got_s, ref_dw) < 2e-2
    per_row = (got_s - ref_dw).norm(dim=1) / ref_dw.norm(dim=1).clamp_min(1e-30)
    assert per_row.max().item() < 5e-2, (per_row.argmax().item(), per_row.max().item())
    assert rel_l2(dh_s, dh.float()) < 5e-3 and rel_l2(dw_s, dw.float()) < 5e-3


def test_gpt_oss_head_full_shape():
    """Config 5's head at its full shape (16384 x 2880 x 201088; hidden size not a multiple of 128): forward
    on every token and d_weight on spread rows against the fp32 torch reference on the GPU, a token subset of
    forward and d_hidden against the CPU oracle, and linearity of the backward."""
    import math
    n, h, v = 16384, 2880, 201088
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=5)
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    from axon_amd import _ops
    lp, ent, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    assert torch.isfinite(lp).all() and (lp <= 1e-4).all()
    assert (ent >= -1e-4).all() and (ent <= math.log(v) + 1e-3).all()
    idx = torch.arange(0, n, 497)
    o_lp, o_ent = OM.forward(hid[idx], w, lab[idx])
    assert (lp.cpu()[idx] - o_lp).abs().max() < 1e-3 and (ent.cpu()[idx] - o_ent).abs().max() < 1e-3
    gen = torch.Generator().manual_seed(55)
    g_lp = (torch.randn(n, generator=gen) / n).to(DEV)
    dh, dw = _ops.lmhead_backward(g_lp, None, hd, wd, ld, lse, eb, 1.0)
    assert torch.isfinite(dh.float()).all() and torch.isfinite(dw.float()).all()
    rows = _spread_rows(v)
    ref_lp, ref_ent, ref_dw = _fp32_torch_head_reference(hd, wd, ld, g_lp, None, rows)
    assert (lp - ref_lp).abs().max().item() < 1e-3 and (ent - ref_ent).abs().max().item() < 1e-3
    assert rel_l2(dw[rows.to(DEV)].double(), ref_dw) < 2e-2
    o_dh, _ = OM.backward(g_lp.cpu()[idx], None, hid[idx], w, lab[idx])
    assert rel_l2(dh[idx.to(DEV)], o_dh) < 2e-2
    dh2, dw2 = _ops.lmhead_backward(2 * g_lp, None, hd, wd, ld, lse, eb, 1.0)
    assert rel_l2(dh2, 2 * dh.float()) < 1e-2 and rel_l2(dw2, 2 * dw.float()) < 1e-2
    del dh2, dw2
    dh_s, dw_s = _stash_backward(hd, wd, ld, g_lp, None, (lp, ent, lse, eb))
    assert rel_l2(dw_s[rows.to(DEV)].double(), ref_dw) < 2e-2 and rel_l2(dh_s[idx.to(DEV)], o_dh) < 2e-2
    assert rel_l2(dh_s, dh.float()) < 5e-3 and rel_l2(dw_s, dw.float()) < 5e-3


def test_micro_batched_dapo_chain_vs_whole_batch_oracle():
    """The GPT-OSS-style configuration at reduced size (hidden 2880 kept: K not a multiple of 128): advantages and
    dynamic sampling over all sequences, then head + DAPO loss per micro-batch of whole sequences with the
    mini-batch-global ``valid_token_count``, dHidden per micro-batch and dWeight accumulated over them.  The
    oracle evaluates the kept sequences as ONE batch: the micro-batch losses must add up to its loss and the
    accumulated gradients must be its gradients."""
    from axon_amd.utils.rl.utils import filter_zero_advantage_samples
    h, v, groups, samples, tmax = 2880, 3000, 4, 3, 80
    g = torch.Generator().manual_seed(61)
    n_seq = groups * samples
    lens = torch.randint(20, tmax + 1, (n_seq,), generator=g).tolist()
    uid = W.uids_for(n_seq, samples)
    score = (torch.rand(n_seq, generator=g) < 0.3).float()
    score[0:3] = 1.0                      # group 0: all equal -> zero advantage -> dropped
    score[3:6] = T_([1.0, 0.0, 0.0])      # the others mixed
    score[6:9] = T_([0.0, 1.0, 1.0])
    score[9:12] = T_([1.0, 0.0, 1.0])
    rewards, mask = torch.zeros(n_seq, tmax), torch.zeros(n_seq, tmax)
    for i, l in enumerate(lens):
        mask[i, 1:l] = 1                   # position 0 is the prompt token
        rewards[i, l - 1] = score[i]
    # 1. advantages over every sequence, then dynamic sampling (row indices bit-exact against the oracle)
    data = DataProto.from_dict(tensors={"token_level_rewards": rewards.to(DEV), "response_mask": mask.to(DEV),
                                        "row": torch.arange(n_seq).to(DEV)})
    data.non_tensor_batch["uid"] = uid
    data = compute_advantage(data, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}})
    gidx = torch.tensor(np.unique(uid, return_inverse=True)[1])
    ref_adv = OA.grpo_advantage(rewards, mask, gidx, 1e-6)
    kept = filter_zero_advantage_samples(data).batch["row"].tolist()
    assert kept == OA.zero_advantage_keep_rows(ref_adv) == list(range(3, 12))
    # 2. the kept sequences, packed, in micro-batches of three sequences
    lens_k = [lens[i] for i in kept]
    n = sum(lens_k)
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=62)
    w = (w.float() * 6).bfloat16()
    cu = W.cu_from_lengths(lens_k).long()
    pack = lambda x: torch.cat([x[i, :lens[i]] for i in kept])  # noqa: E731
    adv_p, mask_p = pack(data.batch["advantages"].cpu()), pack(mask)
    labels = torch.roll(ids, -1)
    old = OM.forward(hid, w, labels)[0]
    old_tok = torch.zeros_like(old)
    old_tok[1:] = old[:-1]
    old_tok = old_tok - 0.05 * torch.randn(n, generator=g)
    valid = int(mask_p.sum())
    wd = w.to(DEV).requires_grad_(True)
    total, dh_parts = 0.0, []
    for first in range(0, len(kept), 3):
        a, b = int(cu[first]), int(cu[min(first + 3, len(kept))])
        cu_mb = (cu[first:first + 4] - a).int().to(DEV)
        hd = hid[a:b].to(DEV).requires_grad_(True)
        from axon_amd.utils.fsdp.forward_utils import packed_logprobs
        lp, _ = packed_logprobs(hd, wd, ids[a:b].to(DEV), cu_mb)
        mb = DataProto.from_dict(
            tensors={"log_probs": lp, "old_log_probs": old_tok[a:b].to(DEV), "advantages": adv_p[a:b].to(DEV),
                     "response_mask": mask_p[a:b].to(DEV),
                     "valid_token_count": torch.full((b - a,), valid, dtype=torch.int64, device=DEV)},
            meta_info={"cu_seqlens": cu_mb})
        loss, _ = compute_loss_fn(mb, "ppo", {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28})
        loss.backward()
        total += loss.item()
        dh_parts.append(hd.grad)
    # 3. the oracle on the whole kept batch
    rl = {"cu_seqlens": cu.int(), "token_level_rewards": pack(rewards), "response_mask": mask_p,
          "uid": uid[kept]}
    # every kept group is complete, so the group statistics of the kept rows equal those of the full batch
    ref = oracle_chain(hid, w, labels, rl, old_tok)
    assert total == pytest.approx(ref[0].item(), rel=1e-4, abs=1e-8)
    assert rel_l2(torch.cat(dh_parts), ref[3]) < 2e-2
    assert rel_l2(wd.grad, ref[4]) < 2e-2


def T_(x):
    return torch.tensor(x)
