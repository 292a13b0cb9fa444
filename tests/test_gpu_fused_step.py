"""GPU parity of the step as ONE autograd node that works block of tokens by block (head forward with a
stash -> loss on the block -> head backward from the stash): against the CPU oracle's chain at small sizes
(PPO, DAPO with entropy bonus and KL penalty, GSPO; block borders on and off sequence ends; one block and many),
against the unfused GPU path, and at the full Qwen3-8B shape against an fp32 torch head + the oracle's loss.

Tolerances: loss 1e-4 relative, bf16 gradients 2e-2 relative L2 against the oracle, 5e-3 against the unfused
GPU path (the stash rounds softmax numerators to fp16 where the recompute keeps fp32), metrics 1e-4 relative."""

import numpy as np
import pytest
import torch

from axon_amd import workloads as W
from axon_amd.protocol import DataProto
from axon_amd.trainer.algos.advantages import compute_advantage
from oracle import advantage as OA
from oracle import lmhead as OM
from oracle import loss as OL

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _inputs(n, h, v, lens, seed, group=3):
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=seed)
    w = (w.float() * 6).bfloat16()
    rl = W.packed_rl_inputs(n, seed=seed + 1, lengths=lens)
    rl["uid"] = W.uids_for(len(lens), group)
    g = torch.Generator().manual_seed(seed + 2)
    labels = torch.roll(ids, -1)
    lp_head, _ = OM.forward(hid, w, labels)
    old = _to_token_positions(lp_head, rl["cu_seqlens"].long()) - 0.05 * torch.randn(n, generator=g)
    ref = old + 0.1 * torch.randn(n, generator=g)
    return hid, w, ids, labels, rl, old, ref


def _to_token_positions(x, cu):
    out = torch.zeros_like(x)
    out[1:] = x[:-1]
    out[cu[:-1][cu[:-1] < x.numel()]] = 0.0
    return out


def _pad(x, cu, tmax):
    return torch.stack([torch.nn.functional.pad(x[a:b], (0, tmax - (b - a))) for a, b in zip(cu[:-1], cu[1:])])


# GRPO advantages add up to zero over a complete group, and GSPO's sequence ratios are within a few 1e-4 of one:
# its loss is then what is left of a cancelling sum, and its relative error is that of the log-probs times the
# cancellation.  The GSPO cases therefore move every advantage by a constant, which makes the loss O(1).
GSPO_ADV_SHIFT = 0.5


def oracle_step(hid, w, labels, rl, old, ref, loss_name, args, dp_replicas=1, n_micro_batches=1, adv_shift=0.0):
    """Head forward -> shift -> GRPO advantage -> actor loss (policy loss, entropy bonus, KL penalty) ->
    backward through the shift -> head backward, all on the CPU oracle."""
    cu = rl["cu_seqlens"].long()
    lens = (cu[1:] - cu[:-1]).tolist()
    tmax = max(lens)
    lp_head, ent_head = OM.forward(hid, w, labels)
    lp_tok, ent_tok = _to_token_positions(lp_head, cu), _to_token_positions(ent_head, cu)
    gidx = torch.tensor(np.unique(rl["uid"], return_inverse=True)[1])
    mask = _pad(rl["response_mask"], cu, tmax)
    adv = OA.grpo_advantage(_pad(rl["token_level_rewards"], cu, tmax), mask, gidx, 1e-6) + adv_shift * mask
    lp_pad = _pad(lp_tok, cu, tmax).requires_grad_(True)
    en_pad = _pad(ent_tok, cu, tmax).requires_grad_(True)
    fn = OL.ppo_loss if loss_name == "ppo" else OL.gspo_loss
    loss, metrics = OL.actor_loss(fn, lp_pad, en_pad, _pad(old, cu, tmax), adv, mask, loss_args=args,
                                  ref_log_prob=_pad(ref, cu, tmax), dp_replicas=dp_replicas,
                                  n_micro_batches=n_micro_batches)
    loss.backward()

    def to_head(g_pad):
        if g_pad is None:
            return None
        g_tok = torch.cat([g_pad[b, :l] for b, l in enumerate(lens)])
        g_head = torch.zeros_like(g_tok)
        g_head[:-1] = g_tok[1:]
        g_head[cu[1:] - 1] = 0.0
        return g_head

    dh, dw = OM.backward(to_head(lp_pad.grad), to_head(en_pad.grad), hid, w, labels)
    return loss.detach(), metrics, lp_tok, ent_tok, dh, dw


def fused_step(hid, w, ids, rl, old, ref, loss_name, args, block_tokens, dp_replicas=1, n_micro_batches=1,
               vocab_chunk=0, extra=None, adv_shift=0.0, dw_group=None):
    from axon_amd.models.fused_head_loss import DEFAULT_DW_GROUP, fused_head_loss
    dw_group = DEFAULT_DW_GROUP if dw_group is None else dw_group
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    cu = rl["cu_seqlens"].to(DEV)
    a_in = DataProto.from_dict(tensors={"token_level_rewards": rl["token_level_rewards"].to(DEV),
                                        "response_mask": rl["response_mask"].to(DEV)}, meta_info={"cu_seqlens": cu})
    a_in.non_tensor_batch["uid"] = rl["uid"]
    adv = compute_advantage(a_in, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}).batch["advantages"]
    adv = adv + adv_shift * rl["response_mask"].to(DEV)
    tensors = {"old_log_probs": old.to(DEV), "advantages": adv, "response_mask": rl["response_mask"].to(DEV),
               "ref_log_prob": ref.to(DEV)}
    tensors.update({k: v.to(DEV) for k, v in (extra or {}).items()})
    data = DataProto.from_dict(tensors=tensors)
    meta = {"loss_fn": loss_name, "loss_fn_args": args, "temperature": 1.0, "dp_replicas": dp_replicas,
            "n_micro_batches": n_micro_batches}
    loss, metrics = fused_head_loss(hd, wd, ids.to(DEV), cu, data, meta, block_tokens=block_tokens,
                                    vocab_chunk=vocab_chunk, dw_group=dw_group)
    loss.backward()
    return loss.detach(), metrics, data, hd.grad, wd.grad


PPO = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28}
DAPO_SIDE = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "entropy_coef": 0.01, "kl_coef": 0.05,
             "kl_type": "low_var_kl"}
GSPO = {"clip_ratio_low": 3e-4, "clip_ratio_high": 4e-4, "token_reduce": "mean", "batch_reduce": "step-mean"}
GSPO_SIDE = dict(GSPO, entropy_coef=0.01, kl_coef=0.05, kl_type="k2")
RAGGED = [400, 33, 500, 64, 300, 203]          # 1500 tokens; no sequence ends on a multiple of 256
ON_BORDERS = [256, 256, 512, 128, 128, 256]     # 1536 tokens; every sequence ends on a block border
ODD_TOTAL = [400, 33, 500, 64, 300, 205]        # 1502 tokens: a last block of 478 or 222 rows cannot be stashed


@pytest.mark.parametrize("lens", [RAGGED, ON_BORDERS, ODD_TOTAL], ids=["ragged", "on-borders", "odd-total"])
@pytest.mark.parametrize("block_tokens", [256, 512, 4096], ids=["b256", "b512", "one-block"])
@pytest.mark.parametrize("case", ["ppo", "dapo-entropy-kl", "gspo", "gspo-entropy-kl"])
def test_fused_step_vs_oracle(case, block_tokens, lens):
    name, args = {"ppo": ("ppo", PPO), "dapo-entropy-kl": ("ppo", DAPO_SIDE), "gspo": ("gspo", GSPO),
                  "gspo-entropy-kl": ("gspo", GSPO_SIDE)}[case]
    if name == "gspo" and block_tokens < max(lens):
        block_tokens = 512  # blocks hold whole sequences
    n, h, v = sum(lens), 128, 2000
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=71)
    shift = GSPO_ADV_SHIFT if name == "gspo" else 0.0
    want = oracle_step(hid, w, labels, rl, old, ref, name, args, dp_replicas=2, n_micro_batches=4, adv_shift=shift)
    got = fused_step(hid, w, ids, rl, old, ref, name, args, block_tokens, dp_replicas=2, n_micro_batches=4,
                     adv_shift=shift)
    data = got[2]
    assert data.meta_info["head_backward"] == "blocked-stash"
    expect_blocks = {256: -(-n // 256), 512: -(-n // 512), 4096: 1}[block_tokens]
    if name == "ppo":
        assert data.meta_info["n_blocks"] == expect_blocks
    else:
        assert data.meta_info["n_blocks"] >= expect_blocks
    assert got[0].item() == pytest.approx(want[0].item(), rel=1e-4, abs=1e-8)
    assert (data.batch["log_probs"].cpu() - want[2]).abs().max() < 1e-3
    assert (data.batch["entropys"].cpu() - want[3]).abs().max() < 1e-3
    assert rel_l2(got[3], want[4]) < 2e-2 and rel_l2(got[4], want[5]) < 2e-2
    keys = ["pg_loss", "entropy", "entropy_token_mean", "pg_clipfrac", "ppo_kl"]
    keys += ["kl_loss", "kl_coef"] if "kl_coef" in args else []
    for k in keys:
        assert got[1][k] == pytest.approx(want[1][k], rel=1e-4, abs=1e-6), k


@pytest.mark.parametrize("lens", [RAGGED, ODD_TOTAL], ids=["ragged", "odd-total"])
@pytest.mark.parametrize("dw_group", [1, 2, 3, 8])
@pytest.mark.parametrize("case", ["dapo-entropy-kl", "gspo-entropy-kl"])
def test_fused_step_with_grouped_weight_gradient_vs_oracle(case, dw_group, lens):
    """Hidden size 256 and a vocabulary that is a multiple of 8: the weight gradient reads the token-major
    dlogits as a K-major GEMM operand (no vocab-major copy), and `dw_group` consecutive blocks share one such
    GEMM (1: every block its own; 8: one GEMM for the step; 2 and 3: groups with a shorter last one, and with
    blocks that are no multiple of 256 rows inside a group)."""
    name, args = {"dapo-entropy-kl": ("ppo", DAPO_SIDE), "gspo-entropy-kl": ("gspo", GSPO_SIDE)}[case]
    n, h, v = sum(lens), 256, 2000
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=73)
    shift = GSPO_ADV_SHIFT if name == "gspo" else 0.0
    want = oracle_step(hid, w, labels, rl, old, ref, name, args, adv_shift=shift)
    got = fused_step(hid, w, ids, rl, old, ref, name, args, 256 if name == "ppo" else 512, adv_shift=shift,
                     dw_group=dw_group)
    data = got[2]
    assert data.meta_info["head_backward"] == "blocked-stash" and data.meta_info["n_blocks"] >= 3
    assert got[0].item() == pytest.approx(want[0].item(), rel=1e-4, abs=1e-8)
    assert rel_l2(got[3], want[4]) < 2e-2 and rel_l2(got[4], want[5]) < 2e-2


@pytest.mark.parametrize("vocab_chunk", [0, 1024])
@pytest.mark.parametrize("case", ["ppo", "dapo-entropy-kl", "gspo"])
def test_fused_step_vs_unfused_gpu_path(case, vocab_chunk):
    """The same micro-batch through the node and through head -> loss -> autograd: the loss agrees to fp32
    summation order, the gradients to the rounding of the stash, the metrics and the head outputs as well."""
    from axon_amd.models.fsdp_models import loss_from_outputs
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    name, args = {"ppo": ("ppo", PPO), "dapo-entropy-kl": ("ppo", DAPO_SIDE), "gspo": ("gspo", GSPO)}[case]
    g = torch.Generator().manual_seed(5)
    lens = W.uniform_lengths(24, 40, 700, g)
    n, h, v = sum(lens), 256, 8192
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=81, group=4)
    samp = old + 0.01 * torch.randn(n, generator=g)
    extra = {"sampler_log_probs": samp}
    got = fused_step(hid, w, ids, rl, old, ref, name, args, 1024, vocab_chunk=vocab_chunk, extra=extra,
                     adv_shift=GSPO_ADV_SHIFT if name == "gspo" else 0.0)
    assert got[2].meta_info["head_backward"] == "blocked-stash" and got[2].meta_info["n_blocks"] >= 3

    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    cu = rl["cu_seqlens"].to(DEV)
    lp, ent = packed_logprobs(hd, wd, ids.to(DEV), cu)
    b = got[2].batch
    data = DataProto.from_dict(tensors={"old_log_probs": b["old_log_probs"], "advantages": b["advantages"],
                                        "response_mask": rl["response_mask"].to(DEV), "ref_log_prob": b["ref_log_prob"],
                                        "sampler_log_probs": b["sampler_log_probs"]}, meta_info={"cu_seqlens": cu})
    meta = {"loss_fn": name, "loss_fn_args": args, "temperature": 1.0, "dp_replicas": 1}
    loss, metrics = loss_from_outputs(data, lp, ent, meta)
    loss.backward()
    assert got[0].item() == pytest.approx(loss.item(), rel=2e-6, abs=1e-9)
    assert torch.equal(b["log_probs"], lp.detach()) and torch.equal(b["entropys"], ent.detach())
    assert rel_l2(got[3], hd.grad) < 5e-3 and rel_l2(got[4], wd.grad) < 5e-3
    assert set(got[1]) == set(metrics)
    for k, val in metrics.items():
        assert got[1][k] == pytest.approx(val, rel=1e-4, abs=1e-6), k


def test_fused_step_with_sampler_correction_and_global_counts():
    """The correction hook runs once over the whole batch before the blocks (token IS weights, token rejection,
    per-sequence veto); the loss then uses the corrected mask and the weights, the side terms the original mask;
    a ``valid_token_count`` carried by the batch is the denominator of every block."""
    from axon_amd.models.fsdp_models import loss_from_outputs
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    g = torch.Generator().manual_seed(9)
    lens = W.uniform_lengths(20, 30, 500, g)
    n, h, v = sum(lens), 128, 4096
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=91, group=4)
    samp = old + 0.01 * torch.randn(n, generator=g)
    samp[::97] += 1.5  # some tokens outside the rejection bounds
    args = dict(DAPO_SIDE, sampler_is="token", sampler_is_threshold=2.0, sampler_rs="token", sampler_rs_threshold=2.0,
                sampler_token_veto_threshold=1e-4)
    count = torch.full((n,), 3.0 * n, dtype=torch.float32)
    extra = {"sampler_log_probs": samp, "valid_token_count": count}
    got = fused_step(hid, w, ids, rl, old, ref, "ppo", args, 512, extra=extra)
    assert got[2].meta_info["head_backward"] == "blocked-stash"
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    cu = rl["cu_seqlens"].to(DEV)
    lp, ent = packed_logprobs(hd, wd, ids.to(DEV), cu)
    b = got[2].batch
    data = DataProto.from_dict(tensors={"old_log_probs": b["old_log_probs"], "advantages": b["advantages"],
                                        "response_mask": rl["response_mask"].to(DEV), "ref_log_prob": b["ref_log_prob"],
                                        "sampler_log_probs": b["sampler_log_probs"], "valid_token_count": count.to(DEV)},
                               meta_info={"cu_seqlens": cu})
    loss, metrics = loss_from_outputs(data, lp, ent, {"loss_fn": "ppo", "loss_fn_args": args, "temperature": 1.0,
                                                     "dp_replicas": 1})
    loss.backward()
    assert torch.equal(b["response_mask"], data.batch["response_mask"])  # the corrected mask, bit for bit
    assert got[0].item() == pytest.approx(loss.item(), rel=2e-6, abs=1e-9)
    assert rel_l2(got[3], hd.grad) < 5e-3 and rel_l2(got[4], wd.grad) < 5e-3
    assert set(got[1]) == set(metrics)
    for k, val in metrics.items():
        assert got[1][k] == pytest.approx(val, rel=1e-4, abs=1e-6), k


@pytest.mark.parametrize("case", ["ppo", "gspo"])
def test_fused_step_odd_shapes_softcap_temperature_and_integer_operands(case):
    """A token count that is no multiple of four (the last block then has no stash and recomputes its logits), a
    vocabulary that is no multiple of the tile, blocks smaller than a tile, soft-capped logits, a temperature,
    int64 token ids and an int64 response mask (the production dtypes): the node against the unfused path."""
    from axon_amd.models.fsdp_models import loss_from_outputs
    from axon_amd.models.fused_head_loss import fused_head_loss
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    name, args = {"ppo": ("ppo", DAPO_SIDE), "gspo": ("gspo", GSPO)}[case]
    lens = [130, 7, 251, 64, 301, 90]  # 843 tokens
    n, h, v = sum(lens), 96, 1001
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=95)
    cu = rl["cu_seqlens"].to(DEV)
    mask_i64 = rl["response_mask"].to(DEV).long()
    adv = (torch.randn(n, generator=torch.Generator().manual_seed(3)) + (GSPO_ADV_SHIFT if case == "gspo" else 0.0))
    meta = {"loss_fn": name, "loss_fn_args": args, "temperature": 0.7, "dp_replicas": 1}

    def tensors():
        return {"old_log_probs": old.to(DEV), "advantages": adv.to(DEV) * mask_i64, "response_mask": mask_i64.clone(),
                "ref_log_prob": ref.to(DEV)}

    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    data = DataProto.from_dict(tensors=tensors())
    loss, metrics = fused_head_loss(hd, wd, ids.to(DEV).long(), cu, data, meta, block_tokens=384 if case == "gspo" else 200,
                                    logit_softcapping=5.0)
    loss.backward()
    assert data.meta_info["head_backward"] == "blocked-stash" and data.meta_info["n_blocks"] >= 3

    h2, w2 = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = packed_logprobs(h2, w2, ids.to(DEV).long(), cu, 0.7, 5.0)
    data2 = DataProto.from_dict(tensors=tensors(), meta_info={"cu_seqlens": cu})
    loss2, metrics2 = loss_from_outputs(data2, lp, ent, meta)
    loss2.backward()
    assert loss.item() == pytest.approx(loss2.item(), rel=2e-6, abs=1e-9)
    assert torch.equal(data.batch["log_probs"], lp.detach()) and torch.equal(data.batch["entropys"], ent.detach())
    assert rel_l2(hd.grad, h2.grad) < 5e-3 and rel_l2(wd.grad, w2.grad) < 5e-3
    for k, val in metrics2.items():
        assert metrics[k] == pytest.approx(val, rel=1e-4, abs=1e-6), k


def test_fused_step_falls_back_where_blocks_do_not_apply():
    """A loss that selects tokens across the whole batch, and a sequence longer than a block under a
    per-sequence loss, take the unfused path; the node refuses a second backward."""
    lens = RAGGED
    n, h, v = sum(lens), 128, 2000
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=71)
    got = fused_step(hid, w, ids, rl, old, ref, "kl_cov", {"kl_cov_ratio": 0.01}, 256)
    assert got[2].meta_info["head_backward"] == "recompute" and torch.isfinite(got[0]).item()
    got = fused_step(hid, w, ids, rl, old, ref, "gspo", GSPO, 256,  # the 400- and 500-token sequences do not fit
                     adv_shift=GSPO_ADV_SHIFT)
    assert got[2].meta_info["head_backward"] == "recompute"
    want = oracle_step(hid, w, labels, rl, old, ref, "gspo", GSPO, adv_shift=GSPO_ADV_SHIFT)
    assert got[0].item() == pytest.approx(want[0].item(), rel=1e-4, abs=1e-8)
    assert rel_l2(got[3], want[4]) < 2e-2 and rel_l2(got[4], want[5]) < 2e-2

    from axon_amd.models.fused_head_loss import fused_head_loss
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    data = DataProto.from_dict(tensors={"old_log_probs": old.to(DEV), "advantages": torch.ones(n, device=DEV),
                                        "response_mask": rl["response_mask"].to(DEV)})
    loss, _ = fused_head_loss(hd, wd, ids.to(DEV), rl["cu_seqlens"].to(DEV), data,
                              {"loss_fn": "ppo", "loss_fn_args": PPO, "temperature": 1.0, "dp_replicas": 1},
                              block_tokens=512)
    loss.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="second time"):
        loss.backward()


def test_fused_step_scales_the_finished_gradients_by_the_incoming_factor():
    """``dp_replicas`` (and any other factor on the loss) reaches d_hidden and d_weight although they are finished
    before autograd's backward starts."""
    lens = ON_BORDERS
    n, h, v = sum(lens), 128, 2000
    hid, w, ids, labels, rl, old, ref = _inputs(n, h, v, lens, seed=73)
    one = fused_step(hid, w, ids, rl, old, ref, "ppo", PPO, 512, dp_replicas=1)
    four = fused_step(hid, w, ids, rl, old, ref, "ppo", PPO, 512, dp_replicas=4)
    assert four[0].item() == pytest.approx(4 * one[0].item(), rel=1e-6)
    assert rel_l2(four[3], 4 * one[3].float()) < 4e-3 and rel_l2(four[4], 4 * one[4].float()) < 4e-3


def test_qwen3_8b_fused_step_vs_fp32_torch_and_oracle_loss():
    """Config 3 at full size through the node (four blocks of 8192 tokens): log-prob and entropy of every token
    and d_weight on ~120 vocabulary rows against an fp32 torch head on the GPU driven by the CPU oracle's PPO
    loss gradient; d_hidden on a token subset against the CPU oracle; and the loss itself."""
    from head_reference import _fp32_torch_head_reference, _spread_rows
    n, h, v = 32768, 4096, 151936
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=3)
    rl = W.packed_rl_inputs(n, 103, group=8)
    cu = rl["cu_seqlens"].long()
    hd0, wd0, ids_d = hid.to(DEV), w.to(DEV), ids.to(DEV)
    labels_d = torch.roll(ids_d, -1)
    zeros = torch.zeros(n, device=DEV)
    rows = _spread_rows(v)
    ref_lp, ref_ent, _ = _fp32_torch_head_reference(hd0, wd0, labels_d, zeros, None, rows[:1])
    lp_tok = _to_token_positions(ref_lp.cpu(), cu)
    old = lp_tok - 0.05 * torch.randn(n, generator=torch.Generator().manual_seed(7))
    got = fused_step(hid, w, ids, rl, old, old, "ppo", PPO, 8192)
    data = got[2]
    assert data.meta_info["head_backward"] == "blocked-stash" and data.meta_info["n_blocks"] == 4
    assert data.meta_info["stash_bytes"] <= 2 * 8192 * 152064 + (1 << 26)
    assert (data.batch["log_probs"].cpu() - lp_tok).abs().max().item() < 1e-3
    assert (data.batch["entropys"].cpu() - _to_token_positions(ref_ent.cpu(), cu)).abs().max().item() < 1e-3
    # the oracle's loss and its gradient on the reference log-probs, on the padded layout the reference uses
    lens = (cu[1:] - cu[:-1]).tolist()
    tmax = max(lens)
    gidx = torch.tensor(np.unique(rl["uid"], return_inverse=True)[1])
    mask = _pad(rl["response_mask"], cu, tmax)
    adv = OA.grpo_advantage(_pad(rl["token_level_rewards"], cu, tmax), mask, gidx, 1e-6)
    lp_pad = _pad(lp_tok, cu, tmax).requires_grad_(True)
    loss, _ = OL.ppo_loss(lp_pad, _pad(old, cu, tmax), adv, mask, **PPO)
    loss.backward()
    assert got[0].item() == pytest.approx(loss.item(), rel=1e-4, abs=1e-8)
    g_tok = torch.cat([lp_pad.grad[b, :l] for b, l in enumerate(lens)])
    g_head = torch.zeros_like(g_tok)
    g_head[:-1] = g_tok[1:]
    g_head[cu[1:] - 1] = 0.0
    _, _, ref_dw = _fp32_torch_head_reference(hd0, wd0, labels_d, g_head.to(DEV), None, rows)
    got_dw = got[4][rows.to(DEV)].double()
    assert rel_l2(got_dw, ref_dw) < 2e-2
    per_row = (got_dw - ref_dw).norm(dim=1) / ref_dw.norm(dim=1).clamp_min(1e-30)
    assert per_row.max().item() < 5e-2, (per_row.argmax().item(), per_row.max().item())
    idx = torch.cat([torch.arange(0, n, 509), torch.tensor([8191, 8192, 16383, 16384, 24575, 24576, n - 1])])
    o_dh, _ = OM.backward(g_head[idx], None, hid[idx], w, torch.roll(ids, -1)[idx])
    assert rel_l2(got[3][idx.to(DEV)], o_dh) < 2e-2
