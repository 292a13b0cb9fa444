"""Pins oracle.sampler, oracle.advantage and oracle.layout against the known answers held by
the reference's tests (tests/utils/test_rl_sampler.py, tests/utils/test_rl_advantage.py,
tests/trainer/algos/advantages/test_advantages.py, tests/utils/test_rl_utils.py,
tests/utils/torch/test_ops.py — numbers restated as data) and per-token scalar loops."""

import math

import pytest
import torch

from oracle import advantage as A
from oracle import layout as L
from oracle import sampler as S

T = torch.tensor


# ---- rejection sampling, reference test_rl_sampler.py:41-113 ----------------------------------------
def test_rs_token_known_answers():
    mask = torch.ones(2, 4)
    assert torch.equal(S.rejection_mask(torch.zeros(2, 4), mask, "token", 2.0) * mask, mask)
    assert (S.rejection_mask(torch.full((2, 4), 10.0), mask, "token", 2.0) * mask).sum() == 0
    assert (S.rejection_mask(torch.full((2, 4), -5.0), mask, "token", 2.0) * mask).sum() == 0
    _, new, m = S.correction(torch.full((2, 4), 10.0), torch.zeros(2, 4), mask, sampler_rs="token",
                             sampler_rs_threshold=2.0)
    assert m["sampler_rs_masked_fraction"] == pytest.approx(1.0)


def test_rs_sequence_rejects_whole_row():
    lr = T([[10.0] * 4, [0.0] * 4])
    keep = S.rejection_mask(lr, torch.ones(2, 4), "sequence", 2.0)
    assert keep[0].sum() == 0 and keep[1].sum() == 4


def test_rs_errors():
    with pytest.raises(ValueError, match="Invalid sampler_rs"):
        S.rejection_mask(torch.zeros(1, 2), torch.ones(1, 2), "bogus", 2.0)
    with pytest.raises(ValueError, match="must be provided"):
        S.rejection_mask(torch.zeros(1, 2), torch.ones(1, 2), "token", None)


# ---- importance weights, reference test_rl_sampler.py:119-186 -------------------------------------
def test_is_known_answers():
    torch.manual_seed(0)
    lr = torch.randn(3, 5)
    mask = (torch.rand(3, 5) > 0.3).float()
    w, _ = S.is_weights(lr, mask, "token", 2.0)
    assert (w <= 2.0).all() and (w >= 0).all() and not w.requires_grad
    assert (w[mask == 0] == 0).all()
    ws, _ = S.is_weights(lr, torch.ones(3, 5), "sequence", 1e9)
    assert torch.allclose(ws, ws[:, :1].expand_as(ws))
    w0, raw0 = S.is_weights(torch.zeros(2, 3), torch.ones(2, 3), "token", 2.0)
    assert torch.equal(w0, torch.ones(2, 3)) and S.masked_mean(raw0, torch.ones(2, 3)).item() == pytest.approx(1.0)
    wbig, _ = S.is_weights(T([[70.0, -70.0]]), torch.ones(1, 2), "token", 1e12)
    assert torch.isfinite(wbig).all() and wbig[0, 0].item() == pytest.approx(math.exp(20), rel=1e-4)
    with pytest.raises(ValueError, match="must be positive"):
        S.is_weights(lr, mask, "token", 0.0)


# ---- unified interface, reference test_rl_sampler.py:199-310 -------------------------------------
def test_unified_known_answers():
    old = torch.zeros(2, 4)
    samp = torch.zeros(2, 4)
    mask = torch.ones(2, 4)
    w, new, m = S.correction(old, samp, mask, sampler_is="token")
    assert w is not None and torch.equal(new, mask)
    w, new, m = S.correction(old, samp, mask, sampler_rs="token", sampler_rs_threshold=2.0)
    assert w is None
    w, new, m = S.correction(old, samp, mask)
    assert w is None and torch.equal(new, mask)
    # veto: threshold 0.01, one token at log-ratio -10 vetoes row 0 (fraction 0.5)
    old2 = old.clone()
    old2[0, 1] = -10.0
    _, new, m = S.correction(old2, samp, mask, sampler_token_veto_threshold=0.01)
    assert new[0].sum() == 0 and new[1].sum() == 4
    assert m["sampler_is_veto_fraction"] == pytest.approx(0.5)
    with pytest.raises(ValueError, match="must be positive"):
        S.correction(old, samp, mask, sampler_token_veto_threshold=-1.0)
    zero = torch.zeros(2, 4)
    w, new, m = S.correction(old, samp, zero, sampler_is="token", sampler_rs="token")
    assert w is None and new is zero and m == {}


def test_correction_matches_scalar_loop():
    torch.manual_seed(3)
    B, Tn = 5, 9
    old = -torch.rand(B, Tn) * 3
    samp = old + torch.randn(B, Tn) * 0.5
    samp[2, 3] = old[2, 3] + 12.0  # catastrophic token
    mask = (torch.rand(B, Tn) > 0.25).float()
    mask[4] = 0
    for is_l, rs_l in [("token", "token"), ("sequence", "sequence"), ("token", "geometric")]:
        w, new, _ = S.correction(old, samp, mask, sampler_is=is_l, sampler_is_threshold=2.0, sampler_rs=rs_l,
                                 sampler_rs_threshold=2.0, sampler_token_veto_threshold=1e-4)
        for b in range(B):
            lrs = [(old[b, t] - samp[b, t]).item() for t in range(Tn)]
            ms = [mask[b, t].item() for t in range(Tn)]
            ssum = sum(l * m for l, m in zip(lrs, ms))
            smean = ssum / (sum(ms) + 1e-8)
            veto = any(l < math.log(1e-4) and m for l, m in zip(lrs, ms))
            for t in range(Tn):
                src = {"token": lrs[t], "sequence": ssum, "geometric": smean}
                ew = min(math.exp(max(-20, min(20, src[is_l]))) * ms[t], 2.0)
                assert w[b, t].item() == pytest.approx(ew, rel=2e-6, abs=1e-7)
                ratio = math.exp(max(-20, min(20, src[rs_l])))
                if abs(ratio - 2.0) > 1e-5 and abs(ratio - 0.5) > 1e-5:  # away from the fp32 boundary
                    keep = 0.5 <= ratio <= 2.0
                    assert new[b, t].item() == ms[t] * keep * (not veto)


# ---- group_mean_std, reference test_rl_advantage.py:110-220 --------------------------------------
def test_group_mean_std_known_answers():
    m, s, c = A.group_mean_std(T([1.0, 2, 3]), T([0, 0, 0]))
    assert s.item() == pytest.approx(1.0) and m.item() == pytest.approx(2.0)
    _, s, _ = A.group_mean_std(T([1.0, 3, 2, 4]), T([0, 0, 1, 1]))
    assert torch.allclose(s, torch.full((2,), math.sqrt(2.0)))
    m, s, c = A.group_mean_std(T([5.0]), T([0]))
    assert (m.item(), s.item(), c.item()) == (0.0, 1.0, 1.0)
    m, s, c = A.group_mean_std(T([10.0, 1, 2, 3]), T([0, 1, 1, 1]))
    assert torch.allclose(m, T([0.0, 2.0])) and torch.equal(c, T([1.0, 3.0]))
    assert all(x.numel() == 0 for x in A.group_mean_std(torch.empty(0), torch.empty(0, dtype=torch.long)))
    with pytest.raises(ValueError, match="mismatch"):
        A.group_mean_std(T([1.0, 2]), T([0]))
    m, s, c = A.group_mean_std(T([10.0, 20]), T([0, 5]))
    assert c.tolist() == [1, 0, 0, 0, 0, 1] and (m == 0).all()
    m, s, _ = A.group_mean_std(T([5.0, 5, 5]), T([0, 0, 0]))
    assert m.item() == pytest.approx(5.0) and s.item() == pytest.approx(math.sqrt(1e-6))
    x = T([1.0, 3, 5, 7])
    _, s, _ = A.group_mean_std(x, T([0, 0, 0, 0]))
    assert s.item() == pytest.approx(torch.std(x).item())


def test_group_mean_std_matches_torch_std_per_group():
    torch.manual_seed(1)
    x = torch.randn(40)
    g = torch.randint(0, 6, (40,))
    m, s, c = A.group_mean_std(x, g)
    for k in range(6):
        sel = x[g == k]
        if sel.numel() > 1:
            assert m[k].item() == pytest.approx(sel.mean().item(), abs=1e-6)
            assert s[k].item() == pytest.approx(max(sel.std().item(), 1e-3), rel=1e-4)


# ---- GRPO, reference test_advantages.py:70-155,715-755,961-1022 ---------------------------------
def test_grpo_known_answers():
    rew = T([[0.0, 0, 2], [0, 0, 0]])
    mask = torch.ones(2, 3)
    adv = A.grpo_advantage(rew, mask, T([0, 0]), norm_adv_by_std=False)
    assert torch.equal(adv[0], torch.ones(3)) and torch.equal(adv[1], -torch.ones(3))
    assert (A.grpo_advantage(rew, mask, T([0, 1])) == 0).all()  # singleton groups
    mask2 = T([[1.0, 0, 1], [1, 1, 1]])
    assert A.grpo_advantage(rew, mask2, T([0, 0]))[0, 1].item() == 0.0
    same = T([[0.0, 1], [0, 1], [1, 0]])
    assert A.grpo_advantage(same, torch.ones(3, 2), T([0, 0, 0])).abs().max() < 1e-5
    assert (A.grpo_advantage(torch.zeros(4, 2), torch.ones(4, 2), T([0, 0, 1, 1])) == 0).all()
    # sizes 1/2/3: singleton zero, signs follow score - mean
    rew3 = T([[5.0], [1.0], [3.0], [1.0], [2.0], [6.0]])
    adv3 = A.grpo_advantage(rew3, torch.ones(6, 1), T([0, 1, 1, 2, 2, 2])).squeeze(1)
    assert adv3[0] == 0 and adv3[1] < 0 < adv3[2] and adv3[3] < 0 and adv3[5] > 0


def test_grpo_std_floor_and_double_eps():
    """std = sqrt(max(var, eps)) and the divide adds eps again (advantage.py:102)."""
    rew = T([[1.0], [0.0], [1.0], [0.0]])
    adv = A.grpo_advantage(rew, torch.ones(4, 1), T([0, 0, 0, 0]), eps=1e-6)
    std = torch.std(T([1.0, 0, 1, 0])).item()
    assert adv[0, 0].item() == pytest.approx(0.5 / (std + 1e-6), rel=1e-6)


# ---- dynamic sampling, reference test_rl_utils.py:38-104 ------------------------------------------
def test_zero_advantage_filter_known_answers():
    assert A.zero_advantage_keep_rows(T([[1.0, 2], [0, 0], [5, 6]])) == [0, 2]
    assert A.zero_advantage_keep_rows(T([[1e-7, 1e-8]])) == []
    assert A.zero_advantage_keep_rows(T([[1e-5, 0.0]])) == []  # exactly eps is not > eps
    assert A.zero_advantage_keep_rows(T([[-1.0, 0.0]])) == [0]
    assert A.zero_advantage_keep_rows(T([[0.0, 0.0, 0.3]])) == [0]


# ---- mini-batch counts, reference tests/driver/test_driver_utils.py:260-281 -----------------------
def test_mini_batch_counts_known_answer():
    mask = T([[1, 1, 0], [1, 0, 0], [0, 0, 0]])
    rows, tokens, per_row, programs = A.mini_batch_counts(mask, ["program-a", "program-a", "program-padding"])
    assert (rows, tokens, programs) == (2, 3, 1)
    assert per_row.tolist() == [2, 1, 0] and per_row.dtype == torch.long
    assert A.mini_batch_counts(mask)[3] is None


# ---- layout, reference test_ops.py:513-561,723-729 -------------------------------------------------
def test_unpad_known_answers():
    idx, cu, mx = L.unpad_data(T([[1, 1, 1, 0, 0], [1, 1, 0, 0, 0]]))
    assert cu.tolist() == [0, 3, 5] and cu.dtype == torch.int32 and mx == 3
    assert idx.tolist() == [0, 1, 2, 5, 6]
    _, cu, _ = L.unpad_data(T([[1] * 5, [1, 0, 0, 0, 0], [1, 1, 1, 0, 0]]))
    assert cu.tolist() == [0, 5, 6, 9]
    _, cu, mx = L.unpad_data(torch.zeros(2, 4, dtype=torch.long))
    assert cu.tolist() == [0, 0, 0] and mx == 0


def test_shift_contract():
    """result[b,t] = head output at position t-1; result[b,0] = 0 (forward_utils.py:164-171)."""
    am = T([[1, 1, 1, 0], [1, 1, 0, 0]])
    idx, _, _ = L.unpad_data(am)
    out = L.head_outputs_to_token_positions(T([10.0, 11, 12, 20, 21]), idx, 2, 4)
    assert out.tolist() == [[0, 10, 11, 12], [0, 20, 21, 0]]


# ---- diagnostics: known answers of tests/utils/test_rl_sampler.py:158-178, 317-368 ----------------
def test_oracle_offpolicy_known_answers():
    old = torch.tensor([[-1.5, -2.5]])
    samp = torch.tensor([[-1.0, -2.0]])
    m = S.offpolicy_metrics(old, samp, torch.ones(1, 2))
    assert m["kl"] == pytest.approx(0.5)
    assert set(m) == {"training_ppl", "training_log_ppl", "kl", "k3_kl", "sampler_ppl", "sampler_log_ppl",
                      "log_ppl_diff", "log_ppl_abs_diff", "log_ppl_diff_max", "log_ppl_diff_min", "ppl_ratio",
                      "chi2_token", "chi2_seq"}
    same = S.offpolicy_metrics(old, old, torch.ones(1, 2))
    assert same["kl"] == 0 and same["k3_kl"] == 0 and same["chi2_token"] == 0 and same["ppl_ratio"] == 1
    assert S.offpolicy_metrics(old, samp, torch.zeros(1, 2)) == {}
    assert set(S.offpolicy_metrics(old, None, torch.ones(1, 2))) == {"training_ppl", "training_log_ppl"}


def test_oracle_weight_metrics_known_answers():
    lr, mask = torch.zeros(3, 5), torch.ones(3, 5)
    m = S.full_metrics(lr, torch.zeros(3, 5), mask, sampler_is="token", sampler_rs="token")
    assert m["sampler_is_mean"] == pytest.approx(1.0) and m["sampler_is_eff_sample_size"] == pytest.approx(1.0)
    assert m["sampler_rs_masked_fraction"] == 0.0 and m["sampler_rs_seq_masked_fraction"] == 0.0
    # lr = +-70 with a huge threshold: finite, the upper weight is e^20 (the +-20 clamp)
    big = torch.tensor([[70.0, -70.0]])
    mm = S.full_metrics(big, torch.zeros(1, 2), torch.ones(1, 2), sampler_is="token", sampler_is_threshold=1e12)
    assert all(math.isfinite(v) for v in mm.values())
    assert mm["sampler_is_max"] == pytest.approx(math.exp(20.0), rel=1e-4)
    # a row of lr = 10 is rejected whole at sequence level, a row of 0 kept
    seq = S.full_metrics(torch.tensor([[10.0] * 4, [0.0] * 4]), torch.zeros(2, 4), torch.ones(2, 4),
                          sampler_rs="sequence", sampler_rs_threshold=2.0)
    assert seq["sampler_rs_seq_masked_fraction"] == 0.5 and seq["sampler_rs_masked_fraction"] == pytest.approx(0.5)
    assert seq["sampler_rs_ratio_fraction_high"] == 0.5 and seq["sampler_rs_max"] == pytest.approx(math.exp(20.0))


def test_oracle_mismatch_stats_by_hand():
    old = torch.tensor([[-1.0, -2.0, -9.0]])
    samp = torch.tensor([[-1.5, -2.0, -1.0]])
    mask = torch.tensor([[1.0, 1.0, 0.0]])
    s = S.mismatch_stats(old, samp, mask)
    pa, ps = [math.exp(-1.0), math.exp(-2.0)], [math.exp(-1.5), math.exp(-2.0)]
    assert s["_valid_count"] == 2
    assert s["_sum"] == pytest.approx(abs(pa[0] - ps[0])) and s["batch/sampler_probs_diff_min"] == 0.0
    assert s["_logprobs_sum"] == pytest.approx(0.5) and s["batch/sampler_logprobs_diff_max"] == pytest.approx(0.5)
    assert s["_product_sum"] == pytest.approx(pa[0] * ps[0] + pa[1] * ps[1])
    assert S.mismatch_stats(old, samp, torch.zeros(1, 3))["_valid_count"] == 0


def test_oracle_rloo_and_gpg_by_hand():
    # groups: {0,1,2} scores 1,2,6 ; {3} score 5 ; {4,5} scores 0,4
    tlr = torch.zeros(6, 3)
    tlr[:, 1] = torch.tensor([1.0, 2.0, 6.0, 5.0, 0.0, 4.0])
    mask = torch.ones(6, 3)
    mask[2, 2] = 0
    g = torch.tensor([0, 0, 0, 1, 2, 2])
    r = A.rloo_advantage(tlr, mask, g)
    # (n*s - S)/(n-1): (3*1-9)/2=-3, (6-9)/2=-1.5, (18-9)/2=4.5 ; singleton 0 ; (0-4)/1=-4, (8-4)/1=4
    assert r[:, 0].tolist() == pytest.approx([-3.0, -1.5, 4.5, 0.0, -4.0, 4.0])
    assert r[2, 2].item() == 0.0
    gp = A.gpg_advantage(tlr, mask, g, f_norm=2.0)
    alpha = 6 / 5  # one zero score
    assert gp[:, 0].tolist() == pytest.approx([alpha * (1 - 3) / 2, alpha * (2 - 3) / 2, alpha * (6 - 3) / 2,
                                               alpha * 5 / 2, alpha * (0 - 2) / 2, alpha * (4 - 2) / 2])
