"""Pins oracle.returns against the known answers of the reference's tests
(tests/trainer/algos/advantages/test_advantages.py:251-714, 757-960, 1075-1165, 1182-1514 and
tests/trainer/algos/loss/test_loss.py:501-580 — numbers restated as data) and against what the mathematics
fixes: closed forms of the recurrences, brute-force double sums, whitening invariants."""

import pytest
import torch

from oracle import advantage as A
from oracle import returns as R

T = torch.tensor


def _gae_brute(rewards, values, gamma, lam):
    """A_t = sum_l (gamma*lam)^l delta_{t+l} in float64, no mask."""
    r, v = rewards.double(), values.double()
    b, n = r.shape
    vnext = torch.cat([v[:, 1:], torch.zeros(b, 1, dtype=torch.float64)], 1)
    delta = r + gamma * vnext - v
    out = torch.zeros_like(delta)
    for t in range(n):
        for l in range(n - t):
            out[:, t] += (gamma * lam) ** l * delta[:, t + l]
    return out


# ---- GAE ----------------------------------------------------------------------------------------------
def test_gae_reference_orderings():
    rewards = T([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0]])
    values = torch.full((2, 3), 0.5)
    adv, ret = R.gae_advantage(rewards, values, torch.ones(2, 3), 0.99, 0.95)
    assert adv.shape == ret.shape == rewards.shape
    assert ret[0, 2] > ret[0, 0] and ret[1, 1] > ret[1, 2]  # test_advantages.py:286-287


def test_gae_closed_forms():
    torch.manual_seed(1)
    r, v = torch.randn(3, 9), torch.randn(3, 9)
    ones = torch.ones(3, 9)
    raw, ret = R.gae_raw(r, v, ones, 1.0, 1.0)  # lam = gamma = 1: reward-to-go minus the value
    togo = r.flip(-1).cumsum(-1).flip(-1)
    assert torch.allclose(raw, togo - v, atol=1e-5) and torch.allclose(ret, togo, atol=1e-5)
    raw0, _ = R.gae_raw(r, v, ones, 0.9, 0.0)  # lam = 0: the one-step TD error
    vnext = torch.cat([v[:, 1:], torch.zeros(3, 1)], 1)
    assert torch.allclose(raw0, r + 0.9 * vnext - v, atol=1e-6)
    raw2, _ = R.gae_raw(r, v, ones, 0.97, 0.9)
    assert torch.allclose(raw2.double(), _gae_brute(r, v, 0.97, 0.9), atol=1e-5)


def test_gae_mask_skips_observation_tokens():
    """At response tokens the masked recurrence equals the unmasked one over the gathered response tokens; a
    masked token repeats the value of the next response token (advantage.py:66-70)."""
    torch.manual_seed(2)
    r, v = torch.randn(1, 8), torch.randn(1, 8)
    mask = T([[1.0, 0.0, 1.0, 1.0, 0.0, 0.0, 1.0, 0.0]])
    raw, _ = R.gae_raw(r, v, mask, 0.95, 0.9)
    keep = mask[0] > 0
    dense, _ = R.gae_raw(r[:, keep], v[:, keep], torch.ones(1, int(keep.sum())), 0.95, 0.9)
    assert torch.allclose(raw[0, keep], dense[0], atol=1e-6)
    assert raw[0, 1] == raw[0, 2] and raw[0, 4] == raw[0, 6] and raw[0, 5] == raw[0, 6] and raw[0, 7] == 0


def test_whiten_invariants():
    torch.manual_seed(3)
    x = torch.randn(4, 11) * 3 + 2
    mask = (torch.rand(4, 11) > 0.4).float()
    w = R.masked_whiten(x, mask)
    n = mask.sum()
    mean = (w * mask).sum() / n
    var = (((w - mean) ** 2) * mask).sum() / (n - 1)
    assert abs(float(mean)) < 1e-5 and float(var) == pytest.approx(1.0, abs=1e-4)
    # a single selected element: no Bessel factor, variance 0, the output stays finite
    one = torch.zeros(1, 4)
    one[0, 2] = 1
    assert torch.isfinite(R.masked_whiten(torch.randn(1, 4), one)).all()
    assert float(R.masked_var(T([1.0, 3.0]), T([1.0, 1.0]))) == pytest.approx(2.0)
    assert float(R.masked_var(T([1.0, 3.0]), T([1.0, 1.0]), False)) == pytest.approx(1.0)


# ---- chunked GAE, test_advantages.py:757-960, 1132-1165 -----------------------------------------------
def test_chunked_gae_equals_gae_on_response_tokens():
    rewards = T([[0.0, 0.0, 1.0, 0.0, 0.5], [0.0, 1.0, 0.0, 0.0, 0.0]])
    values = torch.full((2, 5), 0.5)
    ones = torch.ones(2, 5)
    raw, ret = R.gae_raw(rewards, values, ones, 0.99, 0.95)
    adv_c, ret_c = R.chunked_gae_advantage(rewards, values, ones, 0.99, 0.95)
    assert torch.allclose(ret_c, ret, atol=1e-5)
    assert torch.allclose(adv_c, R.masked_whiten(raw, ones), atol=1e-5)
    torch.manual_seed(4)
    r, v = torch.randn(3, 13), torch.randn(3, 13)
    mask = (torch.rand(3, 13) > 0.35).float()  # gaps inside the response
    raw, ret = R.gae_raw(r, v, mask, 0.99, 0.95)
    adv_c, ret_c = R.chunked_gae_advantage(r, v, mask, 0.99, 0.95)
    assert torch.allclose(ret_c * mask, ret * mask, atol=1e-5)
    assert (ret_c[mask == 0] == 0).all()
    assert torch.allclose(adv_c, R.masked_whiten(raw * mask, mask), atol=1e-5)


def test_chunked_gae_edge_cases():
    z, _ = R.chunked_gae_advantage(torch.ones(2, 4), torch.ones(2, 4), torch.zeros(2, 4))
    assert (z == 0).all()  # test_all_zero_mask
    adv, ret = R.chunked_gae_advantage(T([[1.0]]), T([[0.25]]), T([[1.0]]), 0.99, 0.95)
    assert float(ret) == pytest.approx(1.0) and torch.isfinite(adv).all()  # single token: delta = r - v
    r = T([[0.0, 0.0, 1.0]])
    _, ret0 = R.chunked_gae_advantage(r, torch.full((1, 3), 0.5), torch.ones(1, 3), 0.0, 0.95)
    assert torch.allclose(ret0, r)  # gamma = 0: returns = rewards


# ---- REINFORCE++, test_advantages.py:310-424 ---------------------------------------------------------
def test_reinforce_pp_known_answers():
    rewards = T([[0.0, 0.0, 1.0], [0.0, 0.0, 2.0], [0.0, 0.0, 0.0]])
    adv, ret = R.reinforce_plus_plus_advantage(rewards, torch.ones(3, 3), 1.0)
    assert torch.allclose(ret, T([[1.0] * 3, [2.0] * 3, [0.0] * 3]))
    _, ret = R.reinforce_plus_plus_advantage(T([[0.0, 0.0, 1.0]]), torch.ones(1, 3), 0.9)
    assert torch.allclose(ret[0], T([0.81, 0.9, 1.0]), atol=1e-6)
    # the running return restarts after the response ends: rewards past the mask do not leak back
    ret = R.reinforce_plus_plus_raw(T([[0.0, 1.0, 5.0]]), T([[1.0, 1.0, 0.0]]), 1.0)
    assert torch.equal(ret, T([[1.0, 1.0, 5.0]]))
    assert torch.isfinite(adv).all()


def test_reinforce_pp_baseline_known_structure():
    rewards = T([[0.0, 0.0, 3.0], [0.0, 0.0, 1.0], [0.0, 0.0, 4.0], [0.0, 0.0, 2.0]])
    adv = R.reinforce_plus_plus_baseline_advantage(rewards, torch.ones(4, 3), T([0, 0, 1, 1]))
    s = adv.sum(-1)
    assert s[0] > 0 and s[1] < 0 and s[2] > 0 and s[3] < 0
    # baselined scores are +1, -1, +1, -1 on every token: whitening divides by the unbiased deviation
    expect = 1.0 / (12.0 / 11.0) ** 0.5
    assert torch.allclose(adv[0], torch.full((3,), expect), atol=1e-5)
    # a group of one keeps its score as the baselined value (baseline 0)
    rewards = T([[0.0, 0.0, 5.0], [0.0, 0.0, 2.0], [0.0, 0.0, 4.0]])
    adv = R.reinforce_plus_plus_baseline_advantage(rewards, torch.ones(3, 3), T([0, 1, 1]))
    base = T([5.0, -1.0, 1.0]).unsqueeze(-1).expand(3, 3)
    assert torch.allclose(adv, R.masked_whiten(base, torch.ones(3, 3)), atol=1e-6)


# ---- ReMax, OPO, pass@k, identity: test_advantages.py:426-514, 577-714, 1075-1112, 1167-1180 ----------
def test_remax_known_answers():
    rewards = T([[0.0, 0.0, 3.0], [0.0, 1.0, 1.0]])
    adv, ret = R.remax_advantage(rewards, torch.ones(2, 3), T([2.0, 1.0]))
    assert torch.equal(ret, T([[3.0, 3.0, 3.0], [2.0, 2.0, 1.0]]))
    assert torch.equal(adv, T([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]]))
    _, ret = R.remax_advantage(T([[1.0, 1.0, 1.0]]), T([[1.0, 1.0, 0.0]]), T([0.0]))
    assert ret[0, 2] == 0 and ret[0, 0] == 2


def test_opo_known_answers():
    adv = R.opo_advantage(T([[0.0, 0.0, 4.0], [0.0, 2.0, 0.0]]), torch.ones(2, 3), T([0, 0]))
    assert torch.allclose(adv.sum(-1), T([3.0, -3.0]), atol=1e-5)
    adv = R.opo_advantage(T([[0.0, 0.0, 5.0]]), torch.ones(1, 3), T([0]))
    assert float(adv.sum()) == pytest.approx(15.0)
    mask = T([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]])
    adv = R.opo_advantage(T([[0.0, 0.0, 6.0], [0.0, 3.0, 0.0]]), mask, T([0, 0]))
    assert torch.allclose(adv, T([[1.2] * 3, [-1.8, -1.8, 0.0]]), atol=1e-5)  # baseline 24/5


def test_passk_known_answers():
    rewards = T([[0.0, 0.0, 5.0], [0.0, 0.0, 3.0], [0.0, 0.0, 1.0]])
    adv = R.grpo_passk_advantage(rewards, torch.ones(3, 3), T([0, 0, 0]), norm_adv_by_std=False)
    assert torch.allclose(adv.sum(-1), T([6.0, 0.0, 0.0]))
    with pytest.raises(ValueError, match="at least 2 samples"):
        R.grpo_passk_advantage(T([[0.0, 0.0, 5.0]]), torch.ones(1, 3), T([0]))
    adv = R.grpo_passk_advantage(T([[0.0, 0.0, 10.0], [0.0, 0.0, 5.0]]), torch.ones(2, 3), T([0, 0]))
    s = adv.sum(-1)
    assert s[1] == 0 and float(s[0]) == pytest.approx(3 * 5.0 / (12.5 ** 0.5 + 1e-6), rel=1e-5)
    same = R.grpo_passk_advantage(torch.ones(3, 2), torch.ones(3, 2), T([0, 0, 0]))
    assert (same == 0).all()  # identical scores: max - second max = 0


def test_identity():
    r, m = T([[1.0, -2.0, 3.0]]), T([[1.0, 1.0, 0.0]])
    assert torch.equal(R.identity_advantage(r, m), T([[1.0, -2.0, 0.0]]))


# ---- Kimi k1.5, test_advantages.py:1182-1514 ---------------------------------------------------------
def _kimi_batch(scores, lengths, max_len=12):
    n = len(scores)
    rewards, mask = torch.zeros(n, max_len), torch.zeros(n, max_len)
    for i in range(n):
        mask[i, : lengths[i]] = 1
        rewards[i, lengths[i] - 1] = scores[i]
    return rewards, mask


def test_kimi_known_answers():
    g = T([0, 0, 0, 0])
    r, m = _kimi_batch([1.0, 1.0, 0.0, 0.0], [3, 6, 4, 8])
    assert torch.allclose(R.kimi_k1_5_advantage(r, m, g, length_coef=0.0), A.grpo_advantage(r, m, g), atol=1e-6)
    r, m = _kimi_batch([1.0, 1.0, 0.0, 0.0], [4, 8, 2, 10])
    adv = R.kimi_k1_5_advantage(r, m, g, length_coef=1.0, norm_adv_by_std=False)
    per_row = adv.sum(-1) / m.sum(-1)
    # lengths span 2..10: lam = 0.5 - (len-2)/8 = .25, -.25, .5, -.5; incorrect rows keep min(0, lam)
    shaped = T([1.25, 0.75, 0.0, -0.5])
    assert torch.allclose(per_row, shaped - shaped.mean(), atol=1e-6)
    r, m = _kimi_batch([1.0, 0.0, 1.0, 0.0], [5, 5, 5, 5])  # no spread: no length pressure
    assert torch.allclose(R.kimi_k1_5_advantage(r, m, g, length_coef=1.0), A.grpo_advantage(r, m, g), atol=1e-6)
    # groups are independent: lengths of one group do not move the other
    r, m = _kimi_batch([1.0, 1.0, 1.0, 1.0], [2, 4, 3, 9])
    a = R.kimi_k1_5_advantage(r, m, T([0, 0, 1, 1]), length_coef=1.0, norm_adv_by_std=False)
    row = a.sum(-1) / m.sum(-1)
    assert torch.allclose(row, T([0.5, -0.5, 0.5, -0.5]), atol=1e-6)


def test_kimi_schedule():
    assert R.kimi_length_coef(0.5, 10, 0, 9) == 0.0
    assert R.kimi_length_coef(0.5, 10, 0, 10) == 0.5
    assert R.kimi_length_coef(1.0, 10, 20, 15) == pytest.approx(0.25)
    assert R.kimi_length_coef(1.0, 10, 20, 30) == 1.0
    assert R.kimi_length_coef(1.0, 0, 0, 0) == 1.0


# ---- value loss, test_loss.py:501-580 -----------------------------------------------------------------
def test_value_loss_known_answers():
    values = T([[1.0, 2.0, 3.0]])
    returns = T([[2.0, 2.0, 2.0]])
    loss, m = R.value_loss(values.clone(), values, returns, torch.ones(1, 3), cliprange_value=10.0)
    assert float(loss) == pytest.approx(1.0 / 3.0, abs=1e-6)
    assert m["vf_clipfrac"] == 0.0 and m["vpred_mean"] == pytest.approx(2.0)


def test_value_loss_clipping_and_gradient():
    """Token by token: inside the clip range both branches agree (gradient vpreds - returns over n); outside
    it the larger squared error wins, and the clipped branch carries no gradient."""
    values = T([[0.0, 0.0, 0.0, 0.0]])
    vpreds = T([[0.2, 1.0, 1.0, -3.0]], requires_grad=True)
    returns = T([[1.0, 0.6, 2.0, -1.0]])
    loss, m = R.value_loss(vpreds, values, returns, torch.ones(1, 4), cliprange_value=0.5)
    # token 1: clipped to .5, (1-.6)^2 = .16 vs (.5-.6)^2 = .01 -> unclipped wins
    # token 2: clipped to .5, (1-2)^2 = 1 vs (.5-2)^2 = 2.25 -> clipped wins, no gradient
    # token 3: clipped to -.5, (-3+1)^2 = 4 vs (-.5+1)^2 = .25 -> unclipped wins
    assert float(loss.detach()) == pytest.approx(0.5 * (0.64 + 0.16 + 2.25 + 4.0) / 4, rel=1e-6)
    loss.backward()
    assert torch.allclose(vpreds.grad, T([[-0.8, 0.4, 0.0, -2.0]]) / 4, atol=1e-6)
    assert m["vf_clipfrac"] == pytest.approx(0.25)
    # a mask of zeros: loss 0, finite
    loss0, _ = R.value_loss(vpreds.detach(), values, returns, torch.zeros(1, 4))
    assert float(loss0) == 0.0
