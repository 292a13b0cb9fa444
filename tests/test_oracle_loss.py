"""Pins oracle.loss against the known answers the reference's own tests hold
(tests/trainer/algos/loss/test_utils.py, test_loss.py — numbers restated as data) and
against a scalar pure-Python evaluation of the PPO/GSPO formulas."""

import math

import pytest
import torch

from oracle import loss as O

T = torch.tensor


# ---- agg_loss known answers: reference tests/trainer/algos/loss/test_utils.py:119-288 -------------
AGG_CASES = [
    # loss, mask, token_reduce, batch_reduce, extra kwargs, expected
    ([[1, 2, 3], [4, 5, 6]], [[1, 1, 0], [1, 1, 1]], "sum", "token-mean", {}, 3.6),
    ([[2, 4], [6, 8]], [[1, 1], [1, 1]], "mean", "step-mean", {}, 5.0),
    ([[1, 2], [3, 4]], [[1, 1], [1, 1]], "sum", "step-mean", {}, 5.0),
    ([[1, 2, 0], [3, 4, 0]], [[1, 1, 0], [1, 1, 0]], "mean-norm", "step-mean", {}, (1 + 7 / 3) / 2),
    ([[1, 999]], [[1, 0]], "sum", "token-mean", {}, 1.0),
    ([[1, 2, 3]], [[1, 1, 1]], "mean-program", "step-mean", {"num_program_tokens": T([6])}, 1.0),
    ([[2, 4], [6, 8], [10, 12]], [[1, 1]] * 3, "mean", "program-mean",
     {"num_program_steps": T([2, 2, 1]), "valid_program_count": 2}, 8.0),
    ([[2, 4], [6, 8], [10, 12]], [[1, 1]] * 3, "mean-program", "program-mean",
     {"num_program_steps": T([2, 2, 1]), "valid_program_count": 2, "num_program_tokens": T([4, 4, 2])}, 6.75),
    ([[2, 4], [6, 8], [999, 999]], [[1, 1], [1, 1], [0, 0]], "mean", "program-mean",
     {"num_program_steps": T([2, 2, 1]), "valid_program_count": 1}, 5.0),
    ([[1, 2], [3, 4], [999, 999]], [[1, 1], [1, 1], [0, 0]], "mean", "step-mean", {}, 2.5),
    ([[1, 2], [3, 4], [999, 999]], [[1, 1], [1, 1], [0, 0]], "sum", "token-mean", {}, 2.5),
    ([[1, 2], [3, 4]], [[0, 0], [0, 0]], "mean", "step-mean", {}, 0.0),
]


@pytest.mark.parametrize("loss,mask,tr,br,kw,expect", AGG_CASES)
def test_agg_loss_known_answers(loss, mask, tr, br, kw, expect):
    out = O.agg_loss(T(loss, dtype=torch.float32), T(mask, dtype=torch.float32), token_reduce=tr, batch_reduce=br, **kw)
    assert out.item() == pytest.approx(expect, rel=1e-6)
    assert not math.isnan(out.item())


def test_agg_loss_errors():
    x = torch.ones(1, 2)
    with pytest.raises(ValueError, match="Invalid token_reduce"):
        O.agg_loss(x, x, token_reduce="bad")
    with pytest.raises(ValueError, match="Invalid batch_reduce"):
        O.agg_loss(x, x, batch_reduce="bad")
    with pytest.raises(AssertionError, match="valid_program_count required"):
        O.agg_loss(x, x, token_reduce="mean", batch_reduce="program-mean", num_program_steps=T([1]))


def test_masked_mean_known_answers():  # reference test_utils.py:17-55
    assert O.masked_mean(T([1.0, 2, 3, 4]), T([1.0, 1, 0, 0])).item() == pytest.approx(1.5)
    assert O.masked_mean(T([1.0, 2]), T([0.0, 0])).item() == 0.0
    assert O.masked_mean(T([[1.0, 2], [3, 4]]), T([[1.0, 0], [1, 1]])).item() == pytest.approx(8 / 3)
    assert O.masked_mean(T([1.0, 2, 3, 4]), T([True, True, False, False])).item() == pytest.approx(1.5)
    v = T([1.0, 2, 3], requires_grad=True)
    O.masked_mean(v, T([1.0, 1, 0])).backward()
    assert torch.allclose(v.grad, T([0.5, 0.5, 0.0]))


# ---- PPO known answers: reference tests/trainer/algos/loss/test_loss.py ------------------------------
def test_ppo_ratio_one():  # :63-87
    lp = T([[-1.0, -2.0, -3.0]], requires_grad=True)
    loss, m = O.ppo_loss(lp, lp.detach().clone(), T([[1.0, 2, 3]]), torch.ones(1, 3), clip_ratio=0.2)
    assert loss.item() == pytest.approx(-2.0)
    assert m["pg_clipfrac"] == 0.0 and m["ppo_kl"] == 0.0


def test_ppo_zero_adv_nan_extreme_and_dual_clip_assert():  # :670-723
    lp = torch.randn(2, 5)
    old = lp + 0.3 * torch.randn(2, 5)
    mask = torch.ones(2, 5)
    assert O.ppo_loss(lp, old, torch.zeros(2, 5), mask)[0].item() == 0.0
    adv = T([[1.0, float("nan"), 3.0]])
    assert math.isnan(O.ppo_loss(T([[0.0, 0, 0]]), T([[0.0, 0, 0]]), adv, torch.ones(1, 3))[0].item())
    big, _ = O.ppo_loss(old + 100.0, old, torch.ones(2, 5), mask)
    assert math.isfinite(big.item())
    for c in (0.5, 1.0):
        with pytest.raises(AssertionError, match="clip_ratio_c must be > 1.0"):
            O.ppo_loss(lp, old, torch.ones(2, 5), mask, clip_ratio_c=c)


def test_gspo_invariants():  # :147-204
    lp = torch.randn(3, 6, requires_grad=True)
    mask = T([[1.0] * 6, [1, 1, 1, 0, 0, 0], [1, 1, 0, 0, 0, 0]])
    loss, m = O.gspo_loss(lp, lp.detach().clone(), torch.randn(3, 6), mask)
    assert loss.dim() == 0 and m["pg_clipfrac"] == 0.0 and m["ppo_kl"] == pytest.approx(0.0, abs=1e-7)
    loss.backward()
    assert lp.grad.abs().sum() > 0 and torch.isfinite(lp.grad).all()
    assert m["pg_clipfrac_lower"] == 0.0


# ---- scalar evaluation of every clip region (A>0 / A<0 x below / inside / above, dual clip) ------
def _ppo_token_scalar(lp, old, A, lo, hi, c):
    """Per-token loss and d loss / d lp, straight from the definition, in Python floats."""
    d = lp - old
    nak = max(-20.0, min(20.0, d))
    passes = -20.0 <= d <= 20.0
    r = math.exp(nak)
    rc = max(1 - lo, min(1 + hi, r))
    l1, g1 = -A * r, -A * r
    l2, g2 = -A * rc, (-A * r if (1 - lo) <= r <= (1 + hi) else 0.0)
    if l1 > l2:
        v, g = l1, g1
    elif l1 < l2:
        v, g = l2, g2
    else:
        v, g = l1, 0.5 * (g1 + g2)
    if A < 0:
        l3 = -A * c
        if l3 < v:
            v, g = l3, 0.0
        elif l3 == v:
            g = 0.5 * g
    return v, (g if passes else 0.0)


REGIONS = [  # (log ratio, advantage)
    (-0.5, 1.5), (0.05, 1.5), (0.5, 1.5),     # A>0: below / inside / above the clip range
    (-0.5, -1.5), (0.05, -1.5), (0.5, -1.5),  # A<0
    (1.5, -1.0),                              # ratio 4.48 > c=3 with A<0: dual clip active
    (25.0, 1.0), (-25.0, -1.0),               # beyond the +-20 safety clamp: no gradient
    (0.0, 0.0),                               # tie everywhere
]


def test_ppo_matches_scalar_definition_all_regions():
    lo, hi, c = 0.2, 0.28, 3.0
    d = T([[x for x, _ in REGIONS]], dtype=torch.float64)
    A = T([[a for _, a in REGIONS]], dtype=torch.float64)
    old = torch.full_like(d, -1.0)
    lp = (old + d).requires_grad_(True)
    mask = torch.ones_like(d)
    loss, _ = O.ppo_loss(lp, old, A, mask, clip_ratio_low=lo, clip_ratio_high=hi, clip_ratio_c=c)
    loss.backward()
    n = len(REGIONS)
    vals, grads = zip(*[_ppo_token_scalar(-1.0 + x, -1.0, a, lo, hi, c) for x, a in REGIONS])
    assert loss.item() == pytest.approx(sum(vals) / n, rel=1e-12)
    for k in range(n):
        assert lp.grad[0, k].item() == pytest.approx(grads[k] / n, rel=1e-12, abs=1e-15), REGIONS[k]


def test_gspo_matches_scalar_definition():
    lo, hi = 3e-4, 4e-4
    torch.manual_seed(0)
    old = -torch.rand(4, 7, dtype=torch.float64)
    lp = (old + 1e-3 * torch.randn(4, 7, dtype=torch.float64)).requires_grad_(True)
    A = torch.randn(4, 7, dtype=torch.float64)
    mask = (torch.rand(4, 7) > 0.3).double()
    mask[3] = 0
    loss, m = O.gspo_loss(lp, old, A, mask, clip_ratio_low=lo, clip_ratio_high=hi, token_reduce="mean",
                          batch_reduce="step-mean")
    loss.backward()
    total, rows_with = 0.0, 0
    for b in range(4):
        cnt = mask[b].sum().item()
        sbar = sum(((lp[b, t] - old[b, t]) * mask[b, t]).item() for t in range(7)) / max(cnt, 1.0)
        s = math.exp(max(-20.0, min(20.0, sbar)))
        sc = max(1 - lo, min(1 + hi, s))
        row = 0.0
        for t in range(7):
            a = A[b, t].item()
            row += max(-a * s, -a * sc) * mask[b, t].item()
            g = -a * s if (-a * s > -a * sc or (1 - lo) <= s <= (1 + hi)) else 0.0
            if -a * s == -a * sc and not ((1 - lo) <= s <= (1 + hi)):
                g = 0.5 * (-a * s)
            expect_g = g * mask[b, t].item() / max(cnt, 1.0)
            got = lp.grad[b, t].item()
            rows_total = (mask.sum(-1) > 0).sum().item()
            assert got == pytest.approx(expect_g / rows_total, rel=1e-9, abs=1e-15)
        total += row / max(cnt, 1.0)
        rows_with += cnt > 0
    assert loss.item() == pytest.approx(total / rows_with, rel=1e-12)


def test_dp_scaling_invariant():
    """Reference tests/trainer/algos/loss/test_loss_scaling.py:224-271: with global counts and
    gradients summed over D shards the gradient equals the single-worker gradient."""
    torch.manual_seed(42)
    B, Tn = 8, 16
    lens = [10, 8, 12, 6, 10, 8, 12, 6]
    mask = torch.zeros(B, Tn)
    for b, l in enumerate(lens):
        mask[b, :l] = 1
    x = torch.randn(B, Tn)
    for tr, br, key in [("sum", "token-mean", "valid_token_count"), ("mean", "step-mean", "valid_batch_size"),
                        ("sum", "step-mean", "valid_batch_size")]:
        w = T(1.0, requires_grad=True)
        count = mask.sum() if key == "valid_token_count" else T(float(B))
        O.agg_loss(x * w, mask, token_reduce=tr, batch_reduce=br, **{key: count}).backward()
        full = w.grad.item()
        acc = 0.0
        for sh in (slice(0, 4), slice(4, 8)):
            w2 = T(1.0, requires_grad=True)
            O.agg_loss(x[sh] * w2, mask[sh], token_reduce=tr, batch_reduce=br, **{key: count}).backward()
            acc += w2.grad.item()
        assert acc == pytest.approx(full, rel=1e-5)


# ---- KL penalty: facts the reference's tests/utils/test_kl.py:178-340 asserts ---------------------
KL_TYPES = ["kl", "k1", "abs", "mse", "k2", "low_var_kl", "k3", "k1+", "k3+"]


def test_oracle_kl_penalty_closed_forms():
    lp = torch.tensor([[-1.0, -2.0, -3.0], [-0.5, -1.5, -2.5]])
    ref = torch.tensor([[-1.5, -1.0, -3.5], [-0.5, -2.0, -2.0]])
    d = (lp - ref).tolist()
    for name, f in [("kl", lambda x: x), ("abs", abs), ("mse", lambda x: 0.5 * x * x),
                    ("low_var_kl", lambda x: math.exp(-x) + x - 1)]:
        got = O.kl_penalty(lp, ref, name).tolist()
        for gr, dr in zip(got, d):
            for g, x in zip(gr, dr):
                assert g == pytest.approx(f(x), abs=1e-6), name
    assert torch.equal(O.kl_penalty(lp, ref, "k1"), O.kl_penalty(lp, ref, "kl"))
    assert torch.equal(O.kl_penalty(lp, ref, "k2"), O.kl_penalty(lp, ref, "mse"))
    assert torch.equal(O.kl_penalty(lp, ref, "k3"), O.kl_penalty(lp, ref, "low_var_kl"))
    assert torch.equal(O.kl_penalty(lp, ref, "k1+"), O.kl_penalty(lp, ref, "k1"))  # forward of "+" = base
    assert torch.equal(O.kl_penalty(lp, ref, "k3+"), O.kl_penalty(lp, ref, "k3"))
    for t in KL_TYPES:
        assert torch.allclose(O.kl_penalty(lp, lp, t), torch.zeros_like(lp), atol=1e-6)
    for t in ("abs", "mse", "low_var_kl"):
        assert (O.kl_penalty(lp, ref, t) >= -1e-7).all()
    big = O.kl_penalty(torch.tensor([[100.0]]), torch.tensor([[-100.0]]), "low_var_kl")
    assert -10.0 <= big.item() <= 10.0
    for t in KL_TYPES:
        assert torch.isfinite(O.kl_penalty(torch.tensor([[100.0, -100.0, 50.0]]),
                                            torch.tensor([[-100.0, 100.0, -50.0]]), t)).all()
    with pytest.raises(NotImplementedError):
        O.kl_penalty(lp, ref, "full")
    with pytest.raises(NotImplementedError):
        O.kl_penalty(lp, ref, "nope")


def test_oracle_kl_penalty_gradients():
    ref = torch.tensor([[-1.5, -1.0, -3.5]])
    for t, g in [("kl", lambda x: 1.0), ("mse", lambda x: x), ("low_var_kl", lambda x: 1 - math.exp(-x)),
                 ("k1+", lambda x: x), ("k3+", lambda x: x), ("abs", lambda x: math.copysign(1.0, x))]:
        lp = torch.tensor([[-1.0, -2.0, -3.0]], requires_grad=True)
        O.kl_penalty(lp, ref, t).sum().backward()
        for got, x in zip(lp.grad[0].tolist(), (lp.detach() - ref)[0].tolist()):
            assert got == pytest.approx(g(x), abs=1e-6), t


def test_oracle_reinforce_known_answers():
    """tests/trainer/algos/loss/test_loss.py:228-259: lp=[1,2], A=[3,4] -> -5.5; IS weight 2 doubles it."""
    lp, adv, m = torch.tensor([[1.0, 2.0]]), torch.tensor([[3.0, 4.0]]), torch.ones(1, 2)
    loss, met = O.reinforce_loss(lp, lp, adv, m)
    assert loss.item() == pytest.approx(-5.5) and met["ppo_kl"] == 0.0
    loss2, _ = O.reinforce_loss(lp, lp, adv, m, sampler_is_weights=torch.full((1, 2), 2.0))
    assert loss2.item() == pytest.approx(-11.0)


def test_oracle_cispo_by_hand():
    old = torch.tensor([[-1.0, -1.0, -1.0, -1.0]])
    lp = (old + torch.tensor([[0.0, 0.5, -0.5, 0.5]])).requires_grad_(True)
    adv, m = torch.tensor([[1.0, 1.0, -2.0, -1.0]]), torch.ones(1, 4)
    loss, met = O.cispo_loss(lp, old, adv, m, clip_ratio_low=0.2, clip_ratio_high=0.28, token_level_mask=True)
    loss.backward()
    r = [1.0, math.exp(0.5), math.exp(-0.5), math.exp(0.5)]
    rc = [min(max(x, 0.8), 1.28) for x in r]
    keep = [1.0, 0.0, 0.0, 1.0]  # A>0 with r>1.28 dropped; A<0 with r<0.8 dropped
    want = sum(-rc[i] * adv[0, i].item() * lp[0, i].item() * keep[i] for i in range(4)) / 4
    assert loss.item() == pytest.approx(want, rel=1e-6)
    for i in range(4):
        assert lp.grad[0, i].item() == pytest.approx(-rc[i] * adv[0, i].item() * keep[i] / 4, rel=1e-6, abs=1e-9)
    assert met["pg_clipfrac"] == pytest.approx(0.75)
    # default: no lower bound, no token mask
    l2, m2 = O.cispo_loss(lp.detach(), old, adv, m)
    assert m2["pg_clipfrac"] == pytest.approx(0.5)  # only r > 1.2 counts


def test_oracle_geo_mean_known_answer_and_by_hand():
    """tests/trainer/algos/loss/test_loss.py:391-403: ratio one, A=[1,2,3] -> -2.0."""
    lp, adv, m = torch.tensor([[-1.0, -2.0, -3.0]]), torch.tensor([[1.0, 2.0, 3.0]]), torch.ones(1, 3)
    loss, met = O.geo_mean_loss(lp, lp, adv, m)
    assert loss.item() == pytest.approx(-2.0, rel=1e-6) and met["pg_clipfrac"] == 0 and met["ppo_kl"] == 0
    # two rows by hand: row 0 A=+1 with nak = [0.5 (clipped to 0.2), -0.5 (kept: min picks the smaller)],
    # row 1 A=-1 with nak = [-0.5 (clipped to -0.2), 0.1]; a fully masked third row is left out of the mean
    old = torch.zeros(3, 2)
    new = torch.tensor([[0.5, -0.5], [-0.5, 0.1], [9.0, 9.0]])
    adv2 = torch.tensor([[1.0, 1.0], [-1.0, -1.0], [5.0, 5.0]])
    m2 = torch.tensor([[1.0, 1.0], [1.0, 1.0], [0.0, 0.0]])
    loss2, met2 = O.geo_mean_loss(new, old, adv2, m2, clip_ratio=0.2)
    r0 = math.exp((0.2 - 0.5) / 2)
    r1 = math.exp((-0.2 + 0.1) / 2)
    assert loss2.item() == pytest.approx((-1.0 * r0 + 1.0 * r1) / 2, rel=1e-6)
    assert met2["pg_clipfrac"] == pytest.approx(0.5) and met2["pg_clipfrac_lower"] == pytest.approx(0.25)


# ---- KL-Cov / Clip-Cov (loss.py:198-352).  The reference's own tests (tests/trainer/algos/loss/test_loss.py:
# 270-365) check shapes, metric keys and the ratio assertion only; the numbers below are worked by hand. ----
def test_kl_cov_worked_example():
    adv = torch.tensor([[1.0, -1.0, 2.0, 0.0]])
    lp = torch.tensor([[-1.0, -2.0, -0.5, -3.0]], requires_grad=True)
    d = torch.tensor([[0.1, -0.2, 0.3, 0.0]])
    old = lp.detach() - d
    # means 0.5 and -1.625: covariances .3125, .5625, 1.6875, .6875 -> k = max(1, int(4 * .25)) = 1 picks token 2
    loss, m, picked = O.kl_cov_loss(lp, old, adv, torch.ones(1, 4), kl_cov_ratio=0.25, ppo_kl_coef=2.0)
    assert picked.tolist() == [2]
    base = [-1.0 * math.exp(0.1), 1.0 * math.exp(-0.2), -2.0 * math.exp(0.3), 0.0]
    assert loss.item() == pytest.approx((sum(base) + 2.0 * 0.3) / 4, rel=1e-6)
    assert m["ppo_kl"] == pytest.approx((0.1 + 0.2 + 0.3) / 4, rel=1e-6)
    loss.backward()
    expect = torch.tensor([[base[0], base[1], base[2] + 2.0, 0.0]]) / 4  # d/dlogp of -A e^d is itself; +coef*sign(d)
    assert torch.allclose(lp.grad, expect, atol=1e-6)
    # masked tokens neither enter the means nor get picked; half the tokens -> k = max(1, int(2 * .25)) = 1
    mask = torch.tensor([[1.0, 1.0, 0.0, 0.0]])
    _, _, picked = O.kl_cov_loss(lp.detach(), old, adv, mask, kl_cov_ratio=0.25)
    assert picked.tolist() == [0]  # means 0 and -1.5: covariances .5 and .5 ... the first of two equal values
    # a larger share picks more tokens: k = int(4 * .75) = 3 -> all but the smallest covariance
    _, _, picked = O.kl_cov_loss(lp.detach(), old, adv, torch.ones(1, 4), kl_cov_ratio=0.75)
    assert sorted(picked.tolist()) == [1, 2, 3]


def test_clip_cov_worked_example():
    adv = torch.tensor([[2.0, -1.0, 1.0, 3.0]])
    lp = torch.tensor([[-1.0, -2.0, -0.5, -3.0]], requires_grad=True)
    d = torch.tensor([[0.5, 0.1, -0.5, 0.0]])
    old = lp.detach() - d
    ones = torch.ones(1, 4)
    # clip 0.2: ratios 1.649 (A>0: clipped at 1.2, pg2 > pg1 -> clipped by origin), 1.105, .607 (A>0: pg1 wins), 1
    cand, clip_num = O.clip_cov_candidates(lp.detach(), old, adv, ones, clip_cov_ratio=0.3, clip_cov_lb=-1.0,
                                            clip_cov_ub=10.0)
    # means 1.25 and -1.625: covariances .46875, .84375, -.28125, -2.40625; token 0 clipped, token 3 below the band
    assert cand.tolist() == [[False, True, True, False]] and clip_num == 1
    sel = torch.tensor([[False, False, True, False]])
    loss, m = O.clip_cov_loss(lp, old, adv, ones, selected=sel, token_reduce="sum")
    terms = [-2.0 * 1.2, 1.0 * math.exp(0.1), 0.0, -3.0]
    assert loss.item() == pytest.approx(sum(terms) / 4, rel=1e-6)
    assert m["pg_clipfrac"] == pytest.approx(0.25) and m["ppo_kl"] == pytest.approx(-0.1 / 4, abs=1e-7)
    loss.backward()
    assert torch.allclose(lp.grad, torch.tensor([[0.0, math.exp(0.1), 0.0, -3.0]]) / 4, atol=1e-6)
    # the random draw takes min(clip_num, candidates) tokens, all of them candidates
    torch.manual_seed(0)
    _, m = O.clip_cov_loss(lp.detach(), old, adv, ones, clip_cov_ratio=0.9, clip_cov_lb=-1.0, clip_cov_ub=10.0)
    assert m["pg_clipfrac"] == pytest.approx(0.5)  # clip_num = int(.9 * 4) = 3, two candidates
