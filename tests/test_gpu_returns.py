"""GPU parity: the return-based and remaining group-based advantage estimators and the value loss, through the
registries (ctypes -> libaxon_amd.so), against the CPU oracle.

Tolerances: the recurrences run as parallel scans, so sums form in another order than the oracle's loop from
the last token to the first: 2e-5 relative-L2 on raw advantages / returns, 1e-4 on whitened advantages (the
whitening divides by a deviation that carries its own rounding); group scalars 1e-5; value loss 1e-4 relative,
its gradient 1e-5 relative-L2; zeros exact."""

import numpy as np
import pytest
import torch

from axon_amd import _ops, workloads as W
from axon_amd.protocol import DataProto
from axon_amd.trainer.algos.advantages import compute_advantage
from axon_amd.trainer.algos.loss import compute_loss_fn
from oracle import returns as OR

pytestmark = pytest.mark.gpu
T = torch.tensor
DEV = "cuda"


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _proto(tensors, uid=None, meta=None, dev=DEV):
    d = DataProto.from_dict(tensors={k: v.to(dev) for k, v in tensors.items()}, meta_info=meta or {})
    if uid is not None:
        d.non_tensor_batch["uid"] = uid
    return d


def _run(name, tensors, args=None, uid=None, meta=None, dev=DEV):
    out = compute_advantage(_proto(tensors, uid, meta, dev), {"advantage": name, "advantage_args": args or {}})
    return out.batch["advantages"], out.batch["returns"]


def _value_batch(b, t, seed, gaps=True, mask_dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    rewards = torch.randn(b, t, generator=g) * (torch.rand(b, t, generator=g) > 0.7)
    values = torch.randn(b, t, generator=g)
    lens = torch.randint(1, t + 1, (b,), generator=g)
    mask = (torch.arange(t)[None, :] < lens[:, None]).float()
    if gaps:  # observation tokens inside the response
        mask = mask * (torch.rand(b, t, generator=g) > 0.25)
    return rewards, values, mask.to(mask_dtype)


# lengths around the scan's sub-block (64) and step (256) sizes, and a long row
SHAPES = [(3, 1), (5, 63), (4, 64), (4, 65), (6, 255), (3, 256), (3, 257), (2, 1500), (17, 333)]


@pytest.mark.parametrize("b,t", SHAPES)
@pytest.mark.parametrize("name", ["gae", "chunked_gae"])
def test_gae_vs_oracle(name, b, t):
    r, v, m = _value_batch(b, t, seed=b * 1000 + t)
    if m.sum() < 2:
        m[0, 0] = 1
        m[-1, 0] = 1
    adv, ret = _run(name, {"token_level_rewards": r, "values": v, "response_mask": m},
                    {"gamma": 0.99, "lam": 0.95, "chunk_size": 16})
    fn = OR.gae_advantage if name == "gae" else OR.chunked_gae_advantage
    ref_adv, ref_ret = fn(r, v, m, 0.99, 0.95)
    assert rel_l2(ret, ref_ret) < 2e-5
    assert rel_l2(adv, ref_adv) < 1e-4
    if name == "chunked_gae":
        assert (ret.cpu()[m == 0] == 0).all()


@pytest.mark.parametrize("mask_dtype", [torch.int64, torch.bool])
def test_gae_other_mask_types_and_defaults(mask_dtype):
    r, v, m = _value_batch(6, 200, seed=5)
    adv, ret = _run("gae", {"token_level_rewards": r, "values": v, "response_mask": m.to(mask_dtype)})
    ref_adv, ref_ret = OR.gae_advantage(r, v, m)  # gamma 0.99, lam 0.95
    assert rel_l2(ret, ref_ret) < 2e-5 and rel_l2(adv, ref_adv) < 1e-4


def test_fractional_masks_blend_like_the_reference():
    """The reference blends with the mask value (``x * m + (1 - m) * carried``); a weight of 0.5 must do so here."""
    r, v, m = _value_batch(5, 300, seed=8)
    g = torch.Generator().manual_seed(9)
    m = m * torch.where(torch.rand(5, 300, generator=g) > 0.5, 1.0, 0.5)
    rows = _ops.rows_of(r.to(DEV))
    adv, ret = _ops.reverse_scan(_ops.SCAN_GAE, r.to(DEV), v.to(DEV), m.to(DEV), rows, gamma=0.99, lam=0.95)
    ref_adv, ref_ret = OR.gae_raw(r, v, m, 0.99, 0.95)
    assert rel_l2(adv, ref_adv) < 2e-5 and rel_l2(ret, ref_ret) < 2e-5
    _, ret = _ops.reverse_scan(_ops.SCAN_DISCOUNTED, r.to(DEV), None, m.to(DEV), rows, gamma=0.9)
    assert rel_l2(ret, OR.reinforce_plus_plus_raw(r, m, 0.9)) < 2e-5


def test_gae_closed_forms_on_the_gpu():
    """Independent of the oracle: lam = gamma = 1 gives reward-to-go minus value; lam = 0 the TD error."""
    g = torch.Generator().manual_seed(11)
    r, v = torch.randn(4, 700, generator=g), torch.randn(4, 700, generator=g)
    ones = torch.ones(4, 700)
    rows = _ops.rows_of(r.to(DEV))
    adv, ret = _ops.reverse_scan(_ops.SCAN_GAE, r.to(DEV), v.to(DEV), ones.to(DEV), rows, gamma=1.0, lam=1.0)
    togo = r.double().flip(-1).cumsum(-1).flip(-1)
    assert rel_l2(ret, togo) < 1e-5 and rel_l2(adv, togo - v.double()) < 1e-5
    adv0, _ = _ops.reverse_scan(_ops.SCAN_GAE, r.to(DEV), v.to(DEV), ones.to(DEV), rows, gamma=0.9, lam=0.0)
    vnext = torch.cat([v[:, 1:], torch.zeros(4, 1)], 1)
    assert torch.allclose(adv0.cpu(), r + 0.9 * vnext - v, atol=1e-6)


def test_gae_known_orderings_and_cpu_staging():
    rewards = T([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0]])
    adv, ret = _run("gae", {"token_level_rewards": rewards, "values": torch.full((2, 3), 0.5),
                            "response_mask": torch.ones(2, 3)}, {"gamma": 0.99, "lam": 0.95}, dev="cpu")
    assert adv.device.type == "cpu" and ret.device.type == "cpu"
    assert ret[0, 2] > ret[0, 0] and ret[1, 1] > ret[1, 2]


def test_chunked_gae_edge_cases_gpu():
    z = {"token_level_rewards": torch.ones(2, 4), "values": torch.ones(2, 4), "response_mask": torch.zeros(2, 4)}
    adv, ret = _run("chunked_gae", z)
    assert (adv == 0).all() and (ret == 0).all()
    one = {"token_level_rewards": T([[1.0]]), "values": T([[0.25]]), "response_mask": T([[1.0]])}
    adv, ret = _run("chunked_gae", one)
    assert ret.item() == pytest.approx(1.0) and torch.isfinite(adv).all()
    r = T([[0.0, 0.0, 1.0]])
    _, ret = _run("chunked_gae", {"token_level_rewards": r, "values": torch.full((1, 3), 0.5),
                                  "response_mask": torch.ones(1, 3)}, {"gamma": 0.0})
    assert torch.allclose(ret.cpu(), r)


def test_gae_packed_layout_matches_padded():
    lens = [700, 33, 1, 1200, 64, 257]
    r, v, m = _value_batch(len(lens), max(lens), seed=21)
    for i, l in enumerate(lens):
        m[i, l:] = 0
    pack = lambda x: torch.cat([x[i, :l] for i, l in enumerate(lens)])  # noqa: E731
    cu = W.cu_from_lengths(lens)
    for name in ("gae", "reinforce_plus_plus"):
        tensors = {"token_level_rewards": r, "values": v, "response_mask": m}
        pad_adv, pad_ret = _run(name, tensors)
        pk_adv, pk_ret = _run(name, {k: pack(x) for k, x in tensors.items()}, meta={"cu_seqlens": cu})
        # padding holds mask 0 and carries nothing back into the row, so the valid part agrees
        assert rel_l2(pk_ret, pack(pad_ret.cpu())) < 1e-6
        assert rel_l2(pk_adv, pack(pad_adv.cpu())) < 1e-5


@pytest.mark.parametrize("b,t", SHAPES)
@pytest.mark.parametrize("gamma", [1.0, 0.9])
def test_reinforce_pp_vs_oracle(b, t, gamma):
    r, _, m = _value_batch(b, t, seed=7 * b + t, gaps=False)
    if m.sum() < 2:
        m[:, 0] = 1
    adv, ret = _run("reinforce_plus_plus", {"token_level_rewards": r, "response_mask": m}, {"gamma": gamma})
    ref_adv, ref_ret = OR.reinforce_plus_plus_advantage(r, m, gamma)
    assert rel_l2(ret, ref_ret) < 2e-5 and rel_l2(adv, ref_adv) < 1e-4
    assert (adv.cpu()[m == 0] == 0).all()


def test_reinforce_pp_known_answers_gpu():
    _, ret = _run("reinforce_plus_plus", {"token_level_rewards": T([[0.0, 0.0, 1.0]]),
                                          "response_mask": torch.ones(1, 3)}, {"gamma": 0.9})
    assert torch.allclose(ret.cpu()[0], T([0.81, 0.9, 1.0]), atol=1e-6)
    _, ret = _run("reinforce_plus_plus", {"token_level_rewards": T([[0.0, 1.0, 5.0]]),
                                          "response_mask": T([[1.0, 1.0, 0.0]])})
    assert torch.equal(ret.cpu(), T([[1.0, 1.0, 5.0]]))


@pytest.mark.parametrize("b,t", [(2, 3), (5, 300), (9, 1025)])
def test_remax_vs_oracle(b, t):
    r, _, m = _value_batch(b, t, seed=3 * b + t)
    base = torch.randn(b)
    adv, ret = _run("remax", {"token_level_rewards": r, "response_mask": m, "reward_baselines": base})
    ref_adv, ref_ret = OR.remax_advantage(r, m, base)
    assert rel_l2(ret, ref_ret) < 2e-5 and rel_l2(adv, ref_adv) < 2e-5


def test_remax_known_answers_gpu():
    adv, ret = _run("remax", {"token_level_rewards": T([[0.0, 0.0, 3.0], [0.0, 1.0, 1.0]]),
                              "response_mask": torch.ones(2, 3), "reward_baselines": T([2.0, 1.0])})
    assert torch.equal(ret.cpu(), T([[3.0, 3.0, 3.0], [2.0, 2.0, 1.0]]))
    assert torch.equal(adv.cpu(), T([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]]))


def test_masked_whiten_gpu():
    g = torch.Generator().manual_seed(13)
    for n in (1, 3, 4, 1023, 70001):
        x = torch.randn(n, generator=g) * 3 + 2
        m = (torch.rand(n, generator=g) > 0.4).float()
        for remask in (False, True):
            out, stats = _ops.masked_whiten(x.to(DEV), m.to(DEV), remask=remask)
            ref = OR.masked_whiten(x, m) * (m if remask else 1)
            assert torch.allclose(out.cpu(), ref, rtol=2e-5, atol=2e-5), (n, remask)
            assert stats[1].item() == m.sum().item()
    out, _ = _ops.masked_whiten(torch.randn(5, 7).to(DEV), torch.ones(5, 7, dtype=torch.int64).to(DEV))
    assert out.shape == (5, 7) and abs(out.mean().item()) < 1e-5


# ---- group scalars ------------------------------------------------------------------------------------
def _group_case(seed=7):
    d = W.c1_loss_only(seed, groups=6, samples=5, seqlen=200)
    uid = d["uid"].copy()
    uid[3] = "alone"
    gidx = T(np.unique(uid, return_inverse=True)[1])
    return d["token_level_rewards"], d["response_mask"], uid, gidx


def test_opo_and_baseline_vs_oracle():
    r, m, uid, gidx = _group_case()
    r = r * torch.randn(r.shape[0], 1)  # real-valued scores
    adv, ret = _run("opo", {"token_level_rewards": r, "response_mask": m}, uid=uid)
    assert torch.allclose(adv.cpu(), OR.opo_advantage(r, m, gidx), rtol=1e-5, atol=1e-6) and ret is adv
    adv, _ = _run("reinforce_plus_plus_baseline", {"token_level_rewards": r, "response_mask": m}, uid=uid)
    assert rel_l2(adv, OR.reinforce_plus_plus_baseline_advantage(r, m, gidx)) < 1e-4
    assert (adv.cpu()[m == 0] == 0).all()


def test_opo_known_answers_gpu():
    run = lambda r, m, u: _run("opo", {"token_level_rewards": r, "response_mask": m}, uid=np.array(u))[0].cpu()  # noqa: E731
    assert torch.allclose(run(T([[0.0, 0.0, 4.0], [0.0, 2.0, 0.0]]), torch.ones(2, 3), ["a", "a"]).sum(-1),
                          T([3.0, -3.0]), atol=1e-5)
    assert run(T([[0.0, 0.0, 5.0]]), torch.ones(1, 3), ["a"]).sum().item() == pytest.approx(15.0)
    adv = run(T([[0.0, 0.0, 6.0], [0.0, 3.0, 0.0]]), T([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]]), ["a", "a"])
    assert torch.allclose(adv, T([[1.2] * 3, [-1.8, -1.8, 0.0]]), atol=1e-5)


@pytest.mark.parametrize("norm", [True, False])
def test_passk_vs_oracle(norm):
    r, m, uid, gidx = _group_case(9)
    uid[3] = uid[4]  # no group of one
    gidx = T(np.unique(uid, return_inverse=True)[1])
    r = r * torch.randn(r.shape[0], 1)
    adv, _ = _run("grpo_passk", {"token_level_rewards": r, "response_mask": m},
                  {"norm_adv_by_std": norm, "epsilon": 1e-6}, uid=uid)
    assert torch.allclose(adv.cpu(), OR.grpo_passk_advantage(r, m, gidx, 1e-6, norm), rtol=1e-5, atol=1e-6)


def test_passk_known_answers_and_error_gpu():
    rewards = T([[0.0, 0.0, 5.0], [0.0, 0.0, 3.0], [0.0, 0.0, 1.0]])
    adv, _ = _run("grpo_passk", {"token_level_rewards": rewards, "response_mask": torch.ones(3, 3)},
                  {"norm_adv_by_std": False}, uid=np.array(["a", "a", "a"]))
    assert torch.allclose(adv.cpu().sum(-1), T([6.0, 0.0, 0.0]))
    with pytest.raises(ValueError, match="at least 2 samples"):
        _run("grpo_passk", {"token_level_rewards": rewards[:1], "response_mask": torch.ones(1, 3)},
             uid=np.array(["a"]))
    same, _ = _run("grpo_passk", {"token_level_rewards": torch.ones(3, 2), "response_mask": torch.ones(3, 2)},
                   uid=np.array(["a", "a", "a"]))
    assert (same == 0).all()


@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("coef", [0.0, 0.5, 1.0])
def test_kimi_vs_oracle(norm, coef):
    r, m, uid, gidx = _group_case(12)
    adv, _ = _run("kimi_k1_5", {"token_level_rewards": r, "response_mask": m},
                  {"length_coef": coef, "norm_adv_by_std": norm, "correct_threshold": 1.0}, uid=uid)
    ref = OR.kimi_k1_5_advantage(r, m, gidx, length_coef=coef, norm_adv_by_std=norm)
    assert torch.allclose(adv.cpu(), ref, rtol=1e-5, atol=2e-6)


def test_kimi_schedule_reads_global_steps():
    r, m, uid, gidx = _group_case(12)
    args = {"length_coef": 1.0, "length_coef_warmup_steps": 10, "length_coef_ramp_steps": 20}
    tensors = {"token_level_rewards": r, "response_mask": m}
    for step, coef in ((0, 0.0), (15, 0.25), (40, 1.0)):
        adv, _ = _run("kimi_k1_5", tensors, args, uid=uid, meta={"global_steps": step})
        ref = OR.kimi_k1_5_advantage(r, m, gidx, length_coef=coef)
        assert torch.allclose(adv.cpu(), ref, rtol=1e-5, atol=2e-6), step
    adv, _ = _run("kimi_k1_5", tensors, args, uid=uid)  # no meta_info: step 0
    assert torch.allclose(adv.cpu(), OR.kimi_k1_5_advantage(r, m, gidx, length_coef=0.0), rtol=1e-5, atol=2e-6)


def test_identity_gpu():
    adv, ret = _run("identity", {"token_level_rewards": T([[1.0, -2.0, 3.0]]), "response_mask": T([[1.0, 1.0, 0.0]])})
    assert torch.equal(adv.cpu(), T([[1.0, -2.0, 0.0]])) and ret is adv


# ---- value loss ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("tr,br", [("sum", "token-mean"), ("mean", "step-mean"), ("mean-norm", "token-mean")])
@pytest.mark.parametrize("clip", [0.5, 0.1])
def test_value_loss_vs_oracle(tr, br, clip):
    g = torch.Generator().manual_seed(31)
    b, t = 9, 517
    values = torch.randn(b, t, generator=g)
    vpreds = values + 0.3 * torch.randn(b, t, generator=g)
    returns = values + torch.randn(b, t, generator=g)
    mask = (torch.rand(b, t, generator=g) > 0.3).float()
    mask[4] = 0
    ref_in = vpreds.clone().requires_grad_(True)
    ref_loss, ref_m = OR.value_loss(ref_in, values, returns, mask, cliprange_value=clip, token_reduce=tr,
                                    batch_reduce=br)
    ref_loss.backward()
    vp = vpreds.to(DEV).requires_grad_(True)
    data = _proto({"values": values, "returns": returns, "response_mask": mask})
    data.batch["vpreds"] = vp
    loss, m = compute_loss_fn(data, "value", {"cliprange_value": clip, "token_reduce": tr, "batch_reduce": br})
    loss.backward()
    assert loss.item() == pytest.approx(ref_loss.item(), rel=1e-4)
    assert rel_l2(vp.grad, ref_in.grad) < 1e-5
    for k in ("vf_loss", "vf_clipfrac", "vpred_mean"):
        assert m[k] == pytest.approx(ref_m[k], rel=1e-4, abs=1e-6), k


def test_value_loss_known_answers_gpu():
    values = T([[1.0, 2.0, 3.0]])
    data = _proto({"vpreds": values.clone(), "values": values, "returns": T([[2.0, 2.0, 2.0]]),
                   "response_mask": torch.ones(1, 3)})
    loss, m = compute_loss_fn(data, "value", {"cliprange_value": 10.0})
    assert loss.item() == pytest.approx(1.0 / 3.0, abs=1e-6) and m["vf_clipfrac"] == 0.0
    vp = T([[0.2, 1.0, 1.0, -3.0]]).to(DEV).requires_grad_(True)
    data = _proto({"values": torch.zeros(1, 4), "returns": T([[1.0, 0.6, 2.0, -1.0]]), "response_mask": torch.ones(1, 4)})
    data.batch["vpreds"] = vp
    loss, m = compute_loss_fn(data, "value", {"cliprange_value": 0.5})
    loss.backward()
    assert loss.item() == pytest.approx(0.5 * (0.64 + 0.16 + 2.25 + 4.0) / 4, rel=1e-6)
    assert torch.allclose(vp.grad.cpu(), T([[-0.8, 0.4, 0.0, -2.0]]) / 4, atol=1e-6)
    assert m["vf_clipfrac"] == pytest.approx(0.25)


# ---- KL-Cov / Clip-Cov -----------------------------------------------------------------------------------
from oracle import loss as OL  # noqa: E402


def _selected(keys, state, n):
    """The selection rule of the library, replayed on the host from its outputs."""
    raw = state.cpu().numpy().tobytes()
    thr, k = np.frombuffer(raw[0:4], np.uint32)[0], np.frombuffer(raw[36:40], np.uint32)[0]
    limit = np.frombuffer(raw[16:24], np.int64)[0]
    key = keys.cpu().numpy()[:n].view(np.uint32)
    idx = np.arange(n)
    hit = (key != 0) & ((key > thr) | ((key == thr) & (idx < limit)))
    return torch.from_numpy(hit if k > 0 else np.zeros(n, bool))


def _cov_batch(b=16, t=512, seed=41):
    g = torch.Generator().manual_seed(seed)
    old = -torch.empty(b, t).exponential_(1.0, generator=g)
    lp = old + 0.1 * torch.randn(b, t, generator=g)
    adv = torch.randn(b, 1, generator=g).expand(b, t).contiguous() + 0.1 * torch.randn(b, t, generator=g)
    mask = (torch.rand(b, t, generator=g) > 0.3).float()
    mask[3] = 0
    isw = torch.rand(b, t, generator=g) + 0.5
    return lp, old, adv, mask, isw


@pytest.mark.parametrize("tr,br", [("sum", "token-mean"), ("mean", "step-mean")])
@pytest.mark.parametrize("ratio,with_isw", [(0.002, False), (0.05, True)])
def test_kl_cov_vs_oracle(ratio, with_isw, tr, br):
    lp, old, adv, mask, isw = _cov_batch()
    ref_in = lp.clone().requires_grad_(True)
    ref_loss, ref_m, picked = OL.kl_cov_loss(ref_in, old, adv, mask, kl_cov_ratio=ratio, ppo_kl_coef=0.7,
                                             sampler_is_weights=isw if with_isw else None, token_reduce=tr,
                                             batch_reduce=br)
    ref_loss.backward()
    # the selected token indices, bit-exact
    rows = _ops.rows_of(lp.to(DEV))
    _, _, keys, state = _ops.cov_policy_loss(0, lp.to(DEV), old.to(DEV), adv.to(DEV), mask.to(DEV), None, rows,
                                             select_ratio=ratio, kl_coef=0.7, token_reduce=tr, batch_reduce=br)
    got = torch.nonzero(_selected(keys, state, lp.numel())).flatten()
    assert got.tolist() == sorted(picked.tolist())
    # loss, gradient and metric through the registry
    x = lp.to(DEV).requires_grad_(True)
    tensors = {"old_log_probs": old, "advantages": adv, "response_mask": mask}
    if with_isw:
        tensors["sampler_is_weights"] = isw
    data = _proto(tensors)
    data.batch["log_probs"] = x
    loss, m = compute_loss_fn(data, "kl_cov", {"kl_cov_ratio": ratio, "ppo_kl_coef": 0.7, "token_reduce": tr,
                                               "batch_reduce": br})
    loss.backward()
    assert loss.item() == pytest.approx(ref_loss.item(), rel=1e-4)
    assert rel_l2(x.grad, ref_in.grad) < 1e-5
    assert m["ppo_kl"] == pytest.approx(ref_m["ppo_kl"], rel=1e-4)


def test_kl_cov_worked_example_ties_and_errors_gpu():
    adv = T([[1.0, -1.0, 2.0, 0.0]])
    lp = T([[-1.0, -2.0, -0.5, -3.0]])
    old = lp - T([[0.1, -0.2, 0.3, 0.0]])
    data = _proto({"log_probs": lp, "old_log_probs": old, "advantages": adv, "response_mask": torch.ones(1, 4)})
    loss, m = compute_loss_fn(data, "kl_cov", {"kl_cov_ratio": 0.25, "ppo_kl_coef": 2.0})
    import math
    base = -1.0 * math.exp(0.1) + 1.0 * math.exp(-0.2) - 2.0 * math.exp(0.3)
    assert loss.item() == pytest.approx((base + 2.0 * 0.3) / 4, rel=1e-5)
    assert m["ppo_kl"] == pytest.approx(0.15, rel=1e-5)
    with pytest.raises(AssertionError, match="kl_cov_ratio must be > 0"):
        compute_loss_fn(data, "kl_cov", {"kl_cov_ratio": 0})
    # every covariance equal (constant advantage): the k lowest-index response tokens are taken
    lp2, old2, _, mask, _ = _cov_batch(4, 300, seed=43)
    adv2 = torch.full_like(lp2, 0.5)
    rows = _ops.rows_of(lp2.to(DEV))
    acc, _, keys, state = _ops.cov_policy_loss(0, lp2.to(DEV), old2.to(DEV), adv2.to(DEV), mask.to(DEV), None, rows,
                                               select_ratio=0.01, kl_coef=1.0, token_reduce="sum",
                                               batch_reduce="token-mean")
    k = max(1, int(int(mask.sum()) * 0.01))
    got = torch.nonzero(_selected(keys, state, lp2.numel())).flatten()
    assert got.tolist() == torch.nonzero(mask.flatten() > 0).flatten()[:k].tolist()
    nak = (lp2 - old2).flatten()
    per_tok = -0.5 * torch.exp(nak)
    per_tok[got] += nak[got].abs()
    assert acc[0].item() == pytest.approx(float((per_tok * mask.flatten()).sum() / mask.sum()), rel=1e-4)
    # an all-zero mask selects nothing and gives a zero loss
    acc, grad, keys, state = _ops.cov_policy_loss(0, lp2.to(DEV), old2.to(DEV), adv2.to(DEV),
                                                  torch.zeros_like(mask).to(DEV), None, rows, select_ratio=0.01,
                                                  token_reduce="sum", batch_reduce="token-mean")
    assert acc[0].item() == 0.0 and not _selected(keys, state, lp2.numel()).any() and (grad == 0).all()


@pytest.mark.parametrize("tr,br", [("mean", "token-mean"), ("sum", "step-mean")])
@pytest.mark.parametrize("ratio", [0.002, 0.5])
def test_clip_cov_vs_oracle_on_the_same_draw(ratio, tr, br):
    lp, old, adv, mask, isw = _cov_batch(seed=47)
    adv = adv * 2
    kw = dict(clip_ratio_low=0.2, clip_ratio_high=0.28, clip_cov_ratio=ratio, clip_cov_lb=0.5, clip_cov_ub=5.0)
    cand, clip_num = OL.clip_cov_candidates(lp, old, adv, mask, **kw)
    rows = _ops.rows_of(lp.to(DEV))
    draws = []
    for seed in (1, 2):
        acc, grad, keys, state = _ops.cov_policy_loss(
            1, lp.to(DEV), old.to(DEV), adv.to(DEV), mask.to(DEV), isw.to(DEV), rows, select_ratio=ratio,
            ratio_lo=1 - 0.2, ratio_hi=1 + 0.28, cov_lb=0.5, cov_ub=5.0, seed=seed, token_reduce=tr, batch_reduce=br)
        sel = _selected(keys, state, lp.numel()).view_as(cand)
        # the draw: exactly min(clip_num, candidates) tokens, every one a candidate
        assert int(sel.sum()) == min(clip_num, int(cand.sum())) and not (sel & ~cand).any()
        draws.append(sel)
        ref_in = lp.clone().requires_grad_(True)
        ref_loss, ref_m = OL.clip_cov_loss(ref_in, old, adv, mask, selected=sel, sampler_is_weights=isw,
                                           token_reduce=tr, batch_reduce=br, **kw)
        ref_loss.backward()
        sums = acc.tolist()
        assert sums[0] == pytest.approx(ref_loss.item(), rel=1e-4)
        assert rel_l2(grad * sums[5], ref_in.grad) < 1e-5
        assert sums[1] / max(sums[4], 1) == pytest.approx(ref_m["pg_clipfrac"], rel=1e-5)
        assert sums[2] / max(sums[4], 1) == pytest.approx(ref_m["ppo_kl"], rel=1e-4, abs=1e-7)
    if clip_num < int(cand.sum()):
        assert not torch.equal(draws[0], draws[1])  # another seed, another draw
    else:
        assert torch.equal(draws[0], cand)  # more wanted than there are: every candidate goes


def test_clip_cov_registry_seed_and_errors():
    lp, old, adv, mask, _ = _cov_batch(seed=49)
    data = _proto({"log_probs": lp, "old_log_probs": old, "advantages": adv * 2, "response_mask": mask})
    args = {"clip_cov_ratio": 0.01, "clip_cov_lb": 0.5}
    torch.manual_seed(5)
    l1, m1 = compute_loss_fn(data, "clip_cov", args)
    torch.manual_seed(5)
    l2, m2 = compute_loss_fn(data, "clip_cov", args)
    assert l1.item() == l2.item() and m1 == m2 and set(m1) == {"pg_clipfrac", "ppo_kl"}
    want = max(int(0.01 * float(mask.sum())), 1)
    assert m1["pg_clipfrac"] == pytest.approx(want / float(mask.sum()), rel=1e-5)
    with pytest.raises(AssertionError, match="clip_cov_ratio must be > 0"):
        compute_loss_fn(data, "clip_cov", {"clip_cov_ratio": 0})


def test_cov_losses_packed_layout():
    lens = [700, 33, 1, 1200, 64, 257]
    n = sum(lens)
    g = torch.Generator().manual_seed(53)
    old = -torch.empty(n).exponential_(1.0, generator=g)
    lp = old + 0.1 * torch.randn(n, generator=g)
    adv = torch.randn(n, generator=g)
    mask = (torch.rand(n, generator=g) > 0.2).float()
    cu = W.cu_from_lengths(lens)
    tmax = max(lens)
    pad = lambda x: torch.stack([torch.nn.functional.pad(x[s:e], (0, tmax - (e - s)))  # noqa: E731
                                 for s, e in zip(cu[:-1].tolist(), cu[1:].tolist())])
    ref_loss, ref_m, _ = OL.kl_cov_loss(pad(lp), pad(old), pad(adv), pad(mask), kl_cov_ratio=0.01,
                                        token_reduce="mean", batch_reduce="step-mean")
    data = _proto({"log_probs": lp, "old_log_probs": old, "advantages": adv, "response_mask": mask},
                  meta={"cu_seqlens": cu})
    loss, m = compute_loss_fn(data, "kl_cov", {"kl_cov_ratio": 0.01, "token_reduce": "mean",
                                               "batch_reduce": "step-mean"})
    assert loss.item() == pytest.approx(ref_loss.item(), rel=1e-4)
    assert m["ppo_kl"] == pytest.approx(ref_m["ppo_kl"], rel=1e-4)


def test_masked_moment_helpers():
    from axon_amd.utils.rl.advantage import masked_mean, masked_var, masked_whiten
    g = torch.Generator().manual_seed(17)
    x = torch.randn(6, 301, generator=g) * 2 + 1
    m = (torch.rand(6, 301, generator=g) > 0.5).float()
    xd, md = x.to(DEV), m.to(DEV)
    assert masked_mean(xd, md).item() == pytest.approx(float(OL.masked_mean(x, m)), rel=1e-5)
    assert masked_var(xd, md).item() == pytest.approx(float(OR.masked_var(x, m)), rel=1e-5)
    assert masked_var(xd, md, False).item() == pytest.approx(float(OR.masked_var(x, m, False)), rel=1e-5)
    assert torch.allclose(masked_whiten(xd, md).cpu(), OR.masked_whiten(x, m), rtol=2e-5, atol=2e-5)
    assert torch.allclose(masked_whiten(xd, md, shift_mean=False).cpu(), OR.masked_whiten(x, m, False), rtol=2e-5,
                          atol=2e-5)
    assert float(masked_var(T([1.0, 3.0]).to(DEV), T([1.0, 1.0]).to(DEV))) == pytest.approx(2.0)
