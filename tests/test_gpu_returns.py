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
