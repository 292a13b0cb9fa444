"""GPU parity: stage 2 (sampler correction) and stage 3 (GRPO advantage, PPO/GSPO loss,
agg_loss) through the product API (ctypes -> libaxon_amd.so) against the CPU oracle.

Tolerances: masks / kept-row indices bit-exact; loss 1e-4 relative; gradients and fp32
per-token outputs 1e-5 relative-L2 (fp32 elementwise work)."""

import math

import numpy as np
import pytest
import torch

from axon_amd import _lib, _ops, workloads as W
from axon_amd.protocol import DataProto
from axon_amd.trainer.algos.advantages import compute_advantage
from axon_amd.trainer.algos.loss import agg_loss, compute_loss_fn, masked_mean
from axon_amd.utils.rl import sampler as S
from axon_amd.utils.rl.advantage import group_mean_std
from axon_amd.utils.rl.utils import filter_zero_advantage_samples
from oracle import advantage as OA
from oracle import loss as OL
from oracle import sampler as OS

pytestmark = pytest.mark.gpu
T = torch.tensor
DEV = "cuda"


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def pad_to_packed(x, lens):
    return torch.cat([x[b, :l] for b, l in enumerate(lens)])


# ---- (b) row statistics --------------------------------------------------------------------------
@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.int64, torch.bool])
def test_row_stats_ragged_vs_torch(mask_dtype):
    g = torch.Generator().manual_seed(0)
    lens = [1, 3, 64, 65, 255, 256, 257, 1023, 4100, 2, 5000, 7]
    n = sum(lens)
    cu = W.cu_from_lengths(lens)
    a, b = torch.randn(n, generator=g), torch.randn(n, generator=g)
    mask = (torch.rand(n, generator=g) > 0.3).to(mask_dtype)
    rows = _ops.rows_of(a.to(DEV), cu.to(DEV))
    cnt, ssum, flag = _ops.row_stats(a.to(DEV), b.to(DEV), mask.to(DEV), rows, flag_mode=1, threshold=-2.5)
    mf = mask.float()
    for r, (s, e) in enumerate(zip(cu[:-1].tolist(), cu[1:].tolist())):
        assert cnt[r].item() == mf[s:e].sum().item()
        assert ssum[r].item() == pytest.approx(((a - b)[s:e] * mf[s:e]).double().sum().item(), abs=1e-3)
        assert bool(flag[r].item()) == bool((((a - b)[s:e] < -2.5) & (mf[s:e] != 0)).any())


def test_row_stats_empty_rows_and_uniform_layout():
    cu = T([0, 0, 5, 5, 5, 9, 9], dtype=torch.int32)
    x = torch.arange(9, dtype=torch.float32)
    rows = _ops.rows_of(x.to(DEV), cu.to(DEV))
    cnt, ssum, _ = _ops.row_stats(x.to(DEV), None, None, rows)
    assert cnt.tolist() == [0, 5, 0, 0, 4, 0] and ssum.tolist() == [0, 10, 0, 0, 26, 0]
    y = torch.randn(7, 333)
    rows2 = _ops.rows_of(y.to(DEV))
    _, s2, _ = _ops.row_stats(y.to(DEV), None, None, rows2)
    assert torch.allclose(s2.cpu(), y.sum(-1), atol=1e-4)


# ---- group_mean_std / GRPO / dynamic sampling (known answers through the HIP path) --------------
def test_group_mean_std_known_answers_gpu():
    m, s, c = group_mean_std(T([1.0, 2, 3], device=DEV), T([0, 0, 0], device=DEV))
    assert s.item() == pytest.approx(1.0) and m.item() == pytest.approx(2.0)
    _, s, _ = group_mean_std(T([1.0, 3, 2, 4], device=DEV), T([0, 0, 1, 1], device=DEV))
    assert torch.allclose(s.cpu(), torch.full((2,), math.sqrt(2.0)))
    m, s, c = group_mean_std(T([5.0], device=DEV), T([0], device=DEV))
    assert (m.item(), s.item(), c.item()) == (0.0, 1.0, 1.0)
    m, s, c = group_mean_std(T([10.0, 20], device=DEV), T([0, 5], device=DEV))
    assert c.tolist() == [1, 0, 0, 0, 0, 1] and (m == 0).all()
    m, s, _ = group_mean_std(T([5.0, 5, 5], device=DEV), T([0, 0, 0], device=DEV))
    assert m.item() == pytest.approx(5.0) and s.item() == pytest.approx(math.sqrt(1e-6))


def _grpo_proto(tlr, mask, uid, dev=DEV, meta=None):
    d = DataProto.from_dict(tensors={"token_level_rewards": tlr.to(dev), "response_mask": mask.to(dev)},
                            meta_info=meta or {})
    d.non_tensor_batch["uid"] = uid  # per row; in the packed layout rows are sequences, tensors are per token
    return d


@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.int64])
def test_grpo_config1_vs_oracle(norm, mask_dtype):
    d = W.c1_loss_only()
    data = _grpo_proto(d["token_level_rewards"], d["response_mask"].to(mask_dtype), d["uid"])
    cfg = {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6, "norm_adv_by_std": norm}}
    out = compute_advantage(data, cfg)
    gidx = T(np.unique(d["uid"], return_inverse=True)[1])
    ref = OA.grpo_advantage(d["token_level_rewards"], d["response_mask"], gidx, 1e-6, norm)
    assert out.batch["advantages"].shape == ref.shape
    assert torch.allclose(out.batch["advantages"].cpu(), ref, rtol=1e-5, atol=1e-6)
    assert out.batch["returns"] is out.batch["advantages"]
    clipped = compute_advantage(data, {"advantage": "grpo", "advantage_args": {"clip_advantages": True}})
    assert clipped.batch["advantages"].abs().max() <= 1.0


def test_grpo_known_answers_and_cpu_staging():
    rew = T([[0.0, 0, 2], [0, 0, 0]])
    data = _grpo_proto(rew, torch.ones(2, 3), np.array(["a", "a"], dtype=object), dev="cpu")
    out = compute_advantage(data, {"advantage": "grpo", "advantage_args": {"norm_adv_by_std": False}})
    adv = out.batch["advantages"]
    assert adv.device.type == "cpu"  # driver-side tensors come back where they lived
    assert torch.equal(adv[0], torch.ones(3)) and torch.equal(adv[1], -torch.ones(3))
    single = _grpo_proto(rew, torch.ones(2, 3), np.array(["a", "b"], dtype=object))
    assert (compute_advantage(single, {"advantage": "grpo"}).batch["advantages"] == 0).all()


def test_grpo_packed_layout():
    d = W.packed_rl_inputs(5000, seed=9, lengths=[700, 33, 1200, 64, 2000, 1003])
    data = _grpo_proto(d["token_level_rewards"], d["response_mask"], W.uids_for(6, 3),
                       meta={"cu_seqlens": d["cu_seqlens"]})
    out = compute_advantage(data, {"advantage": "grpo"}).batch["advantages"].cpu()
    # oracle on the padded equivalent
    tmax = max(d["lengths"])
    pad_r, pad_m = torch.zeros(6, tmax), torch.zeros(6, tmax)
    for b, (s, e) in enumerate(zip(d["cu_seqlens"][:-1].tolist(), d["cu_seqlens"][1:].tolist())):
        pad_r[b, : e - s] = d["token_level_rewards"][s:e]
        pad_m[b, : e - s] = d["response_mask"][s:e]
    ref = OA.grpo_advantage(pad_r, pad_m, T([0, 0, 0, 1, 1, 1]))
    assert torch.allclose(out, pad_to_packed(ref, d["lengths"]), rtol=1e-5, atol=1e-6)


def test_filter_zero_advantage_known_answers_gpu():
    def proto(adv, uid=None):
        nt = {"uid": np.array(uid, dtype=object)} if uid else {}
        return DataProto.from_dict(tensors={"advantages": adv.to(DEV), "other": torch.arange(adv.shape[0]).to(DEV)},
                                   non_tensors=nt)
    out = filter_zero_advantage_samples(proto(T([[1.0, 2], [0, 0], [5, 6]])))
    assert len(out) == 2 and out.batch["other"].tolist() == [0, 2]
    assert len(filter_zero_advantage_samples(proto(T([[0.0, 0], [0, 0]])))) == 2  # no uid: unchanged
    out = filter_zero_advantage_samples(proto(T([[1e-7, 1e-8], [1e-5, 0], [0.0, -1.0]]), ["a", "a", "b"]))
    assert out.batch["other"].tolist() == [2]
    out = filter_zero_advantage_samples(proto(T([[0.0, 0], [0, 0], [0, 0]]), ["a", "b", "a"]))
    assert out.batch["other"].tolist() == [0, 2]  # all zero: keep the first uid's group
    with pytest.raises(AssertionError):
        filter_zero_advantage_samples(DataProto.from_dict(tensors={"x": torch.zeros(2, 2).to(DEV)}))
    d = W.c1_loss_only(seed=5)
    gidx = T(np.unique(d["uid"], return_inverse=True)[1])
    adv = OA.grpo_advantage(d["token_level_rewards"], d["response_mask"], gidx)
    kept = filter_zero_advantage_samples(proto(adv)).batch["other"].tolist()
    assert kept == OA.zero_advantage_keep_rows(adv)  # indices bit-exact


# ---- process_mini_batch (reference tests/driver/test_driver_utils.py:260-281) -------------------
@pytest.mark.parametrize("mask_dtype", [torch.int64, torch.float32, torch.bool])
@pytest.mark.parametrize("where", ["cpu", "gpu"])
def test_process_mini_batch(mask_dtype, where):
    from axon_amd.driver.driver_utils import process_mini_batch
    dev = DEV if where == "gpu" else "cpu"
    mask = T([[1, 1, 0], [1, 0, 0], [0, 0, 0]]).to(mask_dtype).to(dev)
    batch = DataProto.from_dict(
        tensors={"response_mask": mask},
        non_tensors={"program_uids": np.array(["program-a", "program-a", "program-padding"], dtype=object)})
    process_mini_batch(batch)
    assert batch.batch["valid_batch_size"].tolist() == [2, 2, 2]
    assert batch.batch["valid_token_count"].tolist() == [3, 3, 3]
    assert batch.batch["valid_program_count"].tolist() == [1, 1, 1]
    assert batch.batch["per_row_token_count"].tolist() == [2, 1, 0]
    for k in ("valid_batch_size", "valid_token_count", "per_row_token_count"):
        assert batch.batch[k].dtype == torch.long and batch.batch[k].device.type == mask.device.type
    # no mask: untouched; a seeded ragged batch against the oracle
    empty = DataProto.from_dict(tensors={"x": torch.zeros(2, 2)})
    process_mini_batch(empty)
    assert "valid_batch_size" not in empty.batch
    d = W.c1_loss_only(seed=9)
    m = d["response_mask"].clone()
    m[3] = 0
    b2 = DataProto.from_dict(tensors={"response_mask": m.to(mask_dtype).to(dev)})
    process_mini_batch(b2)
    rows, tokens, per_row, _ = OA.mini_batch_counts(m)
    assert b2.batch["valid_batch_size"][0].item() == rows and b2.batch["valid_token_count"][-1].item() == tokens
    assert torch.equal(b2.batch["per_row_token_count"].cpu(), per_row)
    assert "valid_program_count" not in b2.batch


# ---- agg_loss / masked_mean known answers through the HIP path --------------------------------
from tests.test_oracle_loss import AGG_CASES  # noqa: E402  (same table the oracle is pinned with)


@pytest.mark.parametrize("loss,mask,tr,br,kw,expect", AGG_CASES)
def test_agg_loss_known_answers_gpu(loss, mask, tr, br, kw, expect):
    kw = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    out = agg_loss(T(loss, dtype=torch.float32, device=DEV), T(mask, dtype=torch.float32, device=DEV),
                   token_reduce=tr, batch_reduce=br, **kw)
    assert out.dim() == 0 and out.item() == pytest.approx(expect, rel=1e-6)


def test_masked_mean_gpu_with_grad():
    v = T([1.0, 2, 3], device=DEV, requires_grad=True)
    out = masked_mean(v, T([1.0, 1, 0], device=DEV))
    out.backward()
    assert out.item() == pytest.approx(1.5) and torch.allclose(v.grad.cpu(), T([0.5, 0.5, 0.0]))
    assert masked_mean(T([1.0, 2], device=DEV), T([0.0, 0], device=DEV)).item() == 0.0


# ---- PPO / GSPO --------------------------------------------------------------------------------
def _loss_proto(d, keys=("log_probs", "old_log_probs", "advantages", "response_mask"), extra=None, meta=None):
    t = {k: d[k].to(DEV) for k in keys}
    t.update({k: v.to(DEV) for k, v in (extra or {}).items()})
    t["log_probs"] = t["log_probs"].clone().requires_grad_(True)
    return DataProto.from_dict(tensors=t, meta_info=meta or {})


def _check_loss(name, oracle_fn, d, cfg, extra=None, agg=None, meta=None, pad=None):
    data = _loss_proto(d, extra=extra, meta=meta)
    loss, metrics = compute_loss_fn(data, name, cfg)
    loss.backward()
    src = pad if pad is not None else d
    lp = src["log_probs"].clone().requires_grad_(True)
    okw = {k: v for k, v in cfg.items() if k.startswith("clip") or k.endswith("_reduce")}
    ex = {k: v for k, v in (src.get("_extra") or extra or {}).items()}
    ref, ref_m = oracle_fn(lp, src["old_log_probs"], src["advantages"], src["response_mask"].float(), **okw, **ex,
                           **(agg or {}))
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4, abs=1e-9)
    got_g = data.batch["log_probs"].grad.cpu()
    ref_g = lp.grad if pad is None else pad_to_packed(lp.grad, d["lengths"])
    assert rel_l2(got_g, ref_g) < 1e-5
    for k in ("pg_clipfrac", "ppo_kl", "pg_clipfrac_lower"):
        assert metrics[k] == pytest.approx(ref_m[k], rel=1e-4, abs=1e-7)
    return loss


def _c1_with_adv(seed=1, mask_dtype=torch.float32):
    d = W.c1_loss_only(seed)
    gidx = T(np.unique(d["uid"], return_inverse=True)[1])
    d["advantages"] = OA.grpo_advantage(d["token_level_rewards"], d["response_mask"], gidx)
    d["response_mask"] = d["response_mask"].to(mask_dtype)
    return d


@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.int64])
def test_ppo_config1_vs_oracle(mask_dtype):
    _check_loss("ppo", OL.ppo_loss, _c1_with_adv(1, mask_dtype),
                {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "token_reduce": "sum", "batch_reduce": "token-mean"})


@pytest.fixture(params=["one_launch", "two_pass"])
def row_path(request):
    """Operators with a per-row quantity have two implementations, chosen by batch size: run the test on both."""
    keep = _ops.OWNED_ROWS_MAX_SLOTS, _ops.OWNED_ROWS_MIN_MEAN_LEN
    _ops.OWNED_ROWS_MAX_SLOTS = keep[0] if request.param == "one_launch" else 0
    _ops.OWNED_ROWS_MIN_MEAN_LEN = 0  # rows of any length, also the short ones the dispatch would send elsewhere
    yield request.param
    _ops.OWNED_ROWS_MAX_SLOTS, _ops.OWNED_ROWS_MIN_MEAN_LEN = keep


@pytest.mark.parametrize("tr,br", [("sum", "token-mean"), ("mean", "step-mean"), ("sum", "step-mean"),
                                   ("mean-norm", "step-mean"), ("mean", "token-mean")])
@pytest.mark.parametrize("name,fn", [("ppo", OL.ppo_loss), ("gspo", OL.gspo_loss)])
def test_losses_all_reductions_with_is_weights(name, fn, tr, br, row_path):
    d = _c1_with_adv(2)
    d["log_probs"] = d["old_log_probs"] + 0.3 * torch.randn(d["old_log_probs"].shape)  # exercise every clip region
    d["advantages"] = d["advantages"] + 0.0
    d["response_mask"][5] = 0  # a row without tokens
    isw = torch.rand(d["old_log_probs"].shape) * 2
    cfg = {"clip_ratio": 0.2, "clip_ratio_c": 3.0, "token_reduce": tr, "batch_reduce": br}
    if name == "gspo":
        cfg.pop("clip_ratio_c")
        cfg.update(clip_ratio_low=3e-4, clip_ratio_high=4e-4)
    _check_loss(name, fn, d, cfg, extra={"sampler_is_weights": isw})


def test_losses_with_global_counts_and_program_modes(row_path):
    d = _c1_with_adv(3)
    b = d["old_log_probs"].shape[0]
    agg = {"valid_token_count": torch.full((b,), 70000), "per_row_token_count": d["response_mask"].sum(-1).long() + 3}
    _check_loss("ppo", OL.ppo_loss, d, {"token_reduce": "mean", "batch_reduce": "token-mean"}, extra=agg, agg={})
    prog = {"num_program_steps": torch.randint(1, 4, (b,)), "num_program_tokens": torch.randint(500, 3000, (b,)),
            "valid_program_count": torch.full((b,), 40)}
    _check_loss("ppo", OL.ppo_loss, d, {"token_reduce": "mean-program", "batch_reduce": "program-mean"}, extra=prog)
    _check_loss("gspo", OL.gspo_loss, d, {"token_reduce": "mean", "batch_reduce": "step-mean"},
                extra={"valid_batch_size": torch.full((b,), 256)})


def test_ppo_known_answers_gpu():
    # reference tests/trainer/algos/loss/test_loss.py:63-87, 670-714
    lp = T([[-1.0, -2.0, -3.0]], device=DEV)
    data = DataProto.from_dict(tensors={"log_probs": lp.clone().requires_grad_(True), "old_log_probs": lp,
                                        "advantages": T([[1.0, 2, 3]], device=DEV),
                                        "response_mask": torch.ones(1, 3, device=DEV)})
    loss, m = compute_loss_fn(data, "ppo", {"clip_ratio": 0.2})
    assert loss.item() == pytest.approx(-2.0) and m["pg_clipfrac"] == 0.0 and m["ppo_kl"] == 0.0
    data.batch["advantages"] = torch.zeros(1, 3, device=DEV)
    assert compute_loss_fn(data, "ppo", {})[0].item() == 0.0
    data.batch["advantages"] = T([[1.0, float("nan"), 3.0]], device=DEV)
    assert math.isnan(compute_loss_fn(data, "ppo", {})[0].item())
    data.batch["advantages"] = torch.ones(1, 3, device=DEV)
    data.batch["log_probs"] = lp + 100.0
    assert math.isfinite(compute_loss_fn(data, "ppo", {})[0].item())
    loss, m = compute_loss_fn(data, "gspo", {})
    assert math.isfinite(loss.item()) and m["pg_clipfrac_lower"] == 0.0


def test_ppo_clip_regions_table_gpu():
    from tests.test_oracle_loss import REGIONS, _ppo_token_scalar
    lo, hi, c = 0.2, 0.28, 3.0
    dlt = T([[x for x, _ in REGIONS]])
    adv = T([[a for _, a in REGIONS]])
    old = torch.full_like(dlt, -1.0)
    data = DataProto.from_dict(tensors={"log_probs": (old + dlt).to(DEV).requires_grad_(True),
                                        "old_log_probs": old.to(DEV), "advantages": adv.to(DEV),
                                        "response_mask": torch.ones_like(dlt).to(DEV)})
    loss, _ = compute_loss_fn(data, "ppo", {"clip_ratio_low": lo, "clip_ratio_high": hi, "clip_ratio_c": c})
    loss.backward()
    n = len(REGIONS)
    for k, (x, a) in enumerate(REGIONS):
        xs = float(T(-1.0 + x, dtype=torch.float32) - T(-1.0))  # the fp32 difference the kernel sees
        _, g = _ppo_token_scalar(-1.0 + xs, -1.0, a, lo, hi, c)
        assert data.batch["log_probs"].grad[0, k].item() == pytest.approx(g / n, rel=1e-5, abs=1e-9), REGIONS[k]


@pytest.mark.parametrize("n_tokens", [20000, 65536])  # 65536 is the full size of the configuration
def test_gspo_packed_config4_vs_oracle(n_tokens, row_path):
    d = W.c4_correction(n_tokens=n_tokens)
    s = len(d["lengths"])
    gidx = T(np.unique(d["uid"], return_inverse=True)[1])
    tmax = max(d["lengths"])
    pad = {k: torch.zeros(s, tmax) for k in ("log_probs", "old_log_probs", "response_mask", "token_level_rewards")}
    for b, (st, en) in enumerate(zip(d["cu_seqlens"][:-1].tolist(), d["cu_seqlens"][1:].tolist())):
        for k in pad:
            pad[k][b, : en - st] = d[k][st:en]
    pad["advantages"] = OA.grpo_advantage(pad["token_level_rewards"], pad["response_mask"], gidx)
    d["advantages"] = pad_to_packed(pad["advantages"], d["lengths"])
    cfg = {"clip_ratio_low": 3e-4, "clip_ratio_high": 4e-4, "token_reduce": "mean", "batch_reduce": "step-mean"}
    _check_loss("gspo", OL.gspo_loss, d, cfg, meta={"cu_seqlens": d["cu_seqlens"]}, pad=pad)
    _check_loss("ppo", OL.ppo_loss, d, {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28},
                meta={"cu_seqlens": d["cu_seqlens"]}, pad=pad)


# ---- stage 2: sampler correction -------------------------------------------------------------------
def _pad_case(seed=4, b=32, t=700):
    g = torch.Generator().manual_seed(seed)
    old = -torch.empty(b, t).exponential_(1.0, generator=g)
    samp = old + 0.3 * torch.randn(b, t, generator=g)
    samp[3, 17] = old[3, 17] + 11.0
    samp[9, 0] = old[9, 0] + 30.0
    lens = torch.randint(1, t + 1, (b,), generator=g)
    mask = (torch.arange(t)[None] < lens[:, None]).float()
    mask[7] = 0
    return old, samp, mask


@pytest.mark.parametrize("is_l,rs_l", [("token", "token"), ("sequence", "sequence"), ("token", "geometric"),
                                       (None, "token"), ("token", None), (None, None)])
@pytest.mark.parametrize("mask_dtype", [torch.float32, torch.int64])
def test_sampler_correction_vs_oracle(is_l, rs_l, mask_dtype, row_path):
    old, samp, mask = _pad_case()
    kw = dict(sampler_is=is_l, sampler_is_threshold=2.0, sampler_rs=rs_l, sampler_rs_threshold=2.0,
              sampler_token_veto_threshold=1e-4)
    proto, new, m = S.compute_sampler_correction_and_rejection_mask(old.to(DEV), samp.to(DEV),
                                                                    mask.to(mask_dtype).to(DEV), **kw)
    w_ref, new_ref, m_ref = OS.correction(old, samp, mask, **kw)
    if rs_l in (None, "token"):
        assert torch.equal(new.cpu(), new_ref)  # bit-exact
    else:  # row-level ratios depend on summation order: allow rows that sit on the threshold
        diff_rows = (new.cpu() != new_ref).any(-1).sum().item()
        assert diff_rows == 0
    assert new.dtype == torch.float32
    if is_l is None:
        assert proto is None
    else:
        w = proto.batch["sampler_is_weights"]
        assert not w.requires_grad and rel_l2(w, w_ref) < 1e-5 and (w.cpu()[mask == 0] == 0).all()
    for k, v in m_ref.items():
        assert m["sampler_corr/" + k] == pytest.approx(v, rel=1e-4, abs=1e-7), k
    assert all(k.startswith("sampler_corr/") for k in m)


def test_sampler_masks_bit_exact_at_the_thresholds():
    """Tokens whose log-ratio sits within a few ulps of +-ln 2 and of ln(1e-4)."""
    centres = [math.log(2.0), -math.log(2.0), math.log(1e-4)]
    vals = []
    for c in centres:
        x = T(c, dtype=torch.float32)
        up, dn = x.clone(), x.clone()
        vals.append(x.clone())
        for _ in range(20):
            up = torch.nextafter(up, T(math.inf))
            dn = torch.nextafter(dn, T(-math.inf))
            vals += [up.clone(), dn.clone()]
    lr = torch.stack(vals).repeat(40)  # long enough for the oracle's exp to take the vector path
    n = lr.numel()
    lr = lr[: n - n % 8].view(8, -1)
    old, samp, mask = lr.clone(), torch.zeros_like(lr), torch.ones_like(lr)
    for veto in (None, 1e-4):
        kw = dict(sampler_rs="token", sampler_rs_threshold=2.0, sampler_token_veto_threshold=veto)
        _, new, _ = S.compute_sampler_correction_and_rejection_mask(old.to(DEV), samp.to(DEV), mask.to(DEV), **kw)
        _, ref, _ = OS.correction(old, samp, mask, **kw)
        assert torch.equal(new.cpu(), ref)
    # per-row veto flags at the boundary, one token per row
    col = torch.stack(vals)[:, None]
    _, new, _ = S.compute_sampler_correction_and_rejection_mask(col.to(DEV), torch.zeros_like(col).to(DEV),
                                                                torch.ones_like(col).to(DEV),
                                                                sampler_token_veto_threshold=1e-4)
    _, ref, _ = OS.correction(col, torch.zeros_like(col), torch.ones_like(col), sampler_token_veto_threshold=1e-4)
    assert torch.equal(new.cpu(), ref)


def test_sampler_known_answers_gpu():
    # reference tests/utils/test_rl_sampler.py:199-298
    z, one = torch.zeros(2, 4, device=DEV), torch.ones(2, 4, device=DEV)
    proto, new, m = S.compute_sampler_correction_and_rejection_mask(z, z, one, sampler_is="token")
    assert proto is not None and torch.equal(new, one) and torch.equal(proto.batch["sampler_is_weights"], one)
    assert m["sampler_corr/sampler_is_mean"] == pytest.approx(1.0)
    proto, new, _ = S.compute_sampler_correction_and_rejection_mask(z, z, one, sampler_rs="token",
                                                                    sampler_rs_threshold=2.0)
    assert proto is None and torch.equal(new, one)
    proto, new, _ = S.compute_sampler_correction_and_rejection_mask(z, z, one)
    assert proto is None and torch.equal(new, one)
    old = z.clone()
    old[0, 1] = -10.0
    _, new, m = S.compute_sampler_correction_and_rejection_mask(old, z, one, sampler_token_veto_threshold=0.01)
    assert new[0].sum() == 0 and new[1].sum() == 4 and m["sampler_corr/sampler_is_veto_fraction"] == 0.5
    proto, new, m = S.compute_sampler_correction_and_rejection_mask(z, z, z, sampler_is="token", sampler_rs="token")
    assert proto is None and new is z and m == {}
    big = T([[70.0, -70.0]], device=DEV)
    w, _ = S.compute_sampler_correction_weights(big, torch.ones(1, 2, device=DEV), "token", 1e12)
    assert torch.isfinite(w).all() and w[0, 0].item() == pytest.approx(math.exp(20), rel=1e-4)
    keep, mm = S.compute_sampler_rejection_mask(torch.full((2, 4), 10.0, device=DEV), one, "token", 2.0)
    assert keep.sum() == 0 and mm["sampler_rs_masked_fraction"] == pytest.approx(1.0)


def test_correction_hook_in_compute_loss_fn_and_mask_side_effect():
    d = _c1_with_adv(6)
    samp = d["old_log_probs"] + 0.2 * torch.randn(d["old_log_probs"].shape)
    data = _loss_proto(d, extra={"sampler_log_probs": samp})
    args = {"sampler_is": "token", "sampler_is_threshold": 2.0, "sampler_rs": "token", "sampler_rs_threshold": 2.0,
            "sampler_token_veto_threshold": 1e-4, "clip_ratio_low": 0.2, "clip_ratio_high": 0.28}
    loss, metrics = compute_loss_fn(data, "ppo", args)
    loss.backward()
    w, new_mask, _ = OS.correction(d["old_log_probs"], samp, d["response_mask"], sampler_is="token",
                                   sampler_rs="token", sampler_token_veto_threshold=1e-4)
    assert torch.equal(data.batch["response_mask"].cpu(), new_mask)  # the batch's mask is overwritten
    lp = d["log_probs"].clone().requires_grad_(True)
    ref, _ = OL.ppo_loss(lp, d["old_log_probs"], d["advantages"], new_mask, clip_ratio_low=0.2, clip_ratio_high=0.28,
                         sampler_is_weights=w)
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4)
    assert rel_l2(data.batch["log_probs"].grad, lp.grad) < 1e-5
    assert "sampler_corr/sampler_is_mean" in metrics and "pg_clipfrac" in metrics


def test_config4_full_size_masks_bit_exact():
    d = W.c4_correction()
    kw = dict(sampler_is="token", sampler_is_threshold=2.0, sampler_rs="token", sampler_rs_threshold=2.0,
              sampler_token_veto_threshold=1e-4)
    proto, new, m = S.compute_sampler_correction_and_rejection_mask(
        d["old_log_probs"].to(DEV), d["sampler_log_probs"].to(DEV), d["response_mask"].to(DEV),
        cu_seqlens=d["cu_seqlens"].to(DEV), **kw)
    s = len(d["lengths"])
    tmax = max(d["lengths"])
    pad = {k: torch.zeros(s, tmax) for k in ("old_log_probs", "sampler_log_probs", "response_mask")}
    for b, (st, en) in enumerate(zip(d["cu_seqlens"][:-1].tolist(), d["cu_seqlens"][1:].tolist())):
        for k in pad:
            pad[k][b, : en - st] = d[k][st:en]
    w_ref, new_ref, m_ref = OS.correction(pad["old_log_probs"], pad["sampler_log_probs"], pad["response_mask"], **kw)
    assert torch.equal(new.cpu(), pad_to_packed(new_ref, d["lengths"]))
    assert rel_l2(proto.batch["sampler_is_weights"], pad_to_packed(w_ref, d["lengths"])) < 1e-5
    assert m["sampler_corr/sampler_is_veto_fraction"] == pytest.approx(m_ref["sampler_is_veto_fraction"])


# ---- diagnostics: every sampler_is_* / sampler_rs_* metric, off-policy and mismatch statistics ----
def _assert_metrics(got, ref, prefix="", rel=2e-4, abs_=2e-6):
    for k, v in ref.items():
        g = got[prefix + k]
        if math.isinf(v):
            assert math.isinf(g) and (g > 0) == (v > 0), k
        else:
            # variances are differences of fp32 second moments close to 1 (in the reference too):
            # their square roots agree to ~1e-5 absolute, not 1e-4 relative
            tol_abs = 5e-5 if k.endswith("std") else abs_
            assert g == pytest.approx(v, rel=rel, abs=tol_abs), (k, g, v)


@pytest.mark.parametrize("is_l,rs_l", [("token", "token"), ("sequence", "sequence"), ("token", "geometric"),
                                       ("sequence", "token"), (None, "geometric"), ("token", None)])
def test_sampler_full_metrics_vs_oracle(is_l, rs_l):
    old, samp, mask = _pad_case(seed=9, b=24, t=300)
    samp = old + 0.02 * (samp - old)  # keep row sums inside the +-20 clamp for most rows
    samp[3, 17] = old[3, 17] + 3.0
    kw = dict(sampler_is=is_l, sampler_is_threshold=2.0, sampler_rs=rs_l, sampler_rs_threshold=1.5,
              sampler_rs_threshold_lower=0.6)
    _, _, m = S.compute_sampler_correction_and_rejection_mask(old.to(DEV), samp.to(DEV), mask.to(DEV), **kw)
    ref = OS.full_metrics(old, samp, mask, **kw)
    assert set(ref) <= {k[len("sampler_corr/"):] for k in m}
    assert set(m) == {"sampler_corr/" + k for k in ref} | {"sampler_corr/sampler_is_veto_fraction",
                                                            "sampler_corr/sampler_is_catastrophic_token_fraction"}
    _assert_metrics(m, ref, "sampler_corr/")


def test_sampler_full_metrics_packed_layout_matches_padded():
    old, samp, mask = _pad_case(seed=10, b=16, t=200)
    samp = old + 0.05 * (samp - old)
    lens = mask.sum(-1).long().clamp(min=1).tolist()
    cu = W.cu_from_lengths(lens)
    pk = lambda x: pad_to_packed(x, lens)  # noqa: E731
    kw = dict(sampler_is="sequence", sampler_is_threshold=2.0, sampler_rs="geometric", sampler_rs_threshold=1.2)
    _, _, mp = S.compute_sampler_correction_and_rejection_mask(pk(old).to(DEV), pk(samp).to(DEV), pk(mask).to(DEV),
                                                               cu_seqlens=cu.to(DEV), **kw)
    ref = OS.full_metrics(old, samp, mask, **kw)
    _assert_metrics(mp, ref, "sampler_corr/")


def test_offpolicy_metrics_gpu():
    old, samp, mask = _pad_case(seed=11, b=20, t=150)
    samp = old + 0.03 * (samp - old)
    got = S.compute_offpolicy_metrics(old.to(DEV), samp.to(DEV), mask.to(DEV))
    ref = OS.offpolicy_metrics(old, samp, mask)
    assert set(got) == set(ref) and len(got) == 13
    _assert_metrics(got, ref)
    # known answers of the reference's tests
    o2, s2 = T([[-1.5, -2.5]]), T([[-1.0, -2.0]])
    assert S.compute_offpolicy_metrics(o2.to(DEV), s2.to(DEV), torch.ones(1, 2).to(DEV))["kl"] == pytest.approx(0.5)
    same = S.compute_offpolicy_metrics(o2.to(DEV), o2.to(DEV), torch.ones(1, 2).to(DEV))
    assert same["kl"] == 0 and same["k3_kl"] == 0 and same["chi2_token"] == pytest.approx(0, abs=1e-7)
    assert same["ppl_ratio"] == pytest.approx(1.0)
    assert S.compute_offpolicy_metrics(o2.to(DEV), s2.to(DEV), torch.zeros(1, 2).to(DEV)) == {}
    only = S.compute_offpolicy_metrics(o2.to(DEV), None, torch.ones(1, 2).to(DEV))
    assert set(only) == {"training_ppl", "training_log_ppl"} and only["training_log_ppl"] == pytest.approx(2.0)


def test_mismatch_metrics_gpu_and_aggregation():
    from axon_amd.utils.metrics import aggregate_trainer_sampler_metrics, compute_trainer_sampler_mismatch_metrics
    old, samp, mask = _pad_case(seed=12, b=10, t=90)
    samp = old + 0.05 * (samp - old)
    halves = []
    for sl in (slice(0, 5), slice(5, 10)):
        data = DataProto.from_dict(tensors={"old_log_probs": old[sl].to(DEV), "sampler_log_probs": samp[sl].to(DEV),
                                            "response_mask": mask[sl].to(torch.int64).to(DEV)})
        got = compute_trainer_sampler_mismatch_metrics(data)
        ref = OS.mismatch_stats(old[sl], samp[sl], mask[sl])
        assert set(got) == set(ref)
        _assert_metrics(got, ref)
        halves.append(got)
    agg = aggregate_trainer_sampler_metrics(halves)
    mb = mask.bool()
    dp = (old.exp() - samp.exp()).abs()[mb]
    dl = (old - samp).abs()[mb]
    assert agg["batch/sampler_probs_diff_mean"] == pytest.approx(dp.mean().item(), rel=1e-4)
    assert agg["batch/sampler_probs_diff_std"] == pytest.approx(dp.std(unbiased=False).item(), rel=1e-3)
    assert agg["batch/sampler_logprobs_diff_max"] == pytest.approx(dl.max().item(), rel=1e-6)
    pear = torch.corrcoef(torch.stack([old.exp()[mb], samp.exp()[mb]]))[0, 1].item()
    assert agg["batch/sampler_actor_probs_pearson_corr"] == pytest.approx(pear, rel=1e-3)
    assert aggregate_trainer_sampler_metrics([]) == {}
    empty = DataProto.from_dict(tensors={"old_log_probs": old[:2].to(DEV), "sampler_log_probs": samp[:2].to(DEV),
                                         "response_mask": torch.zeros(2, 90).to(DEV)})
    z = aggregate_trainer_sampler_metrics([compute_trainer_sampler_mismatch_metrics(empty)])
    assert len(z) == 9 and all(v == 0.0 for v in z.values())


# ---- KL penalty and the actor-loss side terms ---------------------------------------------------------
@pytest.mark.parametrize("ktype", ["kl", "k1", "abs", "mse", "k2", "low_var_kl", "k3", "k1+", "k3+"])
def test_kl_penalty_gpu_vs_oracle(ktype):
    from axon_amd.utils.rl.kl import kl_penalty, kl_penalty_forward
    g = torch.Generator().manual_seed(21)
    lp = -torch.empty(7, 33).exponential_(1.0, generator=g)
    ref = lp + 0.5 * torch.randn(7, 33, generator=g)
    ref[0, 0], ref[0, 1], ref[0, 2] = lp[0, 0] + 25.0, lp[0, 1] - 25.0, lp[0, 2]  # clamps and the tie at 0
    a = lp.clone().to(DEV).requires_grad_(True)
    out = kl_penalty(a, ref.to(DEV), ktype)
    w = torch.randn(7, 33, generator=g)
    (out * w.to(DEV)).sum().backward()
    b = lp.clone().requires_grad_(True)
    want = OL.kl_penalty(b, ref, ktype)
    (want * w).sum().backward()
    assert torch.allclose(out.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-6)
    assert torch.allclose(a.grad.cpu(), b.grad, rtol=1e-5, atol=1e-6)
    assert torch.allclose(kl_penalty_forward(a.detach(), ref.to(DEV), ktype).cpu(), want.detach(), rtol=1e-5, atol=1e-6)


def test_kl_penalty_errors():
    from axon_amd.utils.rl.kl import kl_penalty
    x = torch.zeros(2, 3, device=DEV)
    with pytest.raises(NotImplementedError):
        kl_penalty(x, x, "full")
    with pytest.raises(NotImplementedError):
        kl_penalty(x, x, "nope")


@pytest.mark.parametrize("loss_name,tr,br", [("ppo", "sum", "token-mean"), ("ppo", "mean", "step-mean"),
                                             ("gspo", "mean", "token-mean")])
@pytest.mark.parametrize("kl_type", ["low_var_kl", "k1+"])
def test_actor_loss_assembly_vs_oracle(loss_name, tr, br, kl_type):
    from axon_amd.models.fsdp_models import CausalLM
    d = _c1_with_adv(3)
    g = torch.Generator().manual_seed(33)
    entropy = torch.rand(d["log_probs"].shape, generator=g) * 3
    ref = d["log_probs"] + 0.1 * torch.randn(d["log_probs"].shape, generator=g)
    args = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "token_reduce": tr, "batch_reduce": br,
            "entropy_coef": 0.01, "kl_coef": 0.05, "kl_type": kl_type}
    meta = {"loss_fn": loss_name, "loss_fn_args": args, "temperature": 1.0, "dp_replicas": 2, "n_micro_batches": 4}
    lp_dev = d["log_probs"].to(DEV).requires_grad_(True)
    ent_dev = entropy.to(DEV).requires_grad_(True)
    data = DataProto.from_dict(tensors={"old_log_probs": d["old_log_probs"].to(DEV), "advantages": d["advantages"].to(DEV),
                                        "response_mask": d["response_mask"].to(DEV), "ref_log_prob": ref.to(DEV)})
    module = lambda inputs, m: {"log_probs": lp_dev, "entropys": ent_dev}  # noqa: E731
    loss, metrics = CausalLM.forward_backward_fn(module, data, meta)
    loss.backward()
    lp = d["log_probs"].clone().requires_grad_(True)
    en = entropy.clone().requires_grad_(True)
    fn = OL.ppo_loss if loss_name == "ppo" else OL.gspo_loss
    want, wm = OL.actor_loss(fn, lp, en, d["old_log_probs"], d["advantages"], d["response_mask"], loss_args=args,
                             ref_log_prob=ref, dp_replicas=2, n_micro_batches=4)
    want.backward()
    assert loss.item() == pytest.approx(want.item(), rel=1e-4)
    assert rel_l2(lp_dev.grad, lp.grad) < 1e-5 and rel_l2(ent_dev.grad, en.grad) < 1e-5
    for k in ("pg_loss", "entropy", "entropy_token_mean", "kl_loss", "kl_coef", "pg_clipfrac", "ppo_kl"):
        assert metrics[k] == pytest.approx(wm[k], rel=1e-4, abs=1e-7), k


def test_actor_loss_without_side_terms_and_with_sampler_metrics():
    from axon_amd.models.fsdp_models import loss_from_outputs
    d = _c1_with_adv(4)
    entropy = torch.ones_like(d["log_probs"])
    samp = d["old_log_probs"] + 0.01
    data = DataProto.from_dict(tensors={"old_log_probs": d["old_log_probs"].to(DEV), "advantages": d["advantages"].to(DEV),
                                        "response_mask": d["response_mask"].to(DEV), "sampler_log_probs": samp.to(DEV)})
    lp_dev = d["log_probs"].to(DEV).requires_grad_(True)
    ent_dev = entropy.to(DEV).requires_grad_(True)
    meta = {"loss_fn": "ppo", "loss_fn_args": {}, "temperature": 1.0, "dp_replicas": 1}
    loss, m = loss_from_outputs(data, lp_dev, ent_dev, meta)
    loss.backward()
    assert ent_dev.grad is None or float(ent_dev.grad.abs().max()) == 0.0  # entropy_coef 0: metric only
    assert m["entropy"] == pytest.approx(1.0, rel=1e-5) and m["entropy_token_mean"] == pytest.approx(1.0, rel=1e-5)
    assert "kl_loss" not in m and m["pg_loss"] == pytest.approx(loss.item(), rel=1e-6)
    ref = OS.offpolicy_metrics(d["log_probs"], samp, d["response_mask"])
    _assert_metrics(m, ref, "sampler_corr/")


# ---- REINFORCE / GPG / CISPO ---------------------------------------------------------------------
@pytest.mark.parametrize("tr,br", [("sum", "token-mean"), ("mean", "step-mean")])
@pytest.mark.parametrize("name", ["reinforce", "gpg", "cispo", "cispo-mask"])
def test_more_registry_losses_vs_oracle(name, tr, br):
    d = _c1_with_adv(5)
    g = torch.Generator().manual_seed(44)
    d["log_probs"] = d["old_log_probs"] + 0.3 * torch.randn(d["old_log_probs"].shape, generator=g)
    isw = (1.0 + 0.2 * torch.randn(d["log_probs"].shape, generator=g)).clamp(0.1, 2.0) * d["response_mask"]
    cfg = {"token_reduce": tr, "batch_reduce": br}
    if name.startswith("cispo"):
        cfg.update(clip_ratio_low=0.2, clip_ratio_high=0.28, token_level_mask=name.endswith("mask"))
        okw = dict(clip_ratio_low=0.2, clip_ratio_high=0.28, token_level_mask=name.endswith("mask"))
        fn, reg = OL.cispo_loss, "cispo"
    else:
        okw = dict(sampler_is_weights=isw)
        fn, reg = OL.reinforce_loss, name
    data = _loss_proto(d, extra={"sampler_is_weights": isw})
    loss, metrics = compute_loss_fn(data, reg, cfg)
    loss.backward()
    lp = d["log_probs"].clone().requires_grad_(True)
    ref, ref_m = fn(lp, d["old_log_probs"], d["advantages"], d["response_mask"], token_reduce=tr, batch_reduce=br, **okw)
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4, abs=1e-9)
    assert rel_l2(data.batch["log_probs"].grad, lp.grad) < 1e-5
    assert set(metrics) == set(ref_m)
    for k, v in ref_m.items():
        assert metrics[k] == pytest.approx(v, rel=1e-4, abs=1e-7), k


def test_reinforce_known_answers_gpu():
    lp, adv = T([[1.0, 2.0]]), T([[3.0, 4.0]])
    data = DataProto.from_dict(tensors={"log_probs": lp.to(DEV), "old_log_probs": lp.to(DEV), "advantages": adv.to(DEV),
                                        "response_mask": torch.ones(1, 2).to(DEV)})
    assert compute_loss_fn(data, "reinforce", {})[0].item() == pytest.approx(-5.5)
    assert compute_loss_fn(data, "gpg", {})[0].item() == pytest.approx(-5.5)
    data.batch["sampler_is_weights"] = torch.full((1, 2), 2.0).to(DEV)
    assert compute_loss_fn(data, "reinforce", {})[0].item() == pytest.approx(-11.0)


# ---- RLOO / LOOP / GPG advantages ------------------------------------------------------------------
@pytest.mark.parametrize("name", ["rloo", "loop", "gpg"])
def test_group_baseline_advantages_vs_oracle(name):
    d = W.c1_loss_only(7)
    d["token_level_rewards"][5] = 0  # a zero score for GPG's alpha
    uid = d["uid"].copy()
    uid[3] = "alone"  # a singleton group
    gidx = T(np.unique(uid, return_inverse=True)[1])
    data = DataProto.from_dict(tensors={"token_level_rewards": d["token_level_rewards"].to(DEV),
                                        "response_mask": d["response_mask"].to(DEV)})
    data.non_tensor_batch["uid"] = uid
    args = {"f_norm": 1.5} if name == "gpg" else {}
    out = compute_advantage(data, {"advantage": name, "advantage_args": args})
    if name == "gpg":
        ref = OA.gpg_advantage(d["token_level_rewards"], d["response_mask"], gidx, f_norm=1.5)
    else:
        ref = OA.rloo_advantage(d["token_level_rewards"], d["response_mask"], gidx)
    got = out.batch["advantages"].cpu()
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-6)
    assert torch.equal(out.batch["returns"].cpu(), got)
    assert (got[d["response_mask"] == 0] == 0).all()


# ---- GMPO (geo_mean) -----------------------------------------------------------------------------------
@pytest.mark.parametrize("with_isw", [False, True])
def test_geo_mean_loss_vs_oracle(with_isw):
    d = _c1_with_adv(6)
    g = torch.Generator().manual_seed(55)
    d["log_probs"] = d["old_log_probs"] + 0.3 * torch.randn(d["old_log_probs"].shape, generator=g)
    d["log_probs"][0, 0] = d["old_log_probs"][0, 0] + 0.2   # on the clip boundary
    d["advantages"][1] = 0.0                                  # sign 0
    d["response_mask"][2] = 0.0                               # a row without tokens
    isw = (1.0 + 0.2 * torch.randn(d["log_probs"].shape, generator=g)).clamp(0.1, 2.0) * d["response_mask"]
    extra = {"sampler_is_weights": isw} if with_isw else None
    data = _loss_proto(d, extra=extra)
    loss, metrics = compute_loss_fn(data, "geo_mean", {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28})
    loss.backward()
    lp = d["log_probs"].clone().requires_grad_(True)
    ref, ref_m = OL.geo_mean_loss(lp, d["old_log_probs"], d["advantages"], d["response_mask"], clip_ratio_low=0.2,
                                  clip_ratio_high=0.28, sampler_is_weights=isw if with_isw else None)
    ref.backward()
    assert loss.item() == pytest.approx(ref.item(), rel=1e-4)
    assert rel_l2(data.batch["log_probs"].grad, lp.grad) < 1e-5
    for k, v in ref_m.items():
        assert metrics[k] == pytest.approx(v, rel=1e-4, abs=1e-7), k


def test_geo_mean_known_answer_and_packed_gpu():
    lp, adv = T([[-1.0, -2.0, -3.0]]), T([[1.0, 2.0, 3.0]])
    data = DataProto.from_dict(tensors={"log_probs": lp.to(DEV), "old_log_probs": lp.to(DEV), "advantages": adv.to(DEV),
                                        "response_mask": torch.ones(1, 3).to(DEV)})
    loss, m = compute_loss_fn(data, "geo_mean", {})
    assert loss.item() == pytest.approx(-2.0, rel=1e-6) and m["pg_clipfrac"] == 0.0
    # packed layout == padded layout
    d = _c1_with_adv(8)
    lens = d["lengths"].tolist()
    pk = {k: pad_to_packed(d[k], lens).to(DEV) for k in ("log_probs", "old_log_probs", "advantages", "response_mask")}
    packed = DataProto.from_dict(tensors=pk, meta_info={"cu_seqlens": W.cu_from_lengths(lens).to(DEV)})
    l_pk, _ = compute_loss_fn(packed, "geo_mean", {})
    l_pad, _ = compute_loss_fn(_loss_proto(d), "geo_mean", {})
    # the mean of +-O(1) row terms cancels to ~3e-4: compare on the scale of the terms
    assert l_pk.item() == pytest.approx(l_pad.item(), abs=1e-6)


# ---- operand checks on the host: a short operand never reaches a kernel ------------------------------------
def test_operand_length_mismatch_raises():
    x = torch.zeros(4, 64, device=DEV)
    short = torch.zeros(4, 32, device=DEV)
    rows = _ops.rows_of(x)
    with pytest.raises(ValueError, match="advantages has 128 elements, expected 256"):
        _ops.policy_loss(0, x, x, short, x, None, rows, token_reduce="sum", batch_reduce="token-mean", ratio_lo=0.8,
                         ratio_hi=1.2, clip_c=3.0)
    with pytest.raises(ValueError, match="mask has 128"):
        _ops.row_stats(x, None, short, rows)
    with pytest.raises(ValueError, match="sampler_log_probs has 128"):
        _ops.sampler_correction(x, short, x, rows, is_mode=1, is_threshold=2.0, rs_mode=0, rs_lr_lo=0.0, rs_lr_hi=0.0,
                                log_veto=None)
    with pytest.raises(ValueError, match="values has 128"):
        _ops.reverse_scan(_ops.SCAN_GAE, x, short, x, rows)
    with pytest.raises(ValueError, match="one per row"):
        _ops.policy_loss(0, x, x, x, x, None, rows, token_reduce="mean-program", batch_reduce="token-mean",
                         ratio_lo=0.8, ratio_hi=1.2, clip_c=3.0, num_program_tokens=torch.ones(3, dtype=torch.int64))
    hid = torch.zeros(8, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(100, 32, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="do not match"):
        _ops.lmhead_forward(hid, w, torch.zeros(8, dtype=torch.int32, device=DEV), 1.0)
    with pytest.raises(ValueError, match="labels has 7"):
        _ops.lmhead_forward(hid, torch.zeros(100, 64, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(7, dtype=torch.int32, device=DEV), 1.0)


def test_views_off_a_16_byte_boundary():
    g = torch.Generator().manual_seed(3)
    big = torch.randn(4 * 64 + 1, generator=g).to(DEV)
    x = big[1:].view(4, 64)  # contiguous, 4 bytes past a 16-byte boundary
    mask = (torch.rand(4 * 64 + 1, generator=g) > 0.3).float().to(DEV)[1:].view(4, 64)
    assert x.data_ptr() % 16 == 4
    out, stats = _ops.masked_whiten(x, mask)
    ref, _ = _ops.masked_whiten(x.clone(), mask.clone())
    assert torch.equal(out, ref)
    rows = _ops.rows_of(x)
    a1, g1 = _ops.policy_loss(0, x, x * 0.9, x, mask, None, rows, token_reduce="sum", batch_reduce="token-mean",
                              ratio_lo=0.8, ratio_hi=1.2, clip_c=3.0)
    a2, g2 = _ops.policy_loss(0, x.clone(), x.clone() * 0.9, x.clone(), mask.clone(), None, rows, token_reduce="sum",
                              batch_reduce="token-mean", ratio_lo=0.8, ratio_hi=1.2, clip_c=3.0)
    assert torch.equal(a1[:5], a2[:5]) and torch.equal(g1, g2)


# ---- KL penalty inside the reward (kl.py:248-322) -----------------------------------------------------------
@pytest.mark.parametrize("ktype", ["kl", "abs", "mse", "low_var_kl"])
@pytest.mark.parametrize("where", ["gpu", "cpu"])
def test_apply_kl_penalty_vs_oracle(ktype, where):
    from axon_amd.utils.rl.kl import AdaptiveKLController, apply_kl_penalty, compute_rewards_with_kl
    g = torch.Generator().manual_seed(71)
    b, t = 7, 333
    scores = torch.randn(b, t, generator=g)
    old = -torch.empty(b, t).exponential_(1.0, generator=g)
    ref = old + 0.3 * torch.randn(b, t, generator=g)
    mask = (torch.rand(b, t, generator=g) > 0.3).float()
    mask[2] = 0
    dev = DEV if where == "gpu" else "cpu"
    ctrl = AdaptiveKLController(init_kl_coef=0.2, target_kl=0.01, horizon=100)
    rewards, m = apply_kl_penalty(scores.to(dev), old.to(dev), ref.to(dev), mask.to(dev), ctrl, ktype)
    ref_rewards, ref_kl = OL.apply_kl_penalty(scores, old, ref, mask, 0.2, ktype)
    assert rewards.device.type == ("cuda" if where == "gpu" else "cpu")
    assert torch.allclose(rewards.cpu(), ref_rewards, rtol=1e-5, atol=1e-6)
    assert m["actor/reward_kl_penalty"] == pytest.approx(ref_kl, rel=1e-4, abs=1e-7)
    assert m["actor/reward_kl_penalty_coeff"] == 0.2
    expect = AdaptiveKLController(0.2, 0.01, 100)
    expect.update(ref_kl, b)
    assert ctrl.value == pytest.approx(expect.value, rel=1e-6)  # the controller saw n_steps = number of sequences
    plain = compute_rewards_with_kl(scores.to(dev), old.to(dev), ref.to(dev), 0.05)
    assert torch.allclose(plain.cpu(), scores - (old - ref) * 0.05, rtol=1e-5, atol=1e-6)


def test_apply_kl_penalty_packed_layout():
    from axon_amd.utils.rl.kl import FixedKLController, apply_kl_penalty
    lens = [700, 33, 1, 1200, 64, 257]
    n = sum(lens)
    g = torch.Generator().manual_seed(73)
    scores, old = torch.randn(n, generator=g), -torch.empty(n).exponential_(1.0, generator=g)
    ref = old + 0.2 * torch.randn(n, generator=g)
    mask = (torch.rand(n, generator=g) > 0.2).float()
    cu = W.cu_from_lengths(lens)
    rewards, m = apply_kl_penalty(scores.to(DEV), old.to(DEV), ref.to(DEV), mask.to(DEV), FixedKLController(0.1),
                                  "low_var_kl", cu_seqlens=cu)
    tmax = max(lens)
    pad = lambda x: torch.stack([torch.nn.functional.pad(x[s:e], (0, tmax - (e - s)))  # noqa: E731
                                 for s, e in zip(cu[:-1].tolist(), cu[1:].tolist())])
    ref_rewards, ref_kl = OL.apply_kl_penalty(pad(scores), pad(old), pad(ref), pad(mask), 0.1, "low_var_kl")
    assert torch.allclose(rewards.cpu(), pad_to_packed(ref_rewards, lens), rtol=1e-5, atol=1e-6)
    assert m["actor/reward_kl_penalty"] == pytest.approx(ref_kl, rel=1e-4)


# ---- reward statistics and pass metrics: known answers of the reference's tests/utils/test_rl_utils.py:107-263 --
def test_reward_statistics_and_pass_metrics_known_answers():
    from axon_amd.utils.rl.utils import compute_pass_metrics, compute_reward_statistics

    def proto(scores, **nt):
        return DataProto.from_dict(tensors={"token_level_scores": T(scores).to(DEV)},
                                   non_tensors={k: np.array(v) for k, v in nt.items()})
    s = compute_reward_statistics(proto([[0.0, 1.0], [0.0, 2.0], [0.0, 100.0]], is_padding=[False, False, True],
                                        is_last_step=[True, True, True]))
    assert (s["batch/reward/mean"], s["batch/reward/max"], s["batch/reward/min"]) == (1.5, 2.0, 1.0)
    s = compute_reward_statistics(proto([[0.0, 1.0], [0.0, 2.0], [0.0, 3.0]], is_padding=[False] * 3,
                                        is_last_step=[True, False, True]))
    assert (s["batch/reward/mean"], s["batch/reward/max"], s["batch/reward/min"]) == (2.0, 3.0, 1.0)
    s = compute_reward_statistics(proto([[0.0, 1.0]], is_padding=[True]))
    assert s == {"reward_mean": 0.0, "reward_max": 0.0, "reward_min": 0.0}
    s = compute_reward_statistics(proto([[-1.0, 0.0], [-2.0, -3.0], [-3.0, 0.0]]))
    assert (s["batch/reward/mean"], s["batch/reward/max"], s["batch/reward/min"]) == (-3.0, -1.0, -5.0)
    m, rates = compute_pass_metrics(proto([[0.0, 1.0], [0.0, 0.0], [0.0, 2.0], [0.0, 1.0]], uid=["a", "a", "b", "b"]))
    assert m == {"batch/solve/none": 0, "batch/solve/all": 1, "batch/solve/partial": 1}
    assert rates["a"] == 0.5 and rates["b"] == 1.0
    m, rates = compute_pass_metrics(proto([[0.0, 100.0], [0.0, 1.0], [0.0, 0.0], [0.0, 2.0]], uid=["a", "a", "b", "b"],
                                          is_last_step=[False, True, False, True]))
    assert rates == {"a": 1.0, "b": 1.0} and m["batch/solve/all"] == 2
    m, rates = compute_pass_metrics(proto([[0.0, 0.0], [0.0, 0.0], [0.0, -1.0]], uid=["a", "a", "b"]))
    assert m == {"batch/solve/none": 2, "batch/solve/all": 0, "batch/solve/partial": 0}
    assert compute_pass_metrics(proto([[0.0, 1.0]], uid=["x"]))[1]["x"] == 1.0
    assert compute_pass_metrics(proto([[0.0, 0.999]], uid=["x"]))[1]["x"] == 0.0


# ---- the operators make no host synchronisation and can be captured into a HIP graph ---------------------------
def test_loss_and_correction_in_a_hip_graph():
    """Captured once, replayed several times with other inputs and with eager work and synchronisations between
    the replays: every replay must equal the eager result bit for bit."""
    g = torch.Generator(device=DEV).manual_seed(1)
    b, t = 32, 777
    old = -torch.empty(b, t, device=DEV).exponential_(1.0, generator=g)
    new = old + 0.05 * torch.randn(b, t, device=DEV, generator=g)
    samp = old + 0.01 * torch.randn(b, t, device=DEV, generator=g)
    adv = torch.randn(b, t, device=DEV, generator=g)
    mask = (torch.rand(b, t, device=DEV, generator=g) > 0.3).float()
    rows = _ops.rows_of(new)
    kw = dict(token_reduce="mean", batch_reduce="step-mean", ratio_lo=0.8, ratio_hi=1.28, clip_c=3.0)
    # token-level weights and rejection, the veto (an integer flag per row) and the PPO loss with per-row token
    # counts: none of these adds floats atomically, so two runs agree bit for bit (the sequence-level modes and
    # GSPO add per-row float sums in whatever order the wavefronts arrive and agree to rounding only)
    ckw = dict(is_mode=1, is_threshold=2.0, rs_mode=1, rs_lr_lo=-math.log(2.0), rs_lr_hi=math.log(2.0),
               log_veto=math.log(1e-4))

    def chain():
        isw, new_mask, cacc = _ops.sampler_correction(old, samp, mask, rows, **ckw)
        acc, grad = _ops.policy_loss(0, new, old, adv, new_mask, isw, rows, **kw)
        return cacc, acc, grad

    side = torch.cuda.Stream()  # warm-up off the capture stream, as torch asks for
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_cacc, g_acc, g_grad = chain()
    for _ in range(4):
        new.copy_(old + 0.05 * torch.randn(b, t, device=DEV, generator=g))
        samp.copy_(old + 0.01 * torch.randn(b, t, device=DEV, generator=g))
        e_cacc, e_acc, e_grad = chain()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_acc[:6], e_acc[:6]) and torch.equal(g_grad, e_grad) and torch.equal(g_cacc[:6], e_cacc[:6])


def test_two_hip_graphs_replayed_in_the_other_order():
    """Two graphs captured one after the other on the same capture stream, the second replayed before the first has
    ever run, eager calls in between: each graph must carry the fill of its own reduction workspace (a workspace
    cached at capture time would reach the second graph unfilled), and eager calls must not share a buffer that a
    replay re-zeroes."""
    g = torch.Generator(device=DEV).manual_seed(2)
    b, t = 24, 1500
    old = -torch.empty(b, t, device=DEV).exponential_(1.0, generator=g)
    new = old + 0.05 * torch.randn(b, t, device=DEV, generator=g)
    adv = torch.randn(b, t, device=DEV, generator=g)
    mask = (torch.rand(b, t, device=DEV, generator=g) > 0.3).float()
    rows = _ops.rows_of(new)
    kw_a = dict(token_reduce="sum", batch_reduce="token-mean", ratio_lo=0.8, ratio_hi=1.28, clip_c=3.0)
    kw_b = dict(token_reduce="mean", batch_reduce="step-mean", ratio_lo=0.8, ratio_hi=1.28, clip_c=3.0)
    keep = dict(_ops._PARTIALS)
    _ops._PARTIALS.clear()  # as in a process whose first call on the capture stream happens under capture
    try:
        graph_a, graph_b = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph_a):
            a_acc, a_grad = _ops.policy_loss(0, new, old, adv, mask, None, rows, **kw_a)
        with torch.cuda.graph(graph_b):
            b_acc, b_grad = _ops.policy_loss(0, new, old, adv, mask, None, rows, **kw_b)
        assert not _ops._PARTIALS, "a workspace created under capture must not be kept"
        for first, second in ((graph_b, graph_a), (graph_a, graph_b), (graph_b, graph_a)):
            new.copy_(old + 0.05 * torch.randn(b, t, device=DEV, generator=g))
            ea_acc, ea_grad = _ops.policy_loss(0, new, old, adv, mask, None, rows, **kw_a)
            eb_acc, eb_grad = _ops.policy_loss(0, new, old, adv, mask, None, rows, **kw_b)
            torch.cuda.synchronize()
            first.replay()
            ea2_acc, _ = _ops.policy_loss(0, new, old, adv, mask, None, rows, **kw_a)  # eager work between replays
            second.replay()
            torch.cuda.synchronize()
            assert torch.equal(a_acc[:6], ea_acc[:6]) and torch.equal(a_grad, ea_grad)
            assert torch.equal(b_acc[:6], eb_acc[:6]) and torch.equal(b_grad, eb_grad)
            assert torch.equal(ea2_acc[:6], ea_acc[:6])
    finally:
        _ops._PARTIALS.update(keep)


# ---- kernels in which a workgroup owns whole rows (GSPO, per-row aggregation, veto, sequence level) --------
def _awkward_packed(lens, seed):
    """Packed inputs over rows of the given lengths (zeros allowed), padded twins for the oracle."""
    g = torch.Generator().manual_seed(seed)
    n = sum(lens)
    old = -torch.empty(n).exponential_(1.0, generator=g)
    d = {"lengths": lens, "cu_seqlens": W.cu_from_lengths(lens), "old_log_probs": old,
         "log_probs": old + 0.3 * torch.randn(n, generator=g), "advantages": torch.randn(n, generator=g),
         "sampler_log_probs": old + 0.2 * torch.randn(n, generator=g),
         "response_mask": (torch.rand(n, generator=g) < 0.8).float()}
    tmax = max(max(lens), 1)
    pad = {}
    for k in ("old_log_probs", "log_probs", "advantages", "sampler_log_probs", "response_mask"):
        pad[k] = torch.zeros(len(lens), tmax)
        for b, (a, e) in enumerate(zip(d["cu_seqlens"][:-1].tolist(), d["cu_seqlens"][1:].tolist())):
            pad[k][b, : e - a] = d[k][a:e]
    return d, pad


AWKWARD = {
    # rows longer than the 4096 tokens a workgroup keeps in registers, next to short ones
    "long_rows": [5000, 17, 8192, 1, 3, 4097, 2048, 2047, 2049, 6000, 31],
    # more than 128 rows begin inside one 2048-token range; empty rows in between, first and last
    "tiny_rows": [0, 0] + [1, 0, 2, 3, 0, 5] * 60 + [700, 0, 0],
    # a single row, a row that ends exactly on range borders
    "borders": [2048, 2048, 4096, 1, 2047, 2048],
    # slot counts that are no multiple of four: the incomplete last 16-byte vector shared by two rows, in a
    # later group of a long row, in the first group of the only row; the smallest input the kernels take
    "tail_two_rows": [3000, 2, 1],
    "tail_in_long_row": [6145],
    "tail_in_first_group": [5],
    "four_slots": [1, 3],
}


@pytest.fixture
def owned_rows_forced():
    """Rows of any length through the kernels in which a workgroup owns whole rows (the dispatch would send
    batches of short rows to the row pass + token pass)."""
    from axon_amd import _ops
    keep = _ops.OWNED_ROWS_MIN_MEAN_LEN
    _ops.OWNED_ROWS_MIN_MEAN_LEN = 0
    yield
    _ops.OWNED_ROWS_MIN_MEAN_LEN = keep


@pytest.mark.parametrize("layout", sorted(AWKWARD))
def test_row_owned_losses_on_awkward_layouts(layout, owned_rows_forced):
    lens = AWKWARD[layout]
    d, pad = _awkward_packed(lens, seed=len(lens))
    meta = {"cu_seqlens": d["cu_seqlens"]}
    for name, fn, cfg in (("gspo", OL.gspo_loss, {"clip_ratio_low": 3e-4, "clip_ratio_high": 4e-4,
                                                   "token_reduce": "mean", "batch_reduce": "step-mean"}),
                          ("gspo", OL.gspo_loss, {"clip_ratio_low": 0.1, "clip_ratio_high": 0.1,
                                                   "token_reduce": "sum", "batch_reduce": "token-mean"}),
                          ("ppo", OL.ppo_loss, {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28,
                                                "token_reduce": "mean", "batch_reduce": "token-mean"})):
        first = _check_loss(name, fn, d, cfg, meta=meta, pad=pad)
        again = _check_loss(name, fn, d, cfg, meta=meta, pad=pad)
        assert first.item() == again.item()  # fixed summation order: bit-identical from run to run


@pytest.mark.parametrize("layout", sorted(AWKWARD))
@pytest.mark.parametrize("is_l,rs_l", [("token", "token"), ("sequence", "sequence"), ("sequence", "geometric")])
def test_row_owned_correction_on_awkward_layouts(layout, is_l, rs_l, owned_rows_forced):
    lens = AWKWARD[layout]
    d, pad = _awkward_packed(lens, seed=100 + len(lens))
    kw = dict(sampler_is=is_l, sampler_is_threshold=2.0, sampler_rs=rs_l, sampler_rs_threshold=2.0,
              sampler_token_veto_threshold=0.4)
    outs = []
    for _ in range(2):
        proto, new, m = S.compute_sampler_correction_and_rejection_mask(
            d["old_log_probs"].to(DEV), d["sampler_log_probs"].to(DEV), d["response_mask"].to(DEV),
            cu_seqlens=d["cu_seqlens"].to(DEV), **kw)
        outs.append((proto.batch["sampler_is_weights"].clone(), new.clone(), m))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])  # run to run
    w_ref, new_ref, m_ref = OS.correction(pad["old_log_probs"], pad["sampler_log_probs"], pad["response_mask"], **kw)
    got_new, got_w = outs[0][1].cpu(), outs[0][0].cpu()
    assert torch.equal(got_new, pad_to_packed(new_ref, lens))
    assert torch.allclose(got_w, pad_to_packed(w_ref, lens), rtol=1e-5, atol=1e-7)
    for k, v in m_ref.items():
        assert outs[0][2]["sampler_corr/" + k] == pytest.approx(v, rel=1e-4, abs=1e-6), k


def test_fractional_valid_count_is_not_truncated():
    """A count averaged over ranks may be fractional; the reference divides by the value as it is
    (loss/utils.py:224-229)."""
    d = _c1_with_adv(5)
    b = d["old_log_probs"].shape[0]
    _check_loss("ppo", OL.ppo_loss, d, {"token_reduce": "sum", "batch_reduce": "token-mean"},
                extra={"valid_token_count": torch.full((b,), 1234.5)})
    _check_loss("gspo", OL.gspo_loss, d, {"token_reduce": "mean", "batch_reduce": "step-mean"},
                extra={"valid_batch_size": torch.full((b,), 77.25)})


def test_packed_layout_without_rows_is_refused():
    """cu_seqlens with a single entry (no row) next to a non-empty token array: every kernel that resolves the
    row of a token returns the shape error instead of reading cu_seqlens[-1]."""
    from axon_amd import _lib
    lib = _lib.load()
    t = torch.zeros(64, device=DEV)
    cu = torch.zeros(1, dtype=torch.int32, device=DEV)
    ws = torch.zeros(lib.axon_reduce_partials_bytes(64) // 4, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda x: x.data_ptr()  # noqa: E731
    assert lib.axon_row_stats(p(t), p(t), p(t), 0, p(cu), 0, 64, 0, 0, 0.0, p(t), p(t), None, None, st) == -2
    assert lib.axon_row_broadcast_mask(p(t), p(t), 0, p(cu), 0, 64, 0, 0.0, p(t), st) == -2
    assert lib.axon_policy_loss(1, p(t), p(t), p(t), p(t), 0, None, p(cu), 0, 64, 0, p(t), p(t), 1.0, 0, None, 0.8,
                                1.2, 3.0, p(t), p(t), p(ws), st) == -2
    assert lib.axon_policy_loss_rows(1, p(t), p(t), p(t), p(t), 0, None, p(cu), 0, 64, 0, 1, 1, None, None, None,
                                     None, 0.8, 1.2, 3.0, p(t), p(t), p(ws), st) == -2
    assert lib.axon_sampler_correction_rows(p(t), p(t), p(t), 0, p(cu), 0, 64, 0, 1, 2.0, 1, -0.7, 0.7, 1, -9.0,
                                            p(t), p(t), None, None, None, p(t), p(ws), st) == -2
    assert lib.axon_reverse_scan(0, p(t), p(t), p(t), 0, p(cu), 0, 64, 0, 1.0, 1.0, None, p(t), p(t), st) == -2
    torch.cuda.synchronize()


def _random_layout(seed):
    """Row lengths drawn from a mixture: empty and tiny rows, rows under a chunk of 1024 slots (which share a step
    in pairs), rows of one to two chunks, rows of several groups of 2048; any slot count modulo four."""
    g = torch.Generator().manual_seed(1000 + seed)
    kinds = torch.randint(0, 5, (40,), generator=g).tolist()
    lens = []
    for k in kinds:
        lo, hi = ((0, 4), (4, 200), (200, 1025), (1025, 2100), (2100, 7000))[k]
        lens.append(int(torch.randint(lo, hi, (1,), generator=g)))
    return lens


@pytest.mark.parametrize("seed", range(8))
def test_row_owned_kernels_on_random_layouts(seed, owned_rows_forced):
    """GSPO (sequence ratio and per-row mean), the veto and sequence-level weights on random mixtures of row
    lengths against the oracle: every kind of step of the row walk next to every other."""
    lens = _random_layout(seed)
    d, pad = _awkward_packed(lens, seed=500 + seed)
    _check_loss("gspo", OL.gspo_loss, d, {"clip_ratio_low": 0.1, "clip_ratio_high": 0.1, "token_reduce": "mean",
                                          "batch_reduce": "step-mean"}, meta={"cu_seqlens": d["cu_seqlens"]}, pad=pad)
    kw = dict(sampler_is="sequence", sampler_is_threshold=2.0, sampler_rs="geometric", sampler_rs_threshold=2.0,
              sampler_token_veto_threshold=0.4)
    proto, new, _ = S.compute_sampler_correction_and_rejection_mask(
        d["old_log_probs"].to(DEV), d["sampler_log_probs"].to(DEV), d["response_mask"].to(DEV),
        cu_seqlens=d["cu_seqlens"].to(DEV), **kw)
    w_ref, new_ref, _ = OS.correction(pad["old_log_probs"], pad["sampler_log_probs"], pad["response_mask"], **kw)
    assert torch.equal(new.cpu(), pad_to_packed(new_ref, lens))
    assert torch.allclose(proto.batch["sampler_is_weights"].cpu(), pad_to_packed(w_ref, lens), rtol=1e-5, atol=1e-7)


def test_sequence_level_decisions_repeat_on_the_short_row_path():
    """A batch whose rows average eleven tokens takes the row pass + token pass (the row-owning kernels want
    longer rows), and one of its rows has 6000 tokens: 24 wavefronts each add a partial sum to that row, in
    whatever order they finish.  Its log-ratio sum is placed on the upper rejection bound to within an fp32
    ulp, so a sum that depended on the order would flip the row's keep / reject bit from call to call: the
    masks and weights of twenty calls must be identical (the sums are added in fixed point, rows.hip)."""
    g = torch.Generator().manual_seed(77)
    lens = [8] * 1000 + [6000] + [8] * 1000
    n = sum(lens)
    cu = W.cu_from_lengths(lens)
    rows = _ops.rows_of(torch.empty(n, device=DEV), cu)
    assert not _ops._own_rows(rows) and rows.cu.is_cuda
    with pytest.raises(_lib.AxonAmdError, match="must live on the GPU"):  # host offsets are refused, not dereferenced
        _ops.row_stats(torch.zeros(n, device=DEV), None, None, _ops.rows_of(torch.empty(n), cu))
    old = -torch.empty(n).exponential_(1.0, generator=g)
    lr = 0.01 * torch.randn(n, generator=g)
    a, e = int(cu[1000]), int(cu[1001])
    hi = math.log(2.0)
    lr[a] += hi - lr[a:e].double().sum().item()  # the long row's sum is ln 2 up to rounding
    assert abs(lr[a:e].double().sum().item() - hi) < 1e-6
    samp = (old.double() - lr.double()).float()
    mask = torch.ones(n)
    od, sd, md = old.to(DEV), samp.to(DEV), mask.to(DEV)
    kw = dict(is_mode=2, is_threshold=2.0, rs_mode=2, rs_lr_lo=-hi, rs_lr_hi=hi, log_veto=None)
    first = None
    sums = set()
    for _ in range(20):
        _, ssum, _ = _ops.row_stats(od, sd, md, rows)
        isw, new_mask, acc = _ops.sampler_correction(od, sd, md, rows, **kw)
        sums.add(ssum[1000].item())
        if first is None:
            first = (isw.clone(), new_mask.clone(), ssum.clone())
        assert torch.equal(new_mask, first[1]) and torch.equal(isw, first[0]) and torch.equal(ssum, first[2])
    assert len(sums) == 1 and abs(sums.pop() - hi) < 1e-5
    # a partial beyond the fixed-point range, an infinity and a NaN reach the sum as fp32 would have them
    big = torch.zeros(n)
    big[a] = 3.0e7
    big[a + 300] = 5.0
    big[0] = float("inf")
    big[8] = float("nan")
    _, ssum, _ = _ops.row_stats(big.to(DEV), None, md, rows)
    assert ssum[1000].item() == torch.tensor(3.0e7 + 5.0, dtype=torch.float32).item()  # the double sum, rounded once
    assert ssum[0].item() == float("inf") and math.isnan(ssum[1].item())
    assert float(ssum[2:1000].abs().max()) == 0.0


def test_row_owned_entry_points_refuse_fewer_than_four_slots():
    """The kernels in which a workgroup owns whole rows read 16-byte vectors: one to three slots are refused
    with the shape error (the host sends such inputs through the row pass + token pass), four are taken."""
    from axon_amd import _lib
    lib = _lib.load()
    t = torch.zeros(8, device=DEV)
    ws = torch.zeros(lib.axon_reduce_partials_bytes(8) // 4, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda x: x.data_ptr()  # noqa: E731
    for n, want in ((1, -2), (3, -2), (4, 0)):
        assert lib.axon_policy_loss_rows(1, p(t), p(t), p(t), p(t), 0, None, None, 1, n, n, 1, 1, None, None, None,
                                         None, 0.8, 1.2, 3.0, p(t), p(t), p(ws), st) == want
        assert lib.axon_sampler_correction_rows(p(t), p(t), p(t), 0, None, 1, n, n, 1, 2.0, 1, -0.7, 0.7, 1, -9.0,
                                                p(t), p(t), None, None, None, p(t), p(ws), st) == want
    torch.cuda.synchronize()


def test_all_padding_micro_batch_is_a_no_op_before_any_validation():
    """sampler.py:368-370: an all-zero mask returns (None, mask, {}) even with arguments that would not
    validate; with a token to correct the same arguments raise."""
    z = torch.zeros(2, 4, device=DEV)
    for kw in (dict(sampler_is="token", sampler_is_threshold=0.0), dict(sampler_rs="bogus", sampler_rs_threshold=2.0),
               dict(sampler_rs="token", sampler_rs_threshold=None), dict(sampler_token_veto_threshold=-1.0)):
        proto, mask, m = S.compute_sampler_correction_and_rejection_mask(z, z, z, **kw)
        assert proto is None and mask is z and m == {}
        with pytest.raises(ValueError):
            S.compute_sampler_correction_and_rejection_mask(z, z, torch.ones_like(z), **kw)
    proto, mask, m = S.compute_sampler_correction_and_rejection_mask(z, torch.zeros(2, 5, device=DEV), z)
    assert proto is None and m == {}
