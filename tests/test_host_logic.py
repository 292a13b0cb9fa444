"""CPU-only checks of the host side: registries, DataProto shim, label ranking, threshold
bisection, argument validation, and the C-ABI surface.  No kernel is launched here."""

import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

from axon_amd import _lib
from axon_amd.protocol import DataProto
from axon_amd.trainer.algos.advantages import AdvantageFn, compute_advantage, get_advantage_fn, register_advantage
from axon_amd.trainer.algos.loss import LossFn, agg_loss, compute_loss_fn, get_loss_fn, register_loss
from axon_amd.utils.registry import FunctionRegistry
from axon_amd.utils.rl import sampler as S
from axon_amd.utils.rl.advantage import as_torch_index, group_mean_std

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI ------------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "axon_amd.h")).read()
    declared = set(re.findall(r"\b(axon_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/axon_amd.h but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes bindings and header disagree"
    m = re.search(r"#define AXON_AMD_ABI_VERSION (\d+)", header)
    assert lib.axon_amd_abi_version() == int(m.group(1)) == _lib.ABI_VERSION
    assert lib.axon_amd_error_string(0) == b"ok"
    assert b"workspace" in lib.axon_amd_error_string(-3)


def test_workspace_queries_and_argument_errors_without_gpu():
    lib = _lib.load()
    assert lib.axon_lmhead_fwd_workspace_bytes(32768, 4096, 151936) > 0
    assert lib.axon_lmhead_fwd_workspace_bytes(16, 100, 50) == -1  # hidden % 32 != 0
    assert lib.axon_lmhead_bwd_workspace_bytes(64, 128, 1000, 100) == -1  # chunk % 256 != 0
    assert lib.axon_lmhead_bwd_workspace_bytes(64, 128, 1000, 256) > 0
    # the forward's optional stash: 128 KB per 256 x 256 tile + the per-part maxima; 0 where shifted edge tiles
    # could not hand rows over in fours; -1 for an invalid shape
    assert lib.axon_lmhead_stash_bytes(32768, 4096, 151936) == 594 * 128 * 131072 + 594 * 2 * 32768 * 4
    assert lib.axon_lmhead_stash_bytes(513, 256, 1500) == 0 and lib.axon_lmhead_stash_bytes(516, 256, 1502) == 0
    assert lib.axon_lmhead_stash_bytes(513, 96, 1501) == 3 * 6 * 131072 + 256 * ((6 * 2 * 513 * 4 + 255) // 256)
    assert lib.axon_lmhead_stash_bytes(16, 100, 50) == -1 and lib.axon_lmhead_stash_bytes(0, 128, 1000) == 0
    # null pointers are rejected before any launch
    assert lib.axon_row_stats(None, None, None, 0, None, 4, 16, 4, 0, 0.0, None, None, None, None, None) == -1
    assert lib.axon_policy_loss(7, None, None, None, None, 0, None, None, 1, 4, 4, None, None, 0.0, 0, None, 0.8, 1.2,
                                3.0, None, None, None, None) == -1
    assert lib.axon_reduce_partials_bytes(4097) == lib.axon_reduce_partials_bytes(1 << 30) == 16384 * 32 + 256 * 32 + 2048 and lib.axon_reduce_partials_bytes(-1) == -1
    assert lib.axon_fill_zero(None, 3, None) == -1


def test_cpu_tensors_fail_loudly():
    x = torch.zeros(2, 4)
    with pytest.raises(_lib.AxonAmdError, match="no CPU fallback"):
        agg_loss(x, x)
    data = DataProto.from_dict(tensors={"log_probs": x, "old_log_probs": x, "advantages": x, "response_mask": x})
    with pytest.raises(_lib.AxonAmdError, match="no CPU fallback"):
        compute_loss_fn(data, "ppo", {})
    with pytest.raises(_lib.AxonAmdError):
        S.compute_sampler_correction_and_rejection_mask(x, x, x, sampler_is="token")
    from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy

    with pytest.raises(_lib.AxonAmdError):
        linear_cross_entropy(torch.zeros(4, 32).bfloat16(), torch.zeros(8, 32).bfloat16(), torch.zeros(4).long(), 1.0,
                             "none")


# ---- registries (reference tests/utils/registry/test_function_registry.py:46-67) -----------------
def test_registry_rules():
    reg = FunctionRegistry(name="thing")

    @reg.register("a")
    def fa(data, config):
        return 1

    reg.register("a")(fa)  # same function again: fine
    with pytest.raises(ValueError, match="already registered with different function"):
        reg.register("a")(lambda d, c: 2)
    with pytest.raises(ValueError, match="Unknown thing"):
        reg.get_fn("missing")
    assert "a" in reg and reg.keys() == ["a"] and reg.compute("a", None, None) == 1


def test_loss_and_advantage_registered():
    assert get_loss_fn("ppo") is get_loss_fn(LossFn.PPO)
    assert callable(get_loss_fn("gspo")) and callable(get_advantage_fn(AdvantageFn.GRPO))
    with pytest.raises(ValueError, match="already registered"):
        register_loss("ppo")(lambda d, c: None)
    with pytest.raises(ValueError, match="already registered"):
        register_advantage("grpo")(lambda d, c: None)
    with pytest.raises(ValueError, match="must have 'advantage'"):
        compute_advantage(DataProto.from_dict(tensors={"x": torch.zeros(1)}), {"advantage": None})


# ---- DataProto shim (reference tests/test_protocol.py:240-400) ------------------------------------
def test_dataproto_shim():
    d = DataProto.from_dict(tensors={"a": torch.arange(6).view(3, 2), "b": torch.ones(3)},
                            non_tensors={"uid": ["x", "y", "x"]}, meta_info={"k": 1})
    assert len(d) == 3 and d.non_tensor_batch["uid"].dtype == object
    assert "a" in d.batch and d.batch.get("zz", None) is None
    sub = d.select_idxs([0, 2])
    assert len(sub) == 2 and sub.non_tensor_batch["uid"].tolist() == ["x", "x"]
    assert d.select(batch_keys=["a"]).batch.keys() == {"a"}
    d.union(DataProto.from_dict(tensors={"c": torch.zeros(3)}))
    assert "c" in d.batch
    with pytest.raises(AssertionError, match="Conflicting"):
        d.union(DataProto.from_dict(tensors={"b": torch.zeros(3)}))
    with pytest.raises(AssertionError, match="Batch size mismatch"):
        DataProto.from_dict(tensors={"a": torch.zeros(3), "b": torch.zeros(4)})
    with pytest.raises(RuntimeError, match="batch dimension mismatch"):
        d.batch["bad"] = torch.zeros(5)


# ---- as_torch_index (reference tests/utils/test_rl_advantage.py:53-102,402-450) --------------------
def test_as_torch_index():
    idx = as_torch_index(np.array(["u1", "u2", "u1", "u3"], dtype=object), device="cpu")
    assert idx[0] == idx[2] and len({int(i) for i in idx}) == 3 and idx.dtype == torch.long
    assert as_torch_index(torch.tensor([True, False, True]), device="cpu").tolist() == [1, 0, 1]
    assert as_torch_index(torch.tensor([0.0, 1.0, 2.0]), device="cpu").tolist() == [0, 1, 2]
    assert as_torch_index(torch.tensor([0.0, 1.0, 2.0]).bfloat16(), device="cpu").tolist() == [0, 1, 2]
    frac = as_torch_index(torch.tensor([0.5, 1.5, 0.5]), device="cpu")
    assert frac[0] == frac[2] != frac[1]
    assert as_torch_index(torch.tensor([5, 5, 10, 10]), device="cpu").tolist() == [5, 5, 10, 10]
    assert as_torch_index([3, -1, 3], device="cpu").tolist() == [3, -1, 3]
    mixed = as_torch_index(np.array([None, "a", None, 1], dtype=object), device="cpu")
    assert mixed[0] == mixed[2] and mixed.numel() == 4


def test_group_mean_std_host_checks():
    with pytest.raises(ValueError, match="mismatch"):
        group_mean_std(torch.zeros(2), torch.zeros(1, dtype=torch.long))
    assert all(t.numel() == 0 for t in group_mean_std(torch.empty(0), torch.empty(0, dtype=torch.long)))


# ---- sampler argument validation (reference tests/utils/test_rl_sampler.py:41-49,153-156,272-287) --
def test_sampler_validation_messages():
    x = torch.zeros(2, 3)
    with pytest.raises(ValueError, match="Invalid sampler_rs"):
        S.compute_sampler_rejection_mask(x, x, "bogus", 2.0)
    with pytest.raises(ValueError, match="must be provided"):
        S.compute_sampler_rejection_mask(x, x, "token", None)
    with pytest.raises(ValueError, match="must be positive"):
        S.compute_sampler_correction_weights(x, x, "token", 0.0)
    with pytest.raises(ValueError, match="Invalid sampler_is"):
        S.compute_sampler_correction_weights(x, x, "geometric", 2.0)
    one = torch.ones(2, 3)  # the unified function validates only when there is a token to correct
    with pytest.raises(ValueError, match="must be positive"):
        S.compute_sampler_correction_and_rejection_mask(x, x, one, sampler_token_veto_threshold=-0.1)
    with pytest.raises(ValueError, match="does not match"):
        S.compute_sampler_correction_and_rejection_mask(x, torch.zeros(2, 4), one)
    with pytest.raises(ValueError, match="must be explicitly provided"):
        S.compute_sampler_correction_and_rejection_mask(x, x, one, sampler_rs="token", sampler_rs_threshold=None)
    # an all-padding micro-batch is a no-op before any validation (sampler.py:368-370)
    assert S.compute_sampler_correction_and_rejection_mask(x, x, x, sampler_token_veto_threshold=-0.1) == (None, x, {})


def test_log_interval_agrees_with_torch_exp_bitwise():
    """lo <= x <= hi  <=>  lower <= exp(clamp(x)) <= upper for every fp32 x near the ends."""
    for lower, upper in [(0.5, 2.0), (1 / 3.0, 3.0), (0.9, 1.1), (1e-3, 5.0)]:
        lo, hi = S.log_interval_for_ratio_bounds(lower, upper)
        for centre in (lo, hi):
            xs = torch.tensor([centre], dtype=torch.float32)
            near = [xs]
            up, dn = xs.clone(), xs.clone()
            for _ in range(40):
                up = torch.nextafter(up, torch.tensor(math.inf))
                dn = torch.nextafter(dn, torch.tensor(-math.inf))
                near += [up.clone(), dn.clone()]
            x = torch.cat(near).repeat(8)
            w = torch.exp(torch.clamp(x, -20.0, 20.0))
            ref = (w >= lower) & (w <= upper)
            got = (x >= lo) & (x <= hi)
            assert torch.equal(ref, got), (lower, upper)
    assert S.log_interval_for_ratio_bounds(1e-12, 1e12) == (-math.inf, math.inf)  # beyond the +-20 clamp
    assert S._log32(1e-4) == float(torch.log(torch.tensor(1e-4)))


def test_loss_config_validation_before_any_launch():
    x = torch.zeros(1, 3)
    data = DataProto.from_dict(tensors={"log_probs": x, "old_log_probs": x, "advantages": x, "response_mask": x})
    for c in (0.5, 1.0):
        with pytest.raises(AssertionError, match="clip_ratio_c must be > 1.0"):
            compute_loss_fn(data, "ppo", {"clip_ratio_c": c})
    with pytest.raises(ValueError, match="Invalid token_reduce"):
        agg_loss(x, x, token_reduce="nope")
    with pytest.raises(ValueError, match="Invalid batch_reduce"):
        agg_loss(x, x, batch_reduce="nope")
    with pytest.raises(AssertionError, match="valid_program_count required"):
        agg_loss(x, x, token_reduce="mean", batch_reduce="program-mean", num_program_steps=torch.ones(1))
    with pytest.raises(ValueError, match="Unknown policy loss"):
        compute_loss_fn(data, "nonexistent", {})


def test_rolled_label_precedence_and_output_type():
    """Label choice of the model-forward mirror (reference dense_common.py:187-196) and its output object."""
    from axon_amd.models.transformers.dense_common import (CausalLMOutputForPPO, final_logit_softcapping,
                                                            select_rolled_labels)
    ids = torch.tensor([[5, 6, 7, 8]])
    labels = torch.tensor([[1, 2, 3, 4]])
    pre = torch.tensor([[9, 9, 9, 9]])
    assert select_rolled_labels(pre, labels, ids) is pre
    assert select_rolled_labels(None, labels, ids).tolist() == [[2, 3, 4, 1]]
    assert select_rolled_labels(None, None, ids).tolist() == [[6, 7, 8, 5]]
    with pytest.raises(RuntimeError):
        select_rolled_labels(None, None, None)
    out = CausalLMOutputForPPO(log_probs=torch.zeros(3), entropy=torch.ones(3))
    assert out.log_probs.shape == (3,) and out.entropy.sum() == 3 and out.past_key_values is None

    class Text:
        final_logit_softcapping = 30.0

    class Multi:
        def get_text_config(self):
            return Text()

    class Plain:
        pass

    assert final_logit_softcapping(Multi()) == 30.0 and final_logit_softcapping(Text()) == 30.0
    assert final_logit_softcapping(Plain()) is None


# ---- KL controllers: known answers of the reference's tests/utils/test_kl.py:26-150 ----------------------------
def test_kl_controllers_known_answers():
    import math
    from types import SimpleNamespace
    from axon_amd.utils.rl.kl import AdaptiveKLController, FixedKLController, get_kl_controller
    c = AdaptiveKLController(init_kl_coef=0.5, target_kl=4.0, horizon=1000)
    c.update(current_kl=8.0, n_steps=10)  # error 1.0 clipped to 0.2
    assert c.value == pytest.approx(0.5 * (1 + 0.2 * 10 / 1000))
    c = AdaptiveKLController(1.0, 10.0, 100)
    c.update(current_kl=0.001, n_steps=10)  # clipped to -0.2
    assert c.value == pytest.approx(1 - 0.2 * 10 / 100)
    c = AdaptiveKLController(1.0, 5.0, 100)
    for _ in range(3):
        c.update(10.0, 10)
    assert c.value == pytest.approx(1.02 ** 3)
    c = AdaptiveKLController(0.1, 6.0, 10000)
    c.update(6.0, 32)
    assert c.value == 0.1  # at the target: unchanged
    c.update(100.0, 0)
    assert c.value == 0.1  # no steps: unchanged
    z = AdaptiveKLController(0.1, 0.0, 10)
    z.update(0.5, 1)  # a zero target does not divide by zero
    assert z.value == pytest.approx(0.1 * (1 + 0.2 / 10)) and math.isfinite(z.value)
    f = FixedKLController(kl_coef=0.05)
    f.update(100.0, 32)
    assert f.value == 0.05
    assert isinstance(get_kl_controller(SimpleNamespace(type="fixed", kl_coef=0.1)), FixedKLController)
    a = get_kl_controller(SimpleNamespace(type="adaptive", kl_coef=0.2, target_kl=6.0, horizon=100))
    assert isinstance(a, AdaptiveKLController) and (a.value, a.target, a.horizon) == (0.2, 6.0, 100)
    with pytest.raises(AssertionError, match="horizon must be larger than 0"):
        get_kl_controller(SimpleNamespace(type="adaptive", kl_coef=0.2, target_kl=6.0, horizon=0))
    with pytest.raises(NotImplementedError):
        get_kl_controller(SimpleNamespace(type="bogus", kl_coef=0.2))


def test_row_owning_dispatch_rule():
    """Operators with a per-row quantity take the one-launch kernel (a workgroup works on one row at a time)
    when the rows average at least OWNED_ROWS_MIN_MEAN_LEN and at most OWNED_ROWS_MAX_MEAN_LEN tokens (a single
    workgroup walks a row alone), the row pass + token pass otherwise."""
    import torch

    from axon_amd import _ops

    assert _ops._own_rows(_ops.rows_of(torch.zeros(128, 1024)))           # padded 128 x 1024
    assert _ops._own_rows(_ops.rows_of(torch.zeros(65536), torch.tensor([0, 30000, 40000, 50000, 65536], dtype=torch.int32)))
    assert not _ops._own_rows(_ops.rows_of(torch.zeros(65536), torch.tensor([0, 30000, 65536], dtype=torch.int32)))
    assert not _ops._own_rows(_ops.rows_of(torch.zeros(1, 1 << 20)))      # one row of a million slots
    assert not _ops._own_rows(_ops.rows_of(torch.zeros(4096, 8)))         # rows of 8 tokens
    assert not _ops._own_rows(_ops.rows_of(torch.zeros(12), torch.arange(0, 13, 3, dtype=torch.int32)))
    keep = _ops.OWNED_ROWS_MAX_SLOTS
    try:
        _ops.OWNED_ROWS_MAX_SLOTS = 0
        assert not _ops._own_rows(_ops.rows_of(torch.zeros(128, 1024)))
    finally:
        _ops.OWNED_ROWS_MAX_SLOTS = keep
    keep = _ops.OWNED_ROWS_MIN_MEAN_LEN
    try:  # whatever the threshold: never fewer slots than one 16-byte vector
        _ops.OWNED_ROWS_MIN_MEAN_LEN = 0
        assert _ops._own_rows(_ops.rows_of(torch.zeros(1, 4)))
        assert not _ops._own_rows(_ops.rows_of(torch.zeros(1, 3)))
    finally:
        _ops.OWNED_ROWS_MIN_MEAN_LEN = keep


def test_which_shapes_write_the_dlogits_once_and_may_group_blocks():
    """Host-side shape rules of the head's backward (no GPU call): the dlogits are written once when the
    weight-gradient GEMM can read them K-major (hidden >= 256, vocab % 8 == 0, every chunk at least 256 rows),
    twice otherwise; blocks may share a weight-gradient GEMM when, in addition, a block takes the whole vocabulary
    in one chunk."""
    from axon_amd import _lib
    lib = _lib.load()
    copies, group = lib.axon_lmhead_bwd_dlogit_copies, lib.axon_lmhead_block_can_group
    assert copies(4096, 151936, 0) == 1 and copies(4096, 151936, 152064) == 1      # Qwen3-8B, chunks of 32768 / one
    assert copies(2880, 201088, 0) == 1 and copies(896, 151936, 0) == 1            # GPT-OSS, Qwen2.5-0.5B
    assert copies(256, 1504, 512) == 1 and copies(256, 1160, 512) == 2             # last chunk of 480 / 136 rows
    assert copies(256, 1500, 512) == 2 and copies(192, 2048, 512) == 2             # vocab % 8, hidden < 256
    assert copies(4096, 151936, 100) < 0 and copies(4097, 151936, 0) < 0           # chunk % 256, hidden % 32
    assert group(4096, 151936, 152064) == 1 and group(4096, 151936, 0) == 0        # one chunk only
    # with vocab % 64 == 0 the workspace holds no transposed weight either: hidden x (vocab + 64) x 2 bytes less
    ws = lib.axon_lmhead_bwd_workspace_bytes
    assert ws(8192, 256, 2048 + 8, 2304) - ws(8192, 256, 2048, 2048) > 256 * 2048 * 2
    assert group(256, 2048, 0) == 1 and group(128, 2048, 0) == 0 and group(256, 2044, 0) == 0


def test_blocks_that_share_a_weight_gradient_gemm_are_placed_on_tile_borders():
    from axon_amd._ops import head_block_groups
    four = [(0, 8192), (8192, 16384), (16384, 24576), (24576, 32768)]
    assert head_block_groups(four, 1) == ([(0, 0, True), (1, 0, True), (2, 0, True), (3, 0, True)], 4, 8192)
    assert head_block_groups(four, 2) == ([(0, 0, False), (0, 8192, True), (1, 0, False), (1, 8192, True)], 2, 16384)
    assert head_block_groups(four, 8) == ([(0, 0, False), (0, 8192, False), (0, 16384, False), (0, 24576, True)], 1,
                                          32768)
    # ragged blocks (sequence cuts, lengthened to a multiple of four rows): rounded up to 256 inside a group
    ragged = [(0, 436), (433, 936), (933, 1500)]
    assert head_block_groups(ragged, 2) == ([(0, 0, False), (0, 512, True), (1, 0, True)], 2, 1024)
    assert head_block_groups(ragged, 3) == ([(0, 0, False), (0, 512, False), (0, 1024, True)], 1, 1792)
    assert head_block_groups([(0, 100)], 2) == ([(0, 0, True)], 1, 256)


def test_fused_step_block_plans():
    from axon_amd.models.fused_head_loss import sequence_blocks, token_blocks
    assert token_blocks(32768, 8192) == [(0, 8192), (8192, 16384), (16384, 24576), (24576, 32768)]
    assert token_blocks(1500, 512) == [(0, 512), (512, 1024), (1024, 1500)]
    assert token_blocks(1500, 4096) == [(0, 1500)]
    assert token_blocks(33000, 8192) == [(0, 6656), (6656, 13312), (13312, 19968), (19968, 26624), (26624, 33000)]
    assert token_blocks(32768, 12288) == [(0, 12288), (12288, 24576), (24576, 32768)]
    assert token_blocks(1000, 300) == [(0, 512), (512, 1000)]
    cu = [0, 400, 433, 933, 997, 1297, 1500]
    assert sequence_blocks(cu, 512) == [(0, 2), (2, 3), (3, 5), (5, 6)]
    assert sequence_blocks(cu, 499) is None
    assert sequence_blocks([0, 0, 5, 5, 5], 8) == [(0, 4)]
