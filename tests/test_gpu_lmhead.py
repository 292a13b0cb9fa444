"""GPU parity: the fused LM head (forward, backward, autograd wiring) and the MFMA main loop,
through the product API (ctypes -> libaxon_amd.so) against the CPU oracle.

Tolerances (fp): logprob / entropy 1e-3 absolute against the fp32-upcast oracle; gradients
2e-2 relative-L2 in bf16; plain GEMM 1e-5 relative-L2 against an fp32 matmul of the same
bf16 inputs; the backward that decodes the forward's stash against the backward that recomputes
the logits 5e-3 relative-L2 (fp16 numerators, 2^-11, under the bf16 rounding of every dlogit, 2^-9).

The autograd-level backward tests run twice: with the forward's stash (`head_path` "stash") and with
the recompute backward ("recompute")."""

import math

import pytest
import torch

from axon_amd import _ops, workloads as W
from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
from axon_amd.utils.torch.fused_linear import FusedLinearForPPO
from oracle import lmhead as OM

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(params=["stash", "recompute"])
def head_path(request):
    """Which backward `linear_cross_entropy` takes: decode of the forward's stash (where the shape allows
    one), or recompute of the logits."""
    saved = _ops.LMHEAD_STASH
    _ops.LMHEAD_STASH = request.param == "stash"
    yield request.param
    _ops.LMHEAD_STASH = saved


def rel_l2(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (512, 256, 128), (260, 300, 96), (4, 5, 32), (1000, 77, 2880),
                                   (768, 1024, 896)])
def test_gemm_nt_vs_fp32_matmul(m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    b = torch.randn(n, k, generator=g).bfloat16()
    out = _ops.gemm_nt(a.to(DEV), b.to(DEV))
    ref = b.float() @ a.float().t()
    assert out.shape == (n, m) and rel_l2(out, ref) < 1e-5


def _stored(x, kmajor, pad):
    """The logical [rows][k] matrix `x` as the GEMM takes it: row-major, or K-major ([k][rows]), either with
    `pad` unused elements at the end of every stored row."""
    src = x.t() if kmajor else x
    buf = torch.full((src.shape[0], src.shape[1] + pad), float("nan"), dtype=torch.bfloat16, device=DEV)
    buf[:, : src.shape[1]] = src.to(DEV)
    return buf[:, : src.shape[1]]


@pytest.mark.parametrize("a_kmajor,b_kmajor", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (512, 768, 256), (520, 776, 320), (264, 1024, 128),
                                   (4096, 1000, 192)])
def test_gemm_with_k_major_operands_vs_fp32_matmul(m, n, k, a_kmajor, b_kmajor):
    """Operands stored [k][rows] are read as they lie (LDS transpose reads): same result as the NT form, on whole
    tiles, on edge tiles shifted back by a multiple of 8 rows, with padded leading dimensions."""
    g = torch.Generator().manual_seed(3 * m + 5 * n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    b = torch.randn(n, k, generator=g).bfloat16()
    out = _ops.gemm_layouts(_stored(a, a_kmajor, 72), _stored(b, b_kmajor, 8), a_kmajor, b_kmajor)
    ref = b.float() @ a.float().t()
    assert out.shape == (n, m) and rel_l2(out, ref) < 1e-5
    assert torch.equal(out, _ops.gemm_nt(a.to(DEV), b.to(DEV)))  # the same products in the same order


def test_gemm_with_k_major_operands_refuses_what_the_dma_loop_cannot_take():
    a = torch.zeros(64, 260, dtype=torch.bfloat16, device=DEV)   # [k][m], m % 8 != 0
    b = torch.zeros(256, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="axon_gemm_bf16"):
        _ops.gemm_layouts(a[:, :260], b, True, False)
    with pytest.raises(Exception, match="axon_gemm_bf16"):      # fewer than 256 rows: no DMA loop
        _ops.gemm_layouts(torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV), b, True, False)


CASES = [  # n_tokens, hidden, vocab, temperature, label dtype
    (64, 128, 1000, 1.0, torch.int64),
    (300, 96, 777, 0.7, torch.int32),      # hidden % 64 != 0, ragged tiles everywhere
    (257, 256, 2049, 1.3, torch.int64),
    (1, 32, 5, 1.0, torch.int32),
    (513, 2880, 1500, 1.0, torch.int32),   # GPT-OSS hidden size
    (516, 256, 1504, 0.8, torch.int32),    # hidden >= 256, vocab % 8 == 0: the weight gradient reads the dlogits K-major
    (130, 256, 1024, 1.2, torch.int64),    # vocab % 64 == 0: dHidden reads the weight K-major; fewer than 256 tokens
    (700, 320, 1280, 1.0, torch.int32),    # both, ragged token tiles
]


@pytest.mark.parametrize("n,h,v,temp,ldt", CASES)
def test_forward_vs_oracle(n, h, v, temp, ldt):
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=n + v, label_dtype=ldt)
    w = (w.float() * 8).bfloat16()  # peaky enough that entropy is far from ln V
    lp, ent = linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), temp, "none")
    ref_lp, ref_ent = OM.forward(hid, w, lab, temp)
    assert lp.dtype == torch.float32 and lp.shape == (n,) and ent.shape == (n,)
    assert (lp.cpu() - ref_lp).abs().max() < 1e-3
    assert (ent.cpu() - ref_ent).abs().max() < 1e-3


@pytest.mark.parametrize("dt", [torch.float16, torch.float32])
def test_other_float_dtypes_are_rounded_to_bf16(dt):
    """fp16 / fp32 operands (the reference's op takes any float dtype, kernels.py:517-522): the result is that of
    the bf16-rounded operands, and the gradients come back in the operands' own dtype."""
    n, h, v = 300, 128, 1000
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=31)
    w = (w.float() * 8).bfloat16()
    hd, wd = hid.to(DEV).to(dt).requires_grad_(True), w.to(DEV).to(dt).requires_grad_(True)  # exact in fp32; fp16 rounds
    import sys
    sys.modules["axon_amd.utils.kernel.linear_cross_entropy"]._warned_rounding = False
    with pytest.warns(UserWarning, match="rounded to bfloat16"):  # said once per process
        lp, ent = linear_cross_entropy(hd, wd, lab.to(DEV), 1.0, "none")
    hb, wb = hd.detach().bfloat16().cpu(), wd.detach().bfloat16().cpu()
    ref_lp, ref_ent = OM.forward(hb, wb, lab)
    assert lp.dtype == torch.float32 and (lp.cpu() - ref_lp).abs().max() < 1e-3 and (ent.cpu() - ref_ent).abs().max() < 1e-3
    g = torch.Generator().manual_seed(2)
    g_lp = torch.randn(n, generator=g) / n
    (lp * g_lp.to(DEV)).sum().backward()
    assert hd.grad.dtype == dt and wd.grad.dtype == dt
    ref_dh, ref_dw = OM.backward(g_lp, None, hb, wb, lab, 1.0)
    assert rel_l2(hd.grad, ref_dh) < 2e-2 and rel_l2(wd.grad, ref_dw) < 2e-2


def test_forward_closed_forms_gpu():
    n, h, v = 130, 64, 3000
    hid = torch.randn(n, h).bfloat16()
    lab = torch.randint(0, v, (n,))
    lp, ent = linear_cross_entropy(hid.to(DEV), torch.zeros(v, h).bfloat16().to(DEV), lab.to(DEV), 1.0, "none")
    assert torch.allclose(lp.cpu(), torch.full((n,), -math.log(v)), atol=1e-5)
    assert torch.allclose(ent.cpu(), torch.full((n,), math.log(v)), atol=1e-5)
    # extreme logits stay finite; out-of-range label contributes logit 0
    hid2 = torch.full((4, 64), 30.0).bfloat16()
    w2 = torch.cat([torch.full((1, 64), 2.0), torch.full((1, 64), -2.0), torch.zeros(6, 64)]).bfloat16()
    lp2, ent2 = linear_cross_entropy(hid2.to(DEV), w2.to(DEV), torch.tensor([0, 1, 2, 99]).to(DEV), 1.0, "none")
    assert torch.isfinite(lp2).all() and torch.isfinite(ent2).all() and abs(lp2[0].item()) < 1e-5
    ref = OM.forward(hid2, w2, torch.tensor([0, 1, 2, 0]))[0]
    assert lp2[1].item() == pytest.approx(ref[1].item(), abs=1e-2)
    assert lp2[3].item() == pytest.approx(-3840.0, rel=1e-5)  # 0 - logsumexp


def test_3d_hidden_reductions_and_errors():
    hid, w, lab = W.lmhead_inputs(96, 64, 500, seed=3, label_dtype=torch.int64)
    lp, ent = linear_cross_entropy(hid.view(1, 96, 64).to(DEV), w.to(DEV), lab.view(1, 96).to(DEV), 1.0, "none")
    assert lp.shape == (96,)  # flat, like the reference
    ref = OM.forward(hid, w, lab)[0]
    s, _ = linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), 1.0, "sum")
    mn, _ = linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), 1.0, "mean")
    assert s.item() == pytest.approx(ref.sum().item(), rel=1e-5) and mn.item() == pytest.approx(ref.mean().item(), rel=1e-5)
    with pytest.raises(AssertionError, match="temperature must be a float"):
        linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), 1, "none")
    with pytest.raises(Exception):
        linear_cross_entropy(torch.zeros(4, 40).bfloat16().to(DEV), torch.zeros(8, 40).bfloat16().to(DEV),
                             torch.zeros(4).long().to(DEV), 1.0, "none")  # hidden % 32 != 0
    mod = FusedLinearForPPO()
    lp2, ent2 = mod(hid.view(2, 48, 64).to(DEV), w.to(DEV), lab.view(2, 48).to(DEV).int(), temperature=1.0)
    assert lp2.shape == (2, 48) and torch.allclose(lp2.flatten().cpu(), ref, atol=1e-3)
    lp3, ent3 = FusedLinearForPPO(round_outputs_to_input_dtype=True)(hid.view(2, 48, 64).to(DEV), w.to(DEV),
                                                                      lab.view(2, 48).to(DEV), temperature=1.0)
    assert lp3.dtype == torch.bfloat16 and ent3.dtype == torch.bfloat16  # as fused_linear.py:46
    assert torch.equal(lp3, lp2.bfloat16()) and torch.equal(ent3, ent2.bfloat16())


@pytest.mark.parametrize("n,h,v,temp,ldt", CASES)
@pytest.mark.parametrize("with_entropy", [False, True])
def test_backward_vs_oracle(n, h, v, temp, ldt, with_entropy, head_path):
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=n + v + 1, label_dtype=ldt)
    w = (w.float() * 8).bfloat16()
    g = torch.Generator().manual_seed(5)
    g_lp = torch.randn(n, generator=g) / n
    g_en = torch.randn(n, generator=g) / n if with_entropy else None
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = linear_cross_entropy(hd, wd, lab.to(DEV), temp, "none")
    obj = (lp * g_lp.to(DEV)).sum()
    if with_entropy:
        obj = obj + (ent * g_en.to(DEV)).sum()
    obj.backward()
    assert hd.grad.dtype == torch.bfloat16 and wd.grad.dtype == torch.bfloat16
    ref_dh, ref_dw = OM.backward(g_lp, g_en, hid, w, lab, temp)
    assert rel_l2(hd.grad, ref_dh) < 2e-2
    assert rel_l2(wd.grad, ref_dw) < 2e-2


# ---- logit soft-capping (fused_linear.py:19-23,80-83): DMA-loop and register-loop shapes ----------------
SOFTCAP_CASES = [(300, 96, 777, 0.7, 4.0), (513, 256, 1500, 1.0, 30.0), (64, 128, 1000, 1.3, 2.0)]


@pytest.mark.parametrize("n,h,v,temp,cap", SOFTCAP_CASES)
def test_softcap_forward_backward_vs_oracle(n, h, v, temp, cap, head_path):
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=n + v + 2)
    w = (w.float() * 8).bfloat16()
    g = torch.Generator().manual_seed(6)
    g_lp, g_en = torch.randn(n, generator=g) / n, torch.randn(n, generator=g) / n
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = linear_cross_entropy(hd, wd, lab.to(DEV), temp, "none", None, cap)
    ref_lp, ref_ent = OM.forward(hid, w, lab, temp, softcap=cap)
    assert (lp.cpu() - ref_lp).abs().max() < 1e-3 and (ent.cpu() - ref_ent).abs().max() < 1e-3
    if cap < 30:  # the cap changes the answer on these inputs
        assert (ref_lp - OM.forward(hid, w, lab, temp)[0]).abs().max() > 1e-2
    ((lp * g_lp.to(DEV)).sum() + (ent * g_en.to(DEV)).sum()).backward()
    ref_dh, ref_dw = OM.backward(g_lp, g_en, hid, w, lab, temp, softcap=cap)
    assert rel_l2(hd.grad, ref_dh) < 2e-2 and rel_l2(wd.grad, ref_dw) < 2e-2
    # the module face of the same path
    lp2, ent2 = FusedLinearForPPO()(hid.to(DEV), w.to(DEV), lab.to(DEV), temperature=temp, logit_softcapping=cap)
    assert torch.equal(lp2, lp.detach()) and torch.equal(ent2, ent.detach())


def test_softcap_saturated_logits_and_errors():
    # every logit far beyond the cap: capped logits are +-cap exactly, gradients vanish, nothing overflows
    hid = torch.full((256, 64), 30.0).bfloat16()
    w = torch.cat([torch.full((300, 64), 2.0), torch.full((300, 64), -2.0)]).bfloat16()
    lab = torch.arange(256) % 600
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = linear_cross_entropy(hd, wd, lab.to(DEV), 1.0, "none", None, 10.0)
    ref_lp, ref_ent = OM.forward(hid, w, lab, 1.0, softcap=10.0)
    assert torch.isfinite(lp).all() and (lp.cpu() - ref_lp).abs().max() < 1e-3 and (ent.cpu() - ref_ent).abs().max() < 1e-3
    (lp.sum() + ent.sum()).backward()
    assert hd.grad.float().abs().max() == 0 and wd.grad.float().abs().max() == 0
    with pytest.raises(ValueError):
        linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), 1.0, "none", None, -1.0)


# ---- token-aligned packed layout: roll(ids, -1) before and shift-right after the head, inside the kernels --
def _aligned_reference(hid, w, ids, lens, temp, cap=None):
    """forward_utils.py:131,164-182 on the oracle: labels = roll(ids, -1), outputs shifted right inside each
    sequence, 0 at sequence starts."""
    lp, ent = OM.forward(hid, w, torch.roll(ids, -1), temp, softcap=cap)
    out_lp, out_ent = torch.zeros_like(lp), torch.zeros_like(ent)
    out_lp[1:], out_ent[1:] = lp[:-1], ent[:-1]
    cu = torch.tensor([0] + lens).cumsum(0)
    starts = cu[:-1][cu[:-1] < len(ids)]
    out_lp[starts] = 0
    out_ent[starts] = 0
    return out_lp, out_ent, cu


@pytest.mark.parametrize("n,h,v,lens,cap", [
    (300, 96, 777, [1, 0, 120, 1, 78, 100], None),      # single-token and empty sequences, register loop
    (513, 256, 1500, [256, 1, 256], 4.0),               # DMA loop, boundary on a tile edge, soft-capping
    (64, 128, 1000, [64], None),
])
def test_aligned_packed_layout(n, h, v, lens, cap, head_path):
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs, rolled_labels, shift_packed
    assert sum(lens) == n
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=n + v + 3, label_dtype=torch.int64)
    w = (w.float() * 8).bfloat16()
    temp = 0.9
    ref_lp, ref_ent, cu = _aligned_reference(hid, w, ids, lens, temp, cap)
    cu_d = cu.to(torch.int32).to(DEV)
    flags = _ops.seq_start_flags(cu_d, n)[:n].cpu()
    expect = torch.zeros(n, dtype=torch.uint8)
    expect[[int(a) for a, b in zip(cu[:-1], cu[1:]) if b > a]] = 1
    assert torch.equal(flags, expect)  # bit-exact

    g = torch.Generator().manual_seed(9)
    g_lp, g_en = (torch.randn(n, generator=g) / n).to(DEV), (torch.randn(n, generator=g) / n).to(DEV)
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = packed_logprobs(hd, wd, ids.to(DEV).view(1, -1), cu_d, temp, cap)
    assert (lp.cpu() - ref_lp).abs().max() < 1e-3 and (ent.cpu() - ref_ent).abs().max() < 1e-3
    assert (lp[cu_d[:-1].long()[cu_d[:-1] < n]] == 0).all()
    ((lp * g_lp).sum() + (ent * g_en).sum()).backward()

    # the unfused composition of the same kernels gives the same bits, forward and backward
    h2, w2 = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp_h, ent_h = linear_cross_entropy(h2, w2, rolled_labels(ids.to(DEV)), temp, "none", None, cap)
    lp2, ent2 = shift_packed(lp_h, cu_d), shift_packed(ent_h, cu_d)
    ((lp2 * g_lp).sum() + (ent2 * g_en).sum()).backward()
    assert torch.equal(lp, lp2) and torch.equal(ent, ent2)
    assert torch.equal(hd.grad, h2.grad) and torch.equal(wd.grad, w2.grad)


def test_forward_with_hip_backend_on_a_stub_model():
    """The model-forward mirror (reference dense_common.py:147-235): body model -> hidden states, rolled labels,
    fused head, output object; a config with final_logit_softcapping goes through the capped kernels."""
    import types

    from axon_amd.models.transformers.dense_common import CausalLMOutputForPPO, forward_with_hip_backend
    n, h, v = 300, 128, 1000
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=21, label_dtype=torch.int64)
    w = (w.float() * 8).bfloat16()

    class Body(torch.nn.Module):
        def forward(self, input_ids=None, **kw):
            assert kw["use_cache"] is False and "return_dict" in kw
            return (hid.to(DEV).view(1, n, h),)

    class Model(torch.nn.Module):
        def __init__(self, cap):
            super().__init__()
            self.model = Body()
            self.lm_head = torch.nn.Linear(h, v, bias=False, dtype=torch.bfloat16, device=DEV)
            self.lm_head.weight.data.copy_(w)
            self.config = types.SimpleNamespace(output_attentions=False, output_hidden_states=False,
                                                final_logit_softcapping=cap)

    for cap in (None, 5.0):
        model = Model(cap)
        out = forward_with_hip_backend(model, input_ids=ids.to(DEV).view(1, n), use_cache=False, return_dict=True,
                                       temperature=0.8)
        assert isinstance(out, CausalLMOutputForPPO) and out.log_probs.shape == (n,)
        ref_lp, ref_ent = OM.forward(hid, w, torch.roll(ids, -1), 0.8, softcap=cap)
        assert (out.log_probs.cpu() - ref_lp).abs().max() < 1e-3 and (out.entropy.cpu() - ref_ent).abs().max() < 1e-3
        out.log_probs.sum().backward()
        assert model.lm_head.weight.grad is not None and torch.isfinite(model.lm_head.weight.grad.float()).all()
        # the caller's pre-rolled labels win over the model's own roll
        pre = torch.randint(0, v, (1, n)).to(DEV)
        out2 = forward_with_hip_backend(model, input_ids=ids.to(DEV).view(1, n), use_cache=False, return_dict=True,
                                        temperature=0.8, pre_rolled_labels=pre)
        ref2, _ = OM.forward(hid, w, pre.cpu().view(-1), 0.8, softcap=cap)
        assert (out2.log_probs.detach().cpu() - ref2).abs().max() < 1e-3
    with pytest.raises(NotImplementedError):
        forward_with_hip_backend(Model(None), input_ids=ids.to(DEV).view(1, n), use_cache=False, return_dict=False)


@pytest.mark.parametrize("remove_padding", [True, False])
def test_fsdp_model_forward_mirror(remove_padding):
    """Padded [B, T] micro-batch -> (entropy, log_probs) [B, T] through the model-forward mirror, against the
    oracle evaluated row by row (reference forward_utils.py:185-318: position 0 is 0, position t predicts token t)."""
    import types

    from axon_amd.models.transformers.dense_common import forward_with_hip_backend
    from axon_amd.utils.fsdp.forward_utils import fsdp_model_forward
    b, t, h, v = 4, 96, 128, 1000
    g = torch.Generator().manual_seed(33)
    lens = [96, 40, 1, 77]
    ids = torch.randint(0, v, (b, t), generator=g)
    mask = torch.zeros(b, t, dtype=torch.long)
    for r, n in enumerate(lens):
        mask[r, :n] = 1
    emb = torch.randn(v, h, generator=g).bfloat16()      # the stub body model: an embedding lookup
    w = (torch.randn(v, h, generator=g) * 0.3).bfloat16()

    class Body(torch.nn.Module):
        def forward(self, input_ids=None, **kw):
            return (emb.to(DEV)[input_ids],)

    model = types.SimpleNamespace(
        model=Body(), lm_head=types.SimpleNamespace(weight=w.to(DEV).requires_grad_(True)),
        config=types.SimpleNamespace(output_attentions=False, output_hidden_states=False))
    module = lambda **kw: forward_with_hip_backend(model, **kw)  # noqa: E731
    mb = {"input_ids": ids.to(DEV), "attention_mask": mask.to(DEV),
          "position_ids": torch.arange(t).expand(b, t).to(DEV)}
    ent, lp = fsdp_model_forward(module, mb, 0.9, True, use_remove_padding=remove_padding, use_fused_kernels=True,
                                 ulysses_sp_size=1)
    assert lp.shape == (b, t) and ent.shape == (b, t)
    for r, n in enumerate(lens):
        assert lp[r, 0].item() == 0 and ent[r, 0].item() == 0
        if n > 1:
            ref_lp, ref_ent = OM.forward(emb[ids[r, : n - 1]], w, ids[r, 1:n], 0.9)
            assert (lp[r, 1:n].detach().cpu() - ref_lp).abs().max() < 1e-3
            assert (ent[r, 1:n].detach().cpu() - ref_ent).abs().max() < 1e-3
        if remove_padding:  # slot n holds the last token's (meaningless) prediction, as in the reference
            assert (lp[r, n + 1:] == 0).all() and (ent[r, n + 1:] == 0).all()
    (lp * mask.to(DEV)).sum().backward()
    assert torch.isfinite(model.lm_head.weight.grad.float()).all()
    zero = dict(mb, attention_mask=torch.zeros_like(mb["attention_mask"]))
    e0, l0 = fsdp_model_forward(module, zero, 0.9, True, use_remove_padding=True, use_fused_kernels=True)
    assert (l0 == 0).all() and (e0 == 0).all()
    with pytest.raises(NotImplementedError):
        fsdp_model_forward(module, mb, 0.9, use_remove_padding=True, use_fused_kernels=True, ulysses_sp_size=2)


@pytest.mark.parametrize("chunk", [256, 512, 0])
def test_backward_vocab_chunks_agree(chunk):
    n, h, v = 300, 128, 1000
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=8)
    w = (w.float() * 8).bfloat16()
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    lp, ent, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    g_lp = (torch.randn(n) / n).to(DEV)
    g_en = (torch.randn(n) / n).to(DEV)
    dh, dw = _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0, vocab_chunk=chunk)
    ref_dh, ref_dw = OM.backward(g_lp.cpu(), g_en.cpu(), hid, w, lab, 1.0)
    assert rel_l2(dh, ref_dh) < 2e-2 and rel_l2(dw, ref_dw) < 2e-2


# n, hidden, vocab, chunk, softcap, aligned.  DMA-loop shapes (n, vocab >= 256, hidden % 64 == 0) shift their
# edge tiles back inside the matrix: tiles that share rows with a neighbour, in both directions; chunk
# boundaries inside and at the end of the vocabulary; a last chunk of fewer rows than one tile (its tile
# begins before the chunk); register-loop shapes with clamped tiles and rows beyond the matrix.
STASH_CASES = [
    (516, 256, 1500, 512, 0.0, False),
    (516, 256, 1500, 0, 0.0, True),
    (772, 128, 1100, 1024, 0.0, False),
    (256, 64, 256, 256, 0.0, False),
    (1024, 192, 2048, 512, 3.0, False),
    (300, 96, 777, 256, 0.0, False),
    (301, 96, 777, 512, 4.0, True),
    (64, 128, 1000, 0, 0.0, False),
    (1, 32, 5, 0, 0.0, False),
    # hidden >= 256 and vocab % 8 == 0: the dlogits are written once and the weight gradient reads them K-major;
    # chunks of 512 + 512 + 480 and 512 + 512 + 264 rows (edge tiles shifted back by 32 and 248 rows), one chunk,
    # and a last chunk of 136 rows, which sends the whole call back to the two-copy path
    (516, 256, 1504, 512, 0.0, False),
    (772, 320, 1288, 512, 3.0, True),
    (1100, 256, 2048, 0, 0.0, False),
    (516, 256, 1160, 512, 0.0, False),
    # vocab % 64 == 0 as well: no transposed copy of the weight either (dHidden reads it K-major); fewer than 256
    # tokens run that GEMM on 256 rows of which the last are zero
    (100, 256, 1024, 512, 0.0, False),
    (200, 512, 1280, 0, 2.0, True),
    (772, 256, 1536, 512, 0.0, True),
]


@pytest.mark.parametrize("n,h,v,chunk,cap,aligned", STASH_CASES)
def test_backward_from_stash_vs_recompute_and_oracle(n, h, v, chunk, cap, aligned):
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=n + v + 17)
    w = (w.float() * 8).bfloat16()
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    inv_t = 1.0 / 0.9
    flags = None
    if aligned:
        cu = torch.tensor([0, n // 3, n // 3 + 1, n], dtype=torch.int32, device=DEV)
        flags = _ops.seq_start_flags(cu, n)
    saved = _ops.LMHEAD_STASH
    _ops.LMHEAD_STASH = True
    try:
        lp, ent, lse, eb, stash = _ops.lmhead_forward(hd, wd, ld, inv_t, softcap=cap, seq_start=flags, stash=True)
    finally:
        _ops.LMHEAD_STASH = saved
    assert stash is not None and stash.numel() == _ops.lmhead_stash_bytes(n, h, v) > 2 * n * v
    # the stashing forward returns what the plain one does: the same kernels but for the stores
    lp0, ent0, lse0, eb0 = _ops.lmhead_forward(hd, wd, ld, inv_t, softcap=cap, seq_start=flags)
    assert torch.equal(lp, lp0) and torch.equal(ent, ent0) and torch.equal(lse, lse0) and torch.equal(eb, eb0)
    g = torch.Generator().manual_seed(3)
    g_lp, g_en = (torch.randn(n, generator=g) / n).to(DEV), (torch.randn(n, generator=g) / n).to(DEV)
    for ge in (g_en, None):
        dh_s, dw_s = _ops.lmhead_backward(g_lp, ge, hd, wd, ld, lse, eb, inv_t, vocab_chunk=chunk, softcap=cap,
                                          seq_start=flags, stash=stash)
        dh_r, dw_r = _ops.lmhead_backward(g_lp, ge, hd, wd, ld, lse, eb, inv_t, vocab_chunk=chunk, softcap=cap,
                                          seq_start=flags)
        assert torch.isfinite(dh_s.float()).all() and torch.isfinite(dw_s.float()).all()
        assert rel_l2(dh_s, dh_r.float()) < 5e-3 and rel_l2(dw_s, dw_r.float()) < 5e-3
    if not aligned:
        ref_dh, ref_dw = OM.backward(g_lp.cpu(), None, hid, w, lab, 0.9, softcap=cap or None)
        assert rel_l2(dh_s, ref_dh) < 2e-2 and rel_l2(dw_s, ref_dw) < 2e-2


def test_stash_policy_and_refusals():
    """Shapes whose shifted tiles cannot hand rows over in fours have no stash and fall back to the recompute
    backward; the policy switch; a stash of another shape is refused."""
    assert _ops.lmhead_stash_bytes(513, 256, 1500) == 0 and _ops.lmhead_stash_bytes(516, 256, 1502) == 0
    assert _ops.lmhead_stash_bytes(513, 96, 1501) > 0  # clamped tiles: any shape
    assert _ops.lmhead_stash_bytes(32768, 4096, 151936) == 594 * 128 * 131072 + 594 * 2 * 32768 * 4
    hid, w, lab = W.lmhead_inputs(513, 256, 1500, seed=4)
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    saved = _ops.LMHEAD_STASH
    assert saved is False  # opt-in: by default nothing of size tokens x vocab is kept
    try:
        assert _ops.lmhead_forward(hd, wd, ld, 1.0, stash=True)[4] is None
        _ops.LMHEAD_STASH = True
        assert _ops.lmhead_forward(hd, wd, ld, 1.0, stash=True)[4] is None
        hg, wg = hd.clone().requires_grad_(True), wd.clone().requires_grad_(True)
        linear_cross_entropy(hg, wg, ld, 1.0, "none")[0].sum().backward()  # recompute backward
        assert torch.isfinite(hg.grad.float()).all()
        hid2, w2, lab2 = W.lmhead_inputs(516, 256, 1500, seed=4)
        h2, w2d, l2 = hid2.to(DEV), w2.to(DEV), lab2.to(DEV)
        _ops.LMHEAD_STASH = False
        assert _ops.lmhead_forward(h2, w2d, l2, 1.0, stash=True)[4] is None
        _ops.LMHEAD_STASH = "auto"
        _, _, lse, eb, stash = _ops.lmhead_forward(h2, w2d, l2, 1.0, stash=True)
        assert stash is not None
        _ops.LMHEAD_STASH_MAX_BYTES, keep = 1000, _ops.LMHEAD_STASH_MAX_BYTES
        assert _ops.lmhead_forward(h2, w2d, l2, 1.0, stash=True)[4] is None
        _ops.LMHEAD_STASH_MAX_BYTES = keep
        g = torch.ones(516, device=DEV)
        with pytest.raises(ValueError, match="does not belong"):
            _ops.lmhead_backward(g, None, h2, w2d, l2, lse, eb, 1.0, stash=stash[:-256])
        with pytest.raises(ValueError, match="uint8"):
            _ops.lmhead_backward(g, None, h2, w2d, l2, lse, eb, 1.0, stash=stash.view(torch.int16))
        # no gradient wanted: no stash is made (nothing to check but that it runs and agrees)
        with torch.no_grad():
            lp_ng, _ = linear_cross_entropy(h2, w2d, l2, 1.0, "none")
        assert torch.equal(lp_ng, _ops.lmhead_forward(h2, w2d, l2, 1.0)[0])
    finally:
        _ops.LMHEAD_STASH = saved


def test_backward_properties():
    """dentropy absent == zeros; rows of dlogit sum to zero => identical weight rows give d_hidden = 0;
    linearity in the upstream gradient."""
    n, h, v = 200, 64, 600
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=12)
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    _, _, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    gen = torch.Generator(device=DEV).manual_seed(5)
    g1 = torch.randn(n, device=DEV, generator=gen)
    a = _ops.lmhead_backward(g1, None, hd, wd, ld, lse, eb, 1.0)
    b = _ops.lmhead_backward(g1, torch.zeros(n, device=DEV), hd, wd, ld, lse, eb, 1.0)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    c = _ops.lmhead_backward(2 * g1, None, hd, wd, ld, lse, eb, 1.0)
    assert rel_l2(c[0], 2 * a[0].float()) < 1e-2 and rel_l2(c[1], 2 * a[1].float()) < 1e-2
    same = torch.randn(1, h, generator=torch.Generator().manual_seed(6)).expand(v, h).contiguous().bfloat16().to(DEV)
    _, _, lse2, eb2 = _ops.lmhead_forward(hd, same, ld, 1.0)
    g2 = torch.randn(n, device=DEV, generator=gen)
    dh, _ = _ops.lmhead_backward(g1, g2, hd, same, ld, lse2, eb2, 1.0)
    # exact arithmetic gives 0; what is left is the bf16 rounding of each dlogit (2^-9 relative) times |w|
    bound = 2.0 ** -8 * same.float().abs().max().item() * (g1.abs().max().item() + g2.abs().max().item())
    assert dh.float().abs().max().item() < bound


def test_config2_shape_forward():
    """Qwen2.5-0.5B head shape (config 2): 8192 x 896 x 151936, checked on a token subset."""
    hid, w, lab = W.lmhead_inputs(8192, 896, 151936, seed=2)
    lp, ent = linear_cross_entropy(hid.to(DEV), w.to(DEV), lab.to(DEV), 1.0, "none")
    idx = torch.arange(0, 8192, 61)
    ref_lp, ref_ent = OM.forward(hid[idx], w, lab[idx])
    assert (lp.cpu()[idx] - ref_lp).abs().max() < 1e-3 and (ent.cpu()[idx] - ref_ent).abs().max() < 1e-3
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all()


# ---- materialised-logits path (use_fused_kernels off) --------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,v", [(5, 37), (64, 1000), (33, 4099), (3, 151936)])
def test_logits_path_vs_oracle(dtype, n, v):
    from axon_amd.utils.torch.ops import (entropy_from_logits, logprobs_and_entropy_from_logits,
                                          logprobs_from_logits)
    g = torch.Generator().manual_seed(n * 7 + v)
    logits = (torch.randn(n, v, generator=g) * 3).to(dtype)
    labels = torch.randint(0, v, (n,), generator=g)
    ref_in = logits.float().clone().requires_grad_(True)
    ref_lp, ref_en = OM.logprobs_from_logits(ref_in, labels), OM.entropy_from_logits(ref_in)
    g_lp, g_en = torch.randn(n, generator=g), torch.randn(n, generator=g)
    (ref_lp * g_lp + ref_en * g_en).sum().backward()
    x = logits.to(DEV).requires_grad_(True)
    lp, en = logprobs_and_entropy_from_logits(x, labels.to(DEV))
    assert lp.dtype == torch.float32 and lp.shape == (n,)
    assert (lp.cpu() - ref_lp.detach()).abs().max() < 1e-3 and (en.cpu() - ref_en.detach()).abs().max() < 1e-3
    (lp * g_lp.to(DEV) + en * g_en.to(DEV)).sum().backward()
    # fp32: p = exp(z - lse) carries the rounding of lse (about 1e-6 relative at |lse| = 16) and of the fast exp
    tol = 2e-2 if dtype == torch.bfloat16 else 5e-5
    assert rel_l2(x.grad, ref_in.grad) < tol
    # each function on its own
    x2 = logits.to(DEV).requires_grad_(True)
    lp2 = logprobs_from_logits(x2, labels.to(DEV), inplace_backward=False)
    assert torch.equal(lp2, lp)
    (lp2 * g_lp.to(DEV)).sum().backward()
    ref2 = logits.float().clone().requires_grad_(True)
    (OM.logprobs_from_logits(ref2, labels) * g_lp).sum().backward()
    assert rel_l2(x2.grad, ref2.grad) < tol
    assert torch.equal(entropy_from_logits(logits.to(DEV)), en.detach())


def test_logits_path_inplace_backward_shapes_and_strides():
    from axon_amd.utils.torch.ops import entropy_from_logits_with_chunking, logprobs_from_logits
    g = torch.Generator().manual_seed(5)
    b, t, v = 3, 9, 515
    logits = torch.randn(b, t, v, generator=g)
    labels = torch.randint(0, v, (b, t), generator=g)
    ref_in = logits.clone().requires_grad_(True)
    OM.logprobs_from_logits(ref_in, labels).sum().backward()
    # in-place backward: the gradient is written over the logits' storage (the leaf is a product, as in a model)
    w = torch.ones((), device=DEV, requires_grad=True)
    z = logits.to(DEV) * w
    lp = logprobs_from_logits(z, labels.to(DEV), inplace_backward=True)
    assert lp.shape == (b, t)
    lp.sum().backward()
    assert rel_l2(z, ref_in.grad) < 5e-5  # z now holds d loss / d logits
    # a row stride larger than the vocabulary (a column slice) and rows off a 16-byte boundary
    wide = torch.randn(6, v + 5, generator=g)
    x = wide.to(DEV)[:, 1:v + 1]
    lab = torch.randint(0, v, (6,), generator=g)
    got = logprobs_from_logits(x, lab.to(DEV), inplace_backward=False)
    assert (got.cpu() - OM.logprobs_from_logits(wide[:, 1:v + 1], lab)).abs().max() < 1e-5
    ent = entropy_from_logits_with_chunking(x, chunk_size=2)
    assert (ent.cpu() - OM.entropy_from_logits(wide[:, 1:v + 1])).abs().max() < 1e-5
    with pytest.raises(ValueError, match="fp32 or bf16"):
        logprobs_from_logits(x.half(), lab.to(DEV))


@pytest.mark.parametrize("remove_padding", [True, False])
def test_fsdp_model_forward_non_fused(remove_padding):
    """The model returns logits; log-probabilities and entropy must equal those of the fused branch."""
    from types import SimpleNamespace
    from axon_amd.utils.fsdp.forward_utils import fsdp_model_forward
    g = torch.Generator().manual_seed(9)
    b, t, h, v = 3, 12, 64, 300
    emb = (torch.randn(v, h, generator=g) * 0.5).to(DEV)
    w = (torch.randn(v, h, generator=g) * 0.3).to(torch.bfloat16).to(DEV)

    class LogitsModel(torch.nn.Module):
        def forward(self, input_ids=None, attention_mask=None, position_ids=None, use_cache=False):
            hidden = emb[input_ids].to(torch.bfloat16)
            return SimpleNamespace(logits=(hidden.float() @ w.float().t()))

    ids = torch.randint(0, v, (b, t), generator=g)
    mask = torch.ones(b, t, dtype=torch.int64)
    mask[1, 8:] = 0
    mask[2, 5:] = 0
    batch = {"input_ids": ids.to(DEV), "attention_mask": mask.to(DEV),
             "position_ids": torch.arange(t).expand(b, t).to(DEV)}
    ent, lp = fsdp_model_forward(LogitsModel(), batch, 0.7, True, use_remove_padding=remove_padding,
                                 use_fused_kernels=False)
    assert lp.shape == (b, t) and ent.shape == (b, t) and (lp[:, 0] == 0).all() and (ent[:, 0] == 0).all()
    logits = (emb[ids.to(DEV)].to(torch.bfloat16).float() @ w.float().t()).cpu() / 0.7
    ref_lp = OM.logprobs_from_logits(logits[:, :-1], ids[:, 1:])
    ref_en = OM.entropy_from_logits(logits[:, :-1])
    valid = (mask[:, 1:] > 0) if remove_padding else torch.ones(b, t - 1, dtype=torch.bool)
    assert ((lp.cpu()[:, 1:] - ref_lp).abs() * valid).max() < 1e-3
    assert ((ent.cpu()[:, 1:] - ref_en).abs() * valid).max() < 1e-3


# ---- rows without an upstream gradient are left out of the backward's GEMMs --------------------------------
def _head_state(n, h, v, seed, ldt=torch.int32):
    hid, w, lab = W.lmhead_inputs(n, h, v, seed=seed, label_dtype=ldt)
    w = (w.float() * 8).bfloat16()
    hd, wd, ld = hid.to(DEV), w.to(DEV), lab.to(DEV)
    _, _, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
    return hid, w, lab, hd, wd, ld, lse, eb


def test_active_rows_index_known_answers():
    """The C entry point against a list written by hand and against numpy on a ragged case."""
    from axon_amd import _lib
    g_lp = torch.tensor([0.0, 1.0, 0.0, -0.0, 2.0, 0.0, float("nan"), 0.0], device=DEV)
    g_en = torch.tensor([0.0, 0.0, 3.0, 0.0, 0.0, 0.0, 0.0, 0.0], device=DEV)
    idx, rank, cnt = _ops._active_rows(g_lp, g_en, None, 8)
    assert cnt == 4 and idx[:4].tolist() == [1, 2, 4, 6]
    assert rank.tolist() == [-1, 0, 1, -1, 2, -1, 3, -1]
    idx, rank, cnt = _ops._active_rows(g_lp, None, None, 8)
    assert cnt == 3 and idx[:3].tolist() == [1, 4, 6]
    # aligned layout: hidden row n owns position n + 1 (the last row owns position 0); starts never count
    starts = torch.tensor([1, 0, 0, 0, 1, 0, 0, 0], dtype=torch.uint8, device=DEV)
    g = torch.tensor([5.0, 1.0, 0.0, 1.0, 7.0, 0.0, 1.0, 1.0], device=DEV)
    idx, rank, cnt = _ops._active_rows(g, None, starts, 8)
    assert cnt == 4 and idx[:4].tolist() == [0, 2, 5, 6]  # rows 3 and 7 point at starts, 1 and 4 at zeros
    # more rows than one walk of the workgroup, ragged tail
    n = 5000
    gen = torch.Generator().manual_seed(3)
    big = torch.randn(n, generator=gen) * (torch.rand(n, generator=gen) < 0.4)
    idx, rank, cnt = _ops._active_rows(big.to(DEV), None, None, n)
    want = torch.nonzero(big).flatten()
    assert cnt == len(want) and torch.equal(idx[:cnt].cpu().long(), want)
    inv = torch.full((n,), -1, dtype=torch.int32)
    inv[want] = torch.arange(len(want), dtype=torch.int32)
    assert torch.equal(rank.cpu(), inv)
    assert _lib.load().axon_lmhead_active_rows(None, None, None, 4, None, None, None, None) != 0  # no count pointer


@pytest.mark.parametrize("n,h,v,ldt,with_entropy", [(700, 256, 1500, torch.int32, True),
                                                    (300, 96, 777, torch.int64, False),
                                                    (1030, 128, 2000, torch.int32, True)])
def test_backward_skips_rows_without_gradient(n, h, v, ldt, with_entropy):
    hid, w, lab, hd, wd, ld, lse, eb = _head_state(n, h, v, n + v, ldt)
    gen = torch.Generator().manual_seed(n)
    live = torch.rand(n, generator=gen) < 0.45  # the rest are prompt-like rows: exact zeros
    g_lp = torch.randn(n, generator=gen) / n * live
    g_en = torch.randn(n, generator=gen) / n * live if with_entropy else None
    args = (g_lp.to(DEV), None if g_en is None else g_en.to(DEV), hd, wd, ld, lse, eb, 1.0)
    dh, dw = _ops.lmhead_backward(*args, skip_zero_rows=True)
    dh_all, dw_all = _ops.lmhead_backward(*args)  # the default: every row, no readback
    assert (dh[~live.to(DEV)] == 0).all() and (dh_all[~live.to(DEV)] == 0).all()
    # a d_hidden row is a sum over the vocabulary only: the row set does not change it
    assert torch.equal(dh, dh_all)
    assert rel_l2(dw, dw_all) < 1e-3  # d_weight sums over fewer rows, in another order
    ref_dh, ref_dw = OM.backward(g_lp, g_en, hid, w, lab, 1.0)
    assert rel_l2(dh, ref_dh) < 2e-2 and rel_l2(dw, ref_dw) < 2e-2


def test_backward_row_skipping_in_the_aligned_layout_and_all_zero(head_path):
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    n, h, v, lens = 600, 128, 1200, [200, 1, 150, 249]
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=77, label_dtype=torch.int64)
    w = (w.float() * 8).bfloat16()
    cu = W.cu_from_lengths(lens).to(DEV)
    # prompt positions (the first 60 % of every sequence) carry no gradient
    pos = torch.arange(n)
    resp = torch.zeros(n, dtype=torch.bool)
    for a, b in zip(cu.tolist()[:-1], cu.tolist()[1:]):
        resp |= (pos >= a + int(0.6 * (b - a))) & (pos < b)
    gen = torch.Generator().manual_seed(8)
    g_lp = (torch.randn(n, generator=gen) / n * resp).to(DEV)
    grads = []
    for skip in (True, False):
        hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
        lp, _ = packed_logprobs(hd, wd, ids.to(DEV).view(1, -1), cu, 0.9)
        _ops.SKIP_ZERO_GRAD_ROWS = skip
        try:
            (lp * g_lp).sum().backward()
        finally:
            _ops.SKIP_ZERO_GRAD_ROWS = False
        grads.append((hd.grad, wd.grad))
    if head_path == "recompute":  # the same kernels over fewer rows: d_hidden agrees bit for bit
        assert torch.equal(grads[0][0], grads[1][0]) and rel_l2(grads[0][1], grads[1][1]) < 1e-3
    else:  # the row-skipping backward recomputes; the all-rows one decoded the forward's stash
        assert rel_l2(grads[0][0], grads[1][0].float()) < 5e-3 and rel_l2(grads[0][1], grads[1][1].float()) < 5e-3
    assert (grads[0][0].abs().sum(1) > 0).sum().item() <= int(resp.sum())  # only rows that predict a response token
    # nothing to do at all: exact zeros, no GEMM
    _, _, lab, hd, wd, ld, lse, eb = _head_state(64, 64, 500, 5)
    dh, dw = _ops.lmhead_backward(torch.zeros(64, device=DEV), None, hd, wd, ld, lse, eb, 1.0, skip_zero_rows=True)
    assert not dh.any() and not dw.any() and dh.dtype == torch.bfloat16 and dw.shape == wd.shape


def test_packed_logprobs_with_response_mask_leaves_prompt_rows_out(head_path):
    """Optional response mask: prompt positions come back as 0, everything the loss can see is unchanged."""
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    n, h, v, lens = 700, 128, 1300, [300, 1, 0, 250, 149]
    hid, w, ids = W.lmhead_inputs(n, h, v, seed=21, label_dtype=torch.int64)
    w = (w.float() * 8).bfloat16()
    cu = W.cu_from_lengths(lens).to(DEV)
    pos = torch.arange(n)
    resp = torch.zeros(n)
    for a, b in zip(cu.tolist()[:-1], cu.tolist()[1:]):
        resp[(pos >= a + (b - a) // 2) & (pos < b)] = 1  # second half of every sequence (a one-token sequence whole)
    resp_d = resp.to(DEV)
    gen = torch.Generator().manual_seed(2)
    g_lp, g_en = (torch.randn(n, generator=gen) / n).to(DEV), (torch.randn(n, generator=gen) / n).to(DEV)
    outs = []
    for m in (None, resp_d):
        hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
        lp, ent = packed_logprobs(hd, wd, ids.to(DEV), cu, 0.8, None, response_mask=m)
        ((lp * g_lp * resp_d).sum() + (ent * g_en * resp_d).sum()).backward()
        outs.append((lp.detach(), ent.detach(), hd.grad, wd.grad))
    (lp0, ent0, dh0, dw0), (lp1, ent1, dh1, dw1) = outs
    starts = cu[:-1].long()[cu[:-1] < n]
    seen = resp_d.clone()
    seen[starts] = 0
    assert (lp1[seen == 0] == 0).all() and (ent1[seen == 0] == 0).all()
    assert torch.equal(lp1[seen > 0], lp0[seen > 0]) and torch.equal(ent1[seen > 0], ent0[seen > 0])
    if head_path == "recompute":
        assert torch.equal(dh1, dh0) and rel_l2(dw1, dw0) < 1e-3
    else:  # the two runs may differ in which backward their shapes allow
        assert rel_l2(dh1, dh0.float()) < 5e-3 and rel_l2(dw1, dw0.float()) < 5e-3
    ref_lp, ref_ent, _ = _aligned_reference(hid, w, ids, lens, 0.8)
    assert ((lp1.cpu() - ref_lp) * seen.cpu()).abs().max() < 1e-3
    assert ((ent1.cpu() - ref_ent) * seen.cpu()).abs().max() < 1e-3
    # an all-zero mask: nothing runs, zeros come back and the gradients are zero
    hd, wd = hid.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    lp, ent = packed_logprobs(hd, wd, ids.to(DEV), cu, 0.8, None, response_mask=torch.zeros(n, device=DEV))
    (lp.sum() + ent.sum()).backward()
    assert not lp.any() and not ent.any() and not hd.grad.any() and not wd.grad.any()
    with pytest.raises(ValueError):
        packed_logprobs(hd, wd, ids.to(DEV), cu, 0.8, None, response_mask=torch.zeros(n - 1, device=DEV))


@pytest.mark.parametrize("remove_padding", [True, False])
def test_fsdp_model_forward_skip_prompt_rows(remove_padding):
    """Opt-in: positions outside the response mask come back as 0; inside it nothing changes, values or gradients."""
    import types

    from axon_amd.models.transformers.dense_common import forward_with_hip_backend
    from axon_amd.utils.fsdp.forward_utils import fsdp_model_forward
    b, t, h, v = 4, 96, 128, 1000
    g = torch.Generator().manual_seed(35)
    lens, prompts = [96, 40, 1, 77], [30, 39, 0, 20]  # valid tokens and leading prompt tokens per row
    ids = torch.randint(0, v, (b, t), generator=g)
    att, resp = torch.zeros(b, t, dtype=torch.long), torch.zeros(b, t)
    for r, (n, p) in enumerate(zip(lens, prompts)):
        att[r, :n] = 1
        resp[r, p:n] = 1
    emb = torch.randn(v, h, generator=g).bfloat16()
    w = (torch.randn(v, h, generator=g) * 0.3).bfloat16()

    class Body(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Parameter(emb.to(DEV))

        def forward(self, input_ids=None, **kw):
            return (self.emb[input_ids],)

    res = []
    for skip in (False, True):
        model = types.SimpleNamespace(
            model=Body(), lm_head=types.SimpleNamespace(weight=w.to(DEV).requires_grad_(True)),
            config=types.SimpleNamespace(output_attentions=False, output_hidden_states=False))
        module = lambda **kw: forward_with_hip_backend(model, **kw)  # noqa: E731
        mb = {"input_ids": ids.to(DEV), "attention_mask": att.to(DEV), "response_mask": resp.to(DEV),
              "position_ids": torch.arange(t).expand(b, t).to(DEV)}
        ent, lp = fsdp_model_forward(module, mb, 0.9, True, use_remove_padding=remove_padding,
                                     use_fused_kernels=True, skip_prompt_rows=skip)
        ((lp * resp.to(DEV)).sum() + 0.3 * (ent * resp.to(DEV)).sum()).backward()
        res.append((lp.detach(), ent.detach(), model.lm_head.weight.grad, model.model.emb.grad))
    (lp0, ent0, dw0, de0), (lp1, ent1, dw1, de1) = res
    seen = resp.to(DEV).clone()
    seen[:, 0] = 0  # position 0 has no prediction
    assert (lp1[seen == 0] == 0).all() and (ent1[seen == 0] == 0).all()
    # fewer rows can put the head on its other main loop (another summation order over the hidden size)
    assert (lp1 - lp0)[seen > 0].abs().max() < 1e-5 and (ent1 - ent0)[seen > 0].abs().max() < 1e-5
    assert rel_l2(dw1, dw0) < 1e-3 and rel_l2(de1, de0) < 1e-3


@pytest.mark.parametrize("from_stash", [False, True])
def test_default_backward_has_no_readback_and_replays_in_a_hip_graph(from_stash):
    """The default backward only enqueues launches, with or without the forward's stash: it can be captured
    into a HIP graph, and every replay is bit-identical to the eager call (eager work and synchronisations
    between the replays)."""
    n, h, v = 1024, 256, 2048
    hid, w, lab, hd, wd, ld, lse, eb = _head_state(n, h, v, 91)
    kw = {"vocab_chunk": 1024}  # two chunks
    if from_stash:
        saved, _ops.LMHEAD_STASH = _ops.LMHEAD_STASH, True
        try:
            kw["stash"] = _ops.lmhead_forward(hd, wd, ld, 1.0, stash=True)[4]
        finally:
            _ops.LMHEAD_STASH = saved
        assert kw["stash"] is not None
    gen = torch.Generator().manual_seed(9)
    g_lp = (torch.randn(n, generator=gen) / n).to(DEV)
    g_en = (torch.randn(n, generator=gen) / n).to(DEV)
    dh_e, dw_e = _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0, **kw)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            dh_g, dw_g = _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0, **kw)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        dh_g.zero_(); dw_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dh_g, dh_e) and torch.equal(dw_g, dw_e)
        again = _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0, **kw)  # eager work in between
        torch.cuda.synchronize()
        assert torch.equal(again[0], dh_e) and torch.equal(again[1], dw_e)
    with torch.cuda.stream(side):
        with pytest.raises(Exception):
            with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
                _ops.lmhead_backward(g_lp, g_en, hd, wd, ld, lse, eb, 1.0, skip_zero_rows=True)
    torch.cuda.synchronize()
