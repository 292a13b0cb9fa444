"""Pins oracle.lmhead.  The reference's tests hold no vector for the fused LM head
(``linear_cross_entropy``, ``FusedLinearForPPO`` have no test), so the oracle is pinned by
what the mathematics fixes: library routines, closed forms, invariances, fp64 brute force,
autograd of the textbook forward and finite differences."""

import math

import pytest
import torch

from oracle import lmhead as M


def _case(n=6, h=16, v=40, seed=0):
    g = torch.Generator().manual_seed(seed)
    hid = torch.randn(n, h, generator=g).bfloat16()
    w = (torch.randn(v, h, generator=g) * 0.3).bfloat16()
    lab = torch.randint(0, v, (n,), generator=g)
    return hid, w, lab


def test_forward_is_log_softmax_gather_and_entropy():
    # reference tests/utils/torch/test_ops.py:36-42,119-126 define the same identities
    hid, w, lab = _case()
    lp, ent = M.forward(hid, w, lab, temperature=0.7)
    logits = (hid.double() @ w.double().t()) / 0.7
    ref_lp = torch.log_softmax(logits, -1).gather(-1, lab[:, None]).squeeze(-1)
    p = torch.softmax(logits, -1)
    ref_ent = -(p * torch.log(p)).sum(-1)
    assert torch.allclose(lp.double(), ref_lp, atol=1e-5)
    assert torch.allclose(ent.double(), ref_ent, atol=1e-5)


def test_forward_bruteforce_fp64_python_loops():
    hid, w, lab = _case(n=3, h=8, v=11, seed=2)
    lp, ent = M.forward(hid, w, lab, temperature=1.3)
    for i in range(3):
        logits = [sum(float(hid[i, k]) * float(w[j, k]) for k in range(8)) / 1.3 for j in range(11)]
        mx = max(logits)
        z = sum(math.exp(x - mx) for x in logits)
        lse = mx + math.log(z)
        probs = [math.exp(x - lse) for x in logits]
        assert lp[i].item() == pytest.approx(logits[int(lab[i])] - lse, abs=1e-5)
        assert ent[i].item() == pytest.approx(-sum(p * math.log(p) for p in probs), abs=1e-5)


def test_forward_closed_forms_and_invariances():
    n, h, v = 4, 16, 50
    hid = torch.randn(n, h).bfloat16()
    lab = torch.randint(0, v, (n,))
    lp, ent = M.forward(hid, torch.zeros(v, h).bfloat16(), lab)
    assert torch.allclose(lp, torch.full((n,), -math.log(v)), atol=1e-6)  # uniform -> -ln V / ln V
    assert torch.allclose(ent, torch.full((n,), math.log(v)), atol=1e-6)
    # one dominant class -> logprob ~ 0, entropy ~ 0
    w = torch.zeros(v, h)
    w[7] = 50.0 * hid[0].float() / hid[0].float().norm() ** 2 * 4
    lp1, ent1 = M.forward(hid[:1], w.bfloat16(), torch.tensor([7]))
    assert abs(lp1.item()) < 1e-3 and ent1.item() < 1e-2
    # temperature t == scaling the weight by 1/t (exact for powers of two in bf16)
    hid2, w2, lab2 = _case(seed=5)
    a = M.forward(hid2, w2, lab2, temperature=2.0)
    b = M.forward(hid2, (w2.float() / 2).bfloat16(), lab2, temperature=1.0)
    assert torch.allclose(a[0], b[0], atol=1e-6) and torch.allclose(a[1], b[1], atol=1e-6)
    # chunking does not change the result (test_ops.py:140-144)
    c = M.forward(hid2, w2, lab2, temperature=2.0, chunk=2)
    assert torch.allclose(a[0], c[0], atol=1e-6) and torch.allclose(a[1], c[1], atol=1e-6)


def test_forward_extreme_logits_finite():  # test_ops.py:602-618
    hid = torch.full((2, 16), 30.0).bfloat16()
    w = torch.cat([torch.full((1, 16), 2.0), torch.full((1, 16), -2.0), torch.zeros(3, 16)]).bfloat16()
    lp, ent = M.forward(hid, w, torch.tensor([0, 1]))
    assert torch.isfinite(lp).all() and torch.isfinite(ent).all()
    assert lp[0].item() == pytest.approx(0.0, abs=1e-6)


def test_backward_matches_autograd_of_textbook_forward():
    hid, w, lab = _case(n=7, h=16, v=33, seed=7)
    g1, g2 = torch.randn(7), torch.randn(7)
    for temp in (1.0, 0.6):
        hf = hid.float().requires_grad_(True)
        wf = w.float().requires_grad_(True)
        logits = (hf @ wf.t()) / temp
        lp = torch.log_softmax(logits, -1).gather(-1, lab[:, None]).squeeze(-1)
        p = torch.softmax(logits, -1)
        ent = torch.logsumexp(logits, -1) - (p * logits).sum(-1)
        ((lp * g1).sum() + (ent * g2).sum()).backward()
        dh, dw = M.backward(g1, g2, hid, w, lab, temperature=temp, chunk=3)
        assert torch.allclose(dh, hf.grad, atol=1e-5, rtol=1e-4)
        assert torch.allclose(dw, wf.grad, atol=1e-5, rtol=1e-4)
        dh0, dw0 = M.backward(g1, None, hid, w, lab, temperature=temp)  # dentropy absent == zeros
        dh1, dw1 = M.backward(g1, torch.zeros(7), hid, w, lab, temperature=temp)
        assert torch.allclose(dh0, dh1) and torch.allclose(dw0, dw1)


def test_backward_finite_differences_fp64():
    n, h, v = 2, 4, 6
    g = torch.Generator().manual_seed(11)
    hid = torch.randn(n, h, generator=g, dtype=torch.float64)
    w = torch.randn(v, h, generator=g, dtype=torch.float64)
    lab = torch.tensor([1, 4])
    g1 = torch.tensor([0.7, -1.1], dtype=torch.float64)
    g2 = torch.tensor([0.3, 0.9], dtype=torch.float64)

    def f(hm, wm):
        logits = hm @ wm.t()
        lse = torch.logsumexp(logits, -1)
        lp = logits.gather(-1, lab[:, None]).squeeze(-1) - lse
        ent = lse - (torch.softmax(logits, -1) * logits).sum(-1)
        return ((lp * g1).sum() + (ent * g2).sum()).item()

    # the oracle works in fp32 on its inputs; feed values exactly representable in bf16
    hb, wb = hid.bfloat16(), w.bfloat16()
    dh, dw = M.backward(g1.float(), g2.float(), hb, wb, lab)
    hd, wd = hb.double(), wb.double()
    eps = 1e-6
    for i in range(n):
        for k in range(h):
            d = torch.zeros_like(hd); d[i, k] = eps
            fd = (f(hd + d, wd) - f(hd - d, wd)) / (2 * eps)
            assert dh[i, k].item() == pytest.approx(fd, abs=2e-4)
    for j in range(v):
        for k in range(h):
            d = torch.zeros_like(wd); d[j, k] = eps
            fd = (f(hd, wd + d) - f(hd, wd - d)) / (2 * eps)
            assert dw[j, k].item() == pytest.approx(fd, abs=2e-4)


def test_dlogits_rows_sum_to_zero():
    """sum_v dlogit = 0 per token, hence d_hidden = 0 when every weight row is the same."""
    n, h, v = 5, 16, 20
    hid = torch.randn(n, h).bfloat16()
    w = torch.randn(1, h).expand(v, h).contiguous().bfloat16()
    dh, _ = M.backward(torch.randn(n), torch.randn(n), hid, w, torch.randint(0, v, (n,)))
    assert dh.abs().max() < 1e-5


# ---- logit soft-capping (fused_linear.py:19-23,80-83) -------------------------------------------------
def test_softcap_forward_closed_forms():
    hid, w, lab = _case(n=5, h=16, v=24, seed=3)
    w = (w.float() * 8).bfloat16()  # logits large enough for the cap to bite
    lp, ent = M.forward(hid, w, lab, temperature=0.8, softcap=5.0)
    raw = hid.double() @ w.double().t()
    logits = torch.tanh(raw / 5.0) * 5.0 / 0.8  # cap first, temperature second
    ref_lp = torch.log_softmax(logits, -1).gather(-1, lab[:, None]).squeeze(-1)
    p = torch.softmax(logits, -1)
    assert torch.allclose(lp.double(), ref_lp, atol=1e-5)
    assert torch.allclose(ent.double(), -(p * torch.log(p)).sum(-1), atol=1e-5)
    assert (raw.abs() > 5.0).any() and not torch.allclose(lp, M.forward(hid, w, lab, temperature=0.8)[0], atol=1e-2)
    # a cap far above every logit is the identity; capped logits lie in (-cap, cap), so the
    # log-probabilities are bounded below by -(2 cap / T + ln V)
    lp_inf, ent_inf = M.forward(hid, w, lab, temperature=0.8, softcap=1e6)
    lp0, ent0 = M.forward(hid, w, lab, temperature=0.8)
    assert torch.allclose(lp_inf, lp0, atol=1e-4) and torch.allclose(ent_inf, ent0, atol=1e-4)
    assert (lp >= -(2 * 5.0 / 0.8 + math.log(24))).all()


def test_softcap_backward_matches_autograd_and_finite_differences():
    hid, w, lab = _case(n=4, h=8, v=12, seed=5)
    w = (w.float() * 6).bfloat16()
    g1, g2 = torch.randn(4), torch.randn(4)
    cap, temp = 3.0, 0.7

    def f(hm, wm):
        logits = torch.tanh((hm @ wm.t()) / cap) * cap / temp
        lse = torch.logsumexp(logits, -1)
        lp = logits.gather(-1, lab[:, None]).squeeze(-1) - lse
        ent = lse - (torch.softmax(logits, -1) * logits).sum(-1)
        return (lp * g1.to(hm.dtype)).sum() + (ent * g2.to(hm.dtype)).sum()

    hf, wf = hid.float().requires_grad_(True), w.float().requires_grad_(True)
    f(hf, wf).backward()
    dh, dw = M.backward(g1, g2, hid, w, lab, temperature=temp, chunk=3, softcap=cap)
    assert torch.allclose(dh, hf.grad, atol=1e-5, rtol=1e-4)
    assert torch.allclose(dw, wf.grad, atol=1e-5, rtol=1e-4)
    hd, wd = hid.double(), w.double()
    eps = 1e-6
    for (i, k) in [(0, 0), (1, 3), (3, 7)]:
        d = torch.zeros_like(hd); d[i, k] = eps
        fd = (f(hd + d, wd) - f(hd - d, wd)).item() / (2 * eps)
        assert dh[i, k].item() == pytest.approx(fd, abs=2e-4)
    for (j, k) in [(0, 0), (5, 2), (11, 7), (int(lab[0]), 1)]:
        d = torch.zeros_like(wd); d[j, k] = eps
        fd = (f(hd, wd + d) - f(hd, wd - d)).item() / (2 * eps)
        assert dw[j, k].item() == pytest.approx(fd, abs=2e-4)


# ---- materialised-logits path (ops.py:39-120): closed forms and the textbook definitions ---------------------
def test_logits_oracle_closed_forms():
    v = 37
    z = torch.zeros(3, v)
    lab = torch.tensor([0, 5, 36])
    assert torch.allclose(M.logprobs_from_logits(z, lab), torch.full((3,), -math.log(v)), atol=1e-6)
    assert torch.allclose(M.entropy_from_logits(z), torch.full((3,), math.log(v)), atol=1e-6)
    peak = torch.full((1, v), -50.0)
    peak[0, 7] = 50.0
    assert abs(float(M.logprobs_from_logits(peak, torch.tensor([7])))) < 1e-6
    assert abs(float(M.entropy_from_logits(peak))) < 1e-6
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, v, generator=g, dtype=torch.float64)
    lab = torch.randint(0, v, (4,), generator=g)
    p = torch.softmax(x, -1)
    assert torch.allclose(M.entropy_from_logits(x.float()).double(), -(p * p.log()).sum(-1), atol=1e-6)
    assert torch.allclose(M.logprobs_from_logits(x.float(), lab).double(), p.log()[torch.arange(4), lab], atol=1e-6)
    assert torch.allclose(M.entropy_from_logits(x.float() + 3.0), M.entropy_from_logits(x.float()), atol=1e-5)


# ---- the bf16 torch path timed as the CPU baseline (fused_linear.py run in bf16) -----------------------------
def test_bf16_torch_path_against_the_fp32_oracle():
    """`forward_bf16_torch_path` / `backward_bf16_torch_path` are what `bench.py` times on the host cores.  The
    same formulas evaluated in fp32 are `forward` / `backward`; run in bf16 the results agree to bf16 accuracy:
    logits rounded to 8 bits (relative 2^-9) move a log-prob by a few hundredths, gradients by a few per cent.
    In fp32 the two pairs of functions coincide to rounding, which pins the formulas themselves."""
    g = torch.Generator().manual_seed(4)
    n, h, v = 700, 64, 900  # more than one 512-token chunk
    hid = torch.randn(n, h, generator=g)
    w = torch.randn(v, h, generator=g) * 0.2
    lab = torch.randint(0, v, (n,), generator=g)
    dlogp = torch.randn(n, generator=g) / n
    # fp32 inputs: the bf16-path functions are the same arithmetic as the oracle
    lp32, ent32 = M.forward_bf16_torch_path(hid, w, lab, 0.7)
    ref_lp, ref_ent = M.forward(hid, w, lab, 0.7)
    assert torch.allclose(lp32, ref_lp, atol=1e-5) and torch.allclose(ent32, ref_ent, atol=1e-5)
    dh32, dw32 = M.backward_bf16_torch_path(dlogp, hid, w, lab, 0.7)
    ref_dh, ref_dw = M.backward(dlogp, None, hid, w, lab, 0.7, round_dlogits_bf16=False)
    rel = lambda a, b: ((a.double() - b.double()).norm() / b.double().norm()).item()  # noqa: E731
    assert rel(dh32, ref_dh) < 1e-5 and rel(dw32, ref_dw) < 1e-5
    # bf16 inputs: bf16 accuracy
    hb, wb = hid.bfloat16(), w.bfloat16()
    lpb, entb = M.forward_bf16_torch_path(hb, wb, lab, 0.7)
    ref_lp, ref_ent = M.forward(hb, wb, lab, 0.7)
    assert lpb.dtype == torch.bfloat16 and (lpb.float() - ref_lp).abs().max() < 0.1
    assert (entb.float() - ref_ent).abs().max() < 0.1
    dhb, dwb = M.backward_bf16_torch_path(dlogp, hb, wb, lab, 0.7)
    ref_dh, ref_dw = M.backward(dlogp, None, hb, wb, lab, 0.7)
    assert dhb.dtype == torch.bfloat16 and rel(dhb, ref_dh) < 5e-2 and rel(dwb, ref_dw) < 5e-2
