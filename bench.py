#!/usr/bin/env python3
"""Benchmark of the trainer-side per-token hot path on one MI355X.

One step = GRPO advantage -> fused LM-head log-prob/entropy forward (label roll and shift inside) ->
PPO (DAPO clip) loss forward+backward -> LM-head backward (dHidden, dWeight), on
synthetic inputs already resident in HBM.  Default workload: Qwen3-8B head shape,
32768 packed tokens, hidden 4096, vocab 151936, bf16.  The headline runs head forward, loss and
head backward block of tokens by block in one autograd node (a stash of fixed size, no logit
computed twice); the same step with the head as a plain autograd function whose backward
recomputes the logits is timed beside it.

Prints ONE JSON line: trained tokens/s, the MFMA roofline of the dominant kernel
(HIP-event times over the timed region) and the CPU port of the reference torch path
timed on this host's cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published

WORKLOADS = {
    # name: (tokens, hidden, vocab, group size, seed)
    "qwen3-8b": (32768, 4096, 151936, 8, 3),
    "qwen2.5-0.5b": (8192, 896, 151936, 8, 2),
    "gpt-oss": (16384, 2880, 201088, 16, 5),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="qwen3-8b", choices=sorted(WORKLOADS))
    ap.add_argument("--tokens", type=int, default=0, help="override the token count (debugging)")
    ap.add_argument("--vocab-chunk", type=int, default=0)
    ap.add_argument("--head-backward", choices=("blocked-stash", "recompute", "stash"), default="blocked-stash",
                    help="where the headline's backward takes its dlogits from: the stash of one block of tokens "
                         "(forward, loss and backward block by block in one autograd node; 2 bytes x block x vocab "
                         "held whatever the token count), a recompute of the logits (head, loss and backward as "
                         "separate autograd functions, nothing of size tokens x vocab in memory), or a stash of "
                         "ALL tokens kept from the forward to the backward (opt-in)")
    ap.add_argument("--block-tokens", type=int, default=8192, help="tokens per block of the blocked-stash step")
    ap.add_argument("--dw-group", type=int, default=0,
                    help="blocks that share one weight-gradient GEMM in the blocked-stash step (0: the library's default)")
    ap.add_argument("--no-variants", dest="variants", action="store_false",
                    help="skip the short measurements of the same step on the other head-backward paths")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget; 0 disables it")
    ap.add_argument("--prompt-fraction", type=float, default=1 / 3,
                    help="after the headline, time the step again with this leading share of every sequence "
                         "masked as prompt; 0 disables it")
    ap.add_argument("--hbm-tokens", type=int, default=1 << 26,
                    help="token count for the HBM-bound stage-2/3 kernels' bandwidth figures; 0 disables them")
    ap.add_argument("--no-calibrate", dest="calibrate", action="store_false",
                    help="skip the plain-GEMM calibration (torch.matmul and the bare main loop on the dominant shape)")
    ap.add_argument("--no-other-workloads", dest="other_workloads", action="store_false",
                    help="skip the short runs of the other head shapes (Qwen2.5-0.5B, GPT-OSS)")
    ap.add_argument("--gemm-probe", choices=("hipblaslt", "axon"),
                    help="run three plain bf16 GEMMs of the dominant kernel's shape through torch.matmul or through "
                         "the fused kernels' main loop (axon_gemm_nt_bf16), then exit: the command the rocprofv3 --pmc "
                         "passes that compare the two are taken on")
    ap.add_argument("--traffic-probe", choices=("blocked-stash", "recompute", "stash"),
                    help="run a 1 GiB calibration copy, then one head forward and backward on the named "
                         "head-backward path, then exit: the command the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "passes are taken on")
    return ap.parse_args()


def cpu_baseline(hid, w, lab, budget_s, check=None):
    """The reference torch path (bf16 matmul, 512-token chunks) + PPO loss, ported in oracle/,
    timed on a token sample sized to the budget.  Cost is linear in tokens (W is fixed).

    This leg is the only place the benchmark touches `oracle/`.  `check = (idx, logprob)` also
    compares the GPU log-probs of the token subset `idx` (token p is predicted from hidden p - 1)
    with the fp32 restatement and refuses to report a baseline beside a wrong result."""
    import torch

    from oracle import lmhead as OM
    from oracle import loss as OL

    cores = torch.get_num_threads()

    def run(nt):
        h, l = hid[:nt], lab[:nt]
        t0 = time.perf_counter()
        lp, _ = OM.forward_bf16_torch_path(h, w, l)
        lpf = lp.float().view(1, -1).requires_grad_(True)
        old = lpf.detach() - 0.01
        loss, _ = OL.ppo_loss(lpf, old, torch.ones_like(old), torch.ones_like(old), clip_ratio_low=0.2,
                              clip_ratio_high=0.28)
        loss.backward()
        OM.backward_bf16_torch_path(lpf.grad.view(-1), h, w, l)
        return time.perf_counter() - t0

    probe_n = min(512, hid.shape[0])  # one full chunk of the reference's token loop
    t_probe = run(probe_n)
    n = int(min(hid.shape[0], probe_n * budget_s / max(t_probe, 1e-6)))
    n = max(probe_n, (n // 512) * 512)
    t = run(n) if n > probe_n else t_probe
    out = {
        "value": n / t, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"{n} of the workload's tokens, full hidden and vocab, fwd+loss+bwd, {t:.1f} s; linear in tokens",
    }
    out["config1"] = config1_cpu_vs_gpu()
    out["config4"] = config4_cpu_vs_gpu()
    if check is not None:
        idx, got = check
        ref_lp, _ = OM.forward(hid[idx - 1], w, lab[idx])
        err = (got - ref_lp).abs().max().item()
        assert err < 1e-3, f"log-prob parity failed: {err}"
        out["logprob_max_abs_err_subset"] = err
    return out


def graph_replay_ms(chain, reps=200):
    """The launches of `chain` captured once into a HIP graph and replayed: milliseconds per replay (the GPU's
    time for the chain without the host's eager-call cost) and the captured outputs of the last replay."""
    import torch

    side = torch.cuda.Stream()  # warm-up off the capture stream
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = chain()
    for _ in range(5):
        graph.replay()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(reps):
        graph.replay()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / reps, outs


def config1_cpu_vs_gpu():
    """The small published configuration (padded 128 x 1024, 16 groups of 8; GRPO advantage, PPO loss and its
    gradient): the CPU port beside the GPU path on the same inputs, with the errors between the two."""
    import numpy as np
    import torch

    from axon_amd import workloads as W
    from axon_amd.protocol import DataProto
    from axon_amd.trainer.algos.advantages import compute_advantage
    from axon_amd.trainer.algos.loss import compute_loss_fn
    from oracle import advantage as OA
    from oracle import loss as OL

    d = W.c1_loss_only()
    args = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "clip_ratio_c": 3.0, "token_reduce": "sum",
            "batch_reduce": "token-mean"}
    gidx = torch.as_tensor(np.unique(d["uid"], return_inverse=True)[1])

    def cpu():
        adv = OA.grpo_advantage(d["token_level_rewards"], d["response_mask"], gidx, 1e-6, True)
        lp = d["log_probs"].clone().requires_grad_(True)
        loss, _ = OL.ppo_loss(lp, d["old_log_probs"], adv, d["response_mask"], **args)
        loss.backward()
        return loss.detach(), lp.grad

    dev = "cuda:0"
    gpu_in = {k: d[k].to(dev) for k in ("token_level_rewards", "response_mask", "log_probs", "old_log_probs")}

    def gpu():
        a = DataProto.from_dict(tensors={"token_level_rewards": gpu_in["token_level_rewards"],
                                         "response_mask": gpu_in["response_mask"]})
        a.non_tensor_batch["uid"] = d["uid"]
        adv = compute_advantage(a, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}).batch["advantages"]
        lp = gpu_in["log_probs"].detach().requires_grad_(True)
        data = DataProto.from_dict(tensors={"log_probs": lp, "old_log_probs": gpu_in["old_log_probs"],
                                            "advantages": adv, "response_mask": gpu_in["response_mask"]})
        loss, _ = compute_loss_fn(data, "ppo", args)
        loss.backward()
        return loss.detach(), lp.grad

    def timed(fn, reps, sync):
        fn()
        if sync:
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            r = fn()
        if sync:
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps, r

    t_cpu, (l_cpu, g_cpu) = timed(cpu, 20, False)
    t_gpu, (l_gpu, g_gpu) = timed(gpu, 200, True)

    # the same kernels (row sums, group statistics, broadcast, loss + gradient, gradient scaling) as one HIP graph
    from axon_amd import _ops
    rows = _ops.rows_of(gpu_in["token_level_rewards"])
    gidx_d, one = gidx.to(dev), torch.ones((), device=dev)
    hp = dict(token_reduce="sum", batch_reduce="token-mean", ratio_lo=1 - 0.2, ratio_hi=1 + 0.28, clip_c=3.0)

    def chain():
        _, scores, _ = _ops.row_stats(gpu_in["token_level_rewards"], None, None, rows, want_cnt=False)
        scalar = _ops.group_stats(scores, gidx_d, int(gidx.max()) + 1, 1e-6, 1)[3]
        adv = _ops.row_broadcast_mask(scalar, gpu_in["response_mask"], rows)
        acc, grad = _ops.policy_loss(0, gpu_in["log_probs"], gpu_in["old_log_probs"], adv, gpu_in["response_mask"],
                                     None, rows, **hp)
        return acc, _ops.scale_f32(grad, one, acc[5])

    t_graph, (acc_g, grad_g) = graph_replay_ms(chain)
    assert torch.equal(grad_g, g_gpu) and acc_g[0].item() == l_gpu.item(), "graph replay differs from the eager chain"
    g_gpu = g_gpu.cpu().double()
    return {
        "workload": "128 x 1024 padded, GRPO advantage + PPO loss (0.2 / 0.28 / 3.0, sum / token-mean) + gradient",
        "cpu_ms": 1e3 * t_cpu, "cpu_cores": torch.get_num_threads(), "gpu_ms": 1e3 * t_gpu,
        "gpu_graph_ms": t_graph,
        "gpu_graph": "the chain's launches captured once into a HIP graph and replayed: GPU time without the host's "
                     "eager calls (registry lookups, DataProto, autograd, the metrics readback)",
        "loss_rel_err": abs(l_gpu.item() - l_cpu.item()) / abs(l_cpu.item()),
        "grad_rel_l2": ((g_gpu - g_cpu.double()).norm() / g_cpu.double().norm()).item(),
    }


def config4_cpu_vs_gpu():
    """The correction + GSPO configuration at its full size (65536 packed tokens, ragged sequences; token-level
    importance weights capped at 2, token rejection outside [0.5, 2], per-sequence veto at 1e-4, then the GSPO
    loss with clip 3e-4 / 4e-4, mean / step-mean, and its gradient): the CPU port on the padded layout the
    reference uses beside the GPU path on the packed layout, same inputs, with the errors between the two."""
    import numpy as np
    import torch

    from axon_amd import workloads as W
    from axon_amd.protocol import DataProto
    from axon_amd.trainer.algos.loss import compute_loss_fn
    from axon_amd.utils.rl import sampler as S
    from oracle import advantage as OA
    from oracle import loss as OL
    from oracle import sampler as OS

    d = W.c4_correction()
    lens, cu = d["lengths"], d["cu_seqlens"]
    s_, tmax = len(lens), max(lens)
    pad = {}
    for k in ("log_probs", "old_log_probs", "sampler_log_probs", "response_mask", "token_level_rewards"):
        pad[k] = torch.zeros(s_, tmax)
        for b, (a, e) in enumerate(zip(cu[:-1].tolist(), cu[1:].tolist())):
            pad[k][b, : e - a] = d[k][a:e]
    gidx = torch.as_tensor(np.unique(d["uid"], return_inverse=True)[1])
    adv_pad = OA.grpo_advantage(pad["token_level_rewards"], pad["response_mask"], gidx, 1e-6, True)
    unpad = lambda x: torch.cat([x[b, :l] for b, l in enumerate(lens)])  # noqa: E731
    corr = dict(sampler_is="token", sampler_is_threshold=2.0, sampler_rs="token", sampler_rs_threshold=2.0,
                sampler_token_veto_threshold=1e-4)
    gspo = {"clip_ratio_low": 3e-4, "clip_ratio_high": 4e-4, "token_reduce": "mean", "batch_reduce": "step-mean"}

    def cpu():
        w, new_mask, _ = OS.correction(pad["old_log_probs"], pad["sampler_log_probs"], pad["response_mask"], **corr)
        lp = pad["log_probs"].clone().requires_grad_(True)
        loss, _ = OL.gspo_loss(lp, pad["old_log_probs"], adv_pad, new_mask, sampler_is_weights=w, **gspo)
        loss.backward()
        return loss.detach(), unpad(lp.grad), unpad(new_mask), unpad(w)

    dev = "cuda:0"
    g_in = {k: d[k].to(dev) for k in ("log_probs", "old_log_probs", "sampler_log_probs", "response_mask")}
    g_in["advantages"] = unpad(adv_pad).to(dev)
    cu_d = cu.to(dev)

    def gpu():
        proto, new_mask, _ = S.compute_sampler_correction_and_rejection_mask(
            g_in["old_log_probs"], g_in["sampler_log_probs"], g_in["response_mask"], cu_seqlens=cu_d, **corr)
        lp = g_in["log_probs"].detach().requires_grad_(True)
        w = proto.batch["sampler_is_weights"]
        data = DataProto.from_dict(tensors={"log_probs": lp, "old_log_probs": g_in["old_log_probs"],
                                            "advantages": g_in["advantages"], "response_mask": new_mask,
                                            "sampler_is_weights": w}, meta_info={"cu_seqlens": cu_d})
        loss, _ = compute_loss_fn(data, "gspo", gspo)
        loss.backward()
        return loss.detach(), lp.grad, new_mask, w

    def timed(fn, reps, sync):
        fn()
        if sync:
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            r = fn()
        if sync:
            torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps, r

    t_cpu, (l_cpu, g_cpu, m_cpu, w_cpu) = timed(cpu, 10, False)
    t_gpu, (l_gpu, g_gpu, m_gpu, w_gpu) = timed(gpu, 200, True)

    # the same two operators (correction with veto, GSPO loss + gradient) and the gradient scaling as one HIP graph
    import math

    from axon_amd import _ops
    rows = _ops.rows_of(g_in["log_probs"], cu_d)
    lr_lo, lr_hi = S.log_interval_for_ratio_bounds(0.5, 2.0)
    one = torch.ones((), device=dev)

    def chain():
        isw, new_mask, _ = _ops.sampler_correction(g_in["old_log_probs"], g_in["sampler_log_probs"],
                                                   g_in["response_mask"], rows, is_mode=1, is_threshold=2.0, rs_mode=1,
                                                   rs_lr_lo=lr_lo, rs_lr_hi=lr_hi, log_veto=math.log(1e-4))
        acc, grad = _ops.policy_loss(1, g_in["log_probs"], g_in["old_log_probs"], g_in["advantages"], new_mask, isw,
                                     rows, token_reduce="mean", batch_reduce="step-mean", ratio_lo=1 - 3e-4,
                                     ratio_hi=1 + 4e-4, clip_c=3.0)
        return acc, _ops.scale_f32(grad, one, acc[5]), new_mask

    t_graph, (acc_g, grad_g, mask_g) = graph_replay_ms(chain)
    assert torch.equal(mask_g, m_gpu) and torch.equal(grad_g, g_gpu), "graph replay differs from the eager chain"
    g_gpu = g_gpu.cpu().double()
    return {
        "workload": "65536 packed tokens: token IS (cap 2) + token rejection [0.5, 2] + veto 1e-4, then GSPO "
                    "(3e-4 / 4e-4, mean / step-mean) + gradient",
        "cpu_ms": 1e3 * t_cpu, "cpu_cores": torch.get_num_threads(), "gpu_ms": 1e3 * t_gpu,
        "gpu_graph_ms": t_graph, "sequences": s_, "cpu_layout": f"padded {s_} x {tmax}", "gpu_layout": "packed",
        "masks_equal": bool(torch.equal(m_gpu.cpu(), m_cpu)),
        "weights_max_abs_err": (w_gpu.cpu() - w_cpu).abs().max().item(),
        "loss_rel_err": abs(l_gpu.item() - l_cpu.item()) / abs(l_cpu.item()),
        "grad_rel_l2": ((g_gpu - g_cpu.double()).norm() / g_cpu.double().norm()).item(),
    }


def gemm_calibration(dev, n, h, chunk=32768):
    """What a plain bf16 GEMM of the dominant kernel's shape sustains on THIS box, next to the main loop of the
    fused kernels on the same operands: `torch.matmul` (hipBLASLt) and `axon_gemm_nt_bf16`, dHidden shape
    [n, chunk] x [chunk, h], random operands, median of 5 regions of 8 calls."""
    import torch

    from axon_amd import _ops

    g = torch.Generator(device=dev).manual_seed(77)
    a = torch.randn(h, chunk, device=dev, generator=g).bfloat16()  # [m][k], K-contiguous
    b = torch.randn(n, chunk, device=dev, generator=g).bfloat16()  # [n][k]
    out = torch.empty(n, h, device=dev, dtype=torch.bfloat16)
    flops = 2.0 * n * h * chunk

    def tflops(fn):
        for _ in range(3):
            fn()
        ts = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(8):
                fn()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) / 8)
        return flops / (sorted(ts)[2] * 1e-3) / 1e12

    res = {"shape": f"[{n} x {chunk}] x [{chunk} x {h}] bf16, fp32 accumulate",
           "hipblaslt_matmul_tflops": tflops(lambda: torch.matmul(b, a.t(), out=out)),
           "axon_gemm_nt_tflops": tflops(lambda: _ops.gemm_nt(a, b))}
    del a, b, out
    return res


def head_step_summary(workload, dev, steps=3, warmup=1, block_tokens=8192):
    """One of the other head shapes through the same step as the headline (GRPO advantage, then head forward with
    roll and shift inside, PPO loss and backward to dHidden and dWeight block of tokens by block): tokens/s and
    TFLOP/s per kernel class."""
    import torch

    from axon_amd import _ops, workloads as W
    from axon_amd.models.fused_head_loss import fused_head_loss
    from axon_amd.protocol import DataProto
    from axon_amd.trainer.algos.advantages import compute_advantage
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs

    n, h, v, group, seed = WORKLOADS[workload]
    hid, w, lab = W.lmhead_inputs(n, h, v, seed)
    rl = W.packed_rl_inputs(n, seed + 100, group=group)
    hd, wd, ld = hid.to(dev), w.to(dev), lab.to(dev)
    cu, mask, tlr, uid = rl["cu_seqlens"].to(dev), rl["response_mask"].to(dev), rl["token_level_rewards"].to(dev), rl["uid"]
    with torch.no_grad():
        old = packed_logprobs(hd, wd, ld, cu)[0] - 0.05 * torch.randn(n, device=dev)
    loss_args = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "token_reduce": "sum", "batch_reduce": "token-mean"}

    meta = {"loss_fn": "ppo", "loss_fn_args": loss_args, "temperature": 1.0, "dp_replicas": 1}
    info = {}

    def step():
        hg, wg = hd.detach().requires_grad_(True), wd.detach().requires_grad_(True)
        a_in = DataProto.from_dict(tensors={"token_level_rewards": tlr, "response_mask": mask},
                                   meta_info={"cu_seqlens": cu})
        a_in.non_tensor_batch["uid"] = uid
        adv = compute_advantage(a_in, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}).batch["advantages"]
        data = DataProto.from_dict(tensors={"old_log_probs": old, "advantages": adv, "response_mask": mask})
        loss, _ = fused_head_loss(hg, wg, ld, cu, data, meta, block_tokens=block_tokens)
        loss.backward()
        info.update(data.meta_info)
        return loss

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    timer = _ops.Timer()
    _ops.set_timing(timer)
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    el = time.perf_counter() - t0
    _ops.set_timing(None)
    t = timer.collect()
    timer.close()
    assert torch.isfinite(loss).item()
    nhv = float(n) * h * v
    ms = lambda *keys: sum(t.get(k, {"ms": 0})["ms"] for k in keys) / steps  # noqa: E731
    tf = lambda fl, m: fl / (m * 1e-3) / 1e12 if m > 0 else None  # noqa: E731
    return {"workload": workload, "tokens": n, "hidden": h, "vocab": v, "steps": steps,
            "ms_per_step": 1e3 * el / steps, "tokens_per_s": n * steps / el,
            "fwd_tflops": tf(2 * nhv, ms("fwd/logits_stats")),
            "dhidden_dweight_tflops": tf(4 * nhv, ms("bwd/dhidden", "bwd/dweight")),
            "head_backward": info.get("head_backward"), "n_blocks": info.get("n_blocks"),
            "stash_bytes": info.get("stash_bytes"), "dlogit_ms_per_step": ms("bwd/dlogit"),
            "path_algorithmic_tflops": 6 * nhv / (1e-3 * 1e3 * el / steps) / 1e12}


def hbm_kernels(n_tokens, dev, only=None):
    """Stage-2/3 kernels on a packed batch large enough to show the bandwidth asymptote
    (same lognormal length law as the headline workload).  Each figure is algorithmic bytes
    (one read of every input, one write of every output, fp32) over the median of 20 timed
    calls of the whole operator, every launch it makes included."""
    import math

    import torch

    from axon_amd import _ops, workloads as W

    g = torch.Generator().manual_seed(11)
    lens = torch.exp(torch.randn(max(n_tokens // 300, 8), generator=g) * 0.8 + 6.5).round().clamp(32, 8192).long()
    lens = lens[: int((torch.cumsum(lens, 0) <= n_tokens).sum())].tolist()
    if n_tokens - sum(lens):
        lens.append(n_tokens - sum(lens))
    cu = W.cu_from_lengths(lens).to(dev)
    gd = torch.Generator(device=dev).manual_seed(12)
    old = -torch.empty(n_tokens, device=dev).exponential_(1.0, generator=gd)
    new = old + 0.05 * torch.randn(n_tokens, device=dev, generator=gd)
    samp = old + 0.01 * torch.randn(n_tokens, device=dev, generator=gd)
    adv = torch.randn(n_tokens, device=dev, generator=gd)
    mask = torch.ones(n_tokens, device=dev)
    mask[cu[:-1].long()] = 0
    rows = _ops.rows_of(new, cu)
    seq_scalar = torch.randn(len(lens), device=dev, generator=gd)

    def median_ms(fn, iters=12, warm=5, inner=8):
        """Median over `iters` timed regions of `inner` back-to-back calls each, per call: the host enqueues
        call k + 1 while the GPU runs call k, so the figure is the operator's GPU time (every launch it makes
        and the gaps between them), not the host's time to issue one eager call to an idle GPU."""
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(iters):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a.record()
            for _ in range(inner):
                fn()
            b.record()
            b.synchronize()
            ts.append(a.elapsed_time(b) / inner)
        return sorted(ts)[len(ts) // 2]

    def forced_two_pass(fn):
        keep, _ops.OWNED_ROWS_MAX_SLOTS = _ops.OWNED_ROWS_MAX_SLOTS, 0
        try:
            return fn()
        finally:
            _ops.OWNED_ROWS_MAX_SLOTS = keep

    ppo = dict(token_reduce="sum", batch_reduce="token-mean", ratio_lo=0.8, ratio_hi=1.28, clip_c=3.0)
    gspo = dict(token_reduce="mean", batch_reduce="step-mean", ratio_lo=1 - 3e-4, ratio_hi=1 + 4e-4, clip_c=3.0)
    corr = dict(is_mode=1, is_threshold=2.0, rs_mode=1, rs_lr_lo=-math.log(2.0), rs_lr_hi=math.log(2.0))
    x = torch.empty_like(old)
    cases = [  # name, bytes per token, callable
        ("device-to-device copy (calibration)", 8, lambda: x.copy_(old)),
        ("policy_loss_kernel: PPO/DAPO loss + gradient, sum/token-mean (one pass)", 20,
         lambda: _ops.policy_loss(0, new, old, adv, mask, None, rows, **ppo)),
        ("owned_policy_loss_kernel: GSPO loss + gradient in one launch and one read, a workgroup owns whole "
         "sequences (the path taken unless the rows are short)", 20,
         lambda: _ops.policy_loss(1, new, old, adv, mask, None, rows, **gspo)),
        ("row_stats + policy_loss_kernel: GSPO loss + gradient (two reads of log_probs, old, mask; the path for "
         "batches of short rows, forced here)", 32,
         lambda: forced_two_pass(lambda: _ops.policy_loss(1, new, old, adv, mask, None, rows, **gspo))),
        ("sampler_correction_kernel: token IS weights + rejection mask", 20,
         lambda: _ops.sampler_correction(old, samp, mask, rows, log_veto=None, **corr)),
        ("owned_correction_kernel: IS + rejection + per-sequence veto in one launch and one read (the path taken "
         "unless the rows are short)", 20,
         lambda: _ops.sampler_correction(old, samp, mask, rows, log_veto=math.log(1e-4), **corr)),
        ("row_stats + sampler_correction_kernel: IS + rejection + per-sequence veto (two reads; the path for batches "
         "of short rows, forced here)", 32,
         lambda: forced_two_pass(lambda: _ops.sampler_correction(old, samp, mask, rows, log_veto=math.log(1e-4),
                                                                 **corr))),
        ("row_stats_kernel: per-sequence count and masked sum", 12, lambda: _ops.row_stats(new, old, mask, rows)),
        ("sampler_diag kernels: all IS / rejection / off-policy / mismatch diagnostics (token pass + row pass)", 12,
         lambda: _ops.sampler_diag(old, samp, mask, rows, is_mode=1, is_lo=0.5, is_hi=2.0, rs_mode=1, rs_lo=0.5,
                                   rs_hi=2.0, rs_lr_lo=-math.log(2.0), rs_lr_hi=math.log(2.0),
                                   log_is_lo=-math.log(2.0), log_is_hi=math.log(2.0), log_rs_lo=-math.log(2.0),
                                   log_rs_hi=math.log(2.0))),
        ("row_broadcast_kernel: GRPO advantage = per-sequence scalar * mask", 8,
         lambda: _ops.row_broadcast_mask(seq_scalar, mask, rows)),
        ("reverse_scan_kernel: GAE time recurrence per sequence (rewards, values, mask -> advantages, returns)", 20,
         lambda: _ops.reverse_scan(_ops.SCAN_GAE, adv, new, mask, rows, gamma=0.99, lam=0.95)),
        ("masked_whiten kernels: mean pass + variance pass + normalise (three reads of x, two of mask, one write)",
         24, lambda: _ops.masked_whiten(adv, mask)),
        ("policy_loss_kernel: clipped value loss + gradient, sum/token-mean (one pass)", 20,
         lambda: _ops.policy_loss(4, new, old, adv, mask, None, rows, token_reduce="sum", batch_reduce="token-mean",
                                  ratio_lo=0.5, ratio_hi=0.0, clip_c=0.0)),
    ]
    out = []
    for name, bpt, fn in cases:
        if only is not None and not any(o in name for o in only):
            continue
        ms = median_ms(fn)
        gbs = n_tokens * bpt / (ms * 1e-3) / 1e9
        out.append({"kernel": name, "bytes_per_token": bpt, "ms": ms, "achieved": gbs, "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS})
    # the materialised-logits path (use_fused_kernels off): bf16 logits of 8192 tokens at the Qwen vocabulary
    del old, new, samp, adv, x
    ln, lv = min(8192, max(n_tokens // 1024, 64)), 151936
    logits = torch.randn(ln, lv, device=dev, dtype=torch.bfloat16, generator=gd)
    labels = torch.randint(0, lv, (ln,), device=dev, generator=gd)
    lp, ent, lse = _ops.logits_forward(logits, labels, True)
    g1, g2 = torch.randn(ln, device=dev, generator=gd), torch.randn(ln, device=dev, generator=gd)
    dl = torch.empty_like(logits)

    def bwd():
        lib_out = _ops.logits_backward(logits, labels, lse, ent, g1, g2, inplace=False)
        return lib_out

    for name, nbytes, fn in (
            ("logits_stats_kernel: bf16 logits [8192 x 151936] -> log-prob, entropy (one read)", ln * lv * 2,
             lambda: _ops.logits_forward(logits, labels, True)),
            ("logits_grad_kernel: d logits from both gradients (one read, one write)", ln * lv * 4, bwd)):
        if only is not None and not any(o in name for o in only):
            continue
        ms = median_ms(fn, iters=10, warm=2)
        gbs = nbytes / (ms * 1e-3) / 1e9
        out.append({"kernel": name, "bytes_per_token": nbytes // ln, "ms": ms, "achieved": gbs, "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS})
    del dl
    return {"tokens": n_tokens, "sequences": len(lens), "bound": "hbm", "kernels": out}


def baseline_sizes_cold(dev):
    """The loss and correction operators at the two small published sizes (padded 128 x 1024 PPO;
    65536 packed tokens of correction + GSPO), each timed twice: on one set of buffers (inputs
    sit in L2 / Infinity Cache) and rotating through more than 512 MB of distinct input sets, so
    every call reads its inputs from HBM.  Microseconds per call of the whole operator, every
    launch included; at these sizes launches, not bandwidth, set the time."""
    import math

    import torch

    from axon_amd import _ops, workloads as W

    def per_call_us(fn, sets, rounds):
        for k in range(min(sets, 8)):
            fn(k)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(rounds):
            for k in range(sets):
                fn(k)
        b.record()
        b.synchronize()
        return a.elapsed_time(b) * 1e3 / (rounds * sets)

    def stack(t, sets):  # `sets` copies at distinct addresses
        return t.to(dev).unsqueeze(0).repeat(sets, *([1] * t.dim())).contiguous()

    out = []
    c1 = W.c1_loss_only()
    sets = 288  # x 4 inputs x 512 KiB = 576 MiB
    new, old, mask = (stack(c1[k], sets) for k in ("log_probs", "old_log_probs", "response_mask"))
    adv = stack(torch.randn(c1["log_probs"].shape, generator=torch.Generator().manual_seed(5)), sets) * mask
    rows = _ops.rows_of(new[0])
    ppo = dict(token_reduce="sum", batch_reduce="token-mean", ratio_lo=0.8, ratio_hi=1.28, clip_c=3.0)
    f = lambda k: _ops.policy_loss(0, new[k], old[k], adv[k], mask[k], None, rows, **ppo)
    n_slots = rows.n_slots
    for label, s_, r_ in (("cold", sets, 2), ("cached", 1, 400)):
        us = per_call_us(f, s_, r_)
        out.append({"case": "PPO loss + gradient, padded 128 x 1024, sum/token-mean", "inputs": label,
                    "bytes": n_slots * 20, "us_per_call": us, "achieved_GBps": n_slots * 20 / us / 1e3})
    del new, old, mask, adv

    c4 = W.c4_correction()
    sets = 520  # x 4 inputs x 256 KiB = 520 MiB
    old, samp, new, mask = (stack(c4[k], sets) for k in ("old_log_probs", "sampler_log_probs", "log_probs",
                                                           "response_mask"))
    advs = stack(torch.randn(old.shape[1], generator=torch.Generator().manual_seed(6)), sets)
    rows = _ops.rows_of(new[0], c4["cu_seqlens"].to(dev))
    n_slots = rows.n_slots
    corr = dict(is_mode=1, is_threshold=2.0, rs_mode=1, rs_lr_lo=-math.log(2.0), rs_lr_hi=math.log(2.0),
                log_veto=math.log(1e-4))
    gspo = dict(token_reduce="mean", batch_reduce="step-mean", ratio_lo=1 - 3e-4, ratio_hi=1 + 4e-4, clip_c=3.0)
    fc = lambda k: _ops.sampler_correction(old[k], samp[k], mask[k], rows, **corr)
    fg = lambda k: _ops.policy_loss(1, new[k], old[k], advs[k], mask[k], None, rows, **gspo)
    for case, fn, nbytes in (("sampler correction (token IS, token rejection, veto), 65536 packed tokens", fc, 20),
                             ("GSPO loss + gradient, 65536 packed tokens, mean/step-mean", fg, 20)):
        for label, s_, r_ in (("cold", sets, 1), ("cached", 1, 400)):
            us = per_call_us(fn, s_, r_)
            out.append({"case": case, "inputs": label, "bytes": n_slots * nbytes, "us_per_call": us,
                        "achieved_GBps": n_slots * nbytes / us / 1e3})
    return out


def kernel_table(timing, steps, n, h, v, stash_bytes, vocab_chunk=0):
    """Per kernel class of the head: launches and milliseconds per step (HIP events on the launch stream),
    algorithmic and executed TFLOP/s.  With the forward's stash the backward's first kernel is a streaming one:
    per logit it reads 2 bytes of stash and writes the bf16 dlogit (once, token-major, where the weight-gradient
    GEMM can read that K-major; else a vocab-major copy as well), and no flop of the path is executed twice;
    without it that kernel recomputes the logits (2 N H V executed flop that do not count as algorithmic)."""
    from axon_amd import _lib

    nhv = float(n) * h * v
    copies = max(int(_lib.load().axon_lmhead_bwd_dlogit_copies(h, v, vocab_chunk)), 1)
    classes = [
        ("gemm_store_kernel (dHidden + dWeight GEMMs)", ("bwd/dhidden", "bwd/dweight"), 4 * nhv, 4 * nhv, 0.0),
        ("lmhead_fwd_stash_kernel (logits + online softmax statistics + stash)" if stash_bytes else
         "lmhead_fwd_kernel (logits + online softmax statistics)", ("fwd/logits_stats",), 2 * nhv, 2 * nhv, 0.0),
        (f"lmhead_dlogit_stash_kernel (stash -> bf16 dlogit, {copies} cop{'y' if copies == 1 else 'ies'}; HBM-bound)",
         ("bwd/dlogit",), 0.0, 0.0, (2.0 + 2.0 * copies) * n * v) if stash_bytes else
        ("lmhead_dlogit_kernel (logit recompute + dlogit)", ("bwd/dlogit",), 0.0, 2 * nhv, 0.0),
    ]
    kernels = []
    for label, keys, algo, execd, hbm_bytes in classes:
        ms = sum(timing.get(k, {"ms": 0})["ms"] for k in keys)
        launches = sum(timing.get(k, {"launches": 0})["launches"] for k in keys)
        if launches == 0:
            continue
        kernels.append({
            "kernel": label, "launches_per_step": launches / steps, "ms_per_step": ms / steps,
            "avg_launch_ms": ms / launches,
            "algorithmic_tflops": algo * steps / (ms * 1e-3) / 1e12,
            "executed_tflops": execd * steps / (ms * 1e-3) / 1e12,
        })
        if hbm_bytes:
            gbps = hbm_bytes * steps / (ms * 1e-3) / 1e9
            kernels[-1].update({"algorithmic_bytes_per_step": hbm_bytes, "achieved_GBps": gbps,
                                "frac_of_hbm_peak": gbps / HBM_PEAK_GBS})
    return kernels


def kernel_source_digest():
    """Digest of the sources of the LM-head kernels: ties a committed profile to the code it was taken on."""
    import hashlib

    h = hashlib.sha256()
    for name in ("gemm_nt.h", "lmhead.hip", "common.h"):
        with open(os.path.join(ROOT, "axon_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def traffic_from_profile(workload, head_path):
    """HBM-side bytes of ONE launch of the dominant kernel on the named head-backward path, read from the
    committed summary of the two rocprofv3 --pmc passes over `bench.py --traffic-probe <path>`
    (profiles/lmhead_<workload>_hbm_traffic.md carries one line
    `traffic_bytes_per_launch[<path>]: <bytes> kernel_source_digest: <digest>` per path).  None when there is no
    such line or when the kernels have changed since (the digest of their sources differs)."""
    import re

    path = os.path.join(ROOT, "profiles", f"lmhead_{workload}_hbm_traffic.md")
    try:
        text = open(path).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch\[" + re.escape(head_path) +
                  r"\]:\s*([0-9.eE+]+)\s+kernel_source_digest:\s*([0-9a-f]+)", text)
    if not m or m.group(2) != kernel_source_digest():
        return None
    return float(m.group(1))


def traffic_probe(workload, head_path):
    import torch

    from axon_amd import _ops, workloads as W

    n, h, v, _, seed = WORKLOADS[workload]
    hid, w, lab = W.lmhead_inputs(n, h, v, seed)
    hd, wd, ld = hid.to("cuda"), w.to("cuda"), lab.to("cuda")
    src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()  # 1 GiB
    dst = torch.empty_like(src)
    dst.copy_(src)  # calibration kernel: reads 1 GiB, writes 1 GiB
    g = torch.randn(n + 4, device="cuda")
    if head_path == "blocked-stash":  # four blocks of 8192 tokens: forward with stash, backward from it
        hb = _ops.HeadBlocks(hd, wd, ld, 1.0, [(a, min(a + 8192, n)) for a in range(0, n, 8192)])
        for k in range(len(hb.ranges)):
            hb.forward(k)
            hb.backward(k, g, None)
    elif head_path == "recompute":  # the library's default: the backward recomputes the logits
        _, _, lse, eb = _ops.lmhead_forward(hd, wd, ld, 1.0)
        _ops.lmhead_backward(g[:n], torch.zeros(n, device="cuda"), hd, wd, ld, lse, eb, 1.0)
    else:  # the opt-in stash of all tokens
        _ops.LMHEAD_STASH = True
        _, _, lse, eb, stash = _ops.lmhead_forward(hd, wd, ld, 1.0, stash=True)
        _ops.lmhead_backward(g[:n], torch.zeros(n, device="cuda"), hd, wd, ld, lse, eb, 1.0, stash=stash)
    torch.cuda.synchronize()


def gemm_probe(which, workload):
    import torch

    from axon_amd import _ops

    n, h, _, _, _ = WORKLOADS[workload]
    chunk = 32768
    g = torch.Generator(device="cuda").manual_seed(0)
    a = torch.randn(h, chunk, device="cuda", generator=g).bfloat16()
    b = torch.randn(n, chunk, device="cuda", generator=g).bfloat16()
    for _ in range(3):
        c = torch.matmul(b, a.t()) if which == "hipblaslt" else _ops.gemm_nt(a, b)
    torch.cuda.synchronize()
    del c


def main():
    args = parse_args()
    if args.traffic_probe:
        traffic_probe(args.workload, args.traffic_probe)
        return
    if args.gemm_probe:
        gemm_probe(args.gemm_probe, args.workload)
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from axon_amd import _ops, workloads as W
    from axon_amd.protocol import DataProto
    from axon_amd.trainer.algos.advantages import compute_advantage
    from axon_amd.trainer.algos.loss import compute_loss_fn
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    n, h, v, group, seed = WORKLOADS[args.workload]
    if args.tokens:
        n = args.tokens

    hid, w, lab = W.lmhead_inputs(n, h, v, seed)
    rl = W.packed_rl_inputs(n, seed + 100, group=group)
    hd, wd, ld = hid.to(dev), w.to(dev), lab.to(dev)
    cu = rl["cu_seqlens"].to(dev)
    mask = rl["response_mask"].to(dev)
    tlr = rl["token_level_rewards"].to(dev)
    uid = rl["uid"]

    # old log-probs: one forward, detached, perturbed (as the trainer's first pass would give)
    # (`lab` is the packed stream of token ids: the head rolls and shifts inside its kernels)
    with torch.no_grad():
        lp0, _ = packed_logprobs(hd, wd, ld, cu)
        old = lp0 - 0.05 * torch.randn(n, device=dev)
    # token subset whose log-probs the CPU leg checks: token p is predicted from hidden p - 1
    idx = torch.arange(1, n, max(1, n // 48))
    idx = idx[rl["response_mask"][idx] > 0]
    lp_subset = lp0.cpu()[idx]

    loss_args = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "token_reduce": "sum", "batch_reduce": "token-mean"}
    adv_cfg = {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}
    meta = {"loss_fn": "ppo", "loss_fn_args": loss_args, "temperature": 1.0, "dp_replicas": 1}
    from axon_amd.models.fused_head_loss import DEFAULT_DW_GROUP, fused_head_loss

    def advantages(mask):
        adv_in = DataProto.from_dict(tensors={"token_level_rewards": tlr, "response_mask": mask},
                                     meta_info={"cu_seqlens": cu})
        adv_in.non_tensor_batch["uid"] = uid
        return compute_advantage(adv_in, adv_cfg).batch["advantages"]

    def step_unfused(mask=mask, head_mask=None):
        """Head, loss and head backward as separate autograd functions (the reference's structure)."""
        hg, wg = hd.detach().requires_grad_(True), wd.detach().requires_grad_(True)
        lp_tok, _ent = packed_logprobs(hg, wg, ld, cu, response_mask=head_mask)
        data = DataProto.from_dict(tensors={"log_probs": lp_tok, "old_log_probs": old, "advantages": advantages(mask),
                                            "response_mask": mask}, meta_info={"cu_seqlens": cu})
        loss, _ = compute_loss_fn(data, "ppo", loss_args)
        loss.backward()
        return loss, hg.grad, wg.grad

    block_info = {}

    def step_blocked(mask=mask):
        """Head forward, loss and head backward block of tokens by block, one autograd node."""
        hg, wg = hd.detach().requires_grad_(True), wd.detach().requires_grad_(True)
        data = DataProto.from_dict(tensors={"old_log_probs": old, "advantages": advantages(mask), "response_mask": mask})
        loss, _ = fused_head_loss(hg, wg, ld, cu, data, meta, block_tokens=args.block_tokens,
                                  vocab_chunk=args.vocab_chunk, dw_group=args.dw_group or DEFAULT_DW_GROUP)
        loss.backward()
        block_info.update(data.meta_info)
        return loss, hg.grad, wg.grad

    def timed_steps(step_fn, steps, warmup):
        """`warmup` untimed steps, then exactly `steps` steps between two synchronisations, with HIP events
        around every LM-head launch (recorded on the launch stream without synchronising)."""
        for _ in range(warmup):
            step_fn()
        torch.cuda.synchronize()
        timer = _ops.Timer()
        _ops.set_timing(timer)
        t0 = time.perf_counter()
        for _ in range(steps):
            res = step_fn()
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        _ops.set_timing(None)
        timing = timer.collect()  # events of the timed region, read after it has ended
        timer.close()
        return el, timing, res

    def run_path(path, steps, warmup):
        _ops.LMHEAD_STASH = path == "stash"
        try:
            return timed_steps(step_blocked if path == "blocked-stash" else step_unfused, steps, warmup)
        finally:
            _ops.LMHEAD_STASH = False

    _ops.DEFAULT_VOCAB_CHUNK = args.vocab_chunk
    head_path = args.head_backward

    def chunk_of(path):
        """Vocabulary columns per backward chunk on a path: the blocks take the whole vocabulary unless told otherwise."""
        return args.vocab_chunk or ((v + 255) // 256 * 256 if path == "blocked-stash" else 0)

    elapsed, timing, (loss, dh, dw) = run_path(head_path, args.steps, args.warmup)
    assert torch.isfinite(loss).item() and torch.isfinite(dh.float()).all().item()
    if head_path == "blocked-stash":
        assert block_info.get("head_backward") == "blocked-stash", block_info
        stash_bytes = int(block_info["stash_bytes"])
    else:
        stash_bytes = _ops.lmhead_stash_bytes(n, h, v) if head_path == "stash" else 0

    ms_per_step = 1e3 * elapsed / args.steps
    tokens_per_s = n * args.steps / elapsed
    nhv = float(n) * h * v

    # Not the headline: the same step on the other head-backward paths (three steps each)
    variants = {}
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm()).item()  # noqa: E731
    what = {
        "blocked-stash": "head forward, loss and head backward block of tokens by block in one autograd node: one "
                         "block's stash (2 bytes per logit) held, 6 N H V flop executed",
        "recompute": "head as an autograd function whose backward recomputes the logits (the library's default and the "
                     "reference's structure): nothing of size tokens x vocab held, 8 N H V flop executed for 6",
        "stash": "head as an autograd function whose forward keeps 2 bytes per logit for ALL tokens (opt-in): "
                 "tokens x vocab x 2 bytes held from forward to backward, 6 N H V flop executed",
    }
    if args.variants and not args.tokens:
        for path in ("blocked-stash", "recompute", "stash"):
            if path == head_path or (path == "stash" and not _ops.lmhead_stash_bytes(n, h, v)):
                continue
            el, timing_v, (loss_v, dh_v, dw_v) = run_path(path, 3, 1)
            sb = (int(block_info["stash_bytes"]) if path == "blocked-stash" else
                  _ops.lmhead_stash_bytes(n, h, v) if path == "stash" else 0)
            variants[path] = {
                "what": what[path], "stash_bytes": sb, "steps": 3, "ms_per_step": 1e3 * el / 3,
                "tokens_per_s": 3 * n / el, "path_algorithmic_tflops": 6 * nhv / (el / 3) / 1e12,
                "path_frac_of_peak": 6 * nhv / (el / 3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                "loss": loss_v.item(), "headline_loss": loss.item(),
                "dhidden_rel_l2_vs_headline": rel(dh_v, dh), "dweight_rel_l2_vs_headline": rel(dw_v, dw),
                "kernels": kernel_table(timing_v, 3, n, h, v, sb, chunk_of(path)),
            }
            del loss_v, dh_v, dw_v
            torch.cuda.empty_cache()

    # Not the headline: the same step when the first third of every sequence is prompt (response_mask 0), as in
    # the trainer's batches.  Those positions send exact zeros back into the head, whose backward leaves their
    # rows out of its GEMMs while the forward still covers every token, as the reference's does ("backward");
    # with the mask handed to the head as well, the forward leaves them out too ("forward_and_backward").
    prompt_variant = None
    if args.prompt_fraction > 0:
        pos = torch.arange(n, device=dev)
        row = torch.searchsorted(cu.long(), pos, right=True) - 1
        start, length = cu.long()[row], (cu.long()[1:] - cu.long()[:-1])[row]
        mask_p = mask * (pos - start >= (length.float() * args.prompt_fraction).long()).to(mask.dtype)
        prompt_variant = {"prompt_fraction_of_tokens": 1.0 - mask_p.sum().item() / n, "steps": 3,
                          "head_backward": "recompute"}
        for name, head_mask in (("backward", None), ("forward_and_backward", mask_p)):
            # "backward": the opt-in search for rows without a gradient (one readback per backward)
            _ops.SKIP_ZERO_GRAD_ROWS = head_mask is None
            step_unfused(mask_p, head_mask)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                loss_p, dh_p, _ = step_unfused(mask_p, head_mask)
            torch.cuda.synchronize()
            el = time.perf_counter() - t0
            assert torch.isfinite(loss_p).item() and torch.isfinite(dh_p.float()).all().item()
            prompt_variant[name] = {"ms_per_step": 1e3 * el / 3, "tokens_per_s": 3 * n / el, "loss": loss_p.item()}
        _ops.SKIP_ZERO_GRAD_ROWS = False
        del loss_p, dh_p

    # kernel classes: (label, timing keys, algorithmic flops per step, executed flops per step)
    executed = 8 if head_path == "recompute" else 6
    kernels = kernel_table(timing, args.steps, n, h, v, stash_bytes, chunk_of(head_path))
    dom = max(kernels, key=lambda k: k["ms_per_step"])
    roofline = {
        "bound": "mfma", "kernel": dom["kernel"], "achieved": dom["algorithmic_tflops"] or dom["executed_tflops"],
        "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": (dom["algorithmic_tflops"] or dom["executed_tflops"]) / MFMA_BF16_PEAK_TFLOPS,
        "avg_launch_ms": dom["avg_launch_ms"], "launches_per_step": dom["launches_per_step"],
        "traffic": traffic_from_profile(args.workload, head_path) if not args.tokens and not args.vocab_chunk
        and args.block_tokens == 8192 and not args.dw_group and "gemm_store" in dom["kernel"] else None,
        "kernels": kernels,
        "path_algorithmic_tflops": 6 * nhv / (ms_per_step * 1e-3) / 1e12,
        "path_frac_of_peak": 6 * nhv / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        # a backward that recomputes the logits executes 8 N H V for the 6 that count; one that decodes a
        # stash executes the 6
        "path_executed_flop_per_algorithmic": executed / 6,
        "path_executed_tflops": executed * nhv / (ms_per_step * 1e-3) / 1e12,
        "other_phases_ms_per_step": {k: t["ms"] / args.steps for k, t in timing.items()
                                     if k in ("fwd/merge", "fwd/label", "bwd/transpose")},
        "gemm_dhidden_ms_per_step": timing.get("bwd/dhidden", {"ms": 0.0})["ms"] / args.steps,
        "gemm_dweight_ms_per_step": timing.get("bwd/dweight", {"ms": 0.0})["ms"] / args.steps,
    }
    head_ms = sum(t["ms"] for t in timing.values()) / args.steps
    roofline["head_kernels_ms_per_step"] = head_ms  # the rest of the step: advantage, loss kernels, fills, gaps
    roofline["outside_head_kernels_ms_per_step"] = ms_per_step - head_ms
    for path, var in variants.items():  # scalars, so that a reader of the first level sees them
        key = path.replace("-", "_")
        roofline[f"{key}_variant_ms_per_step"] = var["ms_per_step"]
        roofline[f"{key}_variant_path_frac"] = var["path_frac_of_peak"]

    out = {
        "metric": "trained tokens/sec for fused logprob+GRPO loss fwd+bwd, Qwen3-8B shape; % MFMA peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: fused LM-head logprob + GRPO/PPO loss fwd+bwd", "tokens": n,
                   "hidden": h, "vocab": v, "sequences": len(rl["lengths"]), "group": group,
                   "vocab_chunk": args.vocab_chunk or "default",
                   "head_backward": head_path, "stash_bytes": stash_bytes},
        "roofline": roofline,
    }
    if head_path == "blocked-stash":
        out["config"].update(block_tokens=args.block_tokens, n_blocks=int(block_info["n_blocks"]),
                             dw_group=int(block_info["dw_group"]),
                             head_workspace_bytes=int(block_info["head_workspace_bytes"]))
    if args.calibrate:
        cal = gemm_calibration(dev, n, h)
        roofline["calibration_tflops"] = cal
        best = max(cal["hipblaslt_matmul_tflops"], cal["axon_gemm_nt_tflops"])
        share = 6 / executed
        roofline["calibration_hipblaslt_tflops"] = cal["hipblaslt_matmul_tflops"]
        roofline["calibration_axon_gemm_tflops"] = cal["axon_gemm_nt_tflops"]
        roofline["path_ceiling_frac"] = share * best / MFMA_BF16_PEAK_TFLOPS
        roofline["ceiling"] = (f"{share * best / MFMA_BF16_PEAK_TFLOPS:.2f} of peak = {6}/{executed} executed x best "
                               f"plain GEMM of this run ({best:.0f} TFLOP/s, power-limited)")
    if variants:
        out["variants"] = variants
    if prompt_variant:
        out["prompt_rows_variant"] = prompt_variant
    if args.other_workloads and not args.tokens:
        del hd, wd, dh, dw
        hd = wd = dh = dw = None
        torch.cuda.empty_cache()
        out["other_workloads"] = [head_step_summary(name, dev) for name in sorted(WORKLOADS) if name != args.workload]
    if args.hbm_tokens > 0:
        hd = wd = dh = dw = None
        torch.cuda.empty_cache()
        out["hbm_kernels"] = hbm_kernels(args.hbm_tokens, dev)
        out["hbm_kernels"]["baseline_sizes"] = baseline_sizes_cold(dev)
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(hid, w, lab, args.cpu_seconds, check=(idx, lp_subset))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
