#!/usr/bin/env python3
"""Benchmark of the trainer-side per-token hot path on one MI355X.

One step = fused LM-head log-prob/entropy forward -> packed shift -> GRPO advantage ->
PPO (DAPO clip) loss forward+backward -> LM-head backward (dHidden, dWeight), on
synthetic inputs already resident in HBM.  Default workload: Qwen3-8B head shape,
32768 packed tokens, hidden 4096, vocab 151936, bf16.

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
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget; 0 disables it")
    return ap.parse_args()


def cpu_baseline(hid, w, lab, budget_s):
    """The reference torch path (bf16 matmul, 512-token chunks) + PPO loss, ported in oracle/,
    timed on a token sample sized to the budget.  Cost is linear in tokens (W is fixed)."""
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
    return {
        "value": n / t, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"{n} of the workload's tokens, full hidden and vocab, fwd+loss+bwd, {t:.1f} s; linear in tokens",
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from axon_amd import _ops, workloads as W
    from axon_amd.protocol import DataProto
    from axon_amd.trainer.algos.advantages import compute_advantage
    from axon_amd.trainer.algos.loss import compute_loss_fn
    from axon_amd.utils.fsdp.forward_utils import shift_packed
    from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy
    from oracle import lmhead as OM

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
    with torch.no_grad():
        lp0, _ = linear_cross_entropy(hd, wd, ld, 1.0, "none")
        old = shift_packed(lp0, cu) - 0.05 * torch.randn(n, device=dev)
    # parity gate on a token subset before anything is timed
    idx = torch.arange(0, n, max(1, n // 48))
    ref_lp, _ = OM.forward(hid[idx], w, lab[idx])
    lp_err = (lp0.cpu()[idx] - ref_lp).abs().max().item()
    assert lp_err < 1e-3, f"log-prob parity failed: {lp_err}"

    loss_args = {"clip_ratio_low": 0.2, "clip_ratio_high": 0.28, "token_reduce": "sum", "batch_reduce": "token-mean"}

    def step():
        hg, wg = hd.detach().requires_grad_(True), wd.detach().requires_grad_(True)
        lp_head, _ent = linear_cross_entropy(hg, wg, ld, 1.0, "none")
        lp_tok = shift_packed(lp_head, cu)
        adv_in = DataProto.from_dict(tensors={"token_level_rewards": tlr, "response_mask": mask},
                                     meta_info={"cu_seqlens": cu})
        adv_in.non_tensor_batch["uid"] = uid
        adv = compute_advantage(adv_in, {"advantage": "grpo", "advantage_args": {"epsilon": 1e-6}}).batch["advantages"]
        data = DataProto.from_dict(tensors={"log_probs": lp_tok, "old_log_probs": old, "advantages": adv,
                                            "response_mask": mask}, meta_info={"cu_seqlens": cu})
        loss, _ = compute_loss_fn(data, "ppo", loss_args)
        loss.backward()
        return loss, hg.grad, wg.grad

    _ops.DEFAULT_VOCAB_CHUNK = args.vocab_chunk
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    timing: dict = {}
    _ops.set_timing(timing)  # HIP events around every LM-head launch, on the launch stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, dh, dw = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    _ops.set_timing(None)
    assert torch.isfinite(loss).item() and torch.isfinite(dh.float()).all().item()

    ms_per_step = 1e3 * elapsed / args.steps
    tokens_per_s = n * args.steps / elapsed
    nhv = float(n) * h * v

    # kernel classes: (label, timing keys, algorithmic flops per step, executed flops per step)
    classes = [
        ("gemm_store_kernel (dHidden + dWeight GEMMs)", ("bwd/dhidden", "bwd/dweight"), 4 * nhv, 4 * nhv),
        ("lmhead_fwd_kernel (logits + online softmax statistics)", ("fwd/logits_stats",), 2 * nhv, 2 * nhv),
        ("lmhead_dlogit_kernel (logit recompute + dlogit)", ("bwd/dlogit",), 0.0, 2 * nhv),
    ]
    kernels = []
    for label, keys, algo, execd in classes:
        ms = sum(timing.get(k, {"ms": 0})["ms"] for k in keys)
        launches = sum(timing.get(k, {"launches": 0})["launches"] for k in keys)
        if launches == 0:
            continue
        kernels.append({
            "kernel": label, "launches_per_step": launches / args.steps, "ms_per_step": ms / args.steps,
            "avg_launch_ms": ms / launches,
            "algorithmic_tflops": algo * args.steps / (ms * 1e-3) / 1e12,
            "executed_tflops": execd * args.steps / (ms * 1e-3) / 1e12,
        })
    dom = max(kernels, key=lambda k: k["ms_per_step"])
    roofline = {
        "bound": "mfma", "kernel": dom["kernel"], "achieved": dom["algorithmic_tflops"] or dom["executed_tflops"],
        "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": (dom["algorithmic_tflops"] or dom["executed_tflops"]) / MFMA_BF16_PEAK_TFLOPS,
        "avg_launch_ms": dom["avg_launch_ms"], "traffic": None,
        "kernels": kernels,
        "path_algorithmic_tflops": 6 * nhv / (ms_per_step * 1e-3) / 1e12,
        "path_frac_of_peak": 6 * nhv / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "other_phases_ms_per_step": {k: t["ms"] / args.steps for k, t in timing.items()
                                     if k in ("fwd/merge", "fwd/label", "bwd/transpose")},
    }

    out = {
        "metric": "trained tokens/sec for fused logprob+GRPO loss fwd+bwd, Qwen3-8B shape; % MFMA peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: fused LM-head logprob + GRPO/PPO loss fwd+bwd", "tokens": n,
                   "hidden": h, "vocab": v, "sequences": len(rl["lengths"]), "group": group,
                   "vocab_chunk": args.vocab_chunk or "default"},
        "roofline": roofline,
        "parity": {"logprob_max_abs_err_subset": lp_err},
    }
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(hid, w, lab, args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
