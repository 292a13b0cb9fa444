"""Head forward, loss and head backward of one micro-batch as ONE autograd node, block of tokens by block.

The reference's per-micro-batch step (``CausalLM.forward_backward_fn``, axon/models/fsdp_models.py:183-279) runs
the fused head over all tokens, then the registry loss and the entropy / KL side terms, and autograd then runs the
head's backward, which recomputes the logits (axon/utils/kernel/kernels.py:1377-1585): 8 N H V flop executed for
the 6 that count.  Here the three stages run block of consecutive tokens by block: the block's forward over the whole
vocabulary keeps 2 bytes per logit (``axon_lmhead_fwd``'s stash), the loss kernels run on the block's positions
with the batch-wide denominators, the block's backward decodes its dlogits from the stash, and the next block
reuses the same stash buffer.  What is held from a forward to its backward is one block's stash, a fixed number of
bytes whatever the number of tokens, and no logit is computed twice.

Everything the loss needs from outside a block is known before the first block: the sampler correction reads
only ``old_log_probs`` / ``sampler_log_probs`` (it runs once, over the whole batch), and the denominators of
``agg_loss`` (axon/trainer/algos/loss/utils.py:120-251) are counts of the mask.  Given those, PPO / DAPO,
REINFORCE / GPG and CISPO with ``sum`` / ``token-mean`` and the entropy / KL terms are sums over tokens (blocks
may be cut anywhere); GSPO and every per-row ``token_reduce`` / ``batch_reduce`` are sums over sequences (blocks
are cut at sequence ends).  Losses that select tokens across the batch (KL-Cov, Clip-Cov), GEO_MEAN and batches
with a sequence longer than a block take the unfused path (``packed_logprobs`` + ``loss_from_outputs``).

The node returns the loss; its backward hands autograd the finished ``d_hidden`` / ``d_weight`` times the incoming
scalar.
"""

from __future__ import annotations

import torch

from axon_amd import _lib, _ops
from axon_amd.trainer.algos.loss.loss import POLICY_LOSS_KINDS, policy_loss_metrics, policy_loss_spec

# Tokens per block.  One block's stash is 2 bytes x block x vocab (2.5 GB at 8192 x 151936).  The weight
# gradient is formed once per group of DEFAULT_DW_GROUP blocks (their bf16 dlogits, 2 bytes x block x vocab
# each, wait in the workspace) and carried from group to group in fp32, one read-modify-write of
# vocab x hidden x 4 bytes per group.
DEFAULT_BLOCK_TOKENS = 8192
DEFAULT_DW_GROUP = 2
_TILE = 256


def token_blocks(n: int, block_tokens: int):
    """Hidden-row ranges that cover ``n`` rows: blocks of ``block_tokens`` rows (rounded up to the GEMM tile), the
    last one shorter; when that would leave a last block of under a quarter of a block, equal blocks instead."""
    nb = max(-(-int(block_tokens) // _TILE), 1) * _TILE
    n_blocks = max(1, -(-n // nb))
    if n_blocks > 1 and n - (n_blocks - 1) * nb < nb // 4:
        nb = -(-(-(-n // n_blocks)) // _TILE) * _TILE
    return [(a, min(a + nb, n)) for a in range(0, n, nb)]


def sequence_blocks(cu: list, block_tokens: int):
    """Consecutive groups of whole sequences of at most ``block_tokens`` tokens each: ``[(row0, row1), ...]``,
    or None when one sequence alone is longer than a block."""
    out, r0, n_rows = [], 0, len(cu) - 1
    while r0 < n_rows:
        r1 = r0 + 1
        if cu[r1] - cu[r0] > block_tokens:
            return None
        while r1 < n_rows and cu[r1 + 1] - cu[r0] <= block_tokens:
            r1 += 1
        out.append((r0, r1))
        r0 = r1
    return out


def _global_count(mask, rows, batch_reduce, given):
    """The batch-wide denominator of ``agg_loss``'s batch reduction as a device scalar (loss/utils.py:190-214):
    the count the batch carries, else the number of mask tokens (token-mean) or of rows with any (step-mean)."""
    if given is not None:
        return given
    if batch_reduce == "token-mean":
        return mask.sum(dtype=torch.float64).reshape(1)
    if batch_reduce == "step-mean":
        cnt, _, _ = _ops.row_stats(mask if mask.dtype == torch.float32 else mask.float(), None, mask, rows,
                                   want_sum=False)
        return (cnt > 0).sum(dtype=torch.float64).reshape(1)
    raise AssertionError("valid_program_count required for batch_reduce='program-mean'")


_PINNED: dict = {}


def _start_readback(values):
    """Start the device-to-host copy of a small float64 tensor into pinned memory on the current stream and
    return ``(host tensor, event)``: the host waits for the event only, so launches enqueued after this call
    keep the GPU busy while the host reads the values and goes on.  One pinned buffer per device, reused: read
    the values before the next call."""
    dev = values.device
    n = int(values.numel())
    buf = _PINNED.get(dev.index)
    if buf is None or buf.numel() < n:
        buf = torch.empty(max(n, 128), dtype=torch.float64, pin_memory=True)
        _PINNED[dev.index] = buf
    host = buf[:n]
    host.copy_(values, non_blocking=True)
    event = torch.cuda.Event()
    event.record()
    return host, event


def _rows_slice(x, r0, r1):
    return None if x is None else torch.as_tensor(x).reshape(-1)[r0:r1]


class _BlockedHeadLoss(torch.autograd.Function):
    """(loss, log_probs, entropy, sums) of the whole micro-batch; gradients to ``hidden`` and ``weight``."""

    @staticmethod
    def forward(ctx, hidden, weight, spec):
        n = hidden.shape[0]
        dev = hidden.device
        kind, tensors, hp = spec["kind"], spec["tensors"], spec["hp"]
        side = spec["side"]
        cu, cu_host, seq_mode = spec["cu"], spec["cu_host"], spec["seq_mode"]

        if seq_mode:
            row_blocks = spec["row_blocks"]
            # hidden rows of a block: its sequences, lengthened to a multiple of four rows (the stash needs it);
            # the up to three rows borrowed from the next block carry a zero gradient here and are done again there
            ranges = []
            for r0, r1 in row_blocks:
                a, b = cu_host[r0], cu_host[r1]
                ranges.append((a, min(n, a + (b - a + 3) // 4 * 4)))
            slots = [(cu_host[r0], cu_host[r1]) for r0, r1 in row_blocks]
        else:
            ranges = token_blocks(n, spec["block_tokens"])
            # hidden row r writes position r + 1: a block of rows [a, b) owns positions a + 1 .. b
            slots = [(0 if k == 0 else a + 1, n if k == len(ranges) - 1 else b + 1) for k, (a, b) in enumerate(ranges)]

        hb = _ops.HeadBlocks(hidden, weight, spec["ids"], spec["inv_t"], ranges, softcap=spec["softcap"],
                             seq_start=spec["seq_start"], vocab_chunk=spec["vocab_chunk"], dw_group=spec["dw_group"],
                             timing=_ops.TIMING)
        g_lp = torch.zeros(n + 4, device=dev, dtype=torch.float32)
        want_ent_grad = side is not None and side["entropy_coef"] != 0
        g_en = torch.zeros(n + 4, device=dev, dtype=torch.float32) if want_ent_grad else None
        accs, side_accs = [], []

        out = {}

        def finish():
            """After the last block's loss, before its backward: the step's scalars are complete.  Their readback
            starts here, so that the host can pick them up (and prepare whatever comes next) while the GPU still
            works through the last block's backward."""
            sums = torch.stack(accs).sum(0) if accs else torch.zeros(8, device=dev)
            side_sums = torch.stack(side_accs).sum(0) if side_accs else torch.zeros(8, device=dev)
            loss = sums[0].clone()
            if side is not None:
                if side["entropy_coef"] != 0:
                    loss = loss - side_sums[0] * side["entropy_coef"]
                if side["kl_type"] and side["kl_coef"] != 0:
                    loss = loss + side_sums[1] * side["kl_coef"]
            scalars = [sums[:5].double(), side_sums[:5].double()]
            if spec.get("after_forward") is not None:  # more scalars from the whole-stream outputs (device tensors)
                scalars += [t.double().reshape(-1) for t in spec["after_forward"](hb.logprobs, hb.entropy)]
            spec["readback"] = _start_readback(torch.cat(scalars))
            out.update(loss=loss, sums=sums, side_sums=side_sums)

        for k, (lo, hi) in enumerate(slots):
            hb.forward(k)
            cut = lambda t: None if t is None else t.reshape(-1)[lo:hi]  # noqa: E731
            if seq_mode:
                r0, r1 = spec["row_blocks"][k]
                rows = _ops.Rows(r1 - r0, hi - lo, 0, (cu[r0:r1 + 1] - cu[r0:r0 + 1]).contiguous(), (hi - lo,))
                per_row = {key: _rows_slice(hp[key], r0, r1)
                           for key in ("per_row_token_count", "num_program_tokens", "num_program_steps")}
            else:
                rows = _ops.Rows(1, hi - lo, hi - lo, None, (1, hi - lo))
                per_row = {key: None for key in ("per_row_token_count", "num_program_tokens", "num_program_steps")}
            lp_b = hb.logprobs[lo:hi]
            acc, grad = _ops.policy_loss(
                kind, lp_b, cut(tensors["old_log_probs"]), cut(tensors["advantages"]), cut(tensors["response_mask"]),
                cut(tensors["sampler_is_weights"]), rows, token_reduce=hp["token_reduce"],
                batch_reduce=hp["batch_reduce"], ratio_lo=hp["ratio_lo"], ratio_hi=hp["ratio_hi"],
                clip_c=hp["clip_c"], valid_count=hp["valid_count"], **per_row)
            accs.append(acc)
            torch.mul(grad.reshape(-1), acc[5], out=g_lp[lo:hi])
            if side is not None:
                s_acc, agg_w, grad_kl = _ops.side_terms(
                    hb.entropy[lo:hi], lp_b if side["kl_type"] else None, cut(side["ref"]), cut(side["mask"]), rows,
                    token_reduce=hp["token_reduce"], batch_reduce=hp["batch_reduce"], kl_type=side["kl_type"],
                    kl_plus=side["kl_plus"], valid_count=side["valid_count"], **per_row)
                side_accs.append(s_acc)
                if want_ent_grad:
                    torch.mul(agg_w.reshape(-1), s_acc[5] * (-side["entropy_coef"]), out=g_en[lo:hi])
                if side["kl_type"] and side["kl_coef"] != 0:
                    g_lp[lo:hi].addcmul_(grad_kl.reshape(-1), s_acc[5], value=side["kl_coef"])
            if k == len(slots) - 1:
                finish()
            hb.backward(k, g_lp, g_en)

        loss, sums, side_sums = out["loss"], out["sums"], out["side_sums"]
        ctx.grads = (hb.d_hidden, hb.d_weight)
        ctx.head_workspace_bytes = hb.workspace_bytes
        spec["stash_bytes"], spec["workspace_bytes"], spec["n_blocks"] = hb.stash_bytes, hb.workspace_bytes, len(ranges)
        spec["dw_group_used"] = hb.dw_group
        log_probs, entropy = hb.logprobs, hb.entropy
        hb.d_hidden = hb.d_weight = None
        ctx.mark_non_differentiable(log_probs, entropy, sums, side_sums)
        return loss, log_probs, entropy, sums, side_sums

    @staticmethod
    def backward(ctx, g_loss, _g_lp, _g_en, _g_sums, _g_side):
        if ctx.grads is None:
            raise RuntimeError("the fused head-and-loss node finishes its gradients in the forward and hands them "
                               "over once: backward through it a second time is not possible")
        d_hidden, d_weight = ctx.grads
        ctx.grads = None
        _ops.scale_bf16_unless_one(d_hidden, g_loss)
        _ops.scale_bf16_unless_one(d_weight, g_loss)
        return d_hidden, d_weight, None


def blocked_spec(hidden, weight, packed_ids, cu_seqlens, data, loss_fn, loss_fn_args, temperature, *,
                 block_tokens=DEFAULT_BLOCK_TOKENS, vocab_chunk=0, dw_group=DEFAULT_DW_GROUP, logit_softcapping=None,
                 side_mask=None, cu_host=None):
    """What ``_BlockedHeadLoss`` needs, or None when this batch has to take the unfused path.  ``data.batch`` holds
    the packed per-token tensors (after the sampler correction); ``side_mask`` the mask of the entropy / KL
    terms (the one from before the correction, fsdp_models.py:197-211) or None for no side terms."""
    if loss_fn not in POLICY_LOSS_KINDS or hidden.dim() != 2 or hidden.shape[0] == 0:
        return None
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        return None
    kind, default_tr = POLICY_LOSS_KINDS[loss_fn]
    n = int(hidden.shape[0])
    b = data.batch
    _, _, tensors, hp = policy_loss_spec(kind, data, loss_fn_args, default_tr, with_log_probs=False)
    for name, t in tensors.items():
        if t is not None and int(t.numel()) != n:
            raise ValueError(f"fused head loss: {name} has {int(t.numel())} entries for {n} packed tokens")
    cu = cu_seqlens.to(device=hidden.device, dtype=torch.int32).contiguous()
    rows_all = _ops.Rows(int(cu.numel()) - 1, n, 0, cu, (n,))
    seq_mode = kind == 1 or hp["token_reduce"] != "sum" or hp["batch_reduce"] != "token-mean"
    spec = dict(kind=kind, tensors=tensors, hp=dict(hp), cu=cu, cu_host=None, seq_mode=seq_mode,
                block_tokens=int(block_tokens), vocab_chunk=int(vocab_chunk), dw_group=int(dw_group),
                ids=packed_ids.reshape(-1),
                inv_t=1.0 / float(temperature), softcap=0.0 if logit_softcapping is None else float(logit_softcapping),
                seq_start=_ops.seq_start_flags(cu, n), side=None)
    if seq_mode:
        if hp["token_reduce"] == "mean-norm":
            return None  # divides by the padded row length: not a packed-layout reduction
        host = cu_host if cu_host is not None else cu.tolist()  # one readback: where the sequences end
        if host[0] != 0 or host[-1] != n:
            raise ValueError(f"fused head loss: cu_seqlens spans {host[0]}..{host[-1]}, the batch has {n} tokens")
        spec["cu_host"] = host
        spec["row_blocks"] = sequence_blocks(host, int(block_tokens))
        if spec["row_blocks"] is None:
            return None
    mask = tensors["response_mask"]
    spec["hp"]["valid_count"] = _global_count(mask, rows_all, hp["batch_reduce"], hp["valid_count"])
    if side_mask is not None:
        entropy_coef = loss_fn_args.get("entropy_coef", 0)
        kl_coef = loss_fn_args.get("kl_coef", 0)
        kl_type, kl_plus, ref = 0, 0, None
        if kl_coef != 0:
            assert "ref_log_prob" in b, "ref_log_prob is required for KL loss"
            ref = b["ref_log_prob"]
            kl_type, kl_plus = _ops.kl_type_of(loss_fn_args.get("kl_type", "low_var_kl"))
        same = side_mask is mask
        spec["side"] = dict(mask=side_mask, ref=ref, kl_type=kl_type, kl_plus=kl_plus, entropy_coef=entropy_coef,
                            kl_coef=kl_coef,
                            valid_count=spec["hp"]["valid_count"] if same else
                            _global_count(side_mask, rows_all, hp["batch_reduce"], hp["valid_count"]))
    return spec


def blocked_head_loss(hidden, weight, spec):
    """Run the node: ``(loss, log_probs, entropy, sums, side_sums)``; ``loss`` carries the gradient."""
    _lib.require_device(hidden, "fused head loss")
    return _BlockedHeadLoss.apply(hidden, weight, spec)


def fused_head_loss(hidden, weight, packed_ids, cu_seqlens, data, meta_info, *,
                    block_tokens=DEFAULT_BLOCK_TOKENS, vocab_chunk=0, dw_group=DEFAULT_DW_GROUP,
                    logit_softcapping=None, cu_host=None):
    """Everything of ``forward_backward_fn`` from the final hidden states on (fsdp_models.py:203-278): head, sampler
    correction hook, registry loss, sampler-gap metrics, entropy bonus, KL penalty, ``dp_replicas`` scaling.

    ``hidden`` ``[N, H]`` packed final hidden states and ``weight`` ``[V, H]`` (bf16, the tensors that receive the
    gradients), ``packed_ids`` ``[N]`` the packed token ids, ``cu_seqlens`` int32 ``[S + 1]``; ``data.batch``
    holds the packed per-token tensors of the loss (``old_log_probs``, ``advantages``, ``response_mask``, ...);
    ``meta_info`` as for ``forward_backward_fn`` (``loss_fn``, ``loss_fn_args``, ``temperature``, ``dp_replicas``,
    ``n_micro_batches``).  Returns ``(scaled_loss, metrics)`` with the reference's metric names;
    ``data.batch["log_probs"]`` / ``["entropys"]`` are set to the (detached) head outputs and ``meta_info`` of
    ``data`` gets ``head_backward`` ("blocked-stash" or "recompute"), and for the blocked path ``stash_bytes``,
    ``head_workspace_bytes``, ``n_blocks`` and ``dw_group`` (blocks per weight-gradient GEMM).

    ``cu_host``: the same offsets as a Python list, for a caller that has them (saves the one readback that the
    sequence-cut blocks need)."""
    from axon_amd.models.fsdp_models import loss_from_outputs
    from axon_amd.trainer.algos.loss.registry import _SAMPLER_SWITCHES
    from axon_amd.utils.fsdp.forward_utils import packed_logprobs
    from axon_amd.utils.rl.sampler import (compute_sampler_correction_and_add_to_batch, sampler_gap_metrics,
                                           sampler_gap_sums)

    loss_fn = meta_info["loss_fn"]
    loss_fn_args = meta_info["loss_fn_args"] or {}
    dp_replicas = meta_info["dp_replicas"]
    n_micro_batches = meta_info.get("n_micro_batches", 1)
    temperature = meta_info["temperature"]
    if data.meta_info is None:
        data.meta_info = {}
    data.meta_info["cu_seqlens"] = cu_seqlens
    hidden2 = hidden.reshape(-1, hidden.shape[-1])

    b = data.batch
    side_mask = b["response_mask"]  # before the correction can replace it
    spec = None
    if loss_fn in POLICY_LOSS_KINDS and hidden2.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        corr_metrics = {}
        wanted = any(loss_fn_args.get(k, None) is not None for k in _SAMPLER_SWITCHES)
        if wanted and "sampler_log_probs" in b:
            data, corr_metrics = compute_sampler_correction_and_add_to_batch(data, loss_fn_args)
            b = data.batch
        spec = blocked_spec(hidden2, weight, packed_ids, cu_seqlens, data, loss_fn, loss_fn_args, temperature,
                            block_tokens=block_tokens, vocab_chunk=vocab_chunk, dw_group=dw_group,
                            logit_softcapping=logit_softcapping, side_mask=side_mask, cu_host=cu_host)
        if spec is None and wanted and "sampler_log_probs" in b:
            # the unfused path applies the correction itself: hand it the batch as it was
            b["response_mask"] = side_mask
            b.pop("sampler_is_weights", None)
    if spec is None:
        log_prob, entropy = packed_logprobs(hidden2, weight, packed_ids, cu_seqlens, temperature, logit_softcapping)
        data.meta_info["head_backward"] = "recompute"
        return loss_from_outputs(data, log_prob, entropy, meta_info)

    sampler_log_prob = b.get("sampler_log_probs", None)
    if sampler_log_prob is not None:  # the gap between the current policy and the sampler (fsdp_models.py:232-241)
        spec["after_forward"] = lambda lp, _ent: [sampler_gap_sums(lp, sampler_log_prob, side_mask, cu_seqlens)]
    loss, log_prob, entropy, _sums, _side_sums = blocked_head_loss(hidden2, weight, spec)
    b["log_probs"], b["entropys"] = log_prob, entropy
    data.meta_info.update(head_backward="blocked-stash", stash_bytes=spec["stash_bytes"],
                          head_workspace_bytes=spec["workspace_bytes"], n_blocks=spec["n_blocks"],
                          dw_group=spec["dw_group_used"])
    host, event = spec["readback"]  # the one readback of the step's scalars, started before the last block's backward
    event.synchronize()
    vals = host.tolist()
    metrics = {**policy_loss_metrics(spec["kind"], vals[:5]), **corr_metrics}
    if sampler_log_prob is not None:
        metrics.update(sampler_gap_metrics(vals[10:], int(cu_seqlens.numel()) - 1))
    metrics["pg_loss"] = vals[0] * n_micro_batches
    metrics["entropy"] = vals[5] * n_micro_batches
    metrics["entropy_token_mean"] = vals[7] / max(vals[9], 1.0)
    if spec["side"]["kl_coef"] != 0:
        metrics["kl_loss"] = vals[6] * n_micro_batches
        metrics["kl_coef"] = spec["side"]["kl_coef"]
    return loss * dp_replicas, metrics
