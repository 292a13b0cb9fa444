"""The per-micro-batch loss assembly of the FSDP actor on the HIP path.

``CausalLM.forward_backward_fn`` keeps the contract of
axon/models/fsdp_models.py:183-279: run the model forward, evaluate the registry loss
(with the sampler correction hook), subtract the entropy bonus, add the KL penalty, scale by
``dp_replicas`` and report the same metrics.  The model forward itself is the caller's: ``module`` is
any callable ``module(model_inputs, meta_info) -> {"log_probs": ..., "entropys": ...}`` (in the
reference that is ``CausalLM.forward_fn`` around the HF model and the fused LM head).

The two side terms and the two entropy metrics come out of ONE kernel pass
(``axon_side_terms``) instead of three ``agg_loss`` calls and an elementwise KL chain.
"""

from __future__ import annotations

import numpy as np
import torch

from axon_amd import _lib, _ops
from axon_amd.trainer.algos.loss import compute_loss_fn
from axon_amd.utils.rl.sampler import compute_sampler_corr_metrics_from_logprobs


class _SideTerms(torch.autograd.Function):
    """(aggregated entropy, aggregated KL penalty, raw sums) with gradients to entropy / log_probs."""

    @staticmethod
    def forward(ctx, entropy, log_probs, ref_log_probs, mask, rows, kl_type, kl_plus, agg):
        acc, agg_w, grad_kl = _ops.side_terms(entropy, log_probs, ref_log_probs, mask, rows, kl_type=kl_type,
                                              kl_plus=kl_plus, **agg)
        ctx.save_for_backward(agg_w, grad_kl, acc)
        ctx.dtypes = (entropy.dtype if entropy is not None else None, log_probs.dtype if log_probs is not None else None)
        ctx.mark_non_differentiable(acc)
        return acc[0].clone(), acc[1].clone(), acc

    @staticmethod
    def backward(ctx, g_ent, g_kl, _g_acc):
        agg_w, grad_kl, acc = ctx.saved_tensors
        d_ent = d_lp = None
        if agg_w is not None and ctx.needs_input_grad[0]:
            d_ent = _ops.scale_f32(agg_w, g_ent, acc[5]).to(ctx.dtypes[0])
        if grad_kl is not None and ctx.needs_input_grad[1]:
            d_lp = _ops.scale_f32(grad_kl, g_kl, acc[5]).to(ctx.dtypes[1])
        return d_ent, d_lp, None, None, None, None, None, None


def loss_from_outputs(data, log_prob, entropy, meta_info):
    """Everything of ``forward_backward_fn`` after the model forward (fsdp_models.py:224-278).

    Returns ``(scaled_loss, metrics)``.  ``data.batch["log_probs"]`` is set; ``response_mask`` may be
    overwritten by the sampler correction hook, while the side terms keep the mask they were given
    (the reference captures it before the hook, :197-211).
    """
    loss_fn = meta_info["loss_fn"]
    loss_fn_args = meta_info["loss_fn_args"]
    dp_replicas = meta_info["dp_replicas"]
    n_micro_batches = meta_info.get("n_micro_batches", 1)

    b = data.batch
    response_mask = b["response_mask"]  # before compute_loss_fn can replace it
    cu = data.meta_info.get("cu_seqlens", None) if data.meta_info else None
    nps = data.non_tensor_batch.get("num_program_steps", None) if data.non_tensor_batch else None
    if nps is None:
        nps = b.get("num_program_steps", None)
    elif isinstance(nps, np.ndarray):
        nps = torch.from_numpy(nps.astype(np.int64))
    token_reduce = loss_fn_args.get("token_reduce", "sum")
    batch_reduce = loss_fn_args.get("batch_reduce", "token-mean")
    valid = {"token-mean": b.get("valid_token_count", None), "step-mean": b.get("valid_batch_size", None),
             "program-mean": b.get("valid_program_count", None)}[batch_reduce]
    agg = dict(token_reduce=token_reduce, batch_reduce=batch_reduce,
               num_program_tokens=b.get("num_program_tokens", None), num_program_steps=nps, valid_count=valid)

    b["log_probs"] = log_prob
    pg_loss, pg_metrics = compute_loss_fn(data, loss_fn=loss_fn, loss_fn_args=loss_fn_args)
    metrics = dict(pg_metrics)
    loss = pg_loss

    sampler_log_prob = b.get("sampler_log_probs", None)
    if loss_fn != "bypass_mode" and sampler_log_prob is not None:
        metrics.update(compute_sampler_corr_metrics_from_logprobs(log_prob=log_prob, sampler_log_prob=sampler_log_prob,
                                                                  response_mask=response_mask, cu_seqlens=cu))

    entropy_coef = loss_fn_args.get("entropy_coef", 0)
    kl_coef = loss_fn_args.get("kl_coef", 0)
    kl_type, kl_plus = (0, 0)
    ref = None
    if kl_coef != 0:
        assert "ref_log_prob" in b, "ref_log_prob is required for KL loss"
        ref = b["ref_log_prob"]
        kl_type, kl_plus = _ops.kl_type_of(loss_fn_args.get("kl_type", "low_var_kl"))
    _lib.require_device(entropy, "forward_backward_fn")
    rows = _ops.rows_of(entropy, cu)
    ent_in = entropy if entropy_coef != 0 else entropy.detach()
    ent_agg, kl_agg, acc = _SideTerms.apply(ent_in, log_prob if kl_type else None, ref, response_mask, rows, kl_type,
                                            kl_plus, agg)
    if entropy_coef != 0:
        loss = loss - ent_agg * entropy_coef
    if kl_coef != 0:
        loss = loss + kl_agg * kl_coef
    # one readback for pg_loss and the side-term metrics
    vals = torch.stack([pg_loss.detach().float(), acc[0], acc[1], acc[2], acc[4]]).tolist()
    metrics["pg_loss"] = vals[0] * n_micro_batches
    metrics["entropy"] = vals[1] * n_micro_batches
    metrics["entropy_token_mean"] = vals[3] / max(vals[4], 1.0)
    if kl_coef != 0:
        metrics["kl_loss"] = vals[2] * n_micro_batches
        metrics["kl_coef"] = kl_coef
    return loss * dp_replicas, metrics


class CausalLM:
    @staticmethod
    def forward_backward_fn(module, data, meta_info):
        """Per micro-batch forward + loss; ``data`` is a DataProto.  Returns ``(scaled_loss, metrics)``."""
        model_inputs = {**data.batch, **data.non_tensor_batch}
        result = module(model_inputs, {**meta_info, "temperature": meta_info["temperature"], "calculate_entropy": True})
        return loss_from_outputs(data, result["log_probs"], result["entropys"], meta_info)
