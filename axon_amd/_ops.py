"""Tensor-level wrappers over the C ABI (include/axon_amd.h).

Each function validates on the host, allocates outputs/workspace with torch,
passes raw device pointers and the current stream to ``libaxon_amd.so`` and
raises on a non-zero status.  Nothing here computes on the CPU.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib
from ._lib import MASK_F32, MASK_I64, check, ptr, require_device, stream_ptr


@dataclass
class Rows:
    """How a flat array of ``n_slots`` values splits into rows (sequences)."""

    n_rows: int
    n_slots: int
    uniform_len: int  # T for a padded [B, T] layout, 0 for packed
    cu: torch.Tensor | None  # int32 [n_rows + 1] on device for packed
    shape: tuple

    @property
    def cu_ptr(self):
        # the kernels dereference this pointer: offsets that live in host memory would fault the GPU
        if self.cu is not None and not self.cu.is_cuda:
            raise _lib.AxonAmdError(f"cu_seqlens is on {self.cu.device}: the row offsets must live on the GPU "
                                    "(rows_of puts them on the device of the tensor it is given)")
        return ptr(self.cu)


def rows_of(t: torch.Tensor, cu_seqlens: torch.Tensor | None = None) -> Rows:
    """Row layout of ``t``: [B, T] padded, or packed [N] (also [1, N]) with ``cu_seqlens``."""
    if cu_seqlens is not None:
        if cu_seqlens.dtype != torch.int32:
            cu_seqlens = cu_seqlens.to(torch.int32)
        cu = cu_seqlens.to(t.device).contiguous()
        return Rows(int(cu.numel()) - 1, int(t.numel()), 0, cu, tuple(t.shape))
    if t.dim() != 2:
        raise ValueError(f"expected a [batch, seq] tensor or packed data with cu_seqlens, got shape {tuple(t.shape)}")
    b, s = t.shape
    return Rows(int(b), int(b * s), int(s), None, tuple(t.shape))


def _on_16_bytes(t: torch.Tensor) -> torch.Tensor:
    """The kernels move four values per access: a view that starts off a 16-byte boundary is copied."""
    return t if t.data_ptr() % 16 == 0 else t.clone()


def f32(t: torch.Tensor) -> torch.Tensor:
    if t.requires_grad:
        t = t.detach()
    if t.dtype != torch.float32 or not t.is_contiguous():  # the usual operand passes through untouched
        t = t.to(torch.float32).contiguous()
    return _on_16_bytes(t)


def mask_arg(mask: torch.Tensor):
    """Normalise a response mask once: fp32 and int64 are read natively by the kernels."""
    if mask.requires_grad:
        mask = mask.detach()
    if not mask.is_contiguous():
        mask = mask.contiguous()
    if mask.dtype == torch.int64:
        return _on_16_bytes(mask), MASK_I64
    if mask.dtype != torch.float32:
        mask = mask.to(torch.float32)
    return _on_16_bytes(mask), MASK_F32


def _same_len(what: str, n: int, **tensors) -> None:
    """The kernels index every operand with the same token (or row) index: a shorter operand would be read
    out of bounds, so the lengths are checked here, on the host."""
    for name, t in tensors.items():
        if t is not None and int(t.numel()) != n:
            raise ValueError(f"{what}: {name} has {int(t.numel())} elements, expected {n}")


def _zeros(n, device, dtype=torch.float32):
    return torch.zeros(n, device=device, dtype=dtype)


def _acc8(n_slots, device):
    """The eight scalar sums a kernel returns; the library writes all of them unless there are no tokens.  Under
    stream capture they start as NaN: a replay whose reduction never finished would then show."""
    if n_slots == 0:
        return _zeros(8, device)
    if torch.cuda.is_current_stream_capturing():
        return torch.full((8,), float("nan"), device=device, dtype=torch.float32)
    return torch.empty(8, device=device, dtype=torch.float32)


_PARTIALS: dict = {}


def _partials(n_slots, device):
    """Workspace of the per-workgroup partial sums (and the ticket counter behind them) of the elementwise
    kernels.  The counter has to be zero before the first launch and every launch leaves it zero, so one
    zero-filled buffer per (device, stream) is kept and reused: launches on one stream are ordered.

    Under stream capture nothing is kept: the fill of a buffer created there is recorded, not executed, and the
    buffer lives in the graph's own pool, so every captured call gets a workspace of its own whose fill is a node
    of the same graph (graphs then do not depend on each other's replays, and eager calls never share a buffer
    that a replay re-zeroes)."""
    nbytes = _lib.load().axon_reduce_partials_bytes(int(n_slots))
    if torch.cuda.is_current_stream_capturing():
        return torch.zeros(nbytes // 4, device=device, dtype=torch.float32)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr())
    ws = _PARTIALS.get(key)
    if ws is None:
        ws = torch.zeros(nbytes // 4, device=device, dtype=torch.float32)
        _PARTIALS[key] = ws
    return ws


def row_stats(a, b, mask, rows: Rows, *, flag_mode=0, threshold=0.0, want_cnt=True, want_sum=True):
    """Per-row (count, sum of (a-b)*mask, any-flag); see axon_row_stats."""
    lib = _lib.load()
    require_device(a, "row_stats")
    _same_len("row_stats", rows.n_slots, a=a, b=b, mask=mask)
    dev = a.device
    a = f32(a)
    b = f32(b) if b is not None else None
    mk = (None, MASK_F32) if mask is None else mask_arg(mask)
    # one zero-filled buffer (one fill launch) carries the up to three per-row outputs and, in front of them, the
    # workspace of the sums (an int64 and a float per row: 8-byte aligned at the start of the allocation)
    parts = [want_cnt, want_sum, bool(flag_mode)]
    r = max(rows.n_rows, 1)
    ws_floats = 3 * r if want_sum else 0
    buf = _zeros(ws_floats + sum(parts) * r, dev) if any(parts) else None
    ws = buf[:ws_floats] if want_sum else None
    outs = buf[ws_floats:].view(sum(parts), -1) if any(parts) else None
    slots = iter(range(sum(parts)))
    cnt = outs[next(slots)][: rows.n_rows] if want_cnt else None
    ssum = outs[next(slots)][: rows.n_rows] if want_sum else None
    flag = outs[next(slots)][: rows.n_rows].view(torch.int32) if flag_mode else None
    check(
        lib.axon_row_stats(ptr(a), ptr(b), ptr(mk[0]), mk[1], rows.cu_ptr, rows.n_rows, rows.n_slots,
                           rows.uniform_len, flag_mode, float(threshold), ptr(cnt), ptr(ssum), ptr(flag), ptr(ws),
                           stream_ptr()),
        "axon_row_stats",
    )
    return cnt, ssum, flag


def group_stats(scores, gidx, n_groups, eps, norm_by_std=True, want_scalar=True):
    lib = _lib.load()
    require_device(scores, "group_stats")
    dev = scores.device
    scores = f32(scores).reshape(-1)
    gidx = gidx.to(device=dev, dtype=torch.int64).reshape(-1).contiguous()
    n = int(scores.numel())
    stats = _zeros(3 * max(n_groups, 1), dev).view(3, -1)
    _same_len("group_stats", n, gidx=gidx)
    scalar = torch.empty(n, device=dev, dtype=torch.float32) if want_scalar else None
    check(
        lib.axon_group_stats(ptr(scores), ptr(gidx), n, int(n_groups), float(eps), int(norm_by_std),
                             ptr(stats[0]), ptr(stats[1]), ptr(stats[2]), ptr(scalar), stream_ptr()),
        "axon_group_stats",
    )
    return stats[0][:n_groups], stats[1][:n_groups], stats[2][:n_groups], scalar


def row_broadcast_mask(row_scalar, mask, rows: Rows, clamp_abs=0.0):
    lib = _lib.load()
    require_device(row_scalar, "row_broadcast_mask")
    _same_len("row_broadcast_mask", rows.n_slots, mask=mask)
    _same_len("row_broadcast_mask", rows.n_rows, row_scalar=row_scalar)
    mk, kind = mask_arg(mask)
    out = torch.empty(rows.shape, device=row_scalar.device, dtype=torch.float32)
    check(
        lib.axon_row_broadcast_mask(ptr(f32(row_scalar)), ptr(mk), kind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                                    rows.uniform_len, float(clamp_abs), ptr(out), stream_ptr()),
        "axon_row_broadcast_mask",
    )
    return out


SCAN_GAE, SCAN_GAE_RESPONSE_ONLY, SCAN_DISCOUNTED, SCAN_SUFFIX_SUM = 0, 1, 2, 3


def reverse_scan(mode, rewards, values, mask, rows: Rows, *, gamma=1.0, lam=1.0, row_baseline=None):
    """Time recurrence from each row's last token to its first; returns ``(adv | None, ret)``.  See
    axon_reverse_scan."""
    lib = _lib.load()
    require_device(rewards, "reverse_scan")
    _same_len("reverse_scan", rows.n_slots, rewards=rewards, values=values, mask=mask)
    dev = rewards.device
    rewards = f32(rewards)
    values = f32(values) if values is not None else None
    mk, kind = mask_arg(mask)
    base = f32(row_baseline).reshape(-1) if row_baseline is not None else None
    if base is not None and base.numel() != rows.n_rows:
        raise ValueError(f"row_baseline has {base.numel()} entries, batch has {rows.n_rows} rows")
    adv = None if mode == SCAN_DISCOUNTED else torch.empty(rows.shape, device=dev, dtype=torch.float32)
    ret = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    check(
        lib.axon_reverse_scan(mode, ptr(rewards), ptr(values), ptr(mk), kind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                              rows.uniform_len, float(gamma), float(lam), ptr(base), ptr(adv), ptr(ret),
                              stream_ptr()),
        "axon_reverse_scan",
    )
    return adv, ret


def masked_whiten(x, mask, *, remask=False, inplace=False, stats_only=False):
    """``(x - mean) * rsqrt(var + 1e-8)`` with the mean and variance taken over the mask (times the mask when
    ``remask``); returns ``(out, stats)`` with stats = device [mean, n, var, rsqrt(var + 1e-8)]."""
    lib = _lib.load()
    require_device(x, "masked_whiten")
    _same_len("masked_whiten", int(x.numel()), mask=mask)
    dev = x.device
    xf = f32(x)
    mk, kind = mask_arg(mask)
    n = int(xf.numel())
    if stats_only:
        out = None
    else:
        out = xf if (inplace and xf.data_ptr() == x.data_ptr()) else torch.empty_like(xf)
    stats = _zeros(4, dev)
    ws = torch.empty(max(lib.axon_masked_whiten_workspace_bytes(n) // 4, 8), device=dev, dtype=torch.float32)
    check(
        lib.axon_masked_whiten(ptr(xf), ptr(mk), kind, n, int(remask), ptr(out), ptr(stats), ptr(ws), stream_ptr()),
        "axon_masked_whiten",
    )
    return out, stats


GROUP_OPO, GROUP_MEAN_BASELINE, GROUP_PASSK, GROUP_KIMI = 0, 1, 2, 3


def group_scalar(mode, scores, lens, members, offsets, n_groups, *, eps=1e-6, normalize=True, coef=0.0,
                 threshold=1.0):
    """Per-row scalar from group members in compressed form; see axon_group_scalar."""
    lib = _lib.load()
    require_device(scores, "group_scalar")
    dev = scores.device
    scores = f32(scores).reshape(-1)
    lens = f32(lens).reshape(-1) if lens is not None else None
    members = members.to(device=dev, dtype=torch.int32).contiguous()
    offsets = offsets.to(device=dev, dtype=torch.int32).contiguous()
    n = int(scores.numel())
    if members.numel() != n or offsets.numel() != n_groups + 1:
        raise ValueError("members / offsets do not describe the rows of scores")
    out = torch.empty(n, device=dev, dtype=torch.float32)
    check(
        lib.axon_group_scalar(mode, ptr(scores), ptr(lens), ptr(members), ptr(offsets), n, int(n_groups), float(eps),
                              int(bool(normalize)), float(coef), float(threshold), ptr(out), stream_ptr()),
        "axon_group_scalar",
    )
    return out


# Operators that need a per-row quantity run as ONE launch in which a workgroup owns whole rows (one read of every
# input, row sums that repeat bit for bit) when the rows are long enough to fill a workgroup: it works on one or
# two rows at a time, so a batch of rows of a few tokens each would leave most of its threads idle.  Otherwise, and
# beyond ``OWNED_ROWS_MAX_SLOTS`` tokens, a token-parallel row pass followed by a token pass (two reads, float
# atomics per row).  At 2^26 tokens 0.31-0.34 ms against 0.40-0.43; at the sizes of real micro-batches one launch
# instead of four or five.
# A workgroup walks a row it owns 2048 slots at a time, alone: rows of more than ``OWNED_ROWS_MAX_MEAN_LEN`` slots
# (known for a padded layout; for a packed one only the mean is known on the host) take the two passes, which
# spread any row over the whole GPU.
OWNED_ROWS_MAX_SLOTS = 1 << 40
OWNED_ROWS_MIN_MEAN_LEN = 64
OWNED_ROWS_MAX_MEAN_LEN = 16384


def _own_rows(rows: "Rows") -> bool:
    n_rows = max(rows.n_rows, 1)
    return (4 <= rows.n_slots <= OWNED_ROWS_MAX_SLOTS and rows.n_slots >= OWNED_ROWS_MIN_MEAN_LEN * n_rows
            and rows.n_slots <= OWNED_ROWS_MAX_MEAN_LEN * n_rows)


IS_MODES = {None: 0, "token": 1, "sequence": 2}
RS_MODES = {None: 0, "token": 1, "sequence": 2, "geometric": 3}


def sampler_correction(old_lp, samp_lp, mask, rows: Rows, *, is_mode, is_threshold, rs_mode, rs_lr_lo, rs_lr_hi,
                       log_veto):
    """Importance weights and rejection / veto mask.  Without a row-level quantity: one elementwise pass.  With
    one (veto, sequence or geometric level): one launch in which a workgroup owns whole rows, or (short rows, see
    ``OWNED_ROWS_MIN_MEAN_LEN``) a row-stats pass followed by an elementwise pass.

    Returns (is_weights | None, new_mask fp32, acc[8] device tensor).
    """
    lib = _lib.load()
    require_device(old_lp, "sampler_correction")
    _same_len("sampler_correction", rows.n_slots, old_log_probs=old_lp, sampler_log_probs=samp_lp, mask=mask)
    dev = old_lp.device
    old_lp, samp_lp = f32(old_lp), f32(samp_lp)
    mk, kind = mask_arg(mask)
    has_veto = log_veto is not None
    need_row = is_mode == 2 or rs_mode >= 2 or has_veto
    isw = torch.empty(rows.shape, device=dev, dtype=torch.float32) if is_mode else None
    new_mask = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    acc = _acc8(rows.n_slots, dev)
    if need_row and _own_rows(rows):
        # a workgroup owns whole rows: one launch, one pass over the tokens, row sums in a fixed order
        check(
            lib.axon_sampler_correction_rows(ptr(old_lp), ptr(samp_lp), ptr(mk), kind, rows.cu_ptr, rows.n_rows,
                                             rows.n_slots, rows.uniform_len, is_mode, float(is_threshold), rs_mode,
                                             float(rs_lr_lo), float(rs_lr_hi), int(has_veto),
                                             float(log_veto if has_veto else 0.0), ptr(isw), ptr(new_mask), None,
                                             None, None, ptr(acc), ptr(_partials(rows.n_slots, dev)), stream_ptr()),
            "axon_sampler_correction_rows",
        )
        return isw, new_mask, acc
    cnt = ssum = flag = None
    if need_row:  # very large batches: a token-parallel row pass, then a token-parallel elementwise pass
        cnt, ssum, flag = row_stats(old_lp, samp_lp, mk, rows, flag_mode=1 if has_veto else 0,
                                    threshold=log_veto if has_veto else 0.0)
    check(
        lib.axon_sampler_correction(ptr(old_lp), ptr(samp_lp), ptr(mk), kind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                                    rows.uniform_len, is_mode, float(is_threshold), rs_mode, float(rs_lr_lo),
                                    float(rs_lr_hi), int(has_veto), float(log_veto if has_veto else 0.0), ptr(cnt),
                                    ptr(ssum), ptr(flag), ptr(isw), ptr(new_mask), ptr(acc),
                                    ptr(_partials(rows.n_slots, dev)), stream_ptr()),
        "axon_sampler_correction",
    )
    return isw, new_mask, acc


DIAG_OUT = 72


def sampler_diag(old_lp, samp_lp, mask, rows: Rows, *, is_mode, is_lo, is_hi, rs_mode, rs_lo, rs_hi, rs_lr_lo,
                 rs_lr_hi, log_is_lo, log_is_hi, log_rs_lo, log_rs_hi):
    """All mismatch diagnostics as one float64 device tensor of DIAG_OUT raw sums / extrema
    (layout: axon_sampler_diag in include/axon_amd.h).  No host synchronisation."""
    lib = _lib.load()
    require_device(old_lp, "sampler_diag")
    _same_len("sampler_diag", rows.n_slots, old_log_probs=old_lp, sampler_log_probs=samp_lp, mask=mask)
    dev = old_lp.device
    old_lp, samp_lp = f32(old_lp), f32(samp_lp)
    mk, kind = mask_arg(mask)
    nbytes = lib.axon_sampler_diag_workspace_bytes(rows.n_rows, rows.n_slots)
    ws = torch.empty(nbytes // 4, device=dev, dtype=torch.float32)
    ws[: 6 * rows.n_rows].zero_()
    out = torch.empty(DIAG_OUT, device=dev, dtype=torch.float64)
    check(
        lib.axon_sampler_diag(ptr(old_lp), ptr(samp_lp), ptr(mk), kind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                              rows.uniform_len, int(is_mode), float(is_lo), float(is_hi), int(rs_mode), float(rs_lo),
                              float(rs_hi), float(rs_lr_lo), float(rs_lr_hi), float(log_is_lo), float(log_is_hi),
                              float(log_rs_lo), float(log_rs_hi), ptr(ws), ptr(out), stream_ptr()),
        "axon_sampler_diag",
    )
    return out


TOKEN_REDUCE = {"sum": 0, "mean": 1, "mean-norm": 2, "mean-program": 3}
BATCH_REDUCE = {"token-mean": 0, "step-mean": 1, "program-mean": 2}


def _count_dev(x, dev, n=None, what="count"):
    """A count (or one count per row) as float64 on the device: the reference divides by the value as it is
    (loss/utils.py:224-229), so a fractional count, e.g. one averaged over ranks, is not truncated."""
    if x is None:
        return None
    if n is not None and int(x.numel()) != n:
        raise ValueError(f"{what} has {int(x.numel())} entries, expected one per row ({n})")
    t = torch.as_tensor(x)
    return t.to(device=dev, dtype=torch.float64).reshape(-1).contiguous()


def policy_loss(kind, log_probs, old_log_probs, advantages, mask, is_weights, rows: Rows, *, token_reduce,
                batch_reduce, ratio_lo, ratio_hi, clip_c, per_row_token_count=None, num_program_tokens=None,
                num_program_steps=None, valid_count=None):
    """Forward + gradient of the clipped policy loss.  Returns (acc[8], grad like log_probs).

    acc[0] is the loss; acc[1:5] are the metric sums; acc[5] is the factor the returned
    gradient still has to be multiplied by (see axon_policy_loss).
    """
    lib = _lib.load()
    require_device(log_probs, "policy_loss")
    _same_len("policy_loss", rows.n_slots, log_probs=log_probs, old_log_probs=old_log_probs, advantages=advantages,
              mask=mask, is_weights=is_weights)
    dev = log_probs.device
    lp, old, adv = f32(log_probs), f32(old_log_probs), f32(advantages)
    mk, mkind = mask_arg(mask)
    isw = f32(is_weights) if is_weights is not None else None
    tr, br = TOKEN_REDUCE[token_reduce], BATCH_REDUCE[batch_reduce]

    valid = _count_dev(valid_count, dev)
    grad = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    acc = _acc8(rows.n_slots, dev)
    # PPO with sum / token-mean needs no per-row quantity: one pass over the tokens, the
    # division by the token count happens when the last workgroup has the total.
    one_pass = kind != 1 and tr == 0 and br == 0
    prtc = _count_dev(per_row_token_count, dev, rows.n_rows, "per_row_token_count") if tr == 1 else None
    npt = _count_dev(num_program_tokens, dev, rows.n_rows, "num_program_tokens") if tr == 3 else None
    nps = _count_dev(num_program_steps, dev, rows.n_rows, "num_program_steps") if br == 2 else None
    if not one_pass and tr == 2 and not rows.uniform_len:
        raise ValueError("token_reduce='mean-norm' divides by the padded row length: needs a [batch, seq] layout")
    if not one_pass and _own_rows(rows):
        # a workgroup owns whole rows: one launch, still one pass over the tokens
        check(
            lib.axon_policy_loss_rows(kind, ptr(lp), ptr(old), ptr(adv), ptr(mk), mkind, ptr(isw), rows.cu_ptr,
                                      rows.n_rows, rows.n_slots, rows.uniform_len, tr, br, ptr(prtc), ptr(npt),
                                      ptr(nps), ptr(valid), float(ratio_lo), float(ratio_hi), float(clip_c),
                                      ptr(grad), ptr(acc), ptr(_partials(rows.n_slots, dev)), stream_ptr()),
            "axon_policy_loss_rows",
        )
        return acc, grad
    row_scale = row_mean = None
    if not one_pass:  # very large batches: row pass, row scales, token pass
        cnt, ssum, _ = row_stats(lp, old, mk, rows, want_sum=(kind == 1))
        row_scale = torch.empty(rows.n_rows, device=dev, dtype=torch.float32)
        row_mean = torch.empty(rows.n_rows, device=dev, dtype=torch.float32) if kind == 1 else None
        check(
            lib.axon_loss_row_scale(ptr(cnt), ptr(ssum), rows.n_rows, rows.uniform_len if rows.uniform_len else 0, tr,
                                    br, ptr(prtc), ptr(npt), ptr(nps), ptr(valid), ptr(row_scale), ptr(row_mean),
                                    stream_ptr()),
            "axon_loss_row_scale",
        )
    check(
        lib.axon_policy_loss(kind, ptr(lp), ptr(old), ptr(adv), ptr(mk), mkind, ptr(isw), rows.cu_ptr, rows.n_rows,
                             rows.n_slots, rows.uniform_len, ptr(row_scale), ptr(row_mean), 1.0, int(one_pass),
                             ptr(valid if one_pass else None), float(ratio_lo), float(ratio_hi), float(clip_c),
                             ptr(grad), ptr(acc), ptr(_partials(rows.n_slots, dev)), stream_ptr()),
        "axon_policy_loss",
    )
    return acc, grad


def cov_policy_loss(kind, log_probs, old_log_probs, advantages, mask, is_weights, rows: Rows, *, select_ratio,
                    ratio_lo=0.0, ratio_hi=0.0, cov_lb=0.0, cov_ub=0.0, kl_coef=1.0, seed=0, token_reduce,
                    batch_reduce, per_row_token_count=None, num_program_tokens=None, num_program_steps=None,
                    valid_count=None):
    """KL-Cov (kind 0) / Clip-Cov (kind 1): token selection (axon_cov_select) + loss and gradient
    (axon_cov_policy_loss).  Returns ``(acc[8], grad, keys, state)``; acc as in ``policy_loss`` with
    acc[1] = number of selected tokens (mask-weighted)."""
    lib = _lib.load()
    require_device(log_probs, "cov_policy_loss")
    _same_len("cov_policy_loss", rows.n_slots, log_probs=log_probs, old_log_probs=old_log_probs,
              advantages=advantages, mask=mask, is_weights=is_weights)
    dev = log_probs.device
    lp, old, adv = f32(log_probs), f32(old_log_probs), f32(advantages)
    mk, mkind = mask_arg(mask)
    isw = f32(is_weights) if is_weights is not None else None
    tr, br = TOKEN_REDUCE[token_reduce], BATCH_REDUCE[batch_reduce]
    n = rows.n_slots
    keys = torch.empty(max(n, 4), device=dev, dtype=torch.int32)
    state = torch.zeros((int(lib.axon_cov_select_state_bytes()) + 7) // 8, device=dev, dtype=torch.int64)
    ws = torch.empty(max(int(lib.axon_cov_select_workspace_bytes(n)), 16), device=dev, dtype=torch.uint8)
    check(
        lib.axon_cov_select(kind, ptr(lp), ptr(old), ptr(adv), ptr(mk), mkind, n, float(select_ratio), float(cov_lb),
                            float(cov_ub), float(ratio_lo), float(ratio_hi), int(seed) & 0xFFFFFFFF, ptr(keys),
                            ptr(state), ptr(ws), stream_ptr()),
        "axon_cov_select",
    )
    valid = _count_dev(valid_count, dev)
    grad = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    acc = _acc8(n, dev)
    one_pass = tr == 0 and br == 0
    row_scale = None
    if not one_pass:
        cnt, _, _ = row_stats(lp, None, mk, rows, want_sum=False)
        row_scale = torch.empty(rows.n_rows, device=dev, dtype=torch.float32)
        prtc = _count_dev(per_row_token_count, dev, rows.n_rows, "per_row_token_count") if tr == 1 else None
        npt = _count_dev(num_program_tokens, dev, rows.n_rows, "num_program_tokens") if tr == 3 else None
        nps = _count_dev(num_program_steps, dev, rows.n_rows, "num_program_steps") if br == 2 else None
        check(
            lib.axon_loss_row_scale(ptr(cnt), None, rows.n_rows, rows.uniform_len if rows.uniform_len else 0, tr, br,
                                    ptr(prtc), ptr(npt), ptr(nps), ptr(valid), ptr(row_scale), None, stream_ptr()),
            "axon_loss_row_scale",
        )
    check(
        lib.axon_cov_policy_loss(kind, ptr(lp), ptr(old), ptr(adv), ptr(mk), mkind, ptr(isw), rows.cu_ptr, rows.n_rows,
                                 n, rows.uniform_len, ptr(row_scale), 1.0, int(one_pass),
                                 ptr(valid if one_pass else None), float(ratio_lo), float(ratio_hi), float(kl_coef),
                                 ptr(keys), ptr(state), ptr(grad), ptr(acc), ptr(_partials(n, dev)), stream_ptr()),
        "axon_cov_policy_loss",
    )
    return acc, grad, keys, state


def gmpo_loss(log_probs, old_log_probs, advantages, mask, is_weights, rows: Rows, *, clip_low, clip_high):
    """GMPO loss and gradient; returns (acc[8], grad).  See axon_gmpo_loss."""
    lib = _lib.load()
    require_device(log_probs, "gmpo_loss")
    _same_len("gmpo_loss", rows.n_slots, log_probs=log_probs, old_log_probs=old_log_probs, advantages=advantages,
              mask=mask, is_weights=is_weights)
    dev = log_probs.device
    lp, old, adv = f32(log_probs), f32(old_log_probs), f32(advantages)
    mk, mkind = mask_arg(mask)
    isw = f32(is_weights) if is_weights is not None else None
    row_ws = torch.empty(5 * rows.n_rows, device=dev, dtype=torch.float32)
    row_ws[: 4 * rows.n_rows].zero_()
    grad = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    acc = _acc8(rows.n_slots, dev)
    check(
        lib.axon_gmpo_loss(ptr(lp), ptr(old), ptr(adv), ptr(mk), mkind, ptr(isw), rows.cu_ptr, rows.n_rows,
                           rows.n_slots, rows.uniform_len, float(clip_low), float(clip_high), ptr(row_ws), ptr(grad),
                           ptr(acc), ptr(_partials(rows.n_slots, dev)), stream_ptr()),
        "axon_gmpo_loss",
    )
    return acc, grad


KL_TYPES = {"kl": 1, "k1": 1, "abs": 2, "mse": 3, "k2": 3, "low_var_kl": 4, "k3": 4}


def kl_type_of(kl_penalty_type: str):
    """(type code, straight-through flag) of a kl_penalty type string (kl.py:176-187, 216-245)."""
    base = kl_penalty_type.rstrip("+")
    if base == "full":
        raise NotImplementedError("Full KL divergence requires logits, not just log probs")
    if base not in KL_TYPES:
        raise NotImplementedError(f"Unknown KL penalty type: {kl_penalty_type}")
    plus = kl_penalty_type.endswith("+") and kl_penalty_type not in ("mse", "k2")
    return KL_TYPES[base], int(plus)


def kl_penalty(logprob, ref_logprob, kl_type: int, kl_plus: int):
    """Per-token estimate and its derivative w.r.t. logprob (both fp32, shape of logprob)."""
    lib = _lib.load()
    require_device(logprob, "kl_penalty")
    _same_len("kl_penalty", int(logprob.numel()), ref_logprob=ref_logprob)
    lp, ref = f32(logprob), f32(ref_logprob)
    out, grad = torch.empty_like(lp), torch.empty_like(lp)
    check(lib.axon_kl_penalty(ptr(lp), ptr(ref), lp.numel(), kl_type, kl_plus, ptr(out), ptr(grad), stream_ptr()),
          "axon_kl_penalty")
    return out, grad


def kl_reward(scores, old_log_probs, ref_log_probs, mask, rows: Rows, *, kl_type: int, beta: float):
    """``(rewards, row mask sums, row kld sums)``; see axon_kl_reward."""
    lib = _lib.load()
    require_device(scores, "kl_reward")
    _same_len("kl_reward", rows.n_slots, scores=scores, old_log_probs=old_log_probs, ref_log_probs=ref_log_probs,
              mask=mask)
    dev = scores.device
    sc, old, ref = f32(scores), f32(old_log_probs), f32(ref_log_probs)
    mk, kind = mask_arg(mask)
    rewards = torch.empty(rows.shape, device=dev, dtype=torch.float32)
    row_vals = _zeros(2 * max(rows.n_rows, 1), dev).view(2, -1)
    check(
        lib.axon_kl_reward(ptr(sc), ptr(old), ptr(ref), ptr(mk), kind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                           rows.uniform_len, int(kl_type), float(beta), ptr(rewards), ptr(row_vals), stream_ptr()),
        "axon_kl_reward",
    )
    return rewards, row_vals[0][: rows.n_rows], row_vals[1][: rows.n_rows]


def side_terms(entropy, log_probs, ref_log_probs, mask, rows: Rows, *, token_reduce, batch_reduce, kl_type=0,
               kl_plus=0, per_row_token_count=None, num_program_tokens=None, num_program_steps=None,
               valid_count=None):
    """Aggregated entropy and KL penalty with their gradient arrays.  Returns (acc[8], agg_w | None,
    grad_kl | None); see axon_side_terms."""
    lib = _lib.load()
    anchor = entropy if entropy is not None else log_probs
    require_device(anchor, "side_terms")
    _same_len("side_terms", rows.n_slots, entropy=entropy, log_probs=log_probs if kl_type else None,
              ref_log_probs=ref_log_probs if kl_type else None, mask=mask)
    dev = anchor.device
    ent = f32(entropy) if entropy is not None else None
    lp = f32(log_probs) if kl_type else None
    ref = f32(ref_log_probs) if kl_type else None
    mk, mkind = mask_arg(mask)
    tr, br = TOKEN_REDUCE[token_reduce], BATCH_REDUCE[batch_reduce]
    valid = _count_dev(valid_count, dev)
    one_pass = tr == 0 and br == 0
    row_scale = None
    if not one_pass:
        cnt, _, _ = row_stats(anchor, None, mk, rows, want_sum=False)
        row_scale = torch.empty(rows.n_rows, device=dev, dtype=torch.float32)
        prtc = _count_dev(per_row_token_count, dev, rows.n_rows, "per_row_token_count") if tr == 1 else None
        npt = _count_dev(num_program_tokens, dev, rows.n_rows, "num_program_tokens") if tr == 3 else None
        nps = _count_dev(num_program_steps, dev, rows.n_rows, "num_program_steps") if br == 2 else None
        check(
            lib.axon_loss_row_scale(ptr(cnt), None, rows.n_rows, rows.uniform_len if rows.uniform_len else 0, tr, br,
                                    ptr(prtc), ptr(npt), ptr(nps), ptr(valid), ptr(row_scale), None, stream_ptr()),
            "axon_loss_row_scale",
        )
    agg_w = torch.empty(rows.shape, device=dev, dtype=torch.float32) if ent is not None else None
    grad_kl = torch.empty(rows.shape, device=dev, dtype=torch.float32) if kl_type else None
    acc = _acc8(rows.n_slots, dev)
    check(
        lib.axon_side_terms(ptr(ent), ptr(lp), ptr(ref), ptr(mk), mkind, rows.cu_ptr, rows.n_rows, rows.n_slots,
                            rows.uniform_len, ptr(row_scale), 1.0, int(one_pass), ptr(valid if one_pass else None),
                            int(kl_type), int(kl_plus), ptr(agg_w), ptr(grad_kl), ptr(acc),
                            ptr(_partials(rows.n_slots, dev)), stream_ptr()),
        "axon_side_terms",
    )
    return acc, agg_w, grad_kl


# When set (benchmarks only), the LM-head autograd function routes through the timed entry points,
# which record HIP events around every launch into this timer without synchronising.
TIMING: "Timer | None" = None
# vocab chunk of the LM-head backward used when the caller passes 0 (0 = library default)
DEFAULT_VOCAB_CHUNK = 0

_PHASES = ("fwd/logits_stats", "fwd/merge", "fwd/label", "fwd/unused",
           "bwd/transpose", "bwd/dlogit", "bwd/dhidden", "bwd/dweight")


class Timer:
    """HIP-event timer on the current stream (``axon_timer_*``).  ``collect()`` synchronises the stream and
    returns ``{phase: {"ms": .., "launches": ..}}`` for everything recorded since the previous collect."""

    def __init__(self):
        self._lib = _lib.load()
        self.stream = stream_ptr()
        self.handle = self._lib.axon_timer_create(self.stream)
        if not self.handle:
            raise _lib.AxonAmdError("axon_timer_create failed")

    def collect(self) -> dict:
        import ctypes

        ms, cnt = (ctypes.c_float * 8)(), (ctypes.c_int32 * 8)()
        check(self._lib.axon_timer_collect(self.handle, ms, cnt), "axon_timer_collect")
        return {name: {"ms": float(ms[i]), "launches": int(cnt[i])} for i, name in enumerate(_PHASES) if cnt[i]}

    def close(self):
        if self.handle:
            self._lib.axon_timer_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def set_timing(timer: "Timer | None") -> None:
    global TIMING
    TIMING = timer


def seq_start_flags(cu_seqlens, n_tokens: int):
    """uint8 [N] (padded to a multiple of 4): 1 where a non-empty sequence begins."""
    lib = _lib.load()
    require_device(cu_seqlens, "seq_start_flags")
    cu = cu_seqlens.to(torch.int32).contiguous()
    flags = torch.empty((int(n_tokens) + 3) // 4 * 4, device=cu.device, dtype=torch.uint8)
    check(lib.axon_seq_start_flags(ptr(cu), int(cu.numel()) - 1, int(n_tokens), ptr(flags), stream_ptr()),
          "axon_seq_start_flags")
    return flags


def _head_operands(what, hidden, weight, labels, seq_start):
    """Shapes and types the head's kernels assume; returns (tokens, hidden size, vocabulary)."""
    if hidden.dim() != 2 or weight.dim() != 2 or hidden.shape[1] != weight.shape[1]:
        raise ValueError(f"{what}: hidden {tuple(hidden.shape)} and weight {tuple(weight.shape)} do not match")
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError(f"{what}: hidden and weight must be bf16")
    if labels.dtype not in (torch.int32, torch.int64):
        raise ValueError(f"{what}: labels must be int32 or int64")
    if not (hidden.is_contiguous() and weight.is_contiguous() and labels.is_contiguous()):
        raise ValueError(f"{what}: operands must be contiguous")
    if weight.device != hidden.device or labels.device != hidden.device:
        raise ValueError(f"{what}: operands live on different devices")
    n = int(hidden.shape[0])
    _same_len(what, n, labels=labels)
    if seq_start is not None and int(seq_start.numel()) < n:
        raise ValueError(f"{what}: seq_start has {int(seq_start.numel())} flags for {n} tokens")
    return n, int(hidden.shape[1]), int(weight.shape[0])


# Opt-in: the forward can leave a stash for its backward (2 bytes per logit: every softmax numerator as fp16
# relative to the maximum of its 128-row part of the vocabulary), from which the backward decodes the dlogits
# instead of recomputing the logits: 6 N H V flop per forward + backward instead of 8, for tokens x vocab x 2
# bytes held from forward to backward (10 GB at 32768 x 151936).  Off by default: like the reference's kernels,
# the default path never holds anything of size tokens x vocab.  ``LMHEAD_STASH``: False never; True whenever
# the shape allows it; "auto" when it is at most ``LMHEAD_STASH_MAX_BYTES`` and (outside stream capture) at
# most half of the free device memory.
LMHEAD_STASH = False
LMHEAD_STASH_MAX_BYTES = 64 << 30


def lmhead_stash_bytes(n: int, h: int, v: int) -> int:
    """Bytes of the forward's stash for this shape; 0 if the shape cannot be stashed."""
    return max(0, int(_lib.load().axon_lmhead_stash_bytes(int(n), int(h), int(v))))


def _want_stash(n, h, v, dev) -> int:
    """Bytes of the stash to allocate under the module's policy, or 0."""
    if LMHEAD_STASH is False or n == 0:
        return 0
    need = lmhead_stash_bytes(n, h, v)
    if need == 0 or LMHEAD_STASH is True:
        return need
    if need > LMHEAD_STASH_MAX_BYTES:
        return 0
    if not torch.cuda.is_current_stream_capturing():
        free, _total = torch.cuda.mem_get_info(dev)
        reusable = torch.cuda.memory_reserved(dev) - torch.cuda.memory_allocated(dev)
        if need > (free + reusable) // 2:
            return 0
    return need


def lmhead_forward(hidden, weight, labels, inv_temperature, timing: "Timer | None" = None, softcap: float = 0.0,
                   seq_start=None, stash: bool = False):
    """Returns logprobs, entropy, lse, entropy_b (all fp32 [N]), and with ``stash`` a fifth value: the uint8
    tensor that ``lmhead_backward(..., stash=)`` decodes the dlogits from (None when the module's policy,
    ``LMHEAD_STASH``, or the shape says no).  ``softcap`` > 0 soft-caps the logits
    (cap * tanh(logit / cap)) before the temperature.  With ``seq_start`` (``seq_start_flags``) ``labels`` is
    the packed id stream and logprobs / entropy come back aligned to token positions.

    With ``timing`` (a ``Timer``) the timed entry point is used: it records HIP events around every launch
    into the timer and does not synchronise."""
    lib = _lib.load()
    require_device(hidden, "lmhead_forward")
    n, h, v = _head_operands("lmhead_forward", hidden, weight, labels, seq_start)
    dev = hidden.device
    out = torch.empty(4, max(n, 1), device=dev, dtype=torch.float32)
    ws_bytes = lib.axon_lmhead_fwd_workspace_bytes(n, h, v)
    if ws_bytes < 0:
        raise _lib.AxonAmdError(f"axon_lmhead_fwd: unsupported shape tokens={n} hidden={h} vocab={v} (hidden % 32 != 0?)")
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    stash_bytes = _want_stash(n, h, v, dev) if stash else 0
    stash_t = torch.empty(stash_bytes, device=dev, dtype=torch.uint8) if stash_bytes else None
    args = (ptr(hidden), ptr(weight), ptr(labels), int(labels.dtype == torch.int64), n, h, v,
            float(inv_temperature), float(softcap), ptr(seq_start), ptr(out[0]), ptr(out[1]), ptr(out[2]), ptr(out[3]), ptr(ws), ws_bytes,
            ptr(stash_t), stash_bytes, stream_ptr())
    if timing is None:
        check(lib.axon_lmhead_fwd(*args), "axon_lmhead_fwd")
    else:
        check(lib.axon_lmhead_fwd_timed(*args, timing.handle), "axon_lmhead_fwd_timed")
    res = (out[0][:n], out[1][:n], out[2][:n], out[3][:n])
    return res + (stash_t,) if stash else res


# Opt-in: let the LM-head backward look for rows without an upstream gradient and leave them out.  Finding
# them costs a device-to-host readback (a host synchronisation per backward), which the reference's backward
# does not have, so the default backward never does it; a caller that knows its response mask hands it to
# ``packed_logprobs(..., response_mask=)`` instead, which keeps those rows out of forward and backward alike.
SKIP_ZERO_GRAD_ROWS = False
# With the search on, the backward runs over the active rows only when they are at most this share of all rows
# (below that the two row copies cost more than the skipped work saves).
SKIP_ROWS_BELOW = 0.97


def _active_rows(g_lp, g_en, seq_start, n):
    """(row_index, row_rank, number of rows whose upstream gradient is not zero); one readback."""
    lib = _lib.load()
    idx = torch.empty(2, n, device=g_lp.device, dtype=torch.int32)
    cnt = torch.empty(1, device=g_lp.device, dtype=torch.int32)
    check(lib.axon_lmhead_active_rows(ptr(g_lp), ptr(g_en), ptr(seq_start), n, ptr(idx[0]), ptr(idx[1]), ptr(cnt),
                                      stream_ptr()), "axon_lmhead_active_rows")
    return idx[0], idx[1], int(cnt.item())


def lmhead_backward(dlogprobs, dentropy, hidden, weight, labels, lse, entropy_b, inv_temperature, vocab_chunk=0,
                    timing: "Timer | None" = None, softcap: float = 0.0, seq_start=None, skip_zero_rows=None,
                    stash=None):
    """Returns d_hidden [N,H], d_weight [V,H] in bf16 (``timing`` as in ``lmhead_forward``).  By default the
    call only enqueues launches: no readback, no host synchronisation, and it can be captured into a HIP graph.

    ``stash``: what ``lmhead_forward(..., stash=True)`` returned for the same operands; the dlogits are then
    decoded from it and the logits are not recomputed.  (It describes all rows: a backward that leaves rows out
    ignores it and recomputes.)

    With ``skip_zero_rows`` (default: the module switch ``SKIP_ZERO_GRAD_ROWS``, off) the rows whose upstream
    gradients are both exactly zero (prompt positions, where the response mask is zero, rejected or clipped
    tokens) are left out of the three GEMMs: they contribute nothing to ``d_weight`` and their ``d_hidden`` rows
    are zero.  Finding them costs one readback, so it cannot be used while the stream is being captured."""
    vocab_chunk = vocab_chunk or DEFAULT_VOCAB_CHUNK
    if skip_zero_rows is None:
        skip_zero_rows = SKIP_ZERO_GRAD_ROWS
    lib = _lib.load()
    require_device(hidden, "lmhead_backward")
    n, h, v = _head_operands("lmhead_backward", hidden, weight, labels, seq_start)
    _same_len("lmhead_backward", n, dlogprobs=dlogprobs, dentropy=dentropy, lse=lse, entropy_b=entropy_b)
    dev = hidden.device
    if skip_zero_rows and torch.cuda.is_current_stream_capturing():
        raise _lib.AxonAmdError("lmhead_backward: skip_zero_rows reads a count back and cannot run under stream capture")
    if skip_zero_rows and n > 0 and h % 8 == 0:
        g_lp = f32(dlogprobs)
        g_en = f32(dentropy) if dentropy is not None else None
        row_index, row_rank, n_act = _active_rows(g_lp, g_en, seq_start, n)
        if n_act == 0:
            return torch.zeros_like(hidden), torch.zeros_like(weight)
        if n_act <= SKIP_ROWS_BELOW * n:
            hidden_c = torch.empty(n_act, h, device=dev, dtype=hidden.dtype)
            labels_c = torch.empty(n_act, device=dev, dtype=labels.dtype)
            f = torch.empty(4, n_act, device=dev, dtype=torch.float32)
            check(lib.axon_lmhead_gather_rows(ptr(hidden), ptr(labels), int(labels.dtype == torch.int64), ptr(lse),
                                              ptr(entropy_b), ptr(g_lp), ptr(g_en), ptr(seq_start), n, h,
                                              ptr(row_index), n_act, ptr(hidden_c), ptr(labels_c), ptr(f[0]),
                                              ptr(f[1]), ptr(f[2]), ptr(f[3] if g_en is not None else None),
                                              stream_ptr()), "axon_lmhead_gather_rows")
            dh_c, d_weight = lmhead_backward(f[2], f[3] if g_en is not None else None, hidden_c, weight, labels_c,
                                             f[0], f[1], inv_temperature, vocab_chunk, timing, softcap, None,
                                             skip_zero_rows=False)
            d_hidden = torch.empty_like(hidden)
            check(lib.axon_lmhead_scatter_rows(ptr(dh_c), ptr(row_rank), n, h, ptr(d_hidden), stream_ptr()),
                  "axon_lmhead_scatter_rows")
            return d_hidden, d_weight
    d_hidden = torch.empty_like(hidden)
    d_weight = torch.empty_like(weight)
    ws_bytes = lib.axon_lmhead_bwd_workspace_bytes(n, h, v, int(vocab_chunk))
    if ws_bytes < 0:
        raise _lib.AxonAmdError(f"axon_lmhead_bwd: unsupported shape/chunk tokens={n} hidden={h} vocab={v}")
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    g_lp = f32(dlogprobs)  # keep the converted copies alive until the launch is enqueued
    g_en = f32(dentropy) if dentropy is not None else None
    if stash is not None:
        if stash.dtype != torch.uint8 or stash.device != dev or not stash.is_contiguous():
            raise ValueError("lmhead_backward: stash must be the uint8 tensor lmhead_forward returned")
        if int(stash.numel()) != lmhead_stash_bytes(n, h, v) or int(stash.numel()) == 0:
            raise ValueError(f"lmhead_backward: a stash of {int(stash.numel())} bytes does not belong to a forward of "
                             f"tokens={n} hidden={h} vocab={v}")
    args = (ptr(g_lp), ptr(g_en), ptr(hidden), ptr(weight), ptr(labels), int(labels.dtype == torch.int64), ptr(lse),
            ptr(entropy_b), n, h, v, float(inv_temperature), float(softcap), ptr(seq_start), ptr(d_hidden), ptr(d_weight), int(vocab_chunk), ptr(ws),
            ws_bytes, ptr(stash), 0 if stash is None else int(stash.numel()), stream_ptr())
    if timing is None:
        check(lib.axon_lmhead_bwd(*args), "axon_lmhead_bwd")
    else:
        check(lib.axon_lmhead_bwd_timed(*args, timing.handle), "axon_lmhead_bwd_timed")
    return d_hidden, d_weight


DW_STORE, DW_FIRST, DW_ADD, DW_LAST = 0, 1, 2, 3


def head_block_groups(ranges, group):
    """Where the blocks of a step keep their dlogits when ``group`` consecutive blocks share one weight-gradient
    GEMM: per block ``(group index, first token of the block inside the group's workspace, is the group's last
    block)``, then the number of groups and the tokens the workspace must hold.  Inside a group every block
    begins on a multiple of 256 tokens (the blocks before it rounded up)."""
    place = []
    for k, (a, b) in enumerate(ranges):
        pos = 0
        if k % group:
            pa, pb = ranges[k - 1]
            pos = place[-1][1] + (pb - pa + 255) // 256 * 256
        place.append((k // group, pos, k % group == group - 1 or k == len(ranges) - 1))
    ws_tokens = max(pos + (b - a + 255) // 256 * 256 for (_, pos, _), (a, b) in zip(place, ranges))
    return place, place[-1][0] + 1, ws_tokens


class HeadBlocks:
    """One step of the head as blocks of consecutive tokens (``axon_lmhead_block_*``): forward of a block over
    the whole vocabulary with a stash, then (by the caller) the loss on the block's positions, then the block's
    backward from the stash, then the next block.  Holds the step's operands and everything the blocks share:
    the stash and the workspaces (sized for the largest block, allocated once), the transposed weight, the
    fp32 accumulator of the weight gradient, and the whole-stream outputs.

    ``hidden`` ``[N, H]`` and ``weight`` ``[V, H]`` bf16; ``labels`` ``[N]`` (with ``seq_start``: the packed id
    stream, outputs and gradients aligned to token positions, see ``lmhead_forward``).  ``ranges``: the hidden
    rows ``(first, end)`` of every block, in ascending order and covering all rows.  A block may begin before
    the previous one ends: the shared rows must reach the earlier block with a zero gradient (it then adds
    nothing for them), the later block writes their outputs and their ``d_hidden`` again.  ``vocab_chunk``: 0 =
    the backward of a block takes the whole vocabulary in one piece (no fp32 read-modify-write of the block's
    d_hidden; bf16 dlogits of block x vocab x 2 bytes), else a multiple of 256.  ``dw_group``: how many
    consecutive blocks share one weight-gradient GEMM (their dlogits stay in the workspace until the group's
    last block: a longer reduction and fewer passes over the fp32 partial sums for ``dw_group`` x the dlogit
    memory); 1 where the shape does not allow it (``axon_lmhead_block_can_group``)."""

    def __init__(self, hidden, weight, labels, inv_temperature, ranges, *, softcap=0.0, seq_start=None,
                 vocab_chunk=0, stash=True, dw_group=2, timing: "Timer | None" = None):
        self.lib = _lib.load()
        require_device(hidden, "HeadBlocks")
        self.n, self.h, self.v = _head_operands("HeadBlocks", hidden, weight, labels, seq_start)
        self.ranges = [(int(a), int(b)) for a, b in ranges]
        ok = bool(self.ranges) and self.ranges[0][0] == 0 and self.ranges[-1][1] == self.n
        ok = ok and all(a < b for a, b in self.ranges)
        ok = ok and all(a1 < a2 <= b1 <= b2 for (a1, b1), (a2, b2) in zip(self.ranges, self.ranges[1:]))
        if not ok:
            raise ValueError(f"HeadBlocks: row ranges {self.ranges} do not cover {self.n} rows in ascending order")
        self.hidden, self.weight, self.labels, self.seq_start = hidden, weight, labels, seq_start
        self.inv_t, self.softcap, self.timing = float(inv_temperature), float(softcap), timing
        dev = hidden.device
        n_max = max(b - a for a, b in self.ranges)
        self.chunk = int(vocab_chunk) if vocab_chunk else (self.v + 255) // 256 * 256
        # groups of consecutive blocks that share a weight-gradient GEMM: (group, position in the workspace, last?)
        g = max(int(dw_group), 1)
        if g > 1 and not self.lib.axon_lmhead_block_can_group(self.h, self.v, self.chunk):
            g = 1
        self.dw_group = g
        self.place, self.n_groups, self.ws_tokens = head_block_groups(self.ranges, g)
        self.fwd_ws_bytes = self.lib.axon_lmhead_fwd_workspace_bytes(n_max, self.h, self.v)
        self.bwd_ws_bytes = self.lib.axon_lmhead_bwd_workspace_bytes(self.ws_tokens, self.h, self.v, self.chunk)
        if self.fwd_ws_bytes < 0 or self.bwd_ws_bytes < 0:
            raise _lib.AxonAmdError(f"HeadBlocks: unsupported shape tokens={n_max} hidden={self.h} vocab={self.v}")
        self.fwd_ws = torch.empty(self.fwd_ws_bytes, device=dev, dtype=torch.uint8)
        self.bwd_ws = torch.empty(self.bwd_ws_bytes, device=dev, dtype=torch.uint8)
        self.stash_bytes = max(lmhead_stash_bytes(b - a, self.h, self.v) for a, b in self.ranges) if stash else 0
        self.stash = torch.empty(self.stash_bytes, device=dev, dtype=torch.uint8) if self.stash_bytes else None
        self.stats = torch.empty(2, n_max, device=dev, dtype=torch.float32)  # lse, entropy_b of the current block
        # whole-stream outputs; position 0 is a sequence start (the aligned layout writes it from the last row)
        self.out = torch.zeros(2, max(self.n, 1), device=dev, dtype=torch.float32)
        self.d_hidden = torch.empty_like(hidden)
        self.d_weight = torch.empty_like(weight)
        self.one_block = self.n_groups == 1  # one weight-gradient GEMM: no partial sums to carry
        self.dw_acc_bytes = 0 if self.one_block else int(self.lib.axon_lmhead_block_dw_acc_bytes(self.h, self.v))
        self.dw_acc = torch.empty(self.dw_acc_bytes // 4, device=dev, dtype=torch.float32) if self.dw_acc_bytes else None
        self.wt_ready = False
        self.block_stash_bytes = 0
        self.workspace_bytes = self.fwd_ws_bytes + self.bwd_ws_bytes + self.stash_bytes + self.dw_acc_bytes

    @property
    def logprobs(self):
        return self.out[0][: self.n]

    @property
    def entropy(self):
        return self.out[1][: self.n]

    def _block(self, k):
        n0, n1 = self.ranges[k]
        last_dst = 0 if self.seq_start is None else (n1 - n0 if n1 < self.n else -n0)
        return n0, n1, last_dst

    def _at(self, t, n0):
        """Pointer to element ``n0`` of a whole-stream array (None stays None)."""
        return None if t is None else t.data_ptr() + n0 * t.element_size()

    def forward(self, k):
        """Forward of block ``k``: its positions of ``logprobs`` / ``entropy`` (with ``seq_start``: positions
        ``first + 1 .. end`` of its rows, the stream's last row goes to position 0) are valid once the
        stream reaches the point after the call."""
        n0, n1, last_dst = self._block(k)
        nb = n1 - n0
        self.block_stash_bytes = lmhead_stash_bytes(nb, self.h, self.v) if self.stash is not None else 0
        check(self.lib.axon_lmhead_block_fwd(
            self.hidden.data_ptr() + n0 * self.h * 2, ptr(self.weight), self._at(self.labels, n0),
            int(self.labels.dtype == torch.int64), nb, self.h, self.v, self.inv_t, self.softcap,
            self._at(self.seq_start, n0), last_dst, self._at(self.out[0], n0), self._at(self.out[1], n0),
            ptr(self.stats[0]), ptr(self.stats[1]), ptr(self.fwd_ws), self.fwd_ws_bytes,
            ptr(self.stash) if self.block_stash_bytes else None, self.block_stash_bytes, stream_ptr(),
            self.timing.handle if self.timing else None), "axon_lmhead_block_fwd")

    def backward(self, k, dlogprobs, dentropy):
        """Backward of block ``k`` (after its ``forward``; no other block's forward in between).  ``dlogprobs`` /
        ``dentropy`` (fp32, ``dentropy`` may be None): whole-stream arrays, read at the block's positions."""
        n0, n1, last_dst = self._block(k)
        nb = n1 - n0
        if dlogprobs.dtype != torch.float32 or int(dlogprobs.numel()) < self.n or not dlogprobs.is_contiguous():
            raise ValueError("HeadBlocks.backward: dlogprobs must be a contiguous fp32 array over the whole stream")
        if dentropy is not None and (dentropy.dtype != torch.float32 or int(dentropy.numel()) < self.n
                                     or not dentropy.is_contiguous()):
            raise ValueError("HeadBlocks.backward: dentropy must be a contiguous fp32 array over the whole stream")
        st = stream_ptr()
        th = self.timing.handle if self.timing else None
        if not self.wt_ready:
            check(self.lib.axon_lmhead_block_begin(ptr(self.weight), self.h, self.v, self.chunk, ptr(self.bwd_ws),
                                                   self.bwd_ws_bytes, st, th), "axon_lmhead_block_begin")
            self.wt_ready = True
        group, pos, dw_now = self.place[k]
        mode = (DW_STORE if self.one_block else DW_FIRST if group == 0
                else DW_LAST if group == self.n_groups - 1 else DW_ADD)
        check(self.lib.axon_lmhead_block_bwd(
            self._at(dlogprobs, n0), self._at(dentropy, n0), self.hidden.data_ptr() + n0 * self.h * 2,
            ptr(self.weight), self._at(self.labels, n0), int(self.labels.dtype == torch.int64),
            ptr(self.stats[0]), ptr(self.stats[1]), nb, self.h, self.v, self.inv_t, self.softcap,
            self._at(self.seq_start, n0), last_dst, self.d_hidden.data_ptr() + n0 * self.h * 2,
            ptr(self.d_weight), ptr(self.dw_acc), mode, 1, pos, int(dw_now), self.ws_tokens, self.chunk,
            ptr(self.bwd_ws), self.bwd_ws_bytes,
            ptr(self.stash) if self.block_stash_bytes else None, self.block_stash_bytes, st, th),
            "axon_lmhead_block_bwd")


def scale_f32(x, s1, s2=None):
    """``x * s1 * s2`` for an fp32 array and one or two device scalars (0-d or 1-element fp32 tensors), in one
    launch; a new tensor shaped like ``x``."""
    lib = _lib.load()
    require_device(x, "scale_f32")
    xf = f32(x)

    def scalar(t):
        t = t.detach()
        if t.dtype != torch.float32 or t.device != xf.device:
            t = t.to(device=xf.device, dtype=torch.float32)
        return t

    a = scalar(s1)
    b = scalar(s2) if s2 is not None else None
    out = torch.empty_like(xf)
    check(lib.axon_scale_f32(ptr(xf), ptr(a), ptr(b), ptr(out), int(xf.numel()), stream_ptr()), "axon_scale_f32")
    return out.view(x.shape)


def scale_bf16_unless_one(x, scale):
    """``x *= scale`` in place (bf16 ``x``, ``scale`` a device scalar); no memory traffic when it is exactly 1."""
    lib = _lib.load()
    require_device(x, "scale_bf16_unless_one")
    if x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("scale_bf16_unless_one: x must be contiguous bf16")
    s = scale.detach().to(device=x.device, dtype=torch.float32).reshape(-1)[:1].contiguous()
    check(lib.axon_scale_bf16_unless_one(ptr(x), int(x.numel()), ptr(s), stream_ptr()), "axon_scale_bf16_unless_one")
    return x


_LOGITS_DTYPES = {torch.float32: 0, torch.bfloat16: 1}


def _logits_operands(what, logits, labels):
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise ValueError(f"{what}: logits must be [tokens, vocab] with unit stride over the vocabulary")
    if logits.dtype not in _LOGITS_DTYPES:
        raise ValueError(f"{what}: logits must be fp32 or bf16, got {logits.dtype}")
    n, v = int(logits.shape[0]), int(logits.shape[1])
    if labels is not None:
        if labels.dtype not in (torch.int32, torch.int64) or not labels.is_contiguous():
            raise ValueError(f"{what}: labels must be contiguous int32 or int64")
        if labels.device != logits.device:
            raise ValueError(f"{what}: operands live on different devices")
        _same_len(what, n, labels=labels)
    return n, v, int(logits.stride(0)) if n > 1 else v


def logits_forward(logits, labels=None, want_entropy=True):
    """``(logprob | None, entropy | None, lse)`` fp32 [tokens] from materialised logits; see axon_logits_fwd."""
    lib = _lib.load()
    require_device(logits, "logits_forward")
    n, v, ld = _logits_operands("logits_forward", logits, labels)
    dev = logits.device
    out = torch.empty(3, max(n, 1), device=dev, dtype=torch.float32)
    check(
        lib.axon_logits_fwd(ptr(logits), _LOGITS_DTYPES[logits.dtype], ld, n, v, ptr(labels),
                            int(labels is not None and labels.dtype == torch.int64),
                            ptr(out[0]) if labels is not None else None, ptr(out[1]) if want_entropy else None,
                            ptr(out[2]), stream_ptr()),
        "axon_logits_fwd",
    )
    return (out[0][:n] if labels is not None else None), (out[1][:n] if want_entropy else None), out[2][:n]


def logits_backward(logits, labels, lse, entropy, g_logprob, g_entropy, inplace=False):
    """d loss / d logits in the logits' dtype (written over the logits when ``inplace``); see axon_logits_bwd."""
    lib = _lib.load()
    require_device(logits, "logits_backward")
    n, v, ld = _logits_operands("logits_backward", logits, labels)
    g_lp = f32(g_logprob) if g_logprob is not None else None
    g_en = f32(g_entropy) if g_entropy is not None else None
    _same_len("logits_backward", n, lse=lse, entropy=entropy, g_logprob=g_lp, g_entropy=g_en)
    out = logits if inplace else torch.empty_like(logits, memory_format=torch.contiguous_format)
    ld_d = int(out.stride(0)) if n > 1 else v
    check(
        lib.axon_logits_bwd(ptr(logits), _LOGITS_DTYPES[logits.dtype], ld, n, v, ptr(labels),
                            int(labels is not None and labels.dtype == torch.int64), ptr(lse), ptr(entropy),
                            ptr(g_lp), ptr(g_en), ptr(out), ld_d, stream_ptr()),
        "axon_logits_bwd",
    )
    return out


def gemm_nt(a, b):
    """out[n][m] = sum_k a[m][k] * b[n][k]; bf16 in, fp32 out.  Test/benchmark helper."""
    lib = _lib.load()
    require_device(a, "gemm_nt")
    m, k = a.shape
    n = b.shape[0]
    out = torch.empty(n, m, device=a.device, dtype=torch.float32)
    check(lib.axon_gemm_nt_bf16(ptr(a), a.stride(0), ptr(b), b.stride(0), ptr(out), m, m, n, k, stream_ptr()),
          "axon_gemm_nt_bf16")
    return out


def gemm_layouts(a, b, a_kmajor=False, b_kmajor=False):
    """out[n][m] = sum_k A[m][k] * B[n][k] with `a` given as [m][k], or as [k][m] when a_kmajor (likewise b):
    a K-major operand is read as it lies.  bf16 in, fp32 out.  Test/benchmark helper."""
    lib = _lib.load()
    require_device(a, "gemm_layouts")
    k, m = (a.shape if a_kmajor else a.shape[::-1])
    n = b.shape[1] if b_kmajor else b.shape[0]
    if (b.shape[0] if b_kmajor else b.shape[1]) != k:
        raise ValueError("gemm_layouts: reduction lengths differ")
    out = torch.empty(n, m, device=a.device, dtype=torch.float32)
    check(lib.axon_gemm_bf16(ptr(a), a.stride(0), int(a_kmajor), ptr(b), b.stride(0), int(b_kmajor), ptr(out), m,
                             m, n, k, stream_ptr()), "axon_gemm_bf16")
    return out
