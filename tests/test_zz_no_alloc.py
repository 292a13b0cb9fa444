"""axon_policy_loss_noalloc (the entry point that allocates nothing) against axon_policy_loss.

Both are called through the C ABI on the same inputs; loss, metric sums and the gradient must agree bit for
bit (same kernels, same reduction order).  Two calls in a row, the second on a smaller input, so that what
the first call left in the library's fixed scratch array is there when the second runs."""

import ctypes

import pytest
import torch

from axon_amd import _lib
from axon_amd import workloads as W

pytestmark = pytest.mark.gpu


def _call(fn_name, kind, rl, *, row_scale, row_mean, post_normalize, with_partials):
    lib = _lib.load()
    dev = rl["log_probs"].device
    n = int(rl["log_probs"].numel())
    cu = rl["cu_seqlens"]
    grad = torch.full((n,), float("nan"), device=dev)
    acc = torch.full((8,), float("nan"), device=dev)
    args = [kind, rl["log_probs"].data_ptr(), rl["old_log_probs"].data_ptr(), rl["advantages"].data_ptr(),
            rl["response_mask"].data_ptr(), _lib.MASK_F32, None, cu.data_ptr(), int(cu.numel()) - 1, n, 0,
            None if row_scale is None else row_scale.data_ptr(), None if row_mean is None else row_mean.data_ptr(),
            1.0, post_normalize, None, 0.8, 1.28, 3.0, grad.data_ptr(), acc.data_ptr()]
    keep = None
    if with_partials:
        keep = torch.zeros(lib.axon_reduce_partials_bytes(n) // 4, device=dev)  # the ticket counter starts at zero
        args.append(keep.data_ptr())
    args.append(torch.cuda.current_stream().cuda_stream)
    rc = getattr(lib, fn_name)(*args)
    assert rc == 0, (fn_name, rc, lib.axon_amd_error_string(rc))
    torch.cuda.synchronize()
    return grad, acc


def _inputs(n_tokens, seed, dev):
    rl = W.packed_rl_inputs(n_tokens, seed=seed)
    rl = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in rl.items()}
    g = torch.Generator().manual_seed(seed + 100)
    old = -torch.empty(n_tokens).exponential_(1.0, generator=g)
    rl["old_log_probs"] = old.to(dev)
    rl["log_probs"] = (old + 0.3 * torch.randn(n_tokens, generator=g)).to(dev)
    rl["advantages"] = torch.randn(n_tokens, generator=g).to(dev)
    return rl


@pytest.mark.parametrize("kind", [0, 1])
def test_noalloc_matches_policy_loss_on_two_calls_in_a_row(kind):
    dev = torch.device("cuda:0")
    for n_tokens, seed in ((300_000, 3), (5_000, 4)):  # the second call is the smaller one
        rl = _inputs(n_tokens, seed, dev)
        n_rows = int(rl["cu_seqlens"].numel()) - 1
        row_scale = row_mean = None
        post = 1
        if kind == 1:  # GSPO reads a per-row scale and the per-row mean log-ratio
            g = torch.Generator().manual_seed(seed + 200)
            row_scale = (torch.rand(n_rows, generator=g) * 1e-3).to(dev)
            row_mean = (0.01 * torch.randn(n_rows, generator=g)).to(dev)
            post = 0
        kw = dict(row_scale=row_scale, row_mean=row_mean, post_normalize=post)
        g_ref, a_ref = _call("axon_policy_loss", kind, rl, with_partials=True, **kw)
        g_new, a_new = _call("axon_policy_loss_noalloc", kind, rl, with_partials=False, **kw)
        assert torch.isfinite(a_ref[:6]).all() and torch.isfinite(g_ref).all()
        assert torch.equal(g_new, g_ref), f"gradient differs at {n_tokens} tokens"
        assert torch.equal(a_new[:6], a_ref[:6]), (a_new, a_ref)


def test_noalloc_rejects_inputs_beyond_its_capacity():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    t = torch.zeros(8, device=dev)
    n = (1 << 24) + 1  # the size is rejected before any pointer is read, so small buffers are enough
    rc = lib.axon_policy_loss_noalloc(0, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), _lib.MASK_F32, None,
                                      None, 1, n, n, None, None, 1.0, 1, None, 0.8, 1.28, 3.0, t.data_ptr(),
                                      t.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == -6
    assert b"capacity" in lib.axon_amd_error_string(rc)
    torch.cuda.synchronize()
