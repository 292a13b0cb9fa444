"""An independent reference of the fused head for the full-size GPU tests: plain fp32 torch on the GPU
(library matmul, logsumexp, softmax; nothing of the HIP kernels)."""

import torch


def _fp32_torch_head_reference(hd, wd, ld, g_lp, g_en, rows, token_block=2048):
    """The head in plain fp32 torch on the GPU, block of tokens by block of tokens (library matmul,
    logsumexp, softmax: nothing of the HIP kernels): log-prob and entropy of every token, and d_weight for
    the vocabulary rows ``rows`` under upstream gradients ``g_lp`` (log-prob) and ``g_en`` (entropy),
    dlogit = g_lp (onehot - p) - g_en p (logit - sum p logit), d_weight[r] = sum_n dlogit[n, r] hidden[n]."""
    n = hd.shape[0]
    w32 = wd.float()
    lp = torch.empty(n, device=hd.device)
    ent = torch.empty(n, device=hd.device)
    dw_rows = torch.zeros(len(rows), hd.shape[1], device=hd.device, dtype=torch.float64)
    rows_d = rows.to(hd.device)
    for a in range(0, n, token_block):
        b = min(a + token_block, n)
        h32 = hd[a:b].float()
        logits = h32 @ w32.t()
        lse = torch.logsumexp(logits, -1)
        p = torch.softmax(logits, -1)
        eb = (p * logits).sum(-1)
        lab = ld[a:b].long()
        lp[a:b] = logits.gather(1, lab[:, None])[:, 0] - lse
        ent[a:b] = lse - eb
        pr = p[:, rows_d]
        dl = -g_lp[a:b, None] * pr + g_lp[a:b, None] * (lab[:, None] == rows_d[None, :]).float()
        if g_en is not None:
            dl = dl - g_en[a:b, None] * pr * (logits[:, rows_d] - eb[:, None])
        dw_rows += (dl.t().double() @ h32.double())
        del logits, p
    return lp, ent, dw_rows


def _spread_rows(v, chunk=32768):
    """Vocabulary rows spread over every chunk of the backward, with the edges of the chunks and of the last
    (partial) 256-row tile among them."""
    rows = set(range(0, v, 1571)) | {0, 255, 256, v - 1, v - 2, v - 128, v - 129, v - 256, v - 257}
    for c in range(chunk, v, chunk):
        rows |= {c - 1, c, c + 255, c + 256}
    return torch.tensor(sorted(r for r in rows if 0 <= r < v))
