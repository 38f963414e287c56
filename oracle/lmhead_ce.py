"""CPU oracle for the chunked lm_head cross-entropy over a packed head.

TEST INFRASTRUCTURE (see oracle/__init__.py).  Restates gguf_liger_loss.py:38-186: per row chunk,
logits = hidden @ W^T rounded to bf16 (:109-114), an fp32 softmax cross-entropy that turns the
logits into d(loss)/d(logits) rounded to bf16 (:140-170; Liger's kernel: lse = m + log(sum exp(x-m)),
loss = lse - x[y], gradient softmax - onehot, both divided by the number of non-ignored targets for
reduction "mean"; ignored rows give zero loss and zero gradient), then dHidden = dlogits @ W
(:172-177) and loss = sum of the per-row losses (:179).  Chunking does not change any value.
``n_non_ignore == 0`` divides by zero in the reference (:87,154); defined here as loss 0, grad 0.

The textbook identity pins it: tests/test_oracle_lmhead.py compares with
``torch.nn.functional.cross_entropy(..., ignore_index, reduction)`` and its autograd.
"""

from __future__ import annotations

import torch


def bf16_round64(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float64)


def linear_cross_entropy(hidden, w, labels, ignore_index=-100, reduction="mean", chunk=1024):
    """hidden bf16 [rows,H]; w float64 [V,H] holding bf16 values; labels int64 [rows].
    Returns (loss float64 scalar, dhidden float64 [rows,H] before the final bf16 store,
    loss_1d float64 [rows], lse float64 [rows])."""
    rows = hidden.shape[0]
    valid = labels != ignore_index
    n = int(valid.sum())
    scale = 0.0 if n == 0 else (1.0 / n if reduction == "mean" else 1.0)
    loss_1d = torch.zeros(rows, dtype=torch.float64)
    lse_all = torch.zeros(rows, dtype=torch.float64)
    dh = torch.zeros(rows, hidden.shape[1], dtype=torch.float64)
    for r0 in range(0, rows, chunk):
        r1 = min(r0 + chunk, rows)
        logits = bf16_round64(hidden[r0:r1].to(torch.float64) @ w.T)
        lse = torch.logsumexp(logits, dim=1)
        lse_all[r0:r1] = lse
        p = torch.exp(logits - lse[:, None])
        v = valid[r0:r1]
        y = labels[r0:r1].clamp(min=0)
        p[torch.arange(r1 - r0), y] -= v.to(torch.float64)
        p = bf16_round64(p * scale * v[:, None].to(torch.float64))
        xy = logits[torch.arange(r1 - r0), y]
        loss_1d[r0:r1] = (lse - xy) * scale * v.to(torch.float64)
        dh[r0:r1] = p @ w
    return loss_1d.sum(), dh, loss_1d, lse_all


def predicted_tokens(hidden, w, labels, ignore_index=-100, chunk=1024):
    """Liger's RETURN_PREDICTED_TOKENS / RETURN_TOKEN_ACCURACY outputs as the reference's loop collects them
    (gguf_liger_loss.py:92-101, 117-185): per row the argmax of the bf16 logits, the FIRST maximum (the kernel scans the
    vocabulary in ascending blocks and takes a later block only for a strictly larger maximum), -1 on ignored rows;
    accuracy = rows whose argmax is the label / rows that count (0 when none does, where the reference divides by zero).
    Returns (predicted int64 [rows], accuracy float)."""
    rows = hidden.shape[0]
    valid = labels != ignore_index
    pred = torch.full((rows,), -1, dtype=torch.int64)
    for r0 in range(0, rows, chunk):
        r1 = min(r0 + chunk, rows)
        logits = bf16_round64(hidden[r0:r1].to(torch.float64) @ w.T)
        best = logits.max(dim=1, keepdim=True).values
        first = torch.where(logits == best, torch.arange(logits.shape[1])[None, :], logits.shape[1]).min(dim=1).values
        pred[r0:r1] = torch.where(valid[r0:r1], first, torch.full_like(first, -1))
    n = int(valid.sum())
    acc = float(((pred == labels) & valid).sum()) / n if n else 0.0
    return pred, acc
