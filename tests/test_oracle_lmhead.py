"""Pins oracle/lmhead_ce.py against torch.nn.functional.cross_entropy + autograd (the textbook the
reference's Liger kernel implements, gguf_liger_loss.py:140-170) and against its own invariants."""

import torch

from oracle import lmhead_ce as ce


def _case(seed, rows=37, hid=32, vocab=53, ignored=(3, 11, 36)):
    gen = torch.Generator().manual_seed(seed)
    h = torch.randn(rows, hid, generator=gen).to(torch.bfloat16)
    w = (torch.randn(vocab, hid, generator=gen) * 0.3).to(torch.bfloat16).double()
    y = torch.randint(0, vocab, (rows,), generator=gen)
    for i in ignored:
        y[i] = -100
    return h, w, y


def test_matches_functional_cross_entropy_and_autograd():
    h, w, y = _case(1)
    for reduction in ("mean", "sum"):
        hr = h.double().clone().requires_grad_(True)
        exact = hr @ w.T
        # the path's logits are bf16 values (the reference's mmq returns bf16, gguf_liger_loss.py:109-114);
        # straight-through rounding keeps autograd on the textbook formula
        logits = exact + (ce.bf16_round64(exact.detach()) - exact.detach())
        want = torch.nn.functional.cross_entropy(logits, y, ignore_index=-100, reduction=reduction)
        want.backward()
        loss, dh, loss_1d, lse = ce.linear_cross_entropy(h, w, y, reduction=reduction, chunk=16)
        assert abs(float(loss) - float(want.detach())) <= 1e-9 * max(1.0, abs(float(want.detach())))
        # the logit gradient is rounded to bf16 before the second GEMM (gguf_liger_loss.py:172-177)
        assert float((dh - hr.grad).abs().max()) <= 2.0 ** -7 * float(hr.grad.abs().max())
        assert torch.allclose(lse, torch.logsumexp(logits.detach(), dim=1), atol=1e-12)
        # and the rounding of the logits moves the loss by far less than the path's 2e-2 tolerance class
        unrounded = torch.nn.functional.cross_entropy(exact.detach(), y, ignore_index=-100, reduction="mean")
        mean_loss = float(loss) if reduction == "mean" else float(loss) / int((y != -100).sum())
        assert abs(mean_loss - float(unrounded)) <= 5e-3
        assert not loss_1d[y == -100].any() and not dh[y == -100].any()


def test_sum_is_mean_times_count_and_chunking_is_invisible():
    h, w, y = _case(2)
    n = int((y != -100).sum())
    mean = ce.linear_cross_entropy(h, w, y, reduction="mean", chunk=1024)
    total = ce.linear_cross_entropy(h, w, y, reduction="sum", chunk=1024)
    assert abs(float(total[0]) - n * float(mean[0])) < 1e-9
    for chunk in (1, 7, 37, 64):
        other = ce.linear_cross_entropy(h, w, y, reduction="mean", chunk=chunk)
        for a, b in zip(mean, other):
            assert torch.equal(a, b)


def test_all_rows_ignored_gives_zero_loss_and_gradient():
    h, w, y = _case(3)
    y[:] = -100
    loss, dh, loss_1d, _ = ce.linear_cross_entropy(h, w, y)
    assert float(loss) == 0.0 and not dh.any() and not loss_1d.any()


def test_uniform_logits_closed_form():
    """Zero hidden state: every logit is 0, lse = log V, loss = log V, dlogit = 1/V - onehot."""
    rows, hid, vocab = 4, 8, 16
    h = torch.zeros(rows, hid, dtype=torch.bfloat16)
    w = torch.ones(vocab, hid, dtype=torch.float64)
    y = torch.tensor([0, 5, 15, 7])
    loss, dh, loss_1d, lse = ce.linear_cross_entropy(h, w, y, reduction="sum")
    assert torch.allclose(lse, torch.full((rows,), 16.0, dtype=torch.float64).log())
    assert torch.allclose(loss_1d, lse)
    # sum over vocab of (1/V - onehot) is 0, and every weight row is the same: dh = 0
    assert float(dh.abs().max()) < 1e-6


def test_predicted_tokens_first_maximum_and_accuracy():
    # distinct logits: torch.argmax; tied logits: a brute-force scan that keeps the first maximum
    g = torch.Generator().manual_seed(11)
    hid = torch.randn(9, 16, generator=g).to(torch.bfloat16)
    w = torch.randn(40, 16, generator=g).to(torch.bfloat16).double()
    labels = torch.randint(0, 40, (9,), generator=g)
    labels[2] = -100
    logits = ce.bf16_round64(hid.double() @ w.T)
    pred, acc = ce.predicted_tokens(hid, w, labels, -100, chunk=4)
    for r in range(9):
        best, arg = None, -1
        for c in range(40):
            if best is None or float(logits[r, c]) > best:
                best, arg = float(logits[r, c]), c
        assert int(pred[r]) == (-1 if r == 2 else arg)
    counted = [r for r in range(9) if r != 2]
    assert abs(acc - sum(int(pred[r]) == int(labels[r]) for r in counted) / len(counted)) < 1e-12
    hid[:] = 0  # every logit equal: the first column
    pred, acc = ce.predicted_tokens(hid, w, labels, -100)
    assert pred.tolist() == [0, 0, -1, 0, 0, 0, 0, 0, 0]
    assert ce.predicted_tokens(hid, w, torch.full((9,), -100), -100)[1] == 0.0
