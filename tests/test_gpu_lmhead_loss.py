"""Chunked packed lm_head cross-entropy against the oracle (relations of test_gguf_liger_loss.py:80-156
and test_deepseek_v4_liger_loss.py:41-134)."""

import pytest
import torch

from helpers import assert_close_bf16, bf16_randn, make_payload
from oracle import gguf_blocks as gb
from oracle import lmhead_ce as ref
from oracle import lora_matmul as mm

pytestmark = pytest.mark.gpu


def _case(seed, rows, hidden, vocab, qt, ignore_frac=0.05):
    gen = torch.Generator().manual_seed(seed)
    payload = make_payload(seed, qt, vocab, hidden)
    hid = bf16_randn(gen, rows, hidden)
    labels = torch.randint(0, vocab, (rows,), generator=gen)
    labels[torch.rand(rows, generator=gen) < ignore_frac] = -100
    return payload, hid, labels


@pytest.mark.parametrize("qt,rows,hidden,vocab,chunk,reduction", [
    (gb.Q6_K, 257, 2048, 37, 256, "mean"),      # the reference's test geometry: chunk + 1 rows, 37-row head
    (gb.Q6_K, 300, 512, 9000, 128, "mean"),     # more than one vocabulary block, ragged last tile
    (gb.Q8_0, 130, 256, 1000, 64, "sum"),
    (gb.Q4_K, 64, 512, 8192 + 300, 1024, "mean"),
])
def test_packed_loss_matches_oracle(pkg, dev, qt, rows, hidden, vocab, chunk, reduction):
    payload, hid, labels = _case(12345, rows, hidden, vocab, qt)
    want_loss, want_dh, want_l1, want_lse = ref.linear_cross_entropy(hid, mm.weights_bf16(payload, qt), labels, -100, reduction, chunk)
    h = hid.to(dev).requires_grad_(True)
    loss = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, chunk, -100, reduction)
    loss.backward()
    scale = 1.0 if reduction == "mean" else 1.0 / max(1, int((labels != -100).sum()))
    assert abs(float(loss) - float(want_loss)) * scale <= 1e-3, (float(loss), float(want_loss))
    assert_close_bf16(h.grad, want_dh, "dHidden", ulps=4)
    cos = torch.nn.functional.cosine_similarity(h.grad.double().cpu().reshape(-1), want_dh.reshape(-1), dim=0)
    assert float(cos) > 0.9999
    assert bool((h.grad[(labels == -100).to(dev)] == 0).all()), "ignored rows must get zero gradient"


def test_loss_internals_and_upstream_scale(pkg, dev):
    qt, rows, hidden, vocab = gb.Q6_K, 96, 256, 700
    payload, hid, labels = _case(777, rows, hidden, vocab, qt, ignore_frac=0.2)
    _, want_dh, want_l1, want_lse = ref.linear_cross_entropy(hid, mm.weights_bf16(payload, qt), labels, -100, "mean", 32)
    loss, grad, l1, lse, status, _, _ = pkg.gguf_liger_loss._packed_linear_cross_entropy_forward(
        hid.to(dev), torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, 32, -100, "mean")
    assert int(status[0]) == int((labels != -100).sum()) and int(status[1]) == 0
    assert float((lse.double().cpu() - want_lse).abs().max()) < 2e-3
    assert float((l1.double().cpu() - want_l1).abs().max()) < 1e-4
    h = hid.to(dev).requires_grad_(True)
    out = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, 32)
    (out * 3.0).backward()
    assert_close_bf16(h.grad, 3.0 * want_dh, "scaled dHidden", ulps=6)


def test_all_rows_ignored_gives_zero_loss_and_gradient(pkg, dev):
    qt, rows, hidden, vocab = gb.Q8_0, 20, 256, 50
    payload, hid, _ = _case(1, rows, hidden, vocab, qt)
    labels = torch.full((rows,), -100)
    h = hid.to(dev).requires_grad_(True)
    loss = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, 8)
    loss.backward()
    assert float(loss) == 0.0 and torch.count_nonzero(h.grad) == 0


def test_causal_lm_wrapper_and_guards(pkg, dev):
    L, fl, G = pkg.gguf_liger_loss, pkg.fast_lora, pkg.gguf.GGUFQuantizedTensor
    qt, hidden, vocab = gb.Q6_K, 256, 300
    payload, hid, _ = _case(5, 2 * 9, hidden, vocab, qt)
    head = fl.GGUFLinear(hidden, vocab, G(torch.from_numpy(payload).to(dev), qt, (vocab, hidden)))
    gen = torch.Generator().manual_seed(3)
    labels = torch.randint(0, vocab, (2, 9), generator=gen)
    hs = hid.reshape(2, 9, hidden).to(dev).requires_grad_(True)
    loss = L._packed_for_causal_lm_loss(hs, head, labels.to(dev), hidden)
    shifted = torch.nn.functional.pad(labels, (0, 1), value=-100)[..., 1:].reshape(-1)
    want, want_dh, _, _ = ref.linear_cross_entropy(hid, mm.weights_bf16(payload, qt), shifted, -100, "mean", 256)
    assert abs(float(loss) - float(want)) <= 1e-3
    loss_sum = L._packed_for_causal_lm_loss(hs, head, labels.to(dev), hidden, num_items_in_batch=16)
    assert abs(float(loss_sum) - float(want) * int((shifted != -100).sum()) / 16) <= 1e-3
    out4 = L._packed_for_causal_lm_loss(hs, head, labels.to(dev), hidden, return_token_accuracy=True)
    assert len(out4) == 4 and out4[1] is None and out4[3] is None and 0.0 <= float(out4[2]) <= 1.0  # (loss, z_loss, accuracy, tokens)
    assert abs(float(out4[0]) - float(want)) <= 1e-3
    for bad in ({"return_z_loss": True}, {"ce_weight": torch.ones(3)}, {"label_smoothing": 0.1}, {"lse_square_scale": 1e-4},
                {"final_logit_softcapping": 30.0}, {"use_token_scaling": True}, {"bias": torch.ones(1)}, {"accum_dtype": torch.float16}):
        with pytest.raises(RuntimeError):
            L._packed_for_causal_lm_loss(hs, head, labels.to(dev), hidden, **bad)
    with pytest.raises(RuntimeError):
        L._packed_for_causal_lm_loss(hs, head, labels.to(dev), hidden + 64)
    # higher-order gradients are rejected (gguf_liger_loss.py:241-244)
    h2 = hid.to(dev).requires_grad_(True)
    out = L.packed_linear_cross_entropy(h2, head.weight, shifted.to(dev), qt, vocab)
    with pytest.raises(RuntimeError):
        torch.autograd.grad(out, h2, create_graph=True)
    with pytest.raises(TypeError):
        L.packed_linear_cross_entropy(h2.float(), head.weight, shifted.to(dev), qt, vocab)
    with pytest.raises(ValueError):
        L.packed_linear_cross_entropy(h2, head.weight, shifted.to(dev), qt, vocab, reduction="none")


@pytest.mark.parametrize("qt,rows,hidden,vocab,chunk", [
    (gb.Q6_K, 257, 512, 9000, 128),        # streaming sweep over two vocabulary blocks
    (gb.Q8_0, 130, 256, 8192 * 2 + 5, 64),  # three blocks, the last one five columns wide
    (gb.Q4_K, 200, 512, 700, 4096),        # one chunk covers all rows: the logits are kept
])
def test_token_accuracy_and_predicted_tokens(pkg, dev, qt, rows, hidden, vocab, chunk):
    # Liger's optional outputs (gguf_liger_loss.py:92-101, 117-185): argmax of the bf16 logits per row (-1 on ignored rows)
    # and the share of counted rows whose argmax is the label.  The logits of the two paths agree to bf16 rounding of sums
    # taken in different orders, so a row whose two best logits are within one bf16 step may legitimately differ.
    payload, hid, labels = _case(424242, rows, hidden, vocab, qt, ignore_frac=0.1)
    w = mm.weights_bf16(payload, qt)
    # make the label the clear winner for half of the counted rows: accuracy is then well away from 0 and 1
    logits = hid.double() @ w.T
    best = logits.argmax(dim=1)
    take = (torch.arange(rows) % 2 == 0) & (labels != -100)
    labels[take] = best[take]
    want_pred, want_acc = ref.predicted_tokens(hid, w, labels, -100, chunk)
    h = hid.to(dev).requires_grad_(True)
    loss, acc, pred = pkg.gguf_liger_loss.packed_linear_cross_entropy(h, torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, chunk,
                                                                      -100, "mean", return_token_accuracy=True, return_predicted_tokens=True)
    loss.backward()
    assert pred.dtype == torch.int64 and tuple(pred.shape) == (rows,) and not pred.requires_grad and not acc.requires_grad
    pred = pred.cpu()
    assert bool((pred[labels == -100] == -1).all())
    top2 = torch.topk(ref.bf16_round64(logits), 2, dim=1).values
    clear = (labels != -100) & ((top2[:, 0] - top2[:, 1]) > 2.0 ** -6 * top2[:, 0].abs().clamp(min=1.0))
    assert int(clear.sum()) > rows // 2
    assert torch.equal(pred[clear], want_pred[clear])
    near = (labels != -100) & ~clear  # near-ties: either of the two best columns
    top2i = torch.topk(ref.bf16_round64(logits), 2, dim=1).indices
    assert bool(((pred[near] == top2i[near, 0]) | (pred[near] == top2i[near, 1])).all())
    assert abs(float(acc) - want_acc) <= float(near.sum()) / max(1, int((labels != -100).sum())) + 1e-6
    # the loss and gradient are those of the plain call
    h2 = hid.to(dev).requires_grad_(True)
    plain = pkg.gguf_liger_loss.packed_linear_cross_entropy(h2, torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, chunk)
    plain.backward()
    assert torch.equal(loss.detach(), plain.detach()) and torch.equal(h.grad, h2.grad)


def test_argmax_takes_the_first_of_equal_logits(pkg, dev):
    # an all-zero hidden row makes every logit zero: the first column wins, in the kept-logits form and across the blocks of
    # the streaming form (a later block needs a strictly larger maximum)
    qt, hidden, vocab = gb.Q8_0, 256, 8192 + 100
    payload, hid, labels = _case(9, 8, hidden, vocab, qt, ignore_frac=0.0)
    hid[:4] = 0
    for chunk in (4, 4096):
        _, _, pred = pkg.gguf_liger_loss.packed_linear_cross_entropy(hid.to(dev), torch.from_numpy(payload).to(dev), labels.to(dev), qt, vocab, chunk,
                                                                      return_predicted_tokens=True)
        assert pred[:4].tolist() == [0, 0, 0, 0]


def test_out_of_range_labels_are_ignored_and_reported(pkg, dev):
    qt, rows, hidden, vocab = gb.Q8_0, 40, 256, 300
    payload, hid, labels = _case(31, rows, hidden, vocab, qt, ignore_frac=0.1)
    bad = labels.clone()
    bad[3], bad[17] = vocab, -5  # neither a column nor ignore_index
    clean = labels.clone()
    clean[3] = clean[17] = -100
    L = pkg.gguf_liger_loss
    for chunk in (8, 4096):
        out_bad = L._packed_linear_cross_entropy_forward(hid.to(dev), torch.from_numpy(payload).to(dev), bad.to(dev), qt, vocab, chunk, -100, "mean", True, True)
        out_clean = L._packed_linear_cross_entropy_forward(hid.to(dev), torch.from_numpy(payload).to(dev), clean.to(dev), qt, vocab, chunk, -100, "mean", True, True)
        assert out_bad[4].tolist() == [int((clean != -100).sum()), 2] and out_clean[4].tolist()[1] == 0
        assert torch.equal(out_bad[0], out_clean[0]) and torch.equal(out_bad[1], out_clean[1]) and torch.equal(out_bad[6], out_clean[6])
    L.VALIDATE_LABELS = True
    try:
        with pytest.raises(ValueError):
            L.packed_linear_cross_entropy(hid.to(dev), torch.from_numpy(payload).to(dev), bad.to(dev), qt, vocab, 8)
    finally:
        L.VALIDATE_LABELS = False
