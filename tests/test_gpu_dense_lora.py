"""Dense packed-weight LoRA linear: Y, dX, dA, dB against the dequantize-then-matmul oracle
(relations of test_fast_lora.py:101-145 and test_deepseek_v4_lora.py:56-99)."""

import numpy as np
import pytest
import torch

from helpers import ALL_TYPES, TYPE_NAMES, assert_close_bf16, bf16_bits, bf16_randn, make_payload
from oracle import gguf_blocks as gb
from oracle import lora_matmul as ref

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
def test_mmq_identity_reproduces_decoded_rows_exactly(pkg, dev, qt):
    # X = I: every output is a single product 1 * w, so Y[m, n] must equal bf16(W[n, m]) as a value.
    # This runs the in-register decoders of the matmul kernel against the oracle, element by element.
    k, n = 512, 300
    payload = make_payload(99 + qt, qt, n, k, "random")
    w = torch.from_numpy(gb.dequantize_bf16(payload, qt))
    x = torch.eye(k, dtype=torch.bfloat16, device=dev)
    p = torch.from_numpy(payload).to(dev)
    y = pkg.fast_lora.mmq(x, p, qt, n)
    assert torch.equal(y.float().cpu(), w.T.contiguous()), "forward decode path differs from the oracle"
    dy = torch.eye(n, dtype=torch.bfloat16, device=dev)
    dx = pkg.fast_lora.mmq_grad_input(dy, p, qt, k)
    assert torch.equal(dx.float().cpu(), w), "grad-input decode path differs from the oracle"


@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
@pytest.mark.parametrize("m,n,k", [(33, 37, 2048), (7, 48, 256), (300, 520, 1024)])
def test_mmq_and_grad_input(pkg, dev, qt, m, n, k):
    gen = torch.Generator().manual_seed(2468 + m)
    payload = make_payload(m * n + qt, qt, n, k)
    w = ref.weights_bf16(payload, qt)
    x = bf16_randn(gen, m, k)
    dy = bf16_randn(gen, m, n)
    want = ref.lora_linear(x, w, dy=dy)
    p = torch.from_numpy(payload).to(dev)
    xd = x.to(dev).requires_grad_(True)
    y = pkg.fast_lora.mmq(xd, p, qt, n)
    y.backward(dy.to(dev))
    assert_close_bf16(y, want["y"], "Y")
    assert_close_bf16(xd.grad, want["dx"], "dX")


@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
@pytest.mark.parametrize("m,n,k,r", [(33, 37, 2048, 4), (3 * 11, 64, 512, 16), (257, 300, 768, 24), (130, 256, 1024, 40), (64, 128, 512, 64)])
def test_lora_linear_forward_backward(pkg, dev, qt, m, n, k, r):
    gen = torch.Generator().manual_seed(97531 + r)
    payload = make_payload(k + r + qt, qt, n, k)
    w = ref.weights_bf16(payload, qt)
    x = bf16_randn(gen, m, k)
    a = bf16_randn(gen, r, k, std=k ** -0.5)
    b = bf16_randn(gen, n, r, std=0.02)
    dy = bf16_randn(gen, m, n)
    s = 32.0 / r
    want = ref.lora_linear(x, w, a, b, s, dy)
    p = torch.from_numpy(payload).to(dev)
    xd, ad, bd = (t.to(dev).requires_grad_(True) for t in (x, a, b))
    y = pkg.fast_lora.lora_mmq(xd, p, qt, n, ad, bd, s)
    y.backward(dy.to(dev))
    assert_close_bf16(y, want["y"], "Y")
    assert_close_bf16(xd.grad, want["dx"], "dX")
    assert_close_bf16(ad.grad, want["da"], "dA")
    assert_close_bf16(bd.grad, want["db"], "dB")
    # the LoRA residual really is in Y: against the base-only product the difference is s * xA B^T
    base = pkg.fast_lora.mmq(x.to(dev), p, qt, n)
    delta = (y.detach().double() - base.double()).cpu()
    want_delta = s * (want["xa"] @ b.double().T)
    # both operands of the difference carry one bf16 rounding of |Y|
    assert float((delta - want_delta).abs().max()) <= 2.0 ** -7 * float(want["y"].abs().max())
    assert float(want_delta.abs().max()) > 2.0 ** -5 * float(want["y"].abs().max()), "test would not see a missing LoRA term"


def test_config0_dense_q8_0(pkg, dev):
    # BASELINE configs[0]: W [2048 x 2048] ~ N(0, 0.02^2) -> Q8_0; X bf16 [1, 512, 2048]; r=16, alpha=32
    gen = torch.Generator().manual_seed(19260817)
    n = k = 2048
    w32 = torch.randn(n, k, generator=gen) * 0.02
    payload = gb.quantize(w32.numpy(), gb.Q8_0)
    x = bf16_randn(gen, 1, 512, k)
    a = bf16_randn(gen, 16, k, std=k ** -0.5)
    b = bf16_randn(gen, n, 16, std=0.01)
    dy = bf16_randn(gen, 1, 512, n)
    want = ref.lora_linear(x[0], ref.weights_bf16(payload, gb.Q8_0), a, b, 2.0, dy[0])
    base = pkg.fast_lora.GGUFLinear(k, n, pkg.gguf.GGUFQuantizedTensor(torch.from_numpy(payload).to(dev), gb.Q8_0, (n, k)))
    layer = pkg.fast_lora.FastGGUFLoraLinear(base, r=16, lora_alpha=32)
    with torch.no_grad():
        layer.lora_A["default"].weight.copy_(a.to(dev))
        layer.lora_B["default"].weight.copy_(b.to(dev))
    xd = x.to(dev).requires_grad_(True)
    y = layer(xd)
    y.backward(dy.to(dev))
    assert y.shape == (1, 512, n)
    assert_close_bf16(y[0], want["y"], "Y")
    assert_close_bf16(xd.grad[0], want["dx"], "dX")
    assert_close_bf16(layer.lora_A["default"].weight.grad, want["da"], "dA")
    assert_close_bf16(layer.lora_B["default"].weight.grad, want["db"], "dB")
    assert base.weight.grad is None


def test_dense_guards(pkg, dev):
    fl = pkg.fast_lora
    p = torch.zeros(8, 144, dtype=torch.uint8, device=dev)
    x = torch.zeros(4, 256, dtype=torch.bfloat16, device=dev)
    with pytest.raises(TypeError):
        fl.mmq(x.float(), p, gb.Q4_K, 8)
    with pytest.raises(ValueError):
        fl.mmq(x, torch.zeros(8, 82, dtype=torch.uint8, device=dev), 22, 8)  # IQ2_S: no kernel here, must not be routed anywhere else
    with pytest.raises(ValueError):
        fl.mmq(x, torch.zeros(8, 8 * 18, dtype=torch.uint8, device=dev), 2, 8)  # Q4_0 with a byte count that would fit: no kernel
    with pytest.raises(ValueError):
        fl.mmq(x, p, gb.Q4_K, 9)  # payload rows do not match out_features
    with pytest.raises(ValueError):
        fl.mmq(x.T.contiguous().T, p, gb.Q4_K, 8)  # non-contiguous input is rejected, not repaired
    with pytest.raises(ValueError):
        fl.mmq(torch.zeros(4, 257, dtype=torch.bfloat16, device=dev)[:, 1:], p, gb.Q4_K, 8)  # strided view
    y = fl.mmq(x.requires_grad_(True), p, gb.Q4_K, 8)
    (g,) = torch.autograd.grad(y.sum(), x, create_graph=False)
    assert g.shape == x.shape


@pytest.mark.parametrize("qt,lead,groups,n_group,k", [(gb.Q8_0, (2,), 8, 128, 512), (gb.Q8_0, (3, 43), 8, 64, 256), (gb.Q4_K, (130,), 4, 128, 512)])
def test_fixed_grouped_mmq_equals_per_group_dense_calls(pkg, dev, qt, lead, groups, n_group, k):
    # the relation the reference pins for DeepSeek's eight-group frozen projection (test_deepseek_v4_lora.py:101-151):
    # output and input gradient equal, bit for bit, the per-group dense op on contiguous slices; and both sit on the oracle
    fl = pkg.fast_lora
    gen = torch.Generator().manual_seed(4242)
    payload = np.stack([make_payload(900 + g, qt, n_group, k) for g in range(groups)])
    x = bf16_randn(gen, *lead, groups, k)
    dy = bf16_randn(gen, *lead, groups, n_group)
    pd = torch.from_numpy(payload).to(dev)
    xd = x.to(dev).requires_grad_(True)
    y = fl.fixed_grouped_mmq(xd, pd, qt)
    y.backward(dy.to(dev))
    assert y.shape == (*lead, groups, n_group)
    xr = x.to(dev).requires_grad_(True)
    want = torch.stack([fl.mmq(xr[..., g, :].contiguous(), pd[g].clone(), qt, n_group) for g in range(groups)], dim=-2)
    want.backward(dy.to(dev))
    assert torch.equal(y, want)
    assert torch.equal(xd.grad, xr.grad)
    w = ref.weights_bf16(payload, qt)
    for g in (0, groups - 1):
        res = ref.lora_linear(x[..., g, :].reshape(-1, k), w[g], dy=dy[..., g, :].reshape(-1, n_group))
        assert_close_bf16(y[..., g, :].reshape(-1, n_group), res["y"], "fixed grouped y")
        assert_close_bf16(xd.grad[..., g, :].reshape(-1, k), res["dx"], "fixed grouped dx")
    with pytest.raises(ValueError):
        fl.fixed_grouped_mmq(xd[..., :2, :].contiguous(), pd, qt)
