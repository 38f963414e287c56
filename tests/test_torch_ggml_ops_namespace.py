"""The reference's operator namespace served by this library: the seven ``torch.ops.torch_ggml_ops.*`` entries and the
``torch_ggml_ops`` module its files import (fast_lora.py:20, fast_moe_lora.py:221-262 and :339-374, gguf_liger_loss.py:109-177,
deepseek_v4_lora.py:7)."""

import sys

import numpy as np
import pytest
import torch

from helpers import bf16_randn, make_payload
from oracle import gguf_blocks as gb

OPS = ("mmq", "mmq_grad_input", "grouped_mmq", "grouped_mmq_grad_input", "grouped_mmq_pair", "grouped_mmq_pair_grad_input", "fixed_grouped_mmq",
       "fixed_grouped_mmq_grad_input")


def test_install_registers_the_operator_names_and_the_module(pkg):
    shim = pkg.torch_ggml_ops
    shim.install(as_module=True)
    shim.install(as_module=True)  # idempotent
    import torch_ggml_ops

    assert torch_ggml_ops is shim and sys.modules["torch_ggml_ops"] is shim
    for name in OPS:
        assert hasattr(getattr(torch.ops.torch_ggml_ops, name), "default"), name
    for name in ("mmq", "grouped_mmq", "grouped_mmq_pair", "fixed_grouped_mmq"):  # what the reference imports by name
        assert callable(getattr(torch_ggml_ops, name))


def test_fake_kernels_give_shapes_without_a_device(pkg):
    # FakeTensor / meta registration (docs/plan_qwen3.5.md:148): the entries trace with no data and no GPU
    from torch._subclasses.fake_tensor import FakeTensorMode

    pkg.torch_ggml_ops.install()
    ops = torch.ops.torch_ggml_ops
    n, k, e, rows = 192, 512, 5, 77
    with FakeTensorMode():
        x = torch.empty(3, 37, k, dtype=torch.bfloat16)
        p = torch.empty(n, k // 256 * 144, dtype=torch.uint8)
        y = ops.mmq(x, p, 12, n)
        assert y.shape == (3, 37, n) and y.dtype == torch.bfloat16
        assert ops.mmq_grad_input(y, p, 12, k).shape == (3, 37, k)
        xs = torch.empty(rows, k, dtype=torch.bfloat16)
        pe = torch.empty(e, n, k // 256 * 210, dtype=torch.uint8)
        ids, ends = torch.empty(e, dtype=torch.int64), torch.empty(e, dtype=torch.int32)
        g = ops.grouped_mmq(xs, pe, ids, ends, 14, n)
        assert g.shape == (rows, n)
        a, b = ops.grouped_mmq_pair(xs, pe, pe, ids, ends, 14, n)
        assert a.shape == b.shape == (rows, n)
        assert ops.grouped_mmq_grad_input(g, pe, ids, ends, 14, k).shape == (rows, k)
        assert ops.grouped_mmq_pair_grad_input(a, b, pe, pe, ids, ends, 14, k).shape == (rows, k)
        xg = torch.empty(11, 8, 256, dtype=torch.bfloat16)
        pg = torch.empty(8, 64, 256 // 32 * 34, dtype=torch.uint8)
        yg = ops.fixed_grouped_mmq(xg, pg, 8)
        assert yg.shape == (11, 8, 64) and ops.fixed_grouped_mmq_grad_input(yg, pg, 8, 256).shape == (11, 8, 256)
        with pytest.raises(RuntimeError):
            ops.mmq(x, p, 12, n + 1)  # payload rows against out_features: checked without data
    # registered autograd traces too: the backward of a forward entry is the grad-input entry
    with FakeTensorMode():
        x = torch.empty(4, k, dtype=torch.bfloat16, requires_grad=True)
        p = torch.empty(n, k // 256 * 144, dtype=torch.uint8)
        (gx,) = torch.autograd.grad(ops.mmq(x, p, 12, n).sum(), x)
        assert gx.shape == x.shape


@pytest.mark.gpu
def test_operator_entries_pass_opcheck_and_differentiate(pkg, dev):
    # torch.library.opcheck (docs/plan_qwen3.5.md:148): schema, fake kernel against the real outputs, registered autograd
    pkg.torch_ggml_ops.install()
    ops = torch.ops.torch_ggml_ops
    gen = torch.Generator().manual_seed(5)
    n, k, e = 128, 256, 3
    p = torch.from_numpy(make_payload(11, gb.Q4_K, n, k)).to(dev)
    x = bf16_randn(gen, 2, 9, k).to(dev)
    dy = bf16_randn(gen, 2, 9, n).to(dev)
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(ops.mmq.default, (x.clone().requires_grad_(True), p, gb.Q4_K, n), test_utils=tests)
    torch.library.opcheck(ops.mmq_grad_input.default, (dy, p, gb.Q4_K, k), test_utils=tests)
    sizes = [20, 0, 45]
    rows = sum(sizes)
    ids = torch.arange(e, dtype=torch.int64, device=dev)
    ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32, device=dev)
    p1 = torch.from_numpy(make_payload(12, gb.Q6_K, e * n, k)).reshape(e, n, -1).to(dev)
    p2 = torch.from_numpy(make_payload(13, gb.Q6_K, e * n, k)).reshape(e, n, -1).to(dev)
    xs = bf16_randn(gen, rows, k).to(dev)
    g1, g2 = bf16_randn(gen, rows, n).to(dev), bf16_randn(gen, rows, n).to(dev)
    torch.library.opcheck(ops.grouped_mmq.default, (xs.clone().requires_grad_(True), p1, ids, ends, gb.Q6_K, n), test_utils=tests)
    torch.library.opcheck(ops.grouped_mmq_pair.default, (xs.clone().requires_grad_(True), p1, p2, ids, ends, gb.Q6_K, n), test_utils=tests)
    torch.library.opcheck(ops.grouped_mmq_grad_input.default, (g1, p1, ids, ends, gb.Q6_K, k), test_utils=tests)
    torch.library.opcheck(ops.grouped_mmq_pair_grad_input.default, (g1, g2, p1, p2, ids, ends, gb.Q6_K, k), test_utils=tests)
    pg = torch.from_numpy(make_payload(14, gb.Q8_0, 8 * 64, 256)).reshape(8, 64, -1).to(dev)
    xg = bf16_randn(gen, 5, 8, 256).to(dev)
    torch.library.opcheck(ops.fixed_grouped_mmq.default, (xg.clone().requires_grad_(True), pg, gb.Q8_0), test_utils=tests)
    # values of the registered backward: the dispatcher entries differentiate like the package's functions
    xr = xs.clone().requires_grad_(True)
    a, b = ops.grouped_mmq_pair(xr, p1, p2, ids, ends, gb.Q6_K, n)
    torch.autograd.backward((a, b), (g1, g2))
    assert torch.equal(xr.grad, pkg.fast_moe_lora.grouped_mmq_pair_grad_input(g1, g2, p1, p2, ids, ends, gb.Q6_K, k))
    xr2 = xg.clone().requires_grad_(True)
    ops.fixed_grouped_mmq(xr2, pg, gb.Q8_0).backward(torch.ones(5, 8, 64, dtype=torch.bfloat16, device=dev))
    assert torch.equal(xr2.grad, pkg.fast_lora.fixed_grouped_mmq_grad_input(torch.ones(5, 8, 64, dtype=torch.bfloat16, device=dev), pg, gb.Q8_0, 256))
    # a gradient of a gradient is rejected: the grad-input entries have no autograd formula
    xr3 = x.clone().requires_grad_(True)
    (gx,) = torch.autograd.grad(ops.mmq(xr3, p, gb.Q4_K, n).sum(), xr3, create_graph=True)
    if gx.requires_grad:
        with pytest.raises(RuntimeError):
            gx.sum().backward()


@pytest.mark.gpu
def test_operator_entries_give_the_package_results(pkg, dev):
    shim = pkg.torch_ggml_ops
    shim.install(as_module=True)
    from torch_ggml_ops import fixed_grouped_mmq, grouped_mmq, grouped_mmq_pair, mmq

    ops = torch.ops.torch_ggml_ops
    gen = torch.Generator().manual_seed(3)
    n, k, e = 192, 512, 5
    # dense
    p = torch.from_numpy(make_payload(1, gb.Q4_K, n, k)).to(dev)
    x = bf16_randn(gen, 3, 37, k).to(dev).requires_grad_(True)
    dy = bf16_randn(gen, 3, 37, n).to(dev)
    y = ops.mmq.default(x.detach(), p, gb.Q4_K, n)
    want = pkg.fast_lora.mmq(x, p, gb.Q4_K, n)
    assert torch.equal(y, want.detach()) and y.shape == (3, 37, n)
    assert torch.equal(ops.mmq_grad_input.default(dy, p, gb.Q4_K, k), pkg.fast_lora.mmq_grad_input(dy, p, gb.Q4_K, k))
    mmq(x, p, gb.Q4_K, n).backward(dy)                      # the imported function is differentiable, as the wheel's is
    assert torch.equal(x.grad, pkg.fast_lora.mmq_grad_input(dy, p, gb.Q4_K, k))
    # grouped
    sizes = [40, 0, 130, 7, 64]
    rows = sum(sizes)
    ids = torch.arange(e, dtype=torch.int64, device=dev)
    ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32, device=dev)
    p1 = torch.from_numpy(make_payload(2, gb.Q6_K, e * n, k)).reshape(e, n, -1).to(dev)
    p2 = torch.from_numpy(make_payload(3, gb.Q6_K, e * n, k)).reshape(e, n, -1).to(dev)
    xs = bf16_randn(gen, rows, k).to(dev)
    g1, g2 = bf16_randn(gen, rows, n).to(dev), bf16_randn(gen, rows, n).to(dev)
    ml = pkg.fast_moe_lora
    assert torch.equal(ops.grouped_mmq.default(xs, p1, ids, ends, gb.Q6_K, n), ml.grouped_mmq(xs, p1, ids, ends, gb.Q6_K, n))
    assert torch.equal(grouped_mmq(xs, p1, ids, ends, gb.Q6_K, n), ml.grouped_mmq(xs, p1, ids, ends, gb.Q6_K, n))
    a1, a2 = ops.grouped_mmq_pair.default(xs, p1, p2, ids, ends, gb.Q6_K, n)
    b1, b2 = grouped_mmq_pair(xs, p1, p2, ids, ends, gb.Q6_K, n)
    assert torch.equal(a1, b1) and torch.equal(a2, b2)
    assert torch.equal(ops.grouped_mmq_grad_input.default(g1, p1, ids, ends, gb.Q6_K, k), ml.grouped_mmq_grad_input(g1, p1, ids, ends, gb.Q6_K, k))
    assert torch.equal(ops.grouped_mmq_pair_grad_input.default(g1, g2, p1, p2, ids, ends, gb.Q6_K, k),
                       ml.grouped_mmq_pair_grad_input(g1, g2, p1, p2, ids, ends, gb.Q6_K, k))
    # fixed groups: the imported function takes the packed tensor alone and reads its block format from it
    G = pkg.gguf.GGUFQuantizedTensor
    pg = G(torch.from_numpy(make_payload(4, gb.Q8_0, 8 * 64, 256)).reshape(8, 64, -1).to(dev), gb.Q8_0, (8, 64, 256))
    xg = bf16_randn(gen, 11, 8, 256).to(dev)
    assert torch.equal(fixed_grouped_mmq(xg, pg), pkg.fast_lora.fixed_grouped_mmq(xg, pg, gb.Q8_0))
    assert torch.equal(ops.fixed_grouped_mmq.default(xg, pg.as_subclass(torch.Tensor), gb.Q8_0), pkg.fast_lora.fixed_grouped_mmq(xg, pg, gb.Q8_0))


def test_grouped_mm_stands_in_for_the_aiter_import_and_checks_its_operands(pkg):
    """``from aiter.ops.triton.gmm import gmm, ptgmm`` (fast_moe_lora.py:22) resolves to the package's functions once
    installed; their operand checks run without a device."""
    import importlib
    import sys

    gm = pkg.grouped_mm
    gm.install_as_aiter_gmm()
    gm.install_as_aiter_gmm()  # idempotent
    mod = importlib.import_module("aiter.ops.triton.gmm")
    assert mod.gmm is gm.gmm and mod.ptgmm is gm.ptgmm
    assert sys.modules["aiter"].ops.triton.gmm is mod
    sizes = torch.tensor([2, 2, 2], dtype=torch.int32)
    with pytest.raises(ValueError, match="expects lhs"):
        gm.aiter_grouped_mm(torch.zeros(6, 4, 1, dtype=torch.bfloat16), torch.zeros(3, 4, 5, dtype=torch.bfloat16), sizes)
    with pytest.raises(ValueError, match="expert mismatch"):
        gm.aiter_grouped_mm(torch.zeros(6, 4, dtype=torch.bfloat16), torch.zeros(2, 4, 5, dtype=torch.bfloat16), sizes)
    with pytest.raises(RuntimeError, match="ROCm device"):
        gm.aiter_grouped_mm(torch.zeros(6, 4, dtype=torch.bfloat16), torch.zeros(3, 4, 5, dtype=torch.bfloat16), sizes)


@pytest.mark.gpu
def test_operator_entries_compose_with_torch_compile(pkg, dev):
    """``torch.compile`` composition (docs/plan_qwen3.5.md:125-150): a function over the dispatcher entries is traced through
    their FakeTensor kernels and registered autograd (the ``aot_eager`` backend: no code generation involved) and gives the
    eager bits, forward and backward."""
    pkg.torch_ggml_ops.install()
    ops = torch.ops.torch_ggml_ops
    gen = torch.Generator().manual_seed(9)
    n, k, e = 128, 256, 3
    p = torch.from_numpy(make_payload(21, gb.Q4_K, n, k)).to(dev)
    sizes = [20, 0, 45]
    ids = torch.arange(e, dtype=torch.int64, device=dev)
    ends = torch.tensor(np.cumsum(sizes), dtype=torch.int32, device=dev)
    p1 = torch.from_numpy(make_payload(22, gb.Q4_K, e * n, k)).reshape(e, n, -1).to(dev)
    p2 = torch.from_numpy(make_payload(23, gb.Q4_K, e * n, k)).reshape(e, n, -1).to(dev)

    def fn(x, xs):
        y = ops.mmq(x, p, gb.Q4_K, n)
        a, b = ops.grouped_mmq_pair(xs, p1, p2, ids, ends, gb.Q4_K, n)
        return y.float().square().mean() + (a.float() * torch.sigmoid(b.float())).mean()

    compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
    x0, xs0 = bf16_randn(gen, 2, 9, k).to(dev), bf16_randn(gen, sum(sizes), k).to(dev)
    results = []
    for f in (fn, compiled):
        x, xs = x0.clone().requires_grad_(True), xs0.clone().requires_grad_(True)
        out = f(x, xs)
        out.backward()
        results.append((out.detach(), x.grad, xs.grad))
    for got, want in zip(results[1], results[0]):
        assert torch.equal(got, want)
