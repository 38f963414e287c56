"""The reference's operator namespace served by this library: the seven ``torch.ops.torch_ggml_ops.*`` entries and the
``torch_ggml_ops`` module its files import (fast_lora.py:20, fast_moe_lora.py:221-262 and :339-374, gguf_liger_loss.py:109-177,
deepseek_v4_lora.py:7)."""

import sys

import numpy as np
import pytest
import torch

from helpers import bf16_randn, make_payload
from oracle import gguf_blocks as gb

OPS = ("mmq", "mmq_grad_input", "grouped_mmq", "grouped_mmq_grad_input", "grouped_mmq_pair", "grouped_mmq_pair_grad_input", "fixed_grouped_mmq")


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
