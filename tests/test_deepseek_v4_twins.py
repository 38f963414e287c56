"""The DeepSeek-V4 twins of the dense, expert and loss surfaces (deepseek_v4_lora.py, deepseek_v4_moe_lora.py,
deepseek_v4_liger_loss.py of the reference): same kernels behind DeepSeek's names and guards."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, make_payload
from oracle import gguf_blocks as gb


def _packed(pkg, seed, qt, *shape, device="cpu"):
    rows = int(np.prod(shape[:-1]))
    t = torch.from_numpy(make_payload(seed, qt, rows, shape[-1])).reshape(*shape[:-1], -1).to(device)
    return pkg.gguf.GGUFQuantizedTensor(t, qt, shape)


def test_guards_and_path_helpers(pkg):
    dl, dm, dloss = pkg.deepseek_v4_lora, pkg.deepseek_v4_moe_lora, pkg.deepseek_v4_liger_loss
    assert dm.EXPERTS_IMPLEMENTATION == "deepseek_v4_gguf_dequant_aiter_lora" and dloss._PACKED_LM_HEAD_CHUNK_SIZE == 512
    assert dl.normalize_peft_path("base_model.model.model.layers.3.mlp.experts") == "model.layers.3.mlp.experts"
    assert dl.normalize_peft_path("layers.0.self_attn.q_a_proj") == "model.layers.0.self_attn.q_a_proj"
    assert dl.normalize_peft_path("lm_head") == "lm_head"
    assert dl.is_adapter_parameter("x.experts.lora_B_down.default.weight") and not dl.is_adapter_parameter("x.experts.base_layer.gate_proj")
    gate, up, down = _packed(pkg, 1, gb.IQ2_XXS, 2, 256, 256), _packed(pkg, 2, gb.IQ2_XXS, 2, 256, 256), _packed(pkg, 3, gb.Q2_K, 2, 256, 256)
    with pytest.raises(ValueError, match="swiglu_limit"):
        dm.DeepseekV4GGUFExperts(gate, up, down, swiglu_limit=0.0)
    plain = pkg.fast_moe_lora.GGUFExperts(gate, up, down)
    wrapper = dm.DeepseekV4GGUFMoeLora(plain, r=4, lora_alpha=4)
    x, idx, w = torch.zeros(3, 256, dtype=torch.bfloat16), torch.zeros(3, 1, dtype=torch.int64), torch.ones(3, 1)
    with pytest.raises(TypeError, match="DeepseekV4GGUFExperts"):
        wrapper(x, idx, w)
    with pytest.raises(TypeError, match="DeepseekV4GGUFExperts"):
        dm.deepseek_v4_gguf_dequant_aiter_lora_forward(plain, x, idx, w)
    with pytest.raises(RuntimeError, match="cannot be merged"):
        wrapper.merge()
    head = pkg.fast_lora.GGUFLinear(256, 64, _packed(pkg, 4, gb.Q6_K, 64, 256))
    with pytest.raises(RuntimeError, match="only for Q8_0"):
        dloss.deepseek_v4_packed_liger_causal_lm_loss(torch.zeros(2, 3, 256, dtype=torch.bfloat16), head, torch.zeros(2, 3, dtype=torch.int64), hidden_size=256)
    q8_head = pkg.fast_lora.GGUFLinear(256, 64, _packed(pkg, 5, gb.Q8_0, 64, 256))
    with pytest.raises(RuntimeError, match="label smoothing"):
        dloss.deepseek_v4_packed_liger_causal_lm_loss(torch.zeros(2, 3, 256, dtype=torch.bfloat16), q8_head, torch.zeros(2, 3, dtype=torch.int64),
                                                      hidden_size=256, loss_kwargs={"label_smoothing": 0.1})
    grouped = dl.GGUFGroupedLinear(256, 512, 8, _packed(pkg, 6, gb.Q8_0, 512, 256))
    grouped.input_permutation = torch.arange(256)
    with pytest.raises(RuntimeError, match="layout permutations"):
        grouped(torch.zeros(4, 8, 256, dtype=torch.bfloat16))


@pytest.mark.gpu
def test_twins_give_the_shared_surfaces_results(pkg, dev):
    dl, dm, dloss = pkg.deepseek_v4_lora, pkg.deepseek_v4_moe_lora, pkg.deepseek_v4_liger_loss
    gen = torch.Generator().manual_seed(8)
    # experts: IQ2_XXS gate / up, Q2_K down, clamped SwiGLU
    e, hidden, inter, tokens, top_k, limit = 6, 512, 256, 90, 3, 1.25
    gate, up = _packed(pkg, 11, gb.IQ2_XXS, e, inter, hidden, device=dev), _packed(pkg, 12, gb.IQ2_XXS, e, inter, hidden, device=dev)
    down = _packed(pkg, 13, gb.Q2_K, e, hidden, inter, device=dev)
    twin = dm.DeepseekV4GGUFMoeLora(dm.DeepseekV4GGUFExperts(gate, up, down, swiglu_limit=limit), r=4, lora_alpha=4)
    shared = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down, swiglu_limit=limit), r=4, lora_alpha=4)
    with torch.no_grad():
        for p in twin.parameters():
            p.copy_(bf16_randn(gen, *p.shape, std=0.05).to(dev))
    shared.load_state_dict(twin.state_dict())
    x = bf16_randn(gen, tokens, hidden).to(dev)
    top = torch.topk(torch.randn(tokens, e, generator=gen), top_k, dim=-1)
    idx, w = top.indices.to(dev), torch.softmax(top.values, -1).to(dev)
    dy = bf16_randn(gen, tokens, hidden).to(dev)
    outs = []
    for layer in (twin, shared):
        xi = x.clone().requires_grad_(True)
        out = layer(xi, idx, w)
        out.backward(dy)
        outs.append([out.detach(), xi.grad] + [p.grad for p in layer.parameters()])
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # the eight-group Q8_0 projection: every group is the dense op on its slice
    groups, k, n_group = 8, 256, 64
    lin = dl.GGUFGroupedLinear(k, groups * n_group, groups, _packed(pkg, 14, gb.Q8_0, groups * n_group, k, device=dev))
    xg = bf16_randn(gen, 5, 7, groups, k).to(dev)
    y = lin(xg.float())                                   # the input's dtype comes back (deepseek_v4_lora.py:100, :124)
    assert y.dtype == torch.float32 and y.shape == (5, 7, groups, n_group)
    payload = lin.weight.as_subclass(torch.Tensor).reshape(groups, n_group, -1)
    for g in range(groups):
        want = pkg.fast_lora.mmq(xg[..., g, :].contiguous(), payload[g], gb.Q8_0, n_group)
        assert torch.equal(y[..., g, :].to(torch.bfloat16), want)
    # the loss: chunks of 512 rows, Q8_0 head, sum / num_items reduction
    vocab, hsz = 1000, 256
    head = pkg.fast_lora.GGUFLinear(hsz, vocab, _packed(pkg, 15, gb.Q8_0, vocab, hsz, device=dev))
    hs = bf16_randn(gen, 2, 300, hsz).to(dev).requires_grad_(True)
    labels = torch.randint(0, vocab, (2, 300), generator=gen).to(dev)
    loss = dloss.deepseek_v4_packed_liger_causal_lm_loss(hs, head, labels, hidden_size=hsz, loss_kwargs={"num_items_in_batch": 550})
    loss.backward()
    shifted = torch.nn.functional.pad(labels, (0, 1), value=-100)[..., 1:].reshape(-1)
    hs2 = hs.detach().clone().requires_grad_(True)
    want = pkg.gguf_liger_loss.packed_linear_cross_entropy(hs2.reshape(-1, hsz), head.weight, shifted, gb.Q8_0, vocab, 512, -100, "sum") / 550
    want.backward()
    assert torch.equal(loss, want) and torch.equal(hs.grad, hs2.grad)
