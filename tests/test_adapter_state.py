"""Adapter checkpoints under PEFT's key names (the relations test_deepseek_v4_serialization.py:74-101 pins for the
reference's wrappers): a toy model with one packed dense projection and one packed expert stack, both LoRA-wrapped."""

import numpy as np
import pytest
import torch

from helpers import make_payload
from oracle import gguf_blocks as gb


def _toy(pkg, seed):
    G = pkg.gguf.GGUFQuantizedTensor

    def packed(qt, *shape):
        rows = int(np.prod(shape[:-1]))
        return G(torch.from_numpy(make_payload(seed, qt, rows, shape[-1])).reshape(*shape[:-1], -1), qt, shape)

    class Toy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            lin = pkg.fast_lora.GGUFLinear(256, 64, packed(gb.Q8_0, 64, 256))
            self.q_a_proj = pkg.fast_lora.FastGGUFLoraLinear(lin, r=4, lora_alpha=4)
            experts = pkg.fast_moe_lora.GGUFExperts(packed(gb.Q4_K, 3, 512, 256), packed(gb.Q4_K, 3, 512, 256), packed(gb.Q2_K, 3, 256, 512))
            self.experts = pkg.fast_moe_lora.FastGGUFMoeLora(experts, r=4, lora_alpha=4)

    model = Toy()
    gen = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_((torch.randn(p.shape, generator=gen) * 0.03).to(p.dtype))
    return model


def test_adapter_state_round_trip_contains_only_the_six_lora_factors(pkg):
    fl = pkg.fast_lora
    source = _toy(pkg, 1)
    state = fl.get_adapter_state_dict(source)
    assert sorted(state) == ["experts.lora_A.weight", "experts.lora_A_down.weight", "experts.lora_B.weight", "experts.lora_B_down.weight",
                             "q_a_proj.lora_A.weight", "q_a_proj.lora_B.weight"]
    assert not any("base_layer" in name or "gate_proj" in name or "default" in name for name in state)
    assert state["experts.lora_A_down.weight"].shape == (3, 4, 512) and state["experts.lora_B.weight"].shape == (3, 1024, 4)

    target = _toy(pkg, 2)
    assert not torch.equal(target.experts.lora_B_down["default"].weight, source.experts.lora_B_down["default"].weight)
    missing, unexpected = fl.set_adapter_state_dict(target, state)
    assert missing == [] and unexpected == []
    back = fl.get_adapter_state_dict(target)
    assert back.keys() == state.keys()
    for name in state:
        assert torch.equal(back[name], state[name]), name
    # the packed base weights are untouched and never part of the checkpoint
    assert not torch.equal(target.experts.base_layer.gate_proj.as_subclass(torch.Tensor), source.experts.base_layer.gate_proj.as_subclass(torch.Tensor))
    with pytest.raises(RuntimeError, match="cannot be merged"):
        target.experts.merge()
    with pytest.raises(RuntimeError, match="cannot be merged"):
        target.q_a_proj.merge()


def test_adapter_state_prefix_partial_and_foreign_entries(pkg):
    fl = pkg.fast_lora
    source, target = _toy(pkg, 3), _toy(pkg, 4)
    state = fl.get_adapter_state_dict(source, prefix="base_model.model.")
    assert all(k.startswith("base_model.model.") for k in state)
    partial = {k: v for k, v in state.items() if "lora_A_down" not in k}
    partial["base_model.model.experts.lora_A_up.weight"] = torch.zeros(1)
    before = target.experts.lora_A_down["default"].weight.clone()
    missing, unexpected = fl.set_adapter_state_dict(target, partial, prefix="base_model.model.")
    assert missing == ["experts.lora_A_down.default.weight"]
    assert unexpected == ["experts.lora_A_up.default.weight"]
    assert torch.equal(target.experts.lora_A_down["default"].weight, before)
    assert torch.equal(target.q_a_proj.lora_B["default"].weight, source.q_a_proj.lora_B["default"].weight)
    # another adapter's name selects nothing; a wrong shape is refused
    assert fl.get_adapter_state_dict(source, adapter_name="other") == {}
    bad = dict(state)
    bad["base_model.model.q_a_proj.lora_A.weight"] = torch.zeros(5, 256)
    with pytest.raises(ValueError, match="does not fit"):
        fl.set_adapter_state_dict(target, bad, prefix="base_model.model.")
    # fp32 checkpoints are cast to the factors' dtype
    as32 = {k: v.float() for k, v in state.items()}
    fl.set_adapter_state_dict(target, as32, prefix="base_model.model.")
    assert target.experts.lora_A["default"].weight.dtype == torch.bfloat16
    assert torch.equal(target.experts.lora_A["default"].weight, source.experts.lora_A["default"].weight)
