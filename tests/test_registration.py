"""The functions that install the kernels into a model: ``register_fast_lora`` (fast_lora.py:178-200 of the reference),
``register_fast_moe_lora`` (fast_moe_lora.py:773-802), ``apply_gguf_liger_fused_linear_cross_entropy``
(gguf_liger_loss.py:515-532), ``configure_fast_moe_ranking`` (fast_moe_ranking.py:319-380) and their DeepSeek twins.

PEFT and the reference's transformers fork are not importable here, so the registration functions run against the package's
own config stand-in (the same ``_register_custom_module`` interface) and against transformers' stock Qwen3.5-MoE and
DeepSeek-V4 module classes.  What stays unexercised: ``peft.get_peft_model`` constructing the registered wrappers, and the
fork's ``GGUFExperts`` / ``set_experts_implementation``.  The GPU test runs a small stock ``Qwen3_5MoeForCausalLM`` twice,
as transformers ships it (with the dequantized weights) and with every function above applied, and compares loss and
input gradient.
"""

import copy
import types

import pytest
import torch

from oracle import gguf_blocks as gb


def _fake_packed(pkg, quant_type, shape, device="cpu"):
    """A packed tensor of the right byte shape with zero payload: enough for construction and guards (no compute)."""
    *lead, rows, k = shape
    payload = torch.zeros(*lead, rows, pkg.gguf.row_bytes(quant_type, k), dtype=torch.uint8, device=device)
    return pkg.gguf.GGUFQuantizedTensor(payload, quant_type, tuple(shape))


class _Block(torch.nn.Module):
    def __init__(self, pkg):
        super().__init__()
        self.q_proj = pkg.fast_lora.GGUFLinear(256, 128, _fake_packed(pkg, gb.Q4_K, (128, 256)))
        self.out_proj = torch.nn.Linear(64, 32, bias=True)
        self.norm = torch.nn.LayerNorm(32)
        self.experts = pkg.fast_moe_lora.GGUFExperts(_fake_packed(pkg, gb.Q4_K, (4, 256, 256)), _fake_packed(pkg, gb.Q4_K, (4, 256, 256)),
                                                      _fake_packed(pkg, gb.Q4_K, (4, 256, 256)))


class _Model(torch.nn.Module):
    def __init__(self, pkg):
        super().__init__()
        self.layers = torch.nn.ModuleList([_Block(pkg), _Block(pkg)])
        self.implementation_calls = []

    def set_experts_implementation(self, name):
        self.implementation_calls.append(name)


def test_register_fast_lora_and_injection(pkg):
    fl, pc = pkg.fast_lora, pkg.peft_compat
    with pytest.raises(RuntimeError, match="_register_custom_module"):
        fl.register_fast_lora(types.SimpleNamespace(target_modules=["q_proj"]))
    cfg = pc.LoraConfig(r=4, lora_alpha=8, target_modules=["q_proj", "out_proj"], init_lora_weights=False)
    assert fl.register_fast_lora(cfg) is cfg
    assert list(cfg._custom_modules.items()) == [(fl.GGUFLinear, fl.FastGGUFLoraLinear), (torch.nn.Linear, fl.FastLoraLinear)]
    model = _Model(pkg)
    report = pc.inject_adapter(model, cfg)
    assert report["wrapped"] == ["layers.0.q_proj", "layers.0.out_proj", "layers.1.q_proj", "layers.1.out_proj"]
    assert type(model.layers[0].q_proj) is fl.FastGGUFLoraLinear and type(model.layers[1].out_proj) is fl.FastLoraLinear
    assert model.layers[0].q_proj.get_base_layer() is model.layers[0].q_proj.base_layer
    trainable = [n for n, p in model.named_parameters() if p.requires_grad]
    assert trainable and all(".lora_A." in n or ".lora_B." in n for n in trainable) and sorted(trainable) == report["trainable"]
    assert model.layers[0].q_proj.lora_A["default"].weight.shape == (4, 256) and model.layers[0].q_proj.scaling["default"] == 2.0
    # the float wrapper on the CPU: base + scaling * B(A(x)), and the base alone with adapters disabled
    layer = model.layers[0].out_proj
    x = torch.randn(5, 64)
    want = layer.base_layer(x) + 2.0 * (x @ layer.lora_A["default"].weight.T) @ layer.lora_B["default"].weight.T
    assert torch.allclose(layer(x), want, atol=1e-5)
    layer.disable_adapters = True
    assert torch.equal(layer(x), layer.base_layer(x))
    # options the fast wrappers refuse, from the config or from keywords; a second injection finds nothing new to wrap
    for bad in (dict(use_dora=True), dict(lora_bias=True), dict(init_lora_weights="pissa")):
        with pytest.raises(ValueError):
            fl.FastLoraLinear(torch.nn.Linear(8, 8), "default", r=2, lora_alpha=2, config=pc.LoraConfig(**bad))
    with pytest.raises(ValueError, match="lora_dropout=0"):
        fl.FastGGUFLoraLinear(_Block(pkg).q_proj, "default", r=2, lora_alpha=2, lora_dropout=0.1)
    with pytest.raises(TypeError, match="adapter's name"):
        fl.FastGGUFLoraLinear(_Block(pkg).q_proj, 4, r=2, lora_alpha=2)
    with pytest.raises(ValueError, match="matched no module"):
        pc.inject_adapter(model, cfg)
    # a targeted module with no registered wrapper stops the injection
    cfg2 = fl.register_fast_lora(pc.LoraConfig(r=2, lora_alpha=2, target_modules=["norm"]))
    with pytest.raises(TypeError, match="no registered LoRA wrapper"):
        pc.inject_adapter(_Model(pkg), cfg2)


def test_register_fast_moe_lora(pkg):
    ml, pc = pkg.fast_moe_lora, pkg.peft_compat
    model = _Model(pkg)
    with pytest.raises(RuntimeError, match="_register_custom_module"):
        ml.register_fast_moe_lora(types.SimpleNamespace(target_modules=[], target_parameters=None), model)
    with pytest.raises(ValueError, match="target_parameters"):
        ml.register_fast_moe_lora(pc.LoraConfig(target_modules=["q_proj"], target_parameters=["experts.gate_proj"]), model)
    with pytest.raises(TypeError, match="regex string"):
        ml.register_fast_moe_lora(pc.LoraConfig(target_modules=".*experts"), model)
    for e in (model.layers[0].experts, model.layers[1].experts):
        e.experts_implementation = "something else"
    cfg = pc.LoraConfig(r=4, lora_alpha=4, target_modules=["q_proj"])
    assert ml.register_fast_moe_lora(cfg, model) is cfg
    assert cfg.target_modules == {"q_proj", "experts"}
    assert ml.ALL_GGUF_EXPERTS_FUNCTIONS[ml.EXPERTS_IMPLEMENTATION] is ml.qwen3_5_moe_gguf_mmq_lora_forward
    assert model.implementation_calls == [ml.EXPERTS_IMPLEMENTATION]
    assert all(b.experts.experts_implementation == ml.EXPERTS_IMPLEMENTATION for b in model.layers)
    assert cfg._custom_modules == {ml.GGUFExperts: ml.FastGGUFMoeLora}
    pkg.fast_lora.register_fast_lora(cfg)  # the training script registers both on one config (train_qwen3.5_35b.py:112-113)
    report = pc.inject_adapter(model, cfg)
    assert "layers.1.experts" in report["wrapped"] and type(model.layers[1].experts) is ml.FastGGUFMoeLora
    w = model.layers[1].experts
    assert w.lora_A["default"].weight.shape == (4, 4, 256) and w.lora_B["default"].weight.shape == (4, 512, 4)
    assert w.lora_A_down["default"].weight.shape == (4, 4, 256) and w.lora_B_down["default"].weight.shape == (4, 256, 4)
    assert float(w.lora_B["default"].weight.detach().abs().max()) == 0.0 and float(w.lora_A["default"].weight.detach().abs().max()) > 0.0
    # an unregistered implementation name fails at the call, not silently
    model.layers[0].experts.base_layer.experts_implementation = "nobody"
    with pytest.raises(RuntimeError, match="not registered"):
        model.layers[0].experts.base_layer(torch.zeros(1, 256), torch.zeros(1, 2, dtype=torch.long), torch.zeros(1, 2))
    with pytest.raises(ValueError, match="not registered"):
        ml.set_gguf_experts_implementation(model, "nobody")


def test_deepseek_registration_twins(pkg):
    dl, dm, pc = pkg.deepseek_v4_lora, pkg.deepseek_v4_moe_lora, pkg.peft_compat
    with pytest.raises(ValueError, match="exact indexer-excluding pattern"):
        dl.register_deepseek_v4_lora(pc.LoraConfig(target_modules=["q_a_proj"]))
    cfg = pc.LoraConfig(r=4, lora_alpha=4, target_modules=dl.DEEPSEEK_V4_TARGET_MODULES_PATTERN)
    dl.register_deepseek_v4_lora(cfg)
    assert list(cfg._custom_modules)[0] is dl.GGUFGroupedLinear  # the rejecting entry is looked up first

    class Attn(torch.nn.Module):
        def __init__(self, with_indexer):
            super().__init__()
            self.q_a_proj = pkg.fast_lora.GGUFLinear(256, 64, _fake_packed(pkg, gb.Q8_0, (64, 256)))
            self.o_a_proj = dl.GGUFGroupedLinear(256, 8 * 32, 8, _fake_packed(pkg, gb.Q8_0, (8 * 32, 256)))
            self.o_b_proj = torch.nn.Linear(32, 16, bias=False)
            if with_indexer:
                self.compressor = torch.nn.Module()
                self.compressor.indexer = torch.nn.Module()
                self.compressor.indexer.q_b_proj = torch.nn.Linear(8, 8)

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.self_attn = Attn(True)
            self.experts = dm.DeepseekV4GGUFExperts(_fake_packed(pkg, gb.IQ2_XXS, (4, 256, 256)), _fake_packed(pkg, gb.IQ2_XXS, (4, 256, 256)),
                                                    _fake_packed(pkg, gb.IQ2_XXS, (4, 256, 256)), swiglu_limit=7.0)

    model = torch.nn.Module()
    model.layers = torch.nn.ModuleList([Layer()])
    with pytest.raises(ValueError, match="exact indexer-excluding"):
        dm.register_deepseek_v4_moe_lora(pc.LoraConfig(target_modules=".*"), model)
    dm.register_deepseek_v4_moe_lora(cfg, model)
    assert cfg.target_modules == dl.DEEPSEEK_V4_TARGET_MODULES_PATTERN
    assert dm.ALL_GGUF_EXPERTS_FUNCTIONS[dm.EXPERTS_IMPLEMENTATION] is dm.deepseek_v4_gguf_dequant_aiter_lora_forward
    report = pc.inject_adapter(model, cfg)
    assert sorted(report["wrapped"]) == ["layers.0.experts", "layers.0.self_attn.o_b_proj", "layers.0.self_attn.q_a_proj"]  # not o_a_proj, not the indexer
    attn = model.layers[0].self_attn
    assert type(attn.q_a_proj) is dl.DeepseekV4GGUFLoraLinear and type(attn.o_b_proj) is dl.DeepseekV4LoraLinear
    assert type(model.layers[0].experts) is dm.DeepseekV4GGUFMoeLora and type(attn.o_a_proj) is dl.GGUFGroupedLinear
    assert not any(dl.is_adapter_parameter(n) for n, p in model.named_parameters() if not p.requires_grad)
    # a pattern that reaches the grouped projection stops at the rejecting wrapper
    cfg_bad = pc.LoraConfig(target_modules=["o_a_proj"])
    cfg_bad._register_custom_module(dict(cfg._custom_modules))
    with pytest.raises(RuntimeError, match="grouped o_a_proj LoRA is unsupported"):
        pc.inject_adapter(model, cfg_bad)
    # the grouped forward is installed per instance, once, and the geometry check is the reference's
    report = dl.configure_deepseek_v4_grouped_mmq(model)
    assert report == {"enabled": 1, "paths": ["layers.0.self_attn.o_a_proj"]} and attn.o_a_proj._deepseek_v4_grouped_mmq_enabled
    bound = attn.o_a_proj.forward
    assert dl.configure_deepseek_v4_grouped_mmq(model)["enabled"] == 1 and attn.o_a_proj.forward == bound
    with pytest.raises(RuntimeError, match="4096->1024 contract"):
        dl.configure_deepseek_v4_grouped_mmq(model, require_checkpoint_geometry=True)


def _tiny_qwen_config(**over):
    from transformers.models.qwen3_5_moe.configuration_qwen3_5_moe import Qwen3_5MoeTextConfig

    kw = dict(vocab_size=512, hidden_size=256, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
              moe_intermediate_size=256, shared_expert_intermediate_size=256, num_experts=8, num_experts_per_tok=2,
              linear_num_value_heads=4, linear_num_key_heads=2, linear_key_head_dim=32, linear_value_head_dim=32,
              max_position_embeddings=128, layer_types=["linear_attention", "full_attention"])
    kw.update(over)
    return Qwen3_5MoeTextConfig(**kw)


def test_configure_fast_moe_ranking_on_transformers_modules(pkg):
    from transformers.models.deepseek_v4.modeling_deepseek_v4 import DeepseekV4HashRouter, DeepseekV4TopKRouter
    from transformers.models.qwen3_5_moe.modeling_qwen3_5_moe import Qwen3_5MoeForCausalLM

    rk = pkg.fast_moe_ranking
    model = Qwen3_5MoeForCausalLM(_tiny_qwen_config())
    wrapper = types.SimpleNamespace(get_base_model=lambda: model)  # a PEFT wrapper is unwrapped
    report = rk.configure_fast_moe_ranking(wrapper)
    assert report["qwen"] == 2 and report["paths"]["qwen"] == ["model.layers.0.mlp.gate", "model.layers.1.mlp.gate"]
    assert report["deepseek_topk"] == report["deepseek_hash"] == 0
    assert model.model.layers[0].mlp.gate.forward.__func__ is rk._qwen_router_forward
    with pytest.raises(RuntimeError, match="2048/256/top-8"):
        rk.configure_fast_moe_ranking(model, require_checkpoint_geometry=True)
    with pytest.raises(RuntimeError, match="multiple of 4"):
        rk.configure_fast_moe_ranking(Qwen3_5MoeForCausalLM(_tiny_qwen_config(num_experts=6)))
    # DeepSeek's two router classes, built from the fields their constructors read
    cfg = types.SimpleNamespace(num_experts_per_tok=6, num_local_experts=16, hidden_size=64, scoring_func="sqrtsoftplus", routed_scaling_factor=1.5,
                                vocab_size=32, model_type="deepseek_v4")
    ds = torch.nn.Module()
    ds.config = cfg
    ds.gate = DeepseekV4TopKRouter(cfg)
    ds.hash_gate = DeepseekV4HashRouter(cfg)
    report = rk.configure_fast_moe_ranking(ds)
    assert (report["deepseek_topk"], report["deepseek_hash"]) == (1, 1) and report["paths"]["deepseek_hash"] == ["hash_gate"]
    assert ds.hash_gate.forward.__func__ is rk._deepseek_hash_router_forward
    with pytest.raises(RuntimeError, match="4096/256/top-6"):
        rk.configure_fast_moe_ranking(ds, require_checkpoint_geometry=True)
    cfg.scoring_func = "sigmoid"
    with pytest.raises(RuntimeError, match="sqrtsoftplus"):
        rk.configure_fast_moe_ranking(ds)
    # the hash router's replacement is framework code: it runs here and matches the stock module (fp32 logits, same table)
    cfg.scoring_func = "sqrtsoftplus"
    stock = DeepseekV4HashRouter(cfg)
    torch.nn.init.normal_(stock.weight, std=0.1)
    stock.tid2eid.copy_(torch.stack([torch.randperm(16)[:6] for _ in range(32)]))
    patched = copy.deepcopy(stock)
    holder = torch.nn.Module()
    holder.config, holder.gate = cfg, patched
    rk.configure_fast_moe_ranking(holder)
    h, ids = torch.randn(3, 5, 64), torch.randint(0, 32, (3, 5))
    for got, want in zip(patched(h, ids), stock(h, ids)):
        assert got.shape == want.shape and torch.allclose(got.float(), want.float(), atol=1e-6)


def test_apply_gguf_liger_loss_guards(pkg):
    gl, dl = pkg.gguf_liger_loss, pkg.deepseek_v4_liger_loss

    class Qwen3_5MoeForCausalLM(torch.nn.Module):  # recognised by name, as the fork's and upstream's classes are
        def __init__(self, head):
            super().__init__()
            self.lm_head = head
            self.config = types.SimpleNamespace(hidden_size=256, output_router_logits=False, use_return_dict=True)
            self.vocab_size = 128

        def model(self, input_ids=None, **kw):
            self.seen = kw
            return types.SimpleNamespace(last_hidden_state=torch.zeros(1, 4, 256, dtype=torch.bfloat16))

    head = pkg.fast_lora.GGUFLinear(256, 128, _fake_packed(pkg, gb.Q6_K, (128, 256)))
    with pytest.raises(TypeError, match="requires Qwen3_5MoeForCausalLM"):
        gl.apply_gguf_liger_fused_linear_cross_entropy(torch.nn.Linear(2, 2))
    with pytest.raises(TypeError, match="requires GGUFLinear"):
        gl.apply_gguf_liger_fused_linear_cross_entropy(Qwen3_5MoeForCausalLM(torch.nn.Linear(256, 128)))
    model = Qwen3_5MoeForCausalLM(head)
    target = gl.apply_gguf_liger_fused_linear_cross_entropy(types.SimpleNamespace(get_base_model=lambda: model))
    assert target is model and model.forward.__func__ is gl.gguf_liger_lce_forward
    labels = torch.zeros(1, 4, dtype=torch.long)
    model.train()
    with pytest.raises(RuntimeError, match="logits_to_keep=0"):
        model(input_ids=labels, labels=labels, logits_to_keep=1)
    with pytest.raises(RuntimeError, match="requires labels or shift_labels"):
        model(input_ids=labels, skip_logits=True)
    with pytest.raises(RuntimeError, match="no-full-logits fused loss"):
        model(input_ids=labels, labels=labels, skip_logits=False)
    head.bias = torch.zeros(128)
    with pytest.raises(RuntimeError, match="bias-free"):
        model(input_ids=labels, labels=labels)
    assert "attention_mask" not in model.seen and model.seen["output_router_logits"] is False  # None arguments are not forwarded
    with pytest.raises(TypeError, match="requires DeepseekV4ForCausalLM"):
        dl.apply_deepseek_v4_liger_loss(model)

    class DeepseekV4ForCausalLM(Qwen3_5MoeForCausalLM):
        pass

    ds = DeepseekV4ForCausalLM(pkg.fast_lora.GGUFLinear(256, 128, _fake_packed(pkg, gb.Q8_0, (128, 256))))
    assert dl.apply_deepseek_v4_liger_loss(ds) is ds and ds._deepseek_v4_liger_loss_enabled
    bound = ds.forward
    assert dl.apply_deepseek_v4_liger_loss(ds).forward == bound  # installed once


# ------------------------------------------------------------------------------------------------
def _pack_model(pkg, model, dev):
    """Turns a stock transformers Qwen3.5-MoE model into its packed form in place (what the fork's GGUF loader produces):
    expert weights Q4_K, lm_head Q6_K, every other linear whose input width is a multiple of 256 Q4_K.  Returns a deep copy of
    the original whose weights are the DECODED packed weights, so that both models compute the same function."""
    from transformers.models.qwen3_5_moe.modeling_qwen3_5_moe import Qwen3_5MoeExperts

    G, g = pkg.gguf.GGUFQuantizedTensor, pkg.gguf
    stock = copy.deepcopy(model)

    def pack(w, qt):
        quant = {gb.Q4_K: g.quantize_q4_k, gb.Q6_K: g.quantize_q6_k}[qt]
        payload = quant(w.detach().float())
        return payload, g.dequantize_gguf_tensor(payload, qt, torch.bfloat16)

    for name, module in list(model.named_modules()):
        parent = model.get_submodule(name.rpartition(".")[0]) if "." in name else model
        child = name.rpartition(".")[2]
        twin = stock.get_submodule(name) if name else stock
        if isinstance(module, Qwen3_5MoeExperts):
            e, i, h = module.num_experts, module.intermediate_dim, module.hidden_dim
            gate_p, gate_w = pack(module.gate_up_proj[:, :i], gb.Q4_K)
            up_p, up_w = pack(module.gate_up_proj[:, i:], gb.Q4_K)
            down_p, down_w = pack(module.down_proj, gb.Q4_K)
            with torch.no_grad():
                twin.gate_up_proj.copy_(torch.cat([gate_w, up_w], dim=1))
                twin.down_proj.copy_(down_w)
            setattr(parent, child, pkg.fast_moe_lora.GGUFExperts(G(gate_p, gb.Q4_K, (e, i, h)), G(up_p, gb.Q4_K, (e, i, h)), G(down_p, gb.Q4_K, (e, h, i))))
        elif type(module) is torch.nn.Linear and module.in_features % 256 == 0 and module.out_features % 64 == 0 and module.bias is None \
                and child not in ("shared_expert_gate",):
            qt = gb.Q6_K if child == "lm_head" else gb.Q4_K
            payload, w = pack(module.weight, qt)
            with torch.no_grad():
                twin.weight.copy_(w)
            setattr(parent, child, pkg.fast_lora.GGUFLinear(module.in_features, module.out_features,
                                                            G(payload, qt, (module.out_features, module.in_features))))
    return stock


@pytest.mark.gpu
def test_patched_transformers_model_matches_the_stock_one(pkg, dev):
    from transformers.models.qwen3_5_moe.modeling_qwen3_5_moe import Qwen3_5MoeForCausalLM

    torch.manual_seed(11)
    cfg = _tiny_qwen_config()
    cfg._attn_implementation = "eager"
    model = Qwen3_5MoeForCausalLM(cfg).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        for layer in model.model.layers:  # routers as trained ones are: distinct experts per token, no near-ties
            layer.mlp.gate.weight.normal_(std=0.5)
    stock = _pack_model(pkg, model, dev)
    packed_linears = [n for n, m in model.named_modules() if isinstance(m, pkg.fast_lora.GGUFLinear)]
    assert "lm_head" in packed_linears and any(n.endswith("q_proj") for n in packed_linears) and any(n.endswith("shared_expert.down_proj") for n in packed_linears)

    lora = pkg.peft_compat.LoraConfig(r=8, lora_alpha=16, target_modules=["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj",
                                                                            "out_proj"])
    pkg.fast_lora.register_fast_lora(lora)
    pkg.fast_moe_lora.register_fast_moe_lora(lora, model)
    report = pkg.peft_compat.inject_adapter(model, lora)
    assert sum(n.endswith("experts") for n in report["wrapped"]) == 2
    assert any(type(m) is pkg.fast_lora.FastLoraLinear for m in model.modules())  # linear_attn.out_proj (input width 128) stays a float layer
    assert pkg.fast_moe_ranking.configure_fast_moe_ranking(model)["qwen"] == 2
    pkg.gguf_liger_loss.apply_gguf_liger_fused_linear_cross_entropy(model)

    gen = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 512, (2, 48), generator=gen).to(dev)
    labels = ids.clone()
    labels[0, :5] = -100
    embeds = stock.model.embed_tokens(ids).detach()
    model.train()
    stock.train()
    e1 = embeds.clone().requires_grad_(True)
    out = model(inputs_embeds=e1, labels=labels, use_cache=False)
    assert out.logits is None and out.loss.dtype == torch.float32
    out.loss.backward()
    e2 = embeds.clone().requires_grad_(True)
    ref = stock(inputs_embeds=e2, labels=labels, use_cache=False)
    ref.loss.backward()
    # zero LoRA deltas (B = 0): the same function, computed by the packed kernels on one side and by transformers' bf16 ops
    # on decoded weights on the other
    lo, lr = float(out.loss.detach()), float(ref.loss.detach())
    assert abs(lo - lr) <= 2e-2 * abs(lr), (lo, lr)
    ga, gb_ = e1.grad.float(), e2.grad.float()
    rel = float((ga - gb_).norm() / gb_.norm())
    assert rel < 0.08, rel
    # every adapter factor B received a gradient, nothing else is trainable, and a few optimizer steps lower the loss
    grads = {n: p.grad for n, p in model.named_parameters() if p.requires_grad}
    assert grads and all(".lora_" in n for n in grads)
    assert all(g is not None and float(g.float().abs().max()) > 0 for n, g in grads.items() if ".lora_B" in n), [n for n, g in grads.items() if g is None]
    opt = torch.optim.AdamW([p for p in model.parameters() if p.requires_grad], lr=2e-3)
    first = lo
    for _ in range(8):
        opt.zero_grad(set_to_none=True)
        loss = model(inputs_embeds=embeds, labels=labels, use_cache=False).loss
        loss.backward()
        opt.step()
    assert float(loss.detach()) < first - 0.05, (first, float(loss.detach()))
    # evaluation without labels goes through the head as a layer
    model.eval()
    with torch.no_grad():
        ev = model(inputs_embeds=embeds, use_cache=False, logits_to_keep=1)
    assert ev.logits.shape == (2, 1, 512) and ev.loss is None


@pytest.mark.gpu
def test_patched_routers_match_the_stock_modules(pkg, dev):
    from transformers.models.deepseek_v4.modeling_deepseek_v4 import DeepseekV4TopKRouter
    from transformers.models.qwen3_5_moe.modeling_qwen3_5_moe import Qwen3_5MoeTopKRouter

    torch.manual_seed(5)
    rk = pkg.fast_moe_ranking
    holder = torch.nn.Module()
    holder.config = types.SimpleNamespace(model_type="x", scoring_func="sqrtsoftplus")
    qcfg = types.SimpleNamespace(num_experts_per_tok=8, num_experts=256, hidden_size=512)
    holder.q = Qwen3_5MoeTopKRouter(qcfg).to(dev)
    dcfg = types.SimpleNamespace(num_experts_per_tok=6, num_local_experts=256, hidden_size=512, scoring_func="sqrtsoftplus", routed_scaling_factor=1.5)
    holder.d = DeepseekV4TopKRouter(dcfg).to(dev)
    with torch.no_grad():
        holder.q.weight.normal_(std=0.2)
        holder.d.weight.normal_(std=0.2)
        holder.d.e_score_correction_bias.normal_(std=0.05)
    stock = copy.deepcopy(holder)
    rk.configure_fast_moe_ranking(holder)
    h = torch.randn(4, 100, 512, device=dev)
    for a, b in ((holder.q, stock.q), (holder.d, stock.d)):
        logits, weights, indices = a(h)
        logits0, weights0, indices0 = b(h)
        assert torch.allclose(logits.float(), logits0.float(), atol=1e-4)
        order, order0 = indices.argsort(dim=1), indices0.argsort(dim=1)
        assert torch.equal(indices.gather(1, order), indices0.gather(1, order0))  # the same experts; the stock DeepSeek module leaves them unsorted
        assert torch.allclose(weights.float().gather(1, order), weights0.float().gather(1, order0), rtol=2e-5, atol=1e-6)
    # under autograd the routing weights carry the gradient to the router's input, as the stock modules' do
    probe = torch.randn(400, 8, device=dev)
    for a, b in ((holder.q, stock.q), (holder.d, stock.d)):
        grads = []
        for module in (a, b):
            hr = h.clone().requires_grad_(True)
            _, weights, indices = module(hr)
            order = indices.argsort(dim=1)
            (weights.float().gather(1, order) * probe[:, :weights.shape[1]]).sum().backward()
            grads.append(hr.grad)
        assert float(grads[1].abs().max()) > 0 and float((grads[0] - grads[1]).norm() / grads[1].norm()) < 1e-4
