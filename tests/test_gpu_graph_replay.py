"""The expert layer's forward + backward captured into a HIP graph and replayed: every replay, with new inputs copied into
the captured buffers and eager work and synchronisations in between, gives the bits of the eager step."""

import pytest
import torch

import bench

pytestmark = pytest.mark.gpu


def _iq2xxs_workload(pkg, dev, cfg):
    """A small expert layer on IQ2_XXS weights: 64 rows per expert on average, so the forward launches run the kernel for
    small groups and the grad-input launches wide tiles."""
    g = torch.Generator(device=dev).manual_seed(4242)
    e, h, i, r = cfg["experts"], cfg["hidden"], cfg["inter"], cfg["rank"]
    G = pkg.gguf.GGUFQuantizedTensor
    gate = G(pkg.gguf.random_iq2_xxs((e, i, h), g, dev), 16, (e, i, h))
    up = G(pkg.gguf.random_iq2_xxs((e, i, h), g, dev), 16, (e, i, h))
    down = G(pkg.gguf.random_iq2_xxs((e, h, i), g, dev), 16, (e, h, i))
    layer = pkg.fast_moe_lora.FastGGUFMoeLora(pkg.fast_moe_lora.GGUFExperts(gate, up, down), r=r, lora_alpha=cfg["alpha"])
    with torch.no_grad():
        for name, p in layer.named_parameters():
            p.copy_((torch.randn(p.shape, generator=g, device=dev) * (p.shape[-1] ** -0.5 if "lora_A" in name else 0.01)).to(p.dtype))
    x = torch.randn(cfg["tokens"], h, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
    top = torch.topk(torch.randn(cfg["tokens"], e, generator=g, device=dev), cfg["top_k"], dim=-1)
    weights = torch.softmax(top.values, dim=-1).requires_grad_(True)
    dy = torch.randn(cfg["tokens"], h, generator=g, device=dev).to(torch.bfloat16)
    return layer, x, top.indices.clone(), weights, dy


@pytest.fixture
def factor_gradient_overlap(pkg):
    """Sets the library's switch for one test and puts the default (forked factor gradients) back."""
    lib = pkg._lib.load()
    yield lambda on: pkg._lib.check(lib.ggq_set_factor_gradient_overlap(int(on)))
    lib.ggq_set_factor_gradient_overlap(1)


def test_forked_factor_gradients_give_the_bits_of_the_single_stream_order(pkg, dev, factor_gradient_overlap):
    """The backward calls put dA / dB on the library's side stream (forked and joined inside the call); the results must
    not depend on it, eagerly and back to back (the second step reuses the workspace the first one's side work read)."""
    cfg = dict(bench.CFG, tokens=512, experts=32)
    layer, x, idx, weights, dy = bench.build_workload(pkg, dev, cfg)
    params = list(layer.parameters())
    results = {}
    for on in (1, 0, 1):
        factor_gradient_overlap(on)
        for _ in range(3):
            for p in params:
                p.grad = None
            x.grad = weights.grad = None
            out = layer(x, idx, weights)
            out.backward(dy)
        torch.cuda.synchronize()
        got = [out.detach().clone(), x.grad.clone(), weights.grad.clone()] + [p.grad.clone() for p in params]
        if on in results:
            assert all(torch.equal(a, b) for a, b in zip(got, results[on]))
        results[on] = got
    assert all(torch.equal(a, b) for a, b in zip(results[0], results[1]))
    assert all(float(p.grad.float().abs().sum()) > 0 for p in params)


@pytest.mark.parametrize("overlap", [1, 0])
@pytest.mark.parametrize("kind", ["q4k", "iq2xxs"])
def test_expert_layer_step_replays_from_a_hip_graph(pkg, dev, kind, overlap, factor_gradient_overlap):
    factor_gradient_overlap(overlap)  # 1: the capture holds the fork and join of the factor gradients as graph edges
    if kind == "q4k":
        cfg = dict(bench.CFG, tokens=512, experts=32)
        layer, x, idx, weights, dy = bench.build_workload(pkg, dev, cfg)
    else:
        cfg = dict(bench.CFG, tokens=256, experts=16, hidden=512, inter=256, top_k=4)
        layer, x, idx, weights, dy = _iq2xxs_workload(pkg, dev, cfg)
    params = list(layer.parameters())
    out_static = None

    def step():
        for p in params:
            p.grad = None
        x.grad = None
        weights.grad = None
        out = layer(x, idx, weights)
        out.backward(dy)
        return out

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = step()
    torch.cuda.synchronize()
    captured = [out_static, x.grad, weights.grad] + [p.grad for p in params]

    gen = torch.Generator(device=dev).manual_seed(99)
    for trial in range(3):
        new_x = torch.randn(x.shape, generator=gen, device=dev).to(torch.bfloat16)
        new_dy = torch.randn(dy.shape, generator=gen, device=dev).to(torch.bfloat16)
        new_top = torch.topk(torch.randn(cfg["tokens"], cfg["experts"], generator=gen, device=dev), cfg["top_k"], dim=-1)
        with torch.no_grad():
            x.copy_(new_x)
            dy.copy_(new_dy)
            idx.copy_(new_top.indices)
            weights.copy_(torch.softmax(new_top.values, dim=-1))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        # the same step eagerly, on fresh tensors (also the eager work between two replays)
        xe = new_x.clone().requires_grad_(True)
        we = torch.softmax(new_top.values, dim=-1).requires_grad_(True)
        saved = [p.grad.clone() for p in params]
        for p in params:
            p.grad = None
        oe = layer(xe, new_top.indices, we)
        oe.backward(new_dy)
        torch.cuda.synchronize()
        want = [oe.detach(), xe.grad, we.grad] + [p.grad.clone() for p in params]
        for p, g in zip(params, saved):
            p.grad = g  # hand the captured gradient buffers back to the graph
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (trial, i)
