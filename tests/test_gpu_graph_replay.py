"""The expert layer's forward + backward captured into a HIP graph and replayed: every replay, with new inputs copied into
the captured buffers and eager work and synchronisations in between, gives the bits of the eager step."""

import pytest
import torch

import bench

pytestmark = pytest.mark.gpu


def test_expert_layer_step_replays_from_a_hip_graph(pkg, dev):
    cfg = dict(bench.CFG, tokens=512, experts=32)
    layer, x, idx, weights, dy = bench.build_workload(pkg, dev, cfg)
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
