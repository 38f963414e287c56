"""The committed fixtures under tests/golden/ against the numpy oracle, the independent C
restatement and (on the GPU box) the HIP kernels."""

from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gguf_blocks as gb
from oracle import routing as rt

GOLDEN = Path(__file__).resolve().parent / "golden"
TYPES = ((gb.Q8_0, "q8_0"), (gb.Q2_K, "q2_k"), (gb.Q3_K, "q3_k"), (gb.Q4_K, "q4_k"), (gb.Q5_K, "q5_k"), (gb.Q6_K, "q6_k"), (gb.IQ2_XXS, "iq2_xxs"))


@pytest.fixture(scope="module")
def blocks():
    return np.load(GOLDEN / "block_decode.npz")


@pytest.fixture(scope="module")
def plan():
    return np.load(GOLDEN / "routing_plan.npz")


@pytest.mark.parametrize("qt,name", TYPES)
def test_oracles_reproduce_the_block_fixture(blocks, qt, name):
    from oracle import c_oracle

    payload = blocks[f"{name}_payload"]
    assert payload.dtype == np.uint8 and payload.shape == (6, gb.row_bytes(qt, 512))
    want = blocks[f"{name}_f32"]
    assert np.array_equal(gb.dequantize(payload, qt).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(c_oracle.dequantize(payload, qt).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(gb.to_bf16_bits(want), blocks[f"{name}_bf16_bits"])


def test_oracle_reproduces_the_routing_fixture(plan):
    ids = torch.from_numpy(plan["top_k_index"])
    sorted_ids, perm, inv = rt.plan(ids)
    assert np.array_equal(sorted_ids.numpy(), plan["sorted_ids"])
    assert np.array_equal(perm.numpy(), plan["permutation"])
    assert np.array_equal(inv.numpy(), plan["inverse"])
    counts = rt.expert_counts(ids, 11)
    assert np.array_equal(counts.numpy(), plan["counts"])
    active, ends = rt.active_offsets(counts)
    assert np.array_equal(active.numpy(), plan["active_ids"]) and np.array_equal(ends.numpy(), plan["active_end_offsets"])


@pytest.mark.gpu
@pytest.mark.parametrize("qt,name", TYPES)
def test_hip_decoders_reproduce_the_block_fixture(pkg, dev, blocks, qt, name):
    payload = torch.from_numpy(blocks[f"{name}_payload"]).to(dev)
    f32 = pkg.gguf.dequantize_gguf_tensor(payload, qt, torch.float32)
    assert np.array_equal(f32.cpu().numpy().view(np.uint32), blocks[f"{name}_f32"].view(np.uint32))
    bf = pkg.gguf.dequantize_gguf_tensor(payload, qt, torch.bfloat16)
    assert np.array_equal(bf.view(torch.int16).cpu().numpy().view(np.uint16), blocks[f"{name}_bf16_bits"])


@pytest.mark.gpu
def test_hip_route_plan_reproduces_the_routing_fixture(pkg, dev, plan):
    ids = torch.from_numpy(plan["top_k_index"]).to(dev)
    sorted_ids, perm, inv, counts, ends, active_ids, active_ends, status = pkg.fast_moe_routing.build_route_plan(ids, 11)
    assert np.array_equal(sorted_ids.cpu().numpy(), plan["sorted_ids"])
    assert np.array_equal(perm.cpu().numpy(), plan["permutation"])
    assert np.array_equal(inv.cpu().numpy(), plan["inverse"])
    assert np.array_equal(counts.cpu().numpy(), plan["counts"])
    n_active = int(status[0])
    assert n_active == len(plan["active_ids"]) and int(status[1]) == 0
    assert np.array_equal(active_ids[:n_active].cpu().numpy(), plan["active_ids"])
    assert np.array_equal(active_ends[:n_active].cpu().numpy(), plan["active_end_offsets"])
    assert np.array_equal(ends.cpu().numpy(), np.cumsum(plan["counts"]).astype(np.int32))
