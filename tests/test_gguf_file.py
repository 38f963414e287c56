"""GGUF container reader: a file assembled byte by byte from the published layout (independent of the package's own
writer), the writer's round trip, malformed files, and - on the GPU - packed tensors read from a file against the
decoder oracle."""

import struct

import numpy as np
import pytest
import torch

from helpers import ALL_TYPES, TYPE_NAMES, make_payload
from oracle import gguf_blocks as gb


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _hand_made_file(path, q8_rows, f32_vals):
    """Version 3, alignment 64: three metadata entries, a Q8_0 tensor [3, 64] and an F32 tensor [5]."""
    head = struct.pack("<IIQQ", 0x46554747, 3, 2, 4)
    head += _s("general.architecture") + struct.pack("<I", 8) + _s("qwen35moe")
    head += _s("general.alignment") + struct.pack("<II", 4, 64)
    head += _s("qwen35moe.expert_count") + struct.pack("<IQ", 10, 256)
    head += _s("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, 3) + _s("a") + _s("bc") + _s("")
    # tensor table: name, n_dims, ne (contiguous dimension first), type, offset
    head += _s("blk.0.attn_gate.weight") + struct.pack("<IQQIQ", 2, 64, 3, 8, 0)
    head += _s("blk.0.attn_norm.weight") + struct.pack("<IQIQ", 1, 5, 0, 256)     # 3 rows x 68 bytes = 204 -> next multiple of 64
    data_start = (len(head) + 63) // 64 * 64
    blob = head + b"\0" * (data_start - len(head)) + q8_rows.tobytes() + b"\0" * (256 - 204) + f32_vals.tobytes()
    path.write_bytes(blob)
    return data_start


def test_reads_a_hand_assembled_file(pkg, tmp_path):
    gf = pkg.gguf_file
    q8 = make_payload(5, gb.Q8_0, 3, 64)
    f32 = np.array([1.0, -2.5, 0.0, 3.25, 1e-3], dtype="<f4")
    path = tmp_path / "hand.gguf"
    data_start = _hand_made_file(path, q8, f32)
    with gf.GGUFReader(path) as r:
        assert r.version == 3 and r.alignment == 64 and r.data_offset == data_start
        assert r.fields["general.architecture"] == "qwen35moe"
        assert r.fields["qwen35moe.expert_count"] == 256
        assert r.fields["tokenizer.ggml.tokens"] == ["a", "bc", ""]
        assert [t.name for t in r.tensors] == ["blk.0.attn_gate.weight", "blk.0.attn_norm.weight"]
        t = r.get_tensor("blk.0.attn_gate.weight")
        assert (t.tensor_type, t.shape, t.logical_shape, t.n_elements, t.n_bytes) == (8, (64, 3), (3, 64), 192, 204)
        assert t.data.shape == (3, 68) and np.array_equal(t.data, q8)
        n = r.get_tensor("blk.0.attn_norm.weight")
        assert n.data_offset == data_start + 256 and np.array_equal(n.data, f32)
        with pytest.raises(KeyError):
            r.get_tensor("missing")
        with pytest.raises(ValueError, match="block-quantized"):
            r.plain("blk.0.attn_gate.weight", device="cpu")
        assert torch.equal(r.plain("blk.0.attn_norm.weight", device="cpu"), torch.from_numpy(f32.copy()))


def test_writer_round_trip_every_block_type_and_metadata_kind(pkg, tmp_path):
    gf = pkg.gguf_file
    tensors = []
    for i, qt in enumerate(ALL_TYPES):
        k = 512
        tensors.append((f"blk.{i}.ffn_gate_exps.weight", qt, (4, 6, k), make_payload(20 + i, qt, 24, k).reshape(4, 6, -1)))
    bf = (np.arange(24, dtype=np.uint16) * 257).reshape(2, 12)
    tensors.append(("output_norm.weight", gf.BF16, (2, 12), bf))
    tensors.append(("scalar_like", gf.F16, (7,), np.linspace(-1, 1, 7).astype("<f2")))
    meta = {"general.name": "synthetic", "a.flag": True, "a.count": 7, "a.big": 2 ** 40, "a.huge": 2 ** 63 + 5, "a.scale": 0.5,
            "a.u8": np.uint8(200), "a.f64": np.float64(1e-300), "a.ids": [3, 1, 2], "a.names": ["x", "yz"], "a.nested": [[1, 2], [3]]}
    for alignment in (32, 128):
        path = tmp_path / f"rt{alignment}.gguf"
        gf.write_gguf(path, meta, tensors, alignment=alignment)
        with gf.GGUFReader(path) as r:
            assert r.alignment == alignment
            got = {k: v for k, v in r.fields.items() if k != "general.alignment"}
            assert got == {**meta, "a.u8": 200, "a.f64": 1e-300}
            for (name, qt, logical, data), t in zip(tensors, r.tensors):
                assert (t.name, t.tensor_type, t.logical_shape) == (name, qt, logical)
                assert t.data_offset % alignment == 0
                assert np.array_equal(t.data, data), name
            p = r.packed("blk.2.ffn_gate_exps.weight", device="cpu", rows=slice(1, 3))
            assert isinstance(p, pkg.gguf.GGUFQuantizedTensor) and p.logical_shape == (2, 6, 512) and p.quant_type == ALL_TYPES[2]
            assert np.array_equal(p.as_subclass(torch.Tensor).numpy(), tensors[2][3][1:3])
            assert r.plain("output_norm.weight", device="cpu").dtype == torch.bfloat16
            assert np.array_equal(r.plain("output_norm.weight", device="cpu").view(torch.int16).numpy().view(np.uint16), bf)
            with pytest.raises(ValueError, match="no native kernels"):
                r.packed("output_norm.weight", device="cpu")


def test_malformed_files_are_refused(pkg, tmp_path):
    gf = pkg.gguf_file
    good = tmp_path / "good.gguf"
    gf.write_gguf(good, {"k": 1}, [("w", gb.Q4_K, (2, 256), make_payload(1, gb.Q4_K, 2, 256))])
    blob = good.read_bytes()
    cases = {
        "empty": b"",
        "magic": b"GGML" + blob[4:],
        "version": blob[:4] + struct.pack("<I", 1) + blob[8:],
        "truncated table": blob[:40],
        "truncated data": blob[:-10],
    }
    for name, data in cases.items():
        path = tmp_path / f"{name.replace(' ', '_')}.gguf"
        path.write_bytes(data)
        with pytest.raises(ValueError):
            gf.GGUFReader(path)
    with pytest.raises(ValueError, match="do not hold"):
        gf.write_gguf(tmp_path / "bad.gguf", {}, [("w", gb.Q4_K, (2, 256), np.zeros(100, dtype=np.uint8))])
    with pytest.raises(ValueError, match="unknown GGML type"):
        gf.block_geometry(77)


@pytest.mark.gpu
@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
def test_packed_tensor_from_file_decodes_to_the_oracle(pkg, dev, qt, tmp_path):
    gf = pkg.gguf_file
    payload = make_payload(77, qt, 3 * 5, 1024, kind="random").reshape(3, 5, -1)
    path = tmp_path / "experts.gguf"
    gf.write_gguf(path, {"general.architecture": "synthetic"}, [("pad", gf.F32, (3,), np.zeros(3, "<f4")), ("blk.0.ffn_down_exps.weight", qt, (3, 5, 1024), payload)])
    with gf.GGUFReader(path) as r:
        w = r.packed("blk.0.ffn_down_exps.weight", device=dev)
    assert w.quant_type == qt and w.logical_shape == (3, 5, 1024) and w.device.type == "cuda"
    got = pkg.gguf.dequantize_gguf_tensor(w, qt, torch.float32)
    want = gb.dequantize(payload, qt)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
