"""Bit-exact parity of the HIP block decoders with the CPU oracle (ggml dequantize_row_* + RNE bf16)."""

import numpy as np
import pytest
import torch

from helpers import ALL_TYPES, TYPE_NAMES, bf16_bits, make_payload
from oracle import gguf_blocks as gb

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("qt", ALL_TYPES, ids=[TYPE_NAMES[q] for q in ALL_TYPES])
@pytest.mark.parametrize("kind", ["quantized", "random"])
@pytest.mark.parametrize("rows,k", [(1, 256), (37, 2048), (513, 1024)])
def test_dequantize_bit_exact(pkg, dev, qt, kind, rows, k):
    payload = make_payload(1234 + qt + rows, qt, rows, k, kind)
    want32 = gb.dequantize(payload, qt)
    p = torch.from_numpy(payload).to(dev)
    got32 = pkg.gguf.dequantize_gguf_tensor(p, qt, torch.float32)
    got16 = pkg.gguf.dequantize_gguf_tensor(p, qt, torch.bfloat16)
    torch.cuda.synchronize()
    assert np.array_equal(got32.cpu().numpy().view(np.uint32), want32.view(np.uint32)), "fp32 decode differs in some bit"
    assert np.array_equal(bf16_bits(got16), gb.to_bf16_bits(want32)), "bf16 decode differs in some bit"


def test_dequantize_q8_0_odd_block_count(pkg, dev):
    # K = 32 * odd: rows are not 4-byte multiples of the block pair the matmul path uses
    payload = make_payload(7, gb.Q8_0, 5, 32 * 7, "random")
    got = pkg.gguf.dequantize_gguf_tensor(torch.from_numpy(payload).to(dev), gb.Q8_0, torch.float32)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), gb.dequantize(payload, gb.Q8_0).view(np.uint32))


def test_dequantize_expert_stack_and_constant_payload(pkg, dev):
    # the reference's synthetic expert payload: every byte 32 (test_deepseek_v4_moe_lora.py:55-64)
    payload = np.full((2, 256, 66), 32, dtype=np.uint8)
    got = pkg.gguf.dequantize_gguf_tensor(torch.from_numpy(payload).to(dev), gb.IQ2_XXS, torch.bfloat16)
    assert tuple(got.shape) == (2, 256, 256)
    assert np.array_equal(bf16_bits(got), gb.to_bf16_bits(gb.dequantize(payload, gb.IQ2_XXS)))


def test_device_iq2_xxs_quantizer_matches_the_oracle_quantizer_bit_for_bit(pkg, dev):
    """The torch quantizer that manufactures BASELINE's "N(0, 0.02^2), then quantized" IQ2_XXS experts on the device against
    the oracle's, on the same fp32 weights: identical bytes (scale codes, codebook indices, sign bits), including blocks
    with an all-zero group, an all-zero block and a group whose minus signs are odd in number."""
    rng = np.random.default_rng(20260817)
    w = (rng.standard_normal((512, 4096)) * 0.02).astype(np.float32)
    w[0, :256] = 0.0          # a whole block of zeros
    w[1, 32:64] = 0.0         # one group of zeros
    w[2, :8] = np.abs(w[2, :8]) * np.array([-1, 1, 1, 1, 1, 1, 1, 1], dtype=np.float32)  # one minus sign: the weakest weight flips
    w[3] *= 40.0              # large values
    want = gb.quantize(w, gb.IQ2_XXS)
    got = pkg.gguf.quantize_iq2_xxs(torch.from_numpy(w).to(dev), chunk_groups=1000)
    assert got.dtype == torch.uint8 and tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
    # and the table it reads back through the decoder is the oracle's codebook
    assert np.array_equal(pkg.gguf._iq2xxs_grid(dev).cpu().numpy(), gb._GRID_BYTES.astype(np.float64))


def test_dequantize_rejects_bad_operands(pkg, dev):
    p = torch.zeros(4, 144, dtype=torch.uint8, device=dev)
    with pytest.raises(ValueError):
        pkg.gguf.dequantize_gguf_tensor(torch.zeros(4, 82, dtype=torch.uint8, device=dev), 22, torch.bfloat16)  # IQ2_S (82-byte blocks): no decoder here
    with pytest.raises(ValueError):
        pkg.gguf.dequantize_gguf_tensor(p, 2, torch.bfloat16)  # Q4_0: no decoder here
    with pytest.raises(TypeError):
        pkg.gguf.dequantize_gguf_tensor(p, gb.Q4_K, torch.float16)
    with pytest.raises(ValueError):
        pkg.gguf.dequantize_gguf_tensor(p[:, :100], gb.Q4_K, torch.bfloat16)  # not contiguous / not whole blocks
    with pytest.raises(RuntimeError):
        pkg.gguf.dequantize_gguf_tensor(p.cpu(), gb.Q4_K, torch.bfloat16)
