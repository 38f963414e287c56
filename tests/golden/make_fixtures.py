"""Writes the small golden fixtures in this folder from the CPU oracle (run from the repo root:
``python tests/golden/make_fixtures.py``).  The reference stores no golden vectors for this path and
its decoders live in packages that are not installed, so these files freeze the oracle's answers --
which tests/test_oracle_blocks.py pins by hand-computed blocks -- for the GPU parity tests and as a
regression guard: they are data (packed bytes, expected values, index arrays), not code."""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from oracle import gguf_blocks as gb  # noqa: E402
from oracle import routing as rt  # noqa: E402
from helpers import make_payload  # noqa: E402

HERE = Path(__file__).resolve().parent


def main() -> None:
    out = {}
    for qt, name in ((gb.Q8_0, "q8_0"), (gb.Q2_K, "q2_k"), (gb.Q3_K, "q3_k"), (gb.Q4_K, "q4_k"), (gb.Q5_K, "q5_k"), (gb.Q6_K, "q6_k"),
                     (gb.IQ2_XXS, "iq2_xxs")):
        payload = np.concatenate([make_payload(100 + qt, qt, 3, 512, "quantized"), make_payload(200 + qt, qt, 3, 512, "random")])
        out[f"{name}_payload"] = payload
        out[f"{name}_f32"] = gb.dequantize(payload, qt)
        out[f"{name}_bf16_bits"] = gb.to_bf16_bits(gb.dequantize(payload, qt))
    np.savez_compressed(HERE / "block_decode.npz", **out)

    gen = torch.Generator().manual_seed(19260817)
    ids = torch.randint(0, 11, (37, 4), generator=gen)
    sorted_ids, perm, inv = rt.plan(ids)
    counts = rt.expert_counts(ids, 11)
    active, ends = rt.active_offsets(counts)
    np.savez_compressed(HERE / "routing_plan.npz", top_k_index=ids.numpy(), sorted_ids=sorted_ids.numpy(), permutation=perm.numpy(),
                        inverse=inv.numpy(), counts=counts.numpy(), active_ids=active.numpy(), active_end_offsets=ends.numpy())


if __name__ == "__main__":
    main()
