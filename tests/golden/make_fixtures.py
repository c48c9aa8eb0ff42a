"""Writes tests/golden/fixtures.json: small input/output vectors the CPU and GPU tests replay.

Two kinds.  ``known_answers`` are the literal cases the reference's own tests hold (cited there), typed in by hand:
they pin the oracle.  ``regression`` vectors are computed here by the oracle from seeded inputs after it has passed
its pins: they do not pin anything by themselves, they freeze today's answers so that a later change to the oracle or
to a kernel that moves a bit is seen.  Run from the repository root:  python tests/golden/make_fixtures.py
"""

import json
import pathlib
import sys

import numpy as np

sys.path.insert(0, str(pathlib.Path(__file__).resolve().parents[2]))
from oracle import affine, exl3, routing  # noqa: E402

OUT = pathlib.Path(__file__).with_name("fixtures.json")


def main() -> None:
    rng = np.random.default_rng(20240607)
    known = {
        # tests/test_exl3_format.py:129-134
        "packed_signs": {"words": [0b1000000000000101, 0], "negative_at": [0, 2, 15], "length": 32},
        # tests/cuda/test_experts.py:91-104
        "plan_one_expert": {"rows": 37, "expert": 4, "experts": 9, "tile": 16, "item_counts": [16, 16, 5]},
        # tests/cuda/test_nemotron_kernels.py:71-80
        "ties": {"experts": 128, "top_k": 6, "ids": [0, 1, 2, 3, 4, 5], "weight": float(np.float32(1 / 6))},
        # families/qwen3_5/cuda/qmm.py:132-149: element 8 w + i is bits [4 i, 4 i + 4) of word w
        "nibble_order": {"word": 0x76543210, "codes": [0, 1, 2, 3, 4, 5, 6, 7]},
    }
    words = rng.integers(0, 2 ** 32, size=(2, 16), dtype=np.uint64).astype(np.uint32)
    scales = affine.bf16(rng.uniform(0.002, 0.02, size=(2, 2)).astype(np.float32))
    biases = affine.bf16((-8 * scales).astype(np.float32))
    x = affine.bf16(rng.standard_normal((3, 128)).astype(np.float32))
    logits = rng.standard_normal((4, 17)).astype(np.float32)
    picks, wts = routing.topk_rows(logits, 16, 3, shared=True)
    items, members, distinct = routing.plan(picks, 17, 16)
    reg = {
        "affine": {"words": words.tolist(), "scales_bits": affine.bf16_bits(scales).tolist(),
                   "biases_bits": affine.bf16_bits(biases).tolist(), "gs": 64, "x_bits": affine.bf16_bits(x).tolist(),
                   "y_bits": affine.bf16_bits(affine.linear(x, words, scales, biases, 64)).tolist()},
        "routing": {"logits": logits.tolist(), "experts": 16, "top_k": 3, "picks": picks.tolist(),
                    "weights": wts.astype(np.float64).tolist(), "items": items.tolist(), "members": members.tolist(),
                    "distinct": int(distinct)},
        "exl3": {},
    }
    for cb, bits in (("3inst", 3), ("mcg", 4), ("mul1", 2.5)):
        trellis = rng.integers(-2 ** 15, 2 ** 15, size=(1, 1, int(16 * bits))).astype(np.int16)
        w = exl3.unpack(trellis, bits, cb)
        reg["exl3"][cb] = {"bits": bits, "trellis": trellis.reshape(-1).tolist(),
                           "values_fp16_bits": w.view(np.uint16).reshape(-1).tolist()}
    OUT.write_text(json.dumps({"known_answers": known, "regression": reg}, indent=1))
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
