"""Writes the golden fixtures of the parity tests with this repository's own oracle.

    python tests/golden/make_golden.py

The reference holds no golden vectors for this path (its tests check invariants at run time),
so these fixtures freeze the oracle's answers on small seeded inputs: any later change of the
oracle, the C restatement or the kernels shows up as a diff against committed data.
Inputs and expected outputs only; nothing here is derived from running the reference.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path[:0] = [str(HERE.parent.parent / "oracle"), str(HERE.parent)]

import a2a_oracle as oracle  # noqa: E402
from a2a_cases import Case, bf16_codes, make_world  # noqa: E402
from a2a_harness import rows_needed, run_oracle  # noqa: E402

CASES = [
    Case("golden_small", 12, 256, 8, 2, 2, 4242, routing="uniform"),
    Case("golden_padded_two_nodes", 10, 128, 12, 4, 3, 4243, routing="zipf", zipf_s=1.1, expert_padding=4,
         node_size=2, outliers=True),
]


def build(case: Case, sources: str):
    world = make_world(case, sources)
    rows = rows_needed(case, world)
    res = run_oracle(case, world, rows)
    data = {"rows": np.int64(rows)}
    for r, rd in enumerate(world):
        data[f"x_{r}"] = bf16_codes(rd.x)
        data[f"indices_{r}"] = rd.indices.numpy()
        data[f"weights_{r}"] = rd.weights.numpy()
        data[f"num_tokens_{r}"] = res.num_tokens[r]
        data[f"out_x_{r}"] = res.x[r]
        data[f"out_scale_{r}"] = res.x_scale[r]
        data[f"written_{r}"] = res.written[r]
        data[f"slots_{r}"] = res.slots[r]
        data[f"expert_y_{r}"] = res.expert_y[r]
        data[f"out_tokens_{r}"] = res.out_tokens[r]
    return data


def main() -> None:
    for case in CASES:
        for sources in ("all", "ragged"):
            path = HERE / f"{case.name}_{sources}.npz"
            np.savez_compressed(path, **build(case, sources))
            print(path.name, path.stat().st_size, "bytes")
    # known answers of the fp8 encoder: value -> code
    values = np.array([0.0, -0.0, 2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10, 2.0 ** -6, 0.3, 1.0, 1.0625, 1.1875,
                       240.0, 447.0, 448.0, 464.0, -448.0, -17.5], dtype=np.float32)
    np.savez_compressed(HERE / "e4m3fn_known_answers.npz", values=values, codes=oracle.e4m3fn_encode(values))


if __name__ == "__main__":
    main()
