"""Token rows with NaN, infinities and the largest bf16 value inside otherwise ordinary groups,
and what the quantiser has to make of them, derived by hand from its rule (not by running it)."""

from __future__ import annotations

from typing import Dict, List, Tuple

import numpy as np
import torch

BF16_MAX = 0x7F7F        # 3.3895e38
POS_INF, NEG_INF = 0x7F80, 0xFF80
NAN_POS, NAN_NEG, NAN_PAYLOAD = 0x7FC0, 0xFFC0, 0x7F81


def bad_rows(hidden_dim: int = 1024, seed: int = 7) -> Tuple[np.ndarray, Dict[Tuple[int, int], str]]:
    """bf16 bit patterns [T, H] and {(row, group): kind}, kind = "nan" | "inf" | "max" for the groups
    that hold a special value; every other group is ordinary."""
    assert hidden_dim % 128 == 0 and hidden_dim >= 1024
    T = 10
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn((T, hidden_dim), generator=gen).to(torch.bfloat16)
    x[:, 5] = -0.0                                   # a negative zero in group 0 of every row
    bits = x.view(torch.int16).numpy().view(np.uint16).copy()
    kinds: Dict[Tuple[int, int], str] = {}

    def put(row: int, col: int, pattern: int, kind: str) -> None:
        bits[row, col] = pattern
        key = (row, col // 128)
        kinds[key] = "nan" if "nan" in (kind, kinds.get(key)) else kind

    put(1, 128 + 37, NAN_POS, "nan")                 # one NaN in an ordinary group
    put(2, 256 + 3, POS_INF, "inf")                  # one +inf
    put(3, 64, NEG_INF, "inf")                       # one -inf, same group as the negative zero
    put(4, 384 + 10, NAN_NEG, "nan")                 # NaN and infinity in one group
    put(4, 384 + 90, POS_INF, "inf")
    put(5, 384 + 77, BF16_MAX, "max")                # the largest finite value, either sign
    put(5, 512 + 1, BF16_MAX | 0x8000, "max")
    put(6, 640 + 15, NAN_PAYLOAD, "nan")             # another NaN pattern, at the edge of a 16-element piece
    put(6, 640 + 16, NAN_NEG, "nan")
    put(7, 127, POS_INF, "inf")                      # last element of a group / first of the next
    put(7, 128, NEG_INF, "inf")
    put(7, 128 + 64, POS_INF, "inf")
    for c in range(128):                             # a whole group of NaN, a whole group of infinities
        put(8, 768 + c, NAN_POS if c % 2 else NAN_NEG, "nan")
        put(9, 896 + c, POS_INF if c % 3 else NEG_INF, "inf")
    return bits, kinds


def expected_special_groups(bits: np.ndarray, kinds: Dict[Tuple[int, int], str]) -> List[Tuple[int, int, np.ndarray, int]]:
    """[(row, group, codes[128], scale bits)] for the "nan" and "inf" groups, written out from the rule:
    a NaN poisons the group (scale NaN, every code 0x7F); an infinity makes the scale +inf, an
    infinite value the code 0x7F and a finite one a zero with its sign."""
    out = []
    for (row, group), kind in sorted(kinds.items()):
        g = bits[row, group * 128:(group + 1) * 128]
        if kind == "nan":
            out.append((row, group, np.full(128, 0x7F, dtype=np.uint8), 0x7FC00000))
        elif kind == "inf":
            codes = np.where((g & 0x7FFF) == 0x7F80, 0x7F, (g >> 8) & 0x80).astype(np.uint8)
            out.append((row, group, codes, 0x7F800000))
    return out
