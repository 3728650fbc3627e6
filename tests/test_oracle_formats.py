"""Pins the number formats of the oracle (numpy and C) against torch's casts and
against the mathematical definition (nearest representable value, ties to even)."""

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
import c_oracle


def _torch_e4m3(f: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(f, dtype=np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def _all_bf16_values():
    codes = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    return oracle.bf16_to_f32(codes)


def test_decode_table_is_the_ocp_e4m3fn_grid():
    codes = np.arange(256, dtype=np.uint8)
    mine = oracle.e4m3fn_decode(codes)
    ref = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    finite = ~np.isnan(ref)
    assert np.array_equal(np.isnan(mine), np.isnan(ref))
    np.testing.assert_array_equal(mine[finite], ref[finite])
    assert mine[0x7E] == 448.0 and mine[0x01] == 2.0 ** -9 and mine[0x08] == 2.0 ** -6
    for c in range(256):
        v = c_oracle.lib().oracle_e4m3fn_decode(c)
        assert (np.isnan(v) and np.isnan(mine[c])) or v == mine[c]


def test_encode_matches_torch_on_every_bf16_value():
    f = _all_bf16_values()
    finite = np.isfinite(f)
    np.testing.assert_array_equal(oracle.e4m3fn_encode(f[finite]), _torch_e4m3(f[finite]))
    np.testing.assert_array_equal(c_oracle.encode(f[finite]), _torch_e4m3(f[finite]))
    # NaN and infinities become the NaN code, sign kept
    bad = oracle.e4m3fn_encode(f[~finite])
    assert ((bad & 0x7F) == 0x7F).all()
    assert ((c_oracle.encode(f[~finite]) & 0x7F) == 0x7F).all()


def test_encode_matches_torch_on_random_floats_and_scaled_bf16():
    rng = np.random.default_rng(7)
    f = (rng.standard_normal(1_000_000) * np.exp(rng.uniform(-14, 7, 1_000_000))).astype(np.float32)
    np.testing.assert_array_equal(oracle.e4m3fn_encode(f), _torch_e4m3(f))
    np.testing.assert_array_equal(c_oracle.encode(f), _torch_e4m3(f))
    # every bf16 value times a grid of scales, as the quantiser produces them
    x = _all_bf16_values()
    x = x[np.isfinite(x)]
    for inv in (np.float32(448.0) / np.float32(a) for a in (1e-4, 0.37, 1.0, 3.1875, 50.0, 448.0, 6e4)):
        y = np.clip((x * inv).astype(np.float32), -448, 448)
        np.testing.assert_array_equal(oracle.e4m3fn_encode(y), _torch_e4m3(y))
        np.testing.assert_array_equal(c_oracle.encode(y), _torch_e4m3(y))


def test_encode_is_nearest_value_with_ties_to_even():
    """Brute force: the encoded value is a nearest grid point; at an exact tie the code is even."""
    grid_codes = np.array([c for c in range(0x7F)], dtype=np.uint8)       # non-negative finite codes
    grid = oracle.e4m3fn_decode(grid_codes).astype(np.float64)
    rng = np.random.default_rng(3)
    samples = np.concatenate([
        rng.uniform(0, 460, 20000), rng.uniform(0, 2.0 ** -5, 20000), grid,
        (grid[:-1] + grid[1:]) / 2,                                          # exact midpoints
    ]).astype(np.float32)
    enc = oracle.e4m3fn_encode(samples)
    for x, c in zip(samples.astype(np.float64), enc):
        d = np.abs(grid - x)
        best = d.min()
        assert abs(grid[c] - x) == best, (x, c)
        ties = np.flatnonzero(d == best)
        if len(ties) == 2:
            assert c % 2 == 0, (x, c)
    neg = oracle.e4m3fn_encode(-samples)
    np.testing.assert_array_equal(neg & 0x7F, enc & 0x7F)
    assert ((neg[samples > 2.0 ** -10] & 0x80) == 0x80).all()


@pytest.mark.parametrize("value,code", [
    (448.0, 0x7E), (464.0, 0x7E), (465.0, 0x7F), (500.0, 0x7F), (2.0 ** -9, 0x01), (2.0 ** -10, 0x00),
    (3 * 2.0 ** -10, 0x02), (2.0 ** -6, 0x08), (0.0, 0x00), (-0.0, 0x80), (-448.0, 0xFE), (1.0, 0x38),
])
def test_encode_known_answers(value, code):
    assert int(oracle.e4m3fn_encode(np.array([value], np.float32))[0]) == code
    assert int(c_oracle.lib().oracle_e4m3fn_encode(value)) == code


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(11)
    f = (rng.standard_normal(500_000) * np.exp(rng.uniform(-30, 30, 500_000))).astype(np.float32)
    f = np.concatenate([f, np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    ref = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_bf16(f), ref)
    np.testing.assert_array_equal(oracle.bf16_to_f32(ref), torch.from_numpy(ref.view(np.int16).copy()).view(torch.bfloat16).float().numpy())
    # ties: 1 + 2^-8 is halfway between bf16(1.0) and the next value -> even (1.0)
    assert oracle.f32_to_bf16(np.array([1.00390625], np.float32))[0] == 0x3F80
    assert oracle.f32_to_bf16(np.array([1.01171875], np.float32))[0] == 0x3F82
    assert np.isnan(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([np.nan], np.float32))))[0]


def test_scalar_type_tags_follow_the_reference_order():
    # rust/torch-lib/src/lib.rs:31-49
    assert oracle.SCALAR_TYPES[:3] == ("BOOL", "I8", "U8")
    assert oracle.SCALAR_TYPE["F8_E4M3"] == 9 and oracle.SCALAR_TYPE["F8_E5M2"] == 10
    assert oracle.SCALAR_TYPE["F16"] == 11 and oracle.SCALAR_TYPE["BF16"] == 12
    assert oracle.SCALAR_TYPE["F32"] == 13 and oracle.SCALAR_TYPE["F64"] == 14
    from pplx_garden_amd.native.p2p_all_to_all import SCALAR_TYPE
    assert SCALAR_TYPE[torch.float8_e4m3fn] == 9 and SCALAR_TYPE[torch.bfloat16] == 12
    assert SCALAR_TYPE[torch.float16] == 11 and SCALAR_TYPE[torch.float32] == 13
    assert SCALAR_TYPE[torch.uint32] == 6 and SCALAR_TYPE[torch.int32] == 5
