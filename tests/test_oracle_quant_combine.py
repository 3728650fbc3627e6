"""Pins the quantiser and the combine of the oracle against torch operations, closed forms
and the round-trip identity of the reference's test; numpy against the C restatement."""

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
import c_oracle
from a2a_cases import C0, C1, C2, bf16_codes, make_rank, make_world
from a2a_harness import rows_needed, run_oracle


def _torch_quantize(x_bf16: torch.Tensor):
    """The rule written with torch library routines only."""
    T, H = x_bf16.shape
    g = x_bf16.to(torch.float32).view(T, H // 128, 128)
    amax = g.abs().amax(dim=2).clamp_min(1e-4)
    inv = torch.tensor(448.0) / amax
    q = (g * inv[:, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(T, H).view(torch.uint8).numpy(), (amax / 448.0).numpy()


@pytest.mark.parametrize("case", [C0, C2], ids=lambda c: c.name)
def test_quantize_matches_torch_and_c(case):
    rd = make_rank(case, 0, 48)
    q, s = oracle.quantize_block128(bf16_codes(rd.x))
    tq, ts = _torch_quantize(rd.x)
    np.testing.assert_array_equal(q, tq)
    np.testing.assert_array_equal(s.view(np.uint32), ts.view(np.uint32))
    cq, cs = c_oracle.quantize(bf16_codes(rd.x))
    np.testing.assert_array_equal(cq, q)
    np.testing.assert_array_equal(cs.view(np.uint32), s.view(np.uint32))


def test_quantize_special_groups():
    H = 512
    x = torch.zeros((1, H), dtype=torch.float32)
    x[0, 128:256] = torch.linspace(-3, 3, 128)              # ordinary group
    x[0, 256] = 2.0 ** -20                                  # tiny group: amax clamps to 1e-4
    x[0, 384:512] = torch.randn(128, generator=torch.Generator().manual_seed(1))
    x[0, 400] = 3000.0                                      # outlier dominates its group
    xb = x.to(torch.bfloat16)
    q, s = oracle.quantize_block128(bf16_codes(xb))
    assert (q[0, :128] == 0).all() and s[0, 0] == np.float32(1e-4) / np.float32(448)
    assert s[0, 2] == np.float32(1e-4) / np.float32(448)
    # the group maximum maps to +-448 exactly
    assert q[0, 128] == 0xFE and q[0, 255] == 0x7E
    assert q[0, 400] == 0x7E and s[0, 3] == np.float32(xb[0, 400].float().item()) / np.float32(448)
    cq, cs = c_oracle.quantize(bf16_codes(xb))
    np.testing.assert_array_equal(cq, q)
    np.testing.assert_array_equal(cs, s)


def test_quantize_non_finite_groups():
    """NaN, infinities and the largest bf16 value inside ordinary rows: the hand-written
    expectation, torch's library operations (NaN spelled one way), and the C restatement."""
    from a2a_nonfinite import BF16_MAX, bad_rows, expected_special_groups

    bits, kinds = bad_rows()
    q, s = oracle.quantize_block128(bits)
    sb = s.view(np.uint32)
    special = expected_special_groups(bits, kinds)
    assert len(special) == len([k for k in kinds.values() if k != "max"])
    for row, group, codes, scale_bits in special:
        np.testing.assert_array_equal(q[row, group * 128:(group + 1) * 128], codes, err_msg=f"row {row} group {group}")
        assert sb[row, group] == scale_bits, (row, group, hex(sb[row, group]))
    # every other group is what it is without the special value next door: groups are independent
    clean = bits.copy()
    for (row, group), kind in kinds.items():
        if kind != "max":
            clean[row, group * 128:(group + 1) * 128] = 0
    cq, cs = oracle.quantize_block128(clean)
    for row in range(bits.shape[0]):
        for group in range(bits.shape[1] // 128):
            if kinds.get((row, group)) in ("nan", "inf"):
                continue
            np.testing.assert_array_equal(q[row, group * 128:(group + 1) * 128], cq[row, group * 128:(group + 1) * 128])
            assert sb[row, group] == cs.view(np.uint32)[row, group]
    assert np.isfinite(cs).all() and not ((cq & 0x7F) == 0x7F).any()
    # the largest finite bf16 value is an ordinary maximum: +-448 exactly, scale = value / 448
    big = np.float32(oracle.bf16_to_f32(np.array([BF16_MAX], dtype=np.uint16))[0])
    assert q[5, 384 + 77] == 0x7E and q[5, 512 + 1] == 0xFE
    assert s[5, 3] == big / np.float32(448) and s[5, 4] == big / np.float32(448)
    # a poisoned group dequantises to NaN throughout: the bad activation stays visible
    deq = oracle.dequantize_block128(q, s)
    for row, group, _, _ in special:
        assert np.isnan(deq[row, group * 128:(group + 1) * 128]).all()
    # torch's library operations on the same rows, NaN spelled one way
    xb = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    tq, ts = _torch_quantize(xb)
    tq = np.where((tq & 0x7F) == 0x7F, 0x7F, tq).astype(np.uint8)
    tsb = np.where(np.isnan(ts), 0x7FC00000, ts.view(np.uint32)).astype(np.uint32)
    np.testing.assert_array_equal(q, tq)
    np.testing.assert_array_equal(sb, tsb)
    # the C restatement and the torch twin of the benchmark's CPU baseline
    c_q, c_s = c_oracle.quantize(bits)
    np.testing.assert_array_equal(c_q, q)
    np.testing.assert_array_equal(c_s.view(np.uint32), sb)
    import a2a_oracle_torch
    t2q, t2s = a2a_oracle_torch.quantize_block128(xb)
    np.testing.assert_array_equal(t2q.numpy(), q)
    np.testing.assert_array_equal(t2s.numpy().view(np.uint32), sb)


def test_dequantised_value_is_within_half_a_grid_step():
    rd = make_rank(C2, 0, 64)                                # 1 % outliers x50 stress the scales
    x = oracle.bf16_to_f32(bf16_codes(rd.x))
    q, s = oracle.quantize_block128(bf16_codes(rd.x))
    deq = oracle.dequantize_block128(q, s)
    scale = np.repeat(s, 128, axis=1).astype(np.float64)
    y = np.abs(x.astype(np.float64)) / scale                 # position on the fp8 grid
    step = np.where(y < 2.0 ** -6, 2.0 ** -9, 2.0 ** (np.floor(np.log2(np.maximum(y, 2.0 ** -6))) - 3))
    err = np.abs(deq.astype(np.float64) - x.astype(np.float64)) / scale
    assert (err <= step / 2 * (1 + 1e-5) + 1e-9).all()
    assert not np.isnan(deq).any()


def test_combine_is_the_weighted_sum_and_c_uses_true_fma():
    case = C1
    world = make_world(case, "all")
    rows = rows_needed(case, world)
    res = run_oracle(case, world, rows)
    N, Le = case.world_size, case.experts_per_rank
    # float64 restatement: out = sum_k w[t,k] * y[slot(t,k)]
    for g in (0, N - 1):
        idx = world[g].indices.numpy().astype(np.int64)
        w = world[g].weights.numpy().astype(np.float64)
        acc = np.zeros((idx.shape[0], case.hidden_dim))
        for k in range(case.topk):
            ranks = idx[:, k] // Le
            rows_k = np.stack([oracle.bf16_to_f32(res.expert_y[r][s]) for r, s in zip(ranks, res.slots[g][:, k])])
            acc += w[:, k, None] * rows_k
        got = oracle.bf16_to_f32(res.out_tokens[g]).astype(np.float64)
        np.testing.assert_allclose(got, acc, rtol=2 ** -8, atol=1e-6)     # one bf16 rounding
    # the C restatement (real fmaf) on the same data
    cw = c_oracle.CWorld(case.num_experts, N, N, case.expert_padding, case.hidden_dim, case.topk, rows)
    cw.route_all([rd.indices.numpy() for rd in world])
    cw.dispatch([bf16_codes(rd.x) for rd in world])
    for r in range(N):
        np.testing.assert_array_equal(cw.out_x[r][res.written[r]], res.x[r][res.written[r]])
        np.testing.assert_array_equal(cw.out_s[r][res.written[r]], res.x_scale[r][res.written[r]])
    cw.act()
    for r in range(N):
        np.testing.assert_array_equal(cw.y[r][res.written[r]], res.expert_y[r][res.written[r]])
    outs = cw.combine([rd.weights.numpy() for rd in world])
    for g in range(N):
        same = (outs[g] == res.out_tokens[g]).mean()
        assert same > 0.9999, same                            # float64-emulated fma differs only in rare ties
        np.testing.assert_allclose(oracle.bf16_to_f32(outs[g]), oracle.bf16_to_f32(res.out_tokens[g]), rtol=2 ** -7)


def test_round_trip_identity_of_the_reference_test():
    """combine(2 * dequant(dispatch(x))) == 2 * x up to the fp8 grid, because the weights sum to 1
    (tests/p2p_all_to_all/test_p2p_all_to_all.py:44-50,102,182-189,233-234)."""
    case = C0
    world = make_world(case, "all")
    res = run_oracle(case, world, rows_needed(case, world))
    for g, rd in enumerate(world):
        x = oracle.bf16_to_f32(bf16_codes(rd.x)).astype(np.float64)
        out = oracle.bf16_to_f32(res.out_tokens[g]).astype(np.float64)
        # per group of 128: |2*deq - 2x| <= 2 * amax / 448 * (half a step at the top binade = 16)
        amax = np.abs(x).reshape(x.shape[0], -1, 128).max(axis=2, keepdims=True)
        bound = np.repeat(2 * amax / 448 * 16 + 2 ** -7 * 2 * amax, 128, axis=2).reshape(x.shape)
        assert (np.abs(out - 2 * x) <= bound).all()
        # and the receive counts are the bincount of everything routed here
    counts = sum(np.bincount(rd.indices.numpy().reshape(-1), minlength=case.num_experts) for rd in world)
    Le = case.experts_per_rank
    for r in range(case.world_size):
        np.testing.assert_array_equal(res.num_tokens[r], counts[r * Le:(r + 1) * Le])


def test_combine_accumulate_and_bound_m():
    rng = np.random.default_rng(2)
    E, N, K, H, T = 8, 2, 2, 16, 5
    idx = [rng.integers(0, E, (T, K)).astype(np.int32) for _ in range(N)]
    w = [rng.random((T, K), dtype=np.float32) for _ in range(N)]
    num_routed, toffs, eoffs, slots = oracle.world_routing(idx, E, N, N, 1, bound_m=[3, None])
    assert (slots[0][3:] == -1).all() and (slots[0][:3] >= 0).all()
    assert num_routed[0].sum() == 3 * K
    rows = 64
    y = [oracle.f32_to_bf16(rng.standard_normal((rows, H)).astype(np.float32)) for _ in range(N)]
    prev = [oracle.f32_to_bf16(rng.standard_normal((T, H)).astype(np.float32)) for _ in range(N)]
    plain = oracle.combine_world(y, idx, w, slots, num_experts=E, world_size=N, bound_m=[3, None])
    accum = oracle.combine_world(y, idx, w, slots, num_experts=E, world_size=N, out_prev=prev, bound_m=[3, None])
    assert (plain[0][3:] == 0).all()
    np.testing.assert_array_equal(accum[0][3:], prev[0][3:])          # tokens beyond bound_m untouched
    a = oracle.bf16_to_f32(accum[1]).astype(np.float64)
    p = oracle.bf16_to_f32(plain[1]).astype(np.float64) + oracle.bf16_to_f32(prev[1]).astype(np.float64)
    np.testing.assert_allclose(a, p, rtol=2 ** -6, atol=2 ** -6)


def test_c_oracle_with_threads_equals_scalar():
    """The C oracle splits tokens over threads for the all-cores CPU baseline; tokens are independent,
    so the bytes must not depend on the number of threads."""
    import c_oracle
    from a2a_cases import C0, bf16_codes, make_world
    from a2a_harness import rows_needed
    case = C0
    world = make_world(case, "ragged")
    rows = rows_needed(case, world)
    results = []
    for threads in (1, 3, 8):
        c_oracle.set_threads(threads)
        try:
            cw = c_oracle.CWorld(case.num_experts, case.world_size, case.world_size, case.expert_padding,
                                 case.hidden_dim, case.topk, rows)
            cw.route_all([rd.indices.numpy() for rd in world])
            cw.dispatch([bf16_codes(rd.x) for rd in world])
            cw.act()
            outs = cw.combine([rd.weights.numpy() for rd in world])
            results.append(([a.copy() for a in cw.out_x], [a.copy() for a in cw.out_s], outs))
        finally:
            c_oracle.set_threads(1)
    for other in results[1:]:
        for a, b in zip(results[0][0], other[0]):
            np.testing.assert_array_equal(a, b)
        for a, b in zip(results[0][1], other[1]):
            np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
        for a, b in zip(results[0][2], other[2]):
            np.testing.assert_array_equal(a, b)
