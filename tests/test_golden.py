"""The committed golden fixtures against the oracle (numpy and C) on the CPU and against the
HIP library on the GPU."""

import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import a2a_oracle as oracle
import c_oracle

GOLDEN = Path(__file__).resolve().parent / "golden"
sys.path.insert(0, str(GOLDEN))
from make_golden import CASES, build  # noqa: E402

FIXTURES = [(case, sources) for case in CASES for sources in ("all", "ragged")]


def _load(case, sources):
    with np.load(GOLDEN / f"{case.name}_{sources}.npz") as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("case,sources", FIXTURES, ids=lambda v: v.name if hasattr(v, "name") else v)
def test_oracle_reproduces_the_fixtures(case, sources):
    want = _load(case, sources)
    got = build(case, sources)
    assert sorted(got) == sorted(want)
    for key in want:
        np.testing.assert_array_equal(got[key], want[key], err_msg=key)


@pytest.mark.parametrize("case,sources", FIXTURES, ids=lambda v: v.name if hasattr(v, "name") else v)
def test_c_oracle_reproduces_the_fixtures(case, sources):
    want = _load(case, sources)
    N = case.world_size
    cw = c_oracle.CWorld(case.num_experts, N, case.node_size or N, case.expert_padding, case.hidden_dim,
                         case.topk, int(want["rows"]))
    cw.route_all([want[f"indices_{r}"] for r in range(N)])
    cw.dispatch([want[f"x_{r}"] for r in range(N)])
    for r in range(N):
        w = want[f"written_{r}"]
        np.testing.assert_array_equal(cw.out_x[r][w], want[f"out_x_{r}"][w])
        np.testing.assert_array_equal(cw.out_s[r][w], want[f"out_scale_{r}"][w])
        np.testing.assert_array_equal(cw.tpe[r * cw.Le:(r + 1) * cw.Le], want[f"num_tokens_{r}"][: max(min(cw.Le, case.num_experts - r * cw.Le), 0)])
        cw.y[r][:] = want[f"expert_y_{r}"]
    outs = cw.combine([want[f"weights_{r}"] for r in range(N)])
    for g in range(N):
        a, b = oracle.bf16_to_f32(outs[g]), oracle.bf16_to_f32(want[f"out_tokens_{g}"])
        np.testing.assert_allclose(a, b, rtol=2 ** -7, atol=1e-6)


def test_fp8_known_answers():
    with np.load(GOLDEN / "e4m3fn_known_answers.npz") as z:
        values, codes = z["values"], z["codes"]
    np.testing.assert_array_equal(oracle.e4m3fn_encode(values), codes)
    np.testing.assert_array_equal(c_oracle.encode(values), codes)
    ref = torch.from_numpy(values.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(codes, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("split", [False, True], ids=["group", "split"])
@pytest.mark.parametrize("case,sources", FIXTURES, ids=lambda v: v.name if hasattr(v, "name") else v)
def test_gpu_reproduces_the_fixtures(case, sources, split):
    from a2a_cases import RankData
    from a2a_harness import run_gpu

    want = _load(case, sources)
    N = case.world_size
    def tensor(a, dtype):
        # a fresh torch tensor: zero-row numpy arrays carry zero strides
        return torch.empty(a.shape, dtype=dtype).copy_(torch.from_numpy(np.ascontiguousarray(a)))

    world = [RankData(x=tensor(want[f"x_{r}"].view(np.int16), torch.int16).view(torch.bfloat16),
                      indices=tensor(want[f"indices_{r}"], torch.int32),
                      weights=tensor(want[f"weights_{r}"], torch.float32)) for r in range(N)]
    got = run_gpu(case, world, int(want["rows"]), torch.device("cuda:0"), split=split,
                  expert_y_override=[want[f"expert_y_{r}"] for r in range(N)])
    for r in range(N):
        n_local = max(min(case.experts_per_rank, case.num_experts - r * case.experts_per_rank), 0)
        np.testing.assert_array_equal(got.num_tokens[r][:n_local], want[f"num_tokens_{r}"][:n_local])
        w = want[f"written_{r}"]
        np.testing.assert_array_equal(got.x[r][w], want[f"out_x_{r}"][w])
        np.testing.assert_array_equal(got.x_scale[r][w], want[f"out_scale_{r}"][w])
        a, b = oracle.bf16_to_f32(got.out_tokens[r]), oracle.bf16_to_f32(want[f"out_tokens_{r}"])
        np.testing.assert_allclose(a, b, rtol=1e-2, atol=1e-4)
