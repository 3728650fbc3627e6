"""CPU-side checks of the boundary: the library loads, exports every function the header
declares, rejects bad configurations with the documented codes (no GPU needed: the
configuration is checked before any HIP call), and the host-side Python mirrors the
reference's helpers."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

import a2a_oracle as oracle
from pplx_garden_amd.distributed.loopback import LoopbackWorld
from pplx_garden_amd.native import p2p_all_to_all as native
from pplx_garden_amd.utils.math import Statistics, ceil_div, round_up

REPO = Path(__file__).resolve().parent.parent
HEADER = (REPO / "include" / "a2a.h").read_text()


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    names = re.findall(r"^\s*(?:const\s+char|int|size_t)\s*\**\s*(a2a_\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_library_exports_every_declared_function():
    lib = native.load_library()
    declared = _declared_functions()
    assert len(declared) >= 14, declared
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/a2a.h but not exported"
    assert sorted(native.EXPORTED_SYMBOLS) == declared
    assert lib.a2a_version() == b"0.1"


def test_struct_layouts_match_the_header():
    # field order of the ctypes mirrors is the order in include/a2a.h
    for struct, cname in ((native.A2AConfig, "a2a_config"), (native.A2ADispatchArgs, "a2a_dispatch_args"),
                          (native.A2ACombineArgs, "a2a_combine_args")):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), HEADER, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = re.findall(r"(\w+)\s*;", body)
        assert [f for f, _ in struct._fields_] == fields, cname
    assert ctypes.sizeof(native.A2AConfig) == 18 * 4
    assert ctypes.sizeof(native.A2ADispatchArgs) == 18 * 8
    assert ctypes.sizeof(native.A2ACombineArgs) == 11 * 8


def _config(**over):
    base = dict(struct_size=ctypes.sizeof(native.A2AConfig), hidden_dim=128, hidden_dim_scale=0, in_elemsize=2,
                out_elemsize=2, out_dtype=12, scale_elemsize=0, max_num_tokens=16, max_recv_tokens=64,
                max_private_tokens=0, num_experts=8, expert_padding=1, num_experts_per_token=2, dp_size=1,
                node_size=2, world_size=2, device=0, flags=0)
    base.update(over)
    return native.A2AConfig(**base)


@pytest.mark.parametrize("over,code,needle", [
    (dict(struct_size=4), -1, "struct_size"),
    (dict(world_size=33, node_size=33), -3, "world_size"),
    (dict(dp_size=3, node_size=4, world_size=4), -1, "dp_size"),
    (dict(dp_size=0), -1, "dp_size"),
    (dict(node_size=3), -1, "node_size"),
    (dict(num_experts=2000), -3, "num_experts"),
    (dict(num_experts_per_token=65), -3, "num_experts_per_token"),
    (dict(expert_padding=0), -1, "expert_padding"),
    (dict(hidden_dim=7, in_elemsize=2), -3, "multiple of 16"),
    (dict(in_elemsize=3), -3, "in_elemsize"),
    (dict(out_dtype=14, out_elemsize=8), -3, "out_dtype"),
    (dict(hidden_dim_scale=4, scale_elemsize=2), -3, "scale"),
    (dict(max_num_tokens=0), -1, "max_num_tokens"),
    (dict(flags=8), -1, "flags"),
])
def test_bad_configurations_are_rejected_with_a_message(over, code, needle):
    lib = native.load_library()
    handle = ctypes.c_void_p()
    cfg = _config(**over)
    rc = lib.a2a_ctx_create(ctypes.byref(cfg), ctypes.byref(handle))
    assert rc == code
    assert handle.value is None
    assert needle in lib.a2a_last_error(None).decode()


def test_null_arguments_do_not_crash():
    lib = native.load_library()
    assert lib.a2a_ctx_create(None, None) == -1
    assert lib.a2a_ctx_destroy(None) == 0
    assert lib.a2a_dispatch(None, None, 0, None) == -1
    assert lib.a2a_combine(None, None, 12, 0, None) == -1
    assert lib.a2a_ctx_status(None, None, None) == -1


def test_static_dispatch_refuses_what_its_fixed_tables_cannot_hold():
    """The checks of a2a_dispatch_static run before its first HIP call, so they can be exercised
    without a GPU: a step beyond the fixed array, flags, and more tokens than max_num_tokens."""
    lib = native.load_library()
    big = _config(world_size=32, node_size=32, num_experts=1024, num_experts_per_token=8, max_num_tokens=8192,
                  hidden_dim=7168, in_elemsize=1, hidden_dim_scale=56, scale_elemsize=4)
    args = (native.A2ADispatchArgs * 32)()
    for a in args:
        a.num_tokens = 8192
    assert lib.a2a_dispatch_static(ctypes.byref(big), args, 1, None, None) == -2
    msg = lib.a2a_last_error(None).decode()
    assert "bytes of routing tables" in msg and str(native.STATIC_SCRATCH_BYTES) in msg
    assert lib.a2a_dispatch_static(ctypes.byref(_config(flags=2)), args, 0, None, None) == -1
    assert "flags" in lib.a2a_last_error(None).decode()
    small = _config()
    args[0].num_tokens = 17
    assert lib.a2a_dispatch_static(ctypes.byref(small), args, 0, None, None) == -2
    assert lib.a2a_dispatch_static(None, None, 0, None, None) == -1
    header_bytes = re.search(r"#define A2A_STATIC_SCRATCH_BYTES \((\d+)u << (\d+)\)", HEADER)
    assert int(header_bytes.group(1)) << int(header_bytes.group(2)) == native.STATIC_SCRATCH_BYTES


def test_operator_capacities_match_the_oracle_and_the_reference_values():
    """Rows of a rank's receive region (python/pplx_garden/kernels/p2p_all_to_all.py:92-114): the
    operator's arithmetic against the oracle's on the five baseline shapes, the 1-token configuration
    of the reference's test matrix, dp groups, and the value the reference's sizes give for the
    DeepSeek decode shape (Le 32, average int(4 * 1.2) = 4, private 128, 128 * 8 + 8192 = 9216)."""
    from a2a_cases import BASELINE_CASES
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll
    shapes = [(c.num_tokens, c.num_experts, c.topk, c.world_size, 1, c.expert_padding, None) for c in BASELINE_CASES]
    shapes += [(1, 2, 1, 2, 1, 1, 32), (8, 16, 2, 2, 1, 16, None), (1, 4, 1, 4, 2, 1, None), (8, 4, 4, 4, 2, 1, None),
               (128, 16, 2, 2, 1, 1, 8), (4096, 256, 8, 8, 1, 1, 0), (64, 384, 8, 16, 4, 128, None)]
    for T, E, K, N, D, pad, private in shapes:
        got = P2PAllToAll.receive_capacity(max_num_tokens=T, num_experts=E, expert_padding=pad,
                                           num_experts_per_token=K, world_size=N, dp_size=D,
                                           max_private_tokens=private)
        Le, want_private, want_recv = oracle.buffer_capacity(T, E, K, N, D, pad, private)
        assert got == (want_private, want_recv), (T, E, K, N, D, pad, private)
        assert Le == ceil_div(E, N)
    assert P2PAllToAll.receive_capacity(max_num_tokens=128, num_experts=256, expert_padding=1,
                                        num_experts_per_token=8, world_size=8) == (128, 9216)
    assert P2PAllToAll.receive_capacity(max_num_tokens=1, num_experts=2, expert_padding=1,
                                        num_experts_per_token=1, world_size=2, max_private_tokens=32) == (32, 66)


def test_strides_match_the_oracle():
    lib = native.load_library()
    for H, ie, Hs, se, oe in [(7168, 1, 56, 4, 2), (2048, 1, 16, 4, 2), (128, 4, 0, 0, 4), (16, 2, 0, 0, 2),
                              (4, 4, 0, 0, 4), (7168, 2, 0, 0, 2)]:
        cfg = _config(hidden_dim=H, in_elemsize=ie, hidden_dim_scale=Hs, scale_elemsize=se, out_elemsize=oe)
        assert lib.a2a_dispatch_token_stride(ctypes.byref(cfg)) == oracle.dispatch_token_stride(H, ie, Hs, se)
        assert lib.a2a_combine_token_stride(ctypes.byref(cfg)) == oracle.combine_token_stride(H, oe)


def test_math_helpers_and_statistics():
    assert round_up(7168 + 224, 16) == 7392 and round_up(5, 1) == 5 and ceil_div(33, 8) == 5
    # percentile rule of the reference (python/pplx_garden/utils/math.py:75-79)
    s = Statistics.create([float(v) for v in range(1, 11)])           # n = 10
    assert s.p50 == 6.0            # n*p = 5 is integral -> sorted[5]
    assert s.p25 == (3.0 + 4.0) / 2   # n*p = 2.5 -> mean of sorted[2], sorted[3]
    assert s.p99 == 10.0           # index + 1 >= n -> sorted[index]
    assert s.min == 1.0 and s.max == 10.0 and s.mean == 5.5
    assert abs(s.stddev - 3.0276503540974917) < 1e-12
    assert Statistics.create([]).mean == 0.0 and Statistics.create([4.0]).stddev == 0.0
    assert "p50=6.0" in str(s)


def test_loopback_world_runs_a_collective_when_the_last_rank_posts():
    world = LoopbackWorld(3)
    assert [g.rank for g in world.groups] == [0, 1, 2] and world.group(1).size == 3
    key = ("cfg",)
    assert world.post(key, "dispatch", 1, "b") is None
    assert world.post(key, "dispatch", 0, "a") is None
    assert world.pending(key, "dispatch") == [0, 1]
    with pytest.raises(RuntimeError, match="twice"):
        world.post(key, "dispatch", 1, "again")
    assert world.post(key, "dispatch", 2, "c") == ["a", "b", "c"]      # rank order, not call order
    assert world.pending(key, "dispatch") == []
    assert world.post(key, "combine", 0, 1) is None                   # kinds do not mix
    with pytest.raises(ValueError):
        LoopbackWorld(4, node_size=3)
    with pytest.raises(ValueError):
        world.group(3)


def test_shared_context_is_created_once_and_freed_by_the_last_user():
    world = LoopbackWorld(2)
    made, freed = [], []

    class Fake:
        def destroy(self):
            freed.append(1)

    def factory():
        made.append(1)
        return Fake()

    a = world.acquire_context(("k",), factory)
    b = world.acquire_context(("k",), factory)
    assert a is b and len(made) == 1
    world.release_context(("k",))
    assert not freed
    world.release_context(("k",))
    assert freed == [1]


def test_operator_keeps_the_reference_signature():
    import inspect
    from pplx_garden_amd.kernels.all_to_all import AllToAllKernel
    from pplx_garden_amd.kernels.p2p_all_to_all import P2PAllToAll

    # python/pplx_garden/kernels/all_to_all.py:6-33
    assert list(inspect.signature(AllToAllKernel.dispatch).parameters) == [
        "self", "out_expert_num_tokens", "out_expert_x", "out_expert_x_scale", "dp_x", "dp_x_scale", "indices",
        "weights", "bound_m", "do_send", "do_recv"]
    assert list(inspect.signature(AllToAllKernel.combine).parameters) == [
        "self", "out_tokens", "indices", "weights", "expert_y", "bound_m", "do_send", "do_recv", "accumulate"]
    for name in ("dispatch", "combine", "destroy"):
        assert list(inspect.signature(getattr(P2PAllToAll, name)).parameters) == \
            list(inspect.signature(getattr(AllToAllKernel, name)).parameters)
    # python/pplx_garden/kernels/p2p_all_to_all.py:51-69 (keyword-only constructor)
    ctor = inspect.signature(P2PAllToAll.__init__).parameters
    assert list(ctor)[1:] == ["max_num_tokens", "num_experts", "expert_padding", "hidden_dim", "hidden_dim_scale",
                              "in_dtype", "out_dtype", "scale_dtype", "num_experts_per_token", "nets_per_gpu",
                              "max_private_tokens", "device", "dp_group", "node_group", "global_group"]
    assert all(p.kind is inspect.Parameter.KEYWORD_ONLY for n, p in ctor.items() if n != "self")


def test_context_creation_fails_loudly_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError):
        native.AllToAllContext.create(
            hidden_dim=128, hidden_dim_scale=None, in_elemsize=2, out_elemsize=2, out_dtype=torch.bfloat16,
            scale_elemsize=None, max_num_tokens=4, max_recv_tokens=16, max_private_tokens=0, num_experts=4,
            expert_padding=1, num_experts_per_token=2, dp_size=1, node_size=2, world_size=2, device=0)


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """include/a2a.h must be usable from C (no C++ or torch types): compile a caller with gcc -std=c99
    and g++, link it against the built library and let it read the version and the two stride
    helpers (no GPU work)."""
    import shutil
    import subprocess
    repo = Path(__file__).resolve().parent.parent
    lib = native.library_path()
    src = tmp_path / "caller.c"
    src.write_text("""
#include <stdio.h>
#include <string.h>
#include "a2a.h"
int main(void) {
    a2a_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.struct_size = sizeof cfg; cfg.hidden_dim = 7168; cfg.hidden_dim_scale = 56; cfg.in_elemsize = 1;
    cfg.out_elemsize = 2; cfg.out_dtype = A2A_BF16; cfg.scale_elemsize = 4;
    a2a_dispatch_args d; a2a_combine_args c; (void)d; (void)c;
    printf("%s %zu %zu %d\\n", a2a_version(), a2a_dispatch_token_stride(&cfg), a2a_combine_token_stride(&cfg),
           (int)A2A_FLAG_SEPARATE_ROUTING);
    return 0;
}
""")
    for compiler, std in (("gcc", "-std=c99"), ("g++", "-std=c++11")):
        if shutil.which(compiler) is None:
            pytest.skip(f"{compiler} not installed")
        exe = tmp_path / f"caller_{compiler}"
        unit = src if compiler == "gcc" else tmp_path / "caller.cpp"
        if compiler == "g++":
            unit.write_text(src.read_text())
        subprocess.run([compiler, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", str(repo / "include"), str(unit),
                        "-o", str(exe), "-L", str(lib.parent), "-la2a_mi355", f"-Wl,-rpath,{lib.parent}",
                        "-Wl,--allow-shlib-undefined"], check=True)
        out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
        assert out == ["0.1", "7408", "14336", "2"], out
