"""ctypes binding of the compiled library (`liba2a_mi355.so`).

Plays the part of the reference's pyo3 class `AllToAllContext`
(python-ext/src/py_p2p_all_to_all.rs:17-205, stub
python/pplx_garden/native/p2p_all_to_all.pyi:12-98): methods take integers
(device pointers, strides, a stream handle), `None` becomes a null pointer or 0
(py_p2p_all_to_all.rs:69,73,123-130) and every failure is a `RuntimeError`
carrying the library's message (py_p2p_all_to_all.rs:133).

There is no fallback: if the library has not been built, importing the context
raises.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_size_t, c_uint32, c_uint64, c_void_p
from pathlib import Path
from typing import Optional, Sequence

import torch

_LIB_PATH = Path(__file__).resolve().parent.parent / "lib" / "liba2a_mi355.so"

# Element type tags in the reference's ScalarType order (rust/torch-lib/src/lib.rs:31-49).
SCALAR_TYPE = {
    torch.bool: 0, torch.int8: 1, torch.uint8: 2, torch.int16: 3, torch.uint16: 4,
    torch.int32: 5, torch.uint32: 6, torch.int64: 7, torch.uint64: 8,
    torch.float8_e4m3fn: 9, torch.float8_e5m2: 10, torch.float16: 11,
    torch.bfloat16: 12, torch.float32: 13, torch.float64: 14,
}

TABLE_NUM_ROUTED = 0
TABLE_EXPERT_OFFSETS = 1
TABLE_TOKEN_OFFSET = 2
TABLE_SLOT = 3
TABLE_PADDED_INDEX = 4
TABLE_SOURCE_RANK = 5
TABLE_SOURCE_POSITION = 6
TABLE_NUM_RECV_TOKENS = 7
TABLE_SOURCE_DISPATCH_OFFSET = 8
TABLE_COMBINE_SEND_OFFSET = 9

DEV_BAD_EXPERT_ID = 1
DEV_RECV_OVERFLOW = 2
DEV_BAD_SLOT = 4
DEV_INTERNAL = 0x80000000   # a kernel gave up waiting for its own wavefronts (a guard against a hang)

FLAG_PREALLOC_STAGING = 1
FLAG_SEPARATE_ROUTING = 2   # never take the one-launch paths of small steps
KERNEL_PACK = 0
KERNEL_GATHER = 1
KERNEL_ROUTE = 2
KERNEL_STAGE_SEND = 3
KERNEL_STAGE_RECV = 4
KERNEL_COMBINE_SEND = 5


class A2AConfig(ctypes.Structure):
    _fields_ = [
        ("struct_size", c_uint32), ("hidden_dim", c_uint32), ("hidden_dim_scale", c_uint32),
        ("in_elemsize", c_uint32), ("out_elemsize", c_uint32), ("out_dtype", c_uint32),
        ("scale_elemsize", c_uint32), ("max_num_tokens", c_uint32), ("max_recv_tokens", c_uint32),
        ("max_private_tokens", c_uint32), ("num_experts", c_uint32), ("expert_padding", c_uint32),
        ("num_experts_per_token", c_uint32), ("dp_size", c_uint32), ("node_size", c_uint32),
        ("world_size", c_uint32), ("device", c_int32), ("flags", c_uint32),
    ]


class A2ADispatchArgs(ctypes.Structure):
    _fields_ = [
        ("num_tokens", c_uint64), ("x_ptr", c_void_p), ("x_stride", c_uint64),
        ("x_scale_ptr", c_void_p), ("x_scale_stride_elem", c_uint64),
        ("x_scale_stride_token", c_uint64), ("indices", c_void_p), ("indices_stride", c_uint64),
        ("weights", c_void_p), ("weights_stride", c_uint64), ("bound_m", c_void_p),
        ("out_num_tokens", c_void_p), ("out_x", c_void_p), ("out_x_stride", c_uint64),
        ("out_x_rows", c_uint64), ("out_x_scale", c_void_p),
        ("out_x_scale_stride_elem", c_uint64), ("out_x_scale_stride_token", c_uint64),
    ]


class A2ACombineArgs(ctypes.Structure):
    _fields_ = [
        ("expert_y", c_void_p), ("expert_y_stride", c_uint64), ("expert_y_rows", c_uint64),
        ("num_tokens", c_uint64), ("out_tokens", c_void_p), ("out_tokens_stride", c_uint64),
        ("indices", c_void_p), ("indices_stride", c_uint64), ("weights", c_void_p),
        ("weights_stride", c_uint64), ("bound_m", c_void_p),
    ]


# Every symbol include/a2a.h declares, with its argument types.
_SIGNATURES = {
    "a2a_version": (c_char_p, []),
    "a2a_last_error": (c_char_p, [c_void_p]),
    "a2a_dispatch_token_stride": (c_size_t, [POINTER(A2AConfig)]),
    "a2a_combine_token_stride": (c_size_t, [POINTER(A2AConfig)]),
    "a2a_ctx_create": (c_int, [POINTER(A2AConfig), POINTER(c_void_p)]),
    "a2a_ctx_destroy": (c_int, [c_void_p]),
    "a2a_ctx_status": (c_int, [c_void_p, c_void_p, POINTER(c_uint32)]),
    "a2a_ctx_read_table": (c_int, [c_void_p, c_uint32, c_uint32, POINTER(c_uint32), c_size_t, c_void_p]),
    "a2a_ctx_time_next_kernel": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p]),
    "a2a_dispatch_send": (c_int, [
        c_void_p, c_uint32, c_size_t, c_void_p, c_size_t, c_uint32, c_void_p, c_size_t, c_size_t,
        c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_void_p]),
    "a2a_dispatch_recv": (c_int, [
        c_void_p, c_uint32, c_void_p, c_void_p, c_size_t, c_size_t, c_void_p, c_size_t, c_size_t,
        c_void_p]),
    "a2a_combine_send": (c_int, [c_void_p, c_uint32, c_void_p, c_size_t, c_size_t, c_void_p]),
    "a2a_combine_recv": (c_int, [
        c_void_p, c_uint32, c_size_t, c_size_t, c_uint32, c_void_p, c_size_t, c_void_p, c_size_t,
        c_void_p, c_size_t, c_void_p, c_uint32, c_void_p]),
    "a2a_dispatch": (c_int, [c_void_p, POINTER(A2ADispatchArgs), c_uint32, c_void_p]),
    "a2a_combine": (c_int, [c_void_p, POINTER(A2ACombineArgs), c_uint32, c_uint32, c_void_p]),
    "a2a_dispatch_static": (c_int, [POINTER(A2AConfig), POINTER(A2ADispatchArgs), c_uint32, c_void_p, c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


def library_path() -> Path:
    return _LIB_PATH


def load_library() -> ctypes.CDLL:
    """Load the compiled library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not _LIB_PATH.exists():
        raise ImportError(
            f"{_LIB_PATH} is missing: build it with `python pplx-garden_amd/build.py` "
            "(there is no Python or CPU fallback for this path)")
    lib = ctypes.CDLL(str(_LIB_PATH))
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def _ptr(value: Optional[int]) -> Optional[int]:
    return None if value in (None, 0) else int(value)


def _num(value: Optional[int]) -> int:
    return 0 if value is None else int(value)


STATIC_SCRATCH_BYTES = 8 << 20


def dispatch_static(config: A2AConfig, per_rank: Sequence[A2ADispatchArgs], quantize: bool,
                    device_flags_ptr: Optional[int], stream: int) -> None:
    """`a2a_dispatch_static`: the group dispatch without a context and without any allocation (the
    routing tables of the step live in a fixed array inside the library).  `per_rank` holds one
    A2ADispatchArgs per rank of `config.world_size`; `device_flags_ptr` is an optional device pointer
    to one uint32 that collects the DEV_* bits."""
    lib = load_library()
    if len(per_rank) != config.world_size:
        raise RuntimeError(f"expected arguments of {config.world_size} ranks, got {len(per_rank)}")
    arr = per_rank if isinstance(per_rank, ctypes.Array) else (A2ADispatchArgs * config.world_size)(*per_rank)
    rc = lib.a2a_dispatch_static(ctypes.byref(config), arr, int(quantize), _ptr(device_flags_ptr), _ptr(stream))
    if rc != 0:
        raise RuntimeError(lib.a2a_last_error(None).decode() or f"a2a_dispatch_static failed ({rc})")


class AllToAllContext:
    """One expert-parallel group of logical ranks on one GPU."""

    def __init__(self, handle: int, config: A2AConfig) -> None:
        self._handle = c_void_p(handle)
        self._config = config
        self._lib = load_library()

    @classmethod
    def create(
        cls,
        hidden_dim: int,
        hidden_dim_scale: Optional[int],
        in_elemsize: int,
        out_elemsize: int,
        out_dtype: torch.dtype,
        scale_elemsize: Optional[int],
        max_num_tokens: int,
        max_recv_tokens: int,
        max_private_tokens: int,
        num_experts: int,
        expert_padding: int,
        num_experts_per_token: int,
        dp_size: int,
        node_size: int,
        world_size: int,
        device: int,
        flags: int = 0,
    ) -> "AllToAllContext":
        """Arguments of the reference's `AllToAllContext.create`
        (native/p2p_all_to_all.pyi:13-51) minus `rank` (every call names its
        rank) and the transport handles."""
        lib = load_library()
        if out_dtype not in SCALAR_TYPE:
            raise RuntimeError(f"unsupported out_dtype {out_dtype}")
        cfg = A2AConfig(
            struct_size=ctypes.sizeof(A2AConfig), hidden_dim=hidden_dim,
            hidden_dim_scale=_num(hidden_dim_scale), in_elemsize=in_elemsize,
            out_elemsize=out_elemsize, out_dtype=SCALAR_TYPE[out_dtype],
            scale_elemsize=_num(scale_elemsize), max_num_tokens=max_num_tokens,
            max_recv_tokens=min(max_recv_tokens, 0xFFFFFFFF), max_private_tokens=max_private_tokens,
            num_experts=num_experts, expert_padding=expert_padding,
            num_experts_per_token=num_experts_per_token, dp_size=dp_size, node_size=node_size,
            world_size=world_size, device=device, flags=flags)
        handle = c_void_p()
        rc = lib.a2a_ctx_create(ctypes.byref(cfg), ctypes.byref(handle))
        if rc != 0:
            raise RuntimeError(lib.a2a_last_error(None).decode() or f"a2a_ctx_create failed ({rc})")
        return cls(handle.value, cfg)

    # -- helpers ---------------------------------------------------------

    @property
    def world_size(self) -> int:
        return self._config.world_size

    def _check(self, rc: int) -> None:
        if rc != 0:
            msg = self._lib.a2a_last_error(self._handle).decode()
            raise RuntimeError(msg or f"a2a call failed with code {rc}")

    def _require_open(self) -> None:
        if not self._handle:
            raise RuntimeError("AllToAllContext has been destroyed")

    def destroy(self) -> None:
        if self._handle:
            handle, self._handle = self._handle, c_void_p()
            self._check_destroy(self._lib.a2a_ctx_destroy(handle))

    @staticmethod
    def _check_destroy(rc: int) -> None:
        if rc != 0:
            raise RuntimeError(f"a2a_ctx_destroy failed with code {rc}")

    def __del__(self) -> None:  # Drop => destroy (a2a_context.rs:490-494)
        try:
            self.destroy()
        except Exception:
            pass

    # -- the four split calls (native/p2p_all_to_all.pyi:52-98) -----------

    def dispatch_send(self, rank: int, num_tokens: int, x_ptr: int, x_stride: int,
                      x_scale_ptr: Optional[int], x_scale_stride_elem: Optional[int],
                      x_scale_stride_token: Optional[int], indices_ptr: int, indices_stride: int,
                      weights_ptr: int, weights_stride: int, bound_m_ptr: Optional[int],
                      stream: int, quantize: bool = False) -> None:
        self._require_open()
        self._check(self._lib.a2a_dispatch_send(
            self._handle, rank, num_tokens, _ptr(x_ptr), x_stride, int(quantize),
            _ptr(x_scale_ptr), _num(x_scale_stride_elem), _num(x_scale_stride_token),
            _ptr(indices_ptr), indices_stride, _ptr(weights_ptr), weights_stride,
            _ptr(bound_m_ptr), _ptr(stream)))

    def dispatch_recv(self, rank: int, out_num_tokens_ptr: int, out_x_ptr: int, out_x_stride: int,
                      out_x_rows: int, out_x_scale_ptr: Optional[int],
                      out_x_scale_stride_elem: Optional[int],
                      out_x_scale_stride_token: Optional[int], stream: int) -> None:
        self._require_open()
        self._check(self._lib.a2a_dispatch_recv(
            self._handle, rank, _ptr(out_num_tokens_ptr), _ptr(out_x_ptr), out_x_stride, out_x_rows,
            _ptr(out_x_scale_ptr), _num(out_x_scale_stride_elem), _num(out_x_scale_stride_token),
            _ptr(stream)))

    def combine_send(self, rank: int, expert_x_ptr: int, expert_x_stride: int, expert_x_rows: int,
                     stream: int) -> None:
        self._require_open()
        self._check(self._lib.a2a_combine_send(
            self._handle, rank, _ptr(expert_x_ptr), expert_x_stride, expert_x_rows, _ptr(stream)))

    def combine_recv(self, rank: int, num_tokens: int, num_recv_tokens: int,
                     expert_y_dtype: torch.dtype, out_tokens_ptr: int, out_tokens_stride: int,
                     indices_ptr: int, indices_stride: int, weights_ptr: int, weights_stride: int,
                     bound_m_ptr: Optional[int], accumulate: bool, stream: int) -> None:
        self._require_open()
        if expert_y_dtype not in SCALAR_TYPE:
            raise RuntimeError(f"unsupported expert_y dtype {expert_y_dtype}")
        self._check(self._lib.a2a_combine_recv(
            self._handle, rank, num_tokens, num_recv_tokens, SCALAR_TYPE[expert_y_dtype],
            _ptr(out_tokens_ptr), out_tokens_stride, _ptr(indices_ptr), indices_stride,
            _ptr(weights_ptr), weights_stride, _ptr(bound_m_ptr), int(bool(accumulate)),
            _ptr(stream)))

    # -- the two group calls ------------------------------------------------

    def pack_dispatch_args(self, per_rank: Sequence[A2ADispatchArgs]):
        """The C array `a2a_dispatch` takes; build it once when the buffers do not change."""
        if len(per_rank) != self.world_size:
            raise RuntimeError(f"expected arguments of {self.world_size} ranks, got {len(per_rank)}")
        return (A2ADispatchArgs * self.world_size)(*per_rank)

    def pack_combine_args(self, per_rank: Sequence[A2ACombineArgs]):
        if len(per_rank) != self.world_size:
            raise RuntimeError(f"expected arguments of {self.world_size} ranks, got {len(per_rank)}")
        return (A2ACombineArgs * self.world_size)(*per_rank)

    def dispatch(self, per_rank, quantize: bool, stream: int) -> None:
        """`per_rank`: one A2ADispatchArgs per rank, or the array from pack_dispatch_args."""
        self._require_open()
        arr = per_rank if isinstance(per_rank, ctypes.Array) else self.pack_dispatch_args(per_rank)
        self._check(self._lib.a2a_dispatch(self._handle, arr, int(quantize), _ptr(stream)))

    def combine(self, per_rank, expert_y_dtype: torch.dtype, accumulate: bool, stream: int) -> None:
        self._require_open()
        if expert_y_dtype not in SCALAR_TYPE:
            raise RuntimeError(f"unsupported expert_y dtype {expert_y_dtype}")
        arr = per_rank if isinstance(per_rank, ctypes.Array) else self.pack_combine_args(per_rank)
        self._check(self._lib.a2a_combine(
            self._handle, arr, SCALAR_TYPE[expert_y_dtype], int(bool(accumulate)), _ptr(stream)))

    # -- introspection ------------------------------------------------------

    def status(self, stream: int = 0) -> int:
        """Synchronise `stream`; return and clear the device-side error bits."""
        self._require_open()
        flags = c_uint32(0)
        self._check(self._lib.a2a_ctx_status(self._handle, _ptr(stream), ctypes.byref(flags)))
        return flags.value

    def read_table(self, rank: int, which: int, count: int, stream: int = 0) -> torch.Tensor:
        """Copy `count` entries of a routing table of `rank` to a CPU int64 tensor."""
        self._require_open()
        buf = (c_uint32 * max(count, 1))()
        self._check(self._lib.a2a_ctx_read_table(self._handle, rank, which, buf, count, _ptr(stream)))
        return torch.tensor(list(buf[:count]), dtype=torch.int64)

    def time_next_kernel(self, which: int, start_event: Optional[int], stop_event: Optional[int]) -> None:
        """Have the next call that launches kernel `which` (`KERNEL_PACK`, `KERNEL_ROUTE`: the group
        dispatch; `KERNEL_GATHER`: the group combine or the split combine-recv; `KERNEL_STAGE_SEND`,
        `KERNEL_ROUTE`: the split send; `KERNEL_STAGE_RECV`, `KERNEL_COMBINE_SEND`: those split calls)
        record the two events (raw `hipEvent_t` handles, e.g. `torch.cuda.Event.cuda_event`) at the
        start and end of that kernel itself.  `KERNEL_ROUTE` is the routing launch before the pack or
        the staging of a large step; a step without such a launch leaves those events alone."""
        self._require_open()
        self._check(self._lib.a2a_ctx_time_next_kernel(self._handle, which, _ptr(start_event), _ptr(stop_event)))

    def dispatch_token_stride(self) -> int:
        return int(self._lib.a2a_dispatch_token_stride(ctypes.byref(self._config)))

    def combine_token_stride(self) -> int:
        return int(self._lib.a2a_combine_token_stride(ctypes.byref(self._config)))
