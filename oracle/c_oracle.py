"""ctypes access to oracle/liba2a_oracle.so, the C restatement of the oracle."""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_size_t, c_uint8, c_uint32, c_void_p
from pathlib import Path

import numpy as np

_PATH = Path(__file__).resolve().parent / "liba2a_oracle.so"
_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _PATH.exists():
            raise ImportError(f"{_PATH} is missing: run `make -C oracle`")
        l = ctypes.CDLL(str(_PATH))
        l.oracle_e4m3fn_encode.restype = c_uint8
        l.oracle_e4m3fn_encode.argtypes = [c_float]
        l.oracle_e4m3fn_decode.restype = c_float
        l.oracle_e4m3fn_decode.argtypes = [c_uint8]
        l.oracle_e4m3fn_encode_array.argtypes = [c_void_p, c_void_p, c_size_t]
        l.oracle_route.restype = c_int
        l.oracle_route.argtypes = [c_void_p, c_size_t, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p]
        l.oracle_layout.argtypes = [c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p]
        l.oracle_quantize_row.argtypes = [c_void_p, c_uint32, c_void_p, c_void_p]
        l.oracle_dispatch_rank.argtypes = [c_void_p, c_size_t, c_void_p, c_size_t, c_uint32, c_uint32, c_uint32,
                                           c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
        l.oracle_combine_rank.argtypes = [c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_size_t, c_uint32,
                                          c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p, c_int, c_void_p]
        l.oracle_act_rows.argtypes = [c_void_p, c_void_p, c_size_t, c_uint32, c_void_p]
        l.oracle_set_threads.argtypes = [ctypes.c_int]
        l.oracle_set_threads.restype = None
        _lib = l
    return _lib


def _p(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def encode(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint8)
    lib().oracle_e4m3fn_encode_array(_p(f), _p(out), f.size)
    return out


def route(indices: np.ndarray, num_experts: int, num_tokens=None):
    idx = np.ascontiguousarray(indices, dtype=np.int32)
    T, K = idx.shape
    n = T if num_tokens is None else num_tokens
    count = np.zeros(num_experts, dtype=np.uint32)
    toff = np.zeros(T * K, dtype=np.uint32)
    eoff = np.zeros(num_experts, dtype=np.uint32)
    rc = lib().oracle_route(_p(idx), K, n, K, num_experts, _p(count), _p(toff), _p(eoff))
    if rc:
        raise ValueError("expert id out of range")
    return count, toff, eoff


def layout(num_routed: np.ndarray, node_size: int, expert_padding: int):
    nr = np.ascontiguousarray(num_routed, dtype=np.uint32)
    N, E = nr.shape
    tpe = np.zeros(E, dtype=np.uint32)
    poff = np.zeros(E, dtype=np.uint32)
    base = np.zeros((N, E), dtype=np.uint32)
    lib().oracle_layout(_p(nr), N, E, node_size, expert_padding, _p(tpe), _p(poff), _p(base))
    return tpe, poff, base


def quantize(x_codes: np.ndarray):
    x = np.ascontiguousarray(x_codes, dtype=np.uint16)
    T, H = x.shape
    q = np.empty((T, H), dtype=np.uint8)
    s = np.empty((T, H // 128), dtype=np.float32)
    for t in range(T):
        lib().oracle_quantize_row(_p(x[t]), H, _p(q[t]), _p(s[t]))
    return q, s


def set_threads(n: int) -> None:
    """Threads the C oracle splits the tokens of a dispatch or combine over (1 = the scalar port)."""
    lib().oracle_set_threads(int(n))


class CWorld:
    """dispatch + combine of a whole group with the C oracle (one thread unless set_threads says more)."""

    def __init__(self, num_experts, world_size, node_size, expert_padding, hidden_dim, topk, rows):
        self.E, self.N, self.node, self.pad = num_experts, world_size, node_size, expert_padding
        self.H, self.K, self.rows = hidden_dim, topk, rows
        self.Le = -(-num_experts // world_size)
        self.out_x = [np.zeros((rows, hidden_dim), dtype=np.uint8) for _ in range(world_size)]
        self.out_s = [np.zeros((rows, hidden_dim // 128), dtype=np.float32) for _ in range(world_size)]
        self.y = [np.zeros((rows, hidden_dim), dtype=np.uint16) for _ in range(world_size)]
        self._px = (c_void_p * world_size)(*[_p(a) for a in self.out_x])
        self._ps = (c_void_p * world_size)(*[_p(a) for a in self.out_s])
        self._py = (c_void_p * world_size)(*[_p(a) for a in self.y])
        self._q = np.zeros(hidden_dim, dtype=np.uint8)
        self._s = np.zeros(hidden_dim // 128, dtype=np.float32)
        self._acc = np.zeros(hidden_dim, dtype=np.float32)

    def route_all(self, indices_per_rank):
        self.idx = [np.ascontiguousarray(i, dtype=np.int32) for i in indices_per_rank]
        nr = np.zeros((self.N, self.E), dtype=np.uint32)
        self.toff = []
        for g, idx in enumerate(self.idx):
            c, to, _ = route(idx, self.E) if idx.shape[0] else (np.zeros(self.E, np.uint32), np.zeros(0, np.uint32), None)
            nr[g] = c
            self.toff.append(to)
        self.num_routed = nr
        self.tpe, self.poff, self.base = layout(nr, self.node, self.pad)

    def dispatch(self, x_codes_per_rank):
        for g, x in enumerate(x_codes_per_rank):
            x = np.ascontiguousarray(x, dtype=np.uint16)
            if x.shape[0] == 0:
                continue
            lib().oracle_dispatch_rank(_p(x), self.H, _p(self.idx[g]), self.K, x.shape[0], self.H, self.K,
                                       self.Le, _p(self.toff[g]), _p(self.base[g]), self._px, self._ps,
                                       _p(self._q), _p(self._s))

    def act(self):
        for r in range(self.N):
            lib().oracle_act_rows(_p(self.out_x[r]), _p(self.out_s[r]), self.rows, self.H, _p(self.y[r]))

    def combine(self, weights_per_rank, accumulate=False, out_prev=None):
        outs = []
        for g, w in enumerate(weights_per_rank):
            w = np.ascontiguousarray(w, dtype=np.float32)
            T = w.shape[0]
            out = np.zeros((T, self.H), dtype=np.uint16) if out_prev is None else out_prev[g].copy()
            if T:
                lib().oracle_combine_rank(_p(out), self.H, _p(self.idx[g]), self.K, _p(w), self.K, T, self.H,
                                          self.K, self.Le, _p(self.toff[g]), _p(self.base[g]), self._py,
                                          1 if accumulate else 0, _p(self._acc))
            outs.append(out)
        return outs
