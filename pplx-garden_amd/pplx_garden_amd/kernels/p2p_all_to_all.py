"""`P2PAllToAll`: the MoE dispatch / combine operator, one object per logical rank.

Same constructor keywords, method signatures, tensor checks and per-expert
receive counts as the reference's operator
(python/pplx_garden/kernels/p2p_all_to_all.py:50-534).  What differs:

* `global_group` is a `LoopbackGroup`: all ranks live on one GPU, so the
  constructor sets up no transport (no topology detection, RDMA registration or
  peer-memory exchange, p2p_all_to_all.py:116-278).
* a call with `do_send and do_recv` is a collective: it runs when every rank of
  the world has made it, in one launch sequence that moves every row once.
  Calls with only `do_send` or only `do_recv` run at once, rank by rank, through
  staging buffers; every send of a step must come before the first recv.
* ranks of one `dp_group` must pass the same tokens, indices and weights, as in the reference
  (only one of them sends each copy, all of them receive the combined tokens).
* `dp_x` may be bfloat16 while `in_dtype` is float8_e4m3fn and `dp_x_scale` is
  None: dispatch then quantises, one float32 scale per 128 elements
  (`hidden_dim_scale` must be `hidden_dim // 128`).  The reference only
  transports rows the caller has already quantised.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from pplx_garden_amd.distributed.loopback import LoopbackGroup
from pplx_garden_amd.kernels.all_to_all import AllToAllKernel
from pplx_garden_amd.native.p2p_all_to_all import (
    A2ACombineArgs,
    A2ADispatchArgs,
    AllToAllContext,
)
from pplx_garden_amd.utils.math import ceil_div, round_up

QUANT_GROUP = 128


def _current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class P2PAllToAll(AllToAllKernel):
    def __init__(
        self,
        *,
        max_num_tokens: int,
        num_experts: int,
        expert_padding: int,
        hidden_dim: int,
        hidden_dim_scale: Optional[int],
        in_dtype: torch.dtype,
        out_dtype: torch.dtype,
        scale_dtype: Optional[torch.dtype],
        num_experts_per_token: int,
        nets_per_gpu: int = 1,
        max_private_tokens: Optional[int] = None,
        device: torch.device,
        dp_group: Optional[Any] = None,
        node_group: Optional[Any] = None,
        global_group: LoopbackGroup,
    ) -> None:
        del nets_per_gpu  # no NICs in loopback
        self._hidden_dim = hidden_dim
        self._hidden_dim_scale = hidden_dim_scale
        self._num_experts_per_token = num_experts_per_token
        self._in_dtype = in_dtype
        self._out_dtype = out_dtype
        self._scale_dtype = scale_dtype
        self._device = torch.device(device)
        self._global_group = global_group
        self._all_to_all: Optional[AllToAllContext] = None

        if not isinstance(global_group, LoopbackGroup):
            raise TypeError("global_group must be a LoopbackGroup (see LoopbackWorld.group)")
        # Number of ranks that hold the same tokens (p2p_all_to_all.py:80-87).
        if dp_group is not None:
            self._dp_size = dp_group.size
            if node_group is None and global_group.node_size % dp_group.size != 0:
                node_group = dp_group
        else:
            self._dp_size = 1

        rank = global_group.rank
        world_size = global_group.size
        node_size = node_group.size if node_group is not None else global_group.node_size
        if world_size % node_size != 0:
            raise ValueError(f"node size {node_size} does not divide world size {world_size}")
        self._rank = rank
        self._world_size = world_size
        num_dp_groups = world_size // self._dp_size
        self._num_local_experts = ceil_div(num_experts, world_size)

        max_private_tokens, max_recv_tokens = self.receive_capacity(
            max_num_tokens=max_num_tokens, num_experts=num_experts, expert_padding=expert_padding,
            num_experts_per_token=num_experts_per_token, world_size=world_size, dp_size=self._dp_size,
            max_private_tokens=max_private_tokens)
        self.max_recv_tokens = max_recv_tokens
        self.max_private_tokens = max_private_tokens

        if hidden_dim_scale is not None or scale_dtype is not None:
            assert scale_dtype is not None
            assert hidden_dim_scale is not None
            # the reference supports no other scale type either (p2p_all_to_all.py:164-165)
            assert scale_dtype == torch.float32

        device_index = self._device.index
        if device_index is None:
            device_index = torch.cuda.current_device()

        self._key = (
            hidden_dim, hidden_dim_scale, in_dtype, out_dtype, scale_dtype, max_num_tokens,
            max_recv_tokens, max_private_tokens, num_experts, expert_padding,
            num_experts_per_token, node_size, world_size, device_index, self._dp_size,
        )

        def make_context() -> AllToAllContext:
            return AllToAllContext.create(
                hidden_dim=hidden_dim,
                hidden_dim_scale=hidden_dim_scale,
                in_elemsize=in_dtype.itemsize,
                out_elemsize=out_dtype.itemsize,
                out_dtype=out_dtype,
                scale_elemsize=scale_dtype.itemsize if scale_dtype else None,
                max_num_tokens=max_num_tokens,
                max_recv_tokens=max_recv_tokens,
                max_private_tokens=max_private_tokens,
                num_experts=num_experts,
                expert_padding=expert_padding,
                num_experts_per_token=num_experts_per_token,
                dp_size=self._dp_size,
                node_size=node_size,
                world_size=world_size,
                device=device_index,
                flags=getattr(global_group.world, "context_flags", 0),
            )

        self._all_to_all = global_group.world.acquire_context(self._key, make_context)

    # ------------------------------------------------------------------

    @staticmethod
    def receive_capacity(*, max_num_tokens: int, num_experts: int, expert_padding: int,
                         num_experts_per_token: int, world_size: int, dp_size: int = 1,
                         max_private_tokens: Optional[int] = None):
        """(max_private_tokens, max_recv_tokens): rows of a rank's receive region as the reference
        sizes them (p2p_all_to_all.py:94-114).  Every dp group gets a private region (by default 1.2
        times the average load of the rank's experts); on top of that come the rows all groups share:
        every copy of every group's tokens could land here, but no more than one per (token, local
        expert), and never less than one padded block per local expert."""
        groups = world_size // dp_size
        local_experts = ceil_div(num_experts, world_size)
        if max_private_tokens is None:
            average = int(ceil_div(max_num_tokens * num_experts_per_token, num_experts) * 1.2)
            max_private_tokens = average * local_experts
        assert max_private_tokens >= 0
        tokens = max_num_tokens * groups
        every_copy = tokens * num_experts_per_token + local_experts * (expert_padding - 1)
        shared = max(min(every_copy, tokens * local_experts), local_experts * expert_padding)
        return max_private_tokens, max_private_tokens * groups + round_up(shared, expert_padding)

    @property
    def num_local_experts(self) -> int:
        return self._num_local_experts

    @property
    def context(self) -> AllToAllContext:
        assert self._all_to_all is not None
        return self._all_to_all

    def _is_quantize(self, dp_x: torch.Tensor, dp_x_scale: Optional[torch.Tensor]) -> bool:
        return (
            dp_x_scale is None
            and dp_x.dtype == torch.bfloat16
            and self._in_dtype == torch.float8_e4m3fn
            and self._hidden_dim_scale is not None
        )

    def dispatch(
        self,
        out_expert_num_tokens: torch.Tensor,
        out_expert_x: torch.Tensor,
        out_expert_x_scale: Optional[torch.Tensor],
        dp_x: torch.Tensor,
        dp_x_scale: Optional[torch.Tensor],
        indices: torch.Tensor,
        weights: torch.Tensor,
        bound_m: Optional[torch.Tensor] = None,
        do_send: bool = True,
        do_recv: bool = True,
    ) -> None:
        assert self._all_to_all is not None
        assert do_send or do_recv

        num_tokens, _ = dp_x.shape

        # Output count buffer (p2p_all_to_all.py:336-340).
        assert out_expert_num_tokens.shape == (self._num_local_experts,)
        assert out_expert_num_tokens.stride(0) == 1
        assert out_expert_num_tokens.dtype == torch.int32

        # Output token buffer (p2p_all_to_all.py:342-348).
        num_expert_tokens, _ = out_expert_x.shape
        assert out_expert_x.shape == (num_expert_tokens, self._hidden_dim)
        assert out_expert_x.stride(1) == 1
        assert out_expert_x.dtype == self._in_dtype
        out_x_stride = out_expert_x.stride(0) * out_expert_x.dtype.itemsize

        # Output scale buffer (p2p_all_to_all.py:350-362).
        if out_expert_x_scale is not None:
            assert out_expert_x_scale.dtype == self._scale_dtype
            out_x_scale_ptr = out_expert_x_scale.data_ptr()
            out_x_scale_stride_elem = out_expert_x_scale.stride(1)
            out_x_scale_stride_token = out_expert_x_scale.stride(0)
        else:
            out_x_scale_ptr = None
            out_x_scale_stride_elem = None
            out_x_scale_stride_token = None

        # Input tokens (p2p_all_to_all.py:364-369), plus the quantising mode.
        quantize = self._is_quantize(dp_x, dp_x_scale)
        assert dp_x.shape == (num_tokens, self._hidden_dim)
        assert dp_x.stride(1) == 1
        if quantize:
            assert self._hidden_dim % QUANT_GROUP == 0
            assert self._hidden_dim_scale == self._hidden_dim // QUANT_GROUP
            assert self._scale_dtype == torch.float32
            assert out_expert_x_scale is not None
        else:
            assert dp_x.dtype == self._in_dtype
        x_stride = dp_x.stride(0) * dp_x.dtype.itemsize

        # Input scales (p2p_all_to_all.py:371-388).
        if dp_x_scale is not None:
            assert self._scale_dtype is not None
            assert self._hidden_dim_scale is not None
            assert out_expert_x_scale is not None
            assert dp_x_scale.dtype == self._scale_dtype
            x_scale_ptr = dp_x_scale.data_ptr()
            x_scale_stride_elem = dp_x_scale.stride(1)
            x_scale_stride_token = dp_x_scale.stride(0)
        else:
            if not quantize:
                assert self._scale_dtype is None
                assert self._hidden_dim_scale is None
            x_scale_ptr = None
            x_scale_stride_elem = None
            x_scale_stride_token = None

        # Indices and weights (p2p_all_to_all.py:390-402).
        assert indices.shape == (num_tokens, self._num_experts_per_token)
        assert indices.stride(1) == 1
        assert indices.dtype == torch.uint32
        assert weights.shape == (num_tokens, self._num_experts_per_token)
        assert weights.stride(1) == 1
        assert weights.dtype == torch.float32

        # Dynamic bound on the number of tokens (p2p_all_to_all.py:404-411).
        if bound_m is not None:
            assert bound_m.numel() == 1
            assert bound_m.dtype == torch.int32
            bound_m_ptr = bound_m.data_ptr()
        else:
            bound_m_ptr = None

        stream = _current_stream(self._device)

        if do_send and do_recv:
            args = A2ADispatchArgs(
                num_tokens=num_tokens, x_ptr=dp_x.data_ptr() or None, x_stride=x_stride,
                x_scale_ptr=x_scale_ptr, x_scale_stride_elem=x_scale_stride_elem or 0,
                x_scale_stride_token=x_scale_stride_token or 0,
                indices=indices.data_ptr() or None, indices_stride=indices.stride(0),
                weights=weights.data_ptr() or None, weights_stride=weights.stride(0),
                bound_m=bound_m_ptr, out_num_tokens=out_expert_num_tokens.data_ptr(),
                out_x=out_expert_x.data_ptr() or None, out_x_stride=out_x_stride,
                out_x_rows=num_expert_tokens, out_x_scale=out_x_scale_ptr,
                out_x_scale_stride_elem=out_x_scale_stride_elem or 0,
                out_x_scale_stride_token=out_x_scale_stride_token or 0)
            # keep the tensors alive until the collective has been launched
            keep = (out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x, dp_x_scale,
                    indices, weights, bound_m)
            posted = self._global_group.world.post(
                self._key, "dispatch", self._rank, (args, quantize, keep))
            if posted is not None:
                modes = {q for _, q, _ in posted}
                if len(modes) != 1:
                    raise RuntimeError("every rank must call dispatch() in the same mode")
                self._all_to_all.dispatch([a for a, _, _ in posted], modes.pop(), stream)
            return

        if do_send:
            self._all_to_all.dispatch_send(
                rank=self._rank,
                num_tokens=num_tokens,
                x_ptr=dp_x.data_ptr(),
                x_stride=x_stride,
                x_scale_ptr=x_scale_ptr,
                x_scale_stride_elem=x_scale_stride_elem,
                x_scale_stride_token=x_scale_stride_token,
                indices_ptr=indices.data_ptr(),
                indices_stride=indices.stride(0),
                weights_ptr=weights.data_ptr(),
                weights_stride=weights.stride(0),
                bound_m_ptr=bound_m_ptr,
                stream=stream,
                quantize=quantize,
            )

        if do_recv:
            self._all_to_all.dispatch_recv(
                rank=self._rank,
                out_num_tokens_ptr=out_expert_num_tokens.data_ptr(),
                out_x_ptr=out_expert_x.data_ptr(),
                out_x_stride=out_x_stride,
                out_x_rows=num_expert_tokens,
                out_x_scale_ptr=out_x_scale_ptr,
                out_x_scale_stride_elem=out_x_scale_stride_elem,
                out_x_scale_stride_token=out_x_scale_stride_token,
                stream=stream,
            )

    def combine(
        self,
        out_tokens: torch.Tensor,
        indices: torch.Tensor,
        weights: torch.Tensor,
        expert_y: torch.Tensor,
        bound_m: Optional[torch.Tensor] = None,
        do_send: bool = True,
        do_recv: bool = True,
        accumulate: bool = False,
    ) -> None:
        assert self._all_to_all is not None
        assert do_send or do_recv
        assert not accumulate or self._dp_size == 1

        num_tokens, _ = indices.shape
        num_recv_tokens, _ = expert_y.shape

        # p2p_all_to_all.py:463-484
        assert out_tokens.shape == (num_tokens, self._hidden_dim)
        assert out_tokens.dtype == self._out_dtype
        assert out_tokens.stride(1) == 1
        assert indices.shape == (num_tokens, self._num_experts_per_token)
        assert indices.stride(1) == 1
        assert indices.dtype == torch.uint32
        assert weights.shape == (num_tokens, self._num_experts_per_token)
        assert weights.stride(1) == 1
        assert weights.dtype == torch.float32
        assert expert_y.shape == (num_recv_tokens, self._hidden_dim)
        assert expert_y.stride(1) == 1
        expert_y_stride = expert_y.stride(0) * expert_y.dtype.itemsize

        if bound_m is not None:
            assert bound_m.numel() == 1
            assert bound_m.dtype == torch.int32
            bound_m_ptr = bound_m.data_ptr()
        else:
            bound_m_ptr = None

        stream = _current_stream(self._device)

        if do_send and do_recv:
            args = A2ACombineArgs(
                expert_y=expert_y.data_ptr() or None, expert_y_stride=expert_y_stride,
                expert_y_rows=num_recv_tokens, num_tokens=num_tokens,
                out_tokens=out_tokens.data_ptr() or None, out_tokens_stride=out_tokens.stride(0),
                indices=indices.data_ptr() or None, indices_stride=indices.stride(0),
                weights=weights.data_ptr() or None, weights_stride=weights.stride(0),
                bound_m=bound_m_ptr)
            keep = (out_tokens, indices, weights, expert_y, bound_m)
            posted = self._global_group.world.post(
                self._key, "combine", self._rank, (args, expert_y.dtype, bool(accumulate), keep))
            if posted is not None:
                dtypes = {d for _, d, _, _ in posted}
                accs = {a for _, _, a, _ in posted}
                if len(dtypes) != 1 or len(accs) != 1:
                    raise RuntimeError(
                        "every rank must call combine() with the same expert_y dtype and accumulate")
                self._all_to_all.combine([a for a, _, _, _ in posted], dtypes.pop(), accs.pop(), stream)
            return

        if expert_y.dtype.itemsize != self._out_dtype.itemsize:
            # combine-send copies staging rows sized for out_dtype without knowing the type of
            # expert_y (as the reference's does, a2a_combine_send.cu:261); narrower rows would be over-read
            raise RuntimeError(
                f"split combine needs expert_y ({expert_y.dtype}) with the element size of out_dtype "
                f"({self._out_dtype}); call combine() with do_send and do_recv for mixed types")

        if do_send:
            self._all_to_all.combine_send(
                rank=self._rank,
                expert_x_ptr=expert_y.data_ptr(),
                expert_x_stride=expert_y_stride,
                expert_x_rows=num_recv_tokens,
                stream=stream,
            )

        if do_recv:
            self._all_to_all.combine_recv(
                rank=self._rank,
                num_tokens=num_tokens,
                num_recv_tokens=num_recv_tokens,
                expert_y_dtype=expert_y.dtype,
                out_tokens_ptr=out_tokens.data_ptr(),
                out_tokens_stride=out_tokens.stride(0),
                indices_ptr=indices.data_ptr(),
                indices_stride=indices.stride(0),
                weights_ptr=weights.data_ptr(),
                weights_stride=weights.stride(0),
                bound_m_ptr=bound_m_ptr,
                accumulate=accumulate,
                stream=stream,
            )

    def destroy(self) -> None:
        """Release this rank's share of the context; the last rank frees it."""
        if self._all_to_all is not None:
            self._all_to_all = None
            self._global_group.world.release_context(self._key)
