"""`EPBuffer` / `EPHandle`: the expert-parallel dispatch and combine API, call-compatible with the
reference's deep_ep/buffers/ep.py, backed by the gfx950 kernels of libdeep_ep_hip.so.

One GPU's share: a group of size R describes R partitions of this GPU's arena (a
`deep_ep.comm.LocalGroup`, or a torch ProcessGroup of size 1); there is no transport.
Everything runs on the caller's current stream.
"""
import os
from typing import Optional, Sequence, Tuple, Union

import torch

from .. import _C, comm
from .._C import EventHandle
from ..utils.event import EventOverlap
from ..utils.semantic import value_or
from .allocator import BufferAllocator
from .base import BufferBase

_TensorOrPair = Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]


class EPHandle:
    """What `EPBuffer.dispatch` learned about the routing; replays the layout in a cached dispatch
    and reverses it in `EPBuffer.combine`.

    Attributes (shapes as in the reference, deep_ep/buffers/ep.py:27-51):
        do_expand, num_experts, expert_alignment, num_max_tokens_per_rank, num_sms: call parameters.
        topk_idx: `[num_tokens, num_topk]` int64, held by reference; must stay unmodified.
        psum_num_recv_tokens_per_rank: `[num_ranks]` inclusive prefix sum of received tokens
            (a token counts once per partition however many of its experts live there).
        psum_num_recv_tokens_per_expert: `[num_local_experts]`; entry i = aligned total of the
            experts before i plus the exact count of expert i.
        num_unaligned_recv_tokens_per_expert: `[num_local_experts]` exact counts.
        num_recv_tokens_per_expert_list: aligned counts as a Python list (host-synced dispatch only).
        recv_src_metadata: `[num_recv_tokens, num_topk + 2]` rows `[slot_0..slot_{K-1}, source
            token, last local top-k position]`.
        dst_buffer_slot_idx / dst_gsge_idx: `[num_tokens, num_topk]` send-side slot per partition
            master, and transport descriptor ids (always -1: every copy is local).
        num_recv_tokens / num_expanded_tokens: sizes of the receive stream and of the expanded
            output (upper bounds when the dispatch did not sync with the host).
    """

    def __init__(self, do_expand: bool, num_experts: int, expert_alignment: int, num_max_tokens_per_rank: int,
                 num_sms: int, topk_idx: torch.Tensor, num_recv_tokens: int, num_expanded_tokens: int,
                 num_recv_tokens_per_expert_list: list, psum_num_recv_tokens_per_rank: torch.Tensor,
                 psum_num_recv_tokens_per_expert: torch.Tensor, num_unaligned_recv_tokens_per_expert: torch.Tensor,
                 recv_src_metadata: torch.Tensor, dst_buffer_slot_idx: torch.Tensor, dst_gsge_idx: torch.Tensor):
        assert topk_idx is not None
        self.do_expand, self.num_experts, self.expert_alignment = do_expand, num_experts, expert_alignment
        self.num_max_tokens_per_rank, self.num_sms = num_max_tokens_per_rank, num_sms
        self.num_recv_tokens, self.num_expanded_tokens = num_recv_tokens, num_expanded_tokens
        self.num_recv_tokens_per_expert_list = num_recv_tokens_per_expert_list
        self.psum_num_recv_tokens_per_rank = psum_num_recv_tokens_per_rank
        self.psum_num_recv_tokens_per_expert = psum_num_recv_tokens_per_expert
        self.num_unaligned_recv_tokens_per_expert = num_unaligned_recv_tokens_per_expert
        self.recv_src_metadata = recv_src_metadata
        self.dst_buffer_slot_idx, self.dst_gsge_idx = dst_buffer_slot_idx, dst_gsge_idx
        self.cached_recv_src_metadata_before_sort = None
        self._topk_idx = topk_idx
        # inference tensors carry no version counter
        self._topk_idx_version = None if topk_idx.is_inference() else topk_idx._version

    @property
    def topk_idx(self) -> torch.Tensor:
        if self._topk_idx_version is not None:
            assert self._topk_idx._version == self._topk_idx_version, \
                '`topk_idx` must not be modified while the EP handle is in use'
        return self._topk_idx

    def deterministic_sort(self, do_cpu_sync: bool, is_cached_dispatch: bool, recv_x: torch.Tensor,
                           recv_sf: Optional[torch.Tensor], recv_topk_weights: Optional[torch.Tensor]) -> None:
        """The reference sorts each expert's rows by source token after the fact
        (deep_ep/buffers/ep.py:100-160).  The layout kernels here already assign slots in that
        order -- by (source token, top-k position) inside every expert, padding last -- so the
        expanded tensors and `recv_src_metadata` are canonical as produced and nothing moves."""
        if not is_cached_dispatch:
            self.cached_recv_src_metadata_before_sort = self.recv_src_metadata
        assert self.cached_recv_src_metadata_before_sort is not None


class EPBuffer(BufferBase):
    """Expert-parallel dispatch/combine with the expanded (one row per token-expert pair) layout.

    Stream usage: every operation is enqueued on the current stream.
    """

    barrier = comm.barrier
    get_comm_stream = comm.get_comm_stream
    get_physical_domain_size = comm.get_physical_domain_size
    get_logical_domain_size = comm.get_logical_domain_size

    def __init__(self, group, num_bytes: Optional[int] = None, num_max_tokens_per_rank: int = 0, hidden: int = 0,
                 num_topk: int = 0, use_fp8_dispatch: bool = False,
                 lb_allocation_plan_or_num_bytes: Union[BufferAllocator, int] = 0, deterministic: bool = False,
                 allow_hybrid_mode: bool = True, allow_multiple_reduction: bool = True,
                 prefer_overlap_with_compute: bool = True, sl_idx: Optional[int] = None, num_allocated_qps: int = 0,
                 num_cpu_timeout_secs: int = 300, num_gpu_timeout_secs: int = 100, explicitly_destroy: bool = False,
                 *, use_huge1g_page: bool = True):
        """`group` needs `rank()` and `size()`.  `num_bytes` (without workspace) must be a multiple
        of `get_num_allocation_alignment()`; when None it comes from `get_buffer_size_hint`.
        Load-balancing storage can be reserved; the load-balancing kernels, RDMA service levels
        and explicit QP counts do not exist here."""
        if sl_idx is not None or num_allocated_qps != 0:
            raise NotImplementedError('RDMA service levels and QP configuration are not implemented')
        if not allow_multiple_reduction:
            raise AssertionError('allow_multiple_reduction=True is required')
        if min(num_cpu_timeout_secs, num_gpu_timeout_secs) <= 0:
            raise AssertionError('time-outs are positive numbers of seconds')
        granule = _C.get_num_allocation_alignment()

        # load-balancing storage: a byte count, or a plan whose tensors get their memory below
        lb_plan = lb_allocation_plan_or_num_bytes
        if isinstance(lb_plan, BufferAllocator):
            assert not lb_plan.materialized, 'the allocation plan already has storage'
            num_lb_bytes = lb_plan.num_bytes
        else:
            lb_plan, num_lb_bytes = None, lb_allocation_plan_or_num_bytes
        if not isinstance(num_lb_bytes, int) or num_lb_bytes < 0 or num_lb_bytes % granule:
            raise AssertionError(f'load-balancing storage must be a non-negative multiple of {granule} bytes')

        if num_bytes is None:
            num_bytes = self.get_buffer_size_hint(group, num_max_tokens_per_rank, hidden, num_topk, use_fp8_dispatch,
                                                  allow_hybrid_mode, allow_multiple_reduction)
        if num_bytes < 0 or num_bytes % granule:
            raise AssertionError(f'num_bytes must be a non-negative multiple of {granule}')

        super().__init__(explicitly_destroy)
        rank_idx, num_ranks = group.rank(), group.size()
        vars(self).update(
            group=group, rank_idx=rank_idx, num_ranks=num_ranks, num_bytes=num_bytes, num_lb_bytes=num_lb_bytes,
            num_max_tokens_per_rank=num_max_tokens_per_rank, deterministic=deterministic, num_allocated_qps=0,
            allow_hybrid_mode=allow_hybrid_mode, allow_multiple_reduction=allow_multiple_reduction,
            prefer_overlap_with_compute=prefer_overlap_with_compute,
            hccl_comm_handle=comm.get_hccl_comm_handle(group))
        if os.environ.get('EP_BUFFER_DEBUG'):
            print(f'EP buffer of partition {rank_idx}/{num_ranks}: {num_bytes} bytes + {num_lb_bytes} bytes of storage')

        self._num_compute_units = None
        self.runtime = _C.EPBuffer(rank_idx, num_ranks, self.hccl_comm_handle.get(), num_bytes, num_lb_bytes,
                                   use_huge1g_page, num_cpu_timeout_secs, num_gpu_timeout_secs, explicitly_destroy)
        self.context = self.runtime.context
        node = getattr(group, 'node', None)
        if node is not None:
            node.register(rank_idx, self.runtime)           # the last partition of a node connects them all
        if lb_plan is not None:
            lb_plan.materialize(self.runtime.lb_storage)

        # everything is directly addressable here: one "scale-out" domain holding all partitions
        self.num_scaleout_ranks, self.num_scaleup_ranks = self.get_logical_domain_size()
        self.scaleout_rank_idx, self.scaleup_rank_idx = divmod(rank_idx, self.num_scaleup_ranks)
        self.num_rdma_ranks, self.num_nvlink_ranks = self.get_physical_domain_size()
        torch.cuda.synchronize()

    def destroy(self) -> None:
        super().destroy()
        self.context = self.hccl_comm_handle = None

    def set_exact_sync_sizes(self, enable: bool = True) -> None:
        """No counterpart in the reference (an allocation policy of this library).  By default a dispatch with
        `do_cpu_sync=True` on a single partition allocates its outputs for the call's upper bound, enqueues the copy at
        once and returns views narrowed to the exact sizes, which keep the bound-sized storage alive.  With this switch
        on, such a dispatch waits for the counts first and allocates exactly what its results show, as the reference
        does; the GPU then idles between the layout kernels and the copy (about 10 microseconds a call)."""
        self.runtime.set_exact_sync_sizes(enable)

    @staticmethod
    def get_buffer_size_hint(group, num_max_tokens_per_rank: int, hidden: int, num_topk: int = 0,
                             use_fp8_dispatch: bool = False, allow_hybrid_mode: bool = True,
                             allow_multiple_reduction: bool = True) -> int:
        """Recommended `num_bytes` (2 MiB aligned) for these settings, without building a buffer."""
        assert allow_multiple_reduction
        return _C.calculate_ep_buffer_size(group.size(), num_max_tokens_per_rank, hidden, num_topk, use_fp8_dispatch)

    @staticmethod
    def capture() -> EventHandle:
        """Record an event on the current stream."""
        return EventHandle()

    def get_theoretical_num_sms(self, num_experts: int, num_topk: int, num_scaleout_topk: int = 0,
                                rdma_gbs: float = 0, nvlink_gbs: float = 0,
                                sm_read_gbs: float = 0, sm_write_gbs: float = 0) -> int:
        # launches size themselves; the figure only travels in the handle (asked of the device once)
        if self._num_compute_units is None:
            self._num_compute_units = _C.get_num_ai_cores()
        return self._num_compute_units

    def get_theoretical_num_qps(self, num_sms: int) -> int:
        return 0

    # ------------------------------------------------------------------------------------------
    def dispatch(self, x: _TensorOrPair, topk_idx: Optional[torch.Tensor] = None,
                 topk_weights: Optional[torch.Tensor] = None,
                 cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
                 num_experts: Optional[int] = None, num_max_tokens_per_rank: Optional[int] = None,
                 expert_alignment: Optional[int] = None, num_sms: int = 0, num_qps: int = 0,
                 previous_event: Optional[EventHandle] = None, async_with_compute_stream: bool = False,
                 allocate_on_comm_stream: bool = False, handle: Optional[EPHandle] = None,
                 do_handle_copy: bool = False, do_cpu_sync: Optional[bool] = None, do_expand: bool = False,
                 do_zero_padding: bool = False, use_tma_aligned_col_major_sf: bool = False,
                 defer_epilogue: bool = False, *, fused_fp8_quant: bool = False):
        """Send every token to the experts it selected.

        Arguments (as the reference, deep_ep/buffers/ep.py:340-375):
            x: `[num_tokens, hidden]` bfloat16, or the FP8 pair (`[num_tokens, hidden]`
                float8_e4m3fn, `[num_tokens, num_sf_packs]` 2-byte scale packs, either stride 1).
            topk_idx: `[num_tokens, num_topk]` int64, -1 = no selection; None with a `handle`.
            topk_weights: `[num_tokens, num_topk]` float32, optional (also with a cached handle).
            cumulative_local_expert_recv_stats: `[num_local_experts]` int32 running counter.
            num_experts, num_max_tokens_per_rank, expert_alignment: layout parameters (taken
                from the handle when one is given; alignment defaults to 1).
            num_sms: recorded in the handle; launches size themselves.  num_qps must be 0.
            previous_event: an `EventHandle` the current stream waits for before anything is enqueued.
            allocate_on_comm_stream: accepted and ignored (there is one stream).
            async_with_compute_stream: also return an event for the enqueued work.
            handle: a previous `EPHandle` to replay (no layout pass, no host sync).
            do_cpu_sync: read exact counts on the host (default True without a handle); otherwise
                outputs have worst-case sizes.  With one partition the outputs are allocated for
                this call's own upper bound (`num_tokens * min(num_topk, num_local_experts) +
                (expert_alignment - 1) * num_local_experts` rows) so that the copy can be enqueued
                before the host has the counts, and are returned as views narrowed to the exact
                sizes: while such a view is alive it keeps the whole bound-sized allocation (up to
                about 15 % more rows than its shape shows under uniform routing); `.clone()` it to
                hold only the rows shown, or call `set_exact_sync_sizes()` on the buffer once.  An epilogue deferred with `defer_epilogue` must run
                before the next non-cached dispatch is launched on this buffer: the library
                refuses an epilogue whose dispatch is no longer the buffer's latest.
            do_expand: must be True.  do_handle_copy must be False.
            do_zero_padding: zero the alignment padding rows of the outputs.
            use_tma_aligned_col_major_sf: return the FP8 scales column-major.
            defer_epilogue: return only the `EventOverlap`; `event.current_stream_wait()` then
                runs the copy epilogue and returns `(recv_x, None, recv_topk_weights, handle)`.
            fused_fp8_quant (extension): `x` is bfloat16 and is quantised to e4m3fn with one fp32
                scale per token and 128 channels on the way; returns `(recv_x_fp8, recv_sf_fp32)`
                whose bytes equal `deep_ep.utils.math.per_token_cast_to_fp8(x)` dispatched verbatim, for
                `x` on the GPU (the library's quantiser kernel) and on the CPU (torch's evaluation of
                the reference formula) alike.

        Returns `(recv_x or (recv_x, recv_sf), None, recv_topk_weights, handle, event)`, or the
        `EventOverlap` alone when `defer_epilogue`.
        """
        if num_qps:
            self._no_explicit_qps(num_qps)
        if do_handle_copy:
            raise AssertionError('`do_handle_copy` must be False; handle copying is no longer supported')
        if not do_expand:
            raise AssertionError('only do_expand=True is supported')
        payload, sf = x if isinstance(x, tuple) else (x, None)

        replay = handle is not None
        if replay:
            # the handle fixes the routing and every layout parameter; explicit values may only repeat them
            assert topk_idx is None, 'a cached dispatch takes its routing from the handle'
            assert not do_cpu_sync, 'Cannot do CPU sync with cached handle'
            assert handle.do_expand == do_expand
            layout = (value_or(num_experts, handle.num_experts), value_or(expert_alignment, handle.expert_alignment),
                      value_or(num_max_tokens_per_rank, handle.num_max_tokens_per_rank))
            assert layout == (handle.num_experts, handle.expert_alignment, handle.num_max_tokens_per_rank)
            num_experts, expert_alignment, num_max_tokens_per_rank = layout
            topk_idx, num_sms, do_cpu_sync = handle.topk_idx, handle.num_sms, False
            cached_fields = tuple(getattr(handle, name) for name in self._RUNTIME_CACHED_ORDER)
        else:
            if num_max_tokens_per_rank is None:
                num_max_tokens_per_rank = self.num_max_tokens_per_rank
            if expert_alignment is None:
                expert_alignment = 1
            if do_cpu_sync is None:
                do_cpu_sync = True
            num_sms = num_sms or self._num_compute_units or self.get_theoretical_num_sms(num_experts, topk_idx.size(1))
            cached_fields = self._NO_CACHED_FIELDS

        result, event, deferred = self.runtime.dispatch(
            payload, sf, topk_idx, topk_weights, cumulative_local_expert_recv_stats, *cached_fields,
            num_max_tokens_per_rank, num_experts, expert_alignment, num_sms, previous_event,
            async_with_compute_stream, allocate_on_comm_stream, do_handle_copy, do_cpu_sync, do_expand,
            do_zero_padding, use_tma_aligned_col_major_sf, defer_epilogue, fused_fp8_quant=fused_fp8_quant)
        overlap = EventOverlap(event)

        def finish(native_result: tuple, sort_when_waited: bool):
            recv_x, recv_sf, recv_topk_weights, *layout_fields = native_result
            this_handle = handle if replay else EPHandle(do_expand, num_experts, expert_alignment,
                                                         num_max_tokens_per_rank, num_sms, topk_idx, *layout_fields)
            if self.deterministic:
                def canonical_order():
                    this_handle.deterministic_sort(do_cpu_sync, replay, recv_x, recv_sf, recv_topk_weights)
                if sort_when_waited:
                    overlap.register_hook_after_wait(canonical_order)
                else:
                    canonical_order()
            received = recv_x if recv_sf is None else (recv_x, recv_sf)
            return received, None, recv_topk_weights, this_handle

        if deferred is None:
            return (*finish(result, async_with_compute_stream), overlap)
        overlap.register_hook_after_wait(lambda: finish(deferred(), False))
        return overlap

    _NO_CACHED_FIELDS = (None,) * 9
    # order in which the native runtime takes the fields of a cached handle (csrc/buffers/ep.hpp:96-104)
    _RUNTIME_CACHED_ORDER = ('num_recv_tokens', 'num_expanded_tokens', 'num_recv_tokens_per_expert_list',
                             'psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
                             'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'dst_gsge_idx',
                             'recv_src_metadata')

    @staticmethod
    def _no_explicit_qps(num_qps) -> None:
        if num_qps:
            raise NotImplementedError('Explicit QP counts are not implemented')

    @staticmethod
    def _unpack_bias(bias) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """None, one tensor, or a pair -> always a pair."""
        if bias is None:
            return None, None
        if torch.is_tensor(bias):
            return bias, None
        first, second = bias
        return first, second

    def combine(self, x: torch.Tensor, handle: EPHandle, topk_weights: Optional[torch.Tensor] = None,
                bias: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]] = None, num_sms: int = 0,
                num_qps: int = 0, previous_event: EventHandle = None, async_with_compute_stream: bool = False,
                allocate_on_comm_stream: bool = False, defer_epilogue: bool = False, *,
                apply_weights: bool = False):
        """Reduce expert outputs back to token order.

        Arguments (as the reference, deep_ep/buffers/ep.py:536-550):
            x: `[num_expanded_tokens, hidden]` bfloat16 expert outputs in the dispatch layout.
            handle: the `EPHandle` of the dispatch being reversed.
            topk_weights: `[num_expanded_tokens]` float32; carried back to `[num_tokens, num_topk]`.
            bias: None, one tensor or a pair of `[num_tokens, hidden]` bfloat16 added at the end.
            num_sms: ignored, the handle's value is used; num_qps must be 0.
            defer_epilogue: return only the `EventOverlap`; `event.current_stream_wait()` runs the
                final reduce and returns `(combined_x, combined_topk_weights)`.
            apply_weights (extension): multiply each row by its gate weight before the fp32 sum
                (the reference leaves the gate to the expert GEMM and sums rows unweighted).

        Returns `(combined_x, combined_topk_weights, event)`, or the `EventOverlap` alone.
        """
        if num_qps:
            self._no_explicit_qps(num_qps)
        if handle.recv_src_metadata is None:
            raise AssertionError('the handle comes from a dispatch that ran its epilogue')
        bias_0, bias_1 = self._unpack_bias(bias)
        result, event, deferred = self.runtime.combine(
            x, topk_weights, bias_0, bias_1, handle.recv_src_metadata, handle.topk_idx,
            handle.psum_num_recv_tokens_per_rank, handle.num_experts, handle.num_max_tokens_per_rank,
            handle.num_sms, previous_event, async_with_compute_stream, allocate_on_comm_stream, defer_epilogue,
            apply_weights=apply_weights)
        overlap = EventOverlap(event)
        if deferred is None:
            return (*result, overlap)
        overlap.register_hook_after_wait(deferred)
        return overlap

    # ---- load-balancing entry points: storage exists, kernels do not (csrc/buffers/ep.hpp:75-86) ----
    def lb_get_theoretical_num_sms(self) -> int:
        return _C.get_num_ai_cores()

    def lb_prefetch_weights(self, redundant_expert_weights: Union[Sequence[torch.Tensor], torch.Tensor],
                            expert_weights: Union[Sequence[torch.Tensor], torch.Tensor],
                            redundancy_mapping: torch.Tensor, num_sms: int = 0,
                            previous_event: Optional[EventHandle] = None) -> EventOverlap:
        return EventOverlap(self.runtime.lb_prefetch_weights(
            redundant_expert_weights, expert_weights, redundancy_mapping, num_sms, previous_event))

    def lb_reduce_grads(self, redundant_expert_grads: torch.Tensor, expert_grads: torch.Tensor,
                        redundancy_mapping: torch.Tensor, num_sms: int = 0,
                        previous_event: Optional[EventHandle] = None) -> EventOverlap:
        return EventOverlap(self.runtime.lb_reduce_grads(
            redundant_expert_grads, expert_grads, redundancy_mapping, num_sms, previous_event))
