"""Binding layer over libdeep_ep_hip.so (the C ABI declared in include/deep_ep_hip.h).

It exposes the names the reference's pybind module `deep_ep._C` exports for the EP path
(csrc/python_api.cpp:18-74): `EventHandle`, `EPBuffer` with `.dispatch(27 args)` /
`.combine(14 args)`, `calculate_ep_buffer_size`, the alignment getters, `topk_idx_t` and the
runtime-configuration functions.  Torch tensors are only plumbing here: this module allocates
outputs and passes raw device pointers plus the current HIP stream to the library.  There is no
CPU or torch fallback: if the library or its code object is missing, importing or using this
module raises.
"""
import ctypes
import os
from typing import List, Optional, Tuple

import torch

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'lib')
_LIB_PATH = os.path.join(_LIB_DIR, 'libdeep_ep_hip.so')

if not os.path.exists(_LIB_PATH):
    raise ImportError(f'{_LIB_PATH} is missing: build the native library first (python deepep-ascend_amd/deep_ep/_build.py)')

_lib = ctypes.CDLL(_LIB_PATH)


class _Tensor(ctypes.Structure):
    # ep_tensor_t; size[2] and stride[2] are spelled out so one positional constructor call fills it
    _fields_ = [('data', ctypes.c_void_p), ('dtype', ctypes.c_int32), ('ndim', ctypes.c_int32),
                ('size0', ctypes.c_int64), ('size1', ctypes.c_int64),
                ('stride0', ctypes.c_int64), ('stride1', ctypes.c_int64)]


class _DispatchArgs(ctypes.Structure):
    _fields_ = [(n, _Tensor) for n in (
        'x', 'sf', 'topk_idx', 'topk_weights', 'cumulative_local_expert_recv_stats',
        'psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
        'num_unaligned_recv_tokens_per_expert', 'dst_buffer_slot_idx', 'dst_gsge_idx')] + [
        ('num_max_tokens_per_rank', ctypes.c_int32), ('num_experts', ctypes.c_int32),
        ('expert_alignment', ctypes.c_int32), ('cached_mode', ctypes.c_int32), ('do_cpu_sync', ctypes.c_int32),
        ('fused_fp8_quant', ctypes.c_int32), ('stream', ctypes.c_void_p)]


class _DispatchEpilogueArgs(ctypes.Structure):
    _fields_ = [(n, _Tensor) for n in (
        'x', 'sf', 'topk_weights', 'psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert',
        'recv_x', 'recv_sf', 'recv_sf_staging', 'recv_topk_weights', 'recv_src_metadata')] + [
        ('num_topk', ctypes.c_int32), ('num_max_tokens_per_rank', ctypes.c_int32), ('num_experts', ctypes.c_int32),
        ('expert_alignment', ctypes.c_int32), ('cached_mode', ctypes.c_int32), ('do_zero_padding', ctypes.c_int32),
        ('fused_fp8_quant', ctypes.c_int32), ('recv_sf_layout', ctypes.c_int32), ('stream', ctypes.c_void_p),
        ('dispatch_stamp', ctypes.c_int64)]


class _DispatchRecvArgs(ctypes.Structure):
    _fields_ = [(n, _Tensor) for n in (
        'psum_num_recv_tokens_per_rank', 'psum_num_recv_tokens_per_expert', 'num_unaligned_recv_tokens_per_expert',
        'cumulative_local_expert_recv_stats', 'recv_src_metadata')] + [
        ('hidden_bytes', ctypes.c_int32), ('num_sf_packs', ctypes.c_int32), ('num_topk', ctypes.c_int32),
        ('num_max_tokens_per_rank', ctypes.c_int32), ('num_experts', ctypes.c_int32),
        ('expert_alignment', ctypes.c_int32), ('do_cpu_sync', ctypes.c_int32), ('reserved', ctypes.c_int32),
        ('stream', ctypes.c_void_p), ('dispatch_stamp', ctypes.c_int64)]


class _CombineArgs(ctypes.Structure):
    _fields_ = [(n, _Tensor) for n in (
        'x', 'topk_weights', 'bias_0', 'bias_1', 'src_metadata', 'combined_topk_idx',
        'psum_num_recv_tokens_per_rank', 'combined_x', 'combined_topk_weights')] + [
        ('num_experts', ctypes.c_int32), ('num_max_tokens_per_rank', ctypes.c_int32),
        ('apply_weights', ctypes.c_int32), ('stream', ctypes.c_void_p)]


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_c_int_p = ctypes.POINTER(ctypes.c_int)
_ep_init = _sig('ep_init', ctypes.c_int, ctypes.c_char_p)
_ep_last_error = _sig('ep_last_error', ctypes.c_char_p)
_ep_alloc_align = _sig('ep_get_num_allocation_alignment', ctypes.c_int64)
_ep_tma_align = _sig('ep_get_num_tma_alignment', ctypes.c_int64)
_ep_rdma_align = _sig('ep_get_num_rdma_alignment', ctypes.c_int64)
_ep_num_cus = _sig('ep_get_num_compute_units', ctypes.c_int)
_ep_calc_size = _sig('ep_calculate_buffer_size', ctypes.c_int64, *([ctypes.c_int] * 5))
_ep_dispatch_size = _sig('ep_get_dispatch_buffer_size', ctypes.c_int64, *([ctypes.c_int] * 6))
_ep_combine_size = _sig('ep_get_combine_buffer_size', ctypes.c_int64, *([ctypes.c_int] * 4))
_ep_host_cvt = _sig('ep_host_f32_to_e4m3fn', None, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64)
_ep_selftest = _sig('ep_fp8_selftest', ctypes.c_int, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float,
                    ctypes.POINTER(ctypes.c_uint64))
_ep_set_hw = _sig('ep_set_fp8_hw_convert', None, ctypes.c_int)
_ep_create = _sig('ep_buffer_create', ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                  ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p))
_ep_destroy = _sig('ep_buffer_destroy', ctypes.c_int, ctypes.c_void_p)
_ep_region = _sig('ep_buffer_region', ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int64))
_ep_print_mem = _sig('ep_buffer_print_memory_usage', ctypes.c_int, ctypes.c_void_p)
_ep_dispatch = _sig('ep_dispatch_launch', ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(_DispatchArgs))
_ep_wait = _sig('ep_dispatch_wait_counts', ctypes.c_int, ctypes.c_void_p, _c_int_p, _c_int_p, _c_int_p)
_ep_worst = _sig('ep_dispatch_worst_case_sizes', ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                 ctypes.c_int, ctypes.c_int, _c_int_p, _c_int_p)
_ep_dispatch_recv = _sig('ep_dispatch_recv_launch', ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(_DispatchRecvArgs))
_ep_connect = _sig('ep_buffer_connect', ctypes.c_int, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int)
_ep_set_peers = _sig('ep_buffer_set_peers', ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_int)
_ep_dispatch_epi = _sig('ep_dispatch_epilogue_launch', ctypes.c_int, ctypes.c_void_p,
                        ctypes.POINTER(_DispatchEpilogueArgs))
_ep_stamp = _sig('ep_dispatch_stamp', ctypes.c_int64, ctypes.c_void_p)
_ep_set_fold = _sig('ep_set_layout_fold_max_blocks', None, ctypes.c_int)
_ep_set_combine_cap = _sig('ep_set_combine_blocks_per_cu', None, ctypes.c_int)
_ep_dispatch_static = _sig('ep_dispatch_static_launch', ctypes.c_int, ctypes.POINTER(_DispatchArgs),
                           ctypes.POINTER(_DispatchEpilogueArgs))
_ep_combine = _sig('ep_combine_launch', ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(_CombineArgs), ctypes.c_int)


class EPException(RuntimeError):
    """Raised for contract violations and runtime failures reported by the native library."""


def _check(rc: int) -> None:
    if rc != 0:
        raise EPException(_ep_last_error().decode())


_DTYPES = {torch.bfloat16: 1, torch.float8_e4m3fn: 2, torch.int16: 3, torch.int32: 4, torch.int64: 5,
           torch.float32: 6, torch.uint8: 7}


_ABSENT = _Tensor()


def _desc(t: Optional[torch.Tensor], two_byte_packs: bool = False) -> _Tensor:
    if t is None:
        return _ABSENT
    if not t.is_cuda:
        raise EPException('every tensor handed to the EP kernels must live on the GPU')
    dtype = 3 if (two_byte_packs and t.element_size() == 2) else _DTYPES.get(t.dtype, 0)
    ptr = t.data_ptr() or _nonnull_ptr(t)
    shape, stride = t.shape, t.stride()
    if len(shape) == 2:
        return _Tensor(ptr, dtype, 2, shape[0], shape[1], stride[0], stride[1])
    assert len(shape) == 1
    return _Tensor(ptr, dtype, 1, shape[0], 0, stride[0], 0)


_dummy = {}


def _nonnull_ptr(t: torch.Tensor) -> int:
    # empty tensors have a null data pointer; the ABI uses null for "absent"
    dev = t.device.index or 0
    if dev not in _dummy:
        _dummy[dev] = torch.zeros(64, dtype=torch.uint8, device=t.device)
    return _dummy[dev].data_ptr()


def _stream() -> int:
    # raw hipStream_t of the current stream of the current device
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


# ---- module-level API -------------------------------------------------------------------------
topk_idx_t = torch.int64
_initialised = False
_barrier_in_prologue = False


def init_jit(library_root_path: Optional[str] = None) -> None:
    """Loads the ahead-of-time built gfx950 code object (there is no run-time compiler).  Safe to
    call without a GPU: the load then happens when the first buffer is created."""
    global _initialised
    if _initialised or not torch.cuda.is_available():
        return
    _check(_ep_init(None))
    _initialised = True


def get_num_allocation_alignment() -> int:
    return _ep_alloc_align()


def get_num_tma_alignment() -> int:
    return _ep_tma_align()


def get_num_rdma_alignment() -> int:
    return _ep_rdma_align()


def get_num_ai_cores() -> int:
    """Compute units of the current GPU (the role AI cores play on the reference's hardware)."""
    return _ep_num_cus()


def get_num_vec_cores() -> int:
    return _ep_num_cus()


def set_num_vec_cores(n: int) -> None:
    """Accepted for API compatibility; launches always size themselves from the work."""


def set_barrier_in_prologue(enable: bool) -> bool:
    """Profiling toggle of the reference (csrc/runtime/jit.hpp:61-69).  There is no cross-rank
    barrier on one GPU; the value is only remembered."""
    global _barrier_in_prologue
    previous, _barrier_in_prologue = _barrier_in_prologue, bool(enable)
    return previous


def calculate_ep_buffer_size(num_ranks: int, num_max_tokens_per_rank: int, hidden: int, num_topk: int,
                             use_fp8_dispatch: bool) -> int:
    n = _ep_calc_size(num_ranks, num_max_tokens_per_rank, hidden, num_topk, int(use_fp8_dispatch))
    if n < 0:
        raise EPException(_ep_last_error().decode())
    return n


def get_dispatch_buffer_size(num_max_tokens_per_rank, hidden, num_sf_packs, num_topk, element_size, num_ranks) -> int:
    return _ep_dispatch_size(num_max_tokens_per_rank, hidden, num_sf_packs, num_topk, element_size, num_ranks)


def get_combine_buffer_size(num_ranks, num_max_tokens_per_rank, hidden, num_topk) -> int:
    return _ep_combine_size(num_ranks, num_max_tokens_per_rank, hidden, num_topk)


def host_f32_to_e4m3fn(src: torch.Tensor) -> torch.Tensor:
    """fp32 CPU tensor -> e4m3fn bytes with the integer conversion the device fallback uses."""
    src = src.contiguous().float().cpu()
    dst = torch.empty(src.shape, dtype=torch.uint8)
    _ep_host_cvt(src.data_ptr(), dst.data_ptr(), src.numel())
    return dst


def fp8_selftest(first: int, count: int, limit: float) -> Tuple[int, int]:
    out = (ctypes.c_uint64 * 2)()
    _check(_ep_selftest(first, count, limit, out))
    return int(out[0]), int(out[1])


def set_fp8_hw_convert(enable: bool) -> None:
    _ep_set_hw(int(enable))


def set_combine_blocks_per_cu(num_blocks: int) -> None:
    """Tuning: workgroups of a combine kernel a compute unit holds at once (0: no cap; negative: chosen by
    top-k, the default).  Results do not depend on it."""
    _ep_set_combine_cap(int(num_blocks))


def set_layout_fold_max_blocks(num_blocks: int) -> None:
    """Tuning: up to this many layout workgroups (128 tokens each) the slot-assignment kernel sums the
    per-workgroup histograms itself; beyond, a scan kernel runs in between.  Results do not depend on it."""
    _ep_set_fold(int(num_blocks))


class EventHandle:
    """An event recorded on the current stream when constructed (csrc/utils/event.hpp:10-25)."""

    def __init__(self):
        self.event = torch.cuda.Event()
        self.event.record(torch.cuda.current_stream())

    def current_stream_wait(self) -> None:
        torch.cuda.current_stream().wait_event(self.event)


class Context:
    """The part of the reference's comm::Context the Python API reads."""

    def __init__(self, rank_idx: int, num_ranks: int):
        self.rank_idx, self.num_ranks = rank_idx, num_ranks

    def get_physical_domain_size(self) -> Tuple[int, int]:
        return 1, self.num_ranks

    def get_logical_domain_size(self) -> Tuple[int, int]:
        return 1, self.num_ranks


class _DevicePointer:
    """Exposes a raw device range to torch through the CUDA array interface."""

    def __init__(self, ptr: int, nbytes: int, owner):
        self.owner = owner
        self.__cuda_array_interface__ = {'shape': (nbytes,), 'typestr': '|u1', 'data': (ptr, False), 'version': 3,
                                         'strides': None}


class BufferBase:
    def __init__(self, explicitly_destroy: bool):
        self.explicitly_destroy = explicitly_destroy
        self.destroyed = False
        self.main_context = None


class EPBuffer(BufferBase):
    """Native EP runtime object (host side of csrc/buffers/ep.hpp)."""

    def __init__(self, rank_idx: int, num_ranks: int, group_name: str, num_bytes: int, num_lb_bytes: int,
                 use_huge1g_page: bool, num_cpu_timeout_secs: int, num_gpu_timeout_secs: int,
                 explicitly_destroy: bool):
        super().__init__(explicitly_destroy)
        if not torch.cuda.is_available():
            raise EPException('deep_ep needs a GPU: the EP kernels have no CPU path')
        init_jit()
        self.rank_idx, self.num_ranks, self.group_name = rank_idx, num_ranks, group_name
        self.num_bytes, self.num_lb_bytes = num_bytes, num_lb_bytes
        handle = ctypes.c_void_p()
        _check(_ep_create(rank_idx, num_ranks, num_bytes, num_lb_bytes, num_cpu_timeout_secs, num_gpu_timeout_secs,
                          ctypes.byref(handle)))
        self._h = handle
        self.connected = False
        self.device = torch.device('cuda', torch.cuda.current_device())
        self.context = Context(rank_idx, num_ranks)
        self.main_context = self.context
        if num_lb_bytes > 0:
            n = ctypes.c_int64()
            ptr = _ep_region(self._h, 2, ctypes.byref(n))
            self.lb_storage = torch.as_tensor(_DevicePointer(ptr, n.value, self), device=self.device)
        else:
            self.lb_storage = torch.empty(0, dtype=torch.uint8, device=self.device)

    # ---- lifecycle ----
    def destroy(self) -> None:
        if self.destroyed:
            raise EPException('Assertion exception (_C.py): not destroyed')
        self.lb_storage = None
        _check(_ep_destroy(self._h))
        self._h = None
        self.destroyed = True
        self.context = None
        self.main_context = None

    def __del__(self):
        try:
            if not self.explicitly_destroy and not self.destroyed and self._h is not None:
                self.destroy()
            if not self.destroyed:
                print('`destroy()` is not called before DeepEP EP buffer destruction, which can leak resources.',
                      flush=True)
        except Exception:
            pass

    def print_memory_usage(self) -> None:
        _check(_ep_print_mem(self._h))

    def set_peers(self, arena_bases) -> None:
        """Connects this partition alone, by address: `arena_bases[i]` is where partition i's arena (its
        `region(0)` pointer) is mapped in this process; None disconnects."""
        if arena_bases is None:
            _check(_ep_set_peers(self._h, None, 0))
            self.connected = False
            return
        table = (ctypes.c_void_p * len(arena_bases))(*arena_bases)
        _check(_ep_set_peers(self._h, table, len(arena_bases)))
        self.connected = True

    @staticmethod
    def connect(runtimes) -> None:
        """Makes the given runtime objects (partition i of n at index i) one node: packed rows, row counts
        and combine partials then go straight into the arena of the partition they are meant for."""
        handles = (ctypes.c_void_p * len(runtimes))(*[r._h for r in runtimes])
        _check(_ep_connect(handles, len(runtimes)))
        for r in runtimes:
            r.connected = True

    def region(self, which: int) -> Tuple[int, int]:
        n = ctypes.c_int64()
        ptr = _ep_region(self._h, which, ctypes.byref(n))
        return ptr, n.value

    def buffer_tensor(self) -> torch.Tensor:
        """The communication buffer of the arena (partition-major packed rows after a dispatch with more
        than one partition, the combine buffer of partials during a combine) as a uint8 tensor."""
        ptr, n = self.region(1)
        if n == 0:
            return torch.empty(0, dtype=torch.uint8, device=self.device)
        return torch.as_tensor(_DevicePointer(ptr, n, self), device=self.device)

    def lb_prefetch_weights(self, *args, **kwargs):
        raise EPException('Assertion exception: EPBuffer::lb_prefetch_weights is not implemented')

    def lb_reduce_grads(self, *args, **kwargs):
        raise EPException('Assertion exception: EPBuffer::lb_reduce_grads is not implemented')

    # ---- dispatch (argument order of csrc/buffers/ep.hpp:89-112) ----
    def dispatch(self, x, sf, topk_idx, topk_weights, cumulative_local_expert_recv_stats,
                 cached_num_recv_tokens, cached_num_expanded_tokens, cached_num_recv_tokens_per_expert_list,
                 cached_psum_num_recv_tokens_per_rank, cached_psum_num_recv_tokens_per_expert,
                 cached_num_unaligned_recv_tokens_per_expert, cached_dst_buffer_slot_idx, cached_dst_gsge_idx,
                 cached_recv_src_metadata, num_max_tokens_per_rank, num_experts, expert_alignment, num_ai_cores,
                 previous_event, async_with_compute_stream, allocate_on_comm_stream, do_handle_copy, do_cpu_sync,
                 do_expand, do_zero_padding, use_col_major_sf, defer_epilogue, fused_fp8_quant=False):
        if self.destroyed:
            raise EPException('Assertion exception (_C.py): not destroyed')
        if previous_event is not None:
            previous_event.current_stream_wait()       # the launches below are ordered behind it
        if not do_expand:
            raise EPException('Assertion exception (_C.py): do_expand')
        if do_handle_copy:
            raise EPException('Assertion exception (_C.py): not do_handle_copy')
        if num_ai_cores <= 0:
            raise EPException('Assertion exception (_C.py): num_ai_cores > 0')
        cached_mode = cached_num_recv_tokens is not None
        if cached_mode:
            for item in (cached_num_expanded_tokens, cached_num_recv_tokens_per_expert_list,
                         cached_psum_num_recv_tokens_per_rank, cached_psum_num_recv_tokens_per_expert,
                         cached_num_unaligned_recv_tokens_per_expert, cached_dst_buffer_slot_idx,
                         cached_dst_gsge_idx, cached_recv_src_metadata):
                if item is None:
                    raise EPException('Assertion exception (_C.py): cached handle field has a value')
        if x.dim() != 2 or topk_idx.dim() != 2:
            raise EPException('Assertion exception (_C.py): x.dim() == 2 and topk_idx.dim() == 2')
        num_tokens, hidden = x.shape
        num_topk = topk_idx.size(1)
        num_local_experts = num_experts // self.num_ranks
        dev = x.device

        def ints(*shape):
            return torch.empty(shape, dtype=torch.int32, device=dev)

        if cached_mode:
            psum_rank, psum_expert = cached_psum_num_recv_tokens_per_rank, cached_psum_num_recv_tokens_per_expert
            unaligned = cached_num_unaligned_recv_tokens_per_expert
            dst_slot, dst_gsge = cached_dst_buffer_slot_idx, cached_dst_gsge_idx
        else:
            psum_rank, psum_expert, unaligned = ints(self.num_ranks), ints(num_local_experts), ints(num_local_experts)
            dst_slot, dst_gsge = ints(num_tokens, num_topk), ints(num_tokens, num_topk)

        a = _DispatchArgs()
        a.x, a.sf = _desc(x), _desc(sf, two_byte_packs=True)
        a.topk_idx, a.topk_weights = _desc(topk_idx), _desc(topk_weights)
        a.cumulative_local_expert_recv_stats = _desc(cumulative_local_expert_recv_stats)
        a.psum_num_recv_tokens_per_rank, a.psum_num_recv_tokens_per_expert = _desc(psum_rank), _desc(psum_expert)
        a.num_unaligned_recv_tokens_per_expert = _desc(unaligned)
        a.dst_buffer_slot_idx, a.dst_gsge_idx = _desc(dst_slot), _desc(dst_gsge)
        a.num_max_tokens_per_rank, a.num_experts, a.expert_alignment = num_max_tokens_per_rank, num_experts, expert_alignment
        a.cached_mode, a.do_cpu_sync, a.fused_fp8_quant = int(cached_mode), int(do_cpu_sync), int(fused_fp8_quant)
        a.stream = _stream()
        _check(_ep_dispatch(self._h, ctypes.byref(a)))
        # the epilogue below belongs to this launch: the library refuses it once a later dispatch has
        # taken over the buffer's workspace
        stamp = _ep_stamp(self._h)

        keep_alive = (x, sf, topk_idx, topk_weights, psum_rank, psum_expert)

        def epilogue():
            # the descriptors hold raw pointers: the inputs stay referenced until the copy kernel is enqueued
            assert keep_alive is not None
            per_expert_list: List[int] = []
            partitioned = self.num_ranks > 1
            # rows that can arrive: this partition's own tokens, or everybody's when the partitions form a node
            rows_bound = self.num_ranks * num_max_tokens_per_rank if self.connected else num_tokens
            recv_src_metadata = None
            if partitioned and not cached_mode:
                # receive side: count and rank the rows that arrived in this partition's regions
                c_recv, c_exp = ctypes.c_int(), ctypes.c_int()
                _check(_ep_worst(self._h, num_max_tokens_per_rank, num_topk, num_experts, expert_alignment,
                                 ctypes.byref(c_recv), ctypes.byref(c_exp)))
                recv_src_metadata = ints(rows_bound if do_cpu_sync else c_recv.value, num_topk + 2)
                r = _DispatchRecvArgs()
                r.psum_num_recv_tokens_per_rank, r.psum_num_recv_tokens_per_expert = a.psum_num_recv_tokens_per_rank, \
                    a.psum_num_recv_tokens_per_expert
                r.num_unaligned_recv_tokens_per_expert = a.num_unaligned_recv_tokens_per_expert
                r.cumulative_local_expert_recv_stats = a.cumulative_local_expert_recv_stats
                r.recv_src_metadata = _desc(recv_src_metadata)
                r.hidden_bytes = hidden * (1 if fused_fp8_quant else x.element_size())
                r.num_sf_packs = 2 * ((hidden + 127) // 128) if fused_fp8_quant else (sf.size(1) if sf is not None else 0)
                r.num_topk, r.num_max_tokens_per_rank = num_topk, num_max_tokens_per_rank
                r.num_experts, r.expert_alignment = num_experts, expert_alignment
                r.do_cpu_sync = int(do_cpu_sync)
                r.dispatch_stamp = stamp
                r.stream = _stream()
                _check(_ep_dispatch_recv(self._h, ctypes.byref(r)))

            def wait_counts():
                c_recv, c_exp = ctypes.c_int(), ctypes.c_int()
                c_list = (ctypes.c_int * max(1, num_local_experts))()
                _check(_ep_wait(self._h, ctypes.byref(c_recv), ctypes.byref(c_exp), c_list))
                return c_recv.value, c_exp.value, c_list[:num_local_experts]       # (a slice of a ctypes array is a list)

            if cached_mode:
                num_recv, num_expanded = cached_num_recv_tokens, cached_num_expanded_tokens
                per_expert_list = cached_num_recv_tokens_per_expert_list
                alloc_recv, alloc_expanded = num_recv, num_expanded
            elif do_cpu_sync and self.connected:
                # a node: the bound over every partition's tokens is far above what arrives; wait for the counts
                num_recv, num_expanded, per_expert_list = wait_counts()
                alloc_recv, alloc_expanded = num_recv, num_expanded
                recv_src_metadata = recv_src_metadata[:num_recv]
            elif do_cpu_sync:
                # Exact sizes come from the host count page, but waiting for it here would leave the GPU
                # idle between the layout kernels and the copy.  Allocate for this call's upper bound,
                # enqueue the copy, and read the counts while it runs; the results are narrowed below.
                alloc_recv = num_tokens
                alloc_expanded = num_tokens * min(num_topk, num_local_experts) + (expert_alignment - 1) * num_local_experts
                alloc_expanded = -(-alloc_expanded // expert_alignment) * expert_alignment
                num_recv = num_expanded = None
            else:
                c_recv, c_exp = ctypes.c_int(), ctypes.c_int()
                _check(_ep_worst(self._h, num_max_tokens_per_rank, num_topk, num_experts, expert_alignment,
                                 ctypes.byref(c_recv), ctypes.byref(c_exp)))
                num_recv, num_expanded = c_recv.value, c_exp.value
                alloc_recv, alloc_expanded = num_recv, num_expanded

            out_dtype = torch.float8_e4m3fn if fused_fp8_quant else x.dtype
            recv_x = torch.empty((alloc_expanded, hidden), dtype=out_dtype, device=dev)
            recv_sf = None
            if fused_fp8_quant or sf is not None:
                sf_cols = (hidden + 127) // 128 if fused_fp8_quant else sf.size(1)
                sf_dtype = torch.float32 if fused_fp8_quant else sf.dtype
                sf_staging = None
                if use_col_major_sf:
                    # scale rows go to a staging tensor, a tiled kernel of the library turns them into columns
                    sf_staging = torch.empty((alloc_expanded, sf_cols), dtype=sf_dtype, device=dev)
                    sf_storage = torch.empty((sf_cols * alloc_expanded,), dtype=sf_dtype, device=dev)
                    recv_sf = sf_storage.as_strided((alloc_expanded, sf_cols), (1, alloc_expanded))
                else:
                    recv_sf = torch.empty((alloc_expanded, sf_cols), dtype=sf_dtype, device=dev)
            recv_topk_weights = None
            if topk_weights is not None:
                recv_topk_weights = torch.empty((alloc_expanded,), dtype=topk_weights.dtype, device=dev)
            if cached_mode:
                recv_src_metadata = cached_recv_src_metadata
                if recv_src_metadata.dim() != 2 or recv_src_metadata.size(0) != num_recv:
                    raise EPException('Assertion exception (_C.py): recv_src_metadata.size(0) == num_recv_tokens')
            elif recv_src_metadata is None:
                recv_src_metadata = ints(alloc_recv, num_topk + 2)

            e = _DispatchEpilogueArgs()
            e.x, e.sf, e.topk_weights = a.x, a.sf, a.topk_weights
            e.psum_num_recv_tokens_per_rank = a.psum_num_recv_tokens_per_rank
            e.psum_num_recv_tokens_per_expert = a.psum_num_recv_tokens_per_expert
            e.recv_x, e.recv_sf = _desc(recv_x), _desc(recv_sf, two_byte_packs=not fused_fp8_quant)
            if recv_sf is not None:
                e.recv_sf_staging = _desc(sf_staging, two_byte_packs=not fused_fp8_quant)
            e.recv_topk_weights, e.recv_src_metadata = _desc(recv_topk_weights), _desc(recv_src_metadata)
            e.num_topk, e.num_max_tokens_per_rank = num_topk, num_max_tokens_per_rank
            e.num_experts, e.expert_alignment = num_experts, expert_alignment
            e.cached_mode, e.do_zero_padding = int(cached_mode), int(do_zero_padding)
            e.fused_fp8_quant = int(fused_fp8_quant)
            # sizes still unknown on the host: the column stride is the row count the device computed
            e.recv_sf_layout = (2 if num_recv is None else 1) if use_col_major_sf else 0
            e.stream = _stream()
            e.dispatch_stamp = stamp
            _check(_ep_dispatch_epi(self._h, ctypes.byref(e)))

            if num_recv is None:
                num_recv, num_expanded, per_expert_list = wait_counts()
                if num_recv > alloc_recv or num_expanded > alloc_expanded:
                    raise EPException('Assertion exception (_C.py): received counts exceed this call\'s bound')
                recv_x = recv_x[:num_expanded]
                if recv_sf is not None and use_col_major_sf:
                    recv_sf = sf_storage.as_strided((num_expanded, sf_cols), (1, num_expanded))
                elif recv_sf is not None:
                    recv_sf = recv_sf[:num_expanded]
                recv_topk_weights = recv_topk_weights[:num_expanded] if recv_topk_weights is not None else None
                recv_src_metadata = recv_src_metadata[:num_recv]

            return (recv_x, recv_sf, recv_topk_weights, num_recv, num_expanded, per_expert_list,
                    psum_rank, psum_expert, unaligned, recv_src_metadata, dst_slot, dst_gsge)

        if defer_epilogue:
            if not async_with_compute_stream:
                raise EPException('Assertion exception (_C.py): async_with_compute_stream')
            return None, EventHandle(), epilogue
        result = epilogue()
        return result, (EventHandle() if async_with_compute_stream else None), None

    # ---- combine (argument order of csrc/buffers/ep.hpp:412-425) ----
    def combine(self, x, topk_weights, bias_0, bias_1, src_metadata, combined_topk_idx,
                psum_num_recv_tokens_per_rank, num_experts, num_max_tokens_per_rank, num_sms, previous_event,
                async_with_compute_stream, allocate_on_comm_stream, defer_epilogue, apply_weights=False):
        if self.destroyed:
            raise EPException('Assertion exception (_C.py): not destroyed')
        if previous_event is not None:
            previous_event.current_stream_wait()
        if num_sms <= 0:
            raise EPException('Assertion exception (_C.py): num_sms > 0')
        if x.dim() != 2 or combined_topk_idx.dim() != 2:
            raise EPException('Assertion exception (_C.py): x.dim() == 2 and combined_topk_idx.dim() == 2')
        dev = x.device
        hidden = x.size(1)
        num_combined_tokens, num_topk = combined_topk_idx.shape

        c = _CombineArgs()
        c.x, c.topk_weights, c.bias_0, c.bias_1 = _desc(x), _desc(topk_weights), _desc(bias_0), _desc(bias_1)
        c.src_metadata, c.combined_topk_idx = _desc(src_metadata), _desc(combined_topk_idx)
        c.psum_num_recv_tokens_per_rank = _desc(psum_num_recv_tokens_per_rank)
        c.num_experts, c.num_max_tokens_per_rank = num_experts, num_max_tokens_per_rank
        c.apply_weights = int(apply_weights)
        c.stream = _stream()
        _check(_ep_combine(self._h, ctypes.byref(c), 0))           # owner side (nothing to do for one partition)

        keep_alive = (x, topk_weights, bias_0, bias_1, src_metadata, combined_topk_idx, psum_num_recv_tokens_per_rank)

        def epilogue():
            # the descriptors hold raw pointers: the tensors stay referenced until the reduce is enqueued
            assert keep_alive is not None
            combined_x = torch.empty((num_combined_tokens, hidden), dtype=x.dtype, device=dev)
            combined_topk_weights = None
            if topk_weights is not None:
                combined_topk_weights = torch.empty((num_combined_tokens, num_topk), dtype=topk_weights.dtype,
                                                    device=dev)
            c.combined_x, c.combined_topk_weights = _desc(combined_x), _desc(combined_topk_weights)
            c.stream = _stream()
            _check(_ep_combine(self._h, ctypes.byref(c), 1))       # token side
            return combined_x, combined_topk_weights

        if defer_epilogue:
            if not async_with_compute_stream:
                raise EPException('Assertion exception (_C.py): async_with_compute_stream')
            return None, EventHandle(), epilogue
        result = epilogue()
        return result, (EventHandle() if async_with_compute_stream else None), None


def barrier(context, with_cpu_sync: bool = False, sequential: bool = True, wait_comm_stream: bool = True) -> None:
    if with_cpu_sync:
        torch.cuda.current_stream().synchronize()


def get_comm_stream():
    return torch.cuda.current_stream()


def get_physical_domain_size(group_name: str = '') -> Tuple[int, int]:
    return 1, 1


def get_logical_domain_size(group_name: str = '', allow_hybrid_mode: bool = True) -> Tuple[int, int]:
    return 1, 1
