"""Binding layer over libdeep_ep_hip.so (the C ABI declared in include/deep_ep_hip.h).

It exposes the names the reference's pybind module `deep_ep._C` exports for the EP path
(csrc/python_api.cpp:18-74): `EventHandle`, `EPBuffer` with `.dispatch(27 args)` /
`.combine(14 args)`, `calculate_ep_buffer_size`, the alignment getters, `topk_idx_t` and the
runtime-configuration functions.  Torch tensors are only plumbing here.  The two hot calls,
`EPBuffer.dispatch` and `EPBuffer.combine`, are compiled (`_native`, csrc/python_api.cpp: pybind11 over
the C ABI, as the reference's own binding is); everything else goes through ctypes.  There is no CPU
or torch fallback: if the library, its code object or the compiled binding is missing, importing or
using this module raises.
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

try:
    from . import _native
except ImportError as e:       # pragma: no cover
    raise ImportError(f'the compiled binding deep_ep._native is missing or does not load ({e}): build it first '
                      '(python deepep-ascend_amd/deep_ep/_build.py)') from e


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
_ep_quantise = _sig('ep_per_token_cast_to_fp8', ctypes.c_int, ctypes.POINTER(_Tensor), ctypes.POINTER(_Tensor),
                   ctypes.POINTER(_Tensor), ctypes.c_void_p)
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
_ep_set_recount = _sig('ep_set_layout_recount_limit', None, ctypes.c_int)
_ep_set_combine_cap = _sig('ep_set_combine_blocks_per_cu', None, ctypes.c_int)
_ep_dispatch_static = _sig('ep_dispatch_static_launch', ctypes.c_int, ctypes.POINTER(_DispatchArgs),
                           ctypes.POINTER(_DispatchEpilogueArgs))
_ep_static_bytes = _sig('ep_dispatch_static_scratch_bytes', ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int)
_ep_static_capacity = _sig('ep_dispatch_static_scratch_capacity', ctypes.c_int64)
_ep_combine = _sig('ep_combine_launch', ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(_CombineArgs), ctypes.c_int)


# Raised for contract violations and runtime failures reported by the native library (a RuntimeError).
EPException = _native.EPException


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


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """The caller-side quantiser on the GPU (`x` a contiguous bfloat16 CUDA tensor `[T, H]`, H a multiple of 8):
    the library's own kernel, whose bytes are those of the fused dispatch and of the formula evaluated by torch
    on the CPU."""
    init_jit()
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=torch.float8_e4m3fn, device=x.device)
    sf = torch.empty((rows, (cols + 127) // 128), dtype=torch.float32, device=x.device)
    dx, dq, dsf = _desc(x), _desc(q), _desc(sf)
    _check(_ep_quantise(ctypes.byref(dx), ctypes.byref(dq), ctypes.byref(dsf), _stream()))
    return q, sf


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


def set_layout_recount_limit(blocks_times_topk: int) -> None:
    """Tuning: with one partition and few layout blocks (blocks x top-k up to this limit, at most 48; 0: never) the slot
    assignment counts the ids of all blocks itself and the histogram kernel is not launched.  Results do not depend on it."""
    _ep_set_recount(int(blocks_times_topk))


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
        self._native = _native.Buffer(handle.value, rank_idx, num_ranks)
        # the hot calls are the compiled binding's: dispatch(27 args, fused_fp8_quant=) in the argument order of
        # csrc/buffers/ep.hpp:89-112, combine(14 args, apply_weights=) in that of csrc/buffers/ep.hpp:412-425; both
        # return (result or None, EventHandle or None, deferred epilogue or None)
        self.dispatch = self._native.dispatch
        self.combine = self._native.combine
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

    def set_exact_sync_sizes(self, enable: bool) -> None:
        """Host-synchronised dispatches of a single partition wait for the counts before they allocate (outputs of
        exactly the counted sizes, as csrc/buffers/ep.hpp:300-351 allocates them) instead of allocating for the call's
        upper bound and narrowing."""
        self._native.set_exact_sync_sizes(bool(enable))

    # ---- lifecycle ----
    def destroy(self) -> None:
        if self.destroyed:
            raise EPException('Assertion exception (_C.py): not destroyed')
        self.lb_storage = None
        self._native.invalidate()
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
            self._native.set_connected(False)
            return
        table = (ctypes.c_void_p * len(arena_bases))(*arena_bases)
        _check(_ep_set_peers(self._h, table, len(arena_bases)))
        self.connected = True
        self._native.set_connected(True)

    @staticmethod
    def connect(runtimes) -> None:
        """Makes the given runtime objects (partition i of n at index i) one node: packed rows, row counts
        and combine partials then go straight into the arena of the partition they are meant for."""
        handles = (ctypes.c_void_p * len(runtimes))(*[r._h for r in runtimes])
        _check(_ep_connect(handles, len(runtimes)))
        for r in runtimes:
            r.connected = True
            r._native.set_connected(True)

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


def barrier(context, with_cpu_sync: bool = False, sequential: bool = True, wait_comm_stream: bool = True) -> None:
    if with_cpu_sync:
        torch.cuda.current_stream().synchronize()


def get_comm_stream():
    return torch.cuda.current_stream()


def get_physical_domain_size(group_name: str = '') -> Tuple[int, int]:
    return 1, 1


def get_logical_domain_size(group_name: str = '', allow_hybrid_mode: bool = True) -> Tuple[int, int]:
    return 1, 1
