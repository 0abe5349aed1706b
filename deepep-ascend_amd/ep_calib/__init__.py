"""ctypes binding of libdeep_ep_calib.so (include/deep_ep_calib.h): the calibration kernels the benchmarks
use to price the memory system and the alternatives to the token-major copy kernel.  Not part of the
`deep_ep` product package: nothing there imports this, and this imports nothing from there."""
import ctypes
import os

import torch

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'lib')
_LIB_PATH = os.path.join(_LIB_DIR, 'libdeep_ep_calib.so')
if not os.path.exists(_LIB_PATH):
    raise ImportError(f'{_LIB_PATH} is missing: build it first (python deepep-ascend_amd/deep_ep/_build.py)')
_lib = ctypes.CDLL(_LIB_PATH)

VARIANTS = ('token_major', 'stores_only', 'read_rows', 'ordered_flat', 'ordered_flat_stores_only', 'ordered_steered',
            'ordered_steered_stores_only', 'ordered_steered_loads_only', 'quant_rows', 'copy_ordered_flat',
            'copy_ordered_steered')


class ScatterArgs(ctypes.Structure):
    # ep_calib_scatter_t
    _fields_ = [(n, ctypes.c_void_p) for n in (
        'x', 'topk_weights', 'recv_src_metadata', 'num_recv', 'psum_expert', 'recv_x', 'recv_sf', 'recv_topk_weights',
        'order', 'q_rows', 'q_sf')] + [(n, ctypes.c_int32) for n in (
            'num_tokens', 'hidden', 'num_topk', 'num_experts', 'expert_alignment', 'num_recv_rows', 'num_out_rows',
            'do_zero_padding', 'num_entries', 'entries_per_list', 'num_lists')] + [('stream', ctypes.c_void_p)]


COMBINE_VARIANTS = ('combine', 'combine_loads_only', 'combine_stores_only')


class CombineArgs(ctypes.Structure):
    # ep_calib_combine_t
    _fields_ = [(n, ctypes.c_void_p) for n in (
        'y', 'expanded_weights', 'recv_src_metadata', 'num_recv', 'topk_idx', 'combined_x', 'combined_topk_weights')] + [
            (n, ctypes.c_int32) for n in ('num_tokens', 'hidden', 'num_topk', 'num_experts', 'num_recv_rows', 'num_in_rows',
                                          'blocks_per_cu', 'reserved')] + [('stream', ctypes.c_void_p)]


def _sig(name, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = ctypes.c_int
    fn.argtypes = list(argtypes)
    return fn


_init = _sig('ep_calib_init', ctypes.c_char_p)
_last_error = _lib.ep_calib_last_error
_last_error.restype = ctypes.c_char_p
_fill = _sig('ep_calib_fill', ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p)
_fill_affine = _sig('ep_calib_fill_affine', ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_uint, ctypes.c_void_p)
_fronts = _sig('ep_calib_fronts', ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_uint,
               ctypes.c_void_p)
_mixed = _sig('ep_calib_mixed', ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_uint,
              ctypes.c_void_p)
_scatter = _sig('ep_calib_scatter', ctypes.c_int, ctypes.POINTER(ScatterArgs))
_combine = _sig('ep_calib_combine', ctypes.c_int, ctypes.POINTER(CombineArgs))


class CalibError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise CalibError(_last_error().decode())


def _stream():
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def init():
    _check(_init(None))


def fill(dst: torch.Tensor, shuffled: int = 0, value: int = 0) -> None:
    """Writes the whole of `dst` (a multiple of 4 KiB), one chunk per workgroup: in address order, or with runs
    of `shuffled` chunks in a scrambled order (powers of two)."""
    _check(_fill(dst.data_ptr(), dst.numel() * dst.element_size(), int(shuffled), value, _stream()))


def fill_affine(dst: torch.Tensor, modulus: int, shift: int = 0, value: int = 0) -> None:
    """Writes the whole of `dst` in a scrambled order in which workgroup b writes a chunk with index = b + shift
    modulo `modulus`: every chunk comes from the XCD that is `shift` places after the one address order gives it."""
    _check(_fill_affine(dst.data_ptr(), dst.numel() * dst.element_size(), modulus, shift, value, _stream()))


def fronts(dst: torch.Tensor, num_fronts: int, rows_per_front: int, row_bytes: int, front_pitch_bytes: int) -> None:
    assert dst.numel() * dst.element_size() >= (num_fronts - 1) * front_pitch_bytes + rows_per_front * row_bytes
    _check(_fronts(dst.data_ptr(), num_fronts, rows_per_front, row_bytes, front_pitch_bytes, 1, _stream()))


def mixed(src: torch.Tensor, dst: torch.Tensor, reads_num: int, reads_den: int) -> None:
    """Writes every 4 KiB chunk of `dst` in address order while reading `reads_num` chunks of `src` per
    `reads_den` written."""
    wbytes = dst.numel() * dst.element_size()
    need = -(-(wbytes // 4096) * reads_num // reads_den) * 4096
    assert src.numel() * src.element_size() >= need
    _check(_mixed(src.data_ptr(), dst.data_ptr(), wbytes, reads_num, reads_den, 0, _stream()))


def scatter(variant: str, args: ScatterArgs) -> None:
    args.stream = _stream()
    _check(_scatter(VARIANTS.index(variant), ctypes.byref(args)))


def combine(variant: str, args: CombineArgs) -> None:
    """The single-partition combine at top-6: 'combine' (the product's kernel body), 'combine_loads_only' (its row
    fetches and sums, nothing written), 'combine_stores_only' (its stores of filler rows, nothing fetched but the slots)."""
    args.stream = _stream()
    _check(_combine(COMBINE_VARIANTS.index(variant), ctypes.byref(args)))


def build_order(recv_src_metadata: torch.Tensor, num_topk: int, chunk_tokens: int, steered: bool):
    """(slot, token | position << 24) pairs of every valid (row, position) of a single-partition handle, sorted
    by slot inside chunks of `chunk_tokens` tokens.  Steered: one list per (chunk, token % 8), padded with holes
    to a common length.  Returns (int32 tensor [n, 2], entries_per_list, num_lists)."""
    K = num_topk
    meta = recv_src_metadata.long()
    slots = meta[:, :K]
    tok = meta[:, K:K + 1].expand(-1, K)
    pos = torch.arange(K, device=meta.device).expand_as(slots)
    valid = slots >= 0
    slots, tok, pos = slots[valid], tok[valid], pos[valid]
    chunk = tok // chunk_tokens
    num_chunks = int(chunk.max().item()) + 1
    if not steered:
        key = chunk * (1 << 32) + slots
        idx = torch.argsort(key)
        out = torch.stack([slots[idx], tok[idx] | (pos[idx] << 24)], dim=1).to(torch.int32).contiguous()
        return out, 0, 0
    lst = chunk * 8 + (tok & 7)
    key = lst * (1 << 32) + slots
    idx = torch.argsort(key)
    lst, slots, tok, pos = lst[idx], slots[idx], tok[idx], pos[idx]
    num_lists = num_chunks * 8
    counts = torch.bincount(lst, minlength=num_lists)
    per_list = int(counts.max().item())
    starts = torch.cumsum(counts, 0) - counts
    within = torch.arange(lst.numel(), device=meta.device) - starts[lst]
    out = torch.full((num_lists * per_list, 2), -1, dtype=torch.int32, device=meta.device)
    dst = lst * per_list + within
    out[dst, 0] = slots.to(torch.int32)
    out[dst, 1] = (tok | (pos << 24)).to(torch.int32)
    return out.contiguous(), per_list, num_lists
