"""ep_dispatch_static_launch: the single-partition dispatch that needs no buffer and allocates nothing
(its layout scratch is a device array inside the library).  Called through the C ABI and compared,
bit for bit, with what ep_dispatch_launch + ep_dispatch_epilogue_launch of an ordinary buffer produce
on the same inputs: two calls in a row, the second with a smaller input, so leftovers of the first in
the shared scratch would show.  The first shape is also compared with the CPU oracle, and the second call
must leave the device's free memory where it was."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_routing, make_tokens
from oracle import ep_oracle as O

pytestmark = pytest.mark.gpu

DEV = 'cuda'


def _worst_case(C, T, K, E, A):
    n_recv, n_exp = ctypes.c_int(), ctypes.c_int()
    C._check(C._ep_worst(None, T, K, E, A, ctypes.byref(n_recv), ctypes.byref(n_exp)))
    return n_recv.value, n_exp.value


def _static_dispatch(C, x, topk, w, E, A, fused):
    """One call of the allocation-free entry point; every tensor is allocated here, by the caller."""
    T, H = x.shape
    K = topk.size(1)
    n_recv, n_exp = _worst_case(C, T, K, E, A)
    i32 = dict(dtype=torch.int32, device=DEV)
    out = dict(psum_rank=torch.full((1,), -7, **i32), psum_expert=torch.full((E,), -7, **i32),
               unaligned=torch.full((E,), -7, **i32), dst_slot=torch.full((T, K), -7, **i32),
               dst_gsge=torch.full((T, K), -7, **i32), meta=torch.full((n_recv, K + 2), -7, **i32),
               recv_x=torch.full((n_exp, H), 77, dtype=torch.uint8, device=DEV).view(
                   torch.float8_e4m3fn if fused else torch.uint8),
               recv_w=torch.full((n_exp,), -7.0, dtype=torch.float32, device=DEV))
    if not fused:
        out['recv_x'] = torch.full((n_exp, H), 77, dtype=torch.int16, device=DEV).view(torch.bfloat16)
    out['recv_sf'] = torch.full((n_exp, (H + 127) // 128), -7.0, dtype=torch.float32, device=DEV) if fused else None
    a = C._DispatchArgs()
    a.x, a.topk_idx, a.topk_weights = C._desc(x), C._desc(topk), C._desc(w)
    a.psum_num_recv_tokens_per_rank, a.psum_num_recv_tokens_per_expert = C._desc(out['psum_rank']), C._desc(out['psum_expert'])
    a.num_unaligned_recv_tokens_per_expert = C._desc(out['unaligned'])
    a.dst_buffer_slot_idx, a.dst_gsge_idx = C._desc(out['dst_slot']), C._desc(out['dst_gsge'])
    a.num_max_tokens_per_rank, a.num_experts, a.expert_alignment = T, E, A
    a.cached_mode, a.do_cpu_sync, a.fused_fp8_quant = 0, 0, int(fused)
    a.stream = C._stream()
    e = C._DispatchEpilogueArgs()
    e.x, e.topk_weights = a.x, a.topk_weights
    e.psum_num_recv_tokens_per_rank, e.psum_num_recv_tokens_per_expert = a.psum_num_recv_tokens_per_rank, \
        a.psum_num_recv_tokens_per_expert
    e.recv_x, e.recv_sf = C._desc(out['recv_x']), C._desc(out['recv_sf'])
    e.recv_topk_weights, e.recv_src_metadata = C._desc(out['recv_w']), C._desc(out['meta'])
    e.num_topk, e.num_max_tokens_per_rank, e.num_experts, e.expert_alignment = K, T, E, A
    e.cached_mode, e.do_zero_padding, e.fused_fp8_quant, e.recv_sf_layout = 0, 1, int(fused), 0
    e.stream = a.stream
    C._check(C._ep_dispatch_static(ctypes.byref(a), ctypes.byref(e)))
    out['_args'] = (a, e)          # (the descriptors hold raw pointers into `out` and the inputs: the caller keeps both)
    return out


def _compare_with_oracle(out, x, topk, w, E, A, fused):
    """The allocation-free path against the CPU oracle itself (not only against the buffer path)."""
    T = x.size(0)
    lay = O.rank_share_layout(topk.numpy(), E, 1, 0, A, T)
    n_recv, upto = lay['num_recv_tokens'], lay['num_expanded_tokens']
    assert np.array_equal(out['psum_expert'].cpu().numpy(), lay['psum_num_recv_tokens_per_expert'])
    assert np.array_equal(out['dst_slot'].cpu().numpy(), lay['dst_buffer_slot_idx'])
    assert np.array_equal(out['meta'][:n_recv].cpu().numpy(), lay['recv_src_metadata'])
    if fused:
        q, s = O.quantise(x)
        ex, es, ew = O.rank_share_dispatch(q.numpy(), s.numpy().view(np.uint32), w.numpy(), lay)
        assert np.array_equal(out['recv_x'][:upto].view(torch.uint8).cpu().numpy(), ex[:upto])
        assert np.array_equal(out['recv_sf'][:upto].cpu().numpy().view(np.uint32), es[:upto])
    else:
        ex, _, ew = O.rank_share_dispatch(bf16_bits(x).view(np.int16), None, w.numpy(), lay)
        assert np.array_equal(bf16_bits(out['recv_x'][:upto]).view(np.int16), ex[:upto])
    assert np.array_equal(out['recv_w'][:upto].cpu().numpy().view(np.uint32), ew[:upto].view(np.uint32))


def _buffer_dispatch(de, x, topk, w, E, A, fused):
    T, H = x.shape
    K = topk.size(1)
    buf = de.EPBuffer(de.LocalGroup(), num_max_tokens_per_rank=T, hidden=H, num_topk=K, use_fp8_dispatch=fused,
                      explicitly_destroy=True)
    recv, _, recv_w, h, _ = buf.dispatch(x, topk_idx=topk, topk_weights=w, num_experts=E, expert_alignment=A,
                                         do_expand=True, do_zero_padding=True, do_cpu_sync=False, fused_fp8_quant=fused)
    torch.cuda.synchronize()
    buf.destroy()
    return recv, recv_w, h


def _compare(out, ref, fused, A):
    recv, recv_w, h = ref
    n_recv = int(h.psum_num_recv_tokens_per_rank[-1])
    assert torch.equal(out['psum_rank'], h.psum_num_recv_tokens_per_rank)
    assert torch.equal(out['psum_expert'], h.psum_num_recv_tokens_per_expert)
    assert torch.equal(out['unaligned'], h.num_unaligned_recv_tokens_per_expert)
    assert torch.equal(out['dst_slot'], h.dst_buffer_slot_idx)
    assert torch.equal(out['dst_gsge'], h.dst_gsge_idx)
    assert n_recv > 0 and torch.equal(out['meta'][:n_recv], h.recv_src_metadata[:n_recv])
    # valid rows and zeroed padding alike; the rows behind the last expert's padding are written by neither path
    upto = (int(h.psum_num_recv_tokens_per_expert[-1]) + A - 1) // A * A
    got_x, ref_x = out['recv_x'].view(torch.uint8), (recv[0] if fused else recv).view(torch.uint8)
    assert got_x.shape == ref_x.shape and 0 < upto <= got_x.size(0)
    assert torch.equal(got_x[:upto], ref_x[:upto])
    assert torch.equal(out['recv_w'][:upto].view(torch.int32), recv_w[:upto].view(torch.int32))
    if fused:
        assert torch.equal(out['recv_sf'][:upto].view(torch.int32), recv[1][:upto].view(torch.int32))


@pytest.mark.parametrize('fused', [True, False])
def test_static_dispatch_matches_the_buffer_path_twice(fused):
    import deep_ep as de
    C = de._C
    C.init_jit()
    E, K, A, H = 32, 4, 16, 512
    for T, seed in ((700, 1), (130, 2)):                  # the second call is smaller: the scratch keeps the first's contents
        x = make_tokens(T, H, seed=seed, outliers=True).to(DEV)
        topk_cpu, w_cpu = make_routing(T, E, K, seed=seed, masked=0.15)
        topk, w = topk_cpu.to(DEV), w_cpu.to(DEV)
        out = _static_dispatch(C, x, topk, w, E, A, fused)
        torch.cuda.synchronize()
        if T == 700:
            _compare_with_oracle(out, x.cpu(), topk_cpu, w_cpu, E, A, fused)
        ref = _buffer_dispatch(de, x, topk, w, E, A, fused)
        _compare(out, ref, fused, A)
    # the entry point exists for callers that cannot allocate: a further call (every tensor it needs already
    # exists) leaves the device's free memory untouched
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    a, e = out['_args']
    C._check(C._ep_dispatch_static(ctypes.byref(a), ctypes.byref(e)))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    _compare(out, ref, fused, A)


def test_static_dispatch_rejects_what_does_not_fit():
    import deep_ep as de
    C = de._C
    C.init_jit()
    T, H, E, K, A = 400000, 128, 8, 2, 1                 # slot map 3.2 MB + token -> row map 1.6 MB > 4 MiB
    assert C._ep_static_bytes(T, K, E) > C._ep_static_capacity() >= C._ep_static_bytes(700, 4, 32)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    topk = torch.zeros((T, K), dtype=torch.int64, device=DEV)
    with pytest.raises(C.EPException, match='exceeds the library\'s static scratch'):
        _static_dispatch(C, x, topk, None, E, A, False)
    torch.cuda.synchronize()
